#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on SmolLM2-1.7B shapes with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096] [--layers 24]
                    [--shapes smollm2-1.7b|smollm2-360m|llama-3-8b] [--reps 3]

A step is one decode step of the whole batch through the path that greedy generation uses: ``Engine.step``
(which replays steps of single tokens from HIP graphs) and the device sampler (``sampling.greedy_pending``), the
sampled tokens fed back as the next step's input: the step takes them from the device and the host reads every
one of them while it runs (``--read-back-first`` reads them before the next step is launched, as a caller must
that looks at a token before it feeds it).  The batch is first prefilled (through the same step function, in
portions of 2,048 tokens) so that the last timed step reaches the context length.  K steps are timed ``--reps``
times in a row, each time between synchronisations; ``ms_per_step`` and ``value`` are the mean over the
repetitions and ``reps`` holds their spread; the batch 1 and 64 points are repeated as often, with their spread
beside them (``points.decode_b1_sd``).  ``points.decode_b<batch>_scheduler`` is the same workload as
requests under ``Scheduler.step`` (plan, step, sample, finish), ``points.decode_b<batch>_read_back_first`` the
same steps with the tokens read back before each launch.  Prints one JSON line.  One GPU only: for
--gpus > 1 it says so and exits with 2.
"""
import argparse
import datetime
import json
import os
import statistics
import sys
import time

# SmolLM2-1.7B shapes: the benchmark configuration (the default); the others for measurements at further sizes
SHAPES = {
    "smollm2-1.7b": dict(architectures=["LlamaForCausalLM"], hidden_size=2048, intermediate_size=8192,
                         num_hidden_layers=24, num_attention_heads=32, num_key_value_heads=32, vocab_size=49152,
                         rope_theta=130000.0, rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=8192),
    "smollm2-360m": dict(architectures=["LlamaForCausalLM"], hidden_size=960, intermediate_size=2560,
                         num_hidden_layers=32, num_attention_heads=15, num_key_value_heads=5, vocab_size=49152,
                         rope_theta=100000.0, rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=8192),
    "llama-3-8b": dict(architectures=["LlamaForCausalLM"], hidden_size=4096, intermediate_size=14336,
                       num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=8, vocab_size=128256,
                       rope_theta=500000.0, rms_norm_eps=1e-5, tie_word_embeddings=False, max_position_embeddings=8192),
}
NAMES = {"smollm2-1.7b": "SmolLM2-1.7B shapes", "smollm2-360m": "SmolLM2-360M shapes", "llama-3-8b": "Llama-3-8B shapes"}
PEAK = {"hbm_gbs": 8000.0, "bf16_tflops": 2500.0, "fp32_tflops": 157.3}   # MI355X, dense
PREFILL_TOKENS = 2048


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--shapes", default="smollm2-1.7b", choices=sorted(SHAPES))
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (both numbers are reported)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points")
    ap.add_argument("--only", choices=["decode", "prefill", "portion"], default=None,
                    help="for profiling: run only the decode steps (after their prefill), only the 2,048-token prefill, or "
                         "only a portion of --portion-tokens tokens behind a cached context of --context tokens (a new "
                         "turn behind a long history, the tail of a prompt)")
    ap.add_argument("--portion-tokens", type=int, default=128)
    ap.add_argument("--no-graph", action="store_true", help="run decode steps without HIP graph replay")
    ap.add_argument("--no-layer-tapes", action="store_true",
                    help="walk every layer through the parts' Python (by default layers of a kind share one walk a step)")
    ap.add_argument("--page-size", type=int, default=16, help="tokens a page of the cache (16 as in the reference)")
    ap.add_argument("--reps", type=int, default=3, help="times the K timed steps are repeated (mean and spread are reported)")
    ap.add_argument("--no-scheduler", action="store_true", help="skip the figure through Scheduler.step")
    ap.add_argument("--read-back-first", action="store_true",
                    help="read a step's sampled tokens back before the next step is launched")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="with --only prefill, for profiling: a prompt of another length than the 2,048 tokens of the record")
    a = ap.parse_args()
    if a.prefill_tokens != PREFILL_TOKENS and a.only != "prefill":
        print("bench.py: --prefill-tokens goes with --only prefill; the record's prefill is of 2,048 tokens")
        return 2
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        return 2

    import torch
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.engine import Engine
    from glassbox_amd.engine import Scheduler, SchedulerConfig
    from glassbox_amd.sampling import SamplerConfig, greedy_pending, sample_rows
    from glassbox_amd.weights import build_model, init_random

    MODEL = SHAPES[a.shapes]
    # (a context beyond the model's own limit is measured all the same: the scheduler would end requests at the limit)
    cfg = config_from_dict(dict(MODEL, num_hidden_layers=a.layers or MODEL["num_hidden_layers"],
                                max_position_embeddings=max(MODEL["max_position_embeddings"], a.context + 1)))
    model = build_model(cfg)
    init_random(model, seed=0, dtype=a.dtype, device="cuda:0")
    batches = [a.batch] + ([] if a.no_points else [b for b in (1, 64) if b != a.batch])
    max_tokens = max(max(batches) * (a.context + 64), a.prefill_tokens + 64)
    eng = Engine(model, dtype=a.dtype, max_tokens=max_tokens, max_seqs=max(batches), page_size=a.page_size,
                 graph_decode=False if a.no_graph else None, layer_tapes=not a.no_layer_tapes)
    vocab = cfg.vocab_size
    g = torch.Generator().manual_seed(1)

    d, L, I, qd, kvd = cfg.hidden_size, cfg.num_hidden_layers, cfg.intermediate_size, cfg.q_dim, cfg.kv_dim
    layer_params = d * (qd + 2 * kvd) + qd * d + 2 * I * d + I * d
    esize = 2 if a.dtype == "bfloat16" else 4
    weight_bytes = model.weight_bytes()
    kv_bytes_per_token = 2 * kvd * esize * L

    # ---- prefill: one step of 2,048 tokens, logits for the last one
    def prefill_once(name):
        toks = torch.randint(0, vocab, (a.prefill_tokens,), generator=g).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.step([(name, toks, [a.prefill_tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        eng.end_request(name)
        return dt
    if a.only == "portion":
        # a step of a few hundred rows: the history is cached in portions of 2,048, then the timed step brings the rest
        hist = a.context - a.portion_tokens
        times, host = [], []
        for rep in range(4):
            toks = torch.randint(0, vocab, (a.context,), generator=g).tolist()
            for at in range(0, hist, PREFILL_TOKENS):
                eng.step([("p", toks[at:min(at + PREFILL_TOKENS, hist)], [])])
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            eng.step([("p", toks[hist:], [a.portion_tokens - 1])])
            host.append(time.perf_counter() - t0)              # the launches are made: what the step costs the host
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            eng.end_request("p")
        print(json.dumps({"portion_ms": round(min(times[1:]) * 1e3, 3), "tokens": a.portion_tokens, "context": a.context,
                          "host_ms": round(min(host[1:]) * 1e3, 3), "all_ms": [round(t * 1e3, 3) for t in times]}))
        return 0
    if a.only == "decode":
        pf = float("nan")
    else:
        prefill_once("warm")
        pf = min(prefill_once(f"pf{i}") for i in range(3))
    if a.only == "prefill":
        print(json.dumps({"prefill_ms": round(pf * 1e3, 3), "tokens": a.prefill_tokens}))
        return 0
    T = PREFILL_TOKENS
    pf_flops = 2 * T * layer_params * L + L * 4 * qd * (T * (T + 1) // 2) + 2 * d * vocab
    peak = PEAK["bf16_tflops"] if a.dtype == "bfloat16" else PEAK["fp32_tflops"]
    if a.only == "decode":   # not measured in this run: null, which JSON has and NaN is not
        prefill = {"value": None, "tokens": T, "ms": None, "frac": None}
    else:
        prefill = {"value": round(T / pf, 1), "tokens": T, "ms": round(pf * 1e3, 3),
                   "frac": round(pf_flops / pf / (peak * 1e12), 4)}

    # ---- decode: Engine.step and the device sampler, tokens fed back
    def decode_run(batch, steps, warmup, reps, read_back_first=a.read_back_first):
        start = a.context - reps * steps - warmup
        names = [f"d{batch}_{i}" for i in range(batch)]
        prompts = [torch.randint(0, vocab, (start,), generator=g).tolist() for _ in names]
        for at in range(0, start - 1, PREFILL_TOKENS):        # leave the last prompt token for the first decode step
            n = min(PREFILL_TOKENS, start - 1 - at)
            for name, p in zip(names, prompts):
                eng.step([(name, p[at:at + n], [])])
        tokens = [p[-1] for p in prompts]

        def one_step():
            nonlocal tokens
            # the sampled tokens stay on the device for the next step, which is launched before the host has their
            # values; Engine.step waits for them after the launch (the cache manager keeps every request's tokens)
            logits = eng.step([(name, [t], [0]) for name, t in zip(names, tokens)])
            if read_back_first:
                tokens, _ = sample_rows(logits, [SamplerConfig()] * batch, [0.0] * batch)
            else:
                tokens = greedy_pending(logits)

        for _ in range(warmup):
            one_step()
        times = []
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                one_step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        for name in names:
            eng.end_request(name)
        mean_ctx = a.context - (reps * steps + 1) / 2
        return times, mean_ctx

    # ---- the same workload as requests under the scheduler: plan, step, sample, finish
    def scheduler_run(batch, steps, warmup):
        # tokens that the first requests decode while the last ones are still prompts (a step of prompt portions each)
        slack = batch * -(-a.context // PREFILL_TOKENS) + 8
        budget = warmup + steps + slack
        start = a.context - budget
        sched = Scheduler(eng, SchedulerConfig(token_budget=PREFILL_TOKENS, max_seqs=batch))
        ids = [sched.submit(torch.randint(0, vocab, (start,), generator=g).tolist(), budget) for _ in range(batch)]
        while not all(sched.outputs[i].tokens for i in ids):
            sched.step()                                       # prompts, in portions under the token budget
        for _ in range(warmup):
            sched.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            sched.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if sched.running() != batch:
            raise RuntimeError("a request ended inside the timed steps of the scheduler figure")
        for i in ids:
            sched.abort(i)
        return dt

    times, mean_ctx = decode_run(a.batch, a.steps, a.warmup, a.reps)
    step_s = statistics.mean(times) / a.steps
    value = a.batch / step_s
    bytes_step = weight_bytes + a.batch * mean_ctx * kv_bytes_per_token
    achieved = bytes_step / step_s / 1e9
    points = {}
    if not a.no_scheduler:
        sdt = scheduler_run(a.batch, a.steps, a.warmup)
        points[f"decode_b{a.batch}_scheduler"] = round(a.batch * a.steps / sdt, 1)
    if not a.no_points:
        if not a.read_back_first:
            # the same steps with every step's tokens read back before the next is launched, as a caller must that
            # looks at a token before it feeds it
            k = max(8, min(a.steps, 32))
            pts, _ = decode_run(a.batch, k, min(a.warmup, 4), 1, read_back_first=True)
            points[f"decode_b{a.batch}_read_back_first"] = round(a.batch * k / pts[0], 1)
        for b in (1, 64):
            if b == a.batch:
                points[f"decode_b{b}"] = round(value, 1)
                continue
            k = max(8, min(a.steps, 32))
            pts, _ = decode_run(b, k, min(a.warmup, 4), a.reps)
            rates = [b * k / t for t in pts]
            points[f"decode_b{b}"] = round(statistics.mean(rates), 1)
            points[f"decode_b{b}_sd"] = round(statistics.stdev(rates), 1) if len(rates) > 1 else 0.0
            points[f"decode_b{b}_reps"] = len(rates)

    from glassbox_amd.build import source_version
    ms = [t / a.steps * 1e3 for t in times]

    out = {
        "metric": f"decode tok/s at batch {a.batch}, {NAMES[a.shapes]}, context {a.context} "
                  "(prefill tok/s at 2,048 tokens beside it)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "ms_per_step_sd": round(statistics.stdev(ms), 4) if len(ms) > 1 else 0.0,
        "repetitions": a.reps, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if a.dtype == "bfloat16" else "fp32", "data": "synthetic token ids, random N(0, 0.02) weights",
        "config": {"model": NAMES[a.shapes], "layers": cfg.num_hidden_layers, "layers_of_model": MODEL["num_hidden_layers"],
                   "hidden": d, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_size, "intermediate": I, "vocab": vocab, "rope_theta": cfg.rope_theta,
                   "rms_norm_eps": cfg.rms_norm_eps, "tied": cfg.tie_word_embeddings, "global_batch": a.batch,
                   "seq_len": a.context, "page_size": eng.page_size, "parallelism": "single GPU",
                   "graph": eng.decode_graphs is not None},
        "reps": {"n": a.reps, "ms_per_step": [round(m, 4) for m in ms], "mean_ms": round(statistics.mean(ms), 4),
                 "sd_ms": round(statistics.stdev(ms), 4) if len(ms) > 1 else 0.0},
        "meta": {"gpu": torch.cuda.get_device_name(0), "commit": source_version(),
                 "date": datetime.datetime.now(datetime.timezone.utc).strftime("%Y-%m-%dT%H:%M:%SZ"),
                 "torch": torch.__version__, "path": "Engine.step + sampling." + ("sample_rows" if a.read_back_first else "greedy_pending")},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK["hbm_gbs"], "unit": "GB/s",
                     "frac": round(achieved / PEAK["hbm_gbs"], 4)},
        "points": points,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
