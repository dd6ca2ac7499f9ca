#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on SmolLM2-1.7B shapes with random weights.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096] [--layers 24]
                    [--shapes smollm2-1.7b|smollm2-360m|llama-3-8b]

A step is one decode step of the whole batch through Engine.step and the device sampler, the
sampled tokens fed back as the next step's input.  The batch is first prefilled (through the same
step function, in portions of 2,048 tokens) so that the last timed step reaches the context length.
Prints one JSON line.  One GPU only: for --gpus > 1 it says so and exits with 2.
"""
import argparse
import json
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
    ap.add_argument("--only", choices=["decode", "prefill"], default=None,
                    help="for profiling: run only the decode steps (after their prefill) or only the 2,048-token prefill")
    ap.add_argument("--no-graph", action="store_true", help="run decode steps without HIP graph replay")
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
    from glassbox_amd.engine.decode_loop import DecodeLoop
    from glassbox_amd.weights import build_model, init_random

    MODEL = SHAPES[a.shapes]
    cfg = config_from_dict(dict(MODEL, num_hidden_layers=a.layers or MODEL["num_hidden_layers"]))
    model = build_model(cfg)
    init_random(model, seed=0, dtype=a.dtype, device="cuda:0")
    batches = [a.batch] + ([] if a.no_points else [b for b in (1, 64) if b != a.batch])
    max_tokens = max(max(batches) * (a.context + 64), a.prefill_tokens + 64)
    eng = Engine(model, dtype=a.dtype, max_tokens=max_tokens, max_seqs=max(batches), page_size=16)
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

    # ---- decode
    def decode_run(batch, steps, warmup):
        start = a.context - steps - warmup
        names = [f"d{batch}_{i}" for i in range(batch)]
        prompts = [torch.randint(0, vocab, (start,), generator=g).tolist() for _ in names]
        for at in range(0, start - 1, PREFILL_TOKENS):        # leave the last prompt token for the first decode step
            n = min(PREFILL_TOKENS, start - 1 - at)
            for name, p in zip(names, prompts):
                eng.step([(name, p[at:at + n], [])])
        loop = DecodeLoop(eng, names, [p[-1] for p in prompts], use_graph=not a.no_graph)
        for _ in range(warmup):
            loop.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            loop.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        loop.close()
        for name in names:
            eng.end_request(name)
        mean_ctx = a.context - (steps + 1) / 2
        return dt, mean_ctx

    dt, mean_ctx = decode_run(a.batch, a.steps, a.warmup)
    step_s = dt / a.steps
    value = a.batch / step_s
    bytes_step = weight_bytes + a.batch * mean_ctx * kv_bytes_per_token
    achieved = bytes_step / step_s / 1e9
    points = {}
    if not a.no_points:
        for b in (1, 64):
            if b == a.batch:
                points[f"decode_b{b}"] = round(value, 1)
                continue
            k = max(8, min(a.steps, 32))
            pdt, _ = decode_run(b, k, min(a.warmup, 4))
            points[f"decode_b{b}"] = round(b * k / pdt, 1)

    out = {
        "metric": f"decode tok/s at batch {a.batch}, {NAMES[a.shapes]}, context {a.context} "
                  "(prefill tok/s at 2,048 tokens beside it)",
        "value": round(value, 1), "unit": "tok/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if a.dtype == "bfloat16" else "fp32", "data": "synthetic token ids, random N(0, 0.02) weights",
        "config": {"model": NAMES[a.shapes], "layers": cfg.num_hidden_layers, "layers_of_model": MODEL["num_hidden_layers"],
                   "hidden": d, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                   "head_dim": cfg.head_size, "intermediate": I, "vocab": vocab, "rope_theta": cfg.rope_theta,
                   "rms_norm_eps": cfg.rms_norm_eps, "tied": cfg.tie_word_embeddings, "global_batch": a.batch,
                   "seq_len": a.context, "page_size": eng.page_size, "parallelism": "single GPU",
                   "graph": not a.no_graph},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK["hbm_gbs"], "unit": "GB/s",
                     "frac": round(achieved / PEAK["hbm_gbs"], 4)},
        "points": points,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
