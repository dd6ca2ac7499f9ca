"""Command line in the manner of the reference's `glassbox` and `glassbox-bench`
(crates/glassbox-server/src/main.rs:9-15,71-80; crates/glassbox-bench/src/main.rs:9-15).

Option names and meanings are the reference's where it has them: --model DIR, -n N, --temp,
--top-p, --top-k, --min-p, --repeat-penalty, --seed, --blocks, --budget, --max-seqs,
--no-prefix-cache, --dtype, --out, --label.  Differences: prompts are token ids (--prompt takes
numbers separated by commas or blanks; text and tokenizers are outside this engine), and --dtype
selects bfloat16 or float32 arithmetic rather than a quantized format.
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from typing import List

USAGE = """
  glassbox generate --model DIR --prompt IDS [-n 128] [--dtype bfloat16|float32]
                    [--temp 0] [--top-p 1] [--top-k 0] [--min-p 0] [--repeat-penalty 1] [--seed 0]
                    [--blocks 2048] [--budget 256] [--max-seqs 32] [--no-prefix-cache]
  glassbox batch    --model DIR --prompts FILE [-n 128] ...      (one prompt of ids per line; continuous batching)
  glassbox random   --config FILE.json --out DIR [--seed 0] [--dtype float32|bfloat16] [--norm ones|uniform]
  glassbox bench single --model DIR [--dtype ...] [--label L] [--out FILE]      (pp512 / tg128, as glassbox-bench)
  glassbox bench serve  --model DIR [--dtype ...] [--workload chat|system|long] [--requests N] [--rates R,R,...]
                        [--blocks N] [--budget 512] [--max-seqs 32] [--out FILE]    (requests against the clock)
  glassbox bench kernels [--shapes smollm2-1.7b|smollm2-360m|llama-3-8b] [--rows 1,8,64,...] [--dtype ...] [--out FILE]
                        (each matrix product of a layer alone, as glassbox-bench kernels)
  glassbox replay   --model DIR --dtype D --out DIR --max-tokens N              (same as bin/trace_run)"""


def _ids(text: str) -> List[int]:
    return [int(t) for t in text.replace(",", " ").split()]


def _sampler(a):
    from .sampling import SamplerConfig
    return SamplerConfig(temperature=a.temp, top_k=a.top_k, top_p=a.top_p, min_p=a.min_p,
                         repetition_penalty=a.repeat_penalty, seed=a.seed)


def _add_model(p):
    p.add_argument("--model", required=True)
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "bf16", "float32", "f32", "fp32"])


def _add_sampling(p):
    p.add_argument("-n", type=int, default=128, dest="n")
    p.add_argument("--temp", type=float, default=0.0)
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--top-k", type=int, default=0)
    p.add_argument("--min-p", type=float, default=0.0)
    p.add_argument("--repeat-penalty", type=float, default=1.0)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--stop", default="", help="token ids that end a reply")


def _add_serving(p):
    p.add_argument("--blocks", type=int, default=2048, help="pages of the cache (16 tokens each)")
    p.add_argument("--budget", type=int, default=256, help="most tokens in one step")
    p.add_argument("--max-seqs", type=int, default=32)
    p.add_argument("--no-prefix-cache", action="store_true")


def _engine(a, blocks=None):
    from .engine import Engine
    t0 = time.time()
    eng = Engine(a.model, dtype=a.dtype, max_tokens=(blocks or a.blocks) * 16, max_seqs=getattr(a, "max_seqs", 32),
                 prefix_caching=not getattr(a, "no_prefix_cache", True))
    print(f"loaded {eng.model.config.num_hidden_layers if hasattr(eng.model.config, 'num_hidden_layers') else len(eng.model.blocks)}"
          f" layers, {eng.model.weight_bytes() / 1e6:.0f} MB of weights in {time.time() - t0:.1f}s", file=sys.stderr)
    return eng


def cmd_generate(a) -> int:
    import torch
    from .engine import Generator
    from .sampling import Sampler
    prompt = _ids(a.prompt)
    if not prompt:
        print("the prompt holds no token ids", file=sys.stderr)
        return 2
    # as the reference: a cache of exactly prompt + n + 1 tokens for the one request (main.rs:147)
    eng = _engine(a, blocks=-(-(len(prompt) + a.n + 1) // 16))
    eng.warm_up(len(prompt))     # code loaded, buffers sized, the decode graph captured: the times below are the steps' own
    gen, sampler, stop = Generator(eng), Sampler(_sampler(a)), set(_ids(a.stop))
    torch.cuda.synchronize()
    t0 = time.time()
    logits = gen.feed(prompt)
    torch.cuda.synchronize()
    prefill = time.time() - t0
    t1, out = time.time(), []
    for _ in range(a.n):
        tok = sampler.sample(logits, gen.tokens)
        if tok in stop or len(gen.tokens) + 1 >= gen.capacity():   # main.rs:93
            break
        out.append(tok)
        print(tok, end=" ", flush=True)
        logits = gen.feed([tok])
    torch.cuda.synchronize()
    secs = time.time() - t1
    print()
    print(f"prefill {len(prompt)} tokens: {len(prompt) / prefill:.1f} tok/s; decode {len(out)} tokens: "
          f"{len(out) / max(secs, 1e-9):.1f} tok/s", file=sys.stderr)
    return 0


def cmd_batch(a) -> int:
    from .engine import generate
    with open(a.prompts) as fh:
        prompts = [_ids(line) for line in fh if line.strip()]
    eng = _engine(a)
    eng.warm_up(min(a.budget, 64))
    t0 = time.time()
    outs, sched = generate(eng, prompts, a.n, _sampler(a), _ids(a.stop), a.budget, a.max_seqs, return_scheduler=True)
    secs = time.time() - t0
    for o in outs:
        print(" ".join(map(str, o)))
    m = sched.metrics
    print(f"{m['requests_finished']} requests, {m['generated_tokens']} tokens in {secs:.2f}s "
          f"({m['generated_tokens'] / secs:.1f} tok/s), {m['steps']} steps, {m['preemptions']} preemptions, "
          f"{m['prefix_hit_tokens']} prompt tokens reused", file=sys.stderr)
    return 0


def cmd_random(a) -> int:
    import torch
    from .config import config_from_dict
    from .weights import write_random_model
    with open(a.config) as fh:
        cfg = config_from_dict(json.load(fh))
    write_random_model(cfg, a.out, a.seed, norm_init=a.norm,
                       dtype=torch.float32 if a.dtype in ("float32", "f32", "fp32") else torch.bfloat16)
    print(f"wrote {a.out}/config.json and {a.out}/model.safetensors", file=sys.stderr)
    return 0


def cmd_bench_single(a) -> int:
    """pp512 / tg128 as crates/glassbox-bench/src/main.rs:72-96: a 512-token prompt in one step; 128
    single-token steps from an empty cache; three timed repetitions after a warm-up."""
    import statistics
    import torch
    from .engine import Engine, Generator
    from .sampling import greedy_pending
    pp, tg, reps = 512, 128, 3
    eng = Engine(a.model, dtype=a.dtype, max_tokens=pp + tg + 64, max_seqs=2)
    vocab = eng.model.vocab_size
    prompt = [(i * 7919 + 13) % vocab for i in range(pp)]   # bench main.rs:74
    pps, tgs = [], []
    for rep in range(reps + 1):
        g = Generator(eng, "pp")
        torch.cuda.synchronize(); t = time.time()
        g.feed(prompt)
        torch.cuda.synchronize(); p = pp / (time.time() - t)
        g.close()
        g = Generator(eng, "tg")
        torch.cuda.synchronize(); t = time.time()
        tok = 1
        for _ in range(tg):
            logits = g.feed([tok])
            tok = greedy_pending(logits.reshape(1, -1))[0]   # stays on the device for the next step (as in greedy())
        torch.cuda.synchronize(); d = tg / (time.time() - t)
        g.close()
        if rep > 0:
            pps.append(p); tgs.append(d)
    res = {"engine": "glassbox_amd", "label": a.label or a.model, "model": a.model, "dtype": a.dtype,
           "weight_mb": eng.model.weight_bytes() / 1e6, "pp512_tok_s": statistics.mean(pps),
           "pp512_sd": statistics.pstdev(pps), "tg128_tok_s": statistics.mean(tgs), "tg128_sd": statistics.pstdev(tgs),
           "meta": {"gpu": torch.cuda.get_device_name(0), "date": time.strftime("%Y-%m-%dT%H:%M:%SZ", time.gmtime())}}
    text = json.dumps(res, indent=2)
    if a.out:
        with open(a.out, "w") as fh:
            fh.write(text + "\n")
    else:
        print(text)
    return 0


def _quantile(values, p):
    v = sorted(values)
    return v[round((len(v) - 1) * p)] if v else 0.0


def _serve_run(eng, budget, max_seqs, prompts, outputs, rate):
    """One load through the scheduler in real time (crates/glassbox-bench/src/main.rs:241-288): exponential gaps
    between arrivals at ``rate`` requests a second (all at once when the rate is infinite), greedy replies of
    the given lengths."""
    import math
    from .engine.scheduler import Scheduler, SchedulerConfig
    from .sampling import Rng
    rng, t, times = Rng(42), 0.0, []
    for _ in prompts:
        t += 0.0 if math.isinf(rate) else -math.log(1.0 - rng.next_f32()) / rate
        times.append(t)
    s = Scheduler(eng, SchedulerConfig(token_budget=budget, max_seqs=max_seqs))
    t0, nxt = time.perf_counter(), 0
    while nxt < len(times) or not s.is_idle():
        now = time.perf_counter() - t0
        while nxt < len(times) and times[nxt] <= now:
            s.submit(prompts[nxt], outputs[nxt], arrival=t0 + times[nxt])
            nxt += 1
        if s.is_idle():
            time.sleep(max(0.0, times[nxt] - now))
            continue
        s.step()
    import torch
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    m = s.metrics
    return {"rate_rps": None if math.isinf(rate) else rate, "requests": len(prompts), "wall_s": wall,
            "throughput_tok_s": m["generated_tokens"] / wall,
            "total_tok_s": (m["generated_tokens"] + m["prompt_tokens"] - m["prefix_hit_tokens"]) / wall,
            "ttft_p50_s": _quantile(s.ttft, 0.5), "ttft_p99_s": _quantile(s.ttft, 0.99),
            "itl_p50_s": _quantile(s.itl, 0.5), "itl_p99_s": _quantile(s.itl, 0.99),
            "prefix_hit_tokens": m["prefix_hit_tokens"], "prompt_tokens": m["prompt_tokens"],
            "preemptions": m["preemptions"], "steps": m["steps"],
            "mean_batch_tokens": m["batch_tokens"] / max(1, m["steps"])}


def serve_load(workload: str, n: int, vocab: int):
    """Prompts and reply lengths of a serving load, as seeded random token ids.  ``chat`` and ``system`` are the
    reference's two loads (crates/glassbox-bench/src/main.rs:296-318): prompts of 32-320 tokens with replies of
    32-256; a 384-token prompt that every request shares, 16-64 tokens of its own and replies of 16-64.  ``long``
    has prompts of 32-2048 tokens and replies of 32-256, every other request starting with one 384-token prefix."""
    from .sampling import Rng
    ids, lens = Rng(7), Rng(9)
    toks = lambda k: [int(ids.next_f32() * vocab) for _ in range(k)]
    span = lambda lo, width: lo + int(lens.next_f32() * width)
    if workload == "chat":
        prompts = [toks(span(32, 288)) for _ in range(n)]
        return prompts, [span(32, 224) for _ in range(n)]
    if workload == "system":
        system = toks(384)
        prompts = [system + toks(span(16, 48)) for _ in range(n)]
        return prompts, [span(16, 48) for _ in range(n)]
    if workload == "long":
        system, prompts = toks(384), []
        for i in range(n):
            k = span(32, 2017)
            prompts.append((system + toks(max(1, k - 384))) if i % 2 else toks(k))
        return prompts, [span(32, 225) for _ in range(n)]
    raise ValueError(f"no serving load is called {workload!r}")


def cmd_bench_serve(a) -> int:
    """Requests that arrive against the clock, through the scheduler (crates/glassbox-bench/src/main.rs:290-371):
    throughput, time to the first token and between tokens, with and without the prefix cache where prompts
    share a beginning.  A warm-up pass of a few requests comes first, untimed."""
    import torch
    from .engine import Engine
    rates = [float(r) for r in a.rates.replace(",", " ").split()]
    runs = []
    modes = [("prefix cache", True), ("no prefix cache", False)] if a.workload != "chat" else [("continuous batching", False)]
    for name, prefix in modes:
        for rate in rates:
            # a cache of its own for every run, as the reference builds a scheduler for each (main.rs:245): idle
            # pages keep their prefixes, and a run must not find those of the run before
            eng = Engine(a.model, dtype=a.dtype, max_tokens=a.blocks * 16, max_seqs=a.max_seqs, prefix_caching=prefix)
            vocab = eng.model.vocab_size
            prompts, outputs = serve_load(a.workload, a.requests, vocab)
            warm = [[(i * 7919 + 13 + j) % vocab for i in range(k)] for j, k in enumerate((700, 40, 300, 90))]
            _serve_run(eng, a.budget, a.max_seqs, warm, [8] * len(warm), float("inf"))
            r = _serve_run(eng, a.budget, a.max_seqs, prompts, outputs, rate)
            print(f"{name:20} {rate:5} req/s: {r['throughput_tok_s']:.0f} tok/s, TTFT p50 {r['ttft_p50_s']:.3f}s "
                  f"p99 {r['ttft_p99_s']:.3f}s, ITL p50 {r['itl_p50_s'] * 1e3:.2f}ms, {r['prefix_hit_tokens']} prompt "
                  f"tokens reused, {r['preemptions']} preemptions", file=sys.stderr)
            runs.append({"workload": a.workload, "mode": name, "result": r})
            del eng
    res = {"engine": "glassbox_amd", "model": a.model, "dtype": a.dtype, "token_budget": a.budget,
           "max_seqs": a.max_seqs, "blocks": a.blocks, "runs": runs,
           "meta": {"gpu": torch.cuda.get_device_name(0), "date": time.strftime("%Y-%m-%dT%H:%M:%SZ", time.gmtime())}}
    text = json.dumps(res, indent=2)
    if a.out:
        with open(a.out, "w") as fh:
            fh.write(text + "\n")
    else:
        print(text)
    return 0


KERNEL_SHAPES = {   # hidden, intermediate, query heads, kv heads, head size, vocabulary
    "smollm2-1.7b": (2048, 8192, 32, 32, 64, 49152),
    "smollm2-360m": (960, 2560, 15, 5, 64, 49152),
    "llama-3-8b": (4096, 14336, 32, 8, 128, 128256),
}


def cmd_bench_kernels(a) -> int:
    """The matrix products of one layer and of the head, each alone, at several numbers of rows: time, bytes of
    weights a second and floating-point operations a second, as ``glassbox-bench kernels`` prints for the
    reference's matmul (crates/glassbox-bench/src/main.rs:509-536).  Every product runs as the engine runs it
    (bfloat16: with the workspace that lets it divide k; the feed-forward's first product with its SiLU-multiply
    epilogue, the projections that end a part adding into the 32-bit residual).  The weights are rotated through
    copies of more than 512 MB in all, so that no launch finds them in a cache, and the launches are replayed from
    a HIP graph, so that short kernels are not timed at the pace of their launches."""
    import torch
    from . import ops
    from .weights import compute_dtype
    dt = compute_dtype(a.dtype)
    d, inter, nh, nkv, hd, vocab = KERNEL_SHAPES[a.shapes]
    rows_list = [int(r) for r in a.rows.replace(",", " ").split()]
    products = [("qkv", (nh + 2 * nkv) * hd, d, "store"), ("o", d, nh * hd, "add"), ("gate_up", 2 * inter, d, "silu"),
                ("down", d, inter, "add"), ("head", vocab, d, "f32")]
    dev = torch.device("cuda:0")
    results = []
    print(f"{'product':8} {'N':>6} {'K':>6} {'rows':>5} {'us':>9} {'GB/s':>8} {'TFLOP/s':>8}")
    for name, n_out, k, mode in products:
        w_bytes = n_out * k * (2 if dt == torch.bfloat16 else 4)
        copies = max(2, -(-(512 << 20) // w_bytes))
        ws = [(torch.randn(n_out, k, device=dev) * 0.02).to(dt) for _ in range(copies)]
        for m in rows_list:
            x = (torch.randn(m, k, device=dev) * 0.5).to(dt)
            silu = mode == "silu" and dt == torch.bfloat16
            out_cols = n_out // 2 if silu else n_out
            out = torch.zeros(m, out_cols, device=dev, dtype=torch.float32 if mode in ("add", "f32") else dt)
            floats = ops.gemm_split_floats(m, n_out, k) if dt == torch.bfloat16 and m > 16 else 0
            work = torch.empty(floats, device=dev, dtype=torch.float32) if floats else None

            def run(i):
                ops.gemm(x, ws[i % copies], out, accumulate=mode == "add", silu_mul=silu, workspace=work)
            for i in range(3):
                run(i)
            # the launches of a round are replayed from a graph: issued one by one from here, short kernels would be
            # timed at the pace of their launches
            iters = int(min(64, max(4, 2e11 / (2.0 * n_out * k * max(m, 64)))))
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(iters):
                    run(i)
            graph.replay()
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            start.record()
            for _ in range(3):
                graph.replay()
            end.record()
            torch.cuda.synchronize()
            iters *= 3
            us = start.elapsed_time(end) * 1e3 / iters
            res = {"product": name, "n": n_out, "k": k, "rows": m, "us": us, "weight_gb_s": w_bytes / us / 1e3,
                   "tflop_s": 2.0 * n_out * k * m / us / 1e6}
            results.append(res)
            print(f"{name:8} {n_out:6} {k:6} {m:5} {us:9.1f} {res['weight_gb_s']:8.0f} {res['tflop_s']:8.1f}", flush=True)
        del ws
    if a.out:
        with open(a.out, "w") as fh:
            json.dump({"engine": "glassbox_amd", "shapes": a.shapes, "dtype": a.dtype, "results": results,
                       "meta": {"gpu": torch.cuda.get_device_name(0),
                                "date": time.strftime("%Y-%m-%dT%H:%M:%SZ", time.gmtime())}}, fh, indent=2)
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="glassbox", usage=USAGE)
    sub = ap.add_subparsers(dest="cmd")
    g = sub.add_parser("generate"); _add_model(g); _add_sampling(g); _add_serving(g)
    g.add_argument("--prompt", required=True, help="token ids, separated by commas or blanks")
    b = sub.add_parser("batch"); _add_model(b); _add_sampling(b); _add_serving(b)
    b.add_argument("--prompts", required=True)
    r = sub.add_parser("random")
    r.add_argument("--config", required=True); r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=0); r.add_argument("--dtype", default="float32")
    r.add_argument("--norm", default="ones", choices=["ones", "uniform"])
    be = sub.add_parser("bench")
    bsub = be.add_subparsers(dest="bench_cmd")
    bs = bsub.add_parser("single"); _add_model(bs)
    bs.add_argument("--label", default=None); bs.add_argument("--out", default=None)
    bv = bsub.add_parser("serve"); _add_model(bv)
    bv.add_argument("--workload", default="chat", choices=["chat", "system", "long"])
    bv.add_argument("--requests", type=int, default=48)
    bv.add_argument("--rates", default="inf", help="requests a second, several separated by commas; inf = all at once")
    bv.add_argument("--blocks", type=int, default=4096); bv.add_argument("--budget", type=int, default=512)
    bv.add_argument("--max-seqs", type=int, default=32); bv.add_argument("--out", default=None)
    bk = bsub.add_parser("kernels")
    bk.add_argument("--shapes", default="smollm2-1.7b", choices=sorted(KERNEL_SHAPES))
    bk.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "bf16", "float32", "f32", "fp32"])
    bk.add_argument("--rows", default="1,8,64,128,512,2048", help="numbers of rows, separated by commas")
    bk.add_argument("--out", default=None)
    rp = sub.add_parser("replay"); _add_model(rp)
    rp.add_argument("--out", required=True); rp.add_argument("--max-tokens", type=int, required=True)
    a = ap.parse_args(argv)
    if a.cmd == "generate":
        return cmd_generate(a)
    if a.cmd == "batch":
        return cmd_batch(a)
    if a.cmd == "random":
        return cmd_random(a)
    if a.cmd == "bench" and a.bench_cmd == "single":
        return cmd_bench_single(a)
    if a.cmd == "bench" and a.bench_cmd == "serve":
        return cmd_bench_serve(a)
    if a.cmd == "bench" and a.bench_cmd == "kernels":
        return cmd_bench_kernels(a)
    if a.cmd == "replay":
        import os
        import subprocess
        script = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
        dt = "float32" if a.dtype in ("float32", "f32", "fp32") else "bfloat16"
        return subprocess.call([sys.executable, script, "--model", a.model, "--dtype", dt, "--out", a.out,
                                "--max-tokens", str(a.max_tokens)])
    print(USAGE, file=sys.stderr)
    return 2
