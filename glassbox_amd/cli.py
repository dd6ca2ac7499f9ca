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

USAGE = """usage:
  glassbox generate --model DIR --prompt IDS [-n 128] [--dtype bfloat16|float32]
                    [--temp 0] [--top-p 1] [--top-k 0] [--min-p 0] [--repeat-penalty 1] [--seed 0]
                    [--blocks 2048] [--budget 256] [--max-seqs 32] [--no-prefix-cache]
  glassbox batch    --model DIR --prompts FILE [-n 128] ...      (one prompt of ids per line; continuous batching)
  glassbox random   --config FILE.json --out DIR [--seed 0] [--dtype float32|bfloat16] [--norm ones|uniform]
  glassbox bench single --model DIR [--dtype ...] [--label L] [--out FILE]      (pp512 / tg128, as glassbox-bench)
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
    from .sampling import SamplerConfig, sample_rows
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
            tok = sample_rows(logits.reshape(1, -1), [SamplerConfig()], [0.0])[0][0]
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
    if a.cmd == "replay":
        import os
        import subprocess
        script = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
        dt = "float32" if a.dtype in ("float32", "f32", "fp32") else "bfloat16"
        return subprocess.call([sys.executable, script, "--model", a.model, "--dtype", dt, "--out", a.out,
                                "--max-tokens", str(a.max_tokens)])
    print(USAGE, file=sys.stderr)
    return 2
