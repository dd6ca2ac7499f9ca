"""The engine against the plain implementation under every way of cutting requests into steps:
whole, last 32 tokens one by one, portions of changing size, and mixed batches with so few pages
that they are used again; in 32-bit and in bfloat16."""
import functools
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers

pytestmark = pytest.mark.gpu

# 32-bit: the stated target of the engine.  bfloat16: operands carry 8 bits, about 4e-3 relative
# per rounding; logits here are of order 0.3, a few dozen roundings deep.
TOL = {"float32": 1e-4, "bfloat16": 2.5e-2}

REQUESTS = {
    "A": {"a0": 5, "a1": 17, "a2": 49, "a3": 128, "a4": 70, "a5": 33},
    "B": {"b0": 1, "b1": 33, "b2": 64, "b3": 94, "b4": 200, "b5": 40},
    "C": {"c0": 3, "c1": 47, "c2": 130, "c3": 65, "c4": 257},
    "D": {"d0": 2, "d1": 31, "d2": 150, "d3": 64, "d4": 301},
}
# more requests than are live at once, so that finished requests' pages are handed out again
MORE = {
    "A": {"a6": 100, "a7": 60, "a8": 128, "a9": 20, "a10": 81},
    "B": {"b6": 150, "b7": 17, "b8": 256, "b9": 77},
    "C": {"c5": 90, "c6": 33, "c7": 200, "c8": 16, "c9": 129},
    "D": {"d5": 70, "d6": 129, "d7": 18, "d8": 260},
}


def make_requests_det(name, more=False):
    vocab = helpers.TINY[name]["vocab_size"]
    lengths = dict(REQUESTS[name], **(MORE[name] if more else {}))
    return {rid: helpers.random_tokens(vocab, n, seed=100 * ord(name) + i)
            for i, (rid, n) in enumerate(lengths.items())}


def check(folder, requests, got, dtype, what, tol=None):
    for rid, toks in requests.items():
        want = helpers.plain_logits(folder, tuple(toks))
        assert got[rid].shape == want.shape, f"{what} {rid}: shape {got[rid].shape} vs {want.shape}"
        bad = helpers.first_bad(got[rid], want, tol or TOL[dtype])
        assert bad is None, (f"{what}, request {rid} ({len(toks)} tokens), {dtype}: first wrong position {bad[0]} "
                             f"(page offset {bad[0] % 16}), max abs error {bad[1]:.3e}")


@pytest.fixture(scope="module")
def engines(model_dirs):
    from glassbox_amd.engine import Engine
    made = {}

    def get(name, dtype, max_tokens=1024):
        key = (name, dtype, max_tokens)
        if key not in made:
            made[key] = Engine(model_dirs.get(name), dtype=dtype, max_tokens=max_tokens, max_seqs=8)
        return made[key]
    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
@pytest.mark.parametrize("mode", ["whole", "tail32", "chunks"])
def test_single_request_splits(engines, model_dirs, name, dtype, mode):
    folder = model_dirs.get(name)
    requests = make_requests_det(name)
    steps = {"whole": helpers.schedule_whole, "tail32": helpers.schedule_tail,
             "chunks": helpers.schedule_chunks}[mode](requests)
    eng = engines(name, dtype)
    got = helpers.replay(eng, steps)
    check(folder, requests, got, dtype, mode)
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_mixed_batches_with_page_reuse(model_dirs, name, dtype):
    from glassbox_amd.engine import Engine
    folder = model_dirs.get(name)
    requests = make_requests_det(name, more=True)
    for seed in (0, 1):
        steps, peak = helpers.schedule_mixed(requests, seed=seed)
        eng = Engine(folder, dtype=dtype, max_tokens=peak, max_seqs=4)   # exactly as many pages as are held at the peak
        got = helpers.replay(eng, steps)
        check(folder, requests, got, dtype, f"mixed(seed {seed}, pool {peak})")
        eng.cache.check_invariants()
        assert eng.cache.used_pages() == 0
        assert sum(len(t) for t in requests.values()) > peak, "the schedule did not reuse pages"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_real_width(engines, model_dirs, dtype):
    """Two layers as wide as SmolLM2-360M's: the tiled products run many k-steps, prompt attention pairs
    blocks of 32 tokens over dozens of pages, and a request of 700 tokens is cut in every way."""
    folder = model_dirs.get("M")
    vocab = helpers.TINY["M"]["vocab_size"]
    requests = {"m0": helpers.random_tokens(vocab, 700, seed=31), "m1": helpers.random_tokens(vocab, 129, seed=32)}
    eng = engines("M", dtype, max_tokens=2048)
    # 32-bit: the same 1e-4.  bfloat16: rounding errors grow with the logits, whose root mean square is
    # 0.63 here against 0.19 to 0.3 in the tiny models (measured: mean error 4.3e-3, largest 3.1e-2, the
    # same at the first position as at the last and the same with the plain kernels): the tolerance
    # keeps its ratio to them
    tol = TOL[dtype] * (0.63 / 0.25 if dtype == "bfloat16" else 1.0)
    check = functools.partial(globals()["check"], tol=tol)
    for mode, make in (("whole", helpers.schedule_whole), ("tail32", helpers.schedule_tail),
                       ("chunks", lambda r: helpers.schedule_chunks(r, sizes=(200, 2, 131, 64, 33, 300)))):
        got = helpers.replay(eng, make(requests))
        check(folder, requests, got, dtype, mode)
    steps, peak = helpers.schedule_mixed(requests, seed=3, live=2)
    got = helpers.replay(eng, steps)
    check(folder, requests, got, dtype, "mixed")
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_of_the_benchmark_widths(engines, model_dirs, dtype):
    """One layer as wide as SmolLM2-1.7B's, the shapes of the benchmark: a prompt of 2,100 tokens whole (the
    products with 256 x 256 tiles and operands loaded straight into LDS, their slices of k in the down
    projection), in portions of many sizes, with its last tokens one by one, and mixed with a shorter request."""
    folder = model_dirs.get("W")
    vocab = helpers.TINY["W"]["vocab_size"]
    requests = {"w0": helpers.random_tokens(vocab, 2100, seed=51), "w1": helpers.random_tokens(vocab, 300, seed=52)}
    eng = engines("W", dtype, max_tokens=4096)
    # bfloat16: as in the test above, the tolerance keeps its ratio to the logits' root mean square
    rms = float(np.sqrt(np.mean(helpers.plain_logits(folder, tuple(requests["w1"])) ** 2)))
    tol = TOL[dtype] * (max(1.0, rms / 0.25) if dtype == "bfloat16" else 1.0)
    check = functools.partial(globals()["check"], tol=tol)
    for mode, make in (("whole", helpers.schedule_whole), ("tail32", helpers.schedule_tail),
                       ("chunks", lambda r: helpers.schedule_chunks(r, sizes=(1030, 2, 512, 129, 64, 300)))):
        got = helpers.replay(eng, make(requests))
        check(folder, requests, got, dtype, mode)
    steps, peak = helpers.schedule_mixed(requests, seed=5, live=2)
    got = helpers.replay(eng, steps)
    check(folder, requests, got, dtype, "mixed")
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(engines, model_dirs, dtype):
    folder = model_dirs.get("C")
    toks = helpers.random_tokens(helpers.TINY["C"]["vocab_size"], 300, seed=9)
    steps = helpers.schedule_tail({"long": toks}, tail=290)
    got = helpers.replay(engines("C", dtype), steps)
    check(folder, {"long": toks}, got, dtype, "long decoding")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens(engines, model_dirs, name, dtype):
    folder = model_dirs.get(name)
    toks = helpers.random_tokens(helpers.TINY[name]["vocab_size"], 4, seed=3)
    got = helpers.replay(engines(name, dtype), helpers.schedule_tail({"first": toks}, tail=4))
    check(folder, {"first": toks}, got, dtype, "first tokens")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_dirs, tmp_path, dtype):
    """The program itself, as a child process: mixed steps over a small pool, files and 'done' lines."""
    folder = model_dirs.get("B")
    requests = make_requests_det("B")
    steps, peak = helpers.schedule_mixed(requests, seed=5)
    out = tmp_path / "out"
    lines = []
    for i, st in enumerate(steps):
        lines.append(json.dumps({"step": i, "end": st["end"],
                                 "entries": [{"id": r, "tokens": t, "want": w} for r, t, w in st["entries"]]}))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(peak)], input="\n".join(lines) + "\n",
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == [w for i in range(len(steps)) for w in ("done", str(i))]
    vocab = helpers.TINY["B"]["vocab_size"]
    got = {}
    for i, st in enumerate(steps):
        data = np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, vocab)
        row = 0
        for r, t, w in st["entries"]:
            got.setdefault(r, []).append(data[row:row + len(w)])
            row += len(w)
        assert row == data.shape[0]
    got = {r: np.concatenate(p, 0) for r, p in got.items()}
    check(folder, requests, got, dtype, "trace_run")


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at random (head sizes that the matrix-core kernels take and others, heads in groups of
    one to four, widths, feed-forward sizes and vocabularies that are no power of two, one to three layers, tied
    or not): mixed steps over a pool that is used again, in 32-bit and in bfloat16, against the plain
    implementation."""
    import random
    from plain import llama as plain_llama
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.engine import Engine
    from glassbox_amd.weights import write_random_model
    rng = random.Random(4000 + seed)
    hd = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 24, 40, 8])
    nkv = rng.choice([1, 2, 3, 5])
    nh = nkv * rng.choice([1, 2, 3, 4])
    vocab = rng.randrange(90, 700)
    cfg_d = dict(architectures=["LlamaForCausalLM"], hidden_size=rng.choice([8, 16, 24]) * rng.randrange(3, 12),
                 intermediate_size=16 * rng.randrange(4, 20), num_hidden_layers=rng.choice([1, 2, 3]),
                 num_attention_heads=nh, num_key_value_heads=nkv, head_dim=hd, vocab_size=vocab,
                 rope_theta=float(rng.choice([10000, 130000, 500000])), rms_norm_eps=rng.choice([1e-5, 1e-6, 3e-5]),
                 tie_word_embeddings=rng.random() < 0.5, max_position_embeddings=1024)
    folder = str(tmp_path / "model")
    write_random_model(config_from_dict(cfg_d), folder, seed, norm_init="uniform", dtype=torch.float32)
    requests = {f"r{i}": helpers.random_tokens(vocab, rng.randrange(1, 260), seed=seed * 10 + i) for i in range(4)}
    cfg, w = plain_llama.load_folder(folder)
    want = {r: plain_llama.forward(w, cfg, list(t), torch.float64).numpy() for r, t in requests.items()}
    steps, peak = helpers.schedule_mixed(requests, seed=seed, live=rng.choice([2, 3, 4]))
    rms = max(float(np.sqrt(np.mean(x ** 2))) for x in want.values())
    for dtype in ("float32", "bfloat16"):
        eng = Engine(folder, dtype=dtype, max_tokens=peak, max_seqs=4)
        got = helpers.replay(eng, steps)
        tol = TOL[dtype] * (max(1.0, rms / 0.25) if dtype == "bfloat16" else 1.0)   # as in the tests above
        for r, toks in requests.items():
            bad = helpers.first_bad(got[r], want[r], tol)
            assert bad is None, (f"{cfg_d}, request {r} ({len(toks)} tokens), {dtype}: first wrong position {bad[0]}, "
                                 f"max abs error {bad[1]:.3e}")
        eng.cache.check_invariants()
        assert eng.cache.used_pages() == 0
