"""The engine against the plain implementation under every way of cutting requests into steps:
whole, last 32 tokens one by one, portions of changing size, and mixed batches with so few pages
that they are used again; in 32-bit and in bfloat16."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers

pytestmark = pytest.mark.gpu

# 32-bit: 1e-4 absolute, the stated target of the engine.  bfloat16: against the plain implementation on the
# weights as the engine holds them (rounded), within twice the error of the engine with plain kernels
# (helpers.Bf16Bound), which is itself within 1.5e-2 of the largest logit.
REQUESTS = {
    "A": {"a0": 5, "a1": 17, "a2": 49, "a3": 128, "a4": 70, "a5": 33},
    "B": {"b0": 1, "b1": 33, "b2": 64, "b3": 94, "b4": 200, "b5": 40},
    "C": {"c0": 3, "c1": 47, "c2": 130, "c3": 65, "c4": 257},
    "D": {"d0": 2, "d1": 31, "d2": 150, "d3": 64, "d4": 301},
    "E": {"e0": 4, "e1": 35, "e2": 96, "e3": 161, "e4": 48},
}
# more requests than are live at once, so that finished requests' pages are handed out again
MORE = {
    "A": {"a6": 100, "a7": 60, "a8": 128, "a9": 20, "a10": 81},
    "B": {"b6": 150, "b7": 17, "b8": 256, "b9": 77},
    "C": {"c5": 90, "c6": 33, "c7": 200, "c8": 16, "c9": 129},
    "D": {"d5": 70, "d6": 129, "d7": 18, "d8": 260},
    "E": {"e5": 66, "e6": 19, "e7": 180, "e8": 97},
}


def make_requests_det(name, more=False):
    vocab = helpers.TINY[name]["vocab_size"]
    lengths = dict(REQUESTS[name], **(MORE[name] if more else {}))
    return {rid: helpers.random_tokens(vocab, n, seed=100 * ord(name) + i)
            for i, (rid, n) in enumerate(lengths.items())}


def check(folder, requests, got, dtype, what, tol):
    for rid, toks in requests.items():
        want = helpers.oracle(folder, toks, dtype)
        assert got[rid].shape == want.shape, f"{what} {rid}: shape {got[rid].shape} vs {want.shape}"
        bad = helpers.first_bad(got[rid], want, tol)
        assert bad is None, (f"{what}, request {rid} ({len(toks)} tokens), {dtype}: first wrong position {bad[0]} "
                             f"(page offset {bad[0] % 16}), max abs error {bad[1]:.3e}, allowed {tol:.3e}")


def tolerance(bf16_bound, folder, requests, dtype, page_size=16):
    return helpers.TOL_F32 if dtype == "float32" else bf16_bound.get(folder, requests, page_size)


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
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
@pytest.mark.parametrize("mode", ["whole", "tail32", "chunks"])
def test_single_request_splits(engines, model_dirs, bf16_bound, name, dtype, mode):
    folder = model_dirs.get(name)
    requests = make_requests_det(name)
    steps = {"whole": helpers.schedule_whole, "tail32": helpers.schedule_tail,
             "chunks": helpers.schedule_chunks}[mode](requests)
    eng = engines(name, dtype)
    got = helpers.replay(eng, steps)
    check(folder, requests, got, dtype, mode, tolerance(bf16_bound, folder, requests, dtype))
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_mixed_batches_with_page_reuse(model_dirs, bf16_bound, name, dtype):
    from glassbox_amd.engine import Engine
    folder = model_dirs.get(name)
    requests = make_requests_det(name, more=True)
    for seed in (0, 1):
        steps, peak = helpers.schedule_mixed(requests, seed=seed)
        eng = Engine(folder, dtype=dtype, max_tokens=peak, max_seqs=4)   # exactly as many pages as are held at the peak
        got = helpers.replay(eng, steps)
        check(folder, requests, got, dtype, f"mixed(seed {seed}, pool {peak})", tolerance(bf16_bound, folder, requests, dtype))
        eng.cache.check_invariants()
        assert eng.cache.used_pages() == 0
        assert sum(len(t) for t in requests.values()) > peak, "the schedule did not reuse pages"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_shared_prefixes_recomputation_and_forks(model_dirs, bf16_bound, name, dtype):
    """What the scheduler does to the cache, step by step and with the logits compared at every position
    (crates/glassbox-server/tests/scheduler.rs:84-186, crates/glassbox-core/src/kv.rs:135-187): requests that share
    a 70-token beginning find its four full pages in the cache and run only the rest; a request that is ended in
    the middle of its prompt and added again (preempted and recomputed) finds its own pages; a request forked in
    the middle of a page gets a copy of that page; and with so few pages that idle pages with a prefix are evicted
    for new ones, a later request with the same beginning recomputes it."""
    from glassbox_amd.engine import Engine
    folder = model_dirs.get(name)
    vocab = helpers.TINY[name]["vocab_size"]
    toks = lambda n, seed: helpers.random_tokens(vocab, n, seed=seed)
    prefix = toks(70, 900)
    seqs = {"s0": prefix + toks(21, 901), "s1": prefix + toks(33, 902), "s2": prefix + toks(5, 903),
            "re": toks(75, 904), "parent": toks(37, 905) + toks(20, 906), "child": toks(37, 905) + toks(26, 907),
            "big": toks(150, 908), "s3": prefix + toks(12, 909)}
    tol = tolerance(bf16_bound, folder, seqs, dtype)
    pool = 16 * 16                      # sixteen pages: "big" alone takes ten of them
    eng = Engine(folder, dtype=dtype, max_tokens=pool, max_seqs=4, prefix_caching=True)
    assert eng.cache.share_prefixes
    seen = {}

    def run(entries, what):
        """entries: (request, first position, count, positions wanted).  Compares the wanted rows."""
        logits = eng.step([(r, seqs[r][at:at + n], [p - at for p in want]) for r, at, n, want in entries]).float().cpu().numpy()
        row = 0
        for r, at, n, want in entries:
            ref = helpers.oracle(folder, seqs[r], dtype)
            for p in want:
                err = float(np.abs(logits[row] - ref[p]).max())
                assert err <= tol, f"{what}: request {r}, position {p} (page offset {p % 16}): error {err:.3e}, allowed {tol:.3e}"
                seen.setdefault(r, set()).add(p)
                row += 1
        assert row == logits.shape[0]

    every = lambda at, n: list(range(at, at + n))
    # the first request computes the shared beginning; the second finds it while the first still runs
    assert eng.add_request("s0", seqs["s0"]) == 0
    run([("s0", 0, 80, every(0, 80))], "first request")
    assert eng.add_request("s1", seqs["s1"]) == 64
    run([("s1", 64, 20, every(64, 20)), ("s0", 80, 1, [80])], "a shared beginning beside a single token")
    run([("s1", 84, 19, every(84, 19)), ("s0", 81, 10, every(81, 10))], "both go on")
    eng.end_request("s0")
    # its pages stay in the cache without an owner: the third request takes them back
    assert eng.add_request("s2", seqs["s2"]) == 64
    run([("s2", 64, 11, every(64, 11))], "a beginning found among idle pages")
    eng.end_request("s1"); eng.end_request("s2")
    # preempt and recompute: ended after 40 tokens (two full pages were hashed), added again, finds them
    eng.add_request("re", seqs["re"])
    run([("re", 0, 40, every(0, 40))], "before the preemption")
    eng.end_request("re")
    assert eng.add_request("re", seqs["re"]) == 32
    run([("re", 32, 30, every(32, 30))], "recomputed after a preemption")
    # a fork in the middle of the third page: the child writes into a copy, the parent into the page itself
    eng.add_request("parent")
    run([("parent", 0, 37, every(0, 37)), ("re", 62, 2, [62, 63])], "the parent's first tokens")
    eng.fork_request("parent", "child")
    run([("child", 37, 9, every(37, 9)), ("parent", 37, 1, [37])], "parent and child after the fork")
    run([("parent", 38, 19, every(38, 19)), ("child", 46, 17, every(46, 17)), ("re", 64, 11, every(64, 11))],
        "parent, child and the recomputed request")
    for r in ("parent", "child", "re"):
        eng.end_request(r)
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0
    # a long request needs pages that idle pages with prefixes hold: the oldest of those are evicted
    assert eng.cache.free_pages() == 16
    run([("big", 0, 150, every(0, 150))], "a request that evicts idle pages")
    reused = eng.add_request("s3", seqs["s3"])
    assert reused < 64, "the beginning's first pages were the oldest idle ones and must have been evicted"
    run([("s3", reused, 82 - reused, every(reused, 82 - reused))], "after the eviction")
    eng.end_request("big"); eng.end_request("s3")
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0
    assert seen["s1"] == set(range(64, 103)) and seen["child"] == set(range(37, 63)) and seen["re"] >= set(range(0, 75))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_sharp_attention_shows_a_wrong_key(model_dirs, bf16_bound, name, dtype):
    """With small random weights every softmax is nearly flat and one wrong key among a hundred changes little.  Here
    the query and key projections are scaled so that scores spread over several units and a few keys carry a row's
    attention: mixed steps over an exact-fit pool, and a request cut at every page's edge, must still give the plain
    implementation's logits.  (The test checks first that attention is sharp: the largest probability of a late token
    is many times the uniform one.)"""
    import math
    import torch
    from plain import llama as plain_llama
    from glassbox_amd.engine import Engine
    folder = model_dirs.get(name, sharp=8.0)
    cfg, w = plain_llama.load_folder(folder)
    requests = make_requests_det(name, more=True)
    # how sharp: the first layer's attention of the longest request's last token
    toks = max(requests.values(), key=len)
    x = w["model.embed_tokens.weight"].double()[torch.tensor(toks)]
    h = plain_llama.rms_norm(x, w["model.layers.0.input_layernorm.weight"].double(), cfg["rms_norm_eps"])
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    q = plain_llama.rope((h @ w["model.layers.0.self_attn.q_proj.weight"].double().T).reshape(len(toks), nh, hd), range(len(toks)), cfg["rope_theta"])
    k = plain_llama.rope((h @ w["model.layers.0.self_attn.k_proj.weight"].double().T).reshape(len(toks), nkv, hd), range(len(toks)), cfg["rope_theta"])
    prob = torch.softmax((k[:, 0, :] @ q[-1, 0, :]) / math.sqrt(hd), 0)
    assert prob.max().item() > 10.0 / len(toks), f"attention is not sharp: largest probability {prob.max().item():.3f} over {len(toks)} keys"
    # scores of several units carry bfloat16's rounding of queries and keys into the probabilities: the plain kernels'
    # own error is 2 to 4e-2 here (measured), four times that of the flat model; a wrong key would cost tenths
    tol = helpers.TOL_F32 if dtype == "float32" else bf16_bound.get(folder, requests, plain_rel=8e-2)
    steps, peak = helpers.schedule_mixed(requests, seed=7)
    eng = Engine(folder, dtype=dtype, max_tokens=peak, max_seqs=4)
    got = helpers.replay(eng, steps)
    check(folder, requests, got, dtype, f"sharp attention, mixed (pool {peak})", tol)
    got = helpers.replay(eng, helpers.schedule_chunks(make_requests_det(name), sizes=(16, 15, 17, 1, 32, 31, 2)))
    check(folder, make_requests_det(name), got, dtype, "sharp attention, portions that end at and beside page edges", tol)
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page_size", [("B", 32), ("D", 64), ("C", 48)])
def test_other_page_sizes(model_dirs, bf16_bound, name, page_size, dtype):
    """Pages of 32 and 64 tokens through the whole engine (the tuned attention kernels take powers of two), and of
    48, which they do not: those layers take the plain attention kernel.  Mixed steps over a pool that is used again."""
    from glassbox_amd.engine import Engine
    folder = model_dirs.get(name)
    requests = make_requests_det(name, more=True)
    steps, _ = helpers.schedule_mixed(requests, seed=2)
    # the pool: what live requests hold at the worst moment, each rounded up to whole pages
    eng = Engine(folder, dtype=dtype, max_tokens=4 * (-(-max(len(t) for t in requests.values()) // page_size) * page_size),
                 max_seqs=4, page_size=page_size)
    got = helpers.replay(eng, steps)
    check(folder, requests, got, dtype, f"pages of {page_size}", tolerance(bf16_bound, folder, requests, dtype))
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0
    got = helpers.replay(eng, helpers.schedule_tail(make_requests_det(name)))
    check(folder, make_requests_det(name), got, dtype, f"pages of {page_size}, last tokens one by one",
          tolerance(bf16_bound, folder, requests, dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_real_width(engines, model_dirs, bf16_bound, dtype):
    """Two layers as wide as SmolLM2-360M's: the tiled products run many k-steps, prompt attention pairs
    blocks of 32 tokens over dozens of pages, and a request of 700 tokens is cut in every way."""
    folder = model_dirs.get("M")
    vocab = helpers.TINY["M"]["vocab_size"]
    requests = {"m0": helpers.random_tokens(vocab, 700, seed=31), "m1": helpers.random_tokens(vocab, 129, seed=32)}
    eng = engines("M", dtype, max_tokens=2048)
    tol = tolerance(bf16_bound, folder, requests, dtype)
    for mode, make in (("whole", helpers.schedule_whole), ("tail32", helpers.schedule_tail),
                       ("chunks", lambda r: helpers.schedule_chunks(r, sizes=(200, 2, 131, 64, 33, 300)))):
        got = helpers.replay(eng, make(requests))
        check(folder, requests, got, dtype, mode, tol)
    steps, peak = helpers.schedule_mixed(requests, seed=3, live=2)
    got = helpers.replay(eng, steps)
    check(folder, requests, got, dtype, "mixed", tol)
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_layer_of_the_benchmark_widths(engines, model_dirs, bf16_bound, dtype):
    """One layer as wide as SmolLM2-1.7B's, the shapes of the benchmark: a prompt of 2,100 tokens whole (the
    products with 256 x 256 tiles and operands loaded straight into LDS, their slices of k in the down
    projection), in portions of many sizes, with its last tokens one by one, and mixed with a shorter request."""
    folder = model_dirs.get("W")
    vocab = helpers.TINY["W"]["vocab_size"]
    requests = {"w0": helpers.random_tokens(vocab, 2100, seed=51), "w1": helpers.random_tokens(vocab, 300, seed=52)}
    eng = engines("W", dtype, max_tokens=4096)
    tol = tolerance(bf16_bound, folder, requests, dtype)
    for mode, make in (("whole", helpers.schedule_whole), ("tail32", helpers.schedule_tail),
                       ("chunks", lambda r: helpers.schedule_chunks(r, sizes=(1030, 2, 512, 129, 64, 300)))):
        got = helpers.replay(eng, make(requests))
        check(folder, requests, got, dtype, mode, tol)
    steps, peak = helpers.schedule_mixed(requests, seed=5, live=2)
    got = helpers.replay(eng, steps)
    check(folder, requests, got, dtype, "mixed", tol)
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(engines, model_dirs, bf16_bound, dtype):
    folder = model_dirs.get("C")
    requests = {"long": helpers.random_tokens(helpers.TINY["C"]["vocab_size"], 300, seed=9)}
    steps = helpers.schedule_tail(requests, tail=290)
    got = helpers.replay(engines("C", dtype), steps)
    check(folder, requests, got, dtype, "long decoding", tolerance(bf16_bound, folder, requests, dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens(engines, model_dirs, bf16_bound, name, dtype):
    folder = model_dirs.get(name)
    requests = {"first": helpers.random_tokens(helpers.TINY[name]["vocab_size"], 4, seed=3)}
    got = helpers.replay(engines(name, dtype), helpers.schedule_tail(requests, tail=4))
    # four tokens say little about the plain kernels' error: the bound is that of the longer requests
    check(folder, requests, got, dtype, "first tokens", tolerance(bf16_bound, folder, make_requests_det(name), dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_dirs, bf16_bound, tmp_path, dtype):
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
    check(folder, requests, got, dtype, "trace_run", tolerance(bf16_bound, folder, requests, dtype))


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at random (head sizes that the matrix-core kernels take and others, heads in groups of
    one to four, widths, feed-forward sizes and vocabularies that are no power of two, one to three layers, tied
    or not): mixed steps over a pool that is used again, in 32-bit and in bfloat16, against the plain
    implementation."""
    import random
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
    steps, peak = helpers.schedule_mixed(requests, seed=seed, live=rng.choice([2, 3, 4]))
    bound = helpers.Bf16Bound()
    for dtype in ("float32", "bfloat16"):
        eng = Engine(folder, dtype=dtype, max_tokens=peak, max_seqs=4)
        got = helpers.replay(eng, steps)
        tol = helpers.TOL_F32 if dtype == "float32" else bound.get(folder, requests)
        for r, toks in requests.items():
            bad = helpers.first_bad(got[r], helpers.oracle(folder, toks, dtype), tol)
            assert bad is None, (f"{cfg_d}, request {r} ({len(toks)} tokens), {dtype}: first wrong position {bad[0]}, "
                                 f"max abs error {bad[1]:.3e}, allowed {tol:.3e}")
        eng.cache.check_invariants()
        assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,count", [("B", 12), ("E", 20), ("D", 40), ("M", 33)])
def test_many_requests_decode_together(model_dirs, bf16_bound, name, count, dtype):
    """Twelve, twenty and forty requests whose last 24 tokens are decoded in the same steps: steps of that many single
    tokens (in bfloat16 replayed from graphs, with filler rows up to the graph's size; the products of 9 to 64 rows
    prepare each other's norms), every position against the plain implementation.  Requests end at different steps, so
    the batch shrinks through every size on the way.  Thirty-three requests on SmolLM2-360M's widths: a k of 960 on
    sixteen waves, workgroups of 8 rows of W, short contexts that attention takes whole with four waves."""
    from glassbox_amd.engine import Engine
    folder = model_dirs.get(name)
    vocab = helpers.TINY[name]["vocab_size"]
    requests = {f"r{i}": helpers.random_tokens(vocab, 30 + (7 * i) % 41, seed=500 + i) for i in range(count)}
    tail = 24
    steps = [{"entries": [(r, t[:len(t) - tail], list(range(len(t) - tail)))], "end": []} for r, t in requests.items()]
    longest = max(len(t) for t in requests.values())
    for k in range(tail + longest):
        entries, end = [], []
        for i, (r, t) in enumerate(requests.items()):
            at = len(t) - tail + k - i % 5          # requests start decoding up to four steps apart
            if len(t) - tail <= at < len(t) and k >= i % 5:
                entries.append((r, [t[at]], [0]))
                if at == len(t) - 1:
                    end.append(r)
        if entries:
            steps.append({"entries": entries, "end": end})
    eng = Engine(folder, dtype=dtype, max_tokens=count * 128, max_seqs=count)
    got = helpers.replay(eng, steps)
    assert max(len(s["entries"]) for s in steps) == count
    if eng.decode_graphs is not None:
        assert eng.decode_graphs.replays > 0
    check(folder, requests, got, dtype, f"{count} requests decoding together", tolerance(bf16_bound, folder, requests, dtype))
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_a_context_of_nine_thousand_tokens(model_dirs, bf16_bound, name, dtype):
    """One request of 9,000 tokens: its prompt in portions of 2,048 (each attending to all the pages before it), a
    portion of 100 tokens behind 7,844 (workgroups share a block pair's keys and a second pass adds their sums),
    then 56 tokens one by one over 560 pages (the context in chunks, a pass that merges them; in bfloat16 from graphs):
    every position against the plain implementation."""
    from glassbox_amd.engine import Engine
    folder = model_dirs.get(name)
    toks = helpers.random_tokens(helpers.TINY[name]["vocab_size"], 9000, seed=77)
    requests = {"long": toks}
    cuts = [0, 2048, 4096, 6144, 7844, 7944, 8944]
    steps = [{"entries": [("long", toks[a:b], list(range(b - a)))], "end": []} for a, b in zip(cuts, cuts[1:])]
    steps += [{"entries": [("long", [toks[i]], [0])], "end": ["long"] if i == 8999 else []} for i in range(8944, 9000)]
    eng = Engine(folder, dtype=dtype, max_tokens=9024, max_seqs=1)
    got = helpers.replay(eng, steps)
    check(folder, requests, got, dtype, "nine thousand tokens", tolerance(bf16_bound, folder, requests, dtype))
    assert eng.cache.used_pages() == 0
