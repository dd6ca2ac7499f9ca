"""Schedules that touch the cache in ways the replay schedules do not, at the level of logits and in both
precisions: a block table longer than its request's length (pages kept from a step that found no room), requests
aborted in the middle of their prompts and replies with their pages handed on, a generator truncated into shared and
hashed pages and fed other tokens, stop tokens through the device sampler, more single-token rows than one graph's
skinny products take, and weights loaded again under captured graphs."""
import os
import random

import numpy as np
import pytest
import torch

import helpers
from plain import llama as plain
from test_replay_gpu import check, tolerance
from test_scheduler_gpu import check_records, serve

pytestmark = pytest.mark.gpu


def rows_of(eng, entries):
    """engine.step with every place of every entry wanted; returns {request: rows}."""
    logits = eng.step([(r, t, list(range(len(t)))) for r, t in entries]).float().cpu().numpy()
    out, at = {}, 0
    for r, t in entries:
        out[r] = logits[at:at + len(t)]
        at += len(t)
    return out


def assert_rows(got, folder, full, first, dtype, tol, what):
    want = helpers.oracle(folder, full, dtype)[first:first + got.shape[0]]
    bad = helpers.first_bad(got, want, tol)
    assert bad is None, (f"{what}, {dtype}: first wrong position {first + bad[0]} (page offset {(first + bad[0]) % 16}), "
                         f"error {bad[1]:.3e}, allowed {tol:.3e}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_kept_from_a_step_without_room_do_not_stop_single_token_steps(model_dirs, bf16_bound, dtype):
    """A step's first entry reserves across the edge of the graphs' context bucket, its second finds no room: the
    step raises, the first request keeps the page (by design: nothing was written), and its block table is now longer
    than its length needs.  Single-token steps after that must go on, replayed from graphs, with the right logits."""
    from glassbox_amd.cache import OutOfPages
    from glassbox_amd.engine import Engine
    folder = model_dirs.get("E")
    toks = helpers.random_tokens(helpers.TINY["E"]["vocab_size"], 520, seed=41)
    tol = tolerance(bf16_bound, folder, {"a": toks}, dtype)
    eng = Engine(folder, dtype=dtype, max_tokens=35 * 16, max_seqs=4, graph_decode=True)
    assert eng.decode_graphs is not None
    assert_rows(rows_of(eng, [("a", toks[:500])])["a"], folder, toks, 0, dtype, tol, "the prompt")
    for p in range(500, 503):      # the bucket of 512 tokens: walked, captured, replayed
        assert_rows(rows_of(eng, [("a", toks[p:p + 1])])["a"], folder, toks, p, dtype, tol, "before the failed step")
    with pytest.raises(OutOfPages):
        eng.step([("a", toks[503:513], [9]), ("new", toks[:200], [])])
    sid = eng._ids["a"]
    assert eng.request_len("a") == 503 and len(eng.cache.table(sid)) == 33, "the first entry keeps its reserved page"
    assert not eng.has_request("new")
    replays = eng.decode_graphs.replays
    for p in range(503, 512):
        assert_rows(rows_of(eng, [("a", toks[p:p + 1])])["a"], folder, toks, p, dtype, tol, "after the failed step")
    assert eng.decode_graphs.replays > replays, "the steps after the failed one were not replayed from a graph"
    assert any(bucket > 512 for _, bucket in eng.decode_graphs.shapes), "the longer table needs the next bucket"
    eng.end_request("a")
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_aborts_hand_their_pages_on_and_survivors_keep_their_logits(model_dirs, bf16_bound, name, dtype):
    """crates/glassbox-server/tests/scheduler.rs:125-163 on the device: sixteen requests through a pool of twenty
    pages, every third step a live request is aborted (running ones in the middle of a prompt or a reply, waiting
    ones before their first token), invariants hold after every step, the pages go to the requests behind, and every
    row the scheduler sampled from, of survivors and of aborted requests up to their end, is the plain
    implementation's."""
    from glassbox_amd.engine import Engine
    folder = model_dirs.get(name)
    vocab = helpers.TINY[name]["vocab_size"]
    rng = random.Random(5)
    prompts = [[rng.randrange(vocab) for _ in range(1 + rng.randrange(60))] for _ in range(16)]
    eng = Engine(folder, dtype=dtype, max_tokens=20 * 16, max_seqs=8, prefix_caching=True)
    replies, sched, records = serve(eng, prompts, max_tokens=20, budget=32, max_seqs=8, abort_every=3, abort_seed=1)
    aborted = sched.aborted
    assert aborted["running"] >= 2 and aborted["waiting"] >= 1, aborted
    finishes = [sched.outputs[i].finish for i in sorted(sched.outputs)]
    assert finishes.count("aborted") == aborted["running"] + aborted["waiting"]
    survivors = [i for i, f in enumerate(finishes) if f != "aborted"]
    assert len(survivors) >= 4 and all(len(replies[i]) == 20 for i in survivors)
    assert sum(len(p) + len(r) for p, r in zip(prompts, replies)) > 20 * 16, "the pool was not used twice"
    full = {f"r{i}": p + r for i, (p, r) in enumerate(zip(prompts, replies))}
    tol = helpers.TOL_F32 if dtype == "float32" else bf16_bound.get(folder, full)
    check_records(folder, prompts, replies, records, dtype, tol, "aborts")
    seen = {i for i, _, _ in records}
    assert set(survivors) <= seen
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_a_truncated_generator_is_fed_other_tokens(model_dirs, bf16_bound, name, dtype):
    """``Generator.truncate`` (crates/glassbox-core/src/lib.rs:53-56, kv.rs:237-257) with shared beginnings on and
    single tokens replayed from graphs: cut into the middle of a hashed page and feed other tokens (the rewritten
    page must no longer be found under its old hash), cut at a page's edge, and cut into a page that a forked
    request shares (the generator gets a copy, the twin keeps the page).  Every position against the plain
    implementation."""
    from glassbox_amd.engine import Engine, Generator
    folder = model_dirs.get(name)
    vocab = helpers.TINY[name]["vocab_size"]
    toks = lambda n, seed: helpers.random_tokens(vocab, n, seed=seed)
    X, Y, Z, V, W = toks(40, 1), toks(18, 2), toks(12, 3), toks(14, 4), toks(15, 5)
    seqs = {"x": X, "y": X[:23] + Y, "z": (X[:23] + Y)[:32] + Z, "probe": X + toks(6, 6)}
    seqs["twin"] = seqs["z"] + V
    seqs["w"] = seqs["z"][:37] + W
    tol = tolerance(bf16_bound, folder, seqs, dtype)
    eng = Engine(folder, dtype=dtype, max_tokens=24 * 16, max_seqs=4, prefix_caching=True, graph_decode=True)
    assert eng.cache.share_prefixes and eng.decode_graphs is not None
    g = Generator(eng, name="g")

    def feed(request, full, pieces, what):
        """Feeds ``full[len(request) ...]`` in pieces of the given sizes, every place wanted and compared."""
        at = eng.request_len(request)
        for n in pieces:
            got = rows_of(eng, [(request, full[at:at + n])])[request]
            assert_rows(got, folder, full, at, dtype, tol, f"{what}, {n} tokens from {at}")
            at += n
        if request == "g":
            g.tokens[:] = full[:at]
        return at

    assert feed("g", seqs["x"], [40], "the first forty tokens") == 40
    g.truncate(23)                                   # into the second page, which is full and hashed
    assert eng.request_len("g") == 23 and g.tokens == X[:23]
    assert feed("g", seqs["y"], [2, 1, 1, 1, 1, 1, 1, 10], "after a cut to 23") == 41
    # the second page now holds other tokens: a request with the old beginning finds the first page alone
    assert eng.add_request("probe", seqs["probe"]) == 16
    feed("probe", seqs["probe"], [30], "a request with the old beginning")
    eng.end_request("probe")
    g.truncate(32)                                   # at a page's edge: the third page goes back
    assert len(eng.cache.table(eng._ids["g"])) == 2
    assert feed("g", seqs["z"], [1, 1, 1, 1, 1, 7], "after a cut to 32") == 44
    eng.fork_request("g", "twin")
    g.truncate(37)                                   # into the third page, which the twin shares
    feed("g", seqs["w"], [1], "after a cut into a shared page")            # the generator gets a copy of the page
    feed("twin", seqs["twin"], [1, 1, 1, 11], "the twin goes on in the page itself")
    assert feed("g", seqs["w"], [1, 1, 2, 10], "the generator goes on in its copy") == 52
    assert eng.decode_graphs.replays > 0
    g.close()
    eng.end_request("twin")
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_stop_tokens_end_replies_on_the_device(model_dirs, dtype):
    """``generate(..., stop=...)`` through the device sampler (crates/glassbox-server/src/scheduler.rs:393-399): a reply
    ends before the first stop token, which is neither kept nor counted; the others run to their length."""
    from glassbox_amd import Engine, generate
    folder = model_dirs.get("B")
    cfg, w = helpers._load_rounded(folder) if dtype == "bfloat16" else helpers._load(folder)
    prompts = [helpers.random_tokens(384, n, seed=n) for n in (9, 40, 70, 3)]
    eng = Engine(folder, dtype=dtype, max_tokens=1024, max_seqs=8)
    free = generate(eng, prompts, max_tokens=16, token_budget=16)
    # a token that the first reply reaches at its sixth place or later and not before
    first = free[0]
    at = next(i for i in range(5, 16) if first[i] not in first[:i])
    stop = first[at]
    outs, sched = generate(eng, prompts, max_tokens=16, stop=[stop, 383], token_budget=16, return_scheduler=True)
    for i, (ref, out) in enumerate(zip(free, outs)):
        cut = ref.index(stop) if stop in ref else (ref.index(383) if 383 in ref else 16)
        if 383 in ref[:cut]:
            cut = ref.index(383)
        assert out == ref[:cut], f"prompt {i}: {out} against {ref} cut at {cut}"
        assert sched.outputs[sorted(sched.outputs)[i]].finish == ("stop" if cut < 16 else "length")
    assert outs[0] == first[:at] and len(outs[0]) >= 5
    # and the replies are the plain implementation's greedy ones as far as they go
    for p, out in zip(prompts, outs):
        ref = plain.greedy(w, cfg, p, len(out)) if out else []
        agree = next((i for i, (a, b) in enumerate(zip(out, ref)) if a != b), len(out))
        if agree < len(out):     # two logits within rounding of each other may swap in bfloat16
            logits = plain.forward(w, cfg, list(p) + ref[:agree])[-1]
            top2 = torch.topk(logits, 2).values
            assert (top2[0] - top2[1]).item() < (1e-4 if dtype == "float32" else 1e-2)
    assert sched.metrics["generated_tokens"] == sum(len(o) for o in outs)
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_steps_launched_ahead_of_their_plan_change_nothing(model_dirs, bf16_bound, name, dtype):
    """When every live request decodes greedily the scheduler launches the next step before it has read this one's
    tokens (``SchedulerConfig.run_ahead``).  Replies and finish reasons are those of a scheduler that
    does not; rows that ran ahead were used (most of them) and dropped (a request stopped by a stop token, one
    aborted, requests preempted in a pool of few pages, a request that arrives in the middle and whose prompt runs
    beside rows computed ahead); every row of logits, also of the steps that ran ahead, is the plain
    implementation's; requests that draw with a temperature and a penalty run ahead as well, with the same tokens."""
    from glassbox_amd.engine import Engine, Scheduler, SchedulerConfig
    from glassbox_amd.sampling import SamplerConfig
    folder = model_dirs.get(name)
    vocab = helpers.TINY[name]["vocab_size"]
    prompts = [helpers.random_tokens(vocab, n, seed=200 + n) for n in (9, 40, 70, 3, 25, 17)]
    # free replies first, to find a stop token that the first reply reaches in its middle
    eng = Engine(folder, dtype=dtype, max_tokens=9 * 16, max_seqs=6, prefix_caching=True, graph_decode=True)
    free, _, _ = serve(eng, prompts, max_tokens=20, budget=16, max_seqs=6)
    full = {f"r{i}": p + r for i, (p, r) in enumerate(zip(prompts, free))}
    tol = helpers.TOL_F32 if dtype == "float32" else bf16_bound.get(folder, full)
    first = free[0]
    at = next((i for i in range(4, 20) if first[i] not in first[:i]), None)
    stop = [first[at]] if at is not None else []

    def run(ahead):
        sched = Scheduler(eng, SchedulerConfig(token_budget=16, max_seqs=6, run_ahead=ahead))
        ids = [sched.submit(p, 20, stop=stop) for p in prompts[:5]]
        steps = 0
        while not sched.is_idle():
            sched.step()
            eng.cache.check_invariants()
            steps += 1
            if steps == 9:
                ids.append(sched.submit(prompts[5], 20, stop=stop))     # arrives while the others decode
            if steps == 14:
                sched.abort(ids[1])
        outs = [(sched.outputs[i].tokens, sched.outputs[i].finish) for i in ids]
        assert eng.cache.used_pages() == 0
        return outs, sched

    plain_outs, plain_sched = run(False)
    ahead_outs, ahead_sched = run(True)
    assert ahead_outs == plain_outs
    assert plain_sched.ahead_rows == {"launched": 0, "served": 0}
    rows = ahead_sched.ahead_rows
    assert rows["launched"] >= rows["served"] >= 20, rows    # (launched in vain: for a request that then stopped or was aborted)
    # (the number of steps may differ by a few where the pool is nearly full: the pages of rows that run ahead are
    # taken before the plan looks for room to admit a waiting request, not after)
    for key in ("requests_finished", "generated_tokens"):
        assert ahead_sched.metrics[key] == plain_sched.metrics[key], key
    assert any(f == "stop" for _, f in ahead_outs) or not stop
    assert ahead_outs[1][1] == "aborted"
    # at the level of logits, rows that ran ahead included (serve records them when the reply got that far)
    replies, sched, records = serve(eng, prompts, max_tokens=20, budget=16, max_seqs=6)
    assert replies == free and sched.ahead_rows["served"] >= 20 and sched.metrics["preemptions"] > 0
    check_records(folder, prompts, replies, records, dtype, tol, f"{name}: steps launched ahead")
    # requests that draw, some with a penalty: their steps run ahead too (a row that ran ahead is sampled once the plan
    # has said with which random number), and a seeded run gives the tokens of a scheduler that launches nothing ahead
    drawn = [SamplerConfig(temperature=0.8, top_k=(0, 40)[i % 2], top_p=(1.0, 0.9)[i % 3 == 0],
                           repetition_penalty=(1.0, 1.3)[i % 2], seed=3 + i) for i in range(6)]

    def draw(ahead):
        sched = Scheduler(eng, SchedulerConfig(token_budget=64, max_seqs=6, run_ahead=ahead))
        ids = [sched.submit(p, 14, s) for p, s in zip(prompts, drawn)]
        sched.run()
        assert eng.cache.used_pages() == 0
        return [sched.outputs[i].tokens for i in ids], sched.ahead_rows

    with_ahead, rows = draw(True)
    without, none = draw(False)
    assert rows["served"] >= 20 and none["launched"] == 0, (rows, none)
    assert len({tuple(t) for t in with_ahead}) > 1
    if dtype == "float32":    # (in bfloat16 a row's rounding depends on what else is in its launch, and a draw may tip)
        assert with_ahead == without
    else:
        assert [len(t) for t in with_ahead] == [len(t) for t in without]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,count", [("E", 72), ("M", 96)])
def test_more_than_sixty_four_requests_decode_together(model_dirs, bf16_bound, name, count, dtype):
    """Seventy-two and ninety-six requests whose last twelve tokens are decoded in the same steps: a graph of more
    than 64 rows takes the products that prompt portions take (no skinny kernel, norms by kernels of their own), beside
    attention over that many single tokens.  Requests end three steps apart, so the batch shrinks through 64."""
    from glassbox_amd.engine import Engine
    folder = model_dirs.get(name)
    vocab = helpers.TINY[name]["vocab_size"]
    requests = {f"r{i}": helpers.random_tokens(vocab, 20 + (11 * i) % 37, seed=700 + i) for i in range(count)}
    tail = 12
    steps = []
    names = list(requests)
    for at in range(0, count, 4):     # prompts four at a time
        steps.append({"entries": [(r, requests[r][:-tail], list(range(len(requests[r]) - tail))) for r in names[at:at + 4]],
                      "end": []})
    for k in range(tail + 9):
        entries, end = [], []
        for i, r in enumerate(names):
            t, j = requests[r], k - 3 * (i % 4)      # four groups, three steps apart
            if 0 <= j < tail:
                entries.append((r, [t[len(t) - tail + j]], [0]))
                if j == tail - 1:
                    end.append(r)
        if entries:
            steps.append({"entries": entries, "end": end})
    widths = [len(s["entries"]) for s in steps[count // 4:]]
    assert max(widths) == count and any(w <= 64 for w in widths)
    eng = Engine(folder, dtype=dtype, max_tokens=count * 64, max_seqs=count)
    got = helpers.replay(eng, steps)
    if eng.decode_graphs is not None:
        assert eng.decode_graphs.replays > 0 and any(rows > 64 for rows, _ in eng.decode_graphs.shapes)
    some = dict(list(requests.items())[:6])          # the bound's plain engine need not run all of them
    check(folder, requests, got, dtype, f"{count} requests decoding together", tolerance(bf16_bound, folder, some, dtype))
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


def test_weights_loaded_again_under_captured_graphs(model_dirs):
    """A graph holds the addresses of the weights it was captured on.  After another checkpoint has been loaded into
    the same model, single-token steps must run on the new tensors: the graphs of the old ones are dropped."""
    from glassbox_amd.engine import Engine
    from glassbox_amd.weights import load_weights
    first, second = model_dirs.get("E", seed=0), model_dirs.get("E", seed=7)
    toks = helpers.random_tokens(helpers.TINY["E"]["vocab_size"], 60, seed=3)
    eng = Engine(first, dtype="bfloat16", max_tokens=256, max_seqs=2)
    assert eng.decode_graphs is not None
    bound = helpers.Bf16Bound()
    tol = max(bound.get(first, {"a": toks}), bound.get(second, {"a": toks}))
    assert_rows(rows_of(eng, [("a", toks[:50])])["a"], first, toks, 0, "bfloat16", tol, "the first checkpoint")
    for p in range(50, 55):
        assert_rows(rows_of(eng, [("a", toks[p:p + 1])])["a"], first, toks, p, "bfloat16", tol, "the first checkpoint")
    assert eng.decode_graphs.replays >= 3
    eng.end_request("a")
    load_weights(eng.model, os.path.join(second, "model.safetensors"), torch.bfloat16, eng.device)
    junk = torch.full((1 << 22,), 7.0, device=eng.device)     # what the allocator may put where the old weights lay
    assert_rows(rows_of(eng, [("b", toks[:50])])["b"], second, toks, 0, "bfloat16", tol, "the second checkpoint")
    replays = eng.decode_graphs.replays
    for p in range(50, 60):
        assert_rows(rows_of(eng, [("b", toks[p:p + 1])])["b"], second, toks, p, "bfloat16", tol, "the second checkpoint")
    assert eng.decode_graphs.replays > replays, "graphs are captured again after the reload"
    want = helpers.oracle(second, toks, "bfloat16")[55]
    assert np.abs(want - helpers.oracle(first, toks, "bfloat16")[55]).max() > 1e-2, "the two checkpoints must differ"
    del junk
    eng.end_request("b")
