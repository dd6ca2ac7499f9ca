"""The scheduler on the device, compared at the level of logits: every row that a step of the scheduler asks
for is checked against the plain implementation at that request's position, through preemption and
recomputation, shared beginnings, and portions under a token budget, in 32-bit and in bfloat16.

Tokens alone would not do: a model with tied embeddings and small random weights answers with its last input
token whatever the cache holds (``test_the_tiny_models_do_not_echo`` shows which of the tiny models do)."""
import random

import numpy as np
import pytest
import torch

import helpers
from plain import llama as plain
from plain import sampler as psampler

pytestmark = pytest.mark.gpu


def serve(eng, prompts, max_tokens, samplers=None, budget=16, max_seqs=4, abort_every=0, abort_seed=0, max_aborts=7):
    """Runs the prompts through a scheduler and records, for every step, which request brought which positions and
    the logits that came back.  Returns (replies, scheduler, records); a record is (request index, position, row).
    ``abort_every``: after every so many steps one live request, drawn at random, is aborted (up to ``max_aborts``),
    the cache's invariants are checked after every step, and ``scheduler.aborted`` counts the aborted requests that
    were running and that were waiting (crates/glassbox-server/tests/scheduler.rs:142-151)."""
    from glassbox_amd.engine import Scheduler, SchedulerConfig
    from glassbox_amd.sampling import SamplerConfig
    sched = Scheduler(eng, SchedulerConfig(token_budget=budget, max_seqs=max_seqs))
    ids = [sched.submit(p, max_tokens, (samplers[i] if samplers else SamplerConfig())) for i, p in enumerate(prompts)]
    index = {rid: i for i, rid in enumerate(ids)}
    records = []
    inner = eng.run_reserved

    early = []   # rows of steps launched ahead of their plan: kept if the request got as far as their position

    def spy(entries, validated=False, ahead=None):
        at = [eng.cache.seq_len(sid) + (ahead[j] if ahead else 0) for j, (sid, _, _) in enumerate(entries)]
        logits = inner(entries, validated, ahead)
        rows = logits.float().cpu().numpy()
        row = 0
        for (sid, toks, want), first in zip(entries, at):
            for w in want:
                (early if ahead else records).append((index[sid], first + w, rows[row].copy()))
                row += 1
        assert row == rows.shape[0]
        return logits

    eng.run_reserved = spy
    rng = random.Random(abort_seed)
    sched.aborted = {"running": 0, "waiting": 0}
    try:
        guard = 0
        while not sched.is_idle():
            sched.step()
            guard += 1
            assert guard < 100000
            if abort_every:
                eng.cache.check_invariants()
                live = [rid for rid in ids if sched.outputs[rid].finish is None]
                if guard % abort_every == 0 and live and sum(sched.aborted.values()) < max_aborts:
                    before = sched.running()
                    sched.abort(rng.choice(live))
                    sched.aborted["running" if sched.running() < before else "waiting"] += 1
                    eng.cache.check_invariants()
    finally:
        del eng.run_reserved
    replies = [sched.outputs[i].tokens for i in ids]
    # a row that ran ahead for a request that then stopped or was aborted stands for no position of its reply
    records += [r for r in early if r[1] < len(prompts[r[0]]) + len(replies[r[0]])]
    return replies, sched, records


def check_records(folder, prompts, replies, records, dtype, tol, what):
    assert records
    for i, pos, row in records:
        full = list(prompts[i]) + list(replies[i])
        assert pos < len(full), (i, pos, len(full))
        want = helpers.oracle(folder, full, dtype)[pos]
        err = float(np.abs(row - want).max())
        assert err <= tol, (f"{what}, {dtype}: request {i} ({len(prompts[i])} prompt tokens), position {pos} "
                            f"(page offset {pos % 16}): error {err:.3e}, allowed {tol:.3e}")


def test_the_tiny_models_do_not_echo(model_dirs):
    """Which tiny models' greedy replies depend on the context: B and D (untied heads) do; A (tied, small random
    weights) repeats its last prompt token, so its tokens say nothing about the cache.  Tests that compare tokens
    use B or D."""
    for name, echoes in (("A", True), ("B", False), ("D", False)):
        cfg, w = plain.load_folder(model_dirs.get(name))
        prompt = helpers.random_tokens(cfg["vocab_size"], 12, seed=3)
        reply = plain.greedy(w, cfg, prompt, 6)
        assert (reply == [prompt[-1]] * 6) == echoes, (name, prompt[-1], reply)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D", "A"])
def test_preemption_and_shared_beginnings_at_the_level_of_logits(model_dirs, bf16_bound, name, dtype):
    """Ten requests, half of them behind one 70-token beginning, through fourteen pages with the prefix cache on
    (crates/glassbox-server/tests/scheduler.rs:106-123,165-186): requests are preempted and recomputed, beginnings
    are found in the cache, prompts come in portions of at most sixteen tokens beside decoded tokens.  Every row of
    logits the scheduler sampled from is that of the plain implementation."""
    from glassbox_amd.engine import Engine
    folder = model_dirs.get(name)
    vocab = helpers.TINY[name]["vocab_size"]
    limit = helpers.TINY[name]["max_position_embeddings"]
    rng = random.Random(7)
    system = helpers.random_tokens(vocab, 70, seed=77)
    prompts = [(system if i % 2 else []) + [rng.randrange(vocab) for _ in range(1 + rng.randrange(30))] for i in range(10)]
    eng = Engine(folder, dtype=dtype, max_tokens=14 * 16, max_seqs=6, prefix_caching=True)
    replies, sched, records = serve(eng, prompts, max_tokens=12, budget=16, max_seqs=6)
    assert all(len(r) == 12 or len(p) + len(r) >= limit for p, r in zip(prompts, replies))
    m = sched.metrics
    assert m["preemptions"] > 0, "fourteen pages for ten requests should force preemption"
    assert m["prefix_hit_tokens"] >= 64, "the shared beginning was never found in the cache"
    full = {f"r{i}": p + r for i, (p, r) in enumerate(zip(prompts, replies))}
    tol = helpers.TOL_F32 if dtype == "float32" else bf16_bound.get(folder, full)
    check_records(folder, prompts, replies, records, dtype, tol, "scheduler")
    # recomputation shows: more tokens were run or found in the cache than the requests hold
    assert m["batch_tokens"] + m["prefix_hit_tokens"] > sum(len(t) - 1 for t in full.values())
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0


def test_seeded_temperature_replies_are_the_plain_samplers(model_dirs):
    """The second tiny configuration with the workload it is quoted with: prompts of 1, 9, 40 and 70 tokens, portions of sixteen,
    24 tokens at temperature 0.8, seeded.  In 32-bit every token is the one the plain sampler draws from the plain
    implementation's logits with the same generator (crates/glassbox-core/src/sampler.rs:97-164); the comparison
    of a request ends where a draw falls within 1e-5 of a boundary between two tokens."""
    from glassbox_amd.engine import Engine
    from glassbox_amd.sampling import SamplerConfig
    folder = model_dirs.get("B")
    cfg, w = plain.load_folder(folder)
    prompts = [helpers.random_tokens(384, n, seed=n) for n in (1, 9, 40, 70)]
    # (two of them with a repetition penalty, which the native scheduler counts tokens for, one with every filter)
    samplers = [SamplerConfig(temperature=0.8, seed=1), SamplerConfig(temperature=0.8, repetition_penalty=1.3, seed=2),
                SamplerConfig(temperature=0.8, top_k=40, top_p=0.9, min_p=0.002, repetition_penalty=1.2, seed=3),
                SamplerConfig(temperature=0.8, seed=4)]
    eng = Engine(folder, dtype="float32", max_tokens=2048, max_seqs=8)
    replies, sched, records = serve(eng, prompts, max_tokens=24, samplers=samplers, budget=16, max_seqs=8)
    compared = 0
    for p, reply, s in zip(prompts, replies, samplers):
        assert len(reply) == 24
        rng, toks = psampler.Rng(s.seed), list(p)
        for t in reply:
            logits = plain.forward(w, cfg, toks)[-1].tolist()
            dist = psampler.distribution(logits, toks, s.temperature, s.top_k, s.top_p, s.min_p, s.repetition_penalty)
            u = rng.next_f32() if len(dist) > 1 else 0.0
            acc, want, near = np.float32(0), dist[-1][0], False
            for tok, prob in dist:
                acc = np.float32(acc + np.float32(prob))
                near |= abs(float(acc) - u) < 1e-5
                if u < acc:
                    want = tok
                    break
            if near:
                break
            assert t == want, f"prompt of {len(p)} tokens, token {len(toks) - len(p)}: drew {t}, the plain sampler {want}"
            toks.append(t)
            compared += 1
    assert compared >= 80, "too many draws fell on a boundary for the test to say anything"
    check_records(folder, prompts, replies, records, "float32", helpers.TOL_F32, "temperature 0.8")
    # another seed gives other replies: the draws do depend on the generator
    other, _, _ = serve(eng, prompts, max_tokens=24, samplers=[SamplerConfig(temperature=0.8, seed=s + 10) for s in (1, 2, 3, 4)],
                        budget=16, max_seqs=8)
    assert other != replies


def test_reserve_that_fails_leaves_no_request_and_no_copy_behind(model_dirs):
    """A step whose second entry finds no room: nothing is written, the request that the step would have added is
    not registered, the copy that the first entry's copy-on-write asked for is made (its page stays reserved), and
    the same step goes through once room is made."""
    from glassbox_amd.cache import OutOfPages
    from glassbox_amd.engine import Engine
    folder = model_dirs.get("B")
    toks = helpers.random_tokens(384, 60, seed=12)
    eng = Engine(folder, dtype="float32", max_tokens=3 * 16, max_seqs=4)
    eng.step([("p", toks[:20], [])])                 # two pages, the second partial
    eng.fork_request("p", "c")
    with pytest.raises(OutOfPages):
        eng.step([("c", toks[20:23], [2]), ("new", toks[:17], [])])   # copy-on-write takes the last page; "new" needs two
    assert not eng.has_request("new")
    assert eng.cache.take_copies() == []
    assert eng.request_len("c") == 20 and eng.request_len("p") == 20
    eng.cache.check_invariants()
    got = eng.step([("c", toks[20:23], [2])]).cpu().numpy()
    assert np.abs(got[0] - helpers.plain_logits(folder, tuple(toks[:23]))[22]).max() < 1e-4
    got = eng.step([("p", [5, 6], [1])]).cpu().numpy()      # the parent's page was not disturbed by the child's tokens
    assert np.abs(got[0] - helpers.plain_logits(folder, tuple(toks[:20] + [5, 6]))[21]).max() < 1e-4
    eng.end_request("p"); eng.end_request("c")
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0
