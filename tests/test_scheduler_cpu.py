"""The scheduler's decisions, on the CPU: the real host scheduler and cache manager above a toy
model whose next token depends on the last token and its position only.  The properties are those
of the reference's tests (crates/glassbox-server/tests/scheduler.rs:84-186): batching, chunked
prompts, preemption, aborts and prefix sharing never change the outputs and never leak a page."""
import random
from types import SimpleNamespace

import pytest
import torch

from glassbox_amd.cache import FULL, CacheManager, GroupSpec
from glassbox_amd.engine.scheduler import Scheduler, SchedulerConfig
from glassbox_amd.sampling import SamplerConfig
from plain import sampler as psampler

V = 97


def toy_logits(token, pos):
    g = torch.Generator().manual_seed(token * 1000 + pos)
    return torch.randn(V, generator=g)


class ToyEngine:
    """Stands where Engine stands: a cache manager and run_reserved(); checks what the step is given."""

    def __init__(self, num_pages, max_seqs, share=True, max_positions=4096):
        self.cache = CacheManager(16, [GroupSpec(FULL, 0, num_pages)], max_seqs, share)
        self.max_seqs, self.group_keys = max_seqs, [(0, 0)]
        self.model = SimpleNamespace(vocab_size=V, config=SimpleNamespace(max_position_embeddings=max_positions))
        self.batches = []

    def reset_state(self, sid):
        pass

    def run_reserved(self, entries, validated=False):
        rows = []
        for sid, toks, want in entries:
            start = self.cache.seq_len(sid)
            assert len(self.cache.table(sid)) * 16 >= start + len(toks), "the step was not given its pages"
            rows += [toy_logits(toks[w], start + w) for w in want]
        self.batches.append([(sid, self.cache.seq_len(sid), len(toks), len(want)) for sid, toks, want in entries])
        return torch.stack(rows) if rows else torch.zeros(0, V)


def cpu_sample_rows(logits, configs, uniforms, contexts):
    toks, cands = [], []
    for row, cfg, u, ctx in zip(logits.tolist(), configs, uniforms, contexts):
        dist = psampler.distribution(row, ctx, cfg.temperature, cfg.top_k, cfg.top_p, cfg.min_p, cfg.repetition_penalty)
        acc, pick = 0.0, dist[-1][0]
        for t, p in dist:
            acc += p
            if u < acc:
                pick = t
                break
        toks.append(dist[0][0] if len(dist) == 1 else pick)
        cands.append(len(dist))
    return toks, cands


def alone(prompt, n, cfg=None, stop=()):
    """What the request produces by itself, token by token."""
    cfg = cfg or SamplerConfig()
    rng = psampler.Rng(cfg.seed)
    toks, out = list(prompt), []
    for _ in range(n):
        t = psampler.sample(rng, toy_logits(toks[-1], len(toks) - 1).tolist(), toks, temperature=cfg.temperature,
                            top_k=cfg.top_k, top_p=cfg.top_p, min_p=cfg.min_p, repetition_penalty=cfg.repetition_penalty)
        if t in stop:
            break
        out.append(t)
        toks.append(t)
    return out


def random_prompt(rng, prefix=()):
    return list(prefix) + [rng.randrange(V) for _ in range(1 + rng.randrange(60))]


def run_all(jobs, budget, max_seqs, pages, share=True, samplers=None, check_each=None):
    eng = ToyEngine(pages, max_seqs, share)
    s = Scheduler(eng, SchedulerConfig(budget, max_seqs), trace=True, sample_fn=cpu_sample_rows)
    ids = [s.submit(p, n, samplers[i] if samplers else None) for i, (p, n) in enumerate(jobs)]
    guard = 0
    while not s.is_idle():
        s.step()
        if check_each:
            check_each(s, eng)
        guard += 1
        assert guard < 10_000, "the scheduler made no progress"
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0, "pages leaked"
    assert eng.cache.free_state_slots() == max_seqs
    return [s.outputs[i] for i in ids], s, eng


def test_batched_equals_unbatched():
    for seed in range(4):
        rng = random.Random(seed)
        jobs = [(random_prompt(rng), 1 + rng.randrange(24)) for _ in range(10)]

        def budget_and_order(s, eng):
            batch = eng.batches[-1]
            assert sum(n for _, _, n, _ in batch) <= 16                       # scheduler.rs:284-298
            assert len(batch) <= 6
        outs, s, _ = run_all(jobs, 16, 6, 256, check_each=budget_and_order)
        for (p, n), out in zip(jobs, outs):
            assert out.tokens == alone(p, n) and out.finish == "length"
        m = s.metrics
        assert m["requests_finished"] == 10 and m["generated_tokens"] == sum(n for _, n in jobs)
        assert m["prompt_tokens"] == sum(len(p) for p, _ in jobs) and m["preemptions"] == 0


def test_preemption_keeps_outputs_and_frees_pages():
    rng = random.Random(99)
    jobs = [(random_prompt(rng), 30) for _ in range(12)]
    # 14 pages = 224 token slots for 12 requests that need about 4 each (tests/scheduler.rs:111)
    outs, s, _ = run_all(jobs, 64, 12, 14)
    assert s.metrics["preemptions"] > 0, "the test did not exercise preemption"
    assert any(r.preempted for r in s.trace)
    for (p, n), out in zip(jobs, outs):
        assert out.tokens == alone(p, n)


def test_the_newest_request_is_the_one_preempted():
    eng = ToyEngine(5, 4, share=False)
    s = Scheduler(eng, SchedulerConfig(64, 4), trace=True, sample_fn=cpu_sample_rows)
    a = s.submit([1] * 30, 40)
    b = s.submit([2] * 30, 40)
    while not any(r.preempted for r in s.trace):
        s.step()
    assert s.trace[-1].preempted == [b]            # scheduler.rs:228-236: least work lost
    assert s.queue_depth() == 1 and s.running() == 1
    s.run()
    assert s.outputs[a].tokens == alone([1] * 30, 40) and s.outputs[b].tokens == alone([2] * 30, 40)
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0
    # alone and still too long for the cache: ends with 'length' where the pages end (scheduler.rs:307-315)
    c = s.submit([3] * 30, 80)
    s.run()
    assert s.outputs[c].finish == "length" and 0 < len(s.outputs[c].tokens) < 80
    assert s.outputs[c].tokens == alone([3] * 30, 80)[:len(s.outputs[c].tokens)]
    assert eng.cache.used_pages() == 0


def test_seeded_sampling_survives_preemption():
    rng = random.Random(5)
    jobs = [(random_prompt(rng), 25) for _ in range(10)]
    samplers = [SamplerConfig(temperature=0.8, top_k=[0, 20][i % 2], top_p=[1.0, 0.9][i % 3 == 0], seed=i)
                for i in range(10)]
    outs, s, _ = run_all(jobs, 48, 10, 12, samplers=samplers)
    assert s.metrics["preemptions"] > 0
    for (p, n), cfg, out in zip(jobs, samplers, outs):
        assert out.tokens == alone(p, n, cfg)       # the generator's state is kept across preemption


def test_aborts_free_pages():
    # tests/scheduler.rs:125-163
    rng = random.Random(5)
    eng = ToyEngine(64, 8)
    s = Scheduler(eng, SchedulerConfig(32, 8), sample_fn=cpu_sample_rows)
    ids = [s.submit(random_prompt(rng), 40) for _ in range(16)]
    for step in range(400):
        if s.is_idle():
            break
        s.step()
        if step % 3 == 0:
            s.abort(rng.choice(ids))
        eng.cache.check_invariants()
    s.run()
    eng.cache.check_invariants()
    assert eng.cache.used_pages() == 0
    assert "aborted" in {o.finish for o in s.outputs.values()}
    assert all(o.finish is not None for o in s.outputs.values())


def test_prefix_sharing_never_changes_outputs():
    # tests/scheduler.rs:165-186
    rng = random.Random(11)
    system = [(i * 13) % V for i in range(70)]
    jobs = [(random_prompt(rng, system), 12) for _ in range(8)]
    on, s_on, _ = run_all(jobs, 48, 4, 128, share=True)
    off, s_off, _ = run_all(jobs, 48, 4, 128, share=False)
    assert [o.tokens for o in on] == [o.tokens for o in off] == [alone(p, n) for p, n in jobs]
    assert s_on.metrics["prefix_hit_tokens"] >= 64 and s_off.metrics["prefix_hit_tokens"] == 0
    assert s_on.metrics["batch_tokens"] < s_off.metrics["batch_tokens"]


def test_stop_tokens_zero_budget_and_the_position_cap():
    p = [3, 1, 4, 1, 5]
    full = alone(p, 20)
    stop = full[6]
    eng = ToyEngine(32, 4)
    s = Scheduler(eng, SchedulerConfig(8, 4), sample_fn=cpu_sample_rows)
    a = s.submit(p, 20, stop=[stop])
    b = s.submit(p, 0)
    s.run()
    cut = full.index(stop)
    assert s.outputs[a].tokens == full[:cut] and s.outputs[a].finish == "stop"     # not appended, not emitted
    assert s.outputs[b].tokens == [] and s.outputs[b].finish == "length"           # scheduler.rs:374-378
    eng = ToyEngine(32, 4, max_positions=12)
    s = Scheduler(eng, SchedulerConfig(8, 4), sample_fn=cpu_sample_rows)
    c = s.submit(p, 20)
    s.run()
    assert len(s.outputs[c].tokens) == 12 - len(p) and s.outputs[c].finish == "length"   # scheduler.rs:401
    assert eng.cache.used_pages() == 0


def test_prompts_are_cut_under_the_budget_and_only_the_last_portion_wants_logits():
    eng = ToyEngine(64, 4, share=False)
    s = Scheduler(eng, SchedulerConfig(16, 4), sample_fn=cpu_sample_rows)
    s.submit(list(range(40)), 2)
    s.run()
    sizes = [[(start, n, want) for _, start, n, want in b] for b in eng.batches]
    assert sizes == [[(0, 16, 0)], [(16, 16, 0)], [(32, 8, 1)], [(40, 1, 1)]]
    # a decoding request shares the step with another's prompt portion, and goes first
    eng = ToyEngine(64, 4, share=False)
    s = Scheduler(eng, SchedulerConfig(16, 4), sample_fn=cpu_sample_rows)
    s.submit([1, 2, 3], 5)
    s.step()
    s.submit(list(range(40)), 1)
    s.step()
    assert [(n, want) for _, _, n, want in eng.batches[-1]] == [(1, 1), (15, 0)]


def test_nothing_to_do():
    eng = ToyEngine(8, 2)
    s = Scheduler(eng, sample_fn=cpu_sample_rows, config=SchedulerConfig(16, 2))
    assert s.step() is False and s.is_idle()
    with pytest.raises(ValueError):
        s.submit([], 3)
    with pytest.raises(ValueError):
        s.submit([V], 3)


def test_the_penalty_pairs_count_each_requests_tokens():
    """The native scheduler's (row, token, occurrences, penalty) for the wanted rows of a step are what counting
    each request's context gives (sampler.rs:100-108 walks the context token by token), in steps with portions,
    under preemption, for requests with and without a penalty."""
    import numpy as np
    from collections import Counter
    rng = random.Random(5)
    eng = ToyEngine(14, 6)
    s = None
    seen = {"steps": 0, "pairs": 0}

    def checked(logits, configs, uniforms, contexts):
        lib, h = s._lib, s._h
        m = lib.gbh_sched_penalty_pairs(h, None, None, None, None, 0)
        pairs = np.zeros((4, m), np.int32)
        if m:
            assert lib.gbh_sched_penalty_pairs(h, pairs[0].ctypes.data, pairs[1].ctypes.data, pairs[2].ctypes.data,
                                               pairs[3].ctypes.data, m) == m
        got = {}
        for r, t, c, p in zip(pairs[0].tolist(), pairs[1].tolist(), pairs[2].tolist(), pairs[3].view(np.float32).tolist()):
            assert (r, t) not in got
            got[(r, t)] = (c, p)
        want = {}
        for r, (cfg, ctx) in enumerate(zip(configs, contexts)):
            if cfg.repetition_penalty != 1.0:
                for t, c in Counter(ctx).items():
                    want[(r, t)] = (c, np.float32(cfg.repetition_penalty).item())
        assert got == want
        seen["steps"] += 1
        seen["pairs"] += m
        return cpu_sample_rows(logits, configs, uniforms, contexts)

    s = Scheduler(eng, SchedulerConfig(32, 6), sample_fn=checked)
    for i in range(10):
        cfg = SamplerConfig(temperature=0.8, repetition_penalty=[1.0, 1.3, 2.0][i % 3], seed=i)
        s.submit(random_prompt(rng), 12, cfg)
    s.run()
    assert s.is_idle() and seen["steps"] > 20 and seen["pairs"] > 100
