"""The scheduler's decisions on the CPU, against a stand-in device that reads tokens back
through the block tables (tests/fake_executor.py).  The workloads follow the reference's own
engine test (tests/test_main.cpp:241-302) and its trace simulator (sim/simulate.cpp:120-210)."""

import random

import pytest

from bitwise_amd.config.engine import EngineConfig, SamplingParams
from bitwise_amd.engine.engine import Engine
from fake_executor import FakeExecutor


def run_all(cfg, prompts, params, arrivals=None, cancels=None, guard=20000, run_ahead=False):
    ex = FakeExecutor(cfg.block_size, run_ahead=run_ahead)
    eng = Engine(None, None, cfg, executor=ex)
    ids = [None] * len(prompts)
    arrivals = arrivals or [0] * len(prompts)
    cancels = cancels or [-1] * len(prompts)
    added = 0
    for step in range(guard):
        for i in range(len(prompts)):
            if arrivals[i] == step:
                ids[i] = eng.add_request(prompts[i], params[i])
                added += 1
            if cancels[i] == step and ids[i] is not None:
                eng.cancel(ids[i])
        if added == len(prompts) and eng.idle():
            break
        eng.step()
        eng.manager.check()
    else:
        raise AssertionError("engine did not finish:\n" + eng.debug_state())
    return eng, ex, [eng.result(i) for i in ids]


def solo(cfg_base, prompt, sp):
    cfg = EngineConfig(num_blocks=(len(prompt) + sp.max_new_tokens) // cfg_base.block_size + 2,
                       max_batched_tokens=4096, prefix_caching=False, block_size=cfg_base.block_size)
    _, _, (r,) = run_all(cfg, [prompt], [sp])
    return r


def shared_prefix_workload():
    """Six requests sharing a 37-token prefix plus 3+5r own tokens, odd ones sampled
    (tests/test_main.cpp:244-259)."""
    shared = [(i * 13 + 1) % 97 for i in range(37)]
    prompts = [shared + [(r * 17 + i * 3) % 97 for i in range(3 + 5 * r)] for r in range(6)]
    params = [SamplingParams(temperature=0.8 if r % 2 else 0.0, seed=100 + r, max_new_tokens=20 + r, ignore_eos=True)
              for r in range(6)]
    return prompts, params


@pytest.mark.parametrize("variant", ["chunked+prefix", "tight memory"])
def test_shared_prefix_equals_solo(variant):
    prompts, params = shared_prefix_workload()
    cfg = EngineConfig()
    if variant == "chunked+prefix":
        cfg.max_batched_tokens = 24
    else:
        cfg.num_blocks = 9          # forces preemption and recomputation (tests/test_main.cpp:274)
        cfg.max_batched_tokens = 32
    eng, ex, results = run_all(cfg, prompts, params)
    for p, sp, r in zip(prompts, params, results):
        ref = solo(cfg, p, sp)
        assert r.tokens == ref.tokens
        assert r.logits_fingerprint == ref.logits_fingerprint
        assert r.finished and not r.cancelled
    assert eng.free_blocks == cfg.num_blocks
    assert eng.manager.slots.available() == cfg.max_num_seqs
    if variant == "tight memory":
        assert eng.stats.preemptions > 0
        assert sum(r.preemptions for r in results) == eng.stats.preemptions
    else:
        assert eng.stats.prefix_hit_tokens > 0
        assert sum(r.prefix_cached_tokens for r in results) == eng.stats.prefix_hit_tokens


def test_budget_cuts_prompts_and_running_come_first():
    cfg = EngineConfig(max_batched_tokens=10, prefix_caching=False)
    ex = FakeExecutor(cfg.block_size)
    eng = Engine(None, None, cfg, executor=ex)
    a = eng.add_request(list(range(1, 26)), SamplingParams(max_new_tokens=3, ignore_eos=True))
    b = eng.add_request(list(range(30, 36)), SamplingParams(max_new_tokens=3, ignore_eos=True))
    eng.step()                                   # 10 tokens of a
    assert eng.sched.running[0].computed == 10 and eng.num_waiting == 1 and ex.rows_run == 10
    eng.step()                                   # 10 more of a; b is not admitted on an empty budget
    assert eng.sched.running[0].computed == 20 and eng.num_waiting == 1
    eng.step()                                   # last 5 of a (first token sampled), 5 of b
    assert len(eng.result(a).tokens) == 1 and eng.num_running == 2
    assert eng.sched.running[1].computed == 5
    eng.step()                                   # a decodes (1), b finishes its prompt (1) and samples
    assert len(eng.result(a).tokens) == 2 and len(eng.result(b).tokens) == 1
    while not eng.idle():
        eng.step()
    assert eng.result(a).finished and eng.result(b).finished
    assert eng.stats.prefill_tokens == 31 and eng.stats.decode_rows == 4 and eng.stats.generated_tokens == 6


def test_cut_portions_end_on_whole_blocks():
    """With a budget that leaves room (budget - max_num_seqs >= portion_align) a prompt portion that ends short of its
    prompt ends at a multiple of portion_align unless what it leaves is shorter than that anyway, and a request that
    could only start with a sliver waits a step.  The tokens are those of each request alone."""
    cfg = EngineConfig(num_blocks=64, max_batched_tokens=200, max_num_seqs=4, prefix_caching=False, portion_align=64)
    ex = FakeExecutor(cfg.block_size)
    eng = Engine(None, None, cfg, executor=ex)
    plans = []
    plan = eng.sched.plan

    def spy():
        p = plan()
        plans.append([(w.seq.id, w.start, w.n) for w in p])
        return p
    eng.sched.plan = spy
    prompts = [[(7 * i + r) % 90 + 1 for i in range(n)] for r, n in enumerate((300, 150, 70))]
    sp = SamplingParams(max_new_tokens=6, ignore_eos=True)
    ids = [eng.add_request(p, sp) for p in prompts]
    while not eng.idle():
        eng.step()
        eng.manager.check()
    assert plans[0] == [(0, 0, 192)]                              # 200 fit: cut at 192, since 100 would be left anyway
    assert plans[1] == [(0, 192, 108), (1, 0, 92)]                # a ends; of b all 92 that fit: 58 are left, less than 64
    assert plans[2] == [(0, 300, 1), (1, 92, 58), (2, 0, 70)]
    for step in plans:
        for sid, start, n in step:
            left = len(prompts[sid]) - start - n
            assert left <= 0 or (start + n) % 64 == 0 or left < 64, step
    # a long prompt beside decoded tokens: every portion but the last ends on a multiple of 64, and a request that
    # could only start with a sliver waits for the next step
    long_cfg = EngineConfig(num_blocks=200, max_batched_tokens=256, max_num_seqs=4, prefix_caching=False, portion_align=64)
    eng2 = Engine(None, None, long_cfg, executor=FakeExecutor(long_cfg.block_size))
    seen = []
    plan2 = eng2.sched.plan

    def spy2():
        p = plan2()
        seen.append([(w.seq.id, w.start, w.n) for w in p])
        return p
    eng2.sched.plan = spy2
    eng2.add_request([5] * 20, SamplingParams(max_new_tokens=30, ignore_eos=True))
    eng2.add_request([(3 * i) % 80 + 1 for i in range(1000)], sp)
    eng2.add_request([(5 * i) % 80 + 1 for i in range(900)], sp)
    while not eng2.idle():
        eng2.step()
    assert seen[0] == [(0, 0, 20), (1, 0, 192)]                   # 236 fit beside the 20: cut at 192; 44 left, c waits
    assert seen[1] == [(0, 20, 1), (1, 192, 192)]                 # 255 fit: 192 + 192 = 384
    cuts = [(sid, start + n) for step in seen for sid, start, n in step if sid and start + n < (1000, 900)[sid - 1]]
    assert cuts and all(end % 64 == 0 for _, end in cuts), cuts
    for i, p in zip(ids, prompts):
        assert eng.result(i).tokens == solo(cfg, p, sp).tokens
    # a budget without that room cuts exactly where it ends, as ever
    tight = EngineConfig(num_blocks=64, max_batched_tokens=66, max_num_seqs=4, prefix_caching=False, portion_align=64)
    eng = Engine(None, None, tight, executor=FakeExecutor(tight.block_size))
    eng.add_request(prompts[0], sp)
    eng.step()
    assert eng.sched.running[0].computed == 66
    with pytest.raises(ValueError):
        EngineConfig(portion_align=0).validate()


def test_head_of_line_blocking_and_refusal():
    cfg = EngineConfig(num_blocks=4, block_size=16, prefix_caching=False, max_batched_tokens=64)
    eng = Engine(None, None, cfg, executor=FakeExecutor(16))
    with pytest.raises(ValueError, match="never fit"):
        eng.add_request(list(range(60)), SamplingParams(max_new_tokens=8))
    with pytest.raises(ValueError, match="empty"):
        eng.add_request([], SamplingParams())
    with pytest.raises(ValueError, match="out of range"):
        eng.add_request([1, 97], SamplingParams())
    a = eng.add_request(list(range(40)), SamplingParams(max_new_tokens=4, ignore_eos=True))   # 3 pages
    b = eng.add_request(list(range(40, 70)), SamplingParams(max_new_tokens=4, ignore_eos=True))  # 2 pages: must wait
    c = eng.add_request([5], SamplingParams(max_new_tokens=1, ignore_eos=True))               # would fit, stays behind b
    eng.step()
    assert eng.num_running == 1 and eng.num_waiting == 2
    assert eng.free_blocks == 1                  # b gave back what it took when it could not be admitted
    while not eng.idle():
        eng.step()
    assert all(eng.result(i).finished for i in (a, b, c))
    assert eng.result(b).first_token < eng.result(c).first_token
    assert eng.free_blocks == 4


@pytest.mark.parametrize("num_blocks", [4, 5])
def test_youngest_unscheduled_request_is_preempted_and_recomputes(num_blocks):
    cfg = EngineConfig(num_blocks=num_blocks, block_size=8, prefix_caching=False, max_batched_tokens=64, max_num_seqs=4)
    eng = Engine(None, None, cfg, executor=FakeExecutor(8))
    sp = SamplingParams(max_new_tokens=12, ignore_eos=True)
    ids = [eng.add_request([10 + r] * 7, sp) for r in range(3)]      # one page each; position 8 needs a second
    eng.step()                                   # prompts (positions 0-6)
    eng.step()                                   # position 7: still the first page
    assert eng.num_running == 3 and eng.free_blocks == num_blocks - 3
    eng.step()
    # 4 pages: request 0 takes the free one, request 1 takes the page of the youngest (2), which
    # is not scheduled yet.  5 pages: 0 and 1 take the free ones, 2 finds no victim but itself.
    assert eng.result(ids[2]).preemptions == 1 and eng.result(ids[0]).preemptions == 0
    assert eng.result(ids[1]).preemptions == 0
    assert eng.num_waiting == 1 and eng.sched.waiting[0].id == ids[2]
    assert eng.sched.waiting[0].computed == 0 and eng.sched.waiting[0].cache is None
    kept = list(eng.result(ids[2]).tokens)
    assert len(kept) == 2                        # generated tokens are kept and recomputed as prompt
    while not eng.idle():
        eng.step()
    for n, i in enumerate(ids):
        r = eng.result(i)
        ref = solo(cfg, [10 + n] * 7, sp)
        assert r.tokens == ref.tokens and r.logits_fingerprint == ref.logits_fingerprint
    assert eng.result(ids[2]).tokens[:2] == kept
    assert eng.free_blocks == num_blocks


def test_eos_stops_and_is_kept():
    cfg = EngineConfig(prefix_caching=False)
    ex = FakeExecutor(16, vocab_size=5, eos_token_id=3)
    eng = Engine(None, None, cfg, executor=ex)
    rid = eng.add_request([1, 2], SamplingParams(max_new_tokens=200))
    rid2 = eng.add_request([1, 2], SamplingParams(max_new_tokens=200, ignore_eos=True))
    while not eng.idle():
        eng.step()
    toks = eng.result(rid).tokens
    assert toks[-1] == 3 and 3 not in toks[:-1] and len(toks) < 200
    assert len(eng.result(rid2).tokens) == 200 and eng.result(rid2).tokens[:len(toks)] == toks


def test_cancel_gives_everything_back():
    cfg = EngineConfig(num_blocks=8, block_size=8, max_batched_tokens=16)
    eng = Engine(None, None, cfg, executor=FakeExecutor(8))
    a = eng.add_request(list(range(30)), SamplingParams(max_new_tokens=10, ignore_eos=True))
    b = eng.add_request(list(range(20)), SamplingParams(max_new_tokens=10, ignore_eos=True))
    eng.step()
    eng.cancel(a)                                # running, in the middle of its prompt
    eng.cancel(b)                                # still waiting
    eng.cancel(a)                                # again: no effect
    assert eng.idle() and eng.free_blocks == 8
    assert eng.result(a).cancelled and eng.result(a).finished and eng.result(b).cancelled
    assert eng.manager.slots.available() == cfg.max_num_seqs


@pytest.mark.parametrize("run_ahead", [False, True])
@pytest.mark.parametrize("seed", range(40))
def test_random_traces_equal_solo(seed, run_ahead):
    """The reference's simulator on the CPU (sim/simulate.cpp:120-210): random requests with
    shared and repeated prompts, staggered arrivals, cancellations, tight pools and small
    budgets; every request that was not cancelled must equal its solo run."""
    rng = random.Random(seed)
    ps = rng.choice([8, 16, 32])
    V = 97
    prefixes = [[rng.randrange(4, V) for _ in range(ps * rng.randint(1, 3) if rng.random() < 0.5 else rng.randint(8, 48))]
                for _ in range(3)]
    n = rng.randint(1, 10)
    prompts, params, arrivals, cancels = [], [], [], []
    max_need = 0
    for i in range(n):
        if i > 0 and rng.random() < 0.15:
            p = list(prompts[rng.randrange(i)])
        else:
            p = list(rng.choice(prefixes)) if rng.random() < 0.5 else []
            p += [rng.randrange(V) for _ in range(rng.randint(0 if p else 1, 40))]
        sp = SamplingParams(temperature=0.0 if rng.random() < 0.5 else rng.uniform(0.3, 1.5), seed=rng.getrandbits(63),
                            max_new_tokens=rng.randint(1, 24), ignore_eos=rng.random() < 0.5)
        arr = 0 if rng.random() < 0.3 else rng.randint(0, 30)
        prompts.append(p), params.append(sp), arrivals.append(arr)
        cancels.append(arr + rng.randint(0, 20) if rng.random() < 0.15 else -1)
        max_need = max(max_need, len(p) + sp.max_new_tokens)
    cfg = EngineConfig(block_size=ps, max_batched_tokens=rng.randint(4, 64), max_num_seqs=rng.randint(1, 8),
                       prefix_caching=rng.random() < 0.7)
    cfg.num_blocks = (max_need + 1 + ps - 1) // ps + rng.randint(0, 12)
    eng, ex, results = run_all(cfg, prompts, params, arrivals, cancels, run_ahead=run_ahead)
    assert eng.free_blocks == cfg.num_blocks, "leaked pages"
    assert eng.manager.slots.available() == cfg.max_num_seqs
    for p, sp, r in zip(prompts, params, results):
        if r.cancelled:
            continue
        ref = solo(cfg, p, sp)
        assert r.tokens == ref.tokens
        assert r.logits_fingerprint == ref.logits_fingerprint


def test_steps_are_launched_ahead_and_thrown_away_rows_do_no_harm():
    """Decode steps of an unchanged set of requests are launched before the tokens of the step before are read.
    A request that ends by its end-of-sequence token has had one more row launched: it is thrown away, its
    stale write lands in a page that may already belong to a newcomer, and nobody's tokens change."""
    cfg = EngineConfig(num_blocks=12, block_size=8, max_batched_tokens=32, max_num_seqs=3, prefix_caching=True)
    prompts = [[5, 6, 7, 8, 9], [11, 12, 13], [21, 22, 23, 24, 25, 26, 27, 28, 29], [40, 41], [50, 51, 52, 53]]
    params = [SamplingParams(max_new_tokens=40), SamplingParams(max_new_tokens=40, temperature=0.9, seed=4),
              SamplingParams(max_new_tokens=30, ignore_eos=True), SamplingParams(max_new_tokens=25),
              SamplingParams(max_new_tokens=12, ignore_eos=True)]
    total_ahead = 0
    for vocab in (5, 13, 97):               # small vocabularies: the end-of-sequence token (3) comes early and often
        def run(run_ahead):
            ex = FakeExecutor(cfg.block_size, vocab_size=vocab, run_ahead=run_ahead)
            eng = Engine(None, None, cfg, executor=ex)
            ids = [eng.add_request([t % vocab for t in p], sp) for p, sp in zip(prompts, params)]
            for _ in range(2000):
                if eng.idle():
                    break
                eng.step()
                eng.manager.check()
            assert eng.idle() and eng.free_blocks == cfg.num_blocks and eng.manager.slots.available() == cfg.max_num_seqs
            return ex, [(eng.result(i).tokens, eng.result(i).logits_fingerprint) for i in ids]
        ex_plain, plain = run(False)
        ex_ahead, ahead = run(True)
        assert ahead == plain
        assert ex_plain.steps_ahead == 0
        total_ahead += ex_ahead.steps_ahead
    assert total_ahead > 20


def test_random_traces_do_exercise_preemption_and_prefix_hits():
    """The traces above are only worth something if they reach the hard cases."""
    pre = hits = evict = 0
    for seed in range(40):
        rng = random.Random(1000 + seed)
        ps = 8
        shared = [rng.randrange(4, 97) for _ in range(24)]
        prompts = [shared + [rng.randrange(97) for _ in range(rng.randint(0, 40))] for _ in range(6)]
        params = [SamplingParams(temperature=0.8, seed=r, max_new_tokens=20, ignore_eos=True) for r in range(6)]
        need = max(len(p) for p in prompts) + 21
        cfg = EngineConfig(block_size=ps, num_blocks=(need + ps - 1) // ps + rng.randint(0, 6),
                           max_batched_tokens=rng.randint(8, 48), max_num_seqs=6)
        eng, _, results = run_all(cfg, prompts, params)
        pre += eng.stats.preemptions
        hits += eng.stats.prefix_hit_tokens
        evict += eng.stats.evictions
        for p, sp, r in zip(prompts, params, results):
            ref = solo(cfg, p, sp)
            assert r.tokens == ref.tokens and r.logits_fingerprint == ref.logits_fingerprint
    assert pre > 0 and hits > 0 and evict > 0


@pytest.mark.parametrize("fault", ["prefix_covers_last_page", "register_partial_page", "cancel_leaks"])
def test_injected_faults_are_caught(fault, monkeypatch):
    """Negative controls after the reference's fault sweep (src/engine.h:52-62,
    README.md:86-93): each slip must make the equal-to-solo check, the leak check or the
    hang guard fail."""
    from bitwise_amd.cache import manager as mgr

    if fault == "prefix_covers_last_page":
        orig = mgr.CacheManager.admit_prefix

        def bad(self, rc, tokens):
            return orig(self, rc, list(tokens) + [0])      # may reuse the page holding the last token
        monkeypatch.setattr(mgr.CacheManager, "admit_prefix", bad)
    elif fault == "register_partial_page":
        orig_adv = mgr.CacheManager.advance

        def bad_adv(self, rc, tokens, computed):
            ps = self.page_size
            padded = list(tokens) + [0] * ps
            return_val = orig_adv(self, rc, padded, min((computed + ps - 1) // ps, len(rc.tables[0])) * ps)
            rc.computed = computed
            return return_val
        monkeypatch.setattr(mgr.CacheManager, "advance", bad_adv)
    else:
        from bitwise_amd.engine import scheduler as sch
        orig_remove = sch.Scheduler.remove

        def bad_remove(self, seq):
            if seq.cache is not None and not seq.done and seq.generated() < seq.params.max_new_tokens:
                for t in seq.cache.tables:
                    t.clear()
            return orig_remove(self, seq)
        monkeypatch.setattr(sch.Scheduler, "remove", bad_remove)
    caught = 0
    for seed in range(30):
        try:
            test_random_traces_equal_solo(seed, seed % 2 == 1)
            prompts, params = shared_prefix_workload()
            cfg = EngineConfig(max_batched_tokens=24, num_blocks=40)
            aligned = [[(i * 7 + seed) % 97 for i in range(32)]] * 2      # a repeated prompt that fills its pages
            prompts = prompts + prompts + aligned
            params = params + params + [SamplingParams(max_new_tokens=4, ignore_eos=True)] * 2
            eng, _, results = run_all(cfg, prompts, params, arrivals=[0] * 12 + [0, 40], guard=3000)
            for p, sp, r in zip(prompts, params, results):
                ref = solo(cfg, p, sp)
                assert r.tokens == ref.tokens and r.logits_fingerprint == ref.logits_fingerprint
        except (AssertionError, RuntimeError, KeyError, IndexError, TypeError):
            caught += 1
    assert caught > 0
