"""The product's scheduler (decisions taken natively) beside the plain one of ``plain_scheduler.py``: the same
requests through both, each with a stand-in engine and a cache of its own, and the same decisions step by step,
set-backs and failures included."""
import random

import pytest

from fake_engine import CpuSampler, FakeEngine
from infernum_amd.engine import BatchConfig, Runtime
from infernum_amd.parts import CacheSpec
from infernum_amd.sampling import GenerateOptions, SamplingParams
from plain_scheduler import PlainScheduler


def pair(seed, look_ahead=False):
    rng = random.Random(seed)
    ps = rng.choice((2, 4, 8))
    kw = dict(page_size=ps, num_pages=rng.choice((6, 12, 20, 40)), num_state_slots=5)
    needs = [(CacheSpec("full", 1, 16), None)]
    if seed % 3 == 0:
        needs.append((CacheSpec("window", 1, 16, window=rng.choice((3, 9))), None))
    bc = BatchConfig(max_batch_size=rng.choice((2, 3, 5)), max_prefill_tokens=rng.choice((3, 8, 64)),
                     block_size=ps, num_blocks=kw["num_pages"], max_tokens_per_step=rng.choice((8, 16, 64)),
                     step_token_multiple=random.Random(seed + 977).choice((1, 4, 8, 256)))
    out = []
    for plain in (False, True):
        eng = FakeEngine(50, needs=list(needs), **kw)
        rt = Runtime(eng, None, bc, sampler=CpuSampler())
        assert rt.look_ahead                      # the stand-in engine takes tokens "from the device" too
        rt.look_ahead = look_ahead
        if plain:
            rt.scheduler = PlainScheduler(bc)
        out.append((rt, eng))
    return rng, out[0], out[1]


def digest(plan):
    return ([t.seq.id for t in plan.decode], [(t.seq.id, list(t.token_ids), t.completes) for t in plan.prefill],
            [s.id for s in plan.set_back], [(s.id, s.error) for s in plan.finished])


@pytest.mark.parametrize("look_ahead", [False, True])
@pytest.mark.parametrize("seed", range(12))
def test_native_decisions_equal_plain_decisions(seed, look_ahead):
    """``look_ahead``: a step is decided while the tokens of the step before it are not known yet."""
    rng, (rt_a, eng_a), (rt_b, eng_b) = pair(seed, look_ahead)
    pool_tokens = eng_a.cache.page_size * eng_a.cache.groups[0].allocator.num_pages
    jobs = []
    for i in range(16):
        plen, n_new = rng.randint(1, 30), rng.randint(1, 12)
        if rng.random() < 0.1:
            plen = pool_tokens + rng.randint(0, 5)             # too large for the pool: must fail in both
        sampling = SamplingParams(temperature=0.9, top_p=1.0, seed=i) if rng.random() < 0.5 else None
        jobs.append(([rng.randrange(50) for _ in range(plen)], GenerateOptions(max_new_tokens=n_new, sampling=sampling)))
    pending, seqs_a, seqs_b = list(jobs), [], []
    steps = set_backs = 0
    while pending or not rt_a.scheduler.is_idle():
        while pending and rng.random() < 0.4:
            p, o = pending.pop(0)
            seqs_a.append(rt_a.submit(p, o))
            seqs_b.append(rt_b.submit(p, o))
        if rt_a.scheduler.is_idle():
            continue
        plan_a, plan_b = rt_a.step(), rt_b.step()
        assert digest(plan_a) == digest(plan_b), f"step {steps}"
        set_backs += len(plan_a.set_back)
        assert [s.id for s in rt_a.scheduler.running] == [s.id for s in rt_b.scheduler.running]
        assert [s.id for s in rt_a.scheduler.waiting] == [s.id for s in rt_b.scheduler.waiting]
        assert [g.allocator.num_free for g in eng_a.cache.groups] == [g.allocator.num_free for g in eng_b.cache.groups]
        eng_a.cache.check()
        steps += 1
        assert steps < 5000, "the loop does not end"
    assert rt_b.scheduler.is_idle()
    rt_a.run(), rt_b.run()                        # the tokens of the last step, if they are still on their way
    if seed in (1, 3, 4, 8, 10):
        assert set_backs >= 5, "these loads are meant to run out of pages"
    from fake_engine import reference_generation
    for (p, o), a in zip(jobs, seqs_a):
        if a.error is None:
            assert a.generated_ids == reference_generation(p, o), "a request's tokens depend on its own history only"
    for a, b in zip(seqs_a, seqs_b):
        assert (a.generated_ids, a.error, a.finish_reason, a.times_set_back) == \
               (b.generated_ids, b.error, b.finish_reason, b.times_set_back)
    rt_a.scheduler.reap(eng_a.cache)
    assert all(g.allocator.num_free == g.allocator.num_pages for g in eng_a.cache.groups)
