"""The scheduler's decisions and the generation loop, on the CPU with a stand-in step function."""
import random

import pytest

from fake_engine import CpuSampler, FakeEngine, reference_generation
from infernum_amd.engine import BatchConfig, FinishReason, GenerationError, Runtime, SequencePhase
from infernum_amd.sampling import GenerateOptions, SamplingParams


def runtime(page_size=4, num_pages=16, max_batch=4, chunk=512, budget=64, slots=8, max_seq_len=None, vocab=50,
            look_ahead=False):
    """``look_ahead``: a step is launched while the tokens of the step before it are still where the engine left
    them (the stand-in engine plays along); False: every step waits for its tokens."""
    eng = FakeEngine(vocab, page_size, num_pages, slots)
    bc = BatchConfig(max_batch_size=max_batch, max_prefill_tokens=chunk, block_size=page_size, num_blocks=num_pages,
                     max_tokens_per_step=budget)
    rt = Runtime(eng, None, bc, max_seq_len=max_seq_len, sampler=CpuSampler())
    rt.look_ahead = look_ahead
    return rt, eng


GREEDY = GenerateOptions(max_new_tokens=5)


# ---- the reference's own scheduler tests (infernum-runtime/src/scheduler.rs:435-668) -----------
def test_first_come_first_served_and_batch_limit():
    rt, eng = runtime(max_batch=2)
    seqs = [rt.submit([1, 2, 3], GREEDY) for _ in range(3)]
    plan = rt.step()
    assert [t.seq.id for t in plan.prefill] == [seqs[0].id, seqs[1].id]
    assert rt.scheduler.num_running() == 2 and rt.scheduler.num_waiting() == 1
    plan = rt.step()
    assert [t.seq.id for t in plan.decode] == [seqs[0].id, seqs[1].id] and not plan.prefill


def test_page_exhaustion_stops_admission_without_skipping():
    # 4 pages of 4: the first request takes 1, the second 2 (one page stays in hand for the running request),
    # the third does not fit, and the fourth, which would, must not overtake it
    rt, eng = runtime(page_size=4, num_pages=4, max_batch=8)
    a = rt.submit([1, 2, 3], GenerateOptions(max_new_tokens=1))
    b = rt.submit(list(range(8)), GenerateOptions(max_new_tokens=1))
    c = rt.submit(list(range(9)), GenerateOptions(max_new_tokens=1))      # 3 pages: does not fit beside a and b
    d = rt.submit([1], GenerateOptions(max_new_tokens=1))                 # would fit, but stands behind c
    plan = rt.step()
    assert [t.seq.id for t in plan.prefill] == [a.id, b.id]
    assert rt.scheduler.num_waiting() == 2
    rt.run()
    assert [s.finish_reason for s in (a, b, c, d)] == [FinishReason.LENGTH] * 4
    assert eng.cache.free_pages() == 4 and eng.cache.slots.num_free == 8


def test_finished_are_reaped_at_the_next_step():
    rt, eng = runtime()
    a = rt.submit([1, 2, 3], GenerateOptions(max_new_tokens=1))
    rt.step()
    assert a.phase == SequencePhase.FINISHED and eng.cache.has(a.id)       # still holds its pages
    plan = rt.step()
    assert plan.finished == [a] and not eng.cache.has(a.id) and rt.scheduler.is_idle()


def test_prompt_is_cut_into_portions():
    # scheduler.rs:591-628: 7 tokens with chunks of 3 -> [1,2,3] [4,5,6] [7]
    rt, eng = runtime(chunk=3)
    a = rt.submit([1, 2, 3, 4, 5, 6, 7], GenerateOptions(max_new_tokens=2))
    plans = [rt.step() for _ in range(3)]
    assert [p.prefill[0].token_ids for p in plans] == [[1, 2, 3], [4, 5, 6], [7]]
    assert [p.prefill[0].completes for p in plans] == [False, False, True]
    assert [e[0][2] for e in eng.steps] == [[], [], [0]]              # logits only where the prompt ends
    assert len(a.generated_ids) == 1 and a.phase == SequencePhase.DECODE


def test_decoding_and_portions_share_a_step():
    rt, eng = runtime(chunk=4)
    a = rt.submit([1, 2], GenerateOptions(max_new_tokens=10))
    rt.step()
    b = rt.submit(list(range(10)), GenerateOptions(max_new_tokens=3))
    plan = rt.step()
    assert [t.seq.id for t in plan.decode] == [a.id] and [t.seq.id for t in plan.prefill] == [b.id]
    assert eng.steps[-1] == [(a.id, 1, [0]), (b.id, 4, [])]
    plan = rt.step()
    assert eng.steps[-1] == [(a.id, 1, [0]), (b.id, 4, [])]
    plan = rt.step()
    assert eng.steps[-1] == [(a.id, 1, [0]), (b.id, 2, [1])]


# ---- the budget ------------------------------------------------------------------------------------
def test_token_budget_bounds_every_step_and_decoding_goes_first():
    rt, eng = runtime(num_pages=64, max_batch=4, chunk=16, budget=20, slots=8)
    seqs = [rt.submit(list(range(30)), GenerateOptions(max_new_tokens=6)) for _ in range(4)]
    while not rt.scheduler.is_idle():
        plan = rt.step()
        assert plan.num_tokens <= 20
        decoding = [s for s in rt.scheduler.running if s.phase == SequencePhase.DECODE]
    for e in eng.steps:
        assert sum(n for _, n, _ in e) <= 20
        singles = [n == 1 for _, n, _ in e]
        assert singles == sorted(singles, reverse=True)              # single tokens stand first
    # first step: 16 of the first request, 4 of the second
    assert eng.steps[0] == [(seqs[0].id, 16, []), (seqs[1].id, 4, [])]
    assert all(s.generated_ids == reference_generation(list(range(30)), GenerateOptions(max_new_tokens=6)) for s in seqs)


def _decoding_beside_a_long_prompt(chunk, budget, multiple, decoders, prompt_len):
    """``decoders`` requests decode, then a prompt of ``prompt_len`` tokens arrives; returns the sizes of its portions."""
    eng = FakeEngine(50, 16, 4096, decoders + 2)
    bc = BatchConfig(max_batch_size=decoders + 1, max_prefill_tokens=chunk, block_size=16, num_blocks=4096,
                     max_tokens_per_step=budget, step_token_multiple=multiple)
    rt = Runtime(eng, None, bc, sampler=CpuSampler())
    rt.look_ahead = False
    for _ in range(decoders):
        rt.submit([1, 2, 3], GenerateOptions(max_new_tokens=1000))
    rt.step()
    big = rt.submit(list(range(prompt_len)), GenerateOptions(max_new_tokens=1))
    sizes = []
    while big.phase != SequencePhase.DECODE and not big.generated_ids:
        plan = rt.step()
        assert len(plan.decode) == decoders and plan.num_tokens <= budget
        sizes += [len(t.token_ids) for t in plan.prefill]
    assert sum(sizes) == prompt_len
    return sizes


def test_a_portion_beside_decoded_tokens_leaves_the_step_a_multiple_of_the_tiles_rows():
    # eight decoded tokens and portions of up to 8,192 under a budget of 8,200: the step holds 8,192 tokens, not 8,200
    assert _decoding_beside_a_long_prompt(8192, 8200, 256, 8, 20000) == [8184, 8184, 3632]
    # as the reference cuts them with a multiple of 1
    assert _decoding_beside_a_long_prompt(8192, 8200, 1, 8, 20000) == [8192, 8192, 3616]
    # the defaults' portion of 512 beside twenty decoded tokens: 512 tokens in all
    assert _decoding_beside_a_long_prompt(512, 2048, 256, 20, 1100) == [492, 512 - 20, 116]
    # a portion that reaches its prompt's end is not cut, and none is cut to less than half of what it could take
    assert _decoding_beside_a_long_prompt(512, 2048, 256, 20, 500) == [500]
    assert _decoding_beside_a_long_prompt(100, 2048, 256, 250, 180) == [100, 80]
    assert _decoding_beside_a_long_prompt(100, 2048, 256, 200, 180) == [56, 56, 68]


def test_config_is_checked():
    with pytest.raises(ValueError):
        BatchConfig(max_batch_size=8, max_tokens_per_step=4)
    with pytest.raises(ValueError):
        BatchConfig(block_size=0)
    eng = FakeEngine(page_size=4, num_pages=16)
    with pytest.raises(ValueError, match="block_size"):
        Runtime(eng, None, BatchConfig(block_size=8, num_blocks=16), sampler=CpuSampler())


# ---- ending ------------------------------------------------------------------------------------------
def test_end_of_sequence_token_stops_and_is_not_emitted():
    free = reference_generation([5, 6, 7], GenerateOptions(max_new_tokens=8))
    eos = free[3]
    rt, eng = runtime()
    events = []
    a = rt.submit([5, 6, 7], GenerateOptions(max_new_tokens=8, eos_token_id=eos), lambda ev: events.append(ev) or True)
    rt.run()
    cut = free.index(eos)
    assert a.generated_ids == free[:cut] and a.finish_reason == FinishReason.STOP
    assert [e.kind for e in events] == ["token"] * cut + ["finished"] and events[-1].reason == FinishReason.STOP
    assert eng.cache.free_pages() == 16


def test_max_new_tokens_and_zero():
    rt, eng = runtime()
    a = rt.submit([1], GenerateOptions(max_new_tokens=3))
    z = rt.submit([1], GenerateOptions(max_new_tokens=0))
    assert z.phase == SequencePhase.FINISHED and z.finish_reason == FinishReason.LENGTH
    rt.run()
    assert len(a.generated_ids) == 3 and a.finish_reason == FinishReason.LENGTH and z.generated_ids == []


def test_max_seq_len():
    rt, eng = runtime(max_seq_len=6)
    a = rt.submit([1, 2, 3, 4], GenerateOptions(max_new_tokens=50))
    rt.run()
    assert len(a.generated_ids) == 2 and a.finish_reason == FinishReason.LENGTH
    with pytest.raises(ValueError, match="max_seq_len"):
        rt.submit(list(range(7)), GREEDY)
    with pytest.raises(ValueError, match="at least one"):
        rt.submit([], GREEDY)


def test_receiver_that_goes_away_cancels_and_frees():
    # infernum-runtime/src/engine.rs:463-466
    rt, eng = runtime()
    got = []
    a = rt.submit([1, 2, 3], GenerateOptions(max_new_tokens=50), lambda ev: got.append(ev) or len(got) < 3)
    b = rt.submit([4, 5], GenerateOptions(max_new_tokens=6))
    rt.run()
    assert a.finish_reason == FinishReason.CANCELLED and len(a.generated_ids) == 3
    assert len(b.generated_ids) == 6
    assert eng.cache.free_pages() == 16 and eng.cache.slots.num_free == 8


def test_stream_stopped_early_gives_everything_back():
    rt, eng = runtime()
    it = rt.generate_stream([1, 2, 3], GenerateOptions(max_new_tokens=50))
    first = [next(it) for _ in range(4)]
    it.close()
    assert first == reference_generation([1, 2, 3], GenerateOptions(max_new_tokens=4))
    assert rt.scheduler.is_idle() and eng.cache.free_pages() == 16
    assert list(rt.generate_stream([9], GenerateOptions(max_new_tokens=3))) == \
        reference_generation([9], GenerateOptions(max_new_tokens=3))


# ---- pages run out --------------------------------------------------------------------------------------
def test_out_of_pages_sets_the_last_admitted_back_and_changes_no_token():
    prompts = [[1, 2, 3, 4, 5, 6, 7], [9, 8, 7, 6, 5], [11, 12, 13]]
    opts = GenerateOptions(max_new_tokens=14)
    want = [reference_generation(p, opts) for p in prompts]
    # 8 pages of 4 = 32 tokens; the three requests end at 21 + 19 + 17 = 57 tokens
    rt, eng = runtime(page_size=4, num_pages=8, max_batch=4)
    seqs = [rt.submit(p, opts) for p in prompts]
    set_back = []
    while not rt.scheduler.is_idle():
        plan = rt.step()
        set_back += plan.set_back
        eng.cache.check()
    assert [s.generated_ids for s in seqs] == want
    assert set_back, "the pool was meant to run out"
    assert seqs[0] not in set_back                      # the oldest request is never the one to make room
    assert all(s.times_set_back > 0 for s in set(set_back))
    assert eng.cache.free_pages() == 8 and eng.cache.slots.num_free == 8
    # a request that was set back came again from the front of the queue, its own tokens appended to the prompt
    big = max(n for e in eng.steps for (r, n, w) in e if r == set_back[0].id)
    assert big > len(set_back[0].prompt_ids)


def test_sampled_tokens_do_not_change_when_set_back():
    prompts = [[3, 1, 4, 1, 5, 9], [2, 7, 1, 8], [1, 6, 1, 8, 0, 3]]
    opts = [GenerateOptions(max_new_tokens=12, sampling=SamplingParams(temperature=1.3, top_p=1.0, seed=s)) for s in (7, 8, 9)]
    want = [reference_generation(p, o) for p, o in zip(prompts, opts)]
    rt, eng = runtime(page_size=2, num_pages=14, max_batch=3)
    seqs = [rt.submit(p, o) for p, o in zip(prompts, opts)]
    n_back = 0
    while not rt.scheduler.is_idle():
        n_back += len(rt.step().set_back)
    assert [s.generated_ids for s in seqs] == want and n_back > 0


def test_a_request_larger_than_the_pool_ends_with_an_error():
    rt, eng = runtime(page_size=4, num_pages=2)
    events = []
    a = rt.submit([1, 2, 3], GenerateOptions(max_new_tokens=50), lambda ev: events.append(ev) or True)
    rt.run()
    assert a.error is not None and "too small" in a.error and events[-1].kind == "error"
    assert len(a.generated_ids) == 6                  # 3 + 5 tokens fill the 8 slots; the 6th token is chosen, not stored
    assert eng.cache.free_pages() == 2
    with pytest.raises(GenerationError, match="too small"):
        rt.generate([1, 2, 3], GenerateOptions(max_new_tokens=50))
    # a prompt longer than the pool: its portions fill the pool, then it fails
    b = rt.submit(list(range(12)), GenerateOptions(max_new_tokens=2))
    rt.run()
    assert b.error is not None and eng.cache.free_pages() == 2 and rt.scheduler.is_idle()


def test_a_long_prompt_takes_what_is_free_and_waits_for_the_rest():
    rt, eng = runtime(page_size=4, num_pages=6, max_batch=2, chunk=64)
    a = rt.submit([1, 2, 3, 4, 5, 6], GenerateOptions(max_new_tokens=2))     # 2 pages
    rt.step()
    b = rt.submit(list(range(20)), GenerateOptions(max_new_tokens=2))        # 5 pages + 1 to decode
    rt.run()
    assert a.generated_ids == reference_generation([1, 2, 3, 4, 5, 6], GenerateOptions(max_new_tokens=2))
    assert b.generated_ids == reference_generation(list(range(20)), GenerateOptions(max_new_tokens=2))
    assert a.times_set_back == 0
    assert eng.cache.free_pages() == 6


# ---- everything together, random ---------------------------------------------------------------------------
@pytest.mark.parametrize("look_ahead", [False, True])
@pytest.mark.parametrize("seed", range(5))
def test_random_load_generates_what_each_request_generates_alone(seed, look_ahead):
    rng = random.Random(seed)
    ps = rng.choice((2, 4, 8))
    rt, eng = runtime(page_size=ps, num_pages=rng.choice((12, 20, 40)), max_batch=rng.choice((2, 3, 5)),
                      chunk=rng.choice((3, 8, 64)), budget=rng.choice((8, 16, 64)), slots=5, look_ahead=look_ahead)
    pool_tokens = ps * eng.cache.groups[0].allocator.num_pages
    jobs, seqs = [], []
    for i in range(14):
        plen, n_new = rng.randint(1, 20), rng.randint(1, 12)
        if plen + n_new > pool_tokens:
            plen = 1
        sampling = SamplingParams(temperature=0.9, top_p=1.0, seed=i) if rng.random() < 0.5 else None
        o = GenerateOptions(max_new_tokens=n_new, sampling=sampling)
        jobs.append(([rng.randrange(50) for _ in range(plen)], o))
    pending = list(jobs)
    steps = 0
    while pending or not rt.scheduler.is_idle():
        while pending and rng.random() < 0.4:
            p, o = pending.pop(0)
            seqs.append(rt.submit(p, o))
        if rt.scheduler.is_idle():
            continue
        plan = rt.step()
        assert plan.num_tokens <= rt.batch_config.max_tokens_per_step
        assert rt.scheduler.num_running() <= rt.batch_config.max_batch_size
        eng.cache.check()
        steps += 1
        assert steps < 5000, "the loop does not end"
    rt.run()                                      # the tokens of the last step, if they are still on their way
    rt.scheduler.reap(eng.cache)
    for s, (p, o) in zip(seqs, jobs):
        assert s.error is None
        assert s.generated_ids == reference_generation(p, o), (s.id, s.times_set_back)
    assert eng.cache.free_pages() == eng.cache.groups[0].allocator.num_pages
    assert eng.cache.slots.num_free == 5


def test_generate_batch_and_no_kv_cache():
    rt, eng = runtime(num_pages=64)
    prompts = [[1, 2, 3], [4, 5, 6, 7, 8], [9]]
    o = GenerateOptions(max_new_tokens=7)
    want = [reference_generation(p, o) for p in prompts]
    assert rt.generate_batch(prompts, o) == want
    assert rt.generate(prompts[1], GenerateOptions(max_new_tokens=7, use_kv_cache=False)) == want[1]
    assert eng.cache.free_pages() == 64
    with pytest.raises(GenerationError, match="tokenizer"):
        rt.generate("some text", o)


def test_tokens_still_on_the_device_count_and_arrive_later():
    """A step is launched and its tokens are not on the host yet (``on_launched``): the requests count one token
    more, a request whose last token that is does nothing further but keeps its pages, and the token's arrival
    finishes it; a request that was set back meanwhile and finishes on arrival leaves the queue."""
    from infernum_amd.cache import CacheConfig, CacheManager
    from infernum_amd.engine.scheduler import BatchConfig, FinishReason, Scheduler, SequencePhase
    from infernum_amd.parts import CacheSpec
    from infernum_amd.sampling import GenerateOptions
    cache = CacheManager([(CacheSpec("full", 1, 8), None)], [None], CacheConfig(page_size=4, num_pages=16, num_state_slots=4))
    sch = Scheduler(BatchConfig(max_batch_size=2, max_prefill_tokens=8, block_size=4, num_blocks=16, max_tokens_per_step=16))
    a = sch.add_request([1, 2, 3], GenerateOptions(max_new_tokens=2))
    b = sch.add_request([4, 5, 6, 7, 8], GenerateOptions(max_new_tokens=3))
    c = sch.add_request([9], GenerateOptions(max_new_tokens=1))

    def launch(plan):
        for t in plan.prefill:
            if not cache.has(t.seq.id):
                cache.admit(t.seq.id)
            assert cache.reserve(t.seq.id, len(t.token_ids))
            cache.commit(t.seq.id, len(t.token_ids))
        for t in plan.decode:
            assert cache.reserve(t.seq.id, 1)
            cache.commit(t.seq.id, 1)
        sch.on_launched(plan)

    p1 = sch.step(cache)
    assert [t.seq for t in p1.prefill] == [a, b] and all(t.completes for t in p1.prefill) and sch.num_waiting() == 1
    launch(p1)
    assert a.pending == b.pending == 1 and a.num_tokens == 4 and a.phase == SequencePhase.DECODE and a.generated_ids == []
    p2 = sch.step(cache)                                      # decided with the first tokens still on the device
    assert [t.seq for t in p2.decode] == [a, b] and not p2.prefill
    launch(p2)
    for t in p1.prefill:
        sch.on_prefill_done(t, 50)
    assert a.generated_ids == [50] and a.pending == 1 and a.phase == SequencePhase.DECODE
    p3 = sch.step(cache)                                      # a waits for its last token: only b moves, c cannot come in
    assert [t.seq for t in p3.decode] == [b] and not p3.prefill and sch.num_waiting() == 1 and cache.has(a.id)
    launch(p3)
    for t in p2.decode:
        sch.on_decode_done(t, 51)
    assert a.phase == SequencePhase.FINISHED and a.finish_reason == FinishReason.LENGTH and a.generated_ids == [50, 51]
    assert b.generated_ids == [50, 51] and b.pending == 1
    p4 = sch.step(cache)                                      # a is reaped, c is admitted beside b, which waits
    assert not cache.has(a.id) and [t.seq for t in p4.prefill] == [c] and not p4.decode
    launch(p4)
    for t in p3.decode:
        sch.on_decode_done(t, 52)
    assert b.phase == SequencePhase.FINISHED and b.generated_ids == [50, 51, 52] and b.pending == 0
    # a request set back with a token on the way, which then turns out to be its end
    b2 = sch.add_request([4, 5], GenerateOptions(max_new_tokens=5, eos_token_id=77))
    b2.pending, b2.phase = 1, SequencePhase.WAITING           # as a set-back leaves it
    sch.handle_new_token(b2, 77)
    assert b2.phase == SequencePhase.FINISHED and b2.finish_reason == FinishReason.STOP and b2 not in sch.waiting
    for t in p4.prefill:
        sch.on_prefill_done(t, 9)
    assert c.phase == SequencePhase.FINISHED and c.generated_ids == [9]
    sch.step(cache)
    assert sch.is_idle() and cache.free_pages() == 16


def test_others_wait_for_the_pages_of_a_request_whose_last_token_is_on_its_way():
    """One step ahead, a request that has launched its last step holds pages and does nothing more.  A request
    that needs a page then is neither failed as alone in a pool too small nor set back: it waits a step, until
    the token has come and the pages are free."""
    rt, eng = runtime(page_size=2, num_pages=6, max_batch=2, look_ahead=True)
    a = rt.submit([1, 2, 3, 4], GenerateOptions(max_new_tokens=2))         # 2 pages, a third for its second token
    b = rt.submit([6, 7, 8, 9, 1], GenerateOptions(max_new_tokens=6))   # 3 pages, a fourth after a step
    plans = []
    while not rt.scheduler.is_idle():
        plans.append(rt.step())
        eng.cache.check()
        assert len(plans) < 50
    rt.run()
    assert a.error is None and b.error is None
    assert a.generated_ids == reference_generation([1, 2, 3, 4], GenerateOptions(max_new_tokens=2))
    assert b.generated_ids == reference_generation([6, 7, 8, 9, 1], GenerateOptions(max_new_tokens=6))
    assert a.times_set_back == 0 and b.times_set_back == 0
    # the step after a's last launch has nothing for b to run with: every page is held until a's token is here
    third = plans[2]
    assert not third.decode and not third.prefill and not third.set_back and not third.finished
    assert [t.seq for t in plans[3].decode] == [b] and plans[3].finished == [a]
    assert eng.cache.free_pages() == 6
