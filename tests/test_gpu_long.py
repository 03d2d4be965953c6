"""Long decoding and the first tokens of a sequence, against the plain implementation."""
import pytest
import torch

import plain_llama as P
import tiny_models as TM
import trace_tools as TT

pytestmark = pytest.mark.gpu
TOL = {"float32": 2e-5, "bfloat16": 6e-2}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name in ("B", "C"):
        for dt, tdt in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
            d = str(tmp_path_factory.mktemp(f"long{name}_{dt}"))
            TM.write_tiny(name, d, dtype=tdt)
            out[(name, dt)] = (d,) + P.read_model(d)
    return out


def _engine(d, dtype, ps, pages):
    from infernum_amd import CacheConfig, Engine
    return Engine.from_pretrained(d, dtype=dtype, cache_config=CacheConfig(page_size=ps, num_pages=pages,
                                                                           num_state_slots=4, poison_freed_pages=True))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,ps", [("B", 8), ("C", 16)])
def test_long_decoding(models, name, ps, dtype):
    """A prompt of 20 tokens, then 400 tokens one by one: many pages, many splits of the keys, and (C)
    a window that has long passed the first pages."""
    d, cfg, w = models[(name, dtype)]
    reqs = TT.make_requests(cfg["vocab_size"], (420,), seed=31)
    ref = {r: P.forward(cfg, w, t) for r, t in reqs.items()}
    steps = TT.trace_tail_one_by_one(reqs, tail=400)
    assert len(steps) == 401
    eng = _engine(d, dtype, ps, 64)
    got = TT.run_steps(eng, steps)
    worst, rms, where = TT.error_against(got, ref)
    print(f"{name} {dtype} long decoding: {worst / rms:.2e} at {where}")
    assert worst == worst and worst <= TOL[dtype] * rms, (worst / rms, where)
    eng.cache.check()
    assert all(g.allocator.num_free == 64 for g in eng.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_first_tokens(models, name, dtype):
    """Position 0 sees itself only; prompts of one and of two tokens; the second token decoded."""
    d, cfg, w = models[(name, dtype)]
    from infernum_amd import StepEntry
    eng = _engine(d, dtype, 8, 8)
    toks = [17, 201, 5, 99]
    ref = P.forward(cfg, w, toks)
    rms = ref.pow(2).mean().sqrt().item()

    def close(row, p):
        return (row.double().cpu() - ref[p]).abs().max().item() <= TOL[dtype] * rms
    one = eng.step([StepEntry("a", toks[:1], [0])])
    assert close(one[0], 0)
    nxt = eng.step([StepEntry("a", toks[1:2], [0])])
    assert close(nxt[0], 1)
    two = eng.step([StepEntry("b", toks[:2], [0, 1]), StepEntry("a", toks[2:3], [0])])
    assert close(two[0], 0) and close(two[1], 1) and close(two[2], 2)
    # a token's logits at position 0 are those of a sequence of that token alone
    alone = P.forward(cfg, w, toks[:1])[0]
    assert (one[0].double().cpu() - alone).abs().max().item() <= TOL[dtype] * rms


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n", [40, 100, 150])
@pytest.mark.parametrize("name", ["B", "C"])
def test_many_requests_decoded_together(models, name, n, dtype):
    """Many requests in one decode step, against the plain model.  150: more rows than the decode GEMM kernel
    takes, so the products go the way of many rows while attention and the rest stay on the decode kernels.
    100 (the live requests go from 100 down to about 85): the decode GEMM's variant for 65 to 128 rows, with the
    rotary kernel in front of the attention.  40: the variant for up to 64 rows, rotation inside the attention."""
    import random
    from infernum_amd import CacheConfig, Engine
    from infernum_amd.engine import StepEntry
    d, cfg, w = models[(name, dtype)]
    rng = random.Random(1)
    reqs = {f"r{i}": [rng.randrange(cfg["vocab_size"]) for _ in range(rng.randint(3, 20))] for i in range(n)}
    ref = {r: P.forward(cfg, w, t) for r, t in reqs.items()}
    eng = Engine.from_pretrained(d, dtype=dtype, cache_config=CacheConfig(page_size=8, num_pages=n * 4,
                                                                          num_state_slots=n + 2))
    names = list(reqs)
    fed = {r: max(1, len(reqs[r]) - 4) for r in names}
    for i in range(0, n, 30):
        eng.step([StepEntry(r, reqs[r][:fed[r]], []) for r in names[i:i + 30]])
    worst, live_counts = 0.0, []
    while any(fed[r] < len(reqs[r]) for r in names):
        live = [r for r in names if fed[r] < len(reqs[r])]
        live_counts.append(len(live))
        logits = eng.step([StepEntry(r, [reqs[r][fed[r]]], [0]) for r in live]).double().cpu()
        for k, r in enumerate(live):
            want = ref[r][fed[r]].double()
            worst = max(worst, float((logits[k] - want).abs().max() / want.pow(2).mean().sqrt()))
            fed[r] += 1
    assert worst <= TOL[dtype], f"worst |diff| / rms {worst:.2e}"
    lo, hi = {40: (1, 64), 100: (65, 128), 150: (129, 150)}[n]
    assert all(lo <= c <= hi for c in live_counts), live_counts
    for r in names:
        eng.end(r)
    assert eng.cache.free_pages() == n * 4


def test_recorded_decode_step_of_many_requests_equals_the_eager_one():
    """100 requests a step at layer sizes where the library's large GEMM kernels run: the step is recorded
    with the library's launches inside and replayed six times, with other work of the program between the
    replays; every replay gives the bits of the same step run launch by launch."""
    from infernum_amd import CacheConfig, Engine
    from infernum_amd.config import LlamaConfig
    from infernum_amd.engine import StepEntry
    cfg = LlamaConfig.from_dict({"model_type": "llama", "vocab_size": 32000, "hidden_size": 2048,
                                 "intermediate_size": 8192, "num_hidden_layers": 2, "num_attention_heads": 16,
                                 "num_key_value_heads": 4, "rope_theta": 500000.0, "max_position_embeddings": 4096,
                                 "rms_norm_eps": 1e-5})
    B, steps = 100, 8
    outs = {}
    for graphs in (False, True):
        eng = Engine.from_config(cfg, seed=3, dtype="bfloat16", use_graphs=graphs,
                                 cache_config=CacheConfig(page_size=16, num_pages=B * 8 + 8, num_state_slots=B + 1))
        g = torch.Generator().manual_seed(0)
        prompts = [torch.randint(0, cfg.vocab_size, (40 + (i % 7),), generator=g).tolist() for i in range(B)]
        for i in range(0, B, 25):
            eng.step([StepEntry(j, prompts[j], []) for j in range(i, min(B, i + 25))])
        toks, res = [1 + j for j in range(B)], []
        for _ in range(steps):
            logits = eng.step([StepEntry(j, [toks[j]], [0]) for j in range(B)])
            assert bool(torch.isfinite((logits * 2).sum()))           # eager work and a synchronisation between replays
            res.append(logits.cpu())
            toks = logits.argmax(-1).tolist()
        outs[graphs] = res
        assert eng.graph_replays == (steps - 1 if graphs else 0)
    for s in range(steps):
        assert torch.equal(outs[False][s], outs[True][s]), f"step {s}"
