"""Each part a model is put together from, alone on the GPU against the plain functions;
inputs and weights made so that a fault at a far key, a window's edge or a page's edge shows."""
import math

import pytest
import torch

import plain_llama as P
import tiny_models as TM
from part_harness import DEV, TOL, Steps, build, dense, rel_err, runtime

pytestmark = pytest.mark.gpu
BOTH = pytest.mark.parametrize("dtype", ["float32", "bfloat16"])


def _x(n, h, dtype, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(n, h, generator=g) * scale
    if dtype == "bfloat16":
        x = x.to(torch.bfloat16).float()
    return x


# ------------------------------------------------------------------------------ norm
@BOTH
@pytest.mark.parametrize("H,eps", [(64, 1e-5), (100, 1e-6), (4096, 3e-6)])
def test_norm_alone(dtype, H, eps):
    rt = runtime(dtype)
    norm, w = build("norm", "rmsnorm", {"size": H, "eps": eps, "init": ("uniform", 0.5, 1.5)}, rt)
    h = _x(9, H, "float32", 1)
    delta = _x(9, H, dtype, 2)
    hd = h.to(DEV).clone()
    out = norm.forward(hd, delta.to(DEV).to(rt.dtype))
    s = h.double() + delta.double()
    assert torch.allclose(hd.cpu().double(), s, atol=1e-6)                   # the sum stays 32-bit in h
    assert rel_err(out, P.rms_norm(s, w["weight"], eps)) <= TOL[dtype]
    # rows picked for the head: h stays as it is
    rows = torch.tensor([7, 2], dtype=torch.int32, device=DEV)
    hd2 = h.to(DEV).clone()
    out2 = norm.forward(hd2, delta.to(DEV).to(rt.dtype), rows=rows)
    assert torch.equal(hd2.cpu(), h)
    assert rel_err(out2, P.rms_norm(s[[7, 2]], w["weight"], eps)) <= TOL[dtype]
    # a row near zero shows where eps stands
    tiny = torch.zeros(1, H)
    tiny[0, 0] = 1e-4
    out3 = norm.forward(tiny.to(DEV), None)
    want3 = P.rms_norm(tiny.double(), w["weight"], eps)[0, 0].item()
    assert abs(out3[0, 0].item() - want3) <= (2.0 ** -8 if dtype == "bfloat16" else 1e-6) * abs(want3)
    assert out3[0, 1:].abs().max().item() == 0.0


# -------------------------------------------------------------------------- position
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_position_frequencies(name):
    cfg = TM.tiny_config(name)
    rt = runtime("float32")
    from infernum_amd.parts import PartSpec, make_part
    scaling = cfg.rope_scaling.to_dict() if cfg.rope_scaling else None
    rope = make_part("position", PartSpec("rope", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta,
                                                   "scaling": scaling}), rt)
    want = P.rope_frequencies(cfg.head_dim, cfg.rope_theta, scaling)
    assert rope.inv_freq.dtype == torch.float64 and rope.rotary_dim == cfg.head_dim
    assert torch.allclose(rope.inv_freq.cpu(), want, rtol=1e-15, atol=0)
    if name == "B":      # the three bands: kept, blended, divided by the factor
        plain = P.rope_frequencies(cfg.head_dim, cfg.rope_theta, None)
        r = (rope.inv_freq.cpu().double() / plain)
        assert torch.allclose(r[:2], torch.ones(2, dtype=torch.float64)) and 0.125 < r[2] < 1.0
        assert torch.allclose(r[3:], torch.full((13,), 0.125, dtype=torch.float64))
    none = make_part("position", PartSpec("none", {}), rt)
    assert none.inv_freq is None and none.rotary_dim == 0


# ------------------------------------------------------------------- feed-forward
@BOTH
@pytest.mark.parametrize("H,I,N", [(64, 176, 5), (96, 200, 70), (128, 352, 1)])
def test_feed_forward_alone(dtype, H, I, N):
    rt = runtime(dtype)
    ff, w = build("feed_forward", "swiglu", {"hidden_size": H, "intermediate_size": I}, rt)
    x = _x(N, H, dtype, 3)
    out = dense(ff.forward(x.to(DEV).to(rt.dtype)), rt)
    xd = x.double()
    want = P.linear(P.swiglu(P.linear(xd, w["gate_proj.weight"]), P.linear(xd, w["up_proj.weight"])),
                    w["down_proj.weight"])
    assert out.dtype == rt.dtype and rel_err(out, want) <= TOL[dtype]


# ---------------------------------------------------------------- embedding and head
@BOTH
def test_embedding_and_head_alone(dtype):
    rt = runtime(dtype)
    V, H = 250, 96
    emb, w = build("embedding", "token", {"vocab_size": V, "hidden_size": H}, rt)
    head, wh = build("head", "linear", {"vocab_size": V, "hidden_size": H}, rt, seed=5)
    steps = Steps([], rt)
    ids = [7, 249, 0, 7, 100]
    ctx, packed = steps.begin([("r", len(ids))])
    ctx.token_ids.copy_(torch.tensor(ids, dtype=torch.int32))
    h = emb.forward(ctx)
    assert h.dtype == torch.float32 and torch.equal(h.cpu().double(), w["weight"][ids])
    x = _x(3, H, dtype, 4)
    logits = head.forward(x.to(DEV).to(rt.dtype))
    assert logits.dtype == torch.float32 and tuple(logits.shape) == (3, V)
    assert rel_err(logits, P.linear(x.double(), wh["weight"])) <= (2e-5 if dtype == "float32" else 2e-5)
    # bf16 operands are exact in fp32 products and the sum is fp32: the head does not round its result


# ----------------------------------------------------------------------- attention
def _plain_attention(x, w, nh, nkv, d, freqs, window, scale=None):
    T = x.shape[0]
    q = P.linear(x, w["q_proj.weight"]).reshape(T, nh, d)
    k = P.linear(x, w["k_proj.weight"]).reshape(T, nkv, d)
    v = P.linear(x, w["v_proj.weight"]).reshape(T, nkv, d)
    if freqs is not None:
        pos = torch.arange(T)
        q, k = P.rope(q, pos, freqs), P.rope(k, pos, freqs)
    a = P.causal_attention(q, k, v, scale if scale is not None else 1.0 / math.sqrt(d), window)
    return P.linear(a.reshape(T, nh * d), w["o_proj.weight"])


def _run_attention(att, rt, x, cuts, page_size, window_pages=64):
    """x [T, H] of one request through the mixer, cut into steps of the given sizes."""
    steps = Steps([(att.cache_spec(), None)], rt, page_size=page_size, num_pages=window_pages, poison=True)
    outs, p = [], 0
    for n in cuts:
        ctx, packed = steps.begin([("r", n)])
        outs.append(dense(att.forward(x[p:p + n].to(DEV).to(rt.dtype).contiguous(), ctx, steps.views[0]), rt).cpu())
        steps.end(packed)
        p += n
    assert p == x.shape[0]
    return torch.cat(outs)


ATT_CASES = [
    # H, nh, nkv, d, theta, scaling, window, page size
    (64, 4, 2, 16, 1e4, None, None, 4),
    (128, 4, 1, 32, 5e5, dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                              original_max_position_embeddings=64), None, 8),
    (96, 6, 3, 48, 2e4, None, 24, 16),
    (80, 5, 5, 16, 1e4, None, 7, 4),
]


@BOTH
@pytest.mark.parametrize("case", range(len(ATT_CASES)))
def test_attention_alone_whole_portions_and_token_by_token(dtype, case):
    H, nh, nkv, d, theta, scaling, window, ps = ATT_CASES[case]
    rt = runtime(dtype)
    pos = {"kind": "rope", "params": {"head_dim": d, "theta": theta, "scaling": scaling}}
    att, w = build("mixer", "attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                          "position": pos, "window": window}, rt, seed=case)
    T = 75
    x = _x(T, H, dtype, 10 + case)
    want = _plain_attention(x.double(), w, nh, nkv, d, P.rope_frequencies(d, theta, scaling), window)
    for cuts in ([T], [40] + [1] * 35, [8, 5, 3, 2, 2, 7, 13, 2, 31, 2]):
        got = _run_attention(att, rt, x, cuts, ps)
        assert rel_err(got, want) <= TOL[dtype], cuts


def _picking_weights(nh, nkv):
    """Width 48, head size 16: queries are the values 0..15 of a row, keys 16..31, values 32..47 (for
    every head), and the output projection copies the heads' outputs: scores and outputs can be set
    by hand through the input rows."""
    q, k, v = torch.eye(48)[:16], torch.eye(48)[16:32], torch.eye(48)[32:]
    return {"q_proj.weight": torch.cat([q] * nh), "k_proj.weight": torch.cat([k] * nkv),
            "v_proj.weight": torch.cat([v] * nkv), "o_proj.weight": torch.eye(48, 16 * nh)}


@BOTH
def test_attention_finds_one_far_key_among_hundreds(dtype):
    """Key 3 of 700 is made to stand out for the last query: nearly all of the last row's weight lies
    on it, so a kernel that loses early keys (a wrong first tile, a split that is dropped) shows."""
    H, nh, nkv, d = 48, 2, 1, 16
    rt = runtime(dtype)
    w = _picking_weights(nh, nkv)
    w["o_proj.weight"] = torch.randn(48, 32, generator=torch.Generator().manual_seed(1)) * 0.2
    att, wd = build("mixer", "attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                           "position": {"kind": "none", "params": {}}}, rt, tensors=w)
    T = 700
    x = _x(T, H, dtype, 2, scale=0.3)
    x[3, 16:32] = 4.0
    x[T - 1, :16] = 4.0                                     # score 16 * 16 / 4 = 64 against |others| of a few
    want = _plain_attention(x.double(), wd, nh, nkv, d, None, None)
    near_v3 = P.linear(x[3, 32:].double().repeat(2)[None], wd["o_proj.weight"])[0]
    assert (want[T - 1] - near_v3).abs().max() < 1e-3 * near_v3.abs().max()        # the plain result is v_3
    for cuts, ps in (([T], 16), ([T - 1, 1], 16), ([650] + [1] * 50, 4), ([300, 399, 1], 8)):
        got = _run_attention(att, rt, x, cuts, ps, window_pages=256)
        assert rel_err(got, want) <= TOL[dtype], (cuts, ps)
        assert (got[T - 1].double() - near_v3).abs().max() < 0.05 * near_v3.abs().max()


@BOTH
@pytest.mark.parametrize("ps", [4, 16])
def test_attention_window_edge(dtype, ps):
    """Window 24: for the query at p the key p-23 is the last one inside, p-24 the first one outside.
    Both are made to stand out in turn; the output must follow the one inside and not see the other."""
    H, nh, nkv, d, W = 48, 2, 2, 16, 24
    rt = runtime(dtype)
    w = _picking_weights(nh, nkv)
    att, wd = build("mixer", "attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                           "position": {"kind": "none", "params": {}}, "window": W}, rt, tensors=w)
    T = 90
    for loud in (T - 1 - 23, T - 1 - 24):
        x = _x(T, H, dtype, 3, scale=0.3)
        x[loud, 16:32] = 4.0
        x[T - 1, :16] = 4.0
        want = _plain_attention(x.double(), wd, nh, nkv, d, None, W)
        inside = loud == T - 1 - 23
        follows = (want[T - 1, :16] - x[loud, 32:].double()).abs().max() < 1e-3
        assert follows == inside
        for cuts in ([T], [T - 1, 1], [60] + [1] * 30, [50, 38, 2]):
            got = _run_attention(att, rt, x, cuts, ps)
            assert rel_err(got, want) <= TOL[dtype], (loud, cuts)


@BOTH
def test_attention_key_at_a_pages_edge_with_shuffled_pages(dtype):
    """The loud key stands in the last slot of a page, then in the first slot of the next; the
    request's pages are not in rising order (other requests took and freed pages before)."""
    H, nh, nkv, d, ps = 48, 2, 1, 16, 8
    rt = runtime(dtype)
    w = _picking_weights(nh, nkv)
    att, wd = build("mixer", "attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                           "position": {"kind": "none", "params": {}}}, rt, tensors=w)
    T = 50
    for loud in (23, 24):
        steps = Steps([(att.cache_spec(), None)], rt, page_size=ps, num_pages=12, poison=True)
        # churn: three requests take pages, two give them back, so the free list is out of order
        for r, n in (("a", 20), ("b", 9), ("c", 17)):
            ctx, packed = steps.begin([(r, n)])
            att.forward(_x(n, H, dtype, 9).to(DEV).to(rt.dtype), ctx, steps.views[0])
            steps.end(packed)
        steps.cache.release("a"); steps.cache.release("c")
        x = _x(T, H, dtype, 4, scale=0.3)
        x[loud, 16:32] = 4.0
        x[T - 1, :16] = 4.0
        want = _plain_attention(x.double(), wd, nh, nkv, d, None, None)
        outs, p = [], 0
        for n in (30, 19, 1):
            ctx, packed = steps.begin([("r", n)])
            outs.append(dense(att.forward(x[p:p + n].to(DEV).to(rt.dtype).contiguous(), ctx, steps.views[0]), rt).cpu())
            steps.end(packed)
            p += n
        pages = steps.cache.block_table(0, "r").pages
        assert pages != sorted(pages), "the pages were meant to be out of order"
        got = torch.cat(outs)
        assert rel_err(got, want) <= TOL[dtype], loud
        assert (got[T - 1, :16].double() - x[loud, 32:].double()).abs().max() < 0.05


# --------------------------------------------------------------------------- block
@BOTH
def test_block_alone(dtype):
    """h' = h + mixer(norm1(h + pending)); returns feed_forward(norm2(h')) as the next pending delta."""
    from infernum_amd.parts import block_factory
    H, nh, nkv, d, I, eps = 64, 4, 2, 16, 176, 1e-5
    rt = runtime(dtype)
    pos = {"kind": "rope", "params": {"head_dim": d, "theta": 1e4, "scaling": None}}
    att, wa = build("mixer", "attention", {"hidden_size": H, "num_heads": nh, "num_kv_heads": nkv, "head_dim": d,
                                           "position": pos}, rt, seed=1)
    ff, wf = build("feed_forward", "swiglu", {"hidden_size": H, "intermediate_size": I}, rt, seed=2)
    n1, w1 = build("norm", "rmsnorm", {"size": H, "eps": eps}, rt, seed=3)
    n2, w2 = build("norm", "rmsnorm", {"size": H, "eps": eps}, rt, seed=4)
    block = block_factory("prenorm")(rt, att, ff, n1, n2, {})
    T = 21
    h0, pending = _x(T, H, "float32", 5), _x(T, H, dtype, 6)
    steps = Steps([(att.cache_spec(), None)], rt, page_size=4)
    ctx, packed = steps.begin([("r", T)])
    hd = h0.to(DEV).clone()
    out = dense(block.forward(hd, pending.to(DEV).to(rt.dtype), ctx, steps.views[0]), rt)
    s = h0.double() + pending.double()
    a = _plain_attention(P.rms_norm(s, w1["weight"], eps), wa, nh, nkv, d, P.rope_frequencies(d, 1e4, None), None)
    h1 = s + a
    m = P.rms_norm(h1, w2["weight"], eps)
    want = P.linear(P.swiglu(P.linear(m, wf["gate_proj.weight"]), P.linear(m, wf["up_proj.weight"])),
                    wf["down_proj.weight"])
    assert rel_err(hd, h1) <= TOL[dtype] and rel_err(out, want) <= 2 * TOL[dtype]
