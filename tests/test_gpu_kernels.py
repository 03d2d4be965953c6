"""Each HIP kernel alone against a plain PyTorch fp32 reference of the same
operation, at sizes other than the tiny models': widths and vocabularies that are
no power of two, head sizes in steps of 16, odd page sizes, grouped heads."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def K():
    from infernum_amd.kernels import api
    return api


def _rand(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


# ------------------------------------------------------------------------ rows
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,V", [(100, 77), (4096, 1000), (1536, 333), (5120, 50), (8200, 9)])
def test_embed(dtype, H, V):
    table = _rand(V, H, dtype=dtype)
    ids = torch.tensor([0, V - 1, 5, 5, V // 2], dtype=torch.int32, device=DEV)
    out = torch.empty(5, H, dtype=torch.float32, device=DEV)
    K().embed(table, ids, out)
    assert torch.equal(out, table[ids.long()].float())


def test_embed_bad_id_gives_nan_not_a_fault():
    table = _rand(10, 64)
    ids = torch.tensor([3, 10, -1], dtype=torch.int32, device=DEV)
    out = torch.zeros(3, 64, device=DEV)
    K().embed(table, ids, out)
    assert torch.equal(out[0], table[3]) and out[1].isnan().all() and out[2].isnan().all()


@pytest.mark.parametrize("dtype,wdtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                          (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("H", [4, 100, 2048, 5120])
def test_add_rmsnorm(dtype, wdtype, H):
    N, eps = 7, 1e-6
    h = _rand(N, H, seed=1)
    delta = _rand(N, H, dtype=dtype, seed=2)
    w = (_rand(H, seed=3).abs() + 0.5).to(wdtype)
    h0 = h.clone()
    out = torch.empty(N, H, dtype=dtype, device=DEV)
    K().add_rmsnorm(h, delta, w, eps, out)
    s = h0.double() + delta.double()
    assert torch.allclose(h.double(), s, atol=1e-6)                   # the sum is stored in fp32
    want = s * torch.rsqrt((s * s).mean(-1, keepdim=True) + eps) * w.double()
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(out.double(), want, atol=tol, rtol=tol)
    # without a delta, and on selected rows only (h untouched)
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    h1 = h.clone()
    out2 = torch.empty(3, H, dtype=dtype, device=DEV)
    K().add_rmsnorm(h, delta, w, eps, out2, rows)
    assert torch.equal(h, h1)
    s2 = (h1.double() + delta.double())[rows.long()]
    want2 = s2 * torch.rsqrt((s2 * s2).mean(-1, keepdim=True) + eps) * w.double()
    assert torch.allclose(out2.double(), want2, atol=tol, rtol=tol)


@pytest.mark.parametrize("H", [100, 1024, 4096, 6000])
@pytest.mark.parametrize("S", [1, 3, 8])
def test_add_rmsnorm_joins_partial_sums(H, S):
    """delta as a stack of fp32 partial sums [S, N, H] (what a split matrix product leaves)."""
    api = K()
    N, eps = 5, 1e-5
    h = _rand(N, H, seed=1)
    parts = _rand(S, N, H, seed=2)
    w = (_rand(H, seed=3).abs() + 0.5).to(torch.bfloat16)
    h0 = h.clone()
    out = torch.empty(N, H, dtype=torch.bfloat16, device=DEV)
    api.add_rmsnorm(h, api.SplitSum(parts), w, eps, out)
    s = h0.double() + parts.double().sum(0)
    assert torch.allclose(h.double(), s, atol=1e-5)
    want = s * torch.rsqrt((s * s).mean(-1, keepdim=True) + eps) * w.double()
    assert torch.allclose(out.double(), want, atol=1e-2, rtol=1e-2)
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, H, dtype=torch.bfloat16, device=DEV)
    api.add_rmsnorm(h0.clone(), api.SplitSum(parts), w, eps, out2, rows)
    assert torch.equal(out2, out[rows.long()])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [2048, 3000, 4096, 5120, 1000])
def test_add_rmsnorm_of_many_rows_equals_that_of_few(dtype, H):
    """Many rows take a kernel with fewer threads per row than a few rows do: the same rows in one call of
    1,100 and in calls of 20 leave the same bits (the sums of squares are taken in one order)."""
    N, eps = 1100, 1e-5
    h = _rand(N, H, seed=4)
    delta = _rand(N, H, dtype=dtype, seed=5)
    w = (_rand(H, seed=6).abs() + 0.5).to(dtype)
    h_many, h_few = h.clone(), h.clone()
    out_many = torch.empty(N, H, dtype=dtype, device=DEV)
    out_few = torch.empty(N, H, dtype=dtype, device=DEV)
    K().add_rmsnorm(h_many, delta, w, eps, out_many)
    for n0 in range(0, N, 20):
        K().add_rmsnorm(h_few[n0:n0 + 20], delta[n0:n0 + 20], w, eps, out_few[n0:n0 + 20])
    assert torch.equal(h_many, h_few) and torch.equal(out_many, out_few)
    s = h.double() + delta.double()
    want = s * torch.rsqrt((s * s).mean(-1, keepdim=True) + eps) * w.double()
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert torch.allclose(out_many.double(), want, atol=tol, rtol=tol)


def test_rmsnorm_reference_vector():
    # infernum-cuda/src/inner/cuda/ops/rmsnorm.rs:171-203
    h = torch.tensor([[1.0, 2.0, 3.0, 4.0]], device=DEV)
    out = torch.empty(1, 4, device=DEV)
    K().add_rmsnorm(h, None, torch.ones(4, device=DEV), 1e-6, out)
    assert torch.allclose(out, h / math.sqrt(7.5), atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu(dtype):
    N, I = 5, 172
    gu = _rand(N, 2 * I, dtype=dtype, scale=3.0)
    out = torch.empty(N, I, dtype=dtype, device=DEV)
    K().swiglu(gu, out)
    g, u = gu[:, :I].double(), gu[:, I:].double()
    want = g / (1 + torch.exp(-g)) * u
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    assert torch.allclose(out.double(), want, atol=tol, rtol=tol)


def test_rope_reference_vector_and_pages():
    # infernum-cuda/src/inner/cuda/ops/rope.rs:835-885: [a,b,c,d] at position 1, theta 1e4
    nh, nkv, d, ps = 1, 1, 4, 3
    qkv = torch.tensor([[1.0, 2, 3, 4, 1, 2, 3, 4, 9, 8, 7, 6]], device=DEV)
    inv = torch.tensor([1.0, 0.01], device=DEV)
    kp = torch.zeros(5, nkv, ps, d, device=DEV)
    vp = torch.zeros(5, nkv, d, ps, device=DEV)
    K().rope_kv_append(qkv, torch.tensor([1], dtype=torch.int32, device=DEV), inv, nh, nkv, d, d,
                       torch.tensor([2 * ps + 1], dtype=torch.int32, device=DEV), kp, vp)
    c0, s0, c1, s1 = math.cos(1.0), math.sin(1.0), math.cos(0.01), math.sin(0.01)
    want = torch.tensor([1 * c0 - 3 * s0, 2 * c1 - 4 * s1, 3 * c0 + 1 * s0, 4 * c1 + 2 * s1], device=DEV)
    assert torch.allclose(qkv[0, :4], want, atol=1e-6)
    assert torch.allclose(kp[2, 0, 1], want, atol=1e-6)
    assert torch.equal(vp[2, 0, :, 1], torch.tensor([9.0, 8, 7, 6], device=DEV))     # values lie transposed
    assert kp.abs().sum() == kp[2, 0, 1].abs().sum() and vp.abs().sum() == vp[2, 0, :, 1].abs().sum()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,rot,ps", [(6, 2, 48, 48, 5), (8, 8, 16, 16, 16), (5, 1, 128, 64, 7)])
def test_rope_kv_append(dtype, nh, nkv, d, rot, ps):
    N, pages = 9, 6
    qkv = _rand(N, (nh + 2 * nkv) * d, dtype=dtype)
    q0 = qkv.clone()
    pos = torch.tensor([0, 1, 2, 40, 41, 1000, 7, 8, 9], dtype=torch.int32, device=DEV)
    inv = (10000.0 ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot)).float().to(DEV)
    slots = torch.randperm(pages * ps)[:N].to(torch.int32).to(DEV)
    kp = torch.zeros(pages, nkv, ps, d, dtype=dtype, device=DEV)
    vp = torch.zeros(pages, nkv, d, ps, dtype=dtype, device=DEV)
    K().rope_kv_append(qkv, pos, inv, nh, nkv, d, rot, slots, kp, vp)
    x = q0.double().reshape(N, nh + 2 * nkv, d)
    ang = (pos.float()[:, None] * inv[None, :]).double()      # angles are fp32 products, as in the kernel
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[:, :nh + nkv, :rot // 2], x[:, :nh + nkv, rot // 2:rot]
    roted = x[:, :nh + nkv].clone()
    roted[..., :rot // 2] = a * c - b * s
    roted[..., rot // 2:rot] = a * s + b * c
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(qkv[:, :nh * d].double().reshape(N, nh, d), roted[:, :nh], atol=tol, rtol=tol)
    for n in range(N):
        p, o = int(slots[n]) // ps, int(slots[n]) % ps
        assert torch.allclose(kp[p, :, o].double(), roted[n, nh:], atol=tol, rtol=tol)
        assert torch.equal(vp[p, :, :, o], q0[n].reshape(nh + 2 * nkv, d)[nh + nkv:])
    # queries only (a layer that reads another's keys and values)
    q2 = q0[:, :nh * d].contiguous()
    K().rope_kv_append(q2, pos, inv, nh, nkv, d, rot)
    assert torch.allclose(q2.double().reshape(N, nh, d), roted[:, :nh], atol=tol, rtol=tol)


@pytest.mark.parametrize("N", [6, 40])
def test_rope_angles_at_far_positions(N):
    """With a table of float64 frequencies the angle is formed in float64: positions of a million are rotated as
    exactly as position 1 (an fp32 product would be off by 0.06 rad there); both kernels (few tokens, many)."""
    nh, nkv, d, rot, ps = 2, 1, 64, 64, 8
    qkv = _rand(N, (nh + 2 * nkv) * d, seed=5)
    pos = torch.tensor([1, 1000, 65537, 999983, 1000000, 16777215] * (N // 6 + 1), dtype=torch.int32, device=DEV)[:N].contiguous()
    inv64 = 500000.0 ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot)
    slots = torch.arange(N, dtype=torch.int32, device=DEV)
    kp, vp = torch.zeros(N // ps + 1, nkv, ps, d, device=DEV), torch.zeros(N // ps + 1, nkv, d, ps, device=DEV)
    got = qkv.clone()
    K().rope_kv_append(got, pos, inv64.to(DEV), nh, nkv, d, rot, slots, kp, vp)
    x = qkv.double().cpu().reshape(N, nh + 2 * nkv, d)
    ang = pos.cpu().double()[:, None] * inv64[None, :]
    c, s_ = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[:, :nh, :rot // 2], x[:, :nh, rot // 2:]
    g = got[:, :nh * d].double().cpu().reshape(N, nh, d)
    assert (g[..., :rot // 2] - (a * c - b * s_)).abs().max() <= 3e-6
    assert (g[..., rot // 2:] - (a * s_ + b * c)).abs().max() <= 3e-6
    # the same positions with the table rounded to fp32 are visibly off: the test can tell the two apart
    off = qkv.clone()
    K().rope_kv_append(off, pos, inv64.float().to(DEV), nh, nkv, d, rot)
    assert (off[:, :nh * d].double().cpu().reshape(N, nh, d)[..., :rot // 2] - (a * c - b * s_)).abs().max() > 1e-3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,rot,ps", [(6, 2, 48, 48, 5), (32, 8, 128, 128, 16), (5, 1, 128, 64, 7), (3, 3, 20, 8, 4)])
def test_rope_of_many_tokens_equals_rope_of_few(dtype, nh, nkv, d, rot, ps):
    """A portion of a prompt takes another kernel (one workgroup per token) than a few decoded tokens (one wave
    per token and head): the same tokens in one call of 70 and in calls of 10 leave the same bits."""
    N, pages = 70, 20
    qkv = _rand(N, (nh + 2 * nkv) * d, dtype=dtype, seed=11)
    pos = (torch.arange(N, dtype=torch.int32) * 37 % 2000).to(DEV)
    inv = (10000.0 ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot)).float().to(DEV)
    slots = torch.randperm(pages * ps)[:N].to(torch.int32).to(DEV)
    many, few = qkv.clone(), qkv.clone()
    kp1, vp1 = torch.zeros(pages, nkv, ps, d, dtype=dtype, device=DEV), torch.zeros(pages, nkv, d, ps, dtype=dtype, device=DEV)
    kp2, vp2 = torch.zeros_like(kp1), torch.zeros_like(vp1)
    K().rope_kv_append(many, pos, inv, nh, nkv, d, rot, slots, kp1, vp1)
    for n0 in range(0, N, 10):
        part = few[n0:n0 + 10]
        K().rope_kv_append(part, pos[n0:n0 + 10].contiguous(), inv, nh, nkv, d, rot, slots[n0:n0 + 10].contiguous(), kp2, vp2)
    assert torch.equal(many, few) and torch.equal(kp1, kp2) and torch.equal(vp1, vp2)
    # and both are the rotation: against fp64 at a few places
    x = qkv.double().reshape(N, nh + 2 * nkv, d)
    ang = (pos.float()[:, None] * inv[None, :]).double()
    c, s_ = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[:, :nh, :rot // 2], x[:, :nh, rot // 2:rot]
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    got = many[:, :nh * d].double().reshape(N, nh, d)
    assert torch.allclose(got[..., :rot // 2], a * c - b * s_, atol=tol, rtol=tol)
    assert torch.allclose(got[..., rot // 2:rot], a * s_ + b * c, atol=tol, rtol=tol)
    assert torch.equal(got[..., rot:], x[:, :nh, rot:])
    # a separate output for the queries (the source stays as it is)
    src = qkv.clone()
    q_out = torch.full((N, nh * d), float("nan"), dtype=dtype, device=DEV)
    kp3, vp3 = torch.zeros_like(kp1), torch.zeros_like(vp1)
    K().rope_kv_append(src, pos, inv, nh, nkv, d, rot, slots, kp3, vp3, q_out=q_out)
    assert torch.equal(q_out, many[:, :nh * d]) and torch.equal(src, qkv) and torch.equal(kp3, kp1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,ps", [(40, 40, 128, 16), (8, 2, 64, 8), (4, 4, 256, 32), (6, 3, 48, 24), (4, 2, 32, 12)])
def test_values_of_a_portion_go_to_their_pages_in_runs(dtype, nh, nkv, d, ps):
    """The values of many tokens are written by a launch of their own that takes the tokens which follow each other
    in a page eight at a time: three requests' portions in one call (one starts in the middle of a page, pages in any
    order, a token without a slot between them, a count that is no multiple of sixteen) leave the pages that
    calls of a few tokens leave, which write every value alone."""
    pages = 40
    order = torch.randperm(pages, generator=torch.Generator().manual_seed(ps + d)).tolist()
    slots, pos = [], []
    for first, count in ((5, 45), (0, 33), (ps - 1, 2 * ps + 3)):
        need = (first + count + ps - 1) // ps
        table, order = order[:need], order[need:]
        for p_ in range(first, first + count):
            slots.append(table[p_ // ps] * ps + p_ % ps)
            pos.append(p_)
    slots[50] = -1                                           # a token whose key and value are not kept
    N = len(slots)
    assert N % 16 != 0 and N >= 32
    qkv = _rand(N, (nh + 2 * nkv) * d, dtype=dtype, seed=13)
    slots_t, pos_t = torch.tensor(slots, dtype=torch.int32, device=DEV), torch.tensor(pos, dtype=torch.int32, device=DEV)
    inv = (10000.0 ** (-torch.arange(d // 2, dtype=torch.float64) * 2 / d)).to(DEV)
    kp1 = torch.full((pages, nkv, ps, d), 7.0, dtype=dtype, device=DEV)
    vp1 = torch.full((pages, nkv, d, ps), 7.0, dtype=dtype, device=DEV)
    kp2, vp2 = kp1.clone(), vp1.clone()
    many, few = qkv.clone(), qkv.clone()
    K().rope_kv_append(many, pos_t, inv, nh, nkv, d, d, slots_t, kp1, vp1)
    for n0 in range(0, N, 10):
        K().rope_kv_append(few[n0:n0 + 10], pos_t[n0:n0 + 10].contiguous(), inv, nh, nkv, d, d,
                           slots_t[n0:n0 + 10].contiguous(), kp2, vp2)
    assert torch.equal(many, few) and torch.equal(kp1, kp2) and torch.equal(vp1, vp2)
    # the values themselves, at their places; what no token owns is untouched
    want = torch.full_like(vp1, 7.0)
    v = qkv[:, (nh + nkv) * d:].reshape(N, nkv, d)
    for n, sl in enumerate(slots):
        if sl >= 0:
            want[sl // ps, :, :, sl % ps] = v[n]
    assert torch.equal(vp1, want)


# -------------------------------------------------------------- matrix products
@pytest.mark.parametrize("M,N,K_", [(1, 250, 96), (7, 384, 176), (70, 129, 1000), (300, 64, 33)])
def test_gemm_generic(M, N, K_):
    a, w = _rand(M, K_, seed=4), _rand(N, K_, seed=5)
    out = torch.empty(M, N, device=DEV)
    K().gemm_generic(a, w, out)
    want = a.double() @ w.double().t()
    assert torch.allclose(out.double(), want, atol=1e-4, rtol=1e-5)
    # the same rows alone give the same bits: the order of summation does not depend on M
    one = torch.empty(1, N, device=DEV)
    K().gemm_generic(a[M - 1:M], w, one)
    assert torch.equal(one[0], out[M - 1])
    ab, wb = a.bfloat16(), w.bfloat16()
    outb = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    K().gemm_generic(ab, wb, outb)
    wantb = ab.double() @ wb.double().t()
    assert torch.allclose(outb.double(), wantb, atol=0.3, rtol=2e-2)
    outf = torch.empty(M, N, device=DEV)
    K().gemm_generic(ab, wb, outf)
    assert torch.allclose(outf.double(), wantb, atol=1e-3, rtol=1e-4)


@pytest.mark.parametrize("M", [1, 2, 8, 16, 17, 33, 64, 65, 81, 100, 128])
@pytest.mark.parametrize("N,K_", [(250, 96), (384, 176), (4096, 4096), (1000, 14336), (16, 8), (129, 1000)])
def test_gemm_skinny(M, N, K_):
    api = K()
    a, w = _rand(M, K_, dtype=torch.bfloat16, seed=6), _rand(N, K_, dtype=torch.bfloat16, seed=7)
    want = a.double() @ w.double().t()
    outf = torch.full((M, N), float("nan"), device=DEV)
    api.gemm_skinny(a, w, outf)
    scale = math.sqrt(K_)
    assert (outf.double() - want).abs().max().item() <= 2e-5 * scale + 1e-6 * want.abs().max().item()
    outb = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    api.gemm_skinny(a, w, outb)
    assert torch.equal(outb, outf.bfloat16())
    # a row's result does not depend on how many other rows there are
    one = torch.empty(1, N, device=DEV)
    api.gemm_skinny(a[M - 1:M].contiguous(), w, one)
    assert torch.equal(one[0], outf[M - 1])


@pytest.mark.parametrize("M", [1, 8, 40, 64, 72, 128])
@pytest.mark.parametrize("N,K_", [(352, 128), (4096, 4096), (1000, 14336), (28672, 4096), (130, 1000)])
def test_gemm_skinny_partial_sums_and_swiglu(M, N, K_):
    api = K()
    a, w = _rand(M, K_, dtype=torch.bfloat16, seed=6), _rand(N, K_, dtype=torch.bfloat16, scale=0.05, seed=7)
    plain = api.gemm_skinny(a, w, out_dtype=torch.float32)
    want = a.double() @ w.double().t()
    assert (plain.double() - want).abs().max().item() <= 2e-5 * math.sqrt(K_) * 0.05 + 1e-6 * want.abs().max().item()
    kept = api.gemm_skinny(a, w, keep_split=True)
    S = api.gemm_skinny_splits(N, K_)
    if S > 1:
        assert isinstance(kept, api.SplitSum) and tuple(kept.parts.shape) == (S, M, N)
        total = kept.parts[0].clone()
        for s_ in range(1, S):
            total += kept.parts[s_]                      # the join adds the parts in the order of their index
        assert torch.equal(total, plain)
    else:
        assert torch.equal(kept, plain.bfloat16())
    act = api.gemm_skinny(a, w, epilogue="swiglu", out_dtype=torch.float32)
    assert tuple(act.shape) == (M, N // 2)
    # against the activation of the exact sums: the kernel's sums carry fp32 rounding (a tile of columns walks K from
    # a start of its own, so they are not the sums of the product without the activation bit for bit); silu has a
    # slope of at most 1.1
    g, u = want[:, :N // 2], want[:, N // 2:]
    e = 2e-5 * math.sqrt(K_) * 0.05 + 1e-6 * want.abs().max().item()
    assert bool(((act.double() - g / (1 + torch.exp(-g)) * u).abs() <= e * (1.1 * u.abs() + g.abs() + e) + 1e-6).all())
    actb = api.gemm_skinny(a, w, epilogue="swiglu")
    assert torch.equal(actb, act.bfloat16())


def test_gemm_skinny_takes_the_measured_number_of_parts_for_the_shapes_of_its_table():
    """The table of measured shapes is in force from the library's load on: its shapes are split as it says (the
    chunks of K dealt out evenly), others by the rule of sizes; a product of such a shape is right and its partial sums
    add up to it."""
    api = K()
    assert api.KNOWN_SPLITS[(5120, 13824)] == 6 and api.gemm_skinny_splits(5120, 13824) == 6     # 54 chunks: 6 x 9
    assert api.gemm_skinny_splits(10240, 8192) == 3 and api.gemm_skinny_splits(2048, 8192) == 8
    assert api.gemm_skinny_splits(4096, 14336) == 8 and api.gemm_skinny_splits(4096, 4096) == 8  # the rule: 512 workgroups
    for (N, Kd), parts in api.KNOWN_SPLITS.items():
        assert 1 <= api.gemm_skinny_splits(N, Kd) <= parts
    N, Kd, M = 5120, 5120, 5
    a, w = _rand(M, Kd, dtype=torch.bfloat16, seed=1), _rand(N, Kd, dtype=torch.bfloat16, seed=2)
    out = api.gemm_skinny(a, w, out_dtype=torch.float32)
    want = a.double() @ w.double().t()
    assert ((out.double() - want).abs().max() / want.abs().max()).item() < 1e-5
    kept = api.gemm_skinny(a, w, keep_split=True)
    assert kept.parts.shape[0] == 5 and torch.allclose(kept.parts.sum(0), out, rtol=1e-5, atol=1e-3)


def test_gemm_skinny_refuses_what_it_cannot_do():
    api = K()
    a, w = _rand(129, 64, dtype=torch.bfloat16), _rand(32, 64, dtype=torch.bfloat16)
    with pytest.raises(api.KernelError):
        api.gemm_skinny(a, w)
    with pytest.raises(api.KernelError):
        api.gemm_skinny(_rand(4, 60, dtype=torch.bfloat16), _rand(32, 60, dtype=torch.bfloat16))
    with pytest.raises(api.KernelError):
        api.gemm_skinny(_rand(4, 64, dtype=torch.bfloat16), _rand(33, 64, dtype=torch.bfloat16), epilogue="swiglu")


@pytest.mark.parametrize("tile", ["auto", "256x256", "128x256", "128x128"])
@pytest.mark.parametrize("M,N,K_", [(65, 250, 64), (300, 1003, 192), (257, 516, 1024), (1, 7, 128), (640, 384, 320)])
def test_gemm_mfma(tile, M, N, K_):
    """The LDS-tiled product at sizes that fill no tile: edges in M and N, N that is no multiple of 4 (scalar
    stores), one step of K and many, every tile shape."""
    api = K()
    a, w = _rand(M, K_, dtype=torch.bfloat16, seed=8), _rand(N, K_, dtype=torch.bfloat16, scale=0.1, seed=9)
    want = a.double() @ w.double().t()
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    api.gemm_mfma(a, w, out, tile=tile)
    # fp32 accumulation, one rounding to bf16
    bound = 2e-5 * math.sqrt(K_) * 0.1 + 2.0 ** -8 * want.abs()
    assert bool(((out.double() - want).abs() <= bound).all())
    # a row's result does not depend on the rows beside it, nor on the tile shape
    last = api.gemm_mfma(a[M - 1:M].contiguous(), w, tile=tile)
    assert torch.equal(last[0], out[M - 1])
    assert torch.equal(api.gemm_mfma(a, w, tile="128x128"), out)


def test_gemm_mfma_picks_out_one_product():
    """One large entry in a and one in w, at the last row, column and k: a wrong swizzle, stage or edge row
    would move or lose it."""
    api = K()
    M, N, K_ = 515, 771, 448
    a = torch.zeros(M, K_, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(N, K_, dtype=torch.bfloat16, device=DEV)
    spots = [(0, 0, 0), (M - 1, N - 1, K_ - 1), (256, 255, 64), (129, 513, 71), (300, 2, 447)]
    for i, (m, n, k) in enumerate(spots):
        a[m, k] = 1 + i
        w[n, k] = 2
    want = a.float() @ w.float().t()
    assert torch.equal(api.gemm_mfma(a, w).float(), want)


@pytest.mark.parametrize("M,N,K_,S", [(129, 250, 64, 1), (256, 516, 1024, 4), (200, 1003, 448, 3), (300, 328, 448, 7),
                                      (130, 7, 128, 2), (512, 384, 320, 5)])
def test_gemm_mfma_split(M, N, K_, S):
    """The LDS-tiled product with K split over workgroups: part p of the result holds the fp32 sums over its run of
    the steps of 64 (dealt out evenly, the first parts one more), at sizes that fill no tile, with rows of N that
    are no multiple of 4 (scalar stores), one step a part and many."""
    api = K()
    a, w = _rand(M, K_, dtype=torch.bfloat16, seed=8), _rand(N, K_, dtype=torch.bfloat16, scale=0.1, seed=9)
    parts = torch.full((S, M, N), float("nan"), dtype=torch.float32, device=DEV)
    got = api.gemm_mfma_split(a, w, S, parts)
    assert got.parts.data_ptr() == parts.data_ptr() and tuple(got.shape) == (M, N)
    steps, first = K_ // 64, 0
    for p in range(S):
        n = steps // S + (1 if p < steps % S else 0)
        ka, kb = 64 * first, 64 * (first + n)
        want = a[:, ka:kb].double() @ w[:, ka:kb].double().t()
        assert bool(((parts[p].double() - want).abs() <= 2e-6 * math.sqrt(kb - ka) * 0.1 + 2e-6 * want.abs()).all()), p
        first += n
    # the parts added in the order of their index and rounded once are what the whole product gives (the same
    # sums in the same order within a part; across parts fp32 additions): within one rounding to bf16
    whole = api.gemm_mfma(a, w, tile="128x128")
    joined = got.joined(torch.bfloat16)
    want = a.double() @ w.double().t()
    assert bool(((joined.double() - want).abs() <= 2e-5 * math.sqrt(K_) * 0.1 + 2.0 ** -8 * want.abs()).all())
    assert bool(((joined.double() - whole.double()).abs() <= 2.0 ** -7 * want.abs() + 1e-6).all())
    # a row's sums do not depend on the rows beside it
    last = api.gemm_mfma_split(a[M - 1:M].contiguous(), w, S)
    assert torch.equal(last.parts[:, 0], parts[:, M - 1])


def test_gemm_mfma_split_picks_out_one_product_and_refuses_what_it_cannot_do():
    api = K()
    M, N, K_, S = 200, 771, 448, 3                      # 7 steps of K: parts of 3, 2 and 2
    a = torch.zeros(M, K_, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(N, K_, dtype=torch.bfloat16, device=DEV)
    spots = [(0, 0, 0, 0), (M - 1, N - 1, K_ - 1, 2), (128, 255, 192, 1), (129, 513, 191, 0), (77, 2, 320, 2)]
    for i, (m, n, k, p) in enumerate(spots):
        a[m, k] = 1 + i
        w[n, k] = 2
    got = api.gemm_mfma_split(a, w, S).parts
    want = torch.zeros(S, M, N, device=DEV)
    for i, (m, n, k, p) in enumerate(spots):
        want[p, m, n] = 2 * (1 + i)
    assert torch.equal(got, want)
    with pytest.raises(api.KernelError):
        api.gemm_mfma_split(a, w, 8)                                                                # more parts than steps
    with pytest.raises(api.KernelError):
        api.gemm_mfma_split(a, w, 0)
    with pytest.raises(api.KernelError):
        api.gemm_mfma_split(_rand(80, 96, dtype=torch.bfloat16), _rand(32, 96, dtype=torch.bfloat16), 1)   # K % 64
    with pytest.raises(api.KernelError):
        api.gemm_mfma_split(a, w, S, torch.empty(S, M, N + 1, device=DEV))                           # parts' shape


@pytest.mark.parametrize("M,N,K_", [(64, 1000, 192), (1, 66, 64), (128, 330, 256), (200, 2048, 448), (37, 254, 448),
                                    (130, 260, 1024), (70, 16446, 448), (9, 28672, 512)])
def test_gemm_mfma_swiglu(M, N, K_):
    """The LDS-tiled product with the activation in its epilogue: silu(first half) * second half from the fp32 sums,
    rounded once; tiles of 64 columns of the result at sizes that fill none, half widths that are no multiple of 4
    (scalar stores), more rows than a tile.  Up to 128 rows the weight-streaming kernel's epilogue gives the same
    values but for the order of the fp32 additions (a tile of columns starts its walk over K at a step of its own)."""
    api = K()
    a, w = _rand(M, K_, dtype=torch.bfloat16, seed=8), _rand(N, K_, dtype=torch.bfloat16, scale=0.1, seed=9)
    out = torch.full((M, N // 2), float("nan"), dtype=torch.bfloat16, device=DEV)
    assert api.gemm_mfma_swiglu(a, w, out).data_ptr() == out.data_ptr()
    y = a.double() @ w.double().t()
    gate, up = y[:, :N // 2], y[:, N // 2:]
    want = torch.nn.functional.silu(gate) * up
    # the sums carry fp32 rounding (2e-5 sqrt(K) 0.1 each); silu has slope at most 1.1
    e = 2e-5 * math.sqrt(K_) * 0.1
    bound = 2.0 ** -8 * want.abs() + e * (1.1 * up.abs() + gate.abs() + e)
    assert bool(((out.double() - want).abs() <= bound).all())
    if M <= 128:
        other = api.gemm_skinny(a, w, epilogue="swiglu").double()
        assert bool(((out.double() - other).abs() <= 2.0 ** -7 * want.abs() + 2 * e * (1.1 * up.abs() + gate.abs() + e)).all())
    # a row's result does not depend on the rows beside it
    assert torch.equal(api.gemm_mfma_swiglu(a[M - 1:M].contiguous(), w)[0], out[M - 1])
    # from the copy laid out for the weight-streaming kernel (where that kernel does not split K): the same bits
    if api.gemm_skinny_splits(N, K_) == 1:
        assert torch.equal(api.gemm_mfma_swiglu(a, w, tiled=api.tile_weight(w, "swiglu")), out)
    else:
        with pytest.raises(api.KernelError):
            api.gemm_mfma_swiglu(a, w, tiled=api.tile_weight(w, "swiglu"))
    with pytest.raises(api.KernelError):
        api.gemm_mfma_swiglu(a, w[:N - 1].contiguous())                                             # an odd number of rows
    with pytest.raises(api.KernelError):
        api.gemm_mfma_swiglu(a, w, torch.empty(M, N, dtype=torch.bfloat16, device=DEV))             # out's shape
    with pytest.raises(api.KernelError):
        api.gemm_mfma_swiglu(_rand(8, 96, dtype=torch.bfloat16), _rand(32, 96, dtype=torch.bfloat16))   # K % 64


def test_gemm_mfma_refuses_what_it_cannot_do():
    api = K()
    with pytest.raises(api.KernelError):
        api.gemm_mfma(_rand(80, 96, dtype=torch.bfloat16), _rand(32, 96, dtype=torch.bfloat16))      # K % 64
    with pytest.raises(api.KernelError):
        api.gemm_mfma(_rand(80, 64), _rand(32, 64))                                                  # fp32
    with pytest.raises(api.KernelError):
        api.gemm_mfma(_rand(80, 128, dtype=torch.bfloat16)[:, :64], _rand(32, 64, dtype=torch.bfloat16))


def test_linear_with_the_hand_written_prefill_gemm():
    import importlib
    L = importlib.import_module("infernum_amd.parts.linear")   # the package exports the function under this name
    x, w = _rand(200, 256, dtype=torch.bfloat16, seed=3), _rand(330, 256, dtype=torch.bfloat16, scale=0.1, seed=4)
    lib = L.linear(x, w)
    previous = L.set_prefill_gemm("mfma")
    try:
        own = L.linear(x, w)
        act = L.linear(x, w, epilogue="swiglu")
        odd = L.linear(x[:, :200].contiguous(), w[:, :200].contiguous())   # K = 200: the library takes it
    finally:
        L.set_prefill_gemm(previous)
    want = x.double() @ w.double().t()
    bound = 2e-5 * 16 * 0.1 + 2.0 ** -8 * want.abs()
    assert bool(((own.double() - want).abs() <= bound).all()) and bool(((lib.double() - want).abs() <= bound).all())
    assert torch.equal(act, K().swiglu(own, torch.empty(200, 165, dtype=torch.bfloat16, device=DEV)))
    assert tuple(odd.shape) == (200, 330)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,N,K_", [(65, 100, 72), (67, 31, 9), (300, 1003, 192), (1, 7, 128), (640, 384, 320)])
def test_gemm_library(dtype, M, N, K_):
    """The vendor library's product, called directly: sizes that fill no tile and that are no multiple of
    anything; the second call of a shape takes the kept plan and gives the same bits."""
    api = K()
    a, w = _rand(M, K_, dtype=dtype, seed=8), _rand(N, K_, dtype=dtype, scale=0.1, seed=9)
    want = a.double() @ w.double().t()
    out = torch.full((M, N), float("nan"), dtype=dtype, device=DEV)
    api.gemm_library(a, w, out)
    if dtype == torch.bfloat16:
        bound = 2e-5 * math.sqrt(K_) * 0.1 + 2.0 ** -8 * want.abs()
    else:
        # fp32 throughout: the worst case of K roundings of 2^-24 each on the sum of the products' magnitudes,
        # far below what a reduced-precision matrix mode (2^-11 per product) would leave
        bound = K_ * 2.0 ** -24 * (a.abs().double() @ w.abs().double().t())
    assert bool(((out.double() - want).abs() <= bound).all())
    plans = api.load_library("blaslt").ia_gemm_lt_plans()
    assert torch.equal(api.gemm_library(a, w), out)
    assert api.load_library("blaslt").ia_gemm_lt_plans() == plans


def test_gemm_library_refuses_what_it_cannot_do():
    api = K()
    with pytest.raises(api.KernelError):
        api.gemm_library(_rand(80, 96, dtype=torch.bfloat16), _rand(32, 96))                       # two dtypes
    with pytest.raises(api.KernelError):
        api.gemm_library(_rand(80, 96), _rand(32, 64))                                             # inner sizes
    with pytest.raises(api.KernelError):
        api.gemm_library(_rand(80, 128)[:, :64], _rand(32, 64))                                    # not contiguous


def test_linear_by_the_library_and_by_the_tiled_kernel():
    import importlib
    L = importlib.import_module("infernum_amd.parts.linear")
    x, w = _rand(200, 256, dtype=torch.bfloat16, seed=3), _rand(330, 256, dtype=torch.bfloat16, scale=0.1, seed=4)
    assert L.prefill_gemm() == "library"
    assert [r.kind for r in L.plan(330, 256, torch.bfloat16, torch.bfloat16, None, False)] == ["skinny", "library"]
    direct = L.linear(x, w)
    previous = L.set_prefill_gemm("mfma")
    try:
        assert [r.kind for r in L.plan(330, 256, torch.bfloat16, torch.bfloat16, None, False)] == ["skinny", "mfma"]
        tiled = L.linear(x, w)
    finally:
        L.set_prefill_gemm(previous)
    want = x.double() @ w.double().t()
    bound = 2e-5 * 16 * 0.1 + 2.0 ** -8 * want.abs()
    assert bool(((direct.double() - want).abs() <= bound).all()) and bool(((tiled.double() - want).abs() <= bound).all())
    with pytest.raises(ValueError):
        L.set_prefill_gemm("torch")


def test_linear_fp32_result_of_many_rows_from_bf16_operands():
    """The head of a step that wants many rows: 128 rows at a time through the weight-streaming kernel."""
    import importlib
    L = importlib.import_module("infernum_amd.parts.linear")
    x, w = _rand(300, 96, dtype=torch.bfloat16, seed=5), _rand(1000, 96, dtype=torch.bfloat16, scale=0.1, seed=6)
    assert [r.kind for r in L.plan(1000, 96, torch.bfloat16, torch.float32, None, False)] == ["skinny", "skinny_rows"]
    y = L.linear(x, w, out_dtype=torch.float32)
    want = x.double() @ w.double().t()
    assert y.dtype == torch.float32 and (y.double() - want).abs().max().item() <= 2e-5 * 10 * 0.1
    for m in (1, 128, 129, 256, 257):
        assert torch.equal(L.linear(x[:m].contiguous(), w, out_dtype=torch.float32), y[:m])


def test_known_mid_rows_send_a_few_hundred_rows_to_the_tiled_kernel_with_k_split():
    """Every band of the table is a route of its weight's plan, ahead of the library's, for products that leave
    partial sums; a product that wants a tensor stays with the library; shapes outside the table follow a rule."""
    import importlib
    L = importlib.import_module("infernum_amd.parts.linear")
    assert (129, 256, 4) in L.KNOWN_MID_ROWS[(4096, 14336)]
    for (N, Kd), bands in L.KNOWN_MID_ROWS.items():
        routes = L.plan(N, Kd, torch.bfloat16, torch.bfloat16, None, True)
        last = 0
        for lo, hi, parts in bands:
            assert lo > last and hi >= lo and 1 <= parts <= Kd // 64           # bands follow each other
            for M in (lo, hi):
                r = L.route_of(routes, M)
                assert (r.kind, r.parts) == ("mfma_split", parts), (N, Kd, M)
            if lo > 1:
                assert L.route_of(routes, lo - 1).kind != "mfma_split" or lo - 1 == last
            last = hi
        assert L.route_of(routes, max(last, 128) + 1).kind == "library"
        if not any(lo <= 8 <= hi for lo, hi, _ in bands):                       # few rows: the weight-streaming kernel
            assert L.route_of(routes, 8).kind in ("skinny", "skinny_split")
        assert L.route_of(L.plan(N, Kd, torch.bfloat16, torch.bfloat16, None, False), 200).kind == "library"
        previous = L.set_gemm_route("static")            # the rule of sizes alone
        try:
            at_200 = [parts for lo, hi, parts in L._mid_rows_by_size(N, Kd) if lo <= 200 <= hi]
            r = L.route_of(L.plan(N, Kd, torch.bfloat16, torch.bfloat16, None, True), 200)
            assert (r.kind, r.parts) == (("mfma_split", at_200[0]) if at_200 else ("library", 0))
        finally:
            L.set_gemm_route(previous)
    # gate+up products: the tiled kernel with the activation in its epilogue for the bands of its table
    for (N, Kd), bands in L.KNOWN_GLU_ROWS.items():
        routes = L.plan(N, Kd, torch.bfloat16, torch.bfloat16, "swiglu", False)
        for lo, hi in bands:
            assert L.route_of(routes, lo).kind == L.route_of(routes, hi).kind == "mfma_swiglu"
            assert L.route_of(routes, lo - 1).kind != "mfma_swiglu" and L.route_of(routes, hi + 1).kind != "mfma_swiglu"
        assert all(r.kind != "mfma_swiglu" for r in L.plan(N, Kd, torch.bfloat16, torch.bfloat16, None, False))
    # a shape the table does not hold: as many parts as bring the tiles to a workgroup a compute unit, at least two
    assert L.mid_rows(4096, 11008, True) == ((33, 128, 8), (129, 256, 4), (257, 384, 2)) and L.mid_rows(4096, 11008, False) == ()
    assert L.mid_rows(22016, 4096, True) == () and L.mid_rows(4096, 1000, True) == () and L.mid_rows(64, 448, True) == ()
    # the product through the route is the product: 8B shape's output projection at 200 rows
    x, w = _rand(200, 4096, dtype=torch.bfloat16, seed=5), _rand(4096, 4096, dtype=torch.bfloat16, scale=0.02, seed=6)
    y = L.linear(x, w, keep_split=True)
    assert isinstance(y, K().SplitSum) and tuple(y.parts.shape) == (4, 200, 4096)
    want = x.double() @ w.double().t()
    assert (y.parts.double().sum(0) - want).abs().max().item() <= 2e-5 * 64 * 0.02


def test_linear_fp32_result_of_many_rows_by_the_tiled_kernel():
    """Where the LDS-tiled kernel takes the size (K in steps of 64), the fp32 result of more than 128 rows is its
    one part of fp32 sums: every row as exact as the weight-streaming kernel's, whatever rows stand beside it."""
    import importlib
    L = importlib.import_module("infernum_amd.parts.linear")
    x, w = _rand(300, 192, dtype=torch.bfloat16, seed=5), _rand(1003, 192, dtype=torch.bfloat16, scale=0.1, seed=6)
    assert [r.kind for r in L.plan(1003, 192, torch.bfloat16, torch.float32, None, False)] == ["mfma_f32", "skinny", "skinny_rows"]
    first = L.FP32_TILED_FROM_ROWS[1]
    assert L.route_of(L.plan(1003, 192, torch.bfloat16, torch.float32, None, False), first).kind == "mfma_f32"
    assert L.route_of(L.plan(1003, 192, torch.bfloat16, torch.float32, None, False), first - 1).kind == "skinny"
    assert L.route_of(L.plan(1003, 4096, torch.bfloat16, torch.float32, None, False), L.FP32_TILED_FROM_ROWS[0]).kind == "mfma_f32"
    y = L.linear(x, w, out_dtype=torch.float32)
    want = x.double() @ w.double().t()
    assert y.dtype == torch.float32 and tuple(y.shape) == (300, 1003)
    assert (y.double() - want).abs().max().item() <= 2e-5 * 14 * 0.1
    for m in (129, 256, 257):
        assert torch.equal(L.linear(x[:m].contiguous(), w, out_dtype=torch.float32), y[:m])
    few = L.linear(x[:first - 1].contiguous(), w, out_dtype=torch.float32)     # the weight-streaming kernel
    assert (few.double() - want[:first - 1]).abs().max().item() <= 2e-5 * 14 * 0.1
    assert (few - y[:first - 1]).abs().max().item() <= 4e-6 * 14 * 0.1
    assert torch.equal(L.linear(x[:first].contiguous(), w, out_dtype=torch.float32), y[:first])


@pytest.mark.parametrize("N,Kd,epilogue", [(28672, 4096, "swiglu"), (330, 264, "swiglu"), (1000, 96, None), (6144, 512, None),
                                          (4096, 4096, None), (77, 1032, None), (16640, 264, "swiglu")])
def test_gemm_skinny_with_the_weight_laid_out_for_it(N, Kd, epilogue):
    """A copy of the weight in which a workgroup's rows of a chunk are consecutive memory (rows padded to whole
    workgroups, K to whole chunks): the same sums in the same order, so the same bits, for every number of rows,
    with the activation, with the partial sums kept, and 128 rows at a time."""
    api = K()
    w = _rand(N, Kd, dtype=torch.bfloat16, scale=0.1, seed=N % 97)
    t = api.tile_weight(w, epilogue)
    assert t.dtype == torch.bfloat16 and t.numel() % (64 * 256) == 0 and t.numel() >= N * Kd
    for M in (1, 8, 17, 64, 65, 128):
        x = _rand(M, Kd, dtype=torch.bfloat16, seed=M)
        a, b = api.gemm_skinny(x, w, epilogue=epilogue), api.gemm_skinny(x, w, epilogue=epilogue, tiled=t)
        assert torch.equal(a, b), M
        if epilogue is None:
            a, b = api.gemm_skinny(x, w, keep_split=True), api.gemm_skinny(x, w, keep_split=True, tiled=t)
            parts = lambda y: y.parts if isinstance(y, api.SplitSum) else y
            assert torch.equal(parts(a), parts(b)), M
            a = api.gemm_skinny(x, w, out_dtype=torch.float32)
            assert torch.equal(a, api.gemm_skinny(x, w, out_dtype=torch.float32, tiled=t)), M
    if epilogue is None:
        x = _rand(300, Kd, dtype=torch.bfloat16, seed=5)
        a = api.gemm_skinny_rows(x, w, torch.empty(300, N, device=DEV))
        assert torch.equal(a, api.gemm_skinny_rows(x, w, torch.empty(300, N, device=DEV), tiled=t))


def test_wide_weights_get_a_copy_laid_out_for_the_kernel_and_narrow_ones_do_not():
    import importlib
    L = importlib.import_module("infernum_amd.parts.linear")
    from part_harness import runtime
    rt = runtime("bfloat16")
    wide, narrow = _rand(16640, 264, dtype=torch.bfloat16), _rand(512, 2048, dtype=torch.bfloat16)
    L.prepare_weights(rt, [(wide, "swiglu", False), (wide, None, False), (narrow, None, True)])
    assert L.tiled_copy(wide, "swiglu") is not None and L.tiled_copy(wide, None) is not None
    assert L.tiled_copy(wide, "swiglu") is not L.tiled_copy(wide, None)          # two layouts: with both halves, without
    assert L.tiled_copy(narrow, None) is None and K().gemm_skinny_splits(512, 2048) > 1
    x = _rand(8, 264, dtype=torch.bfloat16, seed=1)
    assert torch.equal(L.linear(x, wide, epilogue="swiglu"), K().gemm_skinny(x, wide, epilogue="swiglu"))
    fp = runtime("float32")
    w32 = _rand(16640, 264)
    L.prepare_weights(fp, [(w32, None, False)])
    assert L.tiled_copy(w32, None) is None
    # no copy where it would take memory that has to stay free: the weight then runs from the file's layout
    other = wide.clone()
    keep, L.COPIES_LEAVE_FREE = L.COPIES_LEAVE_FREE, 1.0
    try:
        L.prepare_weights(rt, [(other, None, False)])
    finally:
        L.COPIES_LEAVE_FREE = keep
    assert L.tiled_copy(other, None) is None
    assert torch.equal(L.linear(x, other), L.linear(x, wide))


def test_known_routes_send_rows_to_the_library_where_the_table_says():
    import importlib
    L = importlib.import_module("infernum_amd.parts.linear")
    key = (15360, 5120, None, True)
    assert L.KNOWN_ROUTES[key] == 0b11111110
    kinds = lambda: {m: L.route_of(L.plan(15360, 5120, torch.bfloat16, torch.bfloat16, None, True), m).kind
                     for m in (1, 16, 17, 64, 128, 129)}
    # (the bands of KNOWN_MID_ROWS stand in front: up to 16 rows and from 97 to 128 the split tiled kernel for this shape)
    assert L.KNOWN_MID_ROWS[(15360, 5120)] == ((1, 16, 2), (97, 128, 2))
    assert kinds() == {1: "mfma_split", 16: "mfma_split", 17: "library", 64: "library", 128: "mfma_split", 129: "library"}
    saved = L.KNOWN_MID_ROWS.pop((15360, 5120))
    try:
        assert L.mid_rows(15360, 5120, True) == ((33, 128, 2),)      # the rule of sizes: 120 tiles of columns, two parts
        assert kinds() == {1: "skinny_split", 16: "skinny_split", 17: "library", 64: "mfma_split", 128: "mfma_split", 129: "library"}
    finally:
        L.KNOWN_MID_ROWS[(15360, 5120)] = saved
    previous = L.set_gemm_route("static")
    try:
        assert kinds() == {1: "skinny_split", 16: "skinny_split", 17: "skinny_split", 64: "mfma_split",
                           128: "mfma_split", 129: "library"}
    finally:
        L.set_gemm_route(previous)


def test_rope_from_partial_sums():
    """The rotary kernel joins a split product itself: same pages and queries as from the joined tensor."""
    api = K()
    nh, nkv, d, ps, N, S = 6, 2, 48, 4, 9, 3
    row = (nh + 2 * nkv) * d
    parts = _rand(S, N, row, seed=4)
    joined = parts.sum(0).bfloat16()
    pos = torch.arange(3, 3 + N, dtype=torch.int32, device=DEV)
    slots = torch.randperm(40)[:N].to(torch.int32).to(DEV)
    inv = (1.0 / (10000.0 ** (torch.arange(0, d, 2).float() / d))).to(DEV)
    kp1, vp1 = torch.zeros(10, nkv, ps, d, dtype=torch.bfloat16, device=DEV), torch.zeros(10, nkv, d, ps, dtype=torch.bfloat16, device=DEV)
    kp2, vp2 = torch.zeros_like(kp1), torch.zeros_like(vp1)
    q1 = api.rope_kv_append(api.SplitSum(parts), pos, inv, nh, nkv, d, d, slots, kp1, vp1)
    # reference: the fp32 sum through the same kernel as one fp32 "part"
    q2 = api.rope_kv_append(api.SplitSum(parts.sum(0, keepdim=True).contiguous()), pos, inv, nh, nkv, d, d, slots, kp2, vp2)
    assert tuple(q1.shape) == (N, nh * d) and q1.dtype == torch.bfloat16
    assert torch.allclose(q1.float(), q2.float(), atol=2e-2) and torch.allclose(kp1.float(), kp2.float(), atol=2e-2)
    assert torch.allclose(vp1.float(), vp2.float(), atol=2e-2)
    # and against the bf16 tensor rotated in place (rounded once more before the rotation)
    q3 = joined.clone()
    kp3, vp3 = torch.zeros_like(kp1), torch.zeros_like(vp1)
    api.rope_kv_append(q3, pos, inv, nh, nkv, d, d, slots, kp3, vp3)
    assert torch.allclose(q1.float(), q3[:, :nh * d].float(), atol=6e-2)
    assert torch.allclose(kp1.float(), kp3.float(), atol=6e-2)


@pytest.mark.parametrize("nh,nkv,d,ps,rot", [(6, 2, 48, 8, 48), (32, 8, 128, 16, 128), (5, 5, 16, 16, 8), (4, 1, 96, 4, 64), (3, 1, 80, 12, 80)])
@pytest.mark.parametrize("S", [1, 2, 5])
def test_rope_of_many_tokens_from_partial_sums(nh, nkv, d, ps, rot, S):
    """From 32 tokens on, a product that comes as one part is rotated by another kernel (a workgroup a token, all
    heads, 16-byte loads; the values to their transposed pages by a launch of their own where pages take eight tokens
    at a time); a stack of partial sums stays with the kernel for few tokens, which adds the parts in the order of
    their index.  Either way the first 9 of 40 tokens alone (the kernel for few tokens) give the same queries and
    the same slots of the pages, bit for bit, and all 40 agree with plain arithmetic on the joined sums."""
    api = K()
    N = 40
    row = (nh + 2 * nkv) * d
    parts = _rand(S, N, row, seed=4 + S)
    pos = torch.arange(3, 3 + N, dtype=torch.int32, device=DEV)
    slots = torch.cat([torch.arange(16, 16 + 24), torch.randperm(16)[:16]]).to(torch.int32).to(DEV)   # a run, then scattered
    num_pages = -(-56 // ps) + 1
    inv = (1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot))).to(DEV)
    kp1 = torch.zeros(num_pages, nkv, ps, d, dtype=torch.bfloat16, device=DEV)
    vp1 = torch.zeros(num_pages, nkv, d, ps, dtype=torch.bfloat16, device=DEV)
    q1 = api.rope_kv_append(api.SplitSum(parts), pos, inv, nh, nkv, d, rot, slots, kp1, vp1)
    kp2, vp2 = torch.zeros_like(kp1), torch.zeros_like(vp1)
    few = api.SplitSum(parts[:, :9].contiguous())
    q2 = api.rope_kv_append(few, pos[:9].contiguous(), inv, nh, nkv, d, rot, slots[:9].contiguous(), kp2, vp2)
    assert torch.equal(q1[:9], q2)
    for n in range(9):
        pg, off = int(slots[n]) // ps, int(slots[n]) % ps
        assert torch.equal(kp1[pg, :, off], kp2[pg, :, off]) and torch.equal(vp1[pg, :, :, off], vp2[pg, :, :, off])
    # and against plain arithmetic on the joined sums
    x = parts.double().sum(0).cpu()
    ang = pos.cpu().double()[:, None] * inv.cpu().double()[None, :]
    cs, sn = torch.cos(ang), torch.sin(ang)
    half = rot // 2
    for h in range(nh + nkv):
        v = x[:, h * d:(h + 1) * d].clone()
        a, b = v[:, :half].clone(), v[:, half:rot].clone()
        v[:, :half], v[:, half:rot] = a * cs - b * sn, b * cs + a * sn
        if h < nh:
            got = q1[:, h * d:(h + 1) * d].double().cpu()
        else:
            got = torch.stack([kp1[int(slots[n]) // ps, h - nh, int(slots[n]) % ps] for n in range(N)]).double().cpu()
        assert (got - v).abs().max().item() <= 2.0 ** -7 * v.abs().max().item() + 1e-3
    for g in range(nkv):
        v = x[:, (nh + nkv + g) * d:(nh + nkv + g + 1) * d]
        got = torch.stack([vp1[int(slots[n]) // ps, g, :, int(slots[n]) % ps] for n in range(N)]).double().cpu()
        assert (got - v).abs().max().item() <= 2.0 ** -7 * v.abs().max().item() + 1e-3


# ------------------------------------------------------------------- attention
def _paged_case(nh, nkv, d, ps, lens, q_lens, dtype, seed=0, scale_one=None, loud=(), q_lift=0.0):
    """Random queries/keys/values of several requests laid out into shuffled pages.
    Returns everything the kernels need plus the dense tensors for the reference.
    ``loud``: (request, key, value) sets the first component of that key (every head) to the value, and
    ``q_lift`` is added to the first component of every query head: the key's score is about
    q_lift * value * scale above the others for every query that sees it."""
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    pages_per = [-(-L // ps) for L in lens]
    num_pages = sum(pages_per) + 3
    perm = torch.randperm(num_pages, generator=g).tolist()
    MB = max(pages_per) + 1
    bt = torch.full((B, MB), -1, dtype=torch.int32)
    kd = [torch.randn(L, nkv, d, generator=g) for L in lens]
    vd = [torch.randn(L, nkv, d, generator=g) for L in lens]
    if scale_one is not None:                      # make one far key stand out
        b, j, factor = scale_one
        kd[b][j] *= factor
    for b, j, value in loud:
        kd[b][j][:, 0] = value
    kp = torch.zeros(num_pages, nkv, ps, d)
    vp = torch.zeros(num_pages, nkv, d, ps)
    it = iter(perm)
    for b in range(B):
        for i in range(pages_per[b]):
            p = next(it)
            bt[b, i] = p
            n = min(ps, lens[b] - i * ps)
            kp[p, :, :n] = kd[b][i * ps:i * ps + n].transpose(0, 1)
            vp[p, :, :, :n] = vd[b][i * ps:i * ps + n].permute(1, 2, 0)
    N = sum(q_lens)
    q = torch.randn(N, nh * d, generator=g)
    if q_lift:
        q[:, ::d] += q_lift
    token_seq = torch.cat([torch.full((ql,), b, dtype=torch.int32) for b, ql in enumerate(q_lens)])
    positions = torch.cat([torch.arange(L - ql, L, dtype=torch.int32) for L, ql in zip(lens, q_lens)])
    to = lambda t: t.to(dtype).to(DEV)
    return dict(q=to(q), kp=to(kp), vp=to(vp), bt=bt.to(DEV), token_seq=token_seq.to(DEV),
                positions=positions.to(DEV), kd=[to(x) for x in kd], vd=[to(x) for x in vd], N=N)


def _ref_attention(case, nh, nkv, d, scale, window):
    out = torch.zeros(case["N"], nh * d, dtype=torch.float64)
    q = case["q"].double().cpu()
    for n in range(case["N"]):
        b, p = int(case["token_seq"][n]), int(case["positions"][n])
        lo = max(0, p - window + 1) if window else 0
        k, v = case["kd"][b].double().cpu()[lo:p + 1], case["vd"][b].double().cpu()[lo:p + 1]
        for h in range(nh):
            gk = h // (nh // nkv)
            w = torch.softmax((k[:, gk] @ q[n, h * d:(h + 1) * d]) * scale, 0)
            out[n, h * d:(h + 1) * d] = w @ v[:, gk]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,nkv,d,ps,window", [(6, 2, 48, 5, 0), (4, 4, 16, 16, 0), (8, 1, 128, 7, 0),
                                                (3, 3, 80, 4, 9), (2, 1, 256, 16, 70)])
def test_attention_generic(dtype, nh, nkv, d, ps, window):
    lens, q_lens = [70, 3, 131, 64], [1, 3, 40, 64]
    case = _paged_case(nh, nkv, d, ps, lens, q_lens, dtype)
    out = torch.full((case["N"], nh * d), float("nan"), dtype=dtype, device=DEV)
    scale = 1.0 / math.sqrt(d)
    K().attention_generic(case["q"], case["kp"], case["vp"], out, case["token_seq"], case["positions"], case["bt"],
                          nh, nkv, d, scale, window)
    want = _ref_attention(case, nh, nkv, d, scale, window)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    assert (out.double().cpu() - want).abs().max().item() <= tol


def test_attention_generic_far_key_and_first_row():
    """One key far back among hundreds carries the softmax; a missed page or a wrong
    block-table entry shows at once.  The first token of a request returns v_0."""
    nh, nkv, d, ps = 2, 1, 32, 8
    case = _paged_case(nh, nkv, d, ps, [500, 1], [1, 1], torch.float32, scale_one=(0, 17, 30.0))
    out = torch.empty(2, nh * d, device=DEV)
    K().attention_generic(case["q"], case["kp"], case["vp"], out, case["token_seq"], case["positions"], case["bt"],
                          nh, nkv, d, 1.0, 0)
    want = _ref_attention(case, nh, nkv, d, 1.0, 0)
    assert (out.double().cpu() - want).abs().max().item() <= 2e-5
    assert torch.allclose(out[1].reshape(nh, d), case["vd"][1][0, 0].expand(nh, d), atol=1e-6)


def test_attention_generic_missing_page_poisons():
    nh, nkv, d, ps = 1, 1, 16, 4
    case = _paged_case(nh, nkv, d, ps, [20], [1], torch.float32)
    case["bt"][0, 2] = -1
    out = torch.zeros(1, d, device=DEV)
    K().attention_generic(case["q"], case["kp"], case["vp"], out, case["token_seq"], case["positions"], case["bt"],
                          nh, nkv, d, 1.0, 0)
    assert out.isnan().all()
    # with a window that has passed the missing page the result is clean
    K().attention_generic(case["q"], case["kp"], case["vp"], out, case["token_seq"], case["positions"], case["bt"],
                          nh, nkv, d, 1.0, 8)
    assert not out.isnan().any()


def _prefill_tiles(q_lens, first_prefill=0):
    tiles = [(s, r) for s in range(first_prefill, len(q_lens)) for r in range(0, q_lens[s], 64)]
    return torch.tensor(tiles, dtype=torch.int32, device=DEV).reshape(-1, 2), len(tiles)


@pytest.mark.parametrize("nh,nkv,d,ps,window", [(8, 2, 128, 16, 0), (6, 3, 48, 4, 0), (4, 4, 16, 8, 0), (32, 8, 128, 16, 0),
                                                (20, 1, 64, 64, 0), (3, 1, 80, 12, 0), (2, 1, 256, 16, 0),
                                                (8, 2, 128, 16, 100), (6, 3, 48, 4, 9), (7, 7, 32, 8, 33)])
def test_attention_mfma_prefill(nh, nkv, d, ps, window):
    """Portions of prompts with earlier context, rows that do not fill a tile, several requests."""
    lens, q_lens = [70, 3, 331, 64, 150], [70, 3, 140, 17, 1]
    case = _paged_case(nh, nkv, d, ps, lens, q_lens, torch.bfloat16, seed=d + nh)
    N = case["N"]
    out = torch.full((N, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    scale = 1.0 / math.sqrt(d)
    starts = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=DEV)
    ctx = torch.tensor([L - q for L, q in zip(lens, q_lens)], dtype=torch.int32, device=DEV)
    tiles, nt = _prefill_tiles(q_lens)
    K().attention_prefill(case["q"], case["kp"], case["vp"], out, starts, ctx, case["bt"], tiles, nt, nh, nkv, d, scale,
                          window)
    want = _ref_attention(case, nh, nkv, d, scale, window)
    err = (out.double().cpu() - want).abs().max().item()
    assert err <= 2e-2, err
    gen = torch.empty_like(out)
    K().attention_generic(case["q"], case["kp"], case["vp"], gen, case["token_seq"], case["positions"], case["bt"], nh,
                          nkv, d, scale, window)
    assert (out.double() - gen.double()).abs().max().item() <= 2e-2
    # one, two or four query heads to a workgroup (four up to a head size of 160), rows of a workgroup from one
    # stretch or from both ends of the request: the same bits
    for hpw in (1, 2, 4):
        for paired in (False, True):
            other = torch.full_like(out, float("nan"))
            if hpw == 4 and d > 160:
                with pytest.raises(K().KernelError):
                    K().attention_prefill(case["q"], case["kp"], case["vp"], other, starts, ctx, case["bt"], tiles, nt,
                                          nh, nkv, d, scale, window, heads_per_workgroup=hpw, paired=paired)
                continue
            K().attention_prefill(case["q"], case["kp"], case["vp"], other, starts, ctx, case["bt"], tiles, nt, nh,
                                  nkv, d, scale, window, heads_per_workgroup=hpw, paired=paired)
            assert torch.equal(other, out), (hpw, paired)
    with pytest.raises(K().KernelError):
        K().attention_prefill(case["q"], case["kp"], case["vp"], other, starts, ctx, case["bt"], tiles, nt, nh, nkv, d,
                              scale, window, heads_per_workgroup=3)


@pytest.mark.parametrize("ctx0", [0, 200])
@pytest.mark.parametrize("nh,nkv,d,ps", [(8, 2, 128, 16), (4, 2, 64, 8), (6, 1, 48, 4)])
def test_attention_mfma_prefill_reference_point_moves_in_late_tiles(nh, nkv, d, ps, ctx0):
    """The prefill kernel takes its exponentials against a reference point that it moves only when a score
    comes out far above it.  Key 300 of 700 has some 2^29 times the weight of everything before it and key
    520 some 2^58 times that: every row that sees them moves its point in its fifth and in its ninth tile of
    keys, with sums of dozens of keys in its accumulators that have to be scaled down; rows of one tile see
    the loud keys, rows of others do not.  Once for a whole prompt, once for a portion after 200 cached tokens
    (whose first rows come before the first loud key); a second, short request rides along."""
    L = 700
    lens, q_lens = [L, 90], [L - ctx0, 90]
    scale = 1.0 / math.sqrt(d)
    lift = 6.0
    case = _paged_case(nh, nkv, d, ps, lens, q_lens, torch.bfloat16, seed=11 + d, q_lift=lift,
                       loud=[(0, 300, 20.0 / (lift * scale)), (0, 520, 60.0 / (lift * scale))])
    N = case["N"]
    starts = torch.tensor([0, q_lens[0], N], dtype=torch.int32, device=DEV)
    ctx = torch.tensor([ctx0, 0], dtype=torch.int32, device=DEV)
    tiles, nt = _prefill_tiles(q_lens)
    want = _ref_attention(case, nh, nkv, d, scale, 0)
    # the plain result itself says that the loud keys carry the rows behind them
    v = case["vd"][0].double().cpu()
    row = lambda p: want[p - ctx0].reshape(nh, d)[0]
    assert (row(400) - v[300, 0]).abs().max() < 1e-3 and (row(699) - v[520, 0]).abs().max() < 1e-3
    assert (row(299) - v[300, 0]).abs().max() > 0.1
    gen = torch.full((N, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    K().attention_generic(case["q"], case["kp"], case["vp"], gen, case["token_seq"], case["positions"], case["bt"], nh,
                          nkv, d, scale, 0)
    assert (gen.double().cpu() - want).abs().max().item() <= 2e-2
    first = None
    for hpw in (1, 2, 4):
        for paired in (False, True):
            out = torch.full((N, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
            K().attention_prefill(case["q"], case["kp"], case["vp"], out, starts, ctx, case["bt"], tiles, nt, nh, nkv,
                                  d, scale, 0, heads_per_workgroup=hpw, paired=paired)
            err = (out.double().cpu() - want).abs().max().item()
            assert err <= 2e-2, (hpw, paired, err)
            first = out if first is None else first
            assert torch.equal(out, first), (hpw, paired)


def test_prefill_launch_shape():
    """Heads per workgroup and pairing of rows for launches of different sizes."""
    api = K()
    dev = torch.device(DEV)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    P = api.PREFILL_PAIRED
    pick = lambda q, c, d=128, nh=32, nkv=8, w=0: api.prefill_launch_shape(nh, nkv, d, q, c, w, dev)
    per_tile = 8                                 # workgroups a block of 64 rows gives with four heads each
    few = [64 * max(1, cus // per_tile // 2)]    # half as many workgroups as compute units: two heads, and
    assert pick(few, [0]) == 2 | P               # still no more workgroups than compute units: paired
    exactly = [64 * (cus // per_tile)]           # one workgroup a compute unit with four heads
    assert pick(exactly, [0]) == 4 | P
    assert pick(exactly, [3 * exactly[0]]) == 4 | P
    assert pick([4 * exactly[0]], [0]) == 4      # many workgroups a compute unit: rows as they come
    assert pick(few, [0], d=64) == 2 | P and pick(few, [0], d=256) == 2 | P
    assert pick([64 * cus], [0], d=64) == 2
    assert pick(few, [0], nh=16) == 2 | P and pick(few, [0], nh=8) == 1 | P
    # under a window nothing is paired; two heads where four would leave one long workgroup a compute unit
    assert pick(few, [0], w=100) == 2 and pick(exactly, [0], w=10 ** 6) == 2 and pick(exactly, [3 * exactly[0]], w=10 ** 6) == 4
    assert pick([], []) == 0


@pytest.mark.parametrize("splits", [None, 1, 3, 7])
@pytest.mark.parametrize("nh,nkv,d,ps,window", [(8, 2, 128, 16, 0), (6, 3, 48, 4, 0), (32, 8, 128, 16, 0), (40, 2, 64, 8, 0),
                                                (5, 5, 16, 16, 0), (2, 1, 256, 64, 0), (8, 2, 128, 16, 100), (4, 1, 96, 4, 17),
                                                (3, 1, 80, 12, 0), (6, 2, 64, 20, 33)])      # pages of 12 and 20: no power of two
def test_attention_mfma_decode(nh, nkv, d, ps, window, splits):
    lens = [70, 1, 331, 64, 150, 16, 17]
    q_lens = [1] * len(lens)
    case = _paged_case(nh, nkv, d, ps, lens, q_lens, torch.bfloat16, seed=d + nh + 1)
    B = len(lens)
    out = torch.full((B, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    scale = 1.0 / math.sqrt(d)
    K().attention_decode(case["q"], case["kp"], case["vp"], out, case["positions"], case["bt"], nh, nkv, d, scale,
                         window, max(lens), num_splits=splits)
    want = _ref_attention(case, nh, nkv, d, scale, window)
    err = (out.double().cpu() - want).abs().max().item()
    assert err <= 2e-2, err


@pytest.mark.parametrize("gemm_splits", [0, 1, 3, 10])   # above eight parts the sums are read one after the other
@pytest.mark.parametrize("splits", [None, 1, 5])
@pytest.mark.parametrize("nh,nkv,d,ps,window,rot", [(8, 2, 128, 16, 0, 128), (6, 3, 48, 4, 0, 48), (32, 8, 128, 16, 0, 128),
                                                    (40, 2, 64, 8, 0, 32), (5, 5, 16, 16, 0, 0), (2, 1, 256, 64, 0, 256),
                                                    (8, 2, 128, 16, 100, 128), (4, 1, 96, 4, 17, 96),
                                                    (3, 1, 80, 12, 0, 80), (6, 2, 64, 20, 33, 64)])   # pages: no power of two
def test_attention_decode_rotating_equals_rotation_then_attention(nh, nkv, d, ps, window, rot, splits, gemm_splits):
    """One launch for rotation, write to the pages and attention against the two kernels one after the other:
    the same attention output and the same pages, bit for bit.  The QKV product comes as bf16 rows
    (gemm_splits 0) or as fp32 partial sums; the slot of the token's own key holds NaN before the call."""
    lens = [70, 1, 331, 64, 150, 16, 17, 65]
    B = len(lens)
    case = _paged_case(nh, nkv, d, ps, lens, [1] * B, torch.bfloat16, seed=d + nh + 7)
    g = torch.Generator().manual_seed(5)
    W = (nh + 2 * nkv) * d
    if gemm_splits == 0:
        qkv = torch.randn(B, W, generator=g).to(torch.bfloat16).to(DEV)
    else:
        qkv = K().SplitSum(torch.randn(gemm_splits, B, W, generator=g).to(DEV))
    inv_freq = None
    if rot:
        inv_freq = (10000.0 ** (-torch.arange(0, rot, 2, dtype=torch.float64) / rot)).to(DEV)
    pos = case["positions"]
    slots = torch.tensor([int(case["bt"][b, (L - 1) // ps]) * ps + (L - 1) % ps for b, L in enumerate(lens)],
                         dtype=torch.int32, device=DEV)
    for b, L in enumerate(lens):                   # whatever lies in the token's own slot must not be read
        pg, off = int(slots[b]) // ps, int(slots[b]) % ps
        case["kp"][pg, :, off] = float("nan")
        case["vp"][pg, :, :, off] = float("nan")
    scale = 1.0 / math.sqrt(d)
    kp1, vp1 = case["kp"].clone(), case["vp"].clone()
    q = K().rope_kv_append(qkv if gemm_splits else qkv.clone(), pos, inv_freq, nh, nkv, d, rot, slots, kp1, vp1)
    want = torch.full((B, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    K().attention_decode(q, kp1, vp1, want, pos, case["bt"], nh, nkv, d, scale, window, max(lens), num_splits=splits)
    assert not want.isnan().any()
    kp2, vp2 = case["kp"].clone(), case["vp"].clone()
    out = torch.full_like(want, float("nan"))
    K().attention_decode_rotating(qkv, pos, inv_freq, rot, slots, kp2, vp2, out, case["bt"], nh, nkv, d, scale, window,
                                  max(lens), num_splits=splits)
    assert torch.equal(out, want)
    assert torch.equal(kp2.view(torch.int16), kp1.view(torch.int16))
    assert torch.equal(vp2.view(torch.int16), vp1.view(torch.int16))
    # without slots: queries only, over pages that already hold the token's key and value
    out2 = torch.full_like(want, float("nan"))
    kp3, vp3 = kp1.clone(), vp1.clone()
    K().attention_decode_rotating(qkv, pos, inv_freq, rot, None, kp3, vp3, out2, case["bt"], nh, nkv, d, scale, window,
                                  max(lens), num_splits=splits)
    assert torch.equal(out2, want)
    assert torch.equal(kp3.view(torch.int16), kp1.view(torch.int16)) and torch.equal(vp3.view(torch.int16), vp1.view(torch.int16))


@pytest.mark.parametrize("nh,nkv,d,ps,window,rot", [(8, 2, 128, 16, 0, 128), (6, 3, 48, 4, 0, 48), (40, 2, 64, 8, 0, 32),
                                                    (5, 5, 16, 16, 0, 0), (2, 1, 256, 64, 0, 256), (4, 1, 96, 4, 17, 96),
                                                    (3, 1, 80, 12, 0, 80)])
def test_attention_decode_of_many_requests(nh, nkv, d, ps, window, rot):
    """A launch with more workgroups than the GPU has compute units gives a workgroup four waves, one with fewer
    eight (up to a head size of 128): the tests above are mostly of the second kind, this one, with 42 requests and
    as many parts of the keys as it takes, is of the first.  Against the plain reference, and the launch that rotates
    and writes the token's key and value against the two kernels one after the other, bit for bit."""
    lens = [70, 1, 331, 64, 150, 16, 17] * 6
    B = len(lens)
    groups = nkv * (-(-(nh // nkv) // 16))
    splits = 256 // (B * groups) + 1
    assert B * groups * splits > 256
    case = _paged_case(nh, nkv, d, ps, lens, [1] * B, torch.bfloat16, seed=d + nh + 3)
    scale = 1.0 / math.sqrt(d)
    out = torch.full((B, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    K().attention_decode(case["q"], case["kp"], case["vp"], out, case["positions"], case["bt"], nh, nkv, d, scale,
                         window, max(lens), num_splits=splits)
    want = _ref_attention(case, nh, nkv, d, scale, window)
    assert (out.double().cpu() - want).abs().max().item() <= 2e-2
    # the same keys in few workgroups (one part, the first seven requests): eight waves a workgroup up to d = 128
    few = torch.full((7, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    K().attention_decode(case["q"][:7], case["kp"], case["vp"], few, case["positions"][:7], case["bt"][:7], nh, nkv, d,
                         scale, window, max(lens), num_splits=1)
    assert (few.double().cpu() - want[:7]).abs().max().item() <= 2e-2
    # rotation inside the launch
    g = torch.Generator().manual_seed(5)
    W = (nh + 2 * nkv) * d
    qkv = K().SplitSum(torch.randn(3, B, W, generator=g).to(DEV))
    inv_freq = (10000.0 ** (-torch.arange(0, rot, 2, dtype=torch.float64) / rot)).to(DEV) if rot else None
    pos = case["positions"]
    slots = torch.tensor([int(case["bt"][b, (L - 1) // ps]) * ps + (L - 1) % ps for b, L in enumerate(lens)],
                         dtype=torch.int32, device=DEV)
    kp1, vp1 = case["kp"].clone(), case["vp"].clone()
    q = K().rope_kv_append(qkv, pos, inv_freq, nh, nkv, d, rot, slots, kp1, vp1)
    two = torch.full((B, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    K().attention_decode(q, kp1, vp1, two, pos, case["bt"], nh, nkv, d, scale, window, max(lens), num_splits=splits)
    kp2, vp2 = case["kp"].clone(), case["vp"].clone()
    one = torch.full_like(two, float("nan"))
    K().attention_decode_rotating(qkv, pos, inv_freq, rot, slots, kp2, vp2, one, case["bt"], nh, nkv, d, scale, window,
                                  max(lens), num_splits=splits)
    assert not two.isnan().any() and torch.equal(one, two)
    assert torch.equal(kp2.view(torch.int16), kp1.view(torch.int16)) and torch.equal(vp2.view(torch.int16), vp1.view(torch.int16))


@pytest.mark.parametrize("splits", [1, 3])
def test_attention_mfma_decode_block_table_longer_than_its_lds_slice(splits):
    """18,000 keys in pages of 4: 4,500 block-table entries, more than the 2,048 the decode kernel keeps in LDS;
    the rest is read from global memory.  One far key is loud, so a wrong page shows."""
    nh, nkv, d, ps = 4, 2, 32, 4
    lens = [18000, 5]
    case = _paged_case(nh, nkv, d, ps, lens, [1, 1], torch.bfloat16, seed=3, scale_one=(0, 17001, 6.0))
    out = torch.full((2, nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    scale = 1.0 / math.sqrt(d)
    K().attention_decode(case["q"], case["kp"], case["vp"], out, case["positions"], case["bt"], nh, nkv, d, scale,
                         0, max(lens), num_splits=splits)
    want = _ref_attention(case, nh, nkv, d, scale, 0)
    assert (out.double().cpu() - want).abs().max().item() <= 2e-2


def test_attention_mfma_far_key_stale_pages_and_missing_page():
    """A far key carries the softmax; pages hold NaN wherever this request has no data;
    a needed key without a page gives NaN instead of a fault."""
    nh, nkv, d, ps = 4, 1, 64, 16
    lens, q_lens = [500, 40, 77], [1, 40, 30]
    case = _paged_case(nh, nkv, d, ps, lens, q_lens, torch.bfloat16, seed=3, scale_one=(0, 17, 6.0))
    # poison every slot that holds no key of these requests
    used_k = torch.zeros_like(case["kp"], dtype=torch.bool)
    used_v = torch.zeros_like(case["vp"], dtype=torch.bool)
    for b, L in enumerate(lens):
        for i in range(-(-L // ps)):
            n = min(ps, L - i * ps)
            pg = int(case["bt"][b, i])
            used_k[pg, :, :n] = True
            used_v[pg, :, :, :n] = True
    case["kp"][~used_k] = float("nan")
    case["vp"][~used_v] = float("nan")
    scale = 1.0 / math.sqrt(d)
    want = _ref_attention(case, nh, nkv, d, scale, 0)
    out = torch.full((case["N"], nh * d), float("nan"), dtype=torch.bfloat16, device=DEV)
    starts = torch.tensor([0, 1, 41, 71], dtype=torch.int32, device=DEV)
    ctx = torch.tensor([499, 0, 47], dtype=torch.int32, device=DEV)
    tiles, nt = _prefill_tiles(q_lens, first_prefill=1)
    K().attention_prefill(case["q"], case["kp"], case["vp"], out, starts, ctx, case["bt"], tiles, nt, nh, nkv, d, scale, 0)
    K().attention_decode(case["q"][:1], case["kp"], case["vp"], out[:1], case["positions"][:1], case["bt"][:1], nh, nkv,
                         d, scale, 0, 500)
    assert not out.isnan().any()
    assert (out.double().cpu() - want).abs().max().item() <= 2e-2
    bt = case["bt"].clone()
    bt[0, 3] = -1
    K().attention_decode(case["q"][:1], case["kp"], case["vp"], out[:1], case["positions"][:1], bt[:1], nh, nkv, d,
                         scale, 0, 500)
    assert out[:1].isnan().all()


# -------------------------------------------------------------------- sampling
@pytest.mark.parametrize("V", [5, 250, 1024, 128256])
def test_argmax(V):
    x = _rand(4, V)
    x[1, V // 3] = 50.0
    x[2, :] = 1.0                                  # all equal: the lowest index wins
    x[3, V - 1] = 60.0
    x[3, V // 2] = 60.0
    out = torch.empty(4, dtype=torch.int32, device=DEV)
    K().argmax(x, out)
    assert out.tolist() == [int(torch.argmax(x[0])), V // 3, 0, V // 2]


def test_repetition_penalty():
    x = torch.tensor([[2.0, -2.0, 1.0, 4.0], [2.0, -2.0, 1.0, 4.0]], device=DEV)
    recent = torch.tensor([[0, 1, 0, 9], [3, 3, 3, 3]], dtype=torch.int32, device=DEV)
    counts = torch.tensor([3, 1], dtype=torch.int32, device=DEV)
    pen = torch.tensor([2.0, 4.0], device=DEV)
    K().repetition_penalty(x, recent, counts, pen)
    # a token that stands twice is penalised twice (infernum-cuda/src/inner/cuda/ops/sample.rs:101-112)
    assert x.tolist() == [[0.5, -4.0, 1.0, 4.0], [2.0, -2.0, 1.0, 1.0]]
    # a row's newest token may still be where an earlier launch left it: row 0 takes entry 2 of `previous` (token 1,
    # once more), row 1 none
    x = torch.tensor([[2.0, -2.0, 1.0, 4.0], [2.0, -2.0, 1.0, 4.0]], device=DEV)
    previous = torch.tensor([3, 0, 1], dtype=torch.int32, device=DEV)
    K().repetition_penalty(x, recent, counts, pen, previous, torch.tensor([2, -1], dtype=torch.int32, device=DEV))
    assert x.tolist() == [[0.5, -8.0, 1.0, 4.0], [2.0, -2.0, 1.0, 1.0]]


def _host_sample(logits, T, top_p, u):
    import plain_llama as P
    return P.sample_token(logits.cpu(), T, top_p, u)


@pytest.mark.parametrize("V", [7, 250, 5000])
def test_sample_matches_host_rule(V):
    import sys, os
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    R = 24
    x = _rand(R, V, scale=2.0, seed=9)
    g = torch.Generator().manual_seed(1)
    T = torch.rand(R, generator=g) * 1.5 + 0.2
    tp = torch.tensor([1.0, 0.9, 0.5, 0.1] * (R // 4))
    u = torch.rand(R, generator=g)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    work = torch.empty(R, V, device=DEV)
    K().sample(x, work, T.to(DEV), tp.to(DEV), u.to(DEV), out)
    bad = 0
    for r in range(R):
        want = _host_sample(x[r], float(T[r]), float(tp[r]), float(u[r]))
        if int(out[r]) != want:
            # only a draw within rounding of a boundary of the CDF may differ
            xr = x[r].double().cpu() / float(T[r])
            e = torch.exp(xr - xr.max())
            bad += 1
            assert e[int(out[r])] > 0
    assert bad <= 1


@pytest.mark.parametrize("V", [50000, 50001, 128256])
def test_sample_of_a_row_alone_and_again(V):
    """A row's token does not depend on the rows beside it nor on the run: masses are integers, their sums exact.
    V = 50001 takes the path of single loads, the others that of 16-byte loads."""
    R = 6
    x = _rand(R, V, scale=3.0, seed=21)
    g = torch.Generator().manual_seed(2)
    T = (torch.rand(R, generator=g) + 0.3).to(DEV)
    tp = torch.tensor([1.0, 0.95, 0.9, 0.5, 0.1, 0.999], device=DEV)
    u = torch.rand(R, generator=g).to(DEV)
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    K().sample(x, torch.empty(R, V, device=DEV), T, tp, u, out)
    again = torch.empty_like(out)
    K().sample(x, torch.empty(R, V, device=DEV), T, tp, u, again)
    assert torch.equal(out, again)
    for r in range(R):
        one = torch.empty(1, dtype=torch.int32, device=DEV)
        K().sample(x[r:r + 1].contiguous(), torch.empty(1, V, device=DEV), T[r:r + 1].contiguous(),
                   tp[r:r + 1].contiguous(), u[r:r + 1].contiguous(), one)
        assert int(one[0]) == int(out[r]), r
    # against the rule worked out on the host in float64: only a draw within 1e-4 of a boundary of the running
    # mass may differ (masses are cut off at 2^-31 of the largest one)
    differ = sum(int(out[r]) != _host_sample(x[r], float(T[r]), float(tp[r]), float(u[r])) for r in range(R))
    assert differ <= 1, differ


def test_sample_limits_and_frequencies():
    V = 50
    x = _rand(1, V, scale=1.5, seed=3)
    # low temperature: the maximum (sample.rs:176-183); same inputs, same token (sample.rs:167-173)
    out = torch.empty(1, dtype=torch.int32, device=DEV)
    work = torch.empty(1, V, device=DEV)
    one = lambda v: torch.tensor([v], device=DEV)
    K().sample(x, work, one(1e-3), one(0.9), one(0.7), out)
    assert int(out[0]) == int(torch.argmax(x[0]))
    # frequencies over many draws follow softmax(x / T)
    R = 20000
    xs = x.expand(R, V).contiguous()
    u = torch.rand(R, generator=torch.Generator().manual_seed(5)).to(DEV)
    outs = torch.empty(R, dtype=torch.int32, device=DEV)
    K().sample(xs, torch.empty(R, V, device=DEV), torch.full((R,), 0.8, device=DEV), torch.ones(R, device=DEV), u, outs)
    freq = torch.bincount(outs.long().cpu(), minlength=V).double() / R
    p = torch.softmax(x[0].double().cpu() / 0.8, 0)
    chi2 = (R * (freq - p) ** 2 / p).sum().item()
    assert chi2 < 100.0, chi2            # 49 degrees of freedom: 100 is far in the tail
    # top_p keeps the nucleus only
    K().sample(xs, torch.empty(R, V, device=DEV), torch.full((R,), 0.8, device=DEV), torch.full((R,), 0.5, device=DEV),
               u, outs)
    srt, idx = torch.sort(p, descending=True)
    n_keep = int(torch.nonzero(torch.cumsum(srt, 0) >= 0.5)[0]) + 1
    assert set(outs.tolist()) <= set(idx[:n_keep].tolist())


# ------------------------------------------------------------------- utilities
def test_cast_rounds_to_nearest_even_and_widens_exactly():
    g = torch.Generator().manual_seed(3)
    x = torch.cat([torch.randn(100003, generator=g) * 7.0,
                   torch.tensor([0.0, -0.0, 1.0, 1.00390625, 1.01171875, float("inf"), -float("inf"), 3.0e38, 1e-40])]).to(DEV)
    down = K().cast(x, torch.bfloat16)
    assert down.dtype == torch.bfloat16 and torch.equal(down, x.to(torch.bfloat16))      # ties to even, as the library
    up = K().cast(down, torch.float32)
    assert torch.equal(up, down.float())
    assert torch.isnan(K().cast(torch.tensor([float("nan")], device=DEV), torch.bfloat16)).all()
    same = K().cast(x, torch.float32)
    assert torch.equal(same, x) and same.data_ptr() != x.data_ptr()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_copy_pages(dtype):
    pool = _rand(9, 3, 5, 6, dtype=dtype)              # pages of 90 values: no multiple of a thread block
    before = pool.clone()
    src = torch.tensor([0, 2, 7, 99, 4, -1], dtype=torch.int32, device=DEV)
    dst = torch.tensor([1, 3, 8, 5, 4, 6], dtype=torch.int32, device=DEV)
    K().copy_pages(pool, src, dst)
    want = before.clone()
    for s, d in ((0, 1), (2, 3), (7, 8)):              # a pair with a page outside the pool, or onto itself, is left out
        want[d] = before[s]
    assert torch.equal(pool, want)
