"""The entry point that allocates nothing, ``ia_gemm_skinny_no_alloc``, called through ctypes as a caller
outside Python would: its output against ``ia_gemm_skinny``'s (the same kernels with a workspace that the
caller brings) on two calls in a row, the second with a smaller input, so that what the first left in the
library's array lies beside what the second writes."""
import ctypes
import gc

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ERR_SCRATCH_TOO_SMALL = 10004


def _lib():
    from infernum_amd.csrc import build
    lib = ctypes.CDLL(build.ensure("core"))
    lib.ia_gemm_skinny_no_alloc_needs.restype = ctypes.c_size_t
    lib.ia_gemm_skinny_no_alloc_capacity.restype = ctypes.c_size_t
    return lib


def _p(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _operands(M, N, K, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).to(DEV)
    return x, w


def _with_workspace(lib, x, w, out_dtype, epilogue, stream):
    """The existing entry point, its workspace allocated here."""
    M, K = x.shape
    N = w.shape[0]
    splits = lib.ia_gemm_skinny_splits(N, K)
    ws = torch.empty(max(splits * M * N, 1), dtype=torch.float32, device=DEV)
    out = torch.empty((M, N // 2 if epilogue else N), dtype=out_dtype, device=DEV)
    rc = lib.ia_gemm_skinny(_p(x), _p(w), _p(out), 0 if out_dtype == torch.float32 else 1, M, N, K, epilogue,
                            _p(ws), ctypes.c_size_t(ws.numel()), stream)
    assert rc == 0
    return out


def _no_alloc(lib, x, w, out, epilogue, stream):
    M, K = x.shape
    return lib.ia_gemm_skinny_no_alloc(_p(x), _p(w), _p(out), 0 if out.dtype == torch.float32 else 1, M, w.shape[0], K,
                                       epilogue, stream)


# (M, N, K, epilogue) of the first call and of the second, smaller one; all split K (N gives few workgroups)
CASES = [
    ((64, 4096, 4096, 0), (8, 1024, 2048, 0)),          # output-projection shapes
    ((33, 6144, 4096, 0), (1, 6144, 4096, 0)),          # QKV, then the same weight with one row
    ((128, 1000, 14336, 0), (5, 328, 1000, 0)),         # widths that are no power of two
    ((16, 2048, 1024, 1), (3, 512, 512, 1)),            # SwiGLU applied while the parts are joined
]


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("first,second", CASES)
def test_two_calls_in_a_row_give_what_the_workspace_entry_point_gives(first, second, out_dtype):
    lib = _lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs, wants = [], []
    operands = [_operands(*c[:3], seed=11 + i) for i, c in enumerate((first, second))]
    for (M, N, K, epi), (x, w) in zip((first, second), operands):
        assert lib.ia_gemm_skinny_splits(N, K) > 1, "the case is meant to use the scratch array"
        assert 0 < lib.ia_gemm_skinny_no_alloc_needs(M, N, K, epi) <= lib.ia_gemm_skinny_no_alloc_capacity()
        wants.append(_with_workspace(lib, x, w, out_dtype, epi, stream))
    torch.cuda.synchronize()
    # the outputs are the caller's: made before the two calls, which then run back to back
    for (M, N, K, epi) in (first, second):
        outs.append(torch.full((M, N // 2 if epi else N), float("nan"), dtype=out_dtype, device=DEV))
    torch.cuda.synchronize()
    gc.collect()            # what earlier tests left in reference cycles goes now, not between the two readings
    before = torch.cuda.memory_allocated()
    for (M, N, K, epi), (x, w), out in zip((first, second), operands, outs):
        assert _no_alloc(lib, x, w, out, epi, stream) == 0
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    for out, want in zip(outs, wants):
        assert torch.equal(out, want)
    # and against the product itself
    (M, N, K, epi), (x, w) = second, operands[1]
    y = x.double() @ w.double().t()
    if epi:
        y = torch.nn.functional.silu(y[:, :N // 2]) * y[:, N // 2:]
    tol = 2e-2 if out_dtype == torch.bfloat16 else 1e-3
    assert torch.allclose(outs[1].double(), y, atol=tol, rtol=tol)


def test_a_product_without_split_needs_no_scratch_and_works():
    lib = _lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    M, N, K = 8, 28672, 512                      # many rows of W: one part
    assert lib.ia_gemm_skinny_splits(N, K) == 1 and lib.ia_gemm_skinny_no_alloc_needs(M, N, K, 1) == 0
    x, w = _operands(M, N, K, seed=5)
    for epi in (0, 1):
        want = _with_workspace(lib, x, w, torch.bfloat16, epi, stream)
        out = torch.empty_like(want)
        assert _no_alloc(lib, x, w, out, epi, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_sizes_beyond_the_array_are_refused_and_nothing_is_written():
    lib = _lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    M, N, K = 128, 6144, 8192
    need = lib.ia_gemm_skinny_no_alloc_needs(M, N, K, 0)
    assert need > lib.ia_gemm_skinny_no_alloc_capacity()
    x, w = _operands(M, N, K, seed=7)
    out = torch.full((M, N), 3.0, dtype=torch.bfloat16, device=DEV)
    assert _no_alloc(lib, x, w, out, 0, stream) == ERR_SCRATCH_TOO_SMALL
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())
    # malformed calls are refused too
    assert lib.ia_gemm_skinny_no_alloc(_p(x), _p(w), None, 1, M, N, K, 0, stream) == 10001
    assert lib.ia_gemm_skinny_no_alloc(_p(x), _p(w), _p(out), 1, 129, N, K, 0, stream) == 10002
    assert lib.ia_gemm_skinny_no_alloc(_p(x), _p(w), _p(out), 1, M, N, 12, 0, stream) == 10002
