"""The matrix product of every projection: y[M, N] = x[M, K] @ W[N, K]^T.

Weights stay in the layout of the file ([out, in]: rows contiguous in K, which
is what a product that streams the weight once wants); the reference transposes
them on the host instead (infernum-cuda/src/inner/weights/generic_impl.rs:107-131)
and calls cuBLAS (infernum-cuda/src/inner/cuda/ops/matmul.rs:68-117).

fp32: the hand-written fp32 kernel, always (no reduced-precision matrix mode).
bf16: up to 64 rows the hand-written MFMA kernel that streams the weight once;
above that the library product (hipBLASLt through torch), as the reference uses
its library there; an fp32 result of many rows comes from the generic kernel.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import api as K


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    M, Kdim = x.shape
    N = w.shape[0]
    out_dtype = out_dtype or x.dtype
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M == 0:
        return out
    if x.dtype == torch.float32:
        return K.gemm_generic(x, w, out)
    if x.dtype != torch.bfloat16:
        raise K.KernelError(f"linear: dtype {x.dtype} is not supported")
    if K.gemm_skinny_available() and K.gemm_skinny_supported(M, N, Kdim) and x.is_contiguous():
        return K.gemm_skinny(x, w, out)
    if out_dtype == torch.bfloat16:
        return torch.mm(x, w.t(), out=out)          # library product, fp32 accumulation
    # fp32 result from bf16 operands, many rows: 64 rows at a time through the skinny kernel
    if K.gemm_skinny_available() and K.gemm_skinny_supported(1, N, Kdim) and x.is_contiguous():
        for m0 in range(0, M, K.SKINNY_MAX_M):
            m1 = min(M, m0 + K.SKINNY_MAX_M)
            K.gemm_skinny(x[m0:m1], w, out[m0:m1])
        return out
    return K.gemm_generic(x, w, out)
