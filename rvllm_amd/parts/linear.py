"""Matrix products of the parts: out = x @ w^T.

The 32-bit path uses the hand-written kernel with 32-bit multiply-adds only.
The bf16 path hands plain products to the library through torch (hipBLASLt /
rocBLAS), as the reference hands its products to cuBLASLt
(v3/crates/rvllm-cutlass/src/cublaslt.rs:277); products with few rows, and
products with 32-bit output from bf16 inputs (the logits), run on the
hand-written kernels.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops


def linear(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, sliced_ok: bool = False):
    """``sliced_ok``: the caller hands the result to a kernel that takes
    ``ops.SlicedSums`` (the unreduced K slices of a product with few rows)."""
    m, k = x.shape
    n = w.shape[0]
    out_dtype = out_dtype or (out.dtype if out is not None else x.dtype)
    if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and m > 0:
        fast = ops.gemm_bf16(x, w, out, out_dtype=out_dtype, sliced_ok=sliced_ok)
        if fast is not None:
            return fast
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    if m == 0:
        return out
    if x.dtype == torch.float32:
        if w.dtype not in (torch.float32, torch.bfloat16):
            raise ops.KernelError(f"linear: unsupported weight dtype {w.dtype}")
        return ops.gemm_plain(x, w, out)
    if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16:
        if out.dtype == torch.bfloat16:
            return torch.matmul(x, w.t(), out=out)
        return ops.gemm_plain(x, w, out)
    raise ops.KernelError(f"linear: unsupported dtypes x={x.dtype} w={w.dtype}")
