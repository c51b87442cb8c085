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


# Whether ``decode_weight`` lays bf16 matrices out in tiles for the few-row product (the engine's setting; the
# matrix row by row is kept beside the tiles for the products that go to the library).
_TILED_WEIGHTS = True


def set_tiled_weights(on: bool) -> None:
    global _TILED_WEIGHTS
    _TILED_WEIGHTS = bool(on)


def decode_weight(w: torch.Tensor):
    """A part's matrix ``[N, K]`` as its products want it: bf16 on the GPU in tiles (``ops.TiledWeight``, the
    rows kept beside them), anything else as it is."""
    if _TILED_WEIGHTS and w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2:
        return ops.TiledWeight(w.contiguous())
    return w


def linear(x: torch.Tensor, w, out: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, sliced_ok: bool = False):
    """``w`` is a matrix ``[N, K]`` or an ``ops.TiledWeight``.  ``sliced_ok``: the caller hands the result to a
    kernel that takes ``ops.SlicedSums`` (the unreduced K slices of a product with few rows)."""
    m, k = x.shape
    n = w.shape[0]
    out_dtype = out_dtype or (out.dtype if out is not None else x.dtype)
    if x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and m > 0:
        fast = ops.gemm_bf16(x, w, out, out_dtype=out_dtype, sliced_ok=sliced_ok)
        if fast is not None:
            return fast
    if isinstance(w, ops.TiledWeight):
        if w.rows is None:
            raise ops.KernelError("linear: this product needs the matrix row by row, which was not kept")
        w = w.rows
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
