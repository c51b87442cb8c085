"""Matrix products of the parts: out = x @ w^T.

The 32-bit path uses the hand-written kernel with 32-bit multiply-adds only.
The bf16 path hands plain products of many rows to the library (hipBLASLt,
called from the kernel library itself: ``csrc/library_gemm.hip``), as the
reference hands its products to cuBLASLt
(v3/crates/rvllm-cutlass/src/cublaslt.rs:277); products with few rows, and
products with 32-bit output from bf16 inputs (the logits), run on the
hand-written kernels.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops


def decode_weight(w: torch.Tensor, tiled: bool = True):
    """A part's matrix ``[N, K]`` as its products want it: with ``tiled`` (the part's ``tiled_weights``, which
    is the engine's setting) a bf16 matrix on the GPU goes into tiles for the few-row product
    (``ops.TiledWeight``; the matrix row by row is kept beside the tiles for the products that go to the
    library), anything else stays as it is."""
    if w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2:
        w = w.contiguous()
        ops.library_matrix_register(w)  # the tuning of the products of many rows takes a shape's matrices in turn
        if tiled:
            return ops.TiledWeight(w)
    return w


def tensor_names(defaults: dict, given) -> dict:
    """A part's table of tensor names: ``defaults`` (role -> name under the layer's prefix, without
    ``.weight``) with the roles that the part's spec names otherwise (``names``) laid over it."""
    names = dict(defaults)
    for role, name in dict(given or {}).items():
        names[str(role)] = str(name)
    return names


def bias_roles(given, roles) -> frozenset:
    """The roles among ``roles`` whose projection has a bias: the spec's ``bias`` is absent or False (none),
    True (all of them) or a list of roles."""
    if not given:
        return frozenset()
    if given is True:
        return frozenset(roles)
    wanted = frozenset(str(r) for r in given)
    unknown = wanted - frozenset(roles)
    if unknown:
        raise ValueError(f"bias for unknown projections {sorted(unknown)}; this part has {sorted(roles)}")
    return wanted


def linear(x: torch.Tensor, w, out: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, sliced_ok: bool = False):
    """``w`` is a matrix ``[N, K]`` or an ``ops.TiledWeight``.  ``sliced_ok``: the caller hands the result to a
    kernel that takes ``ops.SlicedSums`` (the unreduced K slices of a product with few rows)."""
    m, k = x.shape
    n = w.shape[0]
    out_dtype = out_dtype or (out.dtype if out is not None else x.dtype)
    bf16 = x.dtype is torch.bfloat16 and w.dtype is torch.bfloat16
    if bf16 and m > ops.SKINNY_MAX_ROWS and out_dtype in (torch.bfloat16, torch.float32):
        # many rows: the library's, on the matrix row by row
        rows = w.rows if isinstance(w, ops.TiledWeight) else w
        if rows is not None:
            if out is None:
                out = torch.empty((m, n), dtype=out_dtype, device=x.device)
            if ops.library_gemm(x, rows, out) is not None:
                return out
        if out_dtype is torch.float32:  # no algorithm: the few-row kernel, 64 rows at a time
            fast = ops.gemm_bf16(x, w, out, out_dtype=out_dtype, sliced_ok=sliced_ok)
            if fast is not None:
                return fast
    elif bf16 and m > 0:
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
        if out.dtype == torch.bfloat16 and ops.library_gemm(x, w, out) is not None:
            return out
        return ops.gemm_plain(x, w, out)
    raise ops.KernelError(f"linear: unsupported dtypes x={x.dtype} w={w.dtype}")
