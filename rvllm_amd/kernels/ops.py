"""Python face of the HIP kernels.

Every function takes torch tensors that live on the GPU, checks their shapes
and types on the host, and launches on torch's current stream, so the calls
can be captured in a HIP graph.  Nothing here computes on the CPU or falls
back to a library: if the kernel library cannot be loaded the call raises.
"""

from __future__ import annotations

import ctypes
import functools
import threading
from typing import Optional

import torch

from . import build as _build
from . import signatures as _signatures

_lib = None
_lock = threading.Lock()

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


def library():
    """The loaded kernel library; builds it when no current build exists."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                path = _build.ensure_built()
                try:
                    cdll = ctypes.CDLL(str(path))
                except OSError as e:  # pragma: no cover
                    raise KernelError(f"cannot load the kernel library {path}: {e}") from e
                # every entry point's argument types, from the sources the library was built from
                _lib = _signatures.Library(cdll, _signatures.read_signatures(_build.CSRC))
    return _lib


def library_path() -> Optional[str]:
    p = _build.find_library()
    return str(p) if p else None


def _check(code: int) -> None:
    if code != 0:
        raise KernelError(library().rv_last_error().decode())


# torch's current stream as a raw handle.  torch.cuda.current_stream() builds a Python object on the way and costs
# some microseconds, a third of the host's time for a step of several hundred launches; the binding below it does not.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)


# The entry points' argument types are declared (``signatures.py``), so a call takes plain numbers: an address as an
# int or None, a float as a float.  Building a ctypes object for each of the twenty-odd arguments of a launch cost
# more than the rest of the call.
def _stream() -> int:
    if _raw_stream is not None and _current_device is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelError(f"unsupported dtype {t.dtype}; kernels take float32 and bfloat16") from None


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None:
            _need(t.is_cuda, "kernel arguments must live on the GPU")
            _need(t.is_contiguous(), "kernel arguments must be contiguous")


def _i32(*tensors: torch.Tensor) -> None:
    for t in tensors:
        _need(t.dtype == torch.int32, f"index tensors must be int32, got {t.dtype}")


_c_int, _c_float, _c_ll = int, float, int


V_GROUP = 16  # slots whose values of one dimension lie side by side (RV_V_GROUP of csrc/kv_layout.h)


def _cache_geometry(k_pages: torch.Tensor, v_pages: torch.Tensor, what: str) -> tuple[int, int, int, int]:
    """(pages, kv heads, page size, head size) of a layer's cache: keys are
    ``[pages, kv_heads, page_size, head_dim]``, values are transposed inside
    groups of 16 slots, ``[pages, kv_heads, page_size / 16, head_dim, 16]``."""
    _need(k_pages.dim() == 4 and v_pages.dim() == 5, f"{what}: key pages must have four dimensions, value pages five")
    num_pages, nkv, page_size, hd = k_pages.shape
    _need(page_size % V_GROUP == 0 and tuple(v_pages.shape) == (num_pages, nkv, page_size // V_GROUP, hd, V_GROUP),
          f"{what}: keys are {tuple(k_pages.shape)}, so values must be "
          f"{(num_pages, nkv, page_size // V_GROUP, hd, V_GROUP)} with pages a multiple of {V_GROUP}, "
          f"got {tuple(v_pages.shape)}")
    return num_pages, nkv, page_size, hd


class SlicedSums:
    """The result of a product whose K range was split over blocks, not yet
    added up: 32-bit partial sums ``[slices, rows, width]``.  The kernels that
    consume a product's result (norm + residual add, q/k norm and rotation,
    gated activation) add the slices themselves, in their order, which saves a
    kernel and a rounding; anything else calls ``as_tensor``."""

    def __init__(self, data: torch.Tensor, dtype: torch.dtype):
        self.data = data  # [slices, rows, width] float32
        self.dtype = dtype  # what the product's result would be stored as
        self.slices, self.rows, self.width = data.shape

    @property
    def shape(self):
        return (self.rows, self.width)

    @property
    def device(self):
        return self.data.device

    def as_tensor(self) -> torch.Tensor:
        out = torch.empty((self.rows, self.width), dtype=self.dtype, device=self.data.device)
        _check(library().rv_reduce_slices(_stream(), _ptr(self.data), _ptr(out), _dt(out), _c_int(self.slices),
                                          _c_int(self.rows), _c_int(self.width)))
        return out


class TiledWeight:
    """A bf16 matrix ``[N, K]`` stored for the few-row product: in tiles of 16 rows x 32 columns, each tile's
    1 KB in the order in which the 64 lanes of a matrix-core product hold it, a row of tiles (all of K)
    contiguous, so that a wave reads its share of the matrix as one contiguous stream.  ``rows`` is the same
    matrix row by row, kept for the products that go to the library (more than 64 rows), or None."""

    def __init__(self, rows: torch.Tensor, keep_rows: bool = True):
        _gpu(rows)
        _need(rows.dim() == 2 and rows.dtype == torch.bfloat16, "TiledWeight: a bf16 matrix expected")
        self.n, self.k = rows.shape
        lib = library()
        lib.rv_tile_weight_elements.restype = ctypes.c_longlong
        self.tiles = torch.empty(lib.rv_tile_weight_elements(_c_int(self.n), _c_int(self.k)), dtype=torch.bfloat16,
                                 device=rows.device)
        _check(lib.rv_tile_weight(_stream(), _ptr(rows), _ptr(self.tiles), _c_int(self.n), _c_int(self.k),
                                  _c_ll(rows.stride(0))))
        self.rows = rows if keep_rows else None

    @property
    def shape(self):
        return (self.n, self.k)

    @property
    def dtype(self):
        return torch.bfloat16

    @property
    def device(self):
        return self.tiles.device


def as_tensor(x) -> torch.Tensor:
    """A plain tensor from a tensor or from unreduced ``SlicedSums``."""
    return x.as_tensor() if isinstance(x, SlicedSums) else x


def _branch_args(x, what: str):
    """(pointer, slices, slice stride, rows, width, dtype) of a kernel input
    that is a tensor or ``SlicedSums``."""
    if isinstance(x, SlicedSums):
        return _ptr(x.data), x.slices, x.rows * x.width, x.rows, x.width, x.dtype
    _gpu(x)
    _need(x.dim() == 2, f"{what}: a matrix is expected")
    return _ptr(x), 0, 0, x.shape[0], x.shape[1], x.dtype


# --------------------------------------------------------------------------
def embed_gather(table: torch.Tensor, ids: torch.Tensor, scale: float, out: torch.Tensor) -> torch.Tensor:
    _gpu(table, ids, out)
    _i32(ids)
    vocab, hidden = table.shape
    n = ids.numel()
    _need(out.shape == (n, hidden), f"embed_gather: out is {tuple(out.shape)}, expected {(n, hidden)}")
    _check(library().rv_embed_gather(_stream(), _ptr(table), _dt(table), _ptr(ids), _ptr(out), _dt(out), _c_int(n),
                                     _c_int(hidden), _c_int(vocab), _c_float(scale)))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, offset: float,
            out: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Row-wise RMSNorm.  With ``rows`` (int32 indices into the rows of a 2-d
    ``x``, all in range: the caller built them) output row r is the norm of
    x[rows[r]]."""
    width = x.shape[-1]
    if rows is not None:
        _need(x.dim() == 2, "rmsnorm: a row index needs a 2-d input")
        _i32(rows)
        n_rows = rows.numel()
        if out is None:
            out = torch.empty((n_rows, width), dtype=x.dtype, device=x.device)
        _need(out.shape == (n_rows, width) and out.dtype == x.dtype, "rmsnorm: bad out")
    else:
        n_rows = x.numel() // width
        if out is None:
            out = torch.empty_like(x)
        _need(out.shape == x.shape and out.dtype == x.dtype, "rmsnorm: out must match x")
    _gpu(x, weight, out, rows)
    _need(weight.shape == (width,), f"rmsnorm: weight is {tuple(weight.shape)}, expected ({width},)")
    _check(library().rv_rmsnorm(_stream(), _ptr(x), _ptr(rows), _ptr(weight), _c_int(weight.dtype == torch.float32),
                                _ptr(out), _dt(x), _c_int(n_rows), _c_int(width), _c_float(eps), _c_float(offset)))
    return out


def add_rmsnorm(branch, weight: torch.Tensor, eps: float, offset: float, residual: torch.Tensor,
                next_weight: Optional[torch.Tensor] = None, next_eps: float = 0.0, next_offset: float = 0.0,
                next_out: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """residual += rmsnorm(branch); with ``next_weight`` also returns rmsnorm(residual).
    ``branch`` is a tensor or ``SlicedSums``."""
    bptr, slices, stride, rows, width, bdtype = _branch_args(branch, "add_rmsnorm")
    _gpu(weight, residual, next_weight, next_out)
    _need(residual.shape == (rows, width) and residual.dtype == bdtype, "add_rmsnorm: residual must match branch")
    _need(weight.shape == (width,), "add_rmsnorm: bad weight shape")
    if next_weight is not None:
        _need(next_weight.shape == (width,), "add_rmsnorm: bad next weight shape")
        if next_out is None:
            next_out = torch.empty_like(residual)
        _need(next_out.shape == residual.shape and next_out.dtype == residual.dtype, "add_rmsnorm: bad next_out")
    _check(library().rv_add_rmsnorm(
        _stream(), bptr, _c_int(slices), _c_ll(stride), _ptr(weight), _c_int(weight.dtype == torch.float32),
        _ptr(residual), _ptr(next_weight), _c_int(next_weight is not None and next_weight.dtype == torch.float32),
        _ptr(next_out if next_weight is not None else None), _dt(residual), _c_int(rows), _c_int(width), _c_float(eps),
        _c_float(offset), _c_float(next_eps), _c_float(next_offset)))
    return next_out if next_weight is not None else None


ACTIVATIONS = {"gelu_pytorch_tanh": 0, "gelu_tanh": 0, "silu": 1}


# The widths whose gate and up rows may lie in fours (see ``rows_in_fours``): a thread of ``gated_act`` then takes
# its 16 bytes of outputs from 32 neighbouring bytes.
FOURS_WIDTH_MULTIPLE = 8


def rows_in_fours(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The rows of a gate and an up projection ``[I, H]`` as one matrix ``[2 I, H]`` in fours: gates 2q and
    2q + 1, then ups 2q and 2q + 1.  A product against it leaves each gate two places from its up, so that
    ``gemm_bf16_gate_up`` can apply the activation where it holds the sums, and ``gated_act(..., fours=True)``
    reads both from neighbouring bytes."""
    inter, hidden = gate.shape
    _need(up.shape == gate.shape and inter % 2 == 0, "rows_in_fours: two matrices of one shape with an even number of rows")
    return torch.cat([gate.reshape(inter // 2, 2, hidden), up.reshape(inter // 2, 2, hidden)], dim=1).reshape(
        2 * inter, hidden).contiguous()


def gated_act(gate_up, activation: str, out: Optional[torch.Tensor] = None, fours: bool = False) -> torch.Tensor:
    """out[t, i] = act(gate[t, i]) * up[t, i]; ``gate_up`` is a tensor or ``SlicedSums`` whose rows hold the gates
    and then the ups (gate i at i, up i at I + i) or, with ``fours``, what a product against ``rows_in_fours``
    leaves."""
    gptr, slices, stride, rows, two_i, dtype = _branch_args(gate_up, "gated_act")
    _need(two_i % 2 == 0, "gated_act: width must be even")
    inter = two_i // 2
    if out is None:
        out = torch.empty((rows, inter), dtype=dtype, device=gate_up.device)
    _gpu(out)
    _need(out.shape == (rows, inter) and out.dtype == dtype, "gated_act: bad out")
    _need(activation in ACTIVATIONS, f"gated_act: unknown activation {activation!r}")
    _check(library().rv_gated_act(_stream(), gptr, _c_int(slices), _c_ll(stride), _ptr(out), _dt(out), _c_int(rows),
                                  _c_int(inter), _c_int(ACTIVATIONS[activation]), _c_int(int(fours))))
    return out


def add_bias(x, bias: torch.Tensor) -> torch.Tensor:
    """x + bias, row by row: in place for a tensor; unreduced ``SlicedSums`` are added up and the bias with
    them, into a new tensor of the product's type."""
    _gpu(bias)
    if isinstance(x, SlicedSums):
        out = torch.empty((x.rows, x.width), dtype=x.dtype, device=x.device)
        part, slices = x.data, x.slices
    else:
        _gpu(x)
        _need(x.dim() == 2, "add_bias: a matrix is expected")
        out, part, slices = x, None, 0
    rows, width = out.shape
    _need(bias.shape == (width,) and bias.dtype in _DT, f"add_bias: the bias must hold {width} numbers")
    _check(library().rv_add_bias(_stream(), _ptr(out), _dt(out), _ptr(part), _c_int(slices), _ptr(bias),
                                 _c_int(bias.dtype == torch.float32), _c_int(rows), _c_int(width)))
    return out


def softcap_(logits: torch.Tensor, cap: float) -> torch.Tensor:
    _gpu(logits)
    _need(logits.dtype == torch.float32, "softcap: logits must be float32")
    _check(library().rv_softcap(_stream(), _ptr(logits), _c_ll(logits.numel()), _c_float(cap)))
    return logits


def gemm_plain(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[M, N] = a[M, K] @ w[N, K]^T with 32-bit multiply-adds."""
    _need(a.is_cuda and w.is_cuda and out.is_cuda, "gemm: arguments must live on the GPU")
    _need(a.dim() == 2 and w.dim() == 2 and out.dim() == 2, "gemm: matrices expected")
    m, k = a.shape
    n, k2 = w.shape
    _need(k == k2, f"gemm: inner sizes differ: {k} vs {k2}")
    _need(out.shape == (m, n), f"gemm: out is {tuple(out.shape)}, expected {(m, n)}")
    _need(a.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1, "gemm: rows must be contiguous")
    _check(library().rv_gemm_plain(_stream(), _ptr(a), _dt(a), _ptr(w), _dt(w), _ptr(out), _dt(out), _c_int(m),
                                   _c_int(n), _c_int(k), _c_ll(a.stride(0) if m > 1 else k),
                                   _c_ll(w.stride(0) if n > 1 else k), _c_ll(out.stride(0) if m > 1 else n)))
    return out


def rope_table(inv_freq: torch.Tensor, positions: torch.Tensor, num_tokens: int) -> tuple[torch.Tensor, torch.Tensor]:
    """(cos, sin) of float(position) * inv_freq[i] for the first ``num_tokens``
    positions: two 32-bit tensors ``[num_tokens, len(inv_freq)]``."""
    _gpu(inv_freq, positions)
    _i32(positions)
    _need(inv_freq.dtype == torch.float32 and inv_freq.dim() == 1 and inv_freq.numel() > 0, "rope_table: bad inv_freq")
    _need(positions.numel() >= num_tokens, "rope_table: positions too short")
    half = inv_freq.numel()
    cos = torch.empty((num_tokens, half), dtype=torch.float32, device=inv_freq.device)
    sin = torch.empty_like(cos)
    _check(library().rv_rope_table(_stream(), _ptr(inv_freq), _ptr(positions), _ptr(cos), _ptr(sin), _c_int(num_tokens),
                                   _c_int(half)))
    return cos, sin


def qk_norm_rope_kv_write(qkv, q_out: torch.Tensor, q_weight: Optional[torch.Tensor],
                          k_weight: Optional[torch.Tensor], eps: float, offset: float,
                          rope: Optional[tuple[torch.Tensor, torch.Tensor]], rotary_dim: int, positions: torch.Tensor,
                          token_req: torch.Tensor, block_table: Optional[torch.Tensor],
                          k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], num_q_heads: int,
                          num_kv_heads: int, head_dim: int, write_kv: bool = True,
                          values_by_page=None) -> torch.Tensor:
    """Query/key norm and rotation; queries to ``q_out``, keys and values into the cache (``write_kv``).
    ``values_by_page`` is the step (its q_start, chunk_start, num_requests, max_portion) when extra blocks of the
    same launch are to write the values a page at a time, which pays for prompt portions; the projection must
    then be whole, not partial sums."""
    qptr, slices, stride, n, qkv_width, qkv_dtype = _branch_args(qkv, "qk_norm_rope")
    rope_cos, rope_sin = rope if rope is not None else (None, None)
    _gpu(q_out, q_weight, k_weight, rope_cos, rope_sin, positions, token_req, block_table, k_pages, v_pages)
    _i32(positions, token_req)
    _need(qkv_width == (num_q_heads + 2 * num_kv_heads) * head_dim, "qk_norm_rope: bad qkv shape")
    _need(q_out.shape == (n, num_q_heads * head_dim) and q_out.dtype == qkv_dtype, "qk_norm_rope: bad q_out")
    _need(positions.numel() >= n and token_req.numel() >= n, "qk_norm_rope: positions/token_req too short")
    w_f32 = 0
    if q_weight is not None:
        _need(k_weight is not None and q_weight.shape == (head_dim,) and k_weight.shape == (head_dim,),
              "qk_norm_rope: bad norm weights")
        _need(q_weight.dtype == k_weight.dtype, "qk_norm_rope: norm weights must share a dtype")
        w_f32 = int(q_weight.dtype == torch.float32)
    if rope is not None:
        for table in (rope_cos, rope_sin):
            _need(table.dtype == torch.float32 and table.is_contiguous() and table.shape == (n, rotary_dim // 2),
                  f"qk_norm_rope: the table of cosines and sines must be 32-bit [{n}, {rotary_dim // 2}]")
    page_size = num_pages = width = 0
    by_page = bool(write_kv) and values_by_page is not None
    if by_page:
        _need(slices == 0, "qk_norm_rope: values by pages need a projection that is already added up")
        _gpu(values_by_page.q_start, values_by_page.chunk_start)
        _i32(values_by_page.q_start, values_by_page.chunk_start)
    if write_kv:
        _need(k_pages is not None and v_pages is not None and block_table is not None, "qk_norm_rope: no cache given")
        _i32(block_table)
        num_pages, nkv, page_size, hd = _cache_geometry(k_pages, v_pages, "qk_norm_rope")
        _need((nkv, hd) == (num_kv_heads, head_dim), "qk_norm_rope: cache pages do not fit the heads")
        _need(k_pages.dtype == qkv_dtype and v_pages.dtype == qkv_dtype, "qk_norm_rope: cache dtype differs")
        width = block_table.shape[1]
    _check(library().rv_qk_norm_rope_kv_write(
        _stream(), qptr, _c_int(slices), _c_ll(stride), _ptr(q_out), _ptr(q_weight), _ptr(k_weight), _c_int(w_f32),
        _c_float(eps),
        _c_float(offset), _ptr(rope_cos), _ptr(rope_sin), _c_int(rotary_dim if rope is not None else 0), _ptr(positions),
        _ptr(token_req), _ptr(block_table), _c_int(width), _ptr(k_pages), _ptr(v_pages), _c_int(page_size),
        _c_int(num_pages), _dt(q_out), _c_int(n), _c_int(num_q_heads), _c_int(num_kv_heads), _c_int(head_dim),
        _c_int((2 if by_page else 1) if write_kv else 0),
        _ptr(values_by_page.q_start if by_page else None), _ptr(values_by_page.chunk_start if by_page else None),
        _c_int(values_by_page.num_requests if by_page else 0), _c_int(values_by_page.max_portion if by_page else 0)))
    return q_out


# Portions of at least this many tokens have their values written a page at a time.
VALUES_BY_PAGE_MIN_PORTION = 16


def paged_attention_generic(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                            positions: torch.Tensor, token_req: torch.Tensor, out: torch.Tensor, num_q_heads: int,
                            scale: float, window: Optional[int]) -> torch.Tensor:
    _gpu(q, k_pages, v_pages, block_table, positions, token_req, out)
    _i32(block_table, positions, token_req)
    n = q.shape[0]
    num_pages, nkv, page_size, hd = _cache_geometry(k_pages, v_pages, "attention")
    _need(q.shape == (n, num_q_heads * hd), f"attention: q is {tuple(q.shape)}, expected {(n, num_q_heads * hd)}")
    _need(out.shape == q.shape and out.dtype == q.dtype, "attention: out must match q")
    _need(k_pages.dtype == q.dtype and v_pages.dtype == q.dtype, "attention: cache must match q")
    _need(positions.numel() >= n and token_req.numel() >= n, "attention: positions/token_req too short")
    _check(library().rv_paged_attention_generic(
        _stream(), _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table), _c_int(block_table.shape[1]),
        _ptr(positions), _ptr(token_req), _ptr(out), _dt(q), _c_int(n), _c_int(num_q_heads), _c_int(nkv), _c_int(hd),
        _c_int(page_size), _c_int(num_pages), _c_int(window or 0), _c_float(scale)))
    return out


def paged_attention(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor, step,
                    out: torch.Tensor, num_q_heads: int, scale: float, window: Optional[int]) -> torch.Tensor:
    """Attention of the step's tokens over the cache; picks the kernel.

    The 32-bit path always runs the generic kernel.  bf16 runs the
    matrix-core kernel where it covers the head size and grouping, else the
    generic one."""
    if q.dtype == torch.bfloat16 and mfma_attention_covers(k_pages, v_pages, num_q_heads):
        return paged_attention_mfma(q, k_pages, v_pages, block_table, step, out, num_q_heads, scale, window)
    return paged_attention_generic(q, k_pages, v_pages, block_table, step.positions, step.token_req, out,
                                   num_q_heads, scale, window)


MFMA_ATTENTION_MAX_HEAD_DIM = 256
MFMA_ATTENTION_MAX_GROUP = 16
# What the split plan of the decode kernel knows about the machine (measured on MI355X at head sizes 64, 128 and
# 256; microseconds): how many of the kernel's waves the machine holds at once is the library's answer for the
# head size at hand (what the kernel's registers allow: one wave a SIMD, 1024 in all, at head size 256; two at
# 128; four at 64); a wave that waits for nobody takes about 1 + head size / 100 for a block of 32 keys (3.6 at
# 256, 2.3 at 128); the waves together stream about 6.3 TB/s; launches and the first reads cost about 7, and the
# merge 0.1 more per split.
_ATTN_WAVE_SLOTS_FALLBACK = 1024
_ATTN_BLOCK_US = (1.0, 0.01)  # a + b * head size
_ATTN_BYTES_PER_US = 6.3e6
_ATTN_FIXED_US = 7.0
_ATTN_FIXED_UNSPLIT_US = 7.0
_ATTN_MERGE_US_PER_SPLIT = 0.1


@functools.lru_cache(maxsize=None)
def attention_wave_slots(head_dim: int) -> int:
    """How many waves of the matrix-core decode kernel for this head size the GPU holds at once."""
    entry = getattr(library(), f"rv_attn_mfma_wave_slots_g{(head_dim // 16 - 1) // 4}", None)
    slots = entry(_c_int(head_dim)) if entry is not None else -1
    return slots if slots > 0 else _ATTN_WAVE_SLOTS_FALLBACK


def mfma_attention_covers(k_pages: torch.Tensor, v_pages: torch.Tensor, num_q_heads: int) -> bool:
    _, nkv, page_size, hd = k_pages.shape
    return (hd % 16 == 0 and hd <= MFMA_ATTENTION_MAX_HEAD_DIM and page_size % 16 == 0
            and num_q_heads % nkv == 0 and num_q_heads // nkv <= MFMA_ATTENTION_MAX_GROUP)


@functools.lru_cache(maxsize=4096)
def plan_attention_splits(num_requests: int, max_portion: int, max_context: int, nkv: int, group: int,
                          window: Optional[int], head_dim: int = 256,
                          wave_slots: int = _ATTN_WAVE_SLOTS_FALLBACK) -> tuple[int, int, int]:
    """(tiles per request, number of key splits, keys per split) for the
    matrix-core decode kernel.  A tile is 16 / group_pad tokens of one request
    and one key/value head; its keys are split over waves.

    The number of splits is the one a small model of the machine likes best:
    the waves run in rounds of ``wave_slots`` (``attention_wave_slots``: as
    many as the machine holds at once); a round takes what its longest wave
    takes alone or what its bytes take at full streaming rate, whichever is
    longer; a last round that is not full still takes a wave's whole time,
    which is why 1.3 rounds are worse than 1 or 2; every split adds to the
    merge."""
    group_pad = 1
    while group_pad < group:
        group_pad *= 2
    tokens_per_tile = 16 // group_pad
    tiles = -(-max_portion // tokens_per_tile)
    span = max_context
    if window:
        # first key of a tile rounded down to 32, up to the tile's last token
        span = min(span, window - 1 + 31 + tokens_per_tile)
    blocks = -(-span // 32)
    units = num_requests * tiles * nkv
    block_bytes = 32 * head_dim * 2 * 2  # keys and values of a block, bf16
    block_us = _ATTN_BLOCK_US[0] + _ATTN_BLOCK_US[1] * head_dim
    best = None
    for splits in range(1, min(blocks, 512) + 1):
        per = -(-blocks // splits)  # blocks a split
        if per * (splits - 1) >= blocks:
            continue  # the last split would be empty: the same plan as with fewer splits
        waves = units * splits
        full_rounds, rest = divmod(waves, wave_slots)
        alone = per * block_us
        time = full_rounds * max(alone, wave_slots * per * block_bytes / _ATTN_BYTES_PER_US)
        if rest:  # fewer waves draw less than the full rate: about its square root of their share
            rate = _ATTN_BYTES_PER_US * (rest / wave_slots) ** 0.5
            time += max(alone, rest * per * block_bytes / rate)
        time += _ATTN_FIXED_US + _ATTN_MERGE_US_PER_SPLIT * splits if splits > 1 else _ATTN_FIXED_UNSPLIT_US
        if best is None or time < best[0] * (1.0 - 1e-9):
            best = (time, splits, per * 32)
    _, splits, split_len = best
    return tiles, splits, split_len


# The kernel that gives a tile's key splits to the eight waves of one block and merges them there, with no second
# kernel: worth it while a wave walks few blocks of keys (a window, a short context), and possible while the
# tile's columns fit the block's LDS.
_ATTN_IN_BLOCK_WAVES = 8
_ATTN_IN_BLOCK_LDS = 64 * 1024
_ATTN_IN_BLOCK_MAX_KEY_BLOCKS = 6
_ATTN_IN_BLOCK_MIN_TILES = 256


def plan_attention_in_block(max_portion: int, max_context: int, group: int, window: Optional[int],
                            head_dim: int, num_tiles: Optional[int] = None) -> Optional[tuple[int, int]]:
    """(keys per split, columns of a tile kept in LDS) if the decode kernel is
    to merge a tile's splits inside its block, else None.  With ``num_tiles``
    (requests x tiles x key/value heads) the answer is also None while the
    tiles are too few to fill the machine eight waves each: then the keys
    are better split further, over more waves than a block has."""
    if num_tiles is not None and num_tiles < _ATTN_IN_BLOCK_MIN_TILES:
        return None
    group_pad = 1
    while group_pad < group:
        group_pad *= 2
    tokens_per_tile = 16 // group_pad
    cols = min(max_portion, tokens_per_tile) * group
    if _ATTN_IN_BLOCK_WAVES * cols * (head_dim + 2) * 4 > _ATTN_IN_BLOCK_LDS:
        return None
    span = max_context
    if window:
        span = min(span, window - 1 + 31 + tokens_per_tile)
    per = -(-(-(-span // 32)) // _ATTN_IN_BLOCK_WAVES)  # blocks of 32 keys a wave
    if per > _ATTN_IN_BLOCK_MAX_KEY_BLOCKS:
        return None
    return per * 32, cols


# Portions of at least this many tokens go to the kernel whose blocks share key
# tiles through LDS; shorter ones (decoded tokens above all) to the kernel that
# splits a request's keys over many waves.
PREFILL_MIN_PORTION = 16


# The prompt kernel's long tiles in pieces (``plan_prefill_pieces``), as measured on MI355X (microseconds): a
# block walks a block of 64 keys in 0.85 + head size / 400 (1.5 at 256) and has a fixed cost of some nine such
# blocks (its queries and table read, the first keys waited for, its sums written); merging costs a launch and
# the pieces' sums written and read again.  Pieces are taken where they shorten the launch by a tenth at least.
_PREFILL_BLOCK_US = (0.85, 1.0 / 400.0)
_PREFILL_PIECE_FIXED = 9.0
_PREFILL_MERGE_US = 6.0
_PREFILL_BYTES_PER_US = 5.0e6
_PREFILL_PIECES_GAIN = 1.1
_PREFILL_PIECES_MOST = 32
_PREFILL_PIECE_LEAST = 2  # blocks of keys
_PREFILL_CUT_BELOW = 4    # tiles are cut only while they are fewer than a quarter of the blocks the machine holds


@functools.lru_cache(maxsize=None)
def attention_prefill_block_slots(head_dim: int) -> int:
    """How many blocks of the prompt attention kernel for this head size the GPU holds at once."""
    entry = getattr(library(), f"rv_attn_prefill_block_slots_g{(head_dim // 16 - 1) // 4}", None)
    slots = entry(_c_int(head_dim)) if entry is not None else -1
    return slots if slots > 0 else 256


def plan_prefill_pieces(lengths, starts, tokens_per_tile: int, window: Optional[int], portion_min: int,
                        head_dim: int, nkv: int, block_slots: int = 256) -> tuple[int, int]:
    """(blocks of 64 keys a piece at most, pieces a tile at most) for the prompt kernel in this step; (any, 1)
    means a tile a block.  ``lengths`` and ``starts``: the portions' tokens and first positions;
    ``block_slots``: the kernel's blocks that the machine holds at once.

    A tile (``tokens_per_tile`` tokens of a portion) walks the keys its tokens see in blocks of 64.  While the
    blocks all fit the machine at once, a launch lasts as long as its longest block; beyond, as the blocks'
    work spread over the machine and half a longest block for the uneven end.  Cutting the long tiles shortens
    the longest block, adds blocks with their fixed cost and the merge: it pays where few tiles walk many keys
    (a portion of a hundred tokens deep in a long context: 16 blocks for 256 CUs), not where the tiles fill
    the machine already (a prompt of 2 048 tokens in one portion is as many tiles as there are CUs, and cut
    tiles would wait for a second turn).  The cut that makes the launch shortest by this count is taken."""
    import numpy as np

    whole = (1 << 20, 1)
    lengths = np.asarray(lengths, dtype=np.int64)
    starts = np.asarray(starts, dtype=np.int64)
    taken = lengths >= portion_min
    if not taken.any():
        return whole
    lengths, starts = lengths[taken], starts[taken]
    tiles = -(-lengths // tokens_per_tile)
    of = np.repeat(np.arange(len(lengths)), tiles)  # the request of every tile
    first = np.zeros(len(lengths), dtype=np.int64)
    np.cumsum(tiles[:-1], out=first[1:])
    tok0 = (np.arange(int(tiles.sum())) - first[of]) * tokens_per_tile
    ntok = np.minimum(tokens_per_tile, lengths[of] - tok0)
    p_first = starts[of] + tok0
    kmin = np.maximum(0, p_first - window + 1) if window else np.zeros_like(p_first)
    cost = -(-(p_first + ntok - (kmin & ~31)) // 64)
    total, longest = int(cost.sum()), int(cost.max())
    block_us = _PREFILL_BLOCK_US[0] + _PREFILL_BLOCK_US[1] * head_dim
    if len(cost) * nkv * _PREFILL_CUT_BELOW > block_slots:
        return whole  # measured: where the tiles fill a quarter of the machine or more, pieces gain little or lose

    def launch(piece_max):
        pieces = -(-cost // piece_max)
        blocks = int(pieces.sum()) * nkv
        long_one = -(-longest // -(-longest // piece_max)) + _PREFILL_PIECE_FIXED  # the longest tile's pieces are equal
        if blocks <= block_slots:
            time = long_one * block_us
        else:
            time = ((total * nkv + blocks * _PREFILL_PIECE_FIXED) / block_slots + 0.5 * long_one) * block_us
        cut = int(pieces[pieces > 1].sum())
        if cut:
            time += _PREFILL_MERGE_US + cut * nkv * 2 * 64 * head_dim * 4 / _PREFILL_BYTES_PER_US
        return time

    best = (launch(longest), longest, 1)
    for pieces in range(2, _PREFILL_PIECES_MOST + 1):
        piece_max = -(-longest // pieces)
        if piece_max < _PREFILL_PIECE_LEAST:
            break
        time = launch(piece_max)
        if time < best[0]:
            best = (time, piece_max, -(-longest // piece_max))
    if best[2] > 1 and launch(longest) >= _PREFILL_PIECES_GAIN * best[0]:
        return best[1], best[2]
    return whole


def _prefill_pieces(step, window, tokens_per_tile, tiles, portion_min, hd, nkv, device, forced):
    """(piece_max, pieces_max, room for the pieces' sums) for the prompt kernel in this step; made once a step
    for the layers that agree in window and sizes (``step.shared``).  ``forced``: (piece_max, pieces_max)."""
    shared = getattr(step, "shared", None)
    key = ("prefill_pieces", window, tokens_per_tile, tiles, portion_min, hd, nkv, forced)
    if shared is not None and key in shared:
        return shared[key]
    piece_max, pieces_max = 1 << 20, 1
    if forced is not None:
        piece_max, pieces_max = forced
    else:
        starts = getattr(step, "host_q_start", None)
        first = getattr(step, "host_chunk_start", None)
        if starts is not None and first is not None:
            lengths = [int(starts[i + 1] - starts[i]) for i in range(step.num_requests)]
            piece_max, pieces_max = plan_prefill_pieces(lengths, first, tokens_per_tile, window, portion_min, hd, nkv,
                                                        attention_prefill_block_slots(hd))
    part = None
    if pieces_max > 1:
        part = torch.empty(step.num_requests * tiles * nkv * pieces_max * (64 * hd + 128), dtype=torch.float32,
                           device=device)
    result = (int(piece_max), int(pieces_max), part)
    if shared is not None:
        shared[key] = result
    return result


def paged_attention_mfma(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                         step, out: torch.Tensor, num_q_heads: int, scale: float, window: Optional[int],
                         splits: Optional[tuple[int, int]] = None, prefill_kernel: Optional[bool] = None,
                         in_block: Optional[bool] = None,
                         prefill_pieces: Optional[tuple[int, int]] = None) -> torch.Tensor:
    """bf16 attention on the matrix cores.  ``splits`` = (number, keys per
    split) overrides the plan, ``prefill_kernel`` the choice of kernel,
    ``in_block`` whether a tile's splits are merged inside one block and
    ``prefill_pieces`` = (blocks of 64 keys a piece at most, pieces a tile at
    most) how the prompt kernel cuts its long tiles (tests use them to force
    every path)."""
    _gpu(q, k_pages, v_pages, block_table, out)
    _i32(block_table)
    n = q.shape[0]
    num_pages, nkv, page_size, hd = _cache_geometry(k_pages, v_pages, "attention")
    _need(q.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16,
          "attention (matrix cores): bfloat16 only")
    _need(mfma_attention_covers(k_pages, v_pages, num_q_heads),
          f"attention (matrix cores): head_dim {hd} must be a multiple of 16 up to {MFMA_ATTENTION_MAX_HEAD_DIM}, "
          f"at most {MFMA_ATTENTION_MAX_GROUP} query heads per key/value head, pages a multiple of 16")
    _need(q.shape == (n, num_q_heads * hd) and out.shape == q.shape and out.dtype == q.dtype,
          "attention (matrix cores): bad q or out shape")
    _need(n == step.num_tokens, "attention (matrix cores): q must hold the step's tokens")
    group = num_q_heads // nkv
    group_pad = 1
    while group_pad < group:
        group_pad *= 2
    lib = library()
    suffix = f"g{(hd // 16 - 1) // 4}"

    # which requests go to which kernel
    longest = step.max_portion
    if prefill_kernel is None:
        use_prefill = longest >= PREFILL_MIN_PORTION
        portion_min = PREFILL_MIN_PORTION
    else:
        use_prefill, portion_min = prefill_kernel, 1
    shortest_rest = 0  # longest portion left to the split-key kernel
    if use_prefill and portion_min > 1:
        starts = getattr(step, "host_q_start", None)
        if starts is None:
            starts = step.q_start.cpu().numpy()
        lengths = [int(starts[i + 1] - starts[i]) for i in range(step.num_requests)]
        shortest_rest = max([x for x in lengths if x < portion_min], default=0)
    elif not use_prefill:
        shortest_rest = longest

    if use_prefill:
        tokens_per_block = 64 // group_pad
        tiles = -(-longest // tokens_per_block)
        piece_max, pieces_max, part = _prefill_pieces(step, window, tokens_per_block, tiles, portion_min, hd, nkv,
                                                      q.device, prefill_pieces)
        entry = getattr(lib, f"rv_attn_prefill_{suffix}")
        _check(entry(_stream(), _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
                     _c_int(block_table.shape[1]), _ptr(step.q_start), _ptr(step.chunk_start), _ptr(out), _c_int(n),
                     _c_int(step.num_requests), _c_int(tiles), _c_int(num_q_heads), _c_int(nkv), _c_int(hd),
                     _c_int(page_size), _c_int(num_pages), _c_int(window or 0), _c_int(portion_min), _c_float(scale),
                     _c_int(piece_max), _c_int(pieces_max), _ptr(part)))
    if shortest_rest > 0:
        tiles, num_splits, split_len = plan_attention_splits(step.num_requests, shortest_rest, step.max_context, nkv,
                                                             group, window, hd, attention_wave_slots(hd))
        block_cols = 0
        merged = None
        if in_block is not False:
            merged = plan_attention_in_block(shortest_rest, step.max_context, group, window, hd,
                                             None if in_block else step.num_requests * tiles * nkv)
        if in_block:
            _need(merged is not None, "attention: these keys or columns are too many to merge inside a block")
        if merged is not None and (splits is None or in_block):
            num_splits, (split_len, block_cols) = _ATTN_IN_BLOCK_WAVES, merged
        elif splits is not None:
            num_splits, split_len = splits
            need = -(-step.max_context // 32) * 32
            _need(window is not None or num_splits * split_len >= need,
                  "attention: the splits do not cover the context")
        part_o = part_ml = None
        if num_splits > 1 and block_cols == 0:
            units = step.num_requests * tiles * nkv * num_splits
            part_o = torch.empty(units * 16 * hd, dtype=torch.float32, device=q.device)
            part_ml = torch.empty(units * 32, dtype=torch.float32, device=q.device)
        entry = getattr(lib, f"rv_attn_mfma_{suffix}")
        _check(entry(_stream(), _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
                     _c_int(block_table.shape[1]), _ptr(step.q_start), _ptr(step.chunk_start), _ptr(step.token_req),
                     _ptr(out), _ptr(part_o), _ptr(part_ml), _c_int(n), _c_int(step.num_requests), _c_int(tiles),
                     _c_int(num_q_heads), _c_int(nkv), _c_int(hd), _c_int(page_size), _c_int(num_pages),
                     _c_int(window or 0), _c_int(num_splits), _c_int(split_len),
                     _c_int(portion_min - 1 if use_prefill else 0), _c_int(block_cols), _c_float(scale)))
    return out


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _gpu(logits, out)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "argmax: float32 [rows, vocab] expected")
    rows, vocab = logits.shape
    if out is None:
        out = torch.empty(rows, dtype=torch.int32, device=logits.device)
    parts = library().rv_argmax_parts(_c_int(vocab))
    ws_val = torch.empty(rows * parts, dtype=torch.float32, device=logits.device)
    ws_idx = torch.empty(rows * parts, dtype=torch.int32, device=logits.device)
    _check(library().rv_argmax(_stream(), _ptr(logits), _c_int(rows), _c_int(vocab), _c_ll(vocab), _ptr(ws_val),
                               _ptr(ws_idx), _ptr(out)))
    return out


def advance_decode(step, chosen: torch.Tensor) -> None:
    """A step of decoded tokens becomes the next one on the device: request b's
    next token is ``chosen[b]``, one position on.  ``step`` is the step's batch
    (token b belongs to request b); its arrays are changed in place."""
    n = step.num_requests
    _need(step.num_tokens == n and step.max_portion == 1, "advance_decode: a step of single decoded tokens expected")
    _gpu(chosen, step.token_ids, step.positions, step.chunk_start, step.context_len)
    _i32(chosen, step.token_ids, step.positions, step.chunk_start, step.context_len)
    _need(chosen.numel() == n, "advance_decode: one chosen token per request expected")
    _check(library().rv_advance_decode(_stream(), _ptr(chosen), _ptr(step.token_ids), _ptr(step.positions),
                                       _ptr(step.chunk_start), _ptr(step.context_len), _c_int(n)))


def copy_rows_to_device(dst: torch.Tensor, src: torch.Tensor, rows: int, cols: int) -> None:
    """``dst[:rows, :cols] = src[:rows, :cols]`` from a pinned host matrix to a device matrix of the same element
    size as one strided copy in the current stream's order (rows far apart, as a step's block tables are: only
    the pages that the step's requests hold travel)."""
    _gpu(dst)
    _need(not src.is_cuda and src.is_pinned(), "copy_rows: the source must be pinned host memory")
    _need(dst.dim() == 2 and src.dim() == 2 and dst.element_size() == src.element_size()
          and dst.stride(1) == 1 and src.stride(1) == 1, "copy_rows: two matrices with rows of the same elements expected")
    _need(0 <= rows <= min(dst.shape[0], src.shape[0]) and 0 <= cols <= min(dst.shape[1], src.shape[1]),
          f"copy_rows: {rows} x {cols} does not fit {tuple(src.shape)} -> {tuple(dst.shape)}")
    e = dst.element_size()
    _check(library().rv_copy_rows_to_device(_stream(), _ptr(dst), _c_ll(dst.stride(0) * e), _ptr(src),
                                            _c_ll(src.stride(0) * e), _c_ll(cols * e), _c_ll(rows)))


def topk_select(logits: torch.Tensor, k: int, inv_temp: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """The k largest logits of every row, times 1/T, with their ids (unordered)."""
    _gpu(logits, inv_temp)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "topk_select: float32 [rows, vocab] expected")
    rows, vocab = logits.shape
    _need(inv_temp.dtype == torch.float32 and inv_temp.numel() == rows, "topk_select: one 1/T per row expected")
    vals = torch.empty((rows, k), dtype=torch.float32, device=logits.device)
    idx = torch.empty((rows, k), dtype=torch.int32, device=logits.device)
    parts = library().rv_topk_parts(_c_int(vocab))
    cand_val = cand_idx = None
    if parts > 1:  # the parts' candidates, from which the row's are selected
        cand_val = torch.empty((rows, parts * k), dtype=torch.float32, device=logits.device)
        cand_idx = torch.empty((rows, parts * k), dtype=torch.int32, device=logits.device)
    _check(library().rv_topk_select(_stream(), _ptr(logits), _c_int(rows), _c_int(vocab), _c_ll(vocab), _c_int(k),
                                    _ptr(inv_temp), _ptr(vals), _ptr(idx), _ptr(cand_val), _ptr(cand_idx)))
    return vals, idx


def draw(vals: torch.Tensor, ids: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor, rng_state: torch.Tensor,
         out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token a row from the candidates ``vals, ids [rows, k]`` of ``topk_select``, drawn on the device as the
    host draws (``sampling.sampler.sample_rows``): ``top_k`` int32 and ``top_p`` float64 a row, ``rng_state`` int64
    a row, each request's SplitMix64 state, which moves one draw on.  -1 for a row one of whose own ``top_k``
    candidates is no finite number.  A row with ``top_k`` -1 draws nothing: it gets the largest candidate that is
    a number, the lower id among equals, as ``argmax`` gives it."""
    _gpu(vals, ids, top_k, top_p, rng_state, out)
    rows, k = vals.shape
    _need(vals.dtype == torch.float32 and ids.dtype == torch.int32 and ids.shape == vals.shape,
          "draw: float32 values and int32 ids [rows, k] expected")
    _need(top_k.dtype == torch.int32 and top_p.dtype == torch.float64 and rng_state.dtype == torch.int64
          and top_k.numel() == rows and top_p.numel() == rows and rng_state.numel() == rows,
          "draw: top_k int32, top_p float64 and rng_state int64, one a row, expected")
    if out is None:
        out = torch.empty(rows, dtype=torch.int32, device=vals.device)
    _need(out.dtype == torch.int32 and out.numel() == rows, "draw: int32 out, one a row, expected")
    _check(library().rv_draw(_stream(), _ptr(vals), _ptr(ids), _c_int(rows), _c_int(k), _ptr(top_k), _ptr(top_p),
                             _ptr(rng_state), _ptr(out)))
    return out


def gemm_bf16(x: torch.Tensor, w, out: Optional[torch.Tensor] = None,
              out_dtype: Optional[torch.dtype] = None, sliced_ok: bool = False):
    """out = x @ w^T on the matrix cores for bf16 inputs; None when no
    hand-written kernel covers the shape (the caller then uses another path).
    ``w`` is a matrix ``[N, K]`` or a ``TiledWeight``.

    Products with up to 64 rows run the kernel that is built around reading
    ``w`` once.  A 32-bit result of more rows (logits at many positions) runs
    it over blocks of 64 rows; a bf16 result of more rows is left to the
    library product.  With ``sliced_ok`` a product whose K range is split over
    blocks returns its partial sums as ``SlicedSums`` instead of adding them."""
    m, k = x.shape
    tiled = isinstance(w, TiledWeight)
    n = w.shape[0]
    out_dtype = out.dtype if out is not None else (out_dtype or x.dtype)
    if k % 8 or x.stride(1) != 1 or (out is not None and out.stride(1) != 1):
        return None
    if (m > 1 and x.stride(0) % 8) or x.data_ptr() % 16:
        return None
    if not tiled and (w.stride(1) != 1 or (n > 1 and w.stride(0) % 8) or w.data_ptr() % 16):
        return None
    if m > SKINNY_MAX_ROWS and out_dtype != torch.float32:
        return None
    _need(x.is_cuda and w.device.type == "cuda", "gemm: arguments must live on the GPU")
    _need(w.shape[1] == k and (out is None or out.shape == (m, n)), "gemm: shapes do not fit")
    lib = library()
    ldx = x.stride(0) if m > 1 else k
    ldw = 0 if tiled else (w.stride(0) if n > 1 else k)
    wptr = _ptr(w.tiles if tiled else w)
    slices = lib.rv_gemm_skinny_slices(_c_int(n), _c_int(k))
    if sliced_ok and out is None and slices > 1 and m <= SKINNY_MAX_ROWS:
        part = torch.empty((slices, m, n), dtype=torch.float32, device=x.device)
        _check(lib.rv_gemm_skinny(_stream(), _ptr(x), wptr, None, _dt(x), _ptr(part), _c_int(m), _c_int(n),
                                  _c_int(k), _c_ll(ldx), _c_ll(ldw), _c_ll(n), _c_int(0), _c_int(int(tiled))))
        return SlicedSums(part, out_dtype)
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    ldc = out.stride(0) if m > 1 else n
    rows_max = min(m, SKINNY_MAX_ROWS)
    part = torch.empty(slices * rows_max * n, dtype=torch.float32, device=x.device) if slices > 1 else None
    for m0 in range(0, m, SKINNY_MAX_ROWS):
        rows = min(SKINNY_MAX_ROWS, m - m0)
        _check(lib.rv_gemm_skinny(_stream(), ctypes.c_void_p(x.data_ptr() + m0 * ldx * 2), wptr,
                                  ctypes.c_void_p(out.data_ptr() + m0 * ldc * out.element_size()), _dt(out),
                                  _ptr(part), _c_int(rows), _c_int(n), _c_int(k), _c_ll(ldx), _c_ll(ldw),
                                  _c_ll(ldc), _c_int(1), _c_int(int(tiled))))
    return out


SKINNY_MAX_ROWS = 64

# ---- products of many rows: the library's --------------------------------------------------------------------
LIBRARY_WORKSPACE_BYTES = 64 << 20
_library_workspaces: dict = {}
_library_tuning = False


def library_workspace(device) -> torch.Tensor:
    """The device memory that the library's algorithms may use, one allocation a device, made at first use."""
    device = torch.device(device)
    index = torch.cuda.current_device() if device.index is None else device.index
    ws = _library_workspaces.get(index)
    if ws is None:
        ws = _library_workspaces[index] = torch.empty(LIBRARY_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return ws


def set_library_tuning(on: bool) -> None:
    """While on, ``library_gemm`` first times the library's algorithms for every shape it has not tuned yet and
    keeps the fastest (a second or so a shape, with a wait for the device): for warm-up runs, never inside a
    recording."""
    global _library_tuning
    _library_tuning = bool(on)


def _library_args(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor):
    m, k = x.shape
    n = w.shape[0]
    bf16 = torch.bfloat16
    out_f32 = out.dtype is torch.float32
    if not (x.is_cuda and w.is_cuda and out.is_cuda and x.dtype is bf16 and w.dtype is bf16
            and (out.dtype is bf16 or out_f32)
            and w.dim() == 2 and w.shape[1] == k and out.dim() == 2 and out.shape[0] == m and out.shape[1] == n
            and x.stride(1) == 1 and w.stride(1) == 1 and out.stride(1) == 1):
        _need(x.is_cuda and w.is_cuda and out.is_cuda, "library product: arguments must live on the GPU")
        _need(x.dtype == bf16 and w.dtype == bf16 and out.dtype in (bf16, torch.float32),
              "library product: bfloat16 operands, a bfloat16 or float32 result")
        _need(w.dim() == 2 and out.dim() == 2 and w.shape[1] == k and tuple(out.shape) == (m, n),
              f"library product: shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
        _need(False, "library product: rows must be contiguous")
    ws = _library_workspaces.get(x.device.index)
    if ws is None:
        ws = library_workspace(x.device)
    return (x.data_ptr(), w.data_ptr(), out.data_ptr(), m, n, k, x.stride(0) if m > 1 else k,
            w.stride(0) if n > 1 else k, out.stride(0) if m > 1 else n, ws.data_ptr(), LIBRARY_WORKSPACE_BYTES), int(out_f32)


# The matrices that products of many rows may meet, by shape: tuning a shape takes them in turn (``rv_lt_tune``), so
# that its timed calls read from memory as a step's calls do.  Weak references: a model that goes takes its own along.
_library_matrices: dict = {}


def library_matrix_register(w: torch.Tensor) -> None:
    """Tells the tuning of the library's products that ``w`` ([N, K], bf16, on the GPU) is one of the matrices of
    its shape: a part calls it for every matrix it keeps row by row."""
    import weakref

    if w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2 and w.stride(1) == 1:
        key = (w.device.index, w.shape[0], w.shape[1], w.stride(0))
        known = _library_matrices.setdefault(key, [])
        if len(known) >= 1024:  # models come and go: forget the ones that went
            known[:] = [ref for ref in known if ref() is not None]
        known.append(weakref.ref(w))


def _library_matrices_like(w: torch.Tensor):
    """(a C array of the addresses of the registered matrices of ``w``'s shape that are still there, their number);
    (None, 0) if there is none but ``w`` itself."""
    key = (w.device.index, w.shape[0], w.shape[1], w.stride(0))
    alive = [t for t in (ref() for ref in _library_matrices.get(key, ())) if t is not None]
    _library_matrices[key] = [ref for ref in _library_matrices.get(key, ()) if ref() is not None]
    addresses = sorted({t.data_ptr() for t in alive} | {w.data_ptr()})
    if len(addresses) < 2:
        return None, 0
    return (ctypes.c_void_p * len(addresses))(*addresses), len(addresses)


def library_gemm(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> Optional[torch.Tensor]:
    """out[M, N] = x[M, K] @ w[N, K]^T, x and w in bf16, out in bf16 or (logits) float32, with 32-bit sums, by
    hipBLASLt (``csrc/library_gemm.hip``): the product of more rows than the few-row kernel takes.  A shape keeps its plan; see ``set_library_tuning``.
    None, with nothing done, for a shape that the library has no algorithm for."""
    args, out_f32 = _library_args(x, w, out)
    lib = library()
    if _library_tuning:
        others, count = _library_matrices_like(w)
        _check(min(0, lib.rv_lt_tune(_stream(), *args, _c_int(LIBRARY_TUNE_BUDGET_MS), others, _c_int(count), out_f32)))
    status = lib.rv_lt_gemm(_stream(), *args, out_f32)
    if status == 2:  # the library has no algorithm for this shape: nothing ran
        return None
    _check(status)
    return out


LIBRARY_TUNE_BUDGET_MS = 3000
# The environment variable that names a file of tuned plans: ``ModelRunner.warm_up`` reads it before it tunes and
# writes it afterwards, so that a later start finds its shapes tuned.
LIBRARY_PLANS_ENV = "RVLLM_AMD_LIBRARY_PLANS"


def _library_plans_key(device) -> dict:
    """What a file of plans holds for: an algorithm's index means something only to one version of the library on
    one kind of device."""
    kind = ctypes.create_string_buffer(128)
    with torch.cuda.device(device):
        _check(library().rv_lt_device_kind(kind, _c_int(len(kind))))
        return {"device": kind.value.decode(), "hipblaslt": int(library().rv_lt_version())}


def library_plans_save(path: str, device) -> int:
    """Writes the tuned shapes of ``device`` (shape, strides, the algorithm's index, its time, 1 for a 32-bit result) to ``path`` as JSON,
    over what the file held; the number of shapes written."""
    import json
    import os

    lib = library()
    plans = []
    with torch.cuda.device(device):
        while True:
            m, n, k, index, f32 = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
            ldx, ldw, ldc = ctypes.c_longlong(), ctypes.c_longlong(), ctypes.c_longlong()
            us = ctypes.c_float()
            if not lib.rv_lt_tuned_plan(_c_int(len(plans)), ctypes.byref(m), ctypes.byref(n), ctypes.byref(k),
                                        ctypes.byref(ldx), ctypes.byref(ldw), ctypes.byref(ldc), ctypes.byref(index),
                                        ctypes.byref(us), ctypes.byref(f32)):
                break
            plans.append([m.value, n.value, k.value, ldx.value, ldw.value, ldc.value, index.value, round(us.value, 2),
                          f32.value])
        doc = dict(_library_plans_key(device), plans=sorted(plans))
    tmp = f"{path}.{os.getpid()}.tmp"
    with open(tmp, "w") as f:
        json.dump(doc, f, indent=0)
    os.replace(tmp, path)
    return len(plans)


def library_plans_load(path: str, device) -> int:
    """Takes the plans of a file written by ``library_plans_save``: the number of shapes that now count as tuned.
    A file that is missing, unreadable, or of another device or version of the library gives 0 and changes nothing;
    so does a plan that the library does not take."""
    import json

    try:
        with open(path) as f:
            doc = json.load(f)
        plans = [(int(m), int(n), int(k), int(ldx), int(ldw), int(ldc), int(index), float(us), int(f32))
                 for m, n, k, ldx, ldw, ldc, index, us, f32 in doc["plans"]]
    except (OSError, ValueError, KeyError, TypeError):
        return 0
    lib = library()
    taken = 0
    with torch.cuda.device(device):
        if {key: doc.get(key) for key in ("device", "hipblaslt")} != _library_plans_key(device):
            return 0
        room = library_workspace(torch.device(device)).numel()
        for m, n, k, ldx, ldw, ldc, index, us, f32 in plans:
            status = lib.rv_lt_take_plan(_c_int(m), _c_int(n), _c_int(k), _c_ll(ldx), _c_ll(ldw), _c_ll(ldc),
                                         _c_int(index), _c_float(us), _c_ll(room), _c_int(f32))
            if status == 0:
                taken += 1  # anything else: the library does not know the algorithm, or refuses the shape; not taken
    return taken


def library_plan_info(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> tuple[int, int, float]:
    """(1 tuned / 2 a tuned neighbour's algorithm: the nearest row count within one and a half times with the same
    matrix / 0 the library's first suggestion / -1 never seen, the algorithm's index, the time it was tuned to in
    microseconds) for the shape of this product."""
    args, out_f32 = _library_args(x, w, out)
    index, us = ctypes.c_int(-1), ctypes.c_float(0.0)
    state = library().rv_lt_plan_info(*args[3:9], ctypes.byref(index), ctypes.byref(us), out_f32)
    return state, index.value, us.value


def probe_read(data: torch.Tensor, blocks: int = 2048) -> torch.Tensor:
    """Reads ``data`` once with a kernel that does nothing else (a measurement of the memory's read rate);
    returns 64 words folded from what was read."""
    _gpu(data)
    nbytes = data.numel() * data.element_size()
    _need(nbytes % 16 == 0 and data.data_ptr() % 16 == 0, "probe_read: 16-byte aligned data of a multiple of 16 bytes")
    out = torch.zeros(64, dtype=torch.int32, device=data.device)
    _check(library().rv_probe_read(_stream(), _ptr(data), _c_ll(nbytes), _ptr(out), _c_int(blocks)))
    return out


def gemm_bf16_gate_up(x: torch.Tensor, w_fours, activation: str):
    """act(x @ gate^T) * (x @ up^T) in one kernel, for a bf16 ``x`` of at most 64 rows and ``w_fours`` =
    ``rows_in_fours(gate, up)`` (as a matrix or a ``TiledWeight``): the product applies the activation where it
    holds the sums, which saves a kernel and a pass over memory.  None when the kernel does not cover the case
    (rows, alignment, a shape whose product is split along K): the caller then multiplies and applies
    ``gated_act(..., fours=True)``."""
    if x.dtype != torch.bfloat16 or w_fours.dtype != torch.bfloat16:
        return None
    m, k = x.shape
    tiled = isinstance(w_fours, TiledWeight)
    n = w_fours.shape[0]
    if m < 1 or m > SKINNY_MAX_ROWS or w_fours.shape[1] != k or k % 8 or n % 4 or x.stride(1) != 1:
        return None
    if (m > 1 and x.stride(0) % 8) or x.data_ptr() % 16:
        return None
    if not tiled and (w_fours.stride(1) != 1 or (n > 1 and w_fours.stride(0) % 8) or w_fours.data_ptr() % 16):
        return None
    _need(x.is_cuda and w_fours.device.type == "cuda", "gemm: arguments must live on the GPU")
    _need(activation in ACTIVATIONS, f"gemm_bf16_gate_up: unknown activation {activation!r}")
    lib = library()
    if lib.rv_gemm_skinny_slices(_c_int(n), _c_int(k)) != 1:
        return None
    out = torch.empty((m, n // 2), dtype=torch.bfloat16, device=x.device)
    _check(lib.rv_gemm_skinny_gate_up(_stream(), _ptr(x), _ptr(w_fours.tiles if tiled else w_fours), _ptr(out), _dt(out),
                                      _c_int(m), _c_int(n), _c_int(k), _c_ll(x.stride(0) if m > 1 else k),
                                      _c_ll(0 if tiled else (w_fours.stride(0) if n > 1 else k)), _c_ll(n // 2),
                                      _c_int(ACTIVATIONS[activation]), _c_int(int(tiled))))
    return out
