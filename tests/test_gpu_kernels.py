"""Each HIP kernel alone against a plain PyTorch reference of the same
operation, at sizes other than the engine's tiny models: widths and
vocabularies that are no power of two, head sizes in steps of 16, odd head
groupings, pages of every size."""

import math
import types

import pytest
import torch
import torch.nn.functional as F

import plain_gemma as P
from rvllm_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def dev(t, dtype=None):
    return t.to(device=DEV, dtype=dtype or t.dtype).contiguous()


def test_library_is_loaded_from_the_tree():
    assert ops.library() is not None and "librvllm_amd_" in ops.library_path()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,vocab", [(80, 301), (2560, 1000)])
def test_embed_gather(dtype, hidden, vocab):
    g = torch.Generator().manual_seed(1)
    table = torch.randn(vocab, hidden, generator=g).to(dtype)
    ids = torch.tensor([0, vocab - 1, 5, 5, 17], dtype=torch.int32)
    out = torch.empty(5, hidden, dtype=dtype, device=DEV)
    ops.embed_gather(dev(table), dev(ids), math.sqrt(hidden), out)
    want = (table.float()[ids.long()] * math.sqrt(hidden)).to(dtype)
    assert torch.equal(out.cpu(), want)  # one multiplication in 32-bit, one rounding


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [16, 100, 2560, 5376])
@pytest.mark.parametrize("wdtype", DTYPES)
def test_rmsnorm(dtype, width, wdtype):
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(7, width, generator=g) * 3).to(dtype)
    w = (torch.randn(width, generator=g) * 0.1).to(wdtype)
    got = ops.rmsnorm(dev(x), dev(w), 1e-5, 1.0).cpu().float()
    want = P.rmsnorm(x.double(), w.double(), 1e-5).float()
    assert torch.allclose(got, want, **tol(dtype))
    # offset 0: the stored weight is the gain
    got = ops.rmsnorm(dev(x), dev(w), 1e-5, 0.0).cpu().float()
    want = (P.rmsnorm(x.double(), torch.zeros(width).double(), 1e-5) * w.double()).float()
    assert torch.allclose(got, want, **tol(dtype))


def test_rmsnorm_rows_picks_rows():
    x = torch.randn(9, 48)
    w = torch.randn(48) * 0.1
    rows = torch.tensor([8, 0, 3, 3], dtype=torch.int32)
    got = ops.rmsnorm(dev(x), dev(w), 1e-6, 1.0, rows=dev(rows)).cpu()
    assert torch.allclose(got, P.rmsnorm(x[rows.long()], w, 1e-6), atol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [96, 2560])
def test_add_rmsnorm_with_and_without_the_next_norm(dtype, width):
    g = torch.Generator().manual_seed(3)
    branch = (torch.randn(5, width, generator=g) * 2).to(dtype)
    res = torch.randn(5, width, generator=g).to(dtype)
    w1 = (torch.randn(width, generator=g) * 0.1).to(dtype)
    w2 = (torch.randn(width, generator=g) * 0.1).to(dtype)
    want_res = res.double() + P.rmsnorm(branch.double(), w1.double(), 1e-6)
    r = dev(res.clone())
    assert ops.add_rmsnorm(dev(branch), dev(w1), 1e-6, 1.0, r) is None
    assert torch.allclose(r.cpu().float(), want_res.float(), **tol(dtype))
    r2 = dev(res.clone())
    nxt = ops.add_rmsnorm(dev(branch), dev(w1), 1e-6, 1.0, r2, dev(w2), 1e-5, 1.0)
    assert torch.equal(r2, r)
    # the next norm reads the residual as stored
    want_next = P.rmsnorm(r.cpu().double(), w2.double(), 1e-5)
    assert torch.allclose(nxt.cpu().float(), want_next.float(), **tol(dtype))


@pytest.mark.parametrize("width", [96, 1000, 2560, 3072, 5376])
@pytest.mark.parametrize("with_next", [True, False])
def test_add_rmsnorm_of_many_rows(width, with_next):
    """From some hundred rows on a wave takes a whole row (widths up to 3072; wider rows stay with the kernel
    that gives a row to a block): a width that leaves most lanes without values, one that ends inside a turn
    of the wave, whole turns, and rows that do not fill the last block."""
    rows = 301
    g = torch.Generator().manual_seed(33)
    branch = (torch.randn(rows, width, generator=g) * 2).bfloat16()
    res = torch.randn(rows, width, generator=g).bfloat16()
    w1 = (torch.randn(width, generator=g) * 0.1).bfloat16()
    w2 = (torch.randn(width, generator=g) * 0.1).bfloat16()
    r = dev(res.clone())
    nxt = ops.add_rmsnorm(dev(branch), dev(w1), 1e-6, 1.0, r, *((dev(w2), 1e-5, 1.0) if with_next else ()))
    want_res = (res.double() + P.rmsnorm(branch.double(), w1.double(), 1e-6)).bfloat16()
    assert torch.allclose(r.cpu().float(), want_res.float(), **tol(torch.bfloat16))
    # a few rows at a time take the other kernel: the same values up to the order of a row's sum of squares
    few = dev(res[:7].clone())
    few_next = ops.add_rmsnorm(dev(branch[:7]), dev(w1), 1e-6, 1.0, few, *((dev(w2), 1e-5, 1.0) if with_next else ()))
    assert torch.allclose(few.float(), r[:7].float(), rtol=1e-2, atol=1e-2)
    if with_next:
        want_next = P.rmsnorm(r.cpu().double(), w2.double(), 1e-5)  # of the residual as stored
        assert torch.allclose(nxt.cpu().float(), want_next.float(), **tol(torch.bfloat16))
        assert torch.allclose(few_next.float(), nxt[:7].float(), rtol=1e-2, atol=1e-2)
    else:
        assert nxt is None


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_act(dtype):
    g = torch.Generator().manual_seed(4)
    gu = (torch.randn(6, 2 * 173, generator=g) * 2).to(dtype)
    got = ops.gated_act(dev(gu), "gelu_pytorch_tanh").cpu().float()
    want = F.gelu(gu[:, :173].double(), approximate="tanh") * gu[:, 173:].double()
    assert torch.allclose(got, want.float(), **tol(dtype))
    got = ops.gated_act(dev(gu), "silu").cpu().float()
    want = F.silu(gu[:, :173].double()) * gu[:, 173:].double()
    assert torch.allclose(got, want.float(), **tol(dtype))
    with pytest.raises(ops.KernelError, match="unknown activation"):
        ops.gated_act(dev(gu), "relu")


def test_softcap():
    x = torch.tensor([[1000.0, -1000.0, 0.3, 15.0]])
    got = ops.softcap_(dev(x.clone()), 30.0).cpu()
    assert torch.allclose(got, 30.0 * torch.tanh(x / 30.0), atol=1e-5) and abs(got[0, 0] - 30.0) < 0.01


@pytest.mark.parametrize("m,n,k", [(1, 7, 5), (3, 100, 96), (65, 130, 257), (8, 509, 96), (200, 64, 2560)])
def test_gemm_plain_is_true_32_bit_and_independent_of_rows(m, n, k):
    g = torch.Generator().manual_seed(5)
    a, w = torch.randn(m, k, generator=g), torch.randn(n, k, generator=g)
    out = torch.empty(m, n, device=DEV)
    ops.gemm_plain(dev(a), dev(w), out)
    want = (a.double() @ w.double().T)
    # 32-bit products and sums: the error is that of a chain of k roundings, far below any 16-bit mode
    assert (out.cpu().double() - want).abs().max() <= 1e-6 * math.sqrt(k) * want.abs().max()
    # a row's result does not depend on the rows around it
    one = torch.empty(1, n, device=DEV)
    ops.gemm_plain(dev(a[m - 1:m]), dev(w), one)
    assert torch.equal(one[0], out[m - 1])


def test_gemm_plain_bf16_inputs_give_32_bit_logits():
    g = torch.Generator().manual_seed(6)
    a, w = torch.randn(5, 80, generator=g).bfloat16(), torch.randn(301, 80, generator=g).bfloat16()
    out = torch.empty(5, 301, device=DEV, dtype=torch.float32)
    ops.gemm_plain(dev(a), dev(w), out)
    assert torch.allclose(out.cpu(), a.float() @ w.float().T, atol=1e-4, rtol=1e-5)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (8, 4096, 2560), (17, 509, 96), (64, 2560, 10240), (33, 100, 2048),
                                   (3, 20480, 2560), (16, 7, 8), (200, 301, 80)])
def test_gemm_skinny(m, n, k, out_dtype):
    g = torch.Generator().manual_seed(20)
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    out = torch.full((m, n), float("nan"), dtype=out_dtype, device=DEV)
    got = ops.gemm_bf16(dev(x), dev(w), out)
    if m > 64 and out_dtype == torch.bfloat16:
        assert got is None  # left to the library product
        return
    assert got is out
    want = x.double() @ w.double().T
    err = (out.cpu().double() - want).abs().max().item()
    scale = want.abs().max().item()
    assert err <= (2e-6 if out_dtype == torch.float32 else 5e-3) * scale * max(1.0, math.sqrt(k) / 16)
    # a row gives the same bits alone as in the batch
    one = torch.empty((1, n), dtype=out_dtype, device=DEV)
    ops.gemm_bf16(dev(x[m - 1:m]), dev(w), one)
    assert torch.equal(one[0], out[m - 1])


@pytest.mark.parametrize("m,n,k", [(1, 48, 64), (8, 4096, 2560), (17, 509, 96), (64, 2560, 10240), (33, 100, 2048),
                                   (3, 20480, 2560), (16, 7, 8), (5, 1000, 1416), (200, 301, 80), (40, 35, 40)])
def test_a_matrix_stored_in_tiles_gives_the_bits_of_the_matrix_stored_in_rows(m, n, k):
    """The few-row product reads a matrix either row by row or from tiles of 16 rows x 32 columns laid out in the
    order its lanes hold them; rows and columns that do not fill a tile (n no multiple of 16, k no multiple of
    32) are zeros there.  Every sum is the same chain of the same numbers, so the results are equal bit for bit:
    whole, as unreduced slices, and with the activation in the product."""
    g = torch.Generator().manual_seed(40)
    x = dev(torch.randn(m, k, generator=g).bfloat16())
    w = dev((torch.randn(n, k, generator=g) * 0.05).bfloat16())
    tiled = ops.TiledWeight(w)
    assert tiled.shape == (n, k) and tiled.tiles.numel() == -(-n // 16) * -(-k // 32) * 512
    # the layout itself: tile (i, j), lane (c // 8) * 16 + r, holds w[16 i + r, 32 j + c .. c + 8]
    t = tiled.tiles.view(-(-n // 16), -(-k // 32), 4, 16, 8).cpu()
    padded = torch.zeros(-(-n // 16) * 16, -(-k // 32) * 32, dtype=torch.bfloat16)
    padded[:n, :k] = w.cpu()
    assert torch.equal(t, padded.view(-(-n // 16), 16, -(-k // 32), 4, 8).permute(0, 2, 3, 1, 4))
    for out_dtype in (torch.float32, torch.bfloat16):
        rows = ops.gemm_bf16(x, w, out_dtype=out_dtype)
        tiles = ops.gemm_bf16(x, tiled, out_dtype=out_dtype)
        if m > 64 and out_dtype == torch.bfloat16:
            assert rows is None and tiles is None  # left to the library product, which reads the rows
            continue
        assert torch.equal(rows, tiles)
    if m <= 64:
        a, b = ops.gemm_bf16(x, w, sliced_ok=True), ops.gemm_bf16(x, tiled, sliced_ok=True)
        assert type(a) is type(b) and torch.equal(ops.as_tensor(a), ops.as_tensor(b))
        if n % 4 == 0 and ops.gemm_bf16_gate_up(x, w, "silu") is not None:
            assert torch.equal(ops.gemm_bf16_gate_up(x, w, "silu"), ops.gemm_bf16_gate_up(x, tiled, "silu"))
    from rvllm_amd.parts.linear import linear
    want = x.cpu().double() @ w.cpu().double().T
    got = linear(x, tiled)  # more than 64 rows: the library's product on the rows kept beside the tiles
    assert (got.cpu().double() - want).abs().max() <= 1e-2 * max(1.0, want.abs().max().item())
    if m > 64:
        with pytest.raises(ops.KernelError, match="row by row"):
            linear(x, ops.TiledWeight(w, keep_rows=False))


@pytest.mark.parametrize("activation", ["gelu_pytorch_tanh", "silu"])
@pytest.mark.parametrize("m,inter,k", [(1, 40, 64), (8, 96, 128), (64, 10240, 2560), (5, 520, 96), (17, 8, 8)])
def test_gate_and_up_product_with_the_activation_in_it(m, inter, k, activation):
    """act(x gate^T) * (x up^T) in one kernel over the rows in fours: against 64-bit arithmetic, and bit for bit
    against the product followed by the activation kernel, with the rows in fours and with the gates before the
    ups (all round the sums to bf16 before the activation)."""
    g = torch.Generator().manual_seed(22)
    x = (torch.randn(m, k, generator=g) * 1.5).bfloat16()
    gate = (torch.randn(inter, k, generator=g) * 0.08).bfloat16()
    up = (torch.randn(inter, k, generator=g) * 0.08).bfloat16()
    gate[:2], up[:2] = gate[:2] * 40, up[:2] * 0  # far out on the activation, and exact zeros
    fours = ops.rows_in_fours(gate, up)
    assert fours.shape == (2 * inter, k) and torch.equal(fours[0], gate[0]) and torch.equal(fours[1], gate[1])
    assert torch.equal(fours[2], up[0]) and torch.equal(fours[3], up[1]) and torch.equal(fours[4], gate[2])
    fused = ops.gemm_bf16_gate_up(dev(x), dev(fours), activation)
    assert fused is not None and fused.shape == (m, inter) and fused.dtype == torch.bfloat16
    gd, ud = (x.double() @ gate.double().T).bfloat16().double(), (x.double() @ up.double().T).bfloat16().double()
    want = (F.gelu(gd, approximate="tanh") if activation != "silu" else F.silu(gd)) * ud
    assert torch.allclose(fused.cpu().float(), want.float(), **tol(torch.bfloat16))
    in_fours = ops.gated_act(ops.gemm_bf16(dev(x), dev(fours)), activation, fours=True)
    halves = ops.gated_act(ops.gemm_bf16(dev(x), dev(torch.cat([gate, up]))), activation)
    assert torch.equal(fused, in_fours) and torch.equal(fused, halves)
    # another type, more rows than it covers, or a shape whose product is split along K: left to the two kernels
    assert ops.gemm_bf16_gate_up(dev(x.float()), dev(fours.float()), activation) is None
    assert ops.gemm_bf16_gate_up(dev(torch.zeros(65, k).bfloat16()), dev(fours), activation) is None
    assert ops.gemm_bf16_gate_up(dev(torch.zeros(8, 1416).bfloat16()), dev(torch.zeros(192, 1416).bfloat16()), activation) is None


@pytest.mark.parametrize("dtype", DTYPES)
def test_gated_act_over_rows_in_fours(dtype):
    """Whole values and unreduced slices; a width that the kernel cannot take in fours is refused."""
    g = torch.Generator().manual_seed(23)
    gate, up = torch.randn(5, 48, generator=g).to(dtype), torch.randn(5, 48, generator=g).to(dtype)
    gu = ops.rows_in_fours(gate.T.contiguous(), up.T.contiguous()).T.contiguous()  # the columns in fours
    want = (F.silu(gate.double()) * up.double()).float()
    assert torch.allclose(ops.gated_act(dev(gu), "silu", fours=True).cpu().float(), want, **tol(dtype))
    parts = torch.stack([gu.float() * 0.25, gu.float() * 0.75])
    sums = ops.SlicedSums(dev(parts), dtype)
    assert torch.allclose(ops.gated_act(sums, "silu", fours=True).cpu().float(), want, **tol(dtype))
    with pytest.raises(ops.KernelError, match="multiple of"):
        ops.gated_act(dev(torch.zeros(2, 2 * 42, dtype=dtype)), "silu", fours=True)


@pytest.mark.parametrize("m", [1, 8, 33, 64])
def test_gemm_skinny_under_every_plan(m):
    """The plan (waves a block, slices of K) is chosen by a model of the machine, one per shape; here every plan is
    forced in turn, with slices that end inside the last piece of x and blocks that reach past the last row of W."""
    lib = ops.library()
    g = torch.Generator().manual_seed(24)
    n, k = 1000, 1416  # 11.06 pieces of 128 columns; 62.5 tiles of 16 rows
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.05).bfloat16()
    want = x.double() @ w.double().T
    scale = want.abs().max().item()
    try:
        for waves in (4, 5, 6, 7, 8):
            for per in (1, 2, 3, 5, 12):
                lib.rv_gemm_skinny_force_plan(waves, per)
                out = ops.gemm_bf16(dev(x), dev(w), out_dtype=torch.float32)
                err = (out.cpu().double() - want).abs().max().item()
                assert err <= 2e-6 * scale * max(1.0, math.sqrt(k) / 16), (waves, per)
                # the slices handed on unreduced add up to the same bits as the product that adds them itself
                sums = ops.gemm_bf16(dev(x), dev(w), sliced_ok=True)
                whole = ops.gemm_bf16(dev(x), dev(w))
                if isinstance(sums, ops.SlicedSums):
                    assert sums.slices == -(-12 // per) and sums.slices > 1
                    assert torch.equal(sums.as_tensor(), whole), (waves, per)
                else:
                    assert per == 12 and torch.equal(sums, whole)
    finally:
        lib.rv_gemm_skinny_force_plan(0, 0)


def test_gemm_skinny_reads_strided_rows_and_refuses_what_it_cannot():
    g = torch.Generator().manual_seed(21)
    big = dev(torch.randn(6, 96, generator=g).bfloat16())
    x = big[:, :64]  # rows 96 apart
    w = dev(torch.randn(40, 64, generator=g).bfloat16())
    out = torch.empty((6, 40), dtype=torch.float32, device=DEV)
    assert ops.gemm_bf16(x, w, out) is out
    assert torch.allclose(out.cpu(), x.cpu().float() @ w.cpu().float().T, atol=1e-3)
    assert ops.gemm_bf16(dev(torch.zeros(2, 12).bfloat16()), dev(torch.zeros(4, 12).bfloat16()),
                         torch.empty((2, 4), dtype=torch.float32, device=DEV)) is None  # K is no multiple of 8


LIBRARY_SHAPES = [(65, 96, 64), (128, 2048 + 64, 3840), (300, 1000, 2560), (2048, 264, 1152), (77, 112, 72),
                  (200, 333, 40)]


@pytest.mark.parametrize("m,n,k", LIBRARY_SHAPES)
def test_the_librarys_product_against_64_bit(m, n, k):
    """The product of many rows goes to hipBLASLt from the kernel library itself; a shape that the library has no
    algorithm for comes back as None with nothing written, and ``linear`` takes the plain kernel for it."""
    from rvllm_amd.parts.linear import linear

    g = torch.Generator().manual_seed(m + n + k)
    x = dev(torch.randn(m, k, generator=g).bfloat16())
    w = dev((torch.randn(n, k, generator=g) * k ** -0.5).bfloat16())
    want = x.cpu().double() @ w.cpu().double().T
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    got = ops.library_gemm(x, w, out)
    if got is None:
        assert bool(torch.isnan(out).all())
    else:
        assert got is out
        assert torch.allclose(out.cpu().double(), want, atol=2e-2, rtol=1e-2)
    assert torch.allclose(linear(x, w).cpu().double(), want, atol=2e-2, rtol=1e-2)
    # rows that lie apart, in x and in out (a slice of a wider buffer, as the fused projections' outputs are)
    wide_x = dev(torch.randn(m, k + 24, generator=g).bfloat16())
    wide_out = torch.full((m, n + 40), 7.0, dtype=torch.bfloat16, device=DEV)
    xs, outs = wide_x[:, 8:8 + k], wide_out[:, 16:16 + n]
    linear(xs, w, out=outs)
    assert torch.allclose(outs.cpu().double(), xs.cpu().double() @ w.cpu().double().T, atol=2e-2, rtol=1e-2)
    assert bool((wide_out[:, :16] == 7.0).all()) and bool((wide_out[:, 16 + n:] == 7.0).all())


@pytest.mark.parametrize("m,n,k", [(65, 1000, 128), (200, 4096 + 64, 2560), (130, 333, 72)])
def test_the_librarys_product_with_a_32_bit_result(m, n, k):
    """Logits at many positions: bf16 operands, the sums stored in 32 bits, unrounded; through ``linear`` whichever
    kernel takes the shape."""
    from rvllm_amd.parts.linear import linear

    g = torch.Generator().manual_seed(m * n + k)
    x = dev(torch.randn(m, k, generator=g).bfloat16())
    w = dev((torch.randn(n, k, generator=g) * k ** -0.5).bfloat16())
    want = x.cpu().double() @ w.cpu().double().T
    out = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEV)
    got = ops.library_gemm(x, w, out)
    if got is None:
        assert bool(torch.isnan(out).all())
    else:
        assert torch.allclose(out.cpu().double(), want, atol=1e-4, rtol=1e-4)  # no rounding to bf16 at the end
        assert ops.library_plan_info(x, w, out)[0] in (0, 2)
        assert ops.library_plan_info(x, w, torch.empty((m, n), dtype=torch.bfloat16, device=DEV))[0] in (-1, 0, 2)
    logits = linear(x, ops.TiledWeight(w), out_dtype=torch.float32)
    assert logits.dtype == torch.float32
    assert torch.allclose(logits.cpu().double(), want, atol=1e-4, rtol=1e-4)


def test_the_librarys_product_tuned_gives_the_same_and_keeps_its_plan():
    g = torch.Generator().manual_seed(5)
    m, n, k = 160, 512 + 32, 640
    x = dev(torch.randn(m, k, generator=g).bfloat16())
    w = dev((torch.randn(n, k, generator=g) * k ** -0.5).bfloat16())
    want = x.cpu().double() @ w.cpu().double().T
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    assert ops.library_gemm(x, w, out) is out
    assert ops.library_plan_info(x, w, out)[0] == 0  # the library's first suggestion
    first = out.clone()
    ops.set_library_tuning(True)
    try:
        assert ops.library_gemm(x, w, out) is out
    finally:
        ops.set_library_tuning(False)
    state, index, us = ops.library_plan_info(x, w, out)
    assert state == 1 and index >= 0 and 0.0 < us < 1000.0
    assert torch.allclose(out.cpu().double(), want, atol=2e-2, rtol=1e-2)
    assert torch.allclose(out.float(), first.float(), atol=2e-2, rtol=1e-2)
    out.fill_(float("nan"))
    ops.library_gemm(x, w, out)  # the kept plan, with tuning off
    assert ops.library_plan_info(x, w, out) == (state, index, us)
    assert torch.allclose(out.cpu().double(), want, atol=2e-2, rtol=1e-2)


def test_a_shape_nobody_tuned_takes_its_tuned_neighbours_algorithm():
    """A row count that tuning never met runs on the algorithm of the nearest tuned row count with the same matrix
    (within one and a half times), also when it was first seen before its neighbour was tuned; a row count further
    off keeps the library's first suggestion.  The results are right whichever algorithm runs."""
    g = torch.Generator().manual_seed(8)
    n, k = 448 + 32, 576
    w = dev((torch.randn(n, k, generator=g) * k ** -0.5).bfloat16())

    def product(m):
        x = dev(torch.randn(m, k, generator=g).bfloat16())
        out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
        assert ops.library_gemm(x, w, out) is out
        assert torch.allclose(out.cpu().double(), x.cpu().double() @ w.cpu().double().T, atol=2e-2, rtol=1e-2), m
        return ops.library_plan_info(x, w, out)

    early = product(208)  # seen before anything is tuned
    assert early[0] == 0
    ops.set_library_tuning(True)
    try:
        tuned = product(192)
    finally:
        ops.set_library_tuning(False)
    assert tuned[0] == 1
    near = product(200)
    again = product(208)
    far = product(400)
    assert far[0] == 0
    for state, index, _ in (near, again):
        assert state in (0, 2)  # 0 only if the library says that the algorithm does not take this shape
        if state == 2:
            assert index == tuned[1]
    assert 2 in (near[0], again[0])


def test_the_librarys_tuned_plans_go_to_a_file_and_come_back(tmp_path):
    """What tuning found is written as JSON and taken again by index: a plan for a shape this process has not
    seen makes the shape count as tuned (or is refused, if the algorithm does not take the shape) and the product
    is right either way; a file of another version of the library, a broken one and a missing one change nothing."""
    import json

    g = torch.Generator().manual_seed(6)
    m, n, k = 176, 384 + 32, 704
    x = dev(torch.randn(m, k, generator=g).bfloat16())
    w = dev((torch.randn(n, k, generator=g) * k ** -0.5).bfloat16())
    out = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    ops.set_library_tuning(True)
    try:
        ops.library_gemm(x, w, out)
    finally:
        ops.set_library_tuning(False)
    state, index, us = ops.library_plan_info(x, w, out)
    assert state == 1
    path = tmp_path / "plans.json"
    assert ops.library_plans_save(str(path), DEV) >= 1
    doc = json.loads(path.read_text())
    assert [m, n, k, k, k, n, index, 0] in [p[:7] + p[8:] for p in doc["plans"]]  # the last field: a bf16 result
    assert ops.library_plans_load(str(path), DEV) == len(doc["plans"])  # all known already: they stay as they are

    m2 = m + 16  # a shape nobody has tuned here, under the first one's algorithm
    x2 = dev(torch.randn(m2, k, generator=g).bfloat16())
    out2 = torch.empty((m2, n), dtype=torch.bfloat16, device=DEV)
    assert ops.library_plan_info(x2, w, out2)[0] == -1
    other = tmp_path / "other.json"
    other.write_text(json.dumps(dict(doc, plans=[[m2, n, k, k, k, n, index, 12.5, 0]])))
    taken = ops.library_plans_load(str(other), DEV)
    assert taken in (0, 1)
    assert ops.library_plan_info(x2, w, out2)[:2] == ((1, index) if taken else (0, ops.library_plan_info(x2, w, out2)[1]))
    assert ops.library_gemm(x2, w, out2) is out2
    assert torch.allclose(out2.cpu().double(), x2.cpu().double() @ w.cpu().double().T, atol=2e-2, rtol=1e-2)

    m3 = m + 32
    x3 = dev(torch.randn(m3, k, generator=g).bfloat16())
    out3 = torch.empty((m3, n), dtype=torch.bfloat16, device=DEV)
    other.write_text(json.dumps(dict(doc, hipblaslt=doc["hipblaslt"] + 1, plans=[[m3, n, k, k, k, n, index, 12.5, 0]])))
    assert ops.library_plans_load(str(other), DEV) == 0
    other.write_text(json.dumps(dict(doc, plans=[[m3, n, k, k, k, n, 1 << 30, 12.5, 0]])))  # no such algorithm
    assert ops.library_plans_load(str(other), DEV) == 0
    other.write_text(json.dumps(dict(doc, plans=[[-5, n, k, k, k, n, index, 12.5, 0], [m3, n, k, 1, 1, 1, index, 1.0, 0]])))
    assert ops.library_plans_load(str(other), DEV) == 0  # sizes and strides that cannot be: skipped, no error
    other.write_text("{ not json")
    assert ops.library_plans_load(str(other), DEV) == 0
    assert ops.library_plans_load(str(tmp_path / "missing.json"), DEV) == 0
    assert ops.library_plan_info(x3, w, out3)[0] != 1  # not tuned: unseen, or on its neighbour's algorithm
    assert ops.library_gemm(x3, w, out3) is out3
    assert torch.allclose(out3.cpu().double(), x3.cpu().double() @ w.cpu().double().T, atol=2e-2, rtol=1e-2)


def paged_setup(T_total, nkv, hd, page_size, dtype, seed, scramble=True):
    """A cache whose pages are handed out in a scrambled order."""
    g = torch.Generator().manual_seed(seed)
    n_pages = -(-T_total // page_size) + 3
    order = torch.randperm(n_pages, generator=g).tolist() if scramble else list(range(n_pages))
    k_pages = torch.zeros(n_pages, page_size, nkv, hd, dtype=dtype)
    v_pages = torch.zeros_like(k_pages)
    table = torch.full((1, n_pages), -1, dtype=torch.int32)
    for i in range(-(-T_total // page_size)):
        table[0, i] = order[i]
    return g, k_pages, v_pages, table


def to_cache(k_pages, v_pages):
    """The test keeps pages as [page, slot, kv_head, d]; the cache on the
    device holds keys as [page, kv_head, slot, d] and values transposed inside
    groups of 16 slots, [page, kv_head, slot / 16, d, slot % 16]."""
    n_pages, page_size, nkv, hd = v_pages.shape
    v = v_pages.view(n_pages, page_size // 16, 16, nkv, hd).permute(0, 3, 1, 4, 2)
    return dev(k_pages.permute(0, 2, 1, 3)), dev(v)


def from_cache(kp, vp):
    n_pages, nkv, groups, hd, _ = vp.shape
    return kp.cpu().permute(0, 2, 1, 3), vp.cpu().permute(0, 2, 4, 1, 3).reshape(n_pages, groups * 16, nkv, hd)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,hd,rot", [(4, 2, 16, 16), (6, 3, 48, 48), (5, 1, 80, 40), (8, 4, 256, 256), (3, 3, 128, 0),
                                          (2, 1, 36, 12), (2, 2, 512, 512)])  # the last two: the kernel for odd sizes
@pytest.mark.parametrize("page_size", [16, 64])
@pytest.mark.parametrize("T", [37, 301])  # a few tokens: one a wave; a prompt portion: four a wave, the last wave not full
def test_qk_norm_rope_kv_write(dtype, nq, nkv, hd, rot, page_size, T):
    g, k_pages, v_pages, table = paged_setup(T + 100, nkv, hd, page_size, dtype, 7)
    qkv = torch.randn(T, (nq + 2 * nkv) * hd, generator=g).to(dtype)
    qw = (torch.randn(hd, generator=g) * 0.1).to(dtype)
    kw = (torch.randn(hd, generator=g) * 0.1).to(dtype)
    positions = torch.arange(90, 90 + T, dtype=torch.int32)  # straddles page edges
    inv_freq = (10000.0 ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / hd) / 4.0).float()
    q_out = torch.empty(T, nq * hd, dtype=dtype, device=DEV)
    kp_dev, vp_dev = to_cache(k_pages, v_pages)
    rope = ops.rope_table(dev(inv_freq), dev(positions), T) if rot else None
    ops.qk_norm_rope_kv_write(dev(qkv), q_out, dev(qw), dev(kw), 1e-6, 1.0, rope, rot,
                              dev(positions), dev(torch.zeros(T, dtype=torch.int32)), dev(table), kp_dev, vp_dev, nq,
                              nkv, hd)
    kp, vp = from_cache(kp_dev, vp_dev)
    q, k, v = qkv.double().split([nq * hd, nkv * hd, nkv * hd], dim=1)
    q = P.rmsnorm(q.view(T, nq, hd), qw.double(), 1e-6)
    k = P.rmsnorm(k.view(T, nkv, hd), kw.double(), 1e-6)
    if rot:
        full = torch.zeros(hd // 2, dtype=torch.float64)  # dimensions past rot/2 get angle 0: they pass through
        full[: rot // 2] = inv_freq.double()
        q, k = P.rope(q, positions, full), P.rope(k, positions, full)
    assert torch.allclose(q_out.cpu().float().view(T, nq, hd), q.float(), **tol(dtype))
    for t in range(T):
        pos = int(positions[t])
        page, off = int(table[0, pos // page_size]), pos % page_size
        assert torch.allclose(kp[page, off].cpu().float(), k[t].float(), **tol(dtype)), t
        assert torch.equal(vp[page, off].cpu(), v[t].view(nkv, hd).to(dtype)), t  # values are stored as projected
    # nothing else was written
    written = {(int(table[0, int(p) // page_size]), int(p) % page_size) for p in positions}
    mask = torch.ones(kp.shape[:2], dtype=torch.bool)
    for page, off in written:
        mask[page, off] = False
    assert kp.cpu()[mask].abs().sum() == 0 and vp.cpu()[mask].abs().sum() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page_size", [16, 32])
@pytest.mark.parametrize("longest", [70, 333])  # the step's tokens one a wave, and four a wave
def test_values_written_a_page_at_a_time(dtype, page_size, longest):
    """Portions that begin and end inside pages, cover whole pages, and single tokens: the values reach the same
    places as when every token writes its own, and nothing else is touched."""
    nq, nkv, hd = 4, 2, 48
    portions = [(5, longest), (64, 32), (0, 1), (31, 2), (100, 16)]  # (first position, tokens)
    case = Case(portions, nq, nkv, hd, page_size, dtype, 17)
    T = case.q.shape[0]
    g = torch.Generator().manual_seed(18)
    qkv = torch.randn(T, (nq + 2 * nkv) * hd, generator=g).to(dtype)
    results = []
    for by_page in (False, True):
        kp, vp = to_cache(torch.zeros_like(case.k_log), torch.zeros_like(case.v_log))
        q_out = torch.empty(T, nq * hd, dtype=dtype, device=DEV)
        ops.qk_norm_rope_kv_write(dev(qkv), q_out, None, None, 0.0, 0.0, None, 0, case.step.positions,
                                  case.step.token_req, dev(case.table), kp, vp, nq, nkv, hd,
                                  values_by_page=case.step if by_page else None)
        results.append((q_out.cpu(), kp.cpu(), vp.cpu()))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    # and the values are the projection's, at the token's page and slot
    _, vp = from_cache(results[1][1].to(DEV), results[1][2].to(DEV))
    t = 0
    for b, (s, n) in enumerate(portions):
        for pos in range(s, s + n):
            page = int(case.table[b, pos // page_size])
            want = qkv[t, (nq + nkv) * hd:].view(nkv, hd)
            assert torch.equal(vp[page, pos % page_size].cpu(), want), (b, pos)
            t += 1


@pytest.mark.parametrize("nq,nkv,hd,rot", [(8, 4, 256, 256), (5, 1, 128, 64), (7, 3, 64, 64), (3, 2, 16, 16), (6, 2, 32, 0),
                                          (13, 5, 64, 32), (1, 1, 256, 128)])
@pytest.mark.parametrize("page_size", [16, 64])
def test_qk_norm_rope_of_a_prompt_portion(nq, nkv, hd, rot, page_size):
    """Some hundred tokens in bf16 with the values written by pages take the kernel that holds eight dimensions a
    lane and several heads a wave: heads that fill a wave's passes and heads that do not, a rotation of the whole
    head, of a part and none, portions that begin inside pages.  Against the plain formulas, and against the kernel
    that takes a head a wave."""
    dtype = torch.bfloat16
    portions = [(5, 290), (64, 32), (0, 1), (31, 2), (100, 16)]
    case = Case(portions, nq, nkv, hd, page_size, dtype, 23)
    T = case.q.shape[0]
    g = torch.Generator().manual_seed(24)
    qkv = torch.randn(T, (nq + 2 * nkv) * hd, generator=g).to(dtype)
    qw = (torch.randn(hd, generator=g) * 0.1).to(dtype)
    kw = (torch.randn(hd, generator=g) * 0.1).to(dtype)
    inv_freq = (10000.0 ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / hd) / 4.0).float()
    rope = ops.rope_table(dev(inv_freq), case.step.positions, T) if rot else None
    results = []
    for by_page in (False, True):
        kp, vp = to_cache(torch.zeros_like(case.k_log), torch.zeros_like(case.v_log))
        q_out = torch.full((T, nq * hd), float("nan"), dtype=dtype, device=DEV)
        ops.qk_norm_rope_kv_write(dev(qkv), q_out, dev(qw), dev(kw), 1e-5, 1.0, rope, rot, case.step.positions,
                                  case.step.token_req, dev(case.table), kp, vp, nq, nkv, hd,
                                  values_by_page=case.step if by_page else None)
        results.append((q_out.cpu(), kp.cpu(), vp.cpu()))
    # the values are copied, so they are the same bits; the sums of squares are added up in another order
    assert torch.equal(results[0][2].view(torch.int16), results[1][2].view(torch.int16))
    for a, b in zip(results[0][:2], results[1][:2]):
        assert torch.allclose(a.float(), b.float(), **tol(dtype))
    q, k, _ = qkv.double().split([nq * hd, nkv * hd, nkv * hd], dim=1)
    q = P.rmsnorm(q.view(T, nq, hd), qw.double(), 1e-5)
    k = P.rmsnorm(k.view(T, nkv, hd), kw.double(), 1e-5)
    if rot:
        full = torch.zeros(hd // 2, dtype=torch.float64)
        full[: rot // 2] = inv_freq.double()
        q, k = P.rope(q, case.positions, full), P.rope(k, case.positions, full)
    assert torch.allclose(results[1][0].float().view(T, nq, hd), q.float(), **tol(dtype))
    kp, _ = from_cache(results[1][1].to(DEV), results[1][2].to(DEV))
    for t in range(T):
        b, pos = int(case.token_req[t]), int(case.positions[t])
        page = int(case.table[b, pos // page_size])
        assert torch.allclose(kp[page, pos % page_size].cpu().float(), k[t].float(), **tol(dtype)), t


def test_rows_and_columns_of_a_host_matrix_copied_to_the_device():
    """A step sends of its block tables only the requests' rows by the pages of the longest: one strided copy from
    pinned memory, which leaves the rest of the device matrix as it was."""
    host = torch.arange(6 * 40, dtype=torch.int32).view(6, 40).pin_memory()
    on_device = torch.full((8, 50), -7, dtype=torch.int32, device=DEV)
    ops.copy_rows_to_device(on_device, host, 4, 33)
    got = on_device.cpu()
    assert torch.equal(got[:4, :33], host[:4, :33])
    assert (got[4:] == -7).all() and (got[:, 33:] == -7).all()
    ops.copy_rows_to_device(on_device, host, 0, 10)  # nothing to copy is no error
    with pytest.raises(ops.KernelError, match="pinned"):
        ops.copy_rows_to_device(on_device, torch.zeros(6, 40, dtype=torch.int32), 2, 2)
    with pytest.raises(ops.KernelError, match="does not fit"):
        ops.copy_rows_to_device(on_device, host, 7, 10)


def test_rope_table_against_64_bit_angles():
    """cos and sin of float32(position) * inv_freq, positions up to a long context, against 64-bit
    functions of the same 32-bit angle."""
    inv_freq = (1e6 ** (-2.0 * torch.arange(24, dtype=torch.float64) / 48) / 8.0).float()
    positions = torch.tensor([0, 1, 2, 17, 1023, 4096, 65535, 131071, 5, 99999], dtype=torch.int32)
    cos, sin = ops.rope_table(dev(inv_freq), dev(positions), 8)  # fewer tokens than positions: only the first 8
    assert cos.shape == sin.shape == (8, 24) and cos.dtype == torch.float32
    angle = (positions[:8].float()[:, None] * inv_freq[None, :]).double()  # the product is rounded to 32-bit first
    assert torch.allclose(cos.cpu().double(), angle.cos(), atol=2e-7, rtol=0)
    assert torch.allclose(sin.cpu().double(), angle.sin(), atol=2e-7, rtol=0)


def test_qk_norm_rope_without_cache_write_leaves_the_cache_alone():
    nq, nkv, hd, T = 2, 1, 32, 5
    g, k_pages, v_pages, table = paged_setup(64, nkv, hd, 16, torch.float32, 8)
    qkv = torch.randn(T, (nq + 2 * nkv) * hd, generator=g)
    q_out = torch.empty(T, nq * hd, device=DEV)
    kp, vp = to_cache(k_pages, v_pages)
    ops.qk_norm_rope_kv_write(dev(qkv), q_out, None, None, 0.0, 0.0, None, 0, dev(torch.arange(T, dtype=torch.int32)),
                              dev(torch.zeros(T, dtype=torch.int32)), dev(table), kp, vp, nq, nkv, hd, write_kv=False)
    assert kp.abs().sum() == 0 and vp.abs().sum() == 0
    assert torch.equal(q_out.cpu(), qkv[:, : nq * hd])  # no norm, no rotation: queries pass through


def reference_attention(q, k_all, v_all, positions, scale, window):
    """Attention of the query tokens (at ``positions``) over keys 0..p of one request."""
    out = torch.empty_like(q)
    T, nq, hd = q.shape
    group = nq // k_all.shape[1]
    for t in range(T):
        p = int(positions[t])
        lo = max(0, p - window + 1) if window else 0
        for h in range(nq):
            s = scale * (k_all[lo:p + 1, h // group] @ q[t, h])
            out[t, h] = torch.softmax(s, dim=0) @ v_all[lo:p + 1, h // group]
    return out


class Case:
    """Requests with their portions, a scrambled paged cache and the flat batch."""

    def __init__(self, portions, nq, nkv, hd, page_size, dtype, seed, window=None, drop_passed_pages=True):
        # portions: (position of the first query token, number of query tokens) per request
        g = torch.Generator().manual_seed(seed)
        self.nq, self.nkv, self.hd, self.page_size, self.window, self.dtype = nq, nkv, hd, page_size, window, dtype
        self.portions = portions
        B = len(portions)
        lengths = [s + n for s, n in portions]
        pages_per = [-(-L // page_size) for L in lengths]
        n_pages = sum(pages_per) + 5
        order = torch.randperm(n_pages, generator=g).tolist()
        self.k_log = torch.zeros(n_pages, page_size, nkv, hd, dtype=dtype)  # [page, slot, head, d]
        self.v_log = torch.zeros_like(self.k_log)
        self.table = torch.full((B, max(pages_per) + 2), -1, dtype=torch.int32)
        self.k_all, self.v_all = [], []
        nxt = 0
        for b, L in enumerate(lengths):
            k = torch.randn(L, nkv, hd, generator=g).to(dtype)
            v = torch.randn(L, nkv, hd, generator=g).to(dtype)
            self.k_all.append(k)
            self.v_all.append(v)
            for i in range(pages_per[b]):
                page = order[nxt]
                nxt += 1
                self.table[b, i] = page
                rows = slice(i * page_size, min((i + 1) * page_size, L))
                self.k_log[page, : rows.stop - rows.start] = k[rows]
                self.v_log[page, : rows.stop - rows.start] = v[rows]
            if window and drop_passed_pages:
                # pages that the window of the portion's first token has passed are gone:
                # a kernel that touches them reads NaN
                first = max(0, portions[b][0] - window + 1) // page_size
                for i in range(first):
                    self.k_log[int(self.table[b, i])] = float("nan")
                    self.v_log[int(self.table[b, i])] = float("nan")
                    self.table[b, i] = -1
        T = sum(n for _, n in portions)
        self.q = torch.randn(T, nq, hd, generator=g).to(dtype)
        self.positions = torch.cat([torch.arange(s, s + n, dtype=torch.int32) for s, n in portions])
        self.token_req = torch.cat([torch.full((n,), b, dtype=torch.int32) for b, (_, n) in enumerate(portions)])
        starts = [0]
        for _, n in portions:
            starts.append(starts[-1] + n)
        self.step = types.SimpleNamespace(
            num_tokens=T, num_requests=B, positions=dev(self.positions), token_req=dev(self.token_req),
            q_start=dev(torch.tensor(starts, dtype=torch.int32)),
            chunk_start=dev(torch.tensor([s for s, _ in portions], dtype=torch.int32)),
            max_portion=max(n for _, n in portions), max_context=max(lengths), host_q_start=starts)

    def reference(self, scale):
        outs = []
        t = 0
        for b, (s, n) in enumerate(self.portions):
            pos = torch.arange(s, s + n)
            outs.append(reference_attention(self.q[t:t + n].double(), self.k_all[b].double(), self.v_all[b].double(),
                                            pos, scale, self.window))
            t += n
        return torch.cat(outs)

    def run(self, kernel, scale, **kw):
        kp, vp = to_cache(self.k_log, self.v_log)
        T = self.q.shape[0]
        out = torch.full((T, self.nq * self.hd), float("nan"), dtype=self.dtype, device=DEV)
        q = dev(self.q.view(T, -1))
        if kernel == "generic":
            ops.paged_attention_generic(q, kp, vp, dev(self.table), self.step.positions, self.step.token_req, out,
                                        self.nq, scale, self.window)
        else:
            ops.paged_attention_mfma(q, kp, vp, dev(self.table), self.step, out, self.nq, scale, self.window, **kw)
        return out.cpu().view(T, self.nq, self.hd)


MIXED = [(150, 53), (180, 1), (0, 40), (202, 1), (31, 2)]  # portions beside single tokens, page edges, position 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,hd", [(4, 2, 16), (6, 1, 48), (3, 3, 80), (8, 4, 256), (2, 1, 128)])
@pytest.mark.parametrize("window", [None, 7, 100])
def test_paged_attention_generic(dtype, nq, nkv, hd, window):
    case = Case(MIXED, nq, nkv, hd, 16, dtype, 9, window)
    got = case.run("generic", hd ** -0.5)
    assert torch.allclose(got.float(), case.reference(hd ** -0.5).float(), **tol(dtype))


@pytest.mark.parametrize("nq,nkv,hd", [(4, 2, 16), (6, 1, 48), (3, 3, 80), (8, 4, 256), (2, 1, 128), (16, 1, 32),
                                       (5, 5, 240), (12, 4, 64)])
@pytest.mark.parametrize("window", [None, 7, 100])
@pytest.mark.parametrize("page_size", [16, 64])
@pytest.mark.parametrize("kernels", ["both", "split", "shared"])
def test_paged_attention_mfma(nq, nkv, hd, window, page_size, kernels):
    """``both``: as the engine runs a mixed batch, long portions through the
    kernel that shares key tiles in LDS, short ones through the one that
    splits keys; ``split`` / ``shared``: every request through one of them."""
    case = Case(MIXED, nq, nkv, hd, page_size, torch.bfloat16, 9, window)
    want = case.reference(hd ** -0.5).float()
    kw = {"both": {}, "split": {"prefill_kernel": False}, "shared": {"prefill_kernel": True}}[kernels]
    assert torch.allclose(case.run("mfma", hd ** -0.5, **kw).float(), want, **tol(torch.bfloat16))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,hd", [(4, 2, 320), (2, 1, 512), (34, 2, 272)])
@pytest.mark.parametrize("window", [None, 100])
def test_paged_attention_generic_above_256(dtype, nq, nkv, hd, window):
    """Head sizes that no matrix-core kernel takes, up to the largest allowed, and 17 query heads a group."""
    case = Case(MIXED, nq, nkv, hd, 16, dtype, 23, window)
    got = case.run("generic", hd ** -0.5)
    assert torch.allclose(got.float(), case.reference(hd ** -0.5).float(), **tol(dtype))
    kp, vp = to_cache(case.k_log, case.v_log)
    assert not ops.mfma_attention_covers(kp, vp, nq)
    with pytest.raises(ops.KernelError):
        Case([(5, 1)], 1, 1, 528, 16, dtype, 23).run("generic", 1.0)  # beyond the largest head size: refused


@pytest.mark.parametrize("nq,nkv,hd", [(8, 4, 256), (32, 16, 128), (6, 1, 48)])
@pytest.mark.parametrize("window", [None, 100, 1024])
def test_paged_attention_mfma_many_single_tokens_beside_long_portions(nq, nkv, hd, window):
    """A step as a scheduler builds it under load: twenty decoding requests at contexts from a few keys to over
    a thousand, between and around two long prompt portions (one from position 0, one continuing): one launch
    of each attention kernel, each leaving the other's requests alone."""
    singles = [(3 + 61 * i, 1) for i in range(20)]
    portions = singles[:7] + [(0, 300)] + singles[7:15] + [(517, 200)] + singles[15:]
    case = Case(portions, nq, nkv, hd, 16, torch.bfloat16, 24, window)
    want = case.reference(hd ** -0.5).float()
    assert torch.allclose(case.run("mfma", hd ** -0.5).float(), want, **tol(torch.bfloat16))


def test_paged_attention_shared_tiles_long_prompt_portions():
    """Portions as a scheduler cuts a long prompt: from position 0, continuing
    at an odd position, and one that passes a window's edge."""
    for portions, window in (([(0, 300)], None), ([(257, 130), (0, 70)], None), ([(0, 300)], 64), ([(990, 100)], 1024),
                             ([(100, 257)], 100)):
        case = Case(portions, 8, 4, 256, 16, torch.bfloat16, 13, window)
        want = case.reference(1.0 / 16).float()
        assert torch.allclose(case.run("mfma", 1.0 / 16).float(), want, **tol(torch.bfloat16)), (portions, window)


@pytest.mark.parametrize("nq,nkv,hd,page_size", [(8, 4, 256, 16), (6, 2, 64, 64)])
def test_paged_attention_shared_tiles_beyond_the_table_kept_in_lds(nq, nkv, hd, page_size):
    """Portions deep in a long context: the kernel keeps the table entries of 8192 keys at hand and has to fetch
    more of the table on its way, once and twice; with a window it starts far from the table's beginning."""
    for portions, window in (([(8200, 40), (16500, 33)], None), ([(9000, 64)], 1024)):
        case = Case(portions, nq, nkv, hd, page_size, torch.bfloat16, 21, window)
        want = case.reference(hd ** -0.5).float()
        got = case.run("mfma", hd ** -0.5, prefill_kernel=True).float()
        assert torch.allclose(got, want, **tol(torch.bfloat16)), (portions, window)


def _plant(case, b, key, head, dim, value):
    """Key `key` of request b becomes `value` at one dimension and nothing else, in the log and in the pages."""
    k = case.k_all[b]
    k[key, head] = 0
    k[key, head, dim] = value
    case.k_log[int(case.table[b, key // case.page_size]), key % case.page_size, head] = k[key, head]


@pytest.mark.parametrize("far", [0, 17, 31, 32, 63, 64, 200, 255])
def test_shared_tiles_attention_finds_one_key(far):
    """The kernel for prompt portions: one key carries all the weight for every later token, wherever it
    lies in a 64-key stage (first or second half, which different waves multiply and then merge) and
    whichever stage; tokens before it do not see it; at a window's edge it is seen, one further not."""
    nq, nkv, hd, n = 4, 2, 64, 256
    for window in (None, 40):
        case = Case([(0, n)], nq, nkv, hd, 16, torch.bfloat16, 14, window, drop_passed_pages=False)
        for b in range(1):
            case.k_all[b] *= 0.01
            case.k_log *= 0.01
        _plant(case, 0, far, 1, 5, 40.0)
        case.q[:] = 0
        case.q[:, :, 5] = 40.0  # every query looks along dimension 5
        got = case.run("mfma", 1.0, prefill_kernel=True).float()
        want = case.reference(1.0).float()
        assert torch.allclose(got, want, **tol(torch.bfloat16))
        v_far = case.v_all[0][far, 1].float()
        for t in (far, min(far + 39, n - 1), min(far + 40, n - 1), n - 1):
            sees = t >= far and (window is None or t - far < window)
            hit = torch.allclose(got[t, 2:], v_far.expand(2, hd), atol=2e-2)  # heads 2, 3 read kv head 1
            assert hit == sees, (far, window, t)


def test_shared_tiles_attention_when_the_maximum_grows_late():
    """Scores that grow along the sequence by more than the step at which sums are rescaled, by less than
    it, and not at all: the running sums follow in each case."""
    nq, nkv, hd, n = 2, 1, 32, 320
    for step_size in (0.0, 0.05, 3.0, 9.0):
        case = Case([(0, n)], nq, nkv, hd, 16, torch.bfloat16, 15, None)
        ramp = torch.arange(n, dtype=torch.float32) / 32 * step_size  # grows by step_size per 32 keys
        case.k_all[0][:, 0, 7] = ramp.to(torch.bfloat16)
        for j in range(n):
            case.k_log[int(case.table[0, j // 16]), j % 16, 0, 7] = case.k_all[0][j, 0, 7]
        case.q[:, :, 7] = 1.0
        got = case.run("mfma", 1.0, prefill_kernel=True).float()
        assert torch.allclose(got, case.reference(1.0).float(), **tol(torch.bfloat16)), step_size


def test_shared_tiles_attention_missing_page_shows():
    case = Case([(0, 100)], 2, 1, 32, 16, torch.bfloat16, 16)
    case.table[0, 2] = -1  # keys 32..47 are gone: every token from 32 on must not look valid
    got = case.run("mfma", 1.0, prefill_kernel=True)
    assert torch.isnan(got[32:]).all() and not torch.isnan(got[:32]).any()


@pytest.mark.parametrize("nq,nkv,hd", [(8, 4, 256), (32, 16, 128), (6, 1, 48), (5, 5, 240)])
@pytest.mark.parametrize("pieces", [(1, 5), (2, 3), (3, 2), (4, 64), (1, 2)])
def test_prompt_attention_with_long_tiles_in_pieces(nq, nkv, hd, pieces):
    """The prompt kernel with its long tiles cut into pieces, a block each, merged afterwards: pieces of a single
    block of keys, pieces that leave some tiles whole, more pieces allowed than any tile has, fewer than the
    piece length asks for (the pieces are then longer); portions from position 0, continuing ones, short ones
    among them, with and without a window.  The same as a tile a block, and as the 64-bit reference."""
    for portions, window in (([(0, 300)], None), ([(257, 130), (0, 70), (40, 17)], None), ([(0, 300), (5, 2)], 64),
                             ([(990, 100)], 1024), ([(100, 257), (3, 1), (0, 33)], 100)):
        case = Case(portions, nq, nkv, hd, 16, torch.bfloat16, 31, window)
        want = case.reference(hd ** -0.5).float()
        got = case.run("mfma", hd ** -0.5, prefill_pieces=pieces).float()
        assert torch.allclose(got, want, **tol(torch.bfloat16)), (portions, window)
        whole = case.run("mfma", hd ** -0.5, prefill_pieces=(1 << 20, 1)).float()
        assert torch.allclose(got, whole, **tol(torch.bfloat16)), (portions, window)


def test_prompt_attention_cuts_its_tiles_where_few_walk_many_keys():
    """The choice: a short portion deep in a long context (a prompt that arrives in portions of 128 tokens: four
    tiles a key/value head that walk 8 000 keys each, on a machine of 256 CUs) has its tiles cut into pieces;
    a whole prompt of 2 048 tokens is bound by all its blocks of keys together, not by its longest tile, and
    is left a tile a block, as are portions that fill the machine, short ones and decoded tokens."""
    plan = lambda lengths, starts, window=None: ops.plan_prefill_pieces(lengths, starts, 32, window, 16, 256, 4)
    assert plan([128], [8000])[1] > 4
    assert plan([64], [8000], window=1024)[1] > 1    # under the window its tiles see 1 087 keys: 8 blocks for 256 CUs
    assert plan([2048], [0])[1] == 1
    assert plan([1024], [0])[1] == 1
    assert plan([2048] * 4, [30000] * 4)[1] == 1
    assert plan([64] * 8, [0] * 8)[1] == 1
    assert plan([1] * 8, [500] * 8)[1] == 1          # left to the other kernel
    piece_max, pieces_max = plan([128], [30000])
    assert piece_max >= 8 and pieces_max * piece_max >= -(-30128 // 64)  # the pieces cover the longest tile
    # through the kernel, with the plan it makes for itself, at sizes where it cuts
    case = Case([(4000, 100), (700, 1)], 8, 4, 256, 16, torch.bfloat16, 32, None)
    assert ops.plan_prefill_pieces([100, 1], [4000, 700], 32, None, 16, 256, 4)[1] > 1
    want = case.reference(1.0 / 16).float()
    assert torch.allclose(case.run("mfma", 1.0 / 16).float(), want, **tol(torch.bfloat16))


@pytest.mark.parametrize("far", [0, 17, 63, 64, 200, 255])
def test_prompt_attention_in_pieces_finds_one_key(far):
    """One key carries all the weight, wherever it lies among pieces of two blocks of keys: the piece that holds
    it must win the merge for every later token, and no piece of an earlier token may see it; a page that is
    missing shows in exactly the tokens that see it."""
    nq, nkv, hd, n = 4, 2, 64, 256
    for window in (None, 40):
        case = Case([(0, n)], nq, nkv, hd, 16, torch.bfloat16, 14, window, drop_passed_pages=False)
        case.k_all[0] *= 0.01
        case.k_log *= 0.01
        _plant(case, 0, far, 1, 5, 40.0)
        case.q[:] = 0
        case.q[:, :, 5] = 40.0
        got = case.run("mfma", 1.0, prefill_kernel=True, prefill_pieces=(2, 2)).float()
        assert torch.allclose(got, case.reference(1.0).float(), **tol(torch.bfloat16))
        v_far = case.v_all[0][far, 1].float()
        for t in (far, min(far + 39, n - 1), min(far + 40, n - 1), n - 1):
            sees = t >= far and (window is None or t - far < window)
            assert torch.allclose(got[t, 2:], v_far.expand(2, hd), atol=2e-2) == sees, (far, window, t)
    case = Case([(0, 200)], 2, 1, 32, 16, torch.bfloat16, 16)
    case.table[0, 2] = -1  # keys 32..47 are gone
    got = case.run("mfma", 1.0, prefill_kernel=True, prefill_pieces=(1, 4))
    assert torch.isnan(got[32:]).all() and not torch.isnan(got[:32]).any()


@pytest.mark.parametrize("splits", [(1, 224), (2, 128), (7, 32), (4, 64)])
@pytest.mark.parametrize("window", [None, 100])
def test_paged_attention_mfma_every_split(splits, window):
    """One split, splits that end on and off page edges, splits that are empty
    for some tiles: all give the same result."""
    case = Case(MIXED, 8, 4, 256, 16, torch.bfloat16, 10, window)
    want = case.reference(1.0 / 16).float()
    got = case.run("mfma", 1.0 / 16, splits=splits, prefill_kernel=False)
    assert torch.allclose(got.float(), want, **tol(torch.bfloat16))


@pytest.mark.parametrize("nq,nkv,hd", [(6, 1, 48), (3, 3, 80), (8, 4, 256), (16, 1, 32), (4, 2, 128)])
@pytest.mark.parametrize("splits", [(19, 64), (38, 32)])
def test_paged_attention_mfma_merges_many_splits(nq, nkv, hd, splits):
    """Many splits of the keys, merged afterwards: more splits than the merge
    loads at a time, tiles of one, two and three tokens, head counts that
    leave columns of a tile empty, head sizes that are no power of two; and
    again right away, into a workspace that holds the last call's parts."""
    portions = [(1199, 1), (1100, 2), (0, 3), (700, 1), (1213, 1)]
    for window in (None, 300):
        case = Case(portions, nq, nkv, hd, 16, torch.bfloat16, 17, window)
        want = case.reference(hd ** -0.5).float()
        for again in range(3):
            got = case.run("mfma", hd ** -0.5, splits=splits, prefill_kernel=False).float()
            assert torch.allclose(got, want, **tol(torch.bfloat16)), (window, again)


@pytest.mark.parametrize("nq,nkv,hd", [(8, 4, 256), (6, 1, 48), (3, 3, 80), (16, 1, 32), (4, 2, 128), (5, 5, 240)])
@pytest.mark.parametrize("window", [None, 100, 1024])
def test_paged_attention_mfma_merged_inside_the_block(nq, nkv, hd, window):
    """A tile's key splits as the eight waves of one block, merged through
    LDS: decoded tokens and portions of two and three at contexts from one
    key (seven waves without any) to over a thousand, with and without a
    window; the same as with the splits merged by the second kernel."""
    portions = [(0, 1), (5, 1), (31, 2), (32, 1), (700, 1), (1210, 3), (255, 1), (1100, 1), (64, 2)]
    if 8 * 3 * (nq // nkv) * (hd + 2) * 4 > 64 * 1024:
        portions = [(s, 1) for s, _ in portions]  # as many columns of a tile as fit the block's LDS
    case = Case(portions, nq, nkv, hd, 16, torch.bfloat16, 19, window)
    want = case.reference(hd ** -0.5).float()
    got = case.run("mfma", hd ** -0.5, prefill_kernel=False, in_block=True).float()
    assert torch.allclose(got, want, **tol(torch.bfloat16))
    apart = case.run("mfma", hd ** -0.5, prefill_kernel=False, in_block=False).float()
    assert torch.allclose(got, apart, **tol(torch.bfloat16))


def test_paged_attention_mfma_merges_inside_the_block_when_the_tiles_fill_the_machine():
    """Seventy decoded tokens over four key/value heads are 280 tiles: the plan, left to itself, takes the kernel
    that merges in its block; with eight requests it splits the keys over more waves."""
    portions = [(40 + 13 * i, 1) for i in range(70)]
    case = Case(portions, 8, 4, 128, 16, torch.bfloat16, 22, None)
    assert ops.plan_attention_in_block(1, case.step.max_context, 2, None, 128, num_tiles=280) is not None
    assert ops.plan_attention_in_block(1, case.step.max_context, 2, None, 128, num_tiles=32) is None
    want = case.reference(128 ** -0.5).float()
    assert torch.allclose(case.run("mfma", 128 ** -0.5).float(), want, **tol(torch.bfloat16))


def test_paged_attention_mfma_merges_inside_the_block_only_what_fits():
    case = Case([(1700, 1)], 8, 4, 256, 16, torch.bfloat16, 20)  # 54 blocks of 32 keys: seven a wave
    with pytest.raises(ops.KernelError, match="too many to merge inside a block"):
        case.run("mfma", 1.0 / 16, prefill_kernel=False, in_block=True)
    case = Case([(100, 5)], 8, 4, 256, 16, torch.bfloat16, 20)  # ten columns of 256 dimensions from eight waves
    with pytest.raises(ops.KernelError, match="too many to merge inside a block"):
        case.run("mfma", 1.0 / 16, prefill_kernel=False, in_block=True)
    assert ops.plan_attention_in_block(1, 8192, 2, 1024, 256) == (160, 2)  # a decoded token under the 4B model's window
    assert ops.plan_attention_in_block(1, 8192, 2, None, 256) is None


@pytest.mark.parametrize("seed", range(24))
def test_paged_attention_on_batches_drawn_at_random(seed):
    """Head counts, head sizes, pages, windows and the batch itself drawn at random (decoded tokens only, prompts
    only, portions deep in a context, or a mix), through ``ops.paged_attention`` left to its own plans: whichever
    kernels, splits and pieces it takes, the 64-bit reference's output."""
    import random

    rng = random.Random(seed)
    nkv, group = rng.choice([1, 2, 3, 4, 8]), rng.choice([1, 2, 3, 4, 5, 8, 16])
    hd = rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 240, 256])
    page = rng.choice([16, 32, 64])
    window = rng.choice([None, None, 7, 100, 1024])
    kind = rng.choice(["decode", "mixed", "prompts", "deep"])
    portions = []
    for _ in range(rng.randint(1, 10)):
        if kind == "decode":
            portions.append((rng.randint(0, 3000), 1))
        elif kind == "prompts":
            portions.append((rng.choice([0, 0, 17, 500]), rng.randint(1, 300)))
        elif kind == "deep":
            portions.append((rng.randint(1000, 5000), rng.choice([1, 2, 64, 100, 128])))
        else:
            portions.append((rng.randint(0, 2000), rng.choice([1, 1, 1, 2, 3, 40, 64, 65, 130])))
    if sum(s + n for s, n in portions) * nkv * hd > 6e7:
        portions = portions[:2]
    nq = nkv * group
    case = Case(portions, nq, nkv, hd, page, torch.bfloat16, seed, window)
    case.step.host_chunk_start = [s for s, _ in portions]
    case.step.shared = {}
    T = case.q.shape[0]
    out = torch.full((T, nq * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    kp, vp = to_cache(case.k_log, case.v_log)
    ops.paged_attention(dev(case.q.view(T, -1)), kp, vp, dev(case.table), case.step, out, nq, hd ** -0.5, window)
    got = out.cpu().view(T, nq, hd).float()
    assert torch.allclose(got, case.reference(hd ** -0.5).float(), **tol(torch.bfloat16)), (
        f"{nq}:{nkv} heads of {hd}, pages of {page}, window {window}, {kind}: {portions}")


def test_paged_attention_mfma_long_decode_batch():
    """Decode shapes: many requests with one token each at long, different contexts."""
    portions = [(4000 + 37 * i, 1) for i in range(9)]
    for window in (None, 1024):
        case = Case(portions, 8, 4, 256, 16, torch.bfloat16, 11, window)
        want = case.reference(1.0 / 16).float()
        assert torch.allclose(case.run("mfma", 1.0 / 16).float(), want, **tol(torch.bfloat16))


def test_mfma_attention_says_what_it_does_not_cover():
    case = Case([(5, 1)], 34, 2, 32, 16, torch.bfloat16, 12)  # 17 query heads per key/value head
    with pytest.raises(ops.KernelError, match="at most 16 query heads"):
        case.run("mfma", 1.0)
    assert not ops.mfma_attention_covers(*to_cache(case.k_log, case.v_log), 34)


@pytest.mark.parametrize("kernel,dtype", [("generic", torch.float32), ("generic", torch.bfloat16),
                                          ("mfma", torch.bfloat16)])
def test_paged_attention_finds_one_far_key_among_hundreds(kernel, dtype):
    """Random keys hide a wrong mask or table; here one far key carries all
    the weight, so the output is its value exactly."""
    nq, nkv, hd, ctx = 2, 1, 32, 700
    far = 17  # on the second page
    for window, found in ((None, True), (ctx - far, True), (ctx - far - 1, False)):
        # exactly at the window's edge the key is still seen, one further it is not
        case = Case([(ctx - 1, 1)], nq, nkv, hd, 16, dtype, 10, window, drop_passed_pages=False)
        k, v = case.k_all[0], case.v_all[0]
        k *= 0.01
        k[far, 0] = 0
        k[far, 0, 3] = 40.0
        page, slot = int(case.table[0, far // 16]), far % 16
        case.k_log[:] = 0
        for j in range(ctx):
            case.k_log[int(case.table[0, j // 16]), j % 16] = k[j]
        case.q[:] = 0
        case.q[0, :, 3] = 40.0
        got = case.run(kernel, 1.0).float()
        same = torch.allclose(got[0], v[far, 0].float().expand(nq, hd), atol=2e-2 if dtype == torch.bfloat16 else 1e-5)
        assert same == found, (window, found)


@pytest.mark.parametrize("kernel,dtype", [("generic", torch.float32), ("mfma", torch.bfloat16)])
def test_paged_attention_missing_page_shows(kernel, dtype):
    case = Case([(39, 1)], 1, 1, 16, 16, dtype, 11)
    case.table[0, 1] = -1  # a visible page is missing: the result must not look valid
    assert torch.isnan(case.run(kernel, 1.0)).all()


@pytest.mark.parametrize("vocab", [5, 256, 509, 4097, 262208])
def test_argmax(vocab):
    g = torch.Generator().manual_seed(12)
    x = torch.randn(3, vocab, generator=g)
    x[1, vocab // 2] = x[1, vocab - 1] = 50.0  # two equal maxima: the lowest id wins
    x[2, :] = 1.5  # all equal: id 0
    x[0, 0] = float("nan")  # NaN is skipped
    got = ops.argmax(dev(x)).cpu().tolist()
    assert got == [int(torch.nan_to_num(x[0], nan=-1e9).argmax()), vocab // 2, 0]


def test_argmax_golden_rows_of_the_reference():
    # v3/crates/rvllm-invariants/tests/identity.rs:91-128
    assert ops.argmax(dev(torch.tensor([[2.0, 9.0, 4.0, 9.0, 1.0]]))).item() == 1
    assert ops.argmax(dev(torch.tensor([[1.5, 1.5, 1.5, 1.5]]))).item() == 0
    assert ops.argmax(dev(torch.tensor([[0.1, 0.2, 9.9, 0.3], [7.0, 0.0, 1.0, 2.0]]))).cpu().tolist() == [2, 0]


@pytest.mark.parametrize("vocab,k", [(509, 509), (300, 1), (4097, 50), (262208, 1024), (262208, 50), (16385, 1024),
                                     (70001, 64)])  # the row in one part, in 32, in two of which the last is the shorter
def test_topk_select(vocab, k):
    g = torch.Generator().manual_seed(13)
    x = torch.randn(2, vocab, generator=g)
    x[1, : vocab // 2] = 0.25  # many equal values: the lower ids are taken first
    inv_t = torch.tensor([1.0 / 0.8, 2.0])
    vals, idx = ops.topk_select(dev(x), k, dev(inv_t))
    vals, idx = vals.cpu(), idx.cpu().long()
    for r in range(2):
        order = sorted(range(vocab), key=lambda i: (-x[r, i].item(), i))[:k]
        assert sorted(idx[r].tolist()) == sorted(order)
        assert torch.equal(vals[r], x[r][idx[r]] * inv_t[r])


@pytest.mark.parametrize("k", [1, 7, 50, 509, 1024])
def test_the_draw_on_the_device_is_the_hosts(k):
    """The device sorts, weighs, cuts and walks as the host does, with the same stream of numbers: the same tokens
    row by row and draw after draw.  Rows with every kind of cut (all candidates, the first only, a few, a nucleus
    from 0 to 1), equal values among the candidates (the lower id first), values far apart (weights that vanish)
    and both zeros."""
    from rvllm_amd.sampling.sampler import SplitMix64, sample_rows

    rows = 24
    g = torch.Generator().manual_seed(50 + k)
    vals = torch.randn(rows, k, generator=g) * 3
    vals[1] = (vals[1] * 2).round() / 2  # many equal values
    vals[2] = vals[2] * 40  # exp underflows for most
    if k > 2:
        vals[3, :2] = torch.tensor([0.0, -0.0])
    ids = torch.stack([torch.randperm(70000, generator=g)[:k] for _ in range(rows)]).int()
    top_k = [[0, 1, min(k, 5), k][r % 4] for r in range(rows)]
    top_p = [[1.0, 0.9, 0.5, 0.0, 0.999999, 0.3][r % 6] for r in range(rows)]
    seeds = [(0x9E3779B97F4A7C15 * (r + 1)) & ((1 << 64) - 1) for r in range(rows)]
    rngs = [SplitMix64(s) for s in seeds]
    state = dev(torch.tensor([s - (1 << 64) if s >= (1 << 63) else s for s in seeds], dtype=torch.int64))
    d_vals, d_ids = dev(vals), dev(ids)
    d_k, d_p = dev(torch.tensor(top_k, dtype=torch.int32)), dev(torch.tensor(top_p, dtype=torch.float64))
    for draw in range(6):
        want = sample_rows(vals.numpy(), ids.numpy(), top_k, top_p, rngs, 70000)
        got = ops.draw(d_vals, d_ids, d_k, d_p, state).cpu().tolist()
        assert got == want, f"draw {draw}"
    # the streams stand where the host's stand
    assert [s & ((1 << 64) - 1) for s in state.cpu().tolist()] == [r.state for r in rngs]
    # a candidate that is no number: no token, and the stream stays
    vals[0, 0] = float("nan")
    before = state.clone()
    got = ops.draw(dev(vals), d_ids, d_k, d_p, state).cpu().tolist()
    assert got[0] == -1 and all(t >= 0 for t in got[1:]) and state[0] == before[0] and (state[1:] != before[1:]).all()


def test_the_draw_looks_at_a_rows_own_candidates_only():
    """In a batch the device selects for every row as many candidates as the row that asks for most.  Whether a
    row has a token must not depend on who else is in the batch: a row that keeps 3 is judged by its 3 largest
    (a -inf beyond them is nobody's business, one among them is refused as the host refuses it), and a row
    that decodes greedily takes the largest candidate that is a number, as the arg-max does."""
    from rvllm_amd.sampling.sampler import SplitMix64, sample_rows

    k = 8
    vals = torch.tensor([[5.0, 1.0, 3.0, 2.0, float("-inf"), 0.5, 4.0, -1.0],   # keeps 3: -inf lies beyond
                         [5.0, 1.0, float("-inf"), 2.0, 0.0, 0.5, 4.0, -1.0],   # keeps all 8: -inf is among them
                         [float("nan"), 1.0, 7.0, 7.0, 0.0, 0.5, 4.0, -1.0],    # greedy: NaN skipped, 7 twice
                         [float("nan")] * 8,                                    # greedy: nothing is a number
                         [2.0, float("inf"), 3.0, 2.0, 1.0, 0.5, 4.0, -1.0]])   # greedy: +inf is the largest
    ids = torch.tensor([[10, 11, 12, 13, 14, 15, 16, 17]] * 5, dtype=torch.int32)
    ids[2] = torch.tensor([3, 4, 9, 6, 5, 7, 8, 2])  # the two 7s have ids 9 and 6: the lower one
    top_k = torch.tensor([3, 0, -1, -1, -1], dtype=torch.int32)
    top_p = torch.tensor([1.0] * 5, dtype=torch.float64)
    seeds = [11, 12, 13, 14, 15]
    state = dev(torch.tensor(seeds, dtype=torch.int64))
    got = ops.draw(dev(vals), dev(ids), dev(top_k), dev(top_p), state).cpu().tolist()
    want0 = sample_rows(vals[:1, [0, 6, 2]].numpy(), ids[:1, [0, 6, 2]].numpy(), [3], [1.0], [SplitMix64(11)], 100)[0]
    assert got == [want0, -1, 6, -1, 11]
    after = state.cpu().tolist()
    assert after[0] != 11 and after[1:] == seeds[1:]  # only the row that drew moved its stream


def test_kernels_refuse_what_they_cannot_do():
    x = torch.randn(4, 32)
    with pytest.raises(ops.KernelError, match="GPU"):
        ops.rmsnorm(x, torch.zeros(32), 1e-6, 1.0)
    with pytest.raises(ops.KernelError, match="weight"):
        ops.rmsnorm(dev(x), dev(torch.zeros(31)), 1e-6, 1.0)
    with pytest.raises(ops.KernelError, match="dtype"):
        ops.rmsnorm(dev(x.half()), dev(torch.zeros(32)), 1e-6, 1.0)
    with pytest.raises(ops.KernelError, match="inner sizes"):
        ops.gemm_plain(dev(x), dev(torch.randn(8, 31)), torch.empty(4, 8, device=DEV))
    with pytest.raises(ops.KernelError, match="head_dim"):
        hd = 1024
        ops.qk_norm_rope_kv_write(dev(torch.randn(1, 3 * hd)), torch.empty(1, hd, device=DEV), None, None, 0.0, 0.0,
                                  None, 0, dev(torch.zeros(1, dtype=torch.int32)), dev(torch.zeros(1, dtype=torch.int32)),
                                  None, None, None, 1, 1, hd, write_kv=False)
    with pytest.raises(ops.KernelError, match="k="):
        ops.topk_select(dev(torch.randn(1, 5000)), 2000, dev(torch.ones(1)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_consumers_add_up_the_slices_of_a_product(dtype):
    """A product with few rows may hand its K slices to the next kernel
    unreduced; each consumer gives what it gives for the reduced tensor."""
    g = torch.Generator().manual_seed(30)
    slices, rows, width = 5, 7, 96
    part = torch.randn(slices, rows, width, generator=g)
    sums = ops.SlicedSums(dev(part), dtype)
    whole = part.sum(0)
    assert torch.allclose(sums.as_tensor().cpu().float(), whole, **tol(dtype))
    reduced = dev(whole.to(dtype)) if dtype == torch.float32 else None
    # norm + residual add
    w = (torch.randn(width, generator=g) * 0.1).to(dtype)
    res = torch.randn(rows, width, generator=g).to(dtype)
    r1 = dev(res.clone())
    ops.add_rmsnorm(sums, dev(w), 1e-6, 1.0, r1)
    want = res.double() + P.rmsnorm(whole.double(), w.double(), 1e-6)
    assert torch.allclose(r1.cpu().float(), want.float(), **tol(dtype))
    # gated activation
    act = ops.gated_act(sums, "gelu_pytorch_tanh").cpu().float()
    want = F.gelu(whole[:, :48].double(), approximate="tanh") * whole[:, 48:].double()
    assert torch.allclose(act, want.float(), **tol(dtype))
    # q/k norm and rotation: 2 query heads, 2 kv heads of 16
    q_out = torch.empty(rows, 32, dtype=dtype, device=DEV)
    ops.qk_norm_rope_kv_write(sums, q_out, None, None, 0.0, 0.0, None, 0, dev(torch.arange(rows, dtype=torch.int32)),
                              dev(torch.zeros(rows, dtype=torch.int32)), None, None, None, 2, 2, 16, write_kv=False)
    assert torch.allclose(q_out.cpu().float(), whole[:, :32], **tol(dtype))
    if dtype == torch.float32:  # in 32-bit the sliced and the reduced input give the same bits
        r2 = dev(res.clone())
        ops.add_rmsnorm(reduced, dev(w), 1e-6, 1.0, r2)
        assert torch.equal(r1, r2)


def test_sliced_product_through_the_skinny_kernel():
    g = torch.Generator().manual_seed(31)
    x, w = torch.randn(8, 2048, generator=g).bfloat16(), (torch.randn(2560, 2048, generator=g) * 0.05).bfloat16()
    got = ops.gemm_bf16(dev(x), dev(w), sliced_ok=True)
    assert isinstance(got, ops.SlicedSums) and got.slices > 1 and got.shape == (8, 2560)
    want = x.double() @ w.double().T
    assert torch.allclose(got.as_tensor().cpu().double(), want, atol=3e-2, rtol=2e-2)
    assert torch.allclose(got.data.sum(0).cpu().double(), want, atol=1e-3, rtol=1e-4)


def test_sampler_at_a_large_vocabulary_draws_what_one_row_alone_draws():
    """Rows that are greedy, that sample with different temperatures, cuts and seeds, and rows with many equal
    logits, over a vocabulary that the selection cuts into 32 parts: each row's token is the one that the single
    row's draw gives from that row's exact top candidates."""
    from rvllm_amd.sampling.params import SamplingParams
    from rvllm_amd.sampling.sampler import Sampler, SplitMix64, sample_from_candidates

    vocab = 262208
    g = torch.Generator().manual_seed(23)
    logits = torch.randn(7, vocab, generator=g) * 2.0
    logits[3] = torch.round(logits[3])       # many equal values: lower ids first among them
    logits[5, 1000:200000] = 3.5
    params = [SamplingParams(), SamplingParams(0.8, 50, 1.0, seed=1), SamplingParams(1.3, 50, 0.9, seed=2),
              SamplingParams(0.7, 7, 0.5, seed=3), SamplingParams(1.0, 1024, 0.95, seed=4),
              SamplingParams(0.9, 50, 1.0, seed=5), SamplingParams(0.8, 50, 0.0, seed=6)]
    sampler = Sampler(vocab)
    for trial in range(3):
        rngs = [SplitMix64(100 * trial + i) for i in range(7)]
        got = sampler.sample(dev(logits), params, rngs)
        for r, p in enumerate(params):
            row = logits[r]
            if p.is_greedy():
                assert got[r] == int(row.argmax())
                continue
            k = p.kernel_k(vocab)
            order = sorted(range(vocab), key=lambda i: (-row[i].item(), i))[:k] if r in (3, 5) else \
                torch.topk(row, k).indices.tolist()
            cands = [((row[i] * torch.tensor(1.0 / p.temperature)).item(), i) for i in order]
            want = sample_from_candidates(cands, p.top_k, p.top_p, SplitMix64(100 * trial + r), vocab)
            assert got[r] == want, (trial, r)
