"""Each kernel alone against its plain reference, at other sizes than the tiny models use."""
import math
import os

import numpy as np
import pytest
import torch

import plain_model as pm

pytestmark = pytest.mark.gpu
DT = [torch.float32, torch.bfloat16]


def K():
    from prelude_amd.ops import kernels
    return kernels


def tol(dtype, ref, f32=2e-6, bf16=1e-2):
    return (f32 if dtype == torch.float32 else bf16) * max(1.0, float(ref.abs().max()))


def close(got, ref, dtype, **kw):
    err = float((got.double().cpu() - ref.double().cpu()).abs().max())
    assert err <= tol(dtype, ref, **kw), f"max error {err:.3e} > {tol(dtype, ref, **kw):.3e}"


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(*shape, generator=g)).to(dtype)


# ---- embedding, gather ----------------------------------------------------------
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("vocab,hidden", [(509, 96), (1000, 2560), (37, 7)])
def test_embed_gather(gpu, dtype, vocab, hidden):
    table = rnd(vocab, hidden, dtype=dtype)
    ids = torch.tensor([0, vocab - 1, 3, 3, vocab // 2], dtype=torch.int32)
    out = K().embed_gather(ids.to(gpu), table.to(gpu))
    assert torch.equal(out.cpu(), table[ids.long()])


@pytest.mark.parametrize("dtype", DT)
def test_gather_rows(gpu, dtype):
    x = rnd(40, 130, dtype=dtype)
    rows = torch.tensor([39, 0, 7, 7], dtype=torch.int32)
    assert torch.equal(K().gather_rows(x.to(gpu), rows.to(gpu)).cpu(), x[rows.long()])


# ---- norms --------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("rows,hidden,eps", [(5, 2560, 1e-6), (3, 100, 1e-5), (2, 7, 3e-6), (9, 4096, 1e-6), (1, 513, 1e-6)])
def test_rmsnorm(gpu, dtype, rows, hidden, eps):
    x = rnd(rows, hidden, dtype=dtype, scale=3.0)
    w = 1.0 + 0.1 * rnd(hidden, seed=1)
    ref = pm.rms_norm(x.double(), w.double(), eps)
    close(K().rmsnorm(x.to(gpu), w.to(gpu), eps), ref, dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("rows,hidden", [(6, 2560), (4, 96), (3, 1000)])
def test_add_rmsnorm(gpu, dtype, rows, hidden):
    # crates/prelude-core/tests/modules.rs:275-314: the sum is returned, the norm is of the unrounded sum
    x, res = rnd(rows, hidden, dtype=dtype), rnd(rows, hidden, dtype=dtype, seed=2, scale=4.0)
    w = 1.0 + 0.1 * rnd(hidden, seed=1)
    s = x.double() + res.double()
    r_dev = res.to(gpu).clone()
    out = K().rmsnorm(x.to(gpu), w.to(gpu), 1e-6, residual=r_dev)
    close(out, pm.rms_norm(s, w.double(), 1e-6), dtype)
    assert torch.equal(r_dev.cpu(), s.to(dtype))             # the residual holds the sum, rounded once
    # rows variant: compact output, residual untouched
    rows_idx = torch.tensor([rows - 1, 0], dtype=torch.int32)
    r2 = res.to(gpu).clone()
    out2 = K().rmsnorm(x.to(gpu), w.to(gpu), 1e-6, residual=r2, rows=rows_idx.to(gpu))
    close(out2, pm.rms_norm(s[rows_idx.long()], w.double(), 1e-6), dtype)
    assert torch.equal(r2.cpu(), res)


def test_rmsnorm_reference_vector(gpu):
    x = torch.tensor([[3.0, 4.0]])
    out = K().rmsnorm(x.to(gpu), torch.ones(2).to(gpu), 1e-6).cpu()
    assert torch.allclose(out, x / math.sqrt(12.5 + 1e-6), atol=1e-6)


# ---- SiLU * up ----------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("tokens,inter", [(3, 9728), (5, 160), (2, 7), (37, 1000), (4, 12)])
def test_silu_mul(gpu, dtype, tokens, inter):
    gu = rnd(tokens, 2 * inter, dtype=dtype, scale=3.0)
    ref = pm.silu(gu[:, 0::2].double()) * gu[:, 1::2].double()
    close(K().silu_mul(gu.to(gpu)), ref, dtype)


def test_silu_mul_reference_vector(gpu):
    g = torch.tensor([0.0, 1.0, -1.0, 2.0, -2.0, 0.5])
    u = torch.tensor([1.0, 2.0, 3.0, 0.5, 1.0, 4.0])
    out = K().silu_mul(torch.stack([g, u], dim=1).reshape(1, 12).to(gpu)).cpu()[0]
    assert torch.allclose(out, torch.nn.functional.silu(g) * u, atol=1e-6) and float(out[0]) == 0.0


# ---- matrix product ---------------------------------------------------------------------------
@pytest.mark.parametrize("m,n,k", [(1, 509, 96), (33, 70, 45), (64, 64, 16), (130, 257, 160), (7, 2560, 2560)])
def test_gemm_plain_f32(gpu, m, n, k):
    x, w, b = rnd(m, k), rnd(n, k, seed=1), rnd(n, seed=2)
    ref = x.double() @ w.double().T + b.double()
    out = K().gemm_plain(x.to(gpu), w.to(gpu), b.to(gpu))
    close(out, ref, torch.float32, f32=2e-6 * math.sqrt(k))
    # a row's result does not depend on the other rows of the batch
    one = K().gemm_plain(x[m // 2: m // 2 + 1].to(gpu), w.to(gpu), b.to(gpu))
    assert torch.equal(one[0], out[m // 2])


def test_gemm_plain_f32_sums_long_rows_without_drift(gpu):
    """A row of 9,728 terms (the widest inner size of the 4B shape): the sixteens are added with a compensated sum,
    which keeps the error near 1e-7 of the largest output; a plain running sum in 32-bit is off by some 4e-6 there
    and would fail this.  All terms of one sign, so that rounding cannot cancel."""
    m, n, k = 4, 96, 9728
    x, w = rnd(m, k).abs(), rnd(n, k, seed=1).abs()
    ref = x.double() @ w.double().T
    out = K().gemm_plain(x.to(gpu), w.to(gpu))
    err = float((out.double().cpu() - ref).abs().max()) / float(ref.abs().max())
    assert err < 4e-7, f"relative error {err:.2e} of the largest output"


@pytest.mark.parametrize("m,n,k", [(1, 509, 96), (8, 2560, 4096), (40, 331, 80), (300, 192, 96), (64, 6144, 2560)])
def test_linear_bf16(gpu, m, n, k):
    x, w, b = rnd(m, k, dtype=torch.bfloat16), rnd(n, k, dtype=torch.bfloat16, seed=1, scale=0.05), rnd(n, seed=2)
    ref = x.double() @ w.double().T
    close(K().linear(x.to(gpu), w.to(gpu)), ref, torch.bfloat16)
    close(K().linear(x.to(gpu), w.to(gpu), b.to(gpu)), ref + b.double(), torch.bfloat16)
    out32 = K().linear(x.to(gpu), w.to(gpu), out_dtype=torch.float32)
    assert out32.dtype == torch.float32
    close(out32, ref, torch.bfloat16)
    close(K().gemm_plain(x.to(gpu), w.to(gpu), out_dtype=torch.float32), ref, torch.float32, f32=1e-5)


@pytest.mark.parametrize("m,n,k", [(1, 2560, 4096), (8, 6144, 2560), (8, 2560, 9728), (13, 509, 96), (16, 331, 80),
                                   (17, 64, 64), (33, 192, 160), (24, 9728, 2560), (32, 200, 72), (64, 2560, 2560), (5, 19456, 2560), (2, 40, 8),
                                   (3, 151936, 256), (40, 336, 8256), (64, 4112, 8192), (9, 48, 8320),
                                   # the launch shapes that only the weights of larger models reach: 320 tiles or more with
                                   # rows of 128 steps or more (eight wavefronts on two tiles, or on one for few short rows)
                                   (8, 5120, 25600), (1, 5120, 8192), (5, 5120, 8192), (16, 5120, 5120), (24, 24576, 4096)])
def test_gemm_skinny(gpu, m, n, k):
    x, w, b = rnd(m, k, dtype=torch.bfloat16), rnd(n, k, dtype=torch.bfloat16, seed=1, scale=0.05), rnd(n, seed=2)
    ref = x.double() @ w.double().T
    xd, wd = x.to(gpu), w.to(gpu)
    close(K().gemm_skinny(xd, wd, out_dtype=torch.float32), ref, torch.float32, f32=2e-5)
    close(K().gemm_skinny(xd, wd), ref, torch.bfloat16)
    close(K().gemm_skinny(xd, wd, b.to(gpu), out_dtype=torch.float32), ref + b.double(), torch.float32, f32=2e-5)
    # a row's result does not depend on how many rows there are (same weight, same split of K)
    full = K().gemm_skinny(xd, wd, out_dtype=torch.float32)
    one = K().gemm_skinny(xd[m - 1:].contiguous(), wd, out_dtype=torch.float32)
    assert torch.equal(one[0], full[m - 1])
    if n % 2 == 0:
        act = K().gemm_skinny(xd, wd, silu_mul_epilogue=True)
        close(act, pm.silu(ref[:, 0::2]) * ref[:, 1::2], torch.bfloat16)
        close(K().linear_silu_mul(xd, wd), pm.silu(ref[:, 0::2]) * ref[:, 1::2], torch.bfloat16)
    # the weight in tiles (few rows only): the same product, with a split of K of its own
    tiles = K().pack_tiles(wd)
    if m <= 16:
        tiled = K().gemm_skinny(xd, tiles, out_dtype=torch.float32)
        close(tiled, ref, torch.float32, f32=2e-5)
        close(K().gemm_skinny(xd, tiles, b.to(gpu)), ref + b.double(), torch.bfloat16)
        assert torch.equal(K().gemm_skinny(xd[m - 1:].contiguous(), tiles, out_dtype=torch.float32)[0], tiled[m - 1])
        lw = K().LinearWeight(wd, tiles)
        assert torch.equal(K().linear(xd, lw, out_dtype=torch.float32), tiled)
        if n % 2 == 0:
            tact = K().gemm_skinny(xd, tiles, silu_mul_epilogue=True)
            close(tact, pm.silu(ref[:, 0::2]) * ref[:, 1::2], torch.bfloat16)
            # the dispatcher's choice between this kernel and the one with X in LDS follows the shape and the rows
            got = K().linear_silu_mul(xd, lw)
            assert torch.equal(got, tact) or torch.equal(got, K().gemm_mid(xd, tiles, silu_mul_epilogue=True))
            close(got, pm.silu(ref[:, 0::2]) * ref[:, 1::2], torch.bfloat16)
    else:                                # more rows from tiles: the same sums per row as with few rows
        many = K().gemm_skinny(xd, tiles, out_dtype=torch.float32)
        close(many, ref, torch.float32, f32=2e-5)
        # (rows of 8,192 columns or more are summed over 8 wavefronts instead of 16 when there are more than 16 rows)
        fewer = 1 if k < 8192 else 17
        assert torch.equal(K().gemm_skinny(xd[m - fewer:].contiguous(), tiles, out_dtype=torch.float32)[fewer - 1], many[m - 1])
        close(K().linear(xd, K().LinearWeight(wd, tiles)), ref, torch.bfloat16)
        if n % 2 == 0:   # up to 32 rows the gated product stays in the streaming kernel, beyond it is the library's
            close(K().linear_silu_mul(xd, K().LinearWeight(wd, tiles)), pm.silu(ref[:, 0::2]) * ref[:, 1::2],
                  torch.bfloat16, bf16=1.25e-2)


@pytest.mark.parametrize("m,n,k,slices", [(64, 2560, 4096, 8), (33, 331, 1000, 1), (128, 200, 4096, 4), (7, 2560, 9728, 8),
                                          (17, 6144, 2560, 2), (100, 48, 520, 1), (48, 256, 1024, 2), (1, 64, 64, 1),
                                          (80, 36, 72, 1), (96, 132, 1288, 2), (20, 2560, 4096, 8)])
def test_gemm_mid(gpu, m, n, k, slices):
    """The product with X staged in LDS (up to 128 rows, weight in tiles): whole, and cut into slices of the inner
    size whose 32-bit partial sums the reader adds -- the residual add + RMSNorm as it loads them, or sum_slices."""
    x, w, b = rnd(m, k, dtype=torch.bfloat16), rnd(n, k, dtype=torch.bfloat16, seed=1, scale=0.05), rnd(n, seed=2)
    ref = x.double() @ w.double().T
    xd, bd = x.to(gpu), b.to(gpu)
    tiles = K().pack_tiles(w.to(gpu))
    full = K().gemm_mid(xd, tiles, out_dtype=torch.float32)
    close(full, ref, torch.float32, f32=2e-5)
    close(K().gemm_mid(xd, tiles), ref, torch.bfloat16)
    close(K().gemm_mid(xd, tiles, bd, out_dtype=torch.float32), ref + b.double(), torch.float32, f32=2e-5)
    # a row's result does not depend on how many rows there are
    assert torch.equal(K().gemm_mid(xd[m - 1:].contiguous(), tiles, out_dtype=torch.float32)[0], full[m - 1])
    if n % 2 == 0:
        close(K().gemm_mid(xd, tiles, silu_mul_epilogue=True), pm.silu(ref[:, 0::2]) * ref[:, 1::2], torch.bfloat16)
    if slices > 1:
        ss = K().gemm_mid(xd, tiles, bd, slices=slices)
        assert isinstance(ss, K().SliceSums) and tuple(ss.parts.shape) == (slices, m, n) and ss.dtype == torch.bfloat16
        whole = ss.parts.double().sum(0).cpu()
        close(whole, ref + b.double(), torch.float32, f32=2e-5)
        close(ss.materialize(), ref + b.double(), torch.bfloat16)
        # the norm adds the slices itself: residual + product in 32-bit, the residual rounded once, the norm of the unrounded sum
        weight, res = 1 + 0.1 * rnd(n, seed=3), rnd(m, n, dtype=torch.bfloat16, seed=4)
        resd = res.to(gpu)
        normed = K().rmsnorm(ss, weight.to(gpu), 1e-5, residual=resd)
        total = whole + res.double()
        close(resd, total, torch.bfloat16)
        close(normed, pm.rms_norm(total, weight.double(), 1e-5), torch.bfloat16)
        rows = torch.tensor([m - 1, 0], dtype=torch.int32)
        picked = K().rmsnorm(ss, weight.to(gpu), 1e-5, residual=res.to(gpu), rows=rows.to(gpu))
        close(picked, pm.rms_norm(total[rows.long()], weight.double(), 1e-5), torch.bfloat16)
    # what lies behind X is not the product's to read: NaN there must not show
    behind = torch.full((m + 8, k), float("nan"), dtype=torch.bfloat16, device=gpu)
    behind[:m] = xd
    got = K().gemm_mid(behind[:m], tiles, out_dtype=torch.float32)
    assert bool(torch.isfinite(got).all()) and torch.equal(got, full)
    # how many wavefronts share a workgroup (which the launcher picks by the weight's shape) changes no bit
    for waves in (3, 4, 5, 6, 8):
        assert torch.equal(K().gemm_mid(xd, tiles, out_dtype=torch.float32, waves=waves), full), f"{waves} wavefronts"
        if slices > 1:
            assert torch.equal(K().gemm_mid(xd, tiles, bd, slices=slices, waves=waves).parts, ss.parts), f"{waves} wavefronts, slices"


@pytest.mark.parametrize("m,n,k,eps", [(8, 19456, 2560, 1e-6), (1, 64, 64, 1e-5), (16, 200, 4096, 1e-6), (5, 330, 1000, 3e-4),
                                       (13, 36, 72, 1e-6), (9, 1288, 520, 1e-2), (3, 6144, 1024, 1e-6), (16, 512, 256, 1e-6)])
def test_gated_product_behind_its_norm(gpu, m, n, k, eps):
    """Residual add, RMSNorm and gated product in one kernel: the new residual is the sum rounded once, the norm is
    taken of the unrounded sum, and the product is that of the two kernels apart."""
    x, res = rnd(m, k, dtype=torch.bfloat16, scale=0.7), rnd(m, k, dtype=torch.bfloat16, seed=5, scale=3.0)
    res[m - 1] *= 40.0          # a row far larger than the others: every row has a scale of its own
    gain = 1 + 0.3 * rnd(k, seed=3)
    w = rnd(n, k, dtype=torch.bfloat16, seed=1, scale=0.05)
    total = x.double() + res.double()
    h = pm.rms_norm(total, gain.double(), eps)
    g = h @ w.double().T
    ref = pm.silu(g[:, 0::2]) * g[:, 1::2]
    lw = K().LinearWeight(w.to(gpu), K().pack_tiles(w.to(gpu)))
    xd, resd, gd = x.to(gpu), res.to(gpu), gain.to(gpu)
    # the block takes it where it measured faster than the two kernels apart: weights of 40 M elements and more
    assert K().gated_after_norm_supported(xd, resd, lw) == (n * k >= 40 << 20)
    new_res, y = K().linear_gated_after_norm(xd, resd, gd, eps, lw)
    assert torch.equal(resd.cpu(), res) and torch.equal(xd.cpu(), x)          # the inputs stay as they were
    assert torch.equal(new_res.cpu(), (x.float() + res.float()).to(torch.bfloat16))
    close(y, ref, torch.bfloat16, bf16=1.25e-2)
    # beside the two kernels apart: the same residual, a product within rounding of it
    apart_res = resd.clone()
    apart = K().linear_gated(K().rmsnorm(xd, gd, eps, residual=apart_res), lw)
    assert torch.equal(apart_res, new_res)
    close(y, apart.double().cpu(), torch.bfloat16, bf16=1.25e-2)
    # a row's result depends neither on the other rows nor on how many wavefronts share a workgroup
    one_res, one = K().linear_gated_after_norm(xd[m - 1:].contiguous(), resd[m - 1:].contiguous(), gd, eps, lw)
    assert torch.equal(one[0], y[m - 1]) and torch.equal(one_res[0], new_res[m - 1])
    for waves in (3, 4, 5, 6, 8):
        r2, y2 = K().linear_gated_after_norm(xd, resd, gd, eps, lw, waves=waves)
        assert torch.equal(y2, y) and torch.equal(r2, new_res), f"{waves} wavefronts"
    # what lies behind the rows is not the kernel's to read: NaN there must not show
    behind_x = torch.full((m + 8, k), float("nan"), dtype=torch.bfloat16, device=gpu)
    behind_r = torch.full((m + 8, k), float("nan"), dtype=torch.bfloat16, device=gpu)
    behind_x[:m], behind_r[:m] = xd, resd
    r3, y3 = K().linear_gated_after_norm(behind_x[:m], behind_r[:m], gd, eps, lw)
    assert torch.equal(y3, y) and torch.equal(r3, new_res)
    # the other activation, and what it does not take
    import torch.nn.functional as F
    _, y4 = K().linear_gated_after_norm(xd, resd, gd, eps, lw, "gelu_tanh")
    close(y4, F.gelu(g[:, 0::2], approximate="tanh") * g[:, 1::2], torch.bfloat16, bf16=1.25e-2)
    assert not K().gated_after_norm_supported(torch.zeros(17, k, dtype=torch.bfloat16, device=gpu),
                                              torch.zeros(17, k, dtype=torch.bfloat16, device=gpu), lw)
    assert not K().gated_after_norm_supported(xd.float(), resd.float(), lw)
    from prelude_amd._native import NativeError
    with pytest.raises(NativeError, match="buffer of its own"):
        K().check(K().kernels().pa_gemm_mid_normed(None, 1, xd.data_ptr(), resd.data_ptr(), gd.data_ptr(), eps, resd.data_ptr(),
                                                   lw.tiles.data.data_ptr(), y.data_ptr(), m, n, k, k, n // 2, 0))


@pytest.mark.parametrize("m,n,k,slices", [(129, 2560, 4096, 4), (300, 331, 1000, 1), (256, 200, 4096, 2), (513, 2560, 2560, 1),
                                          (192, 6144, 2560, 4), (1030, 72, 640, 1), (260, 1000, 2560, 1), (140, 36, 72, 1),
                                          (576, 2560, 9728, 4), (2, 64, 64, 1)])
def test_gemm_tall(gpu, m, n, k, slices):
    """The product tiled both ways (any number of rows, weight in tiles): whole, with bias, with the gated
    activation in its epilogue, and cut into slices whose 32-bit partial sums the reader adds; at every shape of
    workgroup the same bits, and a row's result whatever the other rows are."""
    x, w, b = rnd(m, k, dtype=torch.bfloat16), rnd(n, k, dtype=torch.bfloat16, seed=1, scale=0.05), rnd(n, seed=2)
    ref = x.double() @ w.double().T
    xd, bd = x.to(gpu), b.to(gpu)
    tiles = K().pack_tiles(w.to(gpu))
    full = K().gemm_tall(xd, tiles)
    close(full, ref, torch.bfloat16)
    close(K().gemm_tall(xd, tiles, bd), ref + b.double(), torch.bfloat16)
    # a row's result does not depend on how many rows there are, nor on which row of a tile it is
    lone = K().gemm_tall(xd[m - 1:].contiguous(), tiles)
    assert torch.equal(lone[0], full[m - 1])
    if m > 70:
        part = K().gemm_tall(xd[37: 37 + 33].contiguous(), tiles)
        assert torch.equal(part, full[37: 37 + 33])
    gated = None
    if n % 2 == 0:
        gated = K().gemm_tall(xd, tiles, silu_mul_epilogue=True)
        close(gated, pm.silu(ref[:, 0::2]) * ref[:, 1::2], torch.bfloat16)
    ss = None
    if slices > 1:
        ss = K().gemm_tall(xd, tiles, bd, slices=slices)
        assert isinstance(ss, K().SliceSums) and tuple(ss.parts.shape) == (slices, m, n) and ss.dtype == torch.bfloat16
        whole = ss.parts.double().sum(0).cpu()
        close(whole, ref + b.double(), torch.float32, f32=2e-5)
        close(ss.materialize(), ref + b.double(), torch.bfloat16)
        weight, res = 1 + 0.1 * rnd(n, seed=3), rnd(m, n, dtype=torch.bfloat16, seed=4)
        resd = res.to(gpu)
        normed = K().rmsnorm(ss, weight.to(gpu), 1e-5, residual=resd)
        total = whole + res.double()
        close(resd, total, torch.bfloat16)
        close(normed, pm.rms_norm(total, weight.double(), 1e-5), torch.bfloat16)
    # what lies behind X is not the product's to read: NaN there must not show
    behind = torch.full((m + 8, k), float("nan"), dtype=torch.bfloat16, device=gpu)
    behind[:m] = xd
    got = K().gemm_tall(behind[:m], tiles)
    assert bool(torch.isfinite(got.float()).all()) and torch.equal(got, full)
    # the workgroup's shape (which the launcher picks by the product's size) changes no bit
    for shape in ((4, 2), (4, 3), (8, 2), (8, 3)):
        assert torch.equal(K().gemm_tall(xd, tiles, shape=shape), full), shape
        if gated is not None:
            assert torch.equal(K().gemm_tall(xd, tiles, silu_mul_epilogue=True, shape=shape), gated), shape
        if ss is not None:
            assert torch.equal(K().gemm_tall(xd, tiles, bd, slices=slices, shape=shape).parts, ss.parts), shape


def test_gemm_tall_refuses_and_is_dispatched(gpu):
    from prelude_amd._native import NativeError
    w = rnd(2560, 4096, dtype=torch.bfloat16, seed=1, scale=0.05).to(gpu)
    tiles = K().pack_tiles(w)
    x = rnd(256, 4096, dtype=torch.bfloat16).to(gpu)
    with pytest.raises(NativeError, match="in tiles"):
        K().gemm_tall(x, w)
    with pytest.raises(NativeError, match="do not cut into"):
        K().gemm_tall(x, tiles, slices=60)
    with pytest.raises(NativeError, match="no kernel of"):
        K().gemm_tall(x, tiles, shape=(5, 2))
    with pytest.raises(NativeError, match="no bias"):
        K().gemm_tall(x, tiles, torch.zeros(2560, device=gpu), silu_mul_epilogue=True)
    # a wide output whose reader adds slices gets them beyond 128 rows too; a narrow one, and a reader that wants a
    # tensor, the library's product
    ww = rnd(4096, 4096, dtype=torch.bfloat16, seed=3, scale=0.05).to(gpu)
    lww = K().LinearWeight(ww, K().pack_tiles(ww))
    got = K().linear(x, lww, slices_ok=True)
    assert isinstance(got, K().SliceSums) and got.parts.shape[0] == 4
    close(K().as_tensor(got), x.double().cpu() @ ww.double().cpu().T, torch.bfloat16)
    assert isinstance(K().linear(x, lww), torch.Tensor)
    assert isinstance(K().linear(x, K().LinearWeight(w, tiles), slices_ok=True), torch.Tensor)
    tall = rnd(700, 4096, dtype=torch.bfloat16, seed=5).to(gpu)
    assert isinstance(K().linear(tall, lww, slices_ok=True), torch.Tensor)                  # beyond the rows it is ahead for
    # the gated product of short rows: the activation in the epilogue, the same bits as asked for directly
    wg = rnd(1024, 2560, dtype=torch.bfloat16, seed=6, scale=0.05).to(gpu)
    lg = K().LinearWeight(wg, K().pack_tiles(wg))
    xg = rnd(200, 2560, dtype=torch.bfloat16, seed=7).to(gpu)
    assert torch.equal(K().linear_silu_mul(xg, lg), K().gemm_tall(xg, lg.tiles, silu_mul_epilogue=True))
    K().set_tall_products(False)
    try:
        off = K().linear_silu_mul(xg, lg)
        assert isinstance(K().linear(x, lww, slices_ok=True), torch.Tensor)
    finally:
        K().set_tall_products(True)
    g = xg.double().cpu() @ wg.double().cpu().T
    close(off, pm.silu(g[:, 0::2]) * g[:, 1::2], torch.bfloat16)
    close(K().linear_silu_mul(xg, lg), pm.silu(g[:, 0::2]) * g[:, 1::2], torch.bfloat16)


def test_dispatch_of_large_weights(gpu):
    """Where the dispatcher sends the products of very large weights at few rows, each against the product in 32-bit
    on the CPU: a weight of 40 M elements whose reader wants a tensor at 9 to 16 rows (the product with X in LDS,
    uncut), rows of 16,384 columns for a reader of slices from 8 rows on, and the gated product of a weight between
    128 M and 200 M elements up to 96 rows (X in LDS, activation in the epilogue) and beyond (the library)."""
    g = torch.Generator().manual_seed(11)
    def weight(n, k):
        return (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16)
    def rows(m, k):
        return torch.randn(m, k, generator=g).to(torch.bfloat16)
    # a reader of tensors, 12 rows
    w = weight(10240, 4096)
    lw = K().LinearWeight(w.to(gpu), K().pack_tiles(w.to(gpu)))
    x = rows(12, 4096)
    got = K().linear(x.to(gpu), lw)
    assert isinstance(got, torch.Tensor) and torch.equal(got, K().gemm_mid(x.to(gpu), lw.tiles))
    close(got, x.float() @ w.float().T, torch.bfloat16)
    del lw
    # long rows, a reader of slices, 8 rows
    w = weight(2560, 16384)
    lw = K().LinearWeight(w.to(gpu), K().pack_tiles(w.to(gpu)))
    x = rows(8, 16384)
    got = K().linear(x.to(gpu), lw, slices_ok=True)
    assert isinstance(got, K().SliceSums)
    close(K().as_tensor(got), x.float() @ w.float().T, torch.bfloat16)
    assert isinstance(K().linear(x[:7].contiguous().to(gpu), lw, slices_ok=True), torch.Tensor)
    del lw
    # the gated product of a very large weight
    w = weight(26624, 5120)
    lw = K().LinearWeight(w.to(gpu), K().pack_tiles(w.to(gpu)))
    for m in (20, 96, 100):
        x = rows(m, 5120)
        ref = x.float() @ w.float().T
        want = pm.silu(ref[:, 0::2].double()) * ref[:, 1::2].double()
        got = K().linear_gated(x.to(gpu), lw)
        if m <= 96:
            assert torch.equal(got, K().gemm_mid(x.to(gpu), lw.tiles, silu_mul_epilogue=True))
            close(got, want, torch.bfloat16)
        else:   # gate and up rounded to bfloat16 by the library before the activation
            close(got, want, torch.bfloat16, bf16=1.25e-2)


def test_gemm_mid_refuses_and_is_dispatched(gpu):
    from prelude_amd._native import NativeError
    w = rnd(2560, 4096, dtype=torch.bfloat16, seed=1, scale=0.05).to(gpu)
    tiles = K().pack_tiles(w)
    with pytest.raises(NativeError, match="exceed 128"):
        K().gemm_mid(torch.zeros(129, 4096, dtype=torch.bfloat16, device=gpu), tiles)
    with pytest.raises(NativeError, match="do not cut into"):
        K().gemm_mid(torch.zeros(8, 4096, dtype=torch.bfloat16, device=gpu), tiles, slices=60)
    with pytest.raises(NativeError, match="in tiles"):
        K().gemm_mid(torch.zeros(8, 4096, dtype=torch.bfloat16, device=gpu), w)
    with pytest.raises(NativeError, match="7 wavefronts"):
        K().gemm_mid(torch.zeros(8, 4096, dtype=torch.bfloat16, device=gpu), tiles, waves=7)
    # linear() hands a narrow weight at 17 to 128 rows to it in slices only when the caller's reader adds slices
    lw = K().LinearWeight(w, tiles)
    x = rnd(40, 4096, dtype=torch.bfloat16).to(gpu)
    assert isinstance(K().linear(x, lw), torch.Tensor)
    got = K().linear(x, lw, slices_ok=True)
    assert isinstance(got, K().SliceSums) and got.parts.shape[0] == K().gemm_mid_slices(2560, 4096) == 4
    close(K().as_tensor(got), x.double().cpu() @ w.double().cpu().T, torch.bfloat16)
    assert isinstance(K().linear(x[:8].contiguous(), lw, slices_ok=True), torch.Tensor)      # few rows: the streaming kernel
    assert isinstance(K().linear(x.float(), w.float(), slices_ok=True), torch.Tensor)      # 32-bit: the plain product
    # a large weight whose reader wants a tensor: the slices and a kernel that adds them, the same bits as asked for
    # directly; a small weight stays with the streaming kernel up to 64 rows
    wl = (torch.randn(10240, 5120, generator=torch.Generator().manual_seed(8)) * 0.03).to(torch.bfloat16).to(gpu)
    ll = K().LinearWeight(wl, K().pack_tiles(wl))
    xl = rnd(56, 5120, dtype=torch.bfloat16, seed=9).to(gpu)
    got = K().linear(xl, ll)
    assert torch.equal(got, K().gemm_mid(xl, ll.tiles, slices=K().gemm_mid_slices(10240, 5120)).materialize())
    close(got, xl.double().cpu() @ wl.double().cpu().T, torch.bfloat16)
    ws = rnd(4096, 1024, dtype=torch.bfloat16, seed=10, scale=0.05).to(gpu)
    ls = K().LinearWeight(ws, K().pack_tiles(ws))
    xs = rnd(64, 1024, dtype=torch.bfloat16, seed=11).to(gpu)
    assert torch.equal(K().linear(xs, ls), K().gemm_skinny(xs, ls.tiles))
    # the gated product beyond 16 rows: activation in this kernel's epilogue (the same bits as asked for directly)
    wg = rnd(1216, 520, dtype=torch.bfloat16, seed=5, scale=0.05).to(gpu)
    lg = K().LinearWeight(wg, K().pack_tiles(wg))
    xg = rnd(40, 520, dtype=torch.bfloat16, seed=6).to(gpu)
    assert torch.equal(K().linear_silu_mul(xg, lg), K().gemm_mid(xg, lg.tiles, silu_mul_epilogue=True))
    K().set_mid_products(False)
    try:
        other = K().linear_silu_mul(xg, lg)
    finally:
        K().set_mid_products(True)
    ref = xg.double().cpu() @ wg.double().cpu().T
    close(other, pm.silu(ref[:, 0::2]) * ref[:, 1::2], torch.bfloat16, bf16=1.25e-2)
    close(K().linear_silu_mul(xg, lg), pm.silu(ref[:, 0::2]) * ref[:, 1::2], torch.bfloat16, bf16=1.25e-2)


@pytest.mark.parametrize("m,n,k,slices", [(8, 2560, 9728, 3), (1, 1024, 3072, 4), (16, 1024, 2048, 4), (5, 200, 520, 2),
                                          (3, 2048, 6144, 2), (12, 331, 1000, 5), (7, 48, 72, 2)])
def test_gemm_skinny_in_slices(gpu, m, n, k, slices):
    """The streaming product of up to 16 rows with K cut into slices, a workgroup a tile and slice, left as 32-bit
    partial sums: their sum against 64-bit, the bias in the first slice, through the norm that adds them."""
    x, w, b = rnd(m, k, dtype=torch.bfloat16), rnd(n, k, dtype=torch.bfloat16, seed=1, scale=0.05), rnd(n, seed=2)
    ref = x.double() @ w.double().T
    xd, bd = x.to(gpu), b.to(gpu)
    tiles = K().pack_tiles(w.to(gpu))
    ss = K().gemm_skinny_sliced(xd, tiles, bd, slices=slices)
    steps = -(-k // 64)
    made = -(-steps // -(-steps // slices))
    assert isinstance(ss, K().SliceSums) and tuple(ss.parts.shape) == (made, m, n) and ss.dtype == torch.bfloat16
    close(ss.parts.double().sum(0), ref + b.double(), torch.float32, f32=2e-5)
    close(ss.parts[1:].double().sum(0), (x[:, 64 * -(-steps // slices):].double() @ w[:, 64 * -(-steps // slices):].double().T),
          torch.float32, f32=2e-5)                                   # the bias is in the first slice alone
    close(ss.materialize(), ref + b.double(), torch.bfloat16)
    none = K().gemm_skinny_sliced(xd, tiles, slices=slices)
    close(none.parts.double().sum(0), ref, torch.float32, f32=2e-5)
    if n % 4 == 0:
        weight, res = 1 + 0.1 * rnd(n, seed=3), rnd(m, n, dtype=torch.bfloat16, seed=4)
        resd = res.to(gpu)
        normed = K().rmsnorm(none, weight.to(gpu), 1e-5, residual=resd)
        total = none.parts.double().sum(0).cpu() + res.double()
        close(resd, total, torch.bfloat16)
        close(normed, pm.rms_norm(total, weight.double(), 1e-5), torch.bfloat16)
    # a row's sums depend neither on the other rows nor on what lies behind X; eight and sixteen wavefronts are both right
    one = K().gemm_skinny_sliced(xd[m - 1:].contiguous(), tiles, slices=slices)
    assert torch.equal(one.parts[:, 0], none.parts[:, m - 1])
    behind = torch.full((m + 8, k), float("nan"), dtype=torch.bfloat16, device=gpu)
    behind[:m] = xd
    assert torch.equal(K().gemm_skinny_sliced(behind[:m], tiles, slices=slices).parts, none.parts)
    for waves in (8, 16):
        close(K().gemm_skinny_sliced(xd, tiles, slices=slices, waves=waves).parts.double().sum(0), ref, torch.float32, f32=2e-5)
    from prelude_amd._native import NativeError
    with pytest.raises(NativeError, match="gemm_skinny_sliced: x"):
        K().gemm_skinny_sliced(torch.zeros(17, k, dtype=torch.bfloat16, device=gpu), tiles, slices=slices)
    with pytest.raises(NativeError, match="slices of"):
        K().check(K().kernels().pa_gemm_skinny_sliced(None, xd.data_ptr(), tiles.data.data_ptr(), None, none.parts.data_ptr(), m, n, k,
                                                       k, steps + 1, 0))


def test_narrow_weights_go_to_the_streaming_kernel_in_slices(gpu):
    """linear() for a reader of slices: weights of few tiles are cut so that the chip has workgroups enough, at the
    rows where that measured faster; the same bits as asked for directly; and not for a reader that wants a tensor."""
    for (n, k, rows, slices) in ((2560, 9728, (4, 8, 12), 3), (2048, 6144, (1, 16), 2), (1024, 3072, (1, 9, 16), 4), (1024, 2048, (2,), 4)):
        w = rnd(n, k, dtype=torch.bfloat16, seed=n, scale=0.03).to(gpu)
        lw = K().LinearWeight(w, K().pack_tiles(w))
        for m in rows:
            x = rnd(m, k, dtype=torch.bfloat16, seed=m).to(gpu)
            got = K().linear(x, lw, slices_ok=True)
            assert isinstance(got, K().SliceSums) and got.parts.shape[0] == slices, (n, k, m)
            assert torch.equal(got.parts, K().gemm_skinny_sliced(x, lw.tiles, slices=slices, waves=8).parts)
            assert isinstance(K().linear(x, lw), torch.Tensor)
            close(K().as_tensor(got), x.double().cpu() @ w.double().cpu().T, torch.bfloat16)
    w = rnd(2560, 9728, dtype=torch.bfloat16, seed=1, scale=0.03).to(gpu)
    lw = K().LinearWeight(w, K().pack_tiles(w))
    for m in (1, 2, 3):       # behind at so few rows: the kernel uncut
        assert isinstance(K().linear(rnd(m, 9728, dtype=torch.bfloat16).to(gpu), lw, slices_ok=True), torch.Tensor)
    K().set_skinny_sliced(False)
    try:
        assert isinstance(K().linear(rnd(8, 9728, dtype=torch.bfloat16).to(gpu), lw, slices_ok=True), torch.Tensor)
    finally:
        K().set_skinny_sliced(True)


@pytest.mark.parametrize("m,n,k", [(30, 24, 16), (4, 76, 24), (16, 48, 40), (1, 32, 8), (39, 2304, 24), (64, 40, 72)])
def test_gemm_skinny_stays_inside_its_rows(gpu, m, n, k):
    """Rows shorter than a step of 64 columns, or ending inside one: what lies behind a row of X is not the
    product's to read.  X is the head of a buffer whose rest is NaN (and a row stride wider than k keeps NaN behind
    every row): a read past a row's end, even one multiplied by the tile's zeros, would show in the result."""
    w = rnd(n, k, dtype=torch.bfloat16, seed=1, scale=0.05)
    x = rnd(m, k, dtype=torch.bfloat16)
    ref = x.double() @ w.double().T
    wd = w.to(gpu)
    tiles = K().pack_tiles(wd)
    behind = torch.full((m + 8, k), float("nan"), dtype=torch.bfloat16, device=gpu)
    behind[:m] = x.to(gpu)
    for weight in (tiles, wd):
        got = K().gemm_skinny(behind[:m], weight, out_dtype=torch.float32)
        assert bool(torch.isfinite(got).all()), f"read behind X with a {'tiled' if weight is tiles else 'row-major'} weight"
        close(got, ref, torch.float32, f32=2e-5)


@pytest.mark.parametrize("seed", list(range(int(os.environ.get("PRELUDE_AMD_DRAWN_PRODUCTS", "12")))))   # widen for a hunt
def test_drawn_products(gpu, seed):
    """Rows, outputs and inner size drawn at random, through the dispatcher and through the weight-streaming kernel
    with the weight in rows and in tiles, with bias, 32-bit output and the SiLU*up epilogue."""
    rng = np.random.default_rng(seed)
    m = int(rng.choice([1, 2, 7, 8, 9, 16, 17, 31, 33, 48, 64, int(rng.integers(1, 65))]))
    n = 2 * int(rng.choice([1, 8, 20, 160, 331, int(rng.integers(1, 1500)), int(rng.integers(1500, 12000))]))
    k = 8 * int(rng.choice([1, 7, 8, 9, 40, 129, int(rng.integers(1, 160)), int(rng.integers(160, 1300))]))
    if n * k > 40e6:
        k = max(8, int(40e6 // n) // 8 * 8)
    what = f"seed {seed}: m {m} n {n} k {k}"
    x, w, b = rnd(m, k, dtype=torch.bfloat16, seed=seed), rnd(n, k, dtype=torch.bfloat16, seed=seed + 1, scale=0.05), rnd(n, seed=2)
    ref = x.double() @ w.double().T
    act = pm.silu(ref[:, 0::2]) * ref[:, 1::2]
    xd, wd, bd = x.to(gpu), w.to(gpu), b.to(gpu)
    tiles = K().pack_tiles(wd)
    lw = K().LinearWeight(wd, tiles)
    for name, got, want, dt in (
            ("rows", K().gemm_skinny(xd, wd, out_dtype=torch.float32), ref, torch.float32),
            ("rows, bias", K().gemm_skinny(xd, wd, bd), ref + b.double(), torch.bfloat16),
            ("rows, SiLU*up", K().gemm_skinny(xd, wd, silu_mul_epilogue=True), act, torch.bfloat16),
            ("tiles", K().gemm_skinny(xd, tiles, out_dtype=torch.float32), ref, torch.float32),
            ("tiles, bias", K().gemm_skinny(xd, tiles, bd), ref + b.double(), torch.bfloat16),
            ("tiles, SiLU*up", K().gemm_skinny(xd, tiles, silu_mul_epilogue=True), act, torch.bfloat16),
            ("linear", K().linear(xd, lw, bd), ref + b.double(), torch.bfloat16),
            # beyond the streaming kernel's rows the library's bfloat16 result is widened: bfloat16's rounding
            ("linear, 32-bit out", K().linear(xd, lw, out_dtype=torch.float32), ref, torch.float32 if m <= 16 else torch.bfloat16),
            ("linear, SiLU*up", K().linear_silu_mul(xd, lw), act, torch.bfloat16)):
        assert tuple(got.shape) == tuple(want.shape), f"{what}, {name}: shape {tuple(got.shape)}"
        err = float((got.double().cpu() - want).abs().max())
        assert err <= tol(dt, want, f32=2e-5), f"{what}, {name}: max error {err:.3e} > {tol(dt, want, f32=2e-5):.3e}"
    # the product with X staged in LDS, at a drawn number of rows up to 128, of wavefronts and of slices
    m3 = int(rng.choice([17, 64, 65, 128, int(rng.integers(1, 129))]))
    x3 = rnd(m3, k, dtype=torch.bfloat16, seed=seed + 5)
    x3d = x3.to(gpu)
    ref3 = x3.double() @ w.double().T
    waves = int(rng.choice([0, 3, 4, 5, 6, 8]))
    steps = (k + 63) // 64
    cuts = [c for c in (2, 3, 4, 8) if c <= steps and -(-steps // -(-steps // c)) == c]
    for name, got, want, dt in (
            ("mid", K().gemm_mid(x3d, tiles, out_dtype=torch.float32, waves=waves), ref3, torch.float32),
            ("mid, bias", K().gemm_mid(x3d, tiles, bd, waves=waves), ref3 + b.double(), torch.bfloat16),
            ("mid, SiLU*up", K().gemm_mid(x3d, tiles, silu_mul_epilogue=True, waves=waves), pm.silu(ref3[:, 0::2]) * ref3[:, 1::2],
             torch.bfloat16),
            ("linear for a reader of slices", K().as_tensor(K().linear(x3d, lw, bd, slices_ok=True)), ref3 + b.double(), torch.bfloat16)):
        err = float((got.double().cpu() - want).abs().max())
        assert err <= tol(dt, want, f32=2e-5), f"{what}, rows {m3}, {waves} wavefronts, {name}: max error {err:.3e}"
    if cuts:
        c = int(rng.choice(cuts))
        parts = K().gemm_mid(x3d, tiles, bd, slices=c, waves=waves).parts
        err = float((parts.double().sum(0).cpu() - ref3 - b.double()).abs().max())
        assert err <= tol(torch.float32, ref3, f32=2e-5), f"{what}, rows {m3}, {waves} wavefronts, {c} slices: max error {err:.3e}"
    # the gated product with the residual add and the norm in front of it, inside it: up to 16 rows
    m5 = int(rng.choice([1, 8, 15, 16, int(rng.integers(1, 17))]))
    eps5 = float(rng.choice([1e-6, 1e-5, 1e-3]))
    x5, res5 = rnd(m5, k, dtype=torch.bfloat16, seed=seed + 9), rnd(m5, k, dtype=torch.bfloat16, seed=seed + 10, scale=float(rng.choice([0.1, 1.0, 30.0])))
    gain5 = 1 + 0.3 * rnd(k, seed=seed + 11)
    total5 = x5.double() + res5.double()
    g5 = pm.rms_norm(total5, gain5.double(), eps5) @ w.double().T
    new5, y5 = K().linear_gated_after_norm(x5.to(gpu), res5.to(gpu), gain5.to(gpu), eps5, lw, waves=waves)
    assert torch.equal(new5.cpu(), (x5.float() + res5.float()).to(torch.bfloat16)), f"{what}, rows {m5}: the new residual"
    want5 = pm.silu(g5[:, 0::2]) * g5[:, 1::2]
    err = float((y5.double().cpu() - want5).abs().max())
    assert err <= tol(torch.bfloat16, want5, bf16=1.25e-2), f"{what}, rows {m5}, {waves} wavefronts, norm + SiLU*up: max error {err:.3e}"
    # the streaming product of up to 16 rows in slices of K
    s6 = int(rng.integers(1, min(steps, 6) + 1))
    parts6 = K().gemm_skinny_sliced(x5.to(gpu), tiles, bd, slices=s6, waves=int(rng.choice([0, 8, 16]))).parts
    ref6 = x5.double() @ w.double().T + b.double()
    err = float((parts6.double().sum(0).cpu() - ref6).abs().max())
    assert err <= tol(torch.float32, ref6, f32=2e-5), f"{what}, rows {m5}, streaming kernel in {s6} slices: max error {err:.3e}"
    # the product tiled both ways, at a drawn number of rows, shape of workgroup, activation and number of slices
    m4 = int(rng.choice([1, 129, 192, 256, 257, int(rng.integers(1, 700))]))
    x4 = rnd(m4, k, dtype=torch.bfloat16, seed=seed + 7)
    x4d = x4.to(gpu)
    ref4 = x4.double() @ w.double().T
    shape = [(0, 0), (4, 2), (4, 3), (8, 2), (8, 3)][int(rng.integers(0, 5))]
    activation = ["silu", "gelu_tanh"][int(rng.integers(0, 2))]
    gate4 = pm.silu(ref4[:, 0::2]) if activation == "silu" else torch.nn.functional.gelu(ref4[:, 0::2], approximate="tanh")
    for name, got, want in (
            ("tall", K().gemm_tall(x4d, tiles, shape=shape), ref4),
            ("tall, bias", K().gemm_tall(x4d, tiles, bd, shape=shape), ref4 + b.double()),
            (f"tall, {activation}*up", K().gemm_tall(x4d, tiles, silu_mul_epilogue=True, shape=shape, activation=activation),
             gate4 * ref4[:, 1::2])):
        assert tuple(got.shape) == tuple(want.shape), f"{what}, rows {m4}, shape {shape}, {name}: shape {tuple(got.shape)}"
        err = float((got.double().cpu() - want).abs().max())
        assert err <= tol(torch.bfloat16, want), f"{what}, rows {m4}, shape {shape}, {name}: max error {err:.3e}"
    if cuts:
        c = int(rng.choice(cuts))
        parts = K().gemm_tall(x4d, tiles, bd, slices=c, shape=shape).parts
        err = float((parts.double().sum(0).cpu() - ref4 - b.double()).abs().max())
        assert err <= tol(torch.float32, ref4, f32=2e-5), f"{what}, rows {m4}, shape {shape}, {c} slices: max error {err:.3e}"
    # many rows through the dispatcher (the library product beyond the streaming kernel's rows)
    m2 = int(rng.integers(65, 400))
    x2 = rnd(m2, k, dtype=torch.bfloat16, seed=seed + 3)
    ref2 = x2.double() @ w.double().T
    close(K().linear(x2.to(gpu), lw, bd), ref2 + b.double(), torch.bfloat16)
    # gate and up are rounded to bfloat16 by the library product, then the activation's result: three roundings of up
    # to 2^-8 each, the gate's weighing up to 1.2 times (x silu'(x) / silu(x)) -- 1.25 % of the largest value at worst
    close(K().linear_silu_mul(x2.to(gpu), lw), pm.silu(ref2[:, 0::2]) * ref2[:, 1::2], torch.bfloat16, bf16=1.25e-2)


def test_pack_tiles_layout(gpu):
    """out[tile][step][half][g][r][j] = w[16 tile + r][64 step + 16 g + 8 half + j], zeros beyond the matrix."""
    n, k = 40, 200
    w = torch.arange(n * k, dtype=torch.float32).reshape(n, k).remainder(251.0).to(torch.bfloat16)
    t = K().pack_tiles(w.to(gpu))
    assert (t.n, t.k) == (n, k) and t.data.numel() == 3 * 4 * 1024
    got = t.data.cpu().reshape(3, 4, 2, 4, 16, 8)
    pad = torch.zeros(48, 256, dtype=torch.bfloat16)
    pad[:n, :k] = w
    want = pad.reshape(3, 16, 4, 4, 2, 8).permute(0, 2, 4, 3, 1, 5)   # [tile, r, step, g, half, j] -> [tile, step, half, g, r, j]
    assert torch.equal(got, want)


def test_gemm_skinny_refuses(gpu):
    from prelude_amd._native import NativeError
    with pytest.raises(NativeError, match="exceed"):
        K().gemm_skinny(torch.zeros(65, 64, dtype=torch.bfloat16, device=gpu), torch.zeros(16, 64, dtype=torch.bfloat16, device=gpu))
    with pytest.raises(NativeError, match="multiples of 8"):
        K().gemm_skinny(torch.zeros(2, 12, dtype=torch.bfloat16, device=gpu), torch.zeros(16, 12, dtype=torch.bfloat16, device=gpu))
    # what it refuses, linear() sends elsewhere
    out = K().linear(torch.ones(2, 12, dtype=torch.bfloat16, device=gpu), torch.ones(16, 12, dtype=torch.bfloat16, device=gpu))
    assert float(out.float().min()) == 12.0


# ---- QK norm + RoPE + cache write ---------------------------------------------------------------
def qk_reference(qkv, qw, kw, cos, sin, pos, nh, nkv, hd, rot, eps):
    t = qkv.shape[0]
    x = qkv.double().reshape(t, nh + 2 * nkv, hd)
    q, k, v = x[:, :nh], x[:, nh:nh + nkv], x[:, nh + nkv:]
    if qw is not None:
        q = pm.rms_norm(q, qw.double(), eps)
    if kw is not None:
        k = pm.rms_norm(k, kw.double(), eps)
    if rot:
        c, s = cos.double()[pos.long()], sin.double()[pos.long()]
        q = torch.cat([pm.apply_rope(q[..., :rot], c, s), q[..., rot:]], -1)
        k = torch.cat([pm.apply_rope(k[..., :rot], c, s), k[..., rot:]], -1)
    return q, k, v


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("nh,nkv,hd,rot,norm", [(32, 8, 128, 128, True), (6, 1, 32, 32, True), (5, 5, 48, 48, True),
                                                 (4, 2, 256, 256, True), (3, 1, 80, 32, True), (2, 2, 16, 16, False),
                                                 (7, 1, 112, 0, True), (4, 4, 64, 64, True)])
def test_qknorm_rope_kv(gpu, dtype, nh, nkv, hd, rot, norm):
    t, page, pages, eps = 11, 4, 9, 1e-5
    qkv = rnd(t, (nh + 2 * nkv) * hd, dtype=dtype, scale=2.0)
    qw = (1.0 + 0.2 * rnd(hd, seed=1)) if norm else None
    kw = (1.0 + 0.2 * rnd(hd, seed=2)) if norm else None
    pos = torch.tensor([0, 1, 2, 3, 17, 18, 99, 5, 6, 7, 255], dtype=torch.int32)
    cos = sin = None
    if rot:
        cos, sin = pm.rope_tables(rot, 256, 10000.0, torch.float32)
    slot_list = [35, 3, 0, 7, 8, 12, -1, 20, 21, 22, 30]                  # one token is not cached
    slots = torch.tensor(slot_list, dtype=torch.int32)
    kc = torch.full((pages, nkv, page, hd), 7.0, dtype=dtype)
    vc = torch.full((pages, nkv, hd, page), 7.0, dtype=dtype)
    dev = lambda x: None if x is None else x.to(gpu)
    kcd, vcd = kc.to(gpu), vc.to(gpu)
    q = K().qknorm_rope_kv(dev(qkv), dev(qw), dev(kw), dev(cos), dev(sin), dev(pos), dev(slots), kcd, vcd, nh, nkv, hd,
                           rot, eps)
    rq, rk, rv = qk_reference(qkv, qw, kw, cos, sin, pos, nh, nkv, hd, rot, eps)
    close(q, rq, dtype)
    touched = torch.zeros(pages, page, dtype=torch.bool)
    for i, s in enumerate(slot_list):
        if s < 0:
            continue
        touched[s // page, s % page] = True
        close(kcd[s // page, :, s % page], rk[i], dtype)
        assert torch.equal(vcd[s // page, :, :, s % page].cpu().double(), rv[i].to(dtype).double())   # V is a copy
    assert bool((kcd.cpu()[~touched[:, None, :].expand(pages, nkv, page)] == 7.0).all())             # nothing else written
    assert bool((vcd.cpu().transpose(2, 3)[~touched[:, None, :].expand(pages, nkv, page)] == 7.0).all())
    # queries only (a layer that reads another layer's cache)
    qonly = qkv[:, : nh * hd].contiguous()
    q2 = K().qknorm_rope_kv(dev(qonly), dev(qw), None, dev(cos), dev(sin), dev(pos), None, None, None, nh, 0, hd, rot, eps)
    assert torch.equal(q2, q)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("page,hd", [(16, 128), (8, 64), (32, 256), (12, 128)])
def test_value_cache_runs(gpu, dtype, page, hd):
    """Value pages written in runs of eight tokens (aligned, consecutive slots) and one by one around them:
    a run that starts in the middle of a group of eight tokens, one broken by an uncached token, one cut off
    by the end of the batch, slots that run backwards, and a page size that allows no runs."""
    nh, nkv, eps = 2, 3, 1e-6
    slot_list = (list(range(32, 40))                # a run: tokens 0..7
                 + list(range(5, 18))               # 5,6,7 alone; 8..15 a run that starts at token 11; 16,17 alone
                 + [48, 49, 50, -1, 52, 53, 54, 55]  # broken by a token that is not cached
                 + list(range(71, 63, -1))          # backwards
                 + list(range(80, 96))              # two runs back to back
                 + [110, 96, 97, 98, 99, 111, 109, 100]   # scattered (and enough tokens for the kernel to look for runs)
                 + list(range(104, 109)))           # cut off by the end of the batch
    t = len(slot_list)
    assert t >= 64
    pages = 112 // page + 1
    qkv = rnd(t, (nh + 2 * nkv) * hd, dtype=dtype, scale=2.0)
    pos = torch.arange(t, dtype=torch.int32)
    cos, sin = pm.rope_tables(hd, 128, 10000.0, torch.float32)
    w = 1.0 + 0.1 * rnd(hd, seed=3)
    kcd = torch.full((pages, nkv, page, hd), 7.0, dtype=dtype, device=gpu)
    vcd = torch.full((pages, nkv, hd, page), 7.0, dtype=dtype, device=gpu)
    K().qknorm_rope_kv(qkv.to(gpu), w.to(gpu), w.to(gpu), cos.to(gpu), sin.to(gpu), pos.to(gpu),
                       torch.tensor(slot_list, dtype=torch.int32, device=gpu), kcd, vcd, nh, nkv, hd, hd, eps)
    want = torch.full((pages, nkv, hd, page), 7.0, dtype=dtype)
    v = qkv[:, (nh + nkv) * hd:].reshape(t, nkv, hd)
    for i, sl in enumerate(slot_list):
        if sl >= 0:
            want[sl // page, :, :, sl % page] = v[i]
    assert torch.equal(vcd.cpu(), want)
    _, rk, _ = qk_reference(qkv, w, w, cos, sin, pos, nh, nkv, hd, hd, eps)
    for i, sl in enumerate(slot_list):
        if sl >= 0:
            close(kcd[sl // page, :, sl % page], rk[i], dtype)


def test_qknorm_rope_refuses_bad_sizes(gpu):
    from prelude_amd._native import NativeError
    qkv = torch.zeros(2, 3 * 272, device=gpu)
    with pytest.raises(NativeError, match="head_dim"):
        K().qknorm_rope_kv(qkv, None, None, None, None, torch.zeros(2, dtype=torch.int32, device=gpu), None, None, None,
                           3, 0, 272, 0, 1e-6)


# ---- attention over the paged cache --------------------------------------------------------------
def capped_plain_attention(q, k, v, scale, cap, window=None, q_offset=0):
    """``pm.attention`` with the scaled scores bent to cap * tanh(s / cap) before the mask: the cap is no formula of
    the reference's Qwen3 (no softcap there, crates/prelude-core/src/models/qwen3.rs:204), so its plain form lives here."""
    sq, nh, hd = q.shape
    sk, nkv, _ = k.shape
    out = torch.empty_like(q)
    qi = torch.arange(sq).reshape(sq, 1) + q_offset
    ki = torch.arange(sk).reshape(1, sk)
    allowed = ki <= qi
    if window is not None:
        allowed &= ki > qi - window
    for h in range(nh):
        s = (q[:, h] @ k[:, h // (nh // nkv)].T) * scale
        s = (cap * torch.tanh(s / cap)).masked_fill(~allowed, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, h // (nh // nkv)]
    return out


def paged_case(gpu, dtype, nh, nkv, hd, page, seqs, window, seed=0, scale_trick=None, kernel="generic", cut=None,
               softcap=0.0):
    """seqs: list of (context_len, q_len): the last q_len tokens of each context are this step's queries.
    Pages are handed out in a scrambled order.  Returns (engine output, plain output)."""
    g = torch.Generator().manual_seed(seed)
    total_pages = sum(-(-c // page) for c, _ in seqs) + 3
    perm = torch.randperm(total_pages, generator=torch.Generator().manual_seed(seed + 77)).tolist()
    kc = torch.zeros(total_pages, nkv, page, hd)
    vc = torch.zeros(total_pages, nkv, hd, page)
    stride = max(-(-c // page) for c, _ in seqs)
    table = torch.full((len(seqs), stride), -1, dtype=torch.int32)
    qs, seq_of, pos, refs = [], [], [], []
    for i, (ctx, ql) in enumerate(seqs):
        k = torch.randn(ctx, nkv, hd, generator=g)
        v = torch.randn(ctx, nkv, hd, generator=g)
        q = torch.randn(ql, nh, hd, generator=g)
        if scale_trick is not None:
            scale_trick(i, q, k, v)
        k, v, q = k.to(dtype).float(), v.to(dtype).float(), q.to(dtype).float()
        for p in range(-(-ctx // page)):
            phys = perm.pop()
            table[i, p] = phys
            n = min(page, ctx - p * page)
            kc[phys, :, :n] = k[p * page: p * page + n].transpose(0, 1)
            vc[phys, :, :, :n] = v[p * page: p * page + n].permute(1, 2, 0)
        if window:   # pages wholly before the first visible key may be gone
            first = max(0, (ctx - ql) - window + 1)
            for p in range(first // page):
                kc[table[i, p]] = float("nan")
                vc[table[i, p]] = float("nan")
                table[i, p] = -1
        qs.append(q)
        seq_of += [i] * ql
        pos += list(range(ctx - ql, ctx))
        if softcap:
            refs.append(capped_plain_attention(q.double(), k.double(), v.double(), 1.0 / math.sqrt(hd), softcap,
                                               window=window or None, q_offset=ctx - ql))
        else:
            refs.append(pm.attention(q.double(), k.double(), v.double(), 1.0 / math.sqrt(hd), window=window or None,
                                     q_offset=ctx - ql))
    q = torch.cat(qs).to(dtype)
    if kernel == "mfma":
        i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
        cu = [0]
        for _, ql in seqs:
            cu.append(cu[-1] + ql)
        dec = [i for i, (_, ql) in enumerate(seqs) if ql == 1]
        pre = [i for i, (_, ql) in enumerate(seqs) if ql > 1]
        qd, kd, vd, td = q.to(gpu), kc.to(dtype).to(gpu), vc.to(dtype).to(gpu), table.to(gpu)
        out = torch.full_like(qd, float("nan"))
        ctxs = i32([c for c, _ in seqs])
        K().attention_decode(qd, kd, vd, td, i32(dec), i32(cu), ctxs, out, max([seqs[i][0] for i in dec], default=0),
                             window, 1.0 / math.sqrt(hd), softcap=softcap)
        if dec and not pre:   # a step of single tokens: the kernels may count the sequences themselves, same bits
            again = torch.full_like(qd, float("nan"))
            K().attention_decode(qd, kd, vd, td, i32(dec), i32(cu), ctxs, again, max(seqs[i][0] for i in dec), window,
                                 1.0 / math.sqrt(hd), every_seq=True, softcap=softcap)
            assert torch.equal(again, out)
        K().attention_prefill(qd, kd, vd, td, i32(pre), i32(cu), ctxs, out, max([seqs[i][1] for i in pre], default=0),
                              window, 1.0 / math.sqrt(hd), cut=cut,
                              min_prefix=min([seqs[i][0] - seqs[i][1] for i in pre], default=0), softcap=softcap)
        return out, torch.cat(refs)
    out = K().attention_generic(q.to(gpu), kc.to(dtype).to(gpu), vc.to(dtype).to(gpu), table.to(gpu),
                                torch.tensor(seq_of, dtype=torch.int32, device=gpu),
                                torch.tensor(pos, dtype=torch.int32, device=gpu), window, 1.0 / math.sqrt(hd), softcap)
    return out, torch.cat(refs)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("nh,nkv,hd,page", [(4, 2, 16, 8), (6, 1, 32, 16), (32, 8, 128, 16), (5, 5, 48, 1), (3, 1, 256, 64),
                                            (8, 2, 80, 4), (2, 1, 112, 16)])
def test_attention_mixed_batch(gpu, dtype, nh, nkv, hd, page):
    seqs = [(70, 70), (130, 1), (33, 7), (1, 1), (64, 2), (257, 1)]
    out, ref = paged_case(gpu, dtype, nh, nkv, hd, page, seqs, 0)
    close(out, ref, dtype, f32=3e-6)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("window,page", [(24, 8), (1, 4), (64, 16), (65, 16), (7, 1)])
def test_attention_window(gpu, dtype, window, page):
    seqs = [(100, 100), (200, 1), (90, 30), (window, 1), (window + 1, 1)]
    out, ref = paged_case(gpu, dtype, 6, 2, 48, page, seqs, window)
    assert not bool(torch.isnan(out).any())
    close(out, ref, dtype, f32=3e-6)


def test_attention_far_key_and_window_edge(gpu):
    """Random keys would hide a key that is never read: one far key is made to stand out so that it
    takes nearly all the weight, once inside the window's edge and once just outside."""
    hd = 32

    def trick(i, q, k, v):
        q[:] = 0
        q[:, :, 0] = 12.0
        k[:, :, 0] = 0
        k[3, :, 0] = 12.0 * math.sqrt(hd)        # key 3 of hundreds

    out, ref = paged_case(gpu, torch.float32, 2, 1, hd, 16, [(300, 1), (300, 300)], 0, scale_trick=trick)
    close(out, ref, torch.float32, f32=3e-6)
    # window edge: the query at position 99 sees keys 80..99 with window 20
    for hot, seen in ((80, True), (79, False)):
        def trick2(i, q, k, v, hot=hot):
            q[:] = 0
            q[:, :, 0] = 12.0
            k[:, :, 0] = 0
            k[hot, :, 0] = 12.0 * math.sqrt(hd)
            v[hot] = 100.0
        out, ref = paged_case(gpu, torch.float32, 2, 1, hd, 16, [(100, 1)], 20, scale_trick=trick2)
        close(out, ref, torch.float32, f32=3e-6)
        assert (float(out.abs().max()) > 50.0) == seen


@pytest.mark.parametrize("nh,nkv,hd,page", [(4, 2, 16, 8), (6, 1, 32, 16), (32, 8, 128, 16), (6, 2, 48, 4), (8, 8, 64, 64),
                                            (24, 1, 96, 32), (16, 2, 128, 128), (3, 3, 64, 16)])
def test_mfma_attention_mixed_batch(gpu, nh, nkv, hd, page):
    seqs = [(70, 70), (130, 1), (33, 7), (1, 1), (64, 2), (700, 1), (257, 1), (300, 150), (16, 16), (513, 1)]
    out, ref = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, 0, kernel="mfma")
    assert not bool(torch.isnan(out).any())
    close(out, ref, torch.bfloat16)


@pytest.mark.parametrize("window,page", [(24, 8), (4, 4), (64, 16), (65, 16), (300, 16), (256, 32)])
def test_mfma_attention_window(gpu, window, page):
    seqs = [(100, 100), (200, 1), (90, 30), (window, 1), (window + 1, 1), (700, 1), (600, 300), (512, 1), (513, 1)]
    out, ref = paged_case(gpu, torch.bfloat16, 6, 2, 48, page, seqs, window, kernel="mfma")
    assert not bool(torch.isnan(out).any())
    close(out, ref, torch.bfloat16)


def test_mfma_attention_far_key_and_edges(gpu):
    hd = 64

    def trick(i, q, k, v):
        q[:] = 0
        q[:, :, 0] = 12.0
        k[:, :, 0] = 0
        k[3, :, 0] = 12.0 * math.sqrt(hd)
        v[3] = 50.0

    out, ref = paged_case(gpu, torch.bfloat16, 4, 1, hd, 16, [(1000, 1), (600, 600)], 0, scale_trick=trick, kernel="mfma")
    close(out, ref, torch.bfloat16)
    assert float(out[0].float().abs().min()) > 40.0            # the far key is found from position 999
    for hot, seen in ((80, True), (79, False)):
        def trick2(i, q, k, v, hot=hot):
            q[:] = 0
            q[:, :, 0] = 12.0
            k[:, :, 0] = 0
            k[hot, :, 0] = 12.0 * math.sqrt(hd)
            v[hot] = 100.0
        for seqs in ([(100, 1)], [(100, 20)]):
            out, ref = paged_case(gpu, torch.bfloat16, 2, 1, hd, 16, seqs, 20, scale_trick=trick2, kernel="mfma")
            close(out, ref, torch.bfloat16)
            assert (float(out[-1].float().abs().max()) > 50.0) == seen


@pytest.mark.parametrize("nh,nkv,hd,page,window,cap", [(8, 2, 128, 16, 0, 2.0), (6, 2, 48, 8, 50, 0.7), (4, 4, 64, 32, 0, 30.0),
                                                       (5, 1, 40, 4, 0, 1.0)])
def test_attention_with_capped_scores(gpu, nh, nkv, hd, page, window, cap):
    """A cap on the scores (cap * tanh(scaled score / cap) before the mask and the softmax) in every attention
    kernel: generic (both precisions), matrix-core decode with its splits, prefill staged and not.  Queries are
    made long so that most scores lie beyond the cap; without the cap the outputs differ by far more than the bound."""
    def trick(i, q, k, v):
        q *= 3.0

    seqs = [(70, 70), (130, 1), (33, 7), (1, 1), (700, 1), (300, 150), (513, 1)]
    for dtype in DT:
        out, ref = paged_case(gpu, dtype, nh, nkv, hd, page, seqs, window, seed=31, scale_trick=trick, softcap=cap)
        close(out, ref, dtype, f32=3e-6)
        plain, other = paged_case(gpu, dtype, nh, nkv, hd, page, seqs, window, seed=31, scale_trick=trick)
        assert float((other - ref).abs().max()) > 20 * tol(dtype, ref) or cap > 10
    if K().mfma_attention_supported(hd, page):
        out, ref = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, window, seed=31, scale_trick=trick,
                              kernel="mfma", softcap=cap)
        assert not bool(torch.isnan(out).any())
        close(out, ref, torch.bfloat16)
        if page >= 8:
            direct, _ = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, window, seed=31, scale_trick=trick,
                                   kernel="mfma", softcap=cap, cut=(-1, -1, -1, 0))
            close(direct, ref, torch.bfloat16)
    from prelude_amd._native import NativeError
    with pytest.raises(NativeError, match="negative"):
        paged_case(gpu, torch.float32, nh, nkv, hd, page, [(5, 1)], 0, softcap=-1.0)


@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
def test_gated_activation_in_every_epilogue(gpu, activation):
    """act(gate) * up with the activation chosen by a code: the pairwise kernel (both precisions) and the gated
    epilogues of the three products, each against the library's own function of that name in 64-bit."""
    import torch.nn.functional as F
    act = (lambda x: F.silu(x)) if activation == "silu" else (lambda x: F.gelu(x, approximate="tanh"))
    for dtype in DT:
        for tokens, inter in ((5, 160), (3, 7), (37, 1000)):
            gu = rnd(tokens, 2 * inter, dtype=dtype, scale=2.0)
            ref = act(gu[:, 0::2].double()) * gu[:, 1::2].double()
            close(K().silu_mul(gu.to(gpu), activation), ref, dtype, f32=3e-6)
    n, k = 1000, 2560
    w = rnd(n, k, dtype=torch.bfloat16, seed=1, scale=0.05)
    tiles = K().pack_tiles(w.to(gpu))
    lw = K().LinearWeight(w.to(gpu), tiles)
    for m, product in ((8, K().gemm_skinny), (40, K().gemm_mid), (200, K().gemm_tall)):
        x = rnd(m, k, dtype=torch.bfloat16, seed=m)
        g = x.double() @ w.double().T
        ref = act(g[:, 0::2]) * g[:, 1::2]
        close(product(x.to(gpu), tiles, silu_mul_epilogue=True, activation=activation), ref, torch.bfloat16)
        close(K().linear_gated(x.to(gpu), lw, activation), ref, torch.bfloat16)
    x = rnd(600, k, dtype=torch.bfloat16, seed=9)          # many rows: the library's product and the pairwise kernel
    g = x.double() @ w.double().T
    close(K().linear_gated(x.to(gpu), lw, activation), act(g[:, 0::2]) * g[:, 1::2], torch.bfloat16)
    from prelude_amd._native import NativeError
    with pytest.raises(NativeError, match="not one of"):
        K().silu_mul(rnd(2, 8).to(gpu), "relu")


@pytest.mark.parametrize("hd,page,window", [(64, 16, 0), (128, 16, 0), (64, 8, 40), (32, 32, 70), (128, 64, 33)])
def test_mfma_attention_first_keys_far_below_zero(gpu, hd, page, window):
    """The first keys a query sees score about -104 (2^-150 as a weight against a reference of 0), the later ones
    around zero: the first step's rescaling factor must not be formed from nothing (2^150 = inf, times the still
    empty sums = NaN).  Contexts that end one key into a step of 32, inside the cold stretch and behind it; with a
    window, queries whose first visible keys are the cold stretch's last ones."""
    cold = 64

    def trick(i, q, k, v):
        q[:, :, 0] = 12.0
        k[:, :, 0] = 0
        k[:cold, :, 0] = -104.0 * math.sqrt(hd) / 12.0

    seqs = [(300, 1), (33, 1), (65, 1), (97, 1), (64, 1), (300, 300), (200, 50), (70, 6), (129, 1)]
    out, ref = paged_case(gpu, torch.bfloat16, 4, 2, hd, page, seqs, window, seed=8, scale_trick=trick, kernel="mfma")
    assert not bool(torch.isnan(out).any())
    close(out, ref, torch.bfloat16)
    out, ref = paged_case(gpu, torch.float32, 4, 2, hd, page, seqs, window, seed=8, scale_trick=trick)
    assert not bool(torch.isnan(out).any())
    # A cold key's dot product starts with one term of 104 sqrt(hd); each of the hd additions behind it rounds at
    # that size (half a unit in the last place: 104 sqrt(hd) 2^-24), which adds up to some sqrt(hd) times that,
    # times the scale 1 / sqrt(hd), in the exponent: a query that sees cold keys only weighs them against each
    # other with a relative error of 104 sqrt(hd) 2^-24 (7e-5 at head_dim 128).  The bound follows the inputs' size;
    # a lost or misread key moves the output by O(1).
    close(out, ref, torch.float32, f32=104.0 * math.sqrt(hd) * 2.0 ** -24)


@pytest.mark.parametrize("nh,nkv,hd,page,window", [(8, 2, 128, 16, 0), (8, 1, 64, 32, 0), (4, 1, 96, 8, 150), (16, 2, 32, 64, 0),
                                                   (8, 2, 128, 128, 0), (4, 2, 64, 256, 100)])
def test_prefill_attention_every_cut(gpu, nh, nkv, hd, page, window):
    """The launcher cuts a prefill by the size of the step (tiles in pairs, unpaired sequence by sequence or unpaired
    with the tiles slowest over the grid; 1, 2 or 4 heads a wavefront, one or two head groups a workgroup, keys
    staged in LDS or not); small cases would only ever see one cut, so each is asked for here, on portions that
    start inside a context, end inside a tile and share a step."""
    seqs = [(333, 333), (500, 70), (1, 1), (129, 128), (64, 64), (700, 450)]
    group = nh // nkv
    most = 4 if hd <= 64 and group % 4 == 0 else 2
    base = None
    for staged in (1, 0):
        for paired in (1, 0, 2):
            for heads in (1, 2, 4):
                for groups in (1, 2):
                    if heads > most or (groups == 2 and (not staged or group % (2 * heads))):
                        continue
                    out, ref = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, window, seed=3, kernel="mfma",
                                          cut=(paired, heads, groups, staged))
                    assert not bool(torch.isnan(out).any()), (staged, paired, heads, groups)
                    close(out, ref, torch.bfloat16)
                    if base is None:
                        base = out
                    # the cut moves no key to another block of 32: the same sums in the same order
                    assert torch.equal(out, base), (staged, paired, heads, groups)


@pytest.mark.parametrize("nh,nkv,hd,page", [(32, 8, 128, 16), (16, 2, 64, 32), (4, 4, 128, 16)])
def test_prefill_attention_far_into_its_context(gpu, nh, nkv, hd, page):
    """Portions with long contexts behind them are cut without pairing and with wider workgroups (the launcher
    goes by the shortest prefix and the number of workgroups); large enough here to take those branches."""
    for seqs in ([(2304, 1024)], [(1500, 600), (3000, 1100)], [(4096, 2048)]):
        out, ref = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, 0, seed=11, kernel="mfma")
        close(out, ref, torch.bfloat16)
        fixed, _ = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, 0, seed=11, kernel="mfma", cut=(1, 1, 1, 1))
        assert torch.equal(out, fixed)


def test_prefill_attention_of_a_few_prompts(gpu):
    """Two to six prompts a step take a branch of their own (pairs only in whole rounds, else unpaired with every
    prompt's long tiles first): sizes that reach each of its cuts, prompts of unequal length among them."""
    for seqs in ([(512, 512)] * 3, [(512, 512)] * 4, [(500, 500), (130, 130), (512, 512), (64, 64), (333, 333), (1, 1)],
                 [(1024, 1024)] * 2, [(1024, 1024), (700, 700), (1000, 1000)], [(2048, 2048)] * 2):
        out, ref = paged_case(gpu, torch.bfloat16, 32, 8, 128, 16, seqs, 0, seed=13, kernel="mfma")
        close(out, ref, torch.bfloat16)
        fixed, _ = paged_case(gpu, torch.bfloat16, 32, 8, 128, 16, seqs, 0, seed=13, kernel="mfma", cut=(1, 1, 1, 1))
        assert torch.equal(out, fixed)
    for nh, nkv in ((40, 8), (16, 8)):
        out, ref = paged_case(gpu, torch.bfloat16, nh, nkv, 128, 16, [(512, 512), (300, 300), (512, 512)], 0, seed=14, kernel="mfma")
        close(out, ref, torch.bfloat16)


def test_prefill_attention_refuses_a_cut_the_shape_does_not_take(gpu):
    from prelude_amd._native import NativeError
    with pytest.raises(NativeError, match="heads a wavefront"):
        paged_case(gpu, torch.bfloat16, 8, 2, 128, 16, [(70, 70)], 0, kernel="mfma", cut=(-1, 4, -1, -1))
    with pytest.raises(NativeError, match="head groups"):
        paged_case(gpu, torch.bfloat16, 3, 3, 64, 16, [(70, 70)], 0, kernel="mfma", cut=(-1, 1, 2, -1))
    with pytest.raises(NativeError, match="not staged"):
        paged_case(gpu, torch.bfloat16, 4, 2, 64, 4, [(70, 70)], 0, kernel="mfma", cut=(-1, -1, -1, 1))


@pytest.mark.parametrize("nh,nkv,hd,page,window,seqs", [
    (2, 1, 128, 16, 0, [(40000, 130), (50001, 1)]),
    (4, 2, 64, 64, 3000, [(45000, 70), (33000, 1)]),
    (2, 2, 128, 128, 0, [(70000, 2), (131072, 1)])])
def test_attention_long_contexts(gpu, nh, nkv, hd, page, window, seqs):
    """Contexts of tens of thousands of tokens: thousands of pages a request, every split of a decoding request
    at work, a window that has passed most of the pages."""
    out, ref = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, window, seed=2, kernel="mfma")
    assert not bool(torch.isnan(out).any())
    close(out, ref, torch.bfloat16)
    if max(c for c, _ in seqs) <= 50001:
        out, ref = paged_case(gpu, torch.float32, nh, nkv, hd, page, seqs, window, seed=2)
        close(out, ref, torch.float32, f32=3e-6)


@pytest.mark.parametrize("nh,nkv,hd,page,window", [(32, 8, 128, 16, 0), (8, 2, 64, 8, 0), (4, 1, 96, 32, 100),
                                                   (6, 3, 128, 128, 0), (2, 2, 32, 4, 0)])
def test_decode_attention_of_single_tokens_only(gpu, nh, nkv, hd, page, window):
    """A step of single tokens: contexts that end at, just before and just behind the edge of a split and of a page
    (the pages of a split are looked up before the length is known, and a key past the end is read from the last
    one there is); table entries behind a sequence's last page are -1."""
    seqs = [(1, 1), (255, 1), (256, 1), (257, 1), (1000, 1), (4097, 1), (31, 1), (33, 1), (512, 1), (769, 1)]
    out, ref = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, window, seed=4, kernel="mfma")
    assert not bool(torch.isnan(out).any())
    close(out, ref, torch.bfloat16)


@pytest.mark.parametrize("nh,nkv,hd,page,window,seqs", [
    (32, 8, 128, 16, 0, [(4096, 1), (4095, 1), (3841, 1), (3840, 1), (2000, 1), (300, 1), (1, 1)]),     # 8 x 16 x 7 = 896
    (16, 4, 64, 32, 700, [(8192, 1), (8000, 1), (7937, 1), (7936, 1), (100, 1), (257, 1), (5000, 1), (31, 1)]),   # 4 x 5 x 8 = 160: four
    (16, 4, 64, 32, 0, [(8192, 1), (8000, 1), (7937, 1), (7936, 1), (100, 1), (257, 1), (5000, 1), (31, 1)]),     # 4 x 32 x 8 = 1,024
    (8, 2, 128, 16, 0, [(12288, 1), (12033, 1), (12032, 1), (1, 1), (256, 1), (6000, 1), (11000, 1), (9999, 1),
                        (77, 1), (4096, 1), (12287, 1), (513, 1), (10000, 1), (2222, 1), (8191, 1), (300, 1)]),   # 2 x 48 x 16 = 1,536
    (3, 3, 48, 8, 0, [(16384, 1), (16129, 1), (2, 1), (9000, 1)])])                                      # 3 x 64 x 4 = 768: four wavefronts
def test_decode_attention_in_grids_that_run_with_two_wavefronts(gpu, nh, nkv, hd, page, window, seqs):
    """Grids of 769 to 1,536 workgroups run with two wavefronts a workgroup, each taking every second step of a
    split; the last case lies at the edge and keeps four."""
    out, ref = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, window, seed=6, kernel="mfma")
    assert not bool(torch.isnan(out).any())
    close(out, ref, torch.bfloat16)


def draw_attention_case(seed: int):
    rng = np.random.default_rng(seed)
    hd = int(rng.choice([16, 32, 48, 64, 96, 128]))
    nkv = int(rng.choice([1, 2, 3, 8]))
    group = int(rng.choice([1, 2, 3, 4, 6, 8]))
    page = int(rng.choice([4, 8, 16, 32, 64, 128]))
    window = int(rng.choice([0, 0, 0, 1, 31, 64, 100, 257, int(rng.integers(2, 500))]))
    seqs = []
    for _ in range(int(rng.integers(1, 7))):
        kind = int(rng.integers(0, 4))
        if kind == 0:                                   # a decoding request
            seqs.append((int(rng.integers(1, 1300)), 1))
        elif kind == 1:                                 # a whole prompt
            n = int(rng.integers(2, 800))
            seqs.append((n, n))
        else:                                           # a portion inside a context, long or down to two tokens
            ctx = int(rng.integers(2, 1500))
            seqs.append((ctx, int(rng.integers(2, min(ctx, 600 if kind == 2 else 9) + 1))))
    return nkv * group, nkv, hd, page, window, seqs


@pytest.mark.parametrize("seed", list(range(int(os.environ.get("PRELUDE_AMD_DRAWN_ATTENTION", "10")))))   # widen for a hunt
def test_drawn_attention(gpu, seed):
    """Head counts, head size, page size, window and the step's requests drawn at random: decoding requests, whole
    prompts and portions inside a context in one step.  Pages a window has passed hold NaN, so a key read from one
    of them shows."""
    nh, nkv, hd, page, window, seqs = draw_attention_case(seed)
    what = f"seed {seed}: {nh} heads over {nkv}, head_dim {hd}, page {page}, window {window}, (context, new) {seqs}"
    out, ref = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, window, seed=seed, kernel="mfma")
    assert not bool(torch.isnan(out).any()), what
    err = float((out.double().cpu() - ref).abs().max())
    assert err <= tol(torch.bfloat16, ref), f"{what}: max error {err:.3e}"
    out, ref = paged_case(gpu, torch.float32, nh, nkv, hd, page, seqs, window, seed=seed)
    assert not bool(torch.isnan(out).any()), what
    err = float((out.double().cpu() - ref).abs().max())
    assert err <= tol(torch.float32, ref, f32=3e-6), f"{what}: 32-bit kernel, max error {err:.3e}"


def draw_two_wavefront_case(seed: int):
    """A step of single tokens whose grid (KV heads x splits of the longest context x sequences) has 769 to 1,536
    workgroups.  The splits are counted as the launcher counts them: from the longest context rounded up."""
    from prelude_amd.ops.kernels import decode_context_bound
    rng = np.random.default_rng(1000 + seed)
    while True:
        hd = int(rng.choice([16, 32, 48, 64, 96, 128]))
        nkv = int(rng.choice([1, 2, 3, 4, 8]))
        group = int(rng.choice([1, 2, 3, 4, 8, 16]))
        page = int(rng.choice([4, 8, 16, 32, 64, 128]))
        nseq = int(rng.integers(2, 11))
        longest = int(rng.integers(300, 16385))
        window = int(rng.choice([0, 0, 0, int(rng.integers(300, 8000))]))
        if window >= longest:
            window = 0
        bound = decode_context_bound(longest, page)
        span = min(bound, window + 256) if window else bound
        grid = nkv * (-(-span // 256) + (1 if window else 0)) * nseq
        if not 768 < grid <= 1536:
            continue
        ctxs = [longest] + [int(rng.integers(1, longest + 1)) for _ in range(nseq - 1)]
        rng.shuffle(ctxs)
        return nkv * group, nkv, hd, page, window, [(int(c), 1) for c in ctxs], grid


@pytest.mark.parametrize("seed", list(range(int(os.environ.get("PRELUDE_AMD_DRAWN_ATTENTION", "10")))))   # widen for a hunt
def test_drawn_attention_in_grids_of_two_wavefronts(gpu, seed):
    nh, nkv, hd, page, window, seqs, grid = draw_two_wavefront_case(seed)
    assert 768 < grid <= 1536
    what = f"seed {seed}: {nh} heads over {nkv}, head_dim {hd}, page {page}, window {window}, (context, new) {seqs}"
    out, ref = paged_case(gpu, torch.bfloat16, nh, nkv, hd, page, seqs, window, seed=seed, kernel="mfma")
    assert not bool(torch.isnan(out).any()), what
    err = float((out.double().cpu() - ref).abs().max())
    assert err <= tol(torch.bfloat16, ref), f"{what}: max error {err:.3e}"


def test_mfma_attention_batch_and_page_independence(gpu):
    one, _ = paged_case(gpu, torch.bfloat16, 8, 2, 128, 16, [(900, 1)], 0, seed=5, kernel="mfma")
    many, _ = paged_case(gpu, torch.bfloat16, 8, 2, 128, 16, [(900, 1), (40, 1), (300, 30)], 0, seed=5, kernel="mfma")
    assert torch.equal(one[0], many[0])                          # same sequence, other company
    other, _ = paged_case(gpu, torch.bfloat16, 8, 2, 128, 64, [(900, 1)], 0, seed=5, kernel="mfma")
    assert torch.equal(one, other)                               # other page size, other pages


def test_decode_attention_on_either_side_of_the_grid_limits(gpu):
    """The same sequence alone (128 workgroups: eight wavefronts a workgroup), among eight (1,024: two), beside one
    other, among six and among thirteen (256, 768 and 1,664: four; dealt out plainly, in stretches, plainly).  Which
    keys a split sums is the same in all of them; the order in which a split's steps are added is not, so the
    results agree to rounding, not to the bit, across the limits -- and to the bit on the same side of them."""
    first = (4096, 1)
    outs = []
    for others in (0, 1, 7, 5, 12):
        seqs = [first] + [(4000 - 50 * i, 1) for i in range(others)]
        out, ref = paged_case(gpu, torch.bfloat16, 32, 8, 128, 16, seqs, 0, seed=21, kernel="mfma")
        close(out, ref, torch.bfloat16)
        outs.append((out[0].double().cpu(), ref[0]))
    (a, ref), (a2, _), (b, _), (c, _), (c2, _) = outs
    assert torch.equal(a2, c) and torch.equal(c, c2)          # four wavefronts every time
    for x, y in ((a, b), (a, c), (b, c)):
        assert float((x - y).abs().max()) <= tol(torch.bfloat16, ref)


@pytest.mark.parametrize("nh,nkv,hd,page,window,norm,ctxs", [
    (32, 8, 128, 16, 0, True, [1, 17, 256, 257, 700, 33, 512]), (8, 8, 64, 8, 0, True, [1, 17, 256, 257, 700, 33, 512]),
    (16, 1, 128, 64, 40, True, [1, 17, 256, 257, 700, 33, 512]), (4, 2, 64, 16, 0, False, [1, 17, 256, 257, 700, 33, 512]),
    # 8 KV heads, 16 splits and 7 listed sequences: 896 workgroups, a grid that runs with two wavefronts a workgroup
    (32, 8, 128, 16, 0, True, [4096, 3841, 3840, 2000, 300, 33, 1, 4095])])
def test_decode_attention_takes_the_raw_projection(gpu, nh, nkv, hd, page, window, norm, ctxs):
    """QK-norm, rotation, cache write and split attention in one kernel against the two kernels one after the
    other: the same outputs and the same keys and values in the cache, for contexts that end at a page's first
    and last place and at a split's edge; sequences outside the list are left alone."""
    raw_projection_case(gpu, nh, nkv, hd, page, window, norm, ctxs)
    assert not K().attention_decode_fused_supported(nh, nkv, hd, hd // 2, page)      # partial rotation
    assert not K().attention_decode_fused_supported(34, 2, 128, 128, 16)             # more than 16 heads per KV head
    assert not K().attention_decode_fused_supported(4, 2, 96, 96, 16)


@pytest.mark.parametrize("nh,nkv,hd,page,window,norm", [(8, 2, 128, 16, 0, True), (4, 4, 64, 8, 0, False),
                                                         (8, 1, 128, 32, 40, True)])
def test_decode_attention_of_the_raw_projection_with_first_keys_far_below_zero(gpu, nh, nkv, hd, page, window, norm):
    """As ``test_mfma_attention_first_keys_far_below_zero``, for the kernel that norms and rotates its own query."""
    raw_projection_case(gpu, nh, nkv, hd, page, window, norm, [300, 33, 65, 97, 66, 40, 129, 4096], cold=64)


@pytest.mark.parametrize("seed", list(range(int(os.environ.get("PRELUDE_AMD_DRAWN_ATTENTION", "10")) // 2)))
def test_drawn_raw_projection_in_grids_of_two_wavefronts(gpu, seed):
    """The one-kernel form in grids of 769 to 1,536 workgroups, drawn: it has a two-wavefront variant of its own."""
    s = seed
    while True:
        nh, nkv, hd, page, window, seqs, grid = draw_two_wavefront_case(10_000 + s)
        if hd in (64, 128) and nh // nkv <= 16 and page >= 8 and len(seqs) >= 5:
            break
        s += 1000
    ctxs = [c for c, _ in seqs]
    ctxs.insert(5, 33)       # the case leaves its sixth sequence out of the step: one that does not count in the grid
    raw_projection_case(gpu, nh, nkv, hd, page, window, bool(seed % 2), ctxs)


def raw_projection_case(gpu, nh, nkv, hd, page, window, norm, ctxs, cold=0):
    """``cold`` > 0: the first ``cold`` keys of every sequence score about -104 against its query (the heads of a
    KV head then share one query, so that one key can be that cold for all of them)."""
    eps = 1e-6
    t = len(ctxs)
    listed = [i for i in range(t) if i != 5]           # the sixth sequence is not in the list
    g = torch.Generator().manual_seed(3)
    group = nh // nkv
    scale = 1.0 / math.sqrt(hd)
    qkv = (2.0 * torch.randn(t, (nh + 2 * nkv) * hd, generator=g)).to(torch.bfloat16)
    if cold:
        heads = qkv[:, : nh * hd].reshape(t, nkv, group, hd)
        heads[:] = heads[:, :, :1]
    qw = (1.0 + 0.2 * rnd(hd, seed=1)) if norm else None
    kw = (1.0 + 0.2 * rnd(hd, seed=2)) if norm else None
    cos, sin = pm.rope_tables(hd, max(ctxs), 10000.0, torch.float32)
    # what the plain functions make of the projection: normed, rotated queries and keys, values as they are
    rq, rk, rv = qk_reference(qkv, qw, kw, cos, sin, torch.tensor([c - 1 for c in ctxs]), nh, nkv, hd, hd, eps)
    total_pages = sum(-(-c // page) for c in ctxs) + 2
    perm = torch.randperm(total_pages, generator=g).tolist()
    stride = max(-(-c // page) for c in ctxs)
    table = torch.full((t, stride), -1, dtype=torch.int32)
    kc = torch.zeros(total_pages, nkv, page, hd, dtype=torch.bfloat16)
    vc = torch.zeros(total_pages, nkv, hd, page, dtype=torch.bfloat16)
    slots, plain = [], []
    for i, c in enumerate(ctxs):
        for p in range(-(-c // page)):
            table[i, p] = perm.pop()
        hist = c - 1                                   # keys before the token's own
        k_hist = torch.randn(hist, nkv, hd, generator=g)
        v_hist = torch.randn(hist, nkv, hd, generator=g).to(torch.bfloat16)
        if cold:
            qdir = rq[i, ::group].float()              # [nkv, hd]: the query all heads of a KV head share
            k_hist[:cold] = -104.0 / scale * qdir / (qdir * qdir).sum(-1, keepdim=True)
        k_hist = k_hist.to(torch.bfloat16)
        for p in range(-(-hist // page)):
            n, ph = min(page, hist - p * page), int(table[i, p])
            kc[ph, :, :n] = k_hist[p * page: p * page + n].transpose(0, 1)
            vc[ph, :, :, :n] = v_hist[p * page: p * page + n].permute(1, 2, 0)
        slots.append(int(table[i, (c - 1) // page]) * page + (c - 1) % page)
        # the plain attention of the token over its history and its own key and value (as the cache will hold them)
        keys = torch.cat([k_hist.double(), rk[i: i + 1].to(torch.bfloat16).double()])
        values = torch.cat([v_hist.double(), rv[i: i + 1]])
        plain.append(pm.attention(rq[i: i + 1].to(torch.bfloat16).double(), keys, values, scale, window=window or None,
                                  q_offset=c - 1)[0])
    dev = lambda x: None if x is None else x.to(gpu)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
    pos, sl, seqs, cu, cl = i32([c - 1 for c in ctxs]), i32(slots), i32(listed), i32(list(range(t + 1))), i32(ctxs)
    assert K().attention_decode_fused_supported(nh, nkv, hd, hd, page)
    # the two kernels
    k1, v1 = kc.to(gpu), vc.to(gpu)
    q = K().qknorm_rope_kv(dev(qkv), dev(qw), dev(kw), dev(cos), dev(sin), pos, sl, k1, v1, nh, nkv, hd, hd, eps)
    out1 = torch.zeros(t, nh, hd, dtype=torch.bfloat16, device=gpu)
    K().attention_decode(q, k1, v1, dev(table), seqs, cu, cl, out1, max(ctxs), window, scale)
    # the one kernel
    k2, v2 = kc.to(gpu), vc.to(gpu)
    out2 = K().attention_decode_fused(dev(qkv), dev(qw), dev(kw), dev(cos), dev(sin), sl, eps, k2, v2, dev(table),
                                      seqs, cu, cl, nh, max(ctxs), window, scale)
    assert not bool(torch.isnan(out2[listed]).any()) and not bool(torch.isnan(out1[listed]).any())
    for i in listed:
        close(out2[i], out1[i].double().cpu(), torch.bfloat16)
        close(out2[i], plain[i], torch.bfloat16)       # and each against the plain functions, not only one another
        close(out1[i], plain[i], torch.bfloat16)
        ph, off = slots[i] // page, slots[i] % page
        assert torch.equal(v2[ph, :, :, off], v1[ph, :, :, off])
        close(k2[ph, :, off], k1[ph, :, off].double().cpu(), torch.bfloat16)
    # the sequence that was not listed: its key and value were not written
    ph, off = slots[5] // page, slots[5] % page
    assert float(k2[ph, :, off].abs().max()) == 0.0 and float(v2[ph, :, :, off].abs().max()) == 0.0
    # nothing else in the caches changed
    mask = torch.ones(total_pages, page, dtype=torch.bool)
    for i in listed:
        mask[slots[i] // page, slots[i] % page] = False
    assert torch.equal(k2.cpu()[mask[:, None, :].expand(total_pages, nkv, page)], kc[mask[:, None, :].expand(total_pages, nkv, page)])
    assert torch.equal(v2.cpu().transpose(2, 3)[mask[:, None, :].expand(total_pages, nkv, page)],
                       vc.transpose(2, 3)[mask[:, None, :].expand(total_pages, nkv, page)])


def test_mfma_attention_refuses_what_it_does_not_take(gpu):
    from prelude_amd._native import NativeError
    assert K().mfma_attention_supported(128, 16) and K().mfma_attention_supported(48, 8)
    assert not K().mfma_attention_supported(80, 16) and not K().mfma_attention_supported(128, 1)
    with pytest.raises(NativeError, match="head_dim"):
        paged_case(gpu, torch.bfloat16, 2, 1, 80, 16, [(20, 1)], 0, kernel="mfma")
    with pytest.raises(NativeError, match="page size"):
        paged_case(gpu, torch.bfloat16, 2, 1, 64, 2, [(20, 1)], 0, kernel="mfma")


def test_attention_is_independent_of_pages_and_batch(gpu):
    a, _ = paged_case(gpu, torch.float32, 4, 2, 64, 16, [(150, 150)], 0, seed=5)
    b, _ = paged_case(gpu, torch.float32, 4, 2, 64, 4, [(150, 150)], 0, seed=5)       # other page size, other pages
    assert torch.equal(a, b)


# ---- sampling ---------------------------------------------------------------------------------
def test_argmax(gpu):
    # crates/prelude-core/src/engine/sampling/logits_processor.rs:144-149 and ties to the lowest index
    x = torch.tensor([[0.1, 0.2, 0.9, 0.3], [0.9, 0.2, 0.9, 0.3], [-1.0, -1.0, -1.0, -1.0]])
    assert K().argmax(x.to(gpu)).tolist() == [2, 0, 0]
    big = rnd(5, 151936)
    big[1, 150000] = 50.0
    big[2, 7] = big[2, 140001] = 60.0
    assert K().argmax(big.to(gpu)).tolist() == torch.argmax(big, dim=-1).tolist()
    assert K().argmax(big.to(gpu)).tolist()[2] == 7


@pytest.mark.parametrize("vocab,wide", [(509, False), (509, True), (151936, False), (151936, True), (40001, True)])
def test_sample_matches_the_plain_draw(gpu, vocab, wide):
    """Both sampling kernels (a workgroup a row; rows cut into slices over many workgroups) against the plain draw."""
    g = torch.Generator().manual_seed(3)
    rows = 24
    logits = 3.0 * torch.randn(rows, vocab, generator=g)
    temps = [0.0, 0.8, 1.0, 0.3, 1.5, 0.8] * 4
    topk = [0, 0, 5, 0, 50, 20] * 4
    topp = [1.0, 1.0, 1.0, 0.9, 0.5, 0.95] * 4
    u = torch.rand(rows, generator=g)
    out = K().sample(logits.to(gpu), torch.tensor(temps).to(gpu), torch.tensor(topk, dtype=torch.int32).to(gpu),
                     torch.tensor(topp).to(gpu), u.to(gpu), wide=wide).tolist()
    checked = 0
    for r in range(rows):
        if temps[r] < 1e-7:
            assert out[r] == int(torch.argmax(logits[r]))
            continue
        prs = pm.sampling_probs(logits[r], temps[r], topk[r] or None, topp[r] if topp[r] < 1.0 else None)
        assert prs[out[r]] > 0, f"row {r}: token {out[r]} is outside the kept set"
        cdf = torch.cumsum(prs, 0)
        target = float(u[r]) * float(cdf[-1])
        # compare only where 32-bit summation cannot move the draw across a boundary
        if float((cdf - target).abs().min()) > 1e-4 * float(cdf[-1]):
            assert out[r] == pm.draw(prs, float(u[r])), f"row {r}"
            checked += 1
    assert checked >= rows // 2


@pytest.mark.parametrize("seed", list(range(int(os.environ.get("PRELUDE_AMD_DRAWN_DRAWS", "8")))))   # widen for a hunt
def test_drawn_draws(gpu, seed):
    """Vocabulary, rows and every row's temperature, top-k and top-p drawn at random, through the one-workgroup
    kernel and the wide one: the token is the plain draw's wherever 32-bit sums cannot move it over a boundary,
    and always one of the kept set."""
    rng = np.random.default_rng(seed)
    vocab = int(rng.choice([2, 17, 509, 4096, 40001, 151936, int(rng.integers(2, 200000))]))
    rows = int(rng.choice([1, 2, 8, 33, int(rng.integers(1, 70))]))
    rows = min(rows, max(1, 400000 // vocab))      # the plain top-p walks the sorted row entry by entry
    g = torch.Generator().manual_seed(seed)
    logits = float(rng.choice([0.5, 3.0, 8.0])) * torch.randn(rows, vocab, generator=g)
    temps = [float(rng.choice([0.0, 0.3, 0.8, 1.0, 1.7])) for _ in range(rows)]
    topk = [int(rng.choice([0, 0, 1, 5, 50, vocab, 2 * vocab])) for _ in range(rows)]
    topp = [float(rng.choice([1.0, 1.0, 0.95, 0.5, 0.05])) for _ in range(rows)]
    u = torch.rand(rows, generator=g)
    for wide in (False, True):
        out = K().sample(logits.to(gpu), torch.tensor(temps).to(gpu), torch.tensor(topk, dtype=torch.int32).to(gpu),
                         torch.tensor(topp).to(gpu), u.to(gpu), wide=wide).tolist()
        for r in range(rows):
            what = f"seed {seed} wide {wide}: vocabulary {vocab}, row {r} of {rows}, T {temps[r]} top-k {topk[r]} top-p {topp[r]}"
            if temps[r] < 1e-7:
                assert out[r] == int(torch.argmax(logits[r])), what
                continue
            prs = pm.sampling_probs(logits[r], temps[r], topk[r] or None, topp[r] if topp[r] < 1.0 else None)
            assert 0 <= out[r] < vocab and prs[out[r]] > 0, f"{what}: token {out[r]} is outside the kept set"
            cdf = torch.cumsum(prs, 0)
            target = float(u[r]) * float(cdf[-1])
            if float((cdf - target).abs().min()) > 1e-4 * float(cdf[-1]):
                assert out[r] == pm.draw(prs, float(u[r])), what


@pytest.mark.parametrize("rows", [1, 3, 70])
def test_sample_wide_takes_only_the_searches_it_is_told_of(gpu, rows):
    """Rows cut into 64, 64 and 14 slices; without top-k and top-p rows the searches are left out, and the
    tokens are those of the one-workgroup kernel (uniform numbers away from the boundaries)."""
    g = torch.Generator().manual_seed(rows)
    vocab = 70001
    logits = (2.0 * torch.randn(rows, vocab, generator=g)).to(gpu)
    u = (0.05 + 0.9 * torch.rand(rows, generator=g)).to(gpu)
    full = lambda v, dt=torch.float32: torch.full((rows,), v, dtype=dt).to(gpu)
    for k, p in ((0, 1.0), (40, 1.0), (0, 0.8), (40, 0.8)):
        args = (logits, full(0.9), full(k, torch.int32), full(p), u)
        one = K().sample(*args, wide=False)
        many = K().sample(*args, any_top_k=k > 0, any_top_p=p < 1.0, wide=True)
        told_more = K().sample(*args, wide=True)
        assert torch.equal(many, told_more)
        assert int((one != many).sum()) <= max(1, rows // 20), (k, p, one.tolist(), many.tolist())


@pytest.mark.parametrize("vocab", [509, 151936, 40001])
def test_logprobs(gpu, vocab):
    """logits[id] - logsumexp(logits), and the k largest entries with ties at the k-th value
    (crates/prelude-core/src/engine/model_runner/postprocess.rs:88-155)."""
    g = torch.Generator().manual_seed(vocab)
    rows = 7
    logits = 4.0 * torch.randn(rows, vocab, generator=g)
    logits[2, 100:104] = logits[2].max() + 1.0          # four equal entries on top
    ids = torch.randint(0, vocab, (rows,), generator=g).to(torch.int32)
    ids[3] = -1
    ref = torch.log_softmax(logits.double(), dim=-1)
    lp, top = K().logprobs(logits.to(gpu), ids.to(gpu))
    assert top is None
    for r in range(rows):
        want = 0.0 if ids[r] < 0 else float(ref[r, ids[r]])
        assert abs(float(lp[r]) - want) < 2e-5 * max(1.0, abs(want))
    for k in (1, 3, 20):
        lp2, (vals, idx, count) = K().logprobs(logits.to(gpu), ids.to(gpu), k)
        assert torch.equal(lp2, lp)
        for r in range(rows):
            n = int(count[r])
            got = sorted(zip(idx[r, :n].tolist(), vals[r, :n].tolist()), key=lambda t: (-t[1], t[0]))
            kth = torch.topk(ref[r], k).values[-1]
            want_ids = sorted(torch.nonzero(ref[r] >= kth).flatten().tolist())      # ties at the k-th value included
            assert sorted(i for i, _ in got) == want_ids, (k, r)
            assert all(abs(v - float(ref[r, i])) < 2e-5 * max(1.0, abs(float(ref[r, i]))) for i, v in got)
            assert [i for i, _ in got[:k]] == torch.topk(ref[r], k).indices.tolist() or r == 2


def test_sample_statistics_and_limits(gpu):
    logits = torch.tensor([[2.0, 1.0, 0.5, -1.0, 0.0]]).repeat(4000, 1)
    g = torch.Generator().manual_seed(0)
    u = torch.rand(4000, generator=g)
    z = lambda v, dt=torch.float32: torch.full((4000,), v, dtype=dt).to(gpu)
    out = K().sample(logits.to(gpu), z(0.8), z(0, torch.int32), z(1.0), u.to(gpu)).cpu()
    freq = torch.bincount(out.long(), minlength=5).double() / 4000
    assert float((freq - torch.softmax(logits[0].double() / 0.8, -1)).abs().max()) < 0.03
    out = K().sample(logits.to(gpu), z(1.0), z(2, torch.int32), z(1.0), u.to(gpu)).cpu()
    assert set(out.tolist()) == {0, 1}                                       # top-2 stays in {0, 1}
    out = K().sample(logits.to(gpu), z(1e-9), z(0, torch.int32), z(1.0), u.to(gpu)).cpu()
    assert set(out.tolist()) == {0}                                          # T -> 0 is the argmax
    out = K().sample(logits.to(gpu), z(1.0), z(0, torch.int32), z(0.4), u.to(gpu)).cpu()
    assert set(out.tolist()) == {0}                                          # the first entry alone reaches p = 0.4
