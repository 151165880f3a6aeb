"""GPU parity of the tap-packed stem conv (few input channels: one activation scale per staged 4 x 10 x 18 tile; src/lp_f8fwd.cuh:153-400)
through lp_conv_fwd_f8 / lp_conv_fwd_f4 against the oracle. Exact-operand cases are bit-exact in every output type; random data within
1e-3 max-abs-rel of the oracle's fp32-accumulated result, MX outputs equal up to neighbouring-code flips."""
import numpy as np
import pytest

import orc
import refnp
from gpuutil import gpu_conv, dev_gn, code_mismatch_fraction, lib

pytestmark = pytest.mark.gpu
GRID = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], np.float32)


def stored(x, xdt, N, Ci, S):
    if xdt >= 3:
        return orc.f32_to_mx(8 if xdt == 3 else 4, x, N, Ci, S)
    return np.ascontiguousarray(x.astype(np.float16).view(np.uint16)) if xdt == 2 else x


@pytest.fixture(params=[0, 2], ids=["zc_auto", "zc2"], autouse=True)
def stem_zc(request):
    """Every case runs with the launch's own choice of z tiles per workgroup (1 at these sizes) and with 2 forced (several tiles per
    workgroup, a ragged last group): the results may not depend on it."""
    lib.mi_conv_stem_zc(request.param)
    yield
    lib.mi_conv_stem_zc(0)


# (input type, Ci, Co, dims): the three channel paddings (4, 8, 16), one and several channel tiles and slices, ragged tiles, odd depths
SHAPES = [(3, 4, 32, (4, 8, 16)), (3, 4, 32, (5, 11, 21)), (3, 3, 16, (3, 9, 17)), (3, 8, 48, (4, 9, 18)), (3, 6, 64, (2, 8, 33)), (3, 4, 160, (3, 8, 16)),
          (4, 4, 32, (3, 8, 16)), (4, 8, 64, (4, 12, 20)), (2, 8, 32, (4, 8, 16)), (0, 16, 32, (3, 10, 17)), (0, 11, 24, (2, 8, 16)), (0, 2, 8, (3, 5, 7))]


@pytest.mark.parametrize("xdt,Ci,Co,dims", SHAPES)
def test_stem_exact_operands(gpu, xdt, Ci, Co, dims):
    rng = np.random.default_rng(xdt * 100 + Ci * 7 + Co)
    D, H, W = dims
    N, S = 2, D * H * W
    x = refnp.gen_exact(rng, (N, Ci, S), force6=False)
    w = refnp.gen_exact(rng, (Co, Ci, 27), force6=False)
    b = (GRID[rng.integers(0, 8, Co)] * 0.25).astype(np.float32)
    xin = stored(x, xdt, N, Ci, S)
    outs = (0, 3, 4) if xdt == 0 else (3, 4) if xdt == 2 else (3, 4)          # same type in and out, or an MX output
    G = 8 if Co % 8 == 0 else 1
    for ydt in outs:
        want, ws = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, ydt, stem_tile=1, acc64=1, Go=G, want_stats=True)
        got, gs = gpu_conv(xin, xdt, N, Ci, D, H, W, w, b, Co, ydt, Go=G, stats=True)      # (48 / 8 = 6 and 24 / 8 = 3 channels per group: per-channel records)
        assert "conv3_stem_k" in lib.mi_last_kernel().decode()
        assert np.array_equal(got, want), ydt
        if gs is not None:
            assert np.abs(gs - ws).max() / np.abs(ws).max() < 1e-5
    if xdt == 4:                                                              # the fp4 entry sends the network input to the same e4m3 kernel (src/lp_f4fwd.cu:37)
        want, _ = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, 4, stem_tile=1, acc64=1)
        got, _ = gpu_conv(xin, xdt, N, Ci, D, H, W, w, b, Co, 4, cbits=4)
        assert "conv3_stem_k" in lib.mi_last_kernel().decode() and np.array_equal(got, want)


@pytest.mark.parametrize("xdt,Ci,Co,dims", [(3, 4, 32, (6, 20, 40)), (3, 8, 64, (5, 9, 35)), (0, 16, 32, (4, 16, 32)), (2, 5, 32, (4, 8, 24))])
def test_stem_random_data(gpu, xdt, Ci, Co, dims):
    rng = np.random.default_rng(xdt + Ci + Co)
    D, H, W = dims
    N, S = 2, D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    x[:, :, S // 3] *= 40.0                                                   # tiles of very different scales
    w = (rng.standard_normal((Co, Ci, 27)) * np.sqrt(2.0 / (Ci * 27))).astype(np.float32)
    b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    xin = stored(x, xdt, N, Ci, S)
    if xdt == 0:
        want, _ = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, 0, stem_tile=1)
        got, _ = gpu_conv(xin, xdt, N, Ci, D, H, W, w, b, Co, 0)
        assert np.abs(got - want).max() / np.abs(want).max() < 2e-4
    wq, ws = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, 3, stem_tile=1, Go=8, want_stats=True, stored_stats=1)
    gq, gs = gpu_conv(xin, xdt, N, Ci, D, H, W, w, b, Co, 3, Go=8, stats=True, stored_stats=1)
    assert "conv3_stem_k" in lib.mi_last_kernel().decode()
    frac, near = code_mismatch_fraction(8, gq, wq, N, Co, S)
    assert frac < 5e-3 and near
    dec = orc.mx_to_f32(8, gq, N, Co, S).astype(np.float64).reshape(N, 8, -1)
    assert np.allclose(gs[:, :, 0], dec.sum(-1), rtol=1e-5, atol=1e-3) and np.allclose(gs[:, :, 1], (dec * dec).sum(-1), rtol=1e-5)
    gq2, gs2 = gpu_conv(xin, xdt, N, Ci, D, H, W, w, b, Co, 3, Go=8, stats=True, stored_stats=1)
    assert np.array_equal(gq, gq2) and np.array_equal(gs, gs2)                # run to run identical


@pytest.mark.parametrize("xdt", [3, 0])
def test_stem_with_groupnorm_input(gpu, xdt):
    rng = np.random.default_rng(40 + xdt)
    N, Ci, Co, D, H, W, G = 2, 8, 32, 4, 12, 20, 2
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci, 27)) * np.sqrt(2.0 / (Ci * 27))).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-.5, .5, Ci).astype(np.float32)
    mean = rng.uniform(-.2, .2, N * G).astype(np.float32); rstd = rng.uniform(.8, 1.2, N * G).astype(np.float32)
    xin = stored(x, xdt, N, Ci, S)
    want, _ = orc.conv3(xin, xdt, N, Ci, D, H, W, w, None, Co, 3, stem_tile=1, gp=orc.gn(gam, bet, mean, rstd, G))
    got, _ = gpu_conv(xin, xdt, N, Ci, D, H, W, w, None, Co, 3, gp=dev_gn(gam, bet, mean, rstd, G))
    assert "conv3_stem_k" in lib.mi_last_kernel().decode()
    frac, near = code_mismatch_fraction(8, got, want, N, Co, S)                # (the sigmoid runs on the hardware's fast exponential)
    assert frac < 2e-2 and near


def test_stem_nonfinite_and_weight_memo(gpu):
    rng = np.random.default_rng(3)
    N, Ci, Co, D, H, W = 1, 4, 32, 4, 16, 32
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci, 27)) * 0.1).astype(np.float32)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    a, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, None, Co, 3, wkey=77)
    b2, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, None, Co, 3, wkey=77)          # second call: prepared weights from the memo
    c, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, None, Co, 3)
    assert np.array_equal(a, b2) and np.array_equal(a, c)
    lib.lp_wmemo_clear()
    # a NaN makes its stored row's scale byte 0xFF, the row decodes to non-finite values, the tile's scale becomes 0xFF as well and every
    # output of the tiles whose halo holds the voxel is non-finite (NaN out of the MFMA's E8M0 0xFF; inf or NaN in the oracle's arithmetic);
    # all other tiles are untouched
    xn = x.copy(); xn[0, 2, 5] = np.nan
    xqn = orc.f32_to_mx(8, xn, N, Ci, S)
    want, _ = orc.conv3(xqn, 3, N, Ci, D, H, W, w, None, Co, 0 + 3, stem_tile=1)
    got, _ = gpu_conv(xqn, 3, N, Ci, D, H, W, w, None, Co, 3)
    dw, dg = orc.mx_to_f32(8, want, N, Co, S), orc.mx_to_f32(8, got, N, Co, S)
    fin = np.isfinite(dg)
    assert np.array_equal(np.isfinite(dw), fin) and not fin.all() and fin.any()
    assert np.array_equal(fin.reshape(Co, D, H, W)[0], fin.reshape(Co, D, H, W).all(0))            # whole voxels
    bad = ~fin.reshape(Co, D, H, W)[0]
    assert bad[:2, :8, :16].all() and bad.sum() == 2 * 8 * 16                                      # voxel 5 = (0, 0, 5): only the first tile's halo holds it
    clean, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, None, Co, 3)
    assert np.array_equal(orc.mx_to_f32(8, clean, N, Co, S)[fin], dg[fin])


# ---- 9 .. 16 channels of an MX or fp16 input: two taps per K block, one activation scale per staged row (src/lp_f8fwd.cuh:447-563) ----
@pytest.mark.parametrize("xdt,Ci,Co,dims", [(3, 16, 32, (4, 8, 16)), (3, 9, 16, (3, 9, 17)), (3, 12, 48, (5, 11, 21)), (4, 16, 32, (3, 8, 33)), (2, 10, 64, (2, 8, 16)), (3, 16, 96, (4, 16, 32))])
def test_row_scale_conv_exact_operands(gpu, xdt, Ci, Co, dims):
    rng = np.random.default_rng(xdt * 100 + Ci * 7 + Co)
    D, H, W = dims
    N, S = 2, D * H * W
    x = refnp.gen_exact(rng, (N, Ci, S), force6=False)
    w = refnp.gen_exact(rng, (Co, Ci, 27), force6=False)
    b = (GRID[rng.integers(0, 8, Co)] * 0.25).astype(np.float32)
    xin = stored(x, xdt, N, Ci, S)
    G = 8 if Co % 8 == 0 else 1
    for ydt in (3, 4):
        want, ws = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, ydt, stem_tile=2, acc64=1, Go=G, want_stats=True)
        got, gs = gpu_conv(xin, xdt, N, Ci, D, H, W, w, b, Co, ydt, Go=G, stats=True)      # (48 / 8 = 6 and 24 / 8 = 3 channels per group: per-channel records)
        assert "conv3_p16_k" in lib.mi_last_kernel().decode()
        assert np.array_equal(got, want), ydt
        if gs is not None:
            assert np.abs(gs - ws).max() / np.abs(ws).max() < 1e-5


@pytest.mark.parametrize("xdt,Ci,Co,dims,gn", [(3, 16, 32, (6, 20, 40), False), (3, 11, 64, (5, 9, 35), False), (2, 16, 32, (4, 8, 24), False), (3, 16, 32, (4, 12, 20), True)])
def test_row_scale_conv_random_data(gpu, xdt, Ci, Co, dims, gn):
    rng = np.random.default_rng(xdt + Ci + Co)
    D, H, W = dims
    N, S = 2, D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    x[:, :, S // 3] *= 40.0                                                   # rows of very different scales
    w = (rng.standard_normal((Co, Ci, 27)) * np.sqrt(2.0 / (Ci * 27))).astype(np.float32)
    b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    xin = stored(x, xdt, N, Ci, S)
    og = dg = None
    if gn:
        G = 4
        p = [rng.uniform(0.5, 1.5, Ci).astype(np.float32), rng.uniform(-.5, .5, Ci).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
        og, dg = orc.gn(*p, G), dev_gn(*p, G)
    wq, ws = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, 3, stem_tile=2, Go=8, want_stats=True, stored_stats=1, gp=og)
    gq, gs = gpu_conv(xin, xdt, N, Ci, D, H, W, w, b, Co, 3, Go=8, stats=True, stored_stats=1, gp=dg)
    assert "conv3_p16_k" in lib.mi_last_kernel().decode()
    frac, near = code_mismatch_fraction(8, gq, wq, N, Co, S)
    assert frac < (2e-2 if gn else 5e-3) and near
    dec = orc.mx_to_f32(8, gq, N, Co, S).astype(np.float64).reshape(N, 8, -1)
    assert np.allclose(gs[:, :, 0], dec.sum(-1), rtol=1e-5, atol=1e-3) and np.allclose(gs[:, :, 1], (dec * dec).sum(-1), rtol=1e-5)
