"""Pins of the oracle's tap-packed stem conv (orc_conv3 with stem_tile; src/lp_f8fwd.cuh:153-400), none of them a retyped formula:
exact operands reduce it to a plain fp64 convolution (pins tap packing, channel padding, tile walk and ragged edges); a single large
value must coarsen exactly the output voxels of the 2 x 8 x 16 tiles whose 4 x 10 x 18 halo holds it (pins the tile geometry and that
the scale is the tile's, not the position's); with one tile per volume the operand equals the tensor quantised with ONE scale."""
import numpy as np
import pytest

import orc
import refnp

GRID = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], np.float32)


def stored(x, xdt, N, Ci, S):
    if xdt >= 3:
        return orc.f32_to_mx(8 if xdt == 3 else 4, x, N, Ci, S)
    return np.ascontiguousarray(x.astype(np.float16).view(np.uint16)) if xdt == 2 else x


@pytest.mark.parametrize("xdt,Ci,Co,dims", [(3, 4, 32, (4, 8, 16)), (3, 4, 32, (5, 11, 21)), (3, 3, 16, (3, 9, 17)), (3, 8, 48, (4, 9, 18)), (3, 6, 64, (2, 8, 33)),
                                            (4, 4, 32, (3, 8, 16)), (2, 8, 32, (4, 8, 16)), (0, 16, 32, (3, 10, 17)), (0, 11, 24, (2, 8, 16)), (0, 2, 8, (3, 5, 7))])
def test_exact_operands_equal_fp64_conv(xdt, Ci, Co, dims):
    rng = np.random.default_rng(xdt * 100 + Ci * 7 + Co)
    D, H, W = dims
    N, S = 2, D * H * W
    x = refnp.gen_exact(rng, (N, Ci, S), force6=False)             # e2m1-grid values: exact under any power-of-two tile scale
    w = refnp.gen_exact(rng, (Co, Ci, 27), force6=False)
    b = (GRID[rng.integers(0, 8, Co)] * 0.25).astype(np.float32)
    want = refnp.conv3d_f64(x.reshape(N, Ci, D, H, W), w, b, 1)
    assert np.array_equal(want.astype(np.float32).astype(np.float64), want)
    xin = stored(x, xdt, N, Ci, S)
    y32, _ = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, 0, stem_tile=1)
    assert np.array_equal(y32.reshape(want.shape), want.astype(np.float32))
    y64, sums = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, 0, stem_tile=1, acc64=1, Go=Co // 8 if Co % 8 == 0 else 1, want_stats=True)
    assert np.array_equal(y64, y32)
    G = sums.shape[1]
    assert np.allclose(sums[:, :, 0], want.reshape(N, G, -1).sum(-1)) and np.allclose(sums[:, :, 1], (want * want).reshape(N, G, -1).sum(-1))
    yq, _ = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, 3, stem_tile=1)
    assert np.array_equal(orc.mx_to_f32(8, yq, N, Co, S), refnp.mx_quant_tensor(want.astype(np.float32).reshape(N, Co, S), 8))


def test_one_large_value_coarsens_exactly_its_tiles():
    rng = np.random.default_rng(5)
    N, Ci, Co, D, H, W = 1, 4, 8, 6, 20, 40
    S = D * H * W
    # small values that need many bits under the spike's scale: 2^-12 multiples, exact under their own tile scale (amax < 2^-6)
    x = (rng.integers(-3, 4, (N, Ci, D, H, W)) * 2.0 ** -10).astype(np.float32)
    zs, ys, xs = 2, 8, 15                                            # at a tile corner: halos of several tiles hold it
    x[0, 1, zs, ys, xs] = 384.0
    w = refnp.gen_exact(rng, (Co, Ci, 27), force6=False)
    y, _ = orc.conv3(np.ascontiguousarray(x.reshape(N, Ci, S)), 0, N, Ci, D, H, W, w, None, Co, 0, stem_tile=1)
    exact = refnp.conv3d_f64(x.astype(np.float64), w, None, 1).astype(np.float32).reshape(N, Co, D, H, W)
    # with the spike's scale (e = mx_exp(384 / 448) = 0 .. the e4m3 quantum near zero is 2^-9) the small values round to 0 or +-2^-9:
    xc = x.copy(); small = np.abs(xc) < 1.0
    steps = np.arange(-8, 9, dtype=np.float32)
    xc[small] = steps[refnp.round_to_grid(xc[small] * 512.0, steps)] / 512.0
    coarse = refnp.conv3d_f64(xc.astype(np.float64), w, None, 1).astype(np.float32).reshape(N, Co, D, H, W)
    y = y.reshape(N, Co, D, H, W)
    hit = np.zeros((D, H, W), bool)
    for tz in range((D + 1) // 2):
        for ty in range((H + 7) // 8):
            for tx in range((W + 15) // 16):
                if 2 * tz - 1 <= zs <= 2 * tz + 2 and 8 * ty - 1 <= ys <= 8 * ty + 8 and 16 * tx - 1 <= xs <= 16 * tx + 16:
                    hit[2 * tz:2 * tz + 2, 8 * ty:8 * ty + 8, 16 * tx:16 * tx + 16] = True
    assert hit.sum() == 8 * 256                                      # the corner position lies in the halo of 2 x 2 x 2 tiles
    assert np.array_equal(y[:, :, ~hit], exact[:, :, ~hit])
    assert np.array_equal(y[:, :, hit], coarse[:, :, hit])
    assert not np.array_equal(coarse[:, :, hit], exact[:, :, hit])


def test_single_tile_uses_one_scale_for_the_whole_operand():
    rng = np.random.default_rng(8)
    N, Ci, Co, D, H, W = 1, 4, 4, 2, 8, 16                           # one tile: the operand is the tensor under one E8M0 scale
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = np.zeros((Co, Ci, 27), np.float32); w[np.arange(4), np.arange(4), 13] = 1.0          # centre-tap identity
    y, _ = orc.conv3(x, 0, N, Ci, D, H, W, w, None, Co, 0, stem_tile=1)
    e = refnp.scale_exp(np.abs(x).max(), 448.0)
    q = np.array([orc.lib().orc_dec_e4m3(orc.lib().orc_enc_e4m3(float(v))) for v in (x * np.float32(2.0 ** -e)).ravel()], np.float32).reshape(x.shape) * np.float32(2.0 ** e)
    assert np.array_equal(y, q)


# ---- the 9 .. 16 channel packed conv: two taps per K block, one activation scale per staged row (src/lp_f8fwd.cuh:447-563) ----
@pytest.mark.parametrize("xdt,Ci,Co,dims", [(3, 16, 32, (4, 8, 16)), (3, 9, 16, (3, 9, 17)), (3, 12, 48, (5, 11, 21)), (4, 16, 32, (3, 8, 33)), (2, 10, 64, (2, 8, 16))])
def test_row_scale_conv_exact_operands_equal_fp64_conv(xdt, Ci, Co, dims):
    rng = np.random.default_rng(xdt * 100 + Ci * 7 + Co)
    D, H, W = dims
    N, S = 2, D * H * W
    x = refnp.gen_exact(rng, (N, Ci, S), force6=False)
    w = refnp.gen_exact(rng, (Co, Ci, 27), force6=False)
    b = (GRID[rng.integers(0, 8, Co)] * 0.25).astype(np.float32)
    want = refnp.conv3d_f64(x.reshape(N, Ci, D, H, W), w, b, 1)
    assert np.array_equal(want.astype(np.float32).astype(np.float64), want)
    xin = stored(x, xdt, N, Ci, S)
    y32, _ = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, 0, stem_tile=2)
    assert np.array_equal(y32.reshape(want.shape), want.astype(np.float32))
    yq, _ = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, 3, stem_tile=2)
    assert np.array_equal(orc.mx_to_f32(8, yq, N, Co, S), refnp.mx_quant_tensor(want.astype(np.float32).reshape(N, Co, S), 8))


def test_row_scale_conv_one_large_value_coarsens_exactly_its_row():
    rng = np.random.default_rng(6)
    N, Ci, Co, D, H, W = 1, 12, 8, 5, 12, 40
    S = D * H * W
    x = (rng.integers(-3, 4, (N, Ci, D, H, W)) * 2.0 ** -10).astype(np.float32)
    zs, ys, xs = 2, 5, 8                                             # inside the first 16-wide x tile only (its rows span x = -1 .. 16)
    x[0, 3, zs, ys, xs] = 384.0
    w = refnp.gen_exact(rng, (Co, Ci, 27), force6=False)
    y, _ = orc.conv3(orc.f32_to_mx(8, x.reshape(N, Ci, S), N, Ci, S), 3, N, Ci, D, H, W, w, None, Co, 0, stem_tile=2)
    xs_in = orc.mx_to_f32(8, orc.f32_to_mx(8, x.reshape(N, Ci, S), N, Ci, S), N, Ci, S).reshape(N, Ci, D, H, W)   # the stored operand (the spike's own
    exact = refnp.conv3d_f64(xs_in.astype(np.float64), w, None, 1).astype(np.float32).reshape(N, Co, D, H, W)   # voxel row is coarse already)
    xc = xs_in.copy()
    steps = np.arange(-8, 9, dtype=np.float32)
    seg = xc[0, :, zs, ys, 0:17]; small = np.abs(seg) < 1.0          # the staged row of tile 0: x = -1 .. 16, under the spike's scale 2^0
    seg[small] = steps[refnp.round_to_grid(seg[small] * 512.0, steps)] / 512.0
    xc[0, :, zs, ys, 0:17] = seg
    coarse = refnp.conv3d_f64(xc.astype(np.float64), w, None, 1).astype(np.float32).reshape(N, Co, D, H, W)
    y = y.reshape(N, Co, D, H, W)
    assert np.array_equal(y[..., :16], coarse[..., :16])             # outputs of the x tile whose row holds the value
    assert np.array_equal(y[..., 16:], exact[..., 16:])              # the next tile quantises x = 15, 16 of that line with its own row scale
    assert not np.array_equal(coarse[..., :16], exact[..., :16])
    far = np.ones((D, H), bool); far[zs - 1:zs + 2, ys - 1:ys + 2] = False
    assert np.array_equal(y[:, :, far], exact[:, :, far])            # only outputs whose taps read that (z, y) line
