"""CPU tests that pin the oracle's convolution, epilogue, GroupNorm, upsample and head against independent numpy statements
(exact-operand construction of tests/test_mx4_wide.c:81-98: every partial sum is exact, so results must be EQUAL, not close)."""
import numpy as np
import pytest

import orc
import refnp


def mx_dec(bits, q, N, C, S):
    return orc.mx_to_f32(bits, q, N, C, S)


@pytest.mark.parametrize("bits,Ci,Co,dims,stride", [
    (8, 32, 32, (4, 6, 9), 1), (8, 64, 48, (3, 5, 7), 1), (4, 32, 64, (4, 6, 9), 1), (4, 96, 32, (3, 4, 5), 1),
    (8, 32, 32, (6, 8, 10), 2), (8, 64, 32, (5, 7, 9), 2), (4, 32, 32, (6, 6, 6), 2), (8, 40, 24, (3, 4, 6), 1)])
def test_exact_operand_conv_equals_fp64(bits, Ci, Co, dims, stride):
    rng = np.random.default_rng(Ci * 7 + Co + bits)
    D, H, W = dims
    N, S = 2, D * H * W
    x = refnp.gen_exact(rng, (N, Ci, S))
    w = refnp.gen_exact(rng, (Co, Ci, 27))
    b = (np.array([0, .5, 1, 1.5, 2, 3, 4, 6], np.float32)[rng.integers(0, 8, Co)] * 0.25).astype(np.float32)
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    assert np.array_equal(mx_dec(bits, xq, N, Ci, S), x)                       # the operand is stored losslessly
    want = refnp.conv3d_f64(x.reshape(N, Ci, D, H, W), w, b, stride)
    assert np.array_equal(want.astype(np.float32).astype(np.float64), want)    # the exactness premise holds
    y32, _ = orc.conv3(xq, 3 if bits == 8 else 4, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride)
    assert np.array_equal(y32.reshape(want.shape), want.astype(np.float32))
    y64, _ = orc.conv3(xq, 3 if bits == 8 else 4, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride, acc64=1)
    assert np.array_equal(y64, y32)
    # MX output == the format-definition quantiser of the exact conv (cmp_mx, tests/test_mx4_wide.c:252-265), both output formats
    So = want.shape[2] * want.shape[3] * want.shape[4]
    for ob in (8, 4):
        yq, _ = orc.conv3(xq, 3 if bits == 8 else 4, N, Ci, D, H, W, w, b, Co, 3 if ob == 8 else 4, cbits=bits, stride=stride)
        assert np.array_equal(mx_dec(ob, yq, N, Co, So), refnp.mx_quant_tensor(want.astype(np.float32).reshape(N, Co, So), ob))


def test_centre_tap_identity_reads_back_operand():
    """A conv whose only non-zero weights are 1 on the centre tap diagonal returns the staged operand (tests/test_mx4_wide.c:13-15)."""
    rng = np.random.default_rng(5)
    N, C, D, H, W = 1, 32, 3, 4, 5
    S = D * H * W
    x = rng.standard_normal((N, C, S)).astype(np.float32)
    w = np.zeros((C, C, 27), np.float32)
    w[np.arange(C), np.arange(C), 13] = 1.0
    for bits in (8, 4):
        xq = orc.f32_to_mx(bits, x, N, C, S)
        y, _ = orc.conv3(xq, 3 if bits == 8 else 4, N, C, D, H, W, w, None, C, 0, cbits=bits)
        assert np.array_equal(y, mx_dec(bits, xq, N, C, S))


def test_plane_input_staging_equals_converter():
    """fp32 planes quantised in staging == lp_f32_to_mx8 of the tensor followed by the copy path when Ci % 32 == 0 (src/lp_f8fwd.cuh:88-113)."""
    rng = np.random.default_rng(6)
    N, C, D, H, W = 1, 64, 3, 4, 6
    S = D * H * W
    x = rng.standard_normal((N, C, S)).astype(np.float32)
    w = (rng.standard_normal((32, C, 27)) * 0.05).astype(np.float32)
    y0, _ = orc.conv3(x, 0, N, C, D, H, W, w, None, 32, 0, cbits=8)
    y1, _ = orc.conv3(orc.f32_to_mx(8, x, N, C, S), 3, N, C, D, H, W, w, None, 32, 0, cbits=8)
    assert np.array_equal(y0, y1)


def test_random_conv_close_to_fp64_of_dequantised_operands():
    """fp32 accumulation of the block products stays within 1e-5 (max-abs-rel) of the fp64 conv of the same dequantised operands."""
    rng = np.random.default_rng(7)
    N, Ci, Co, D, H, W = 1, 64, 32, 4, 5, 6
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci, 27)) * np.sqrt(2 / (27 * Ci))).astype(np.float32)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    xd = mx_dec(8, xq, N, Ci, S)
    wd = np.moveaxis(refnp.quantize_block(np.moveaxis(w.reshape(Co, Ci // 32, 32, 27), 2, -1), 8)[0], -1, 2).reshape(Co, Ci, 27)   # blocks of 32 ci per (co, tap)
    want = refnp.conv3d_f64(xd.reshape(N, Ci, D, H, W), wd)
    y, _ = orc.conv3(xq, 3, N, Ci, D, H, W, w, None, Co, 0, cbits=8)
    assert np.abs(y.reshape(want.shape) - want).max() / np.abs(want).max() < 1e-5


def test_gn_stats_and_finalize():
    rng = np.random.default_rng(8)
    N, Ci, Co, D, H, W, G = 2, 32, 32, 3, 4, 5, 8
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci, 27)) * 0.1).astype(np.float32)
    b = rng.standard_normal(Co).astype(np.float32)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    y32, s0 = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 0, cbits=8, Go=G, want_stats=True)
    g = y32.astype(np.float64).reshape(N, G, -1)
    assert np.allclose(s0[:, :, 0], g.sum(-1), rtol=1e-12) and np.allclose(s0[:, :, 1], (g * g).sum(-1), rtol=1e-12)
    # stored statistics = sums of the decoded stored tensor (tests/test_gn_contract.c:1-2)
    yq, s1 = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 3, cbits=8, Go=G, want_stats=True, stored_stats=1)
    d = mx_dec(8, yq, N, Co, S).astype(np.float64).reshape(N, G, -1)
    assert np.allclose(s1[:, :, 0], d.sum(-1), rtol=1e-12) and np.allclose(s1[:, :, 1], (d * d).sum(-1), rtol=1e-12)
    sums = np.zeros((N * G, 2)); orc.lib().orc_gn_sums_mx(8, orc.ptr(yq), N, Co, G, S, orc.ptr(sums), 0, S)
    assert np.allclose(sums.reshape(N, G, 2), s1, rtol=1e-12)
    # finalize (src/nn_elem.cu:5-11) against numpy, and the constant-group invariant: var 0 -> rstd = 1 / sqrt(eps)
    mean = np.zeros(N * G, np.float32); rstd = np.zeros(N * G, np.float32)
    length = (Co // G) * S
    orc.lib().orc_gn_finalize(orc.ptr(s0), N * G, length, 1e-5, orc.ptr(mean), orc.ptr(rstd))
    assert np.allclose(mean.reshape(N, G), g.mean(-1), rtol=1e-6, atol=1e-7)
    assert np.allclose(rstd.reshape(N, G), 1 / np.sqrt(g.var(-1) + 1e-5), rtol=1e-5)
    const = np.array([[3.5 * length, 3.5 * 3.5 * length]])
    orc.lib().orc_gn_finalize(orc.ptr(const), 1, length, 1e-5, orc.ptr(mean), orc.ptr(rstd))
    assert mean[0] == np.float32(3.5) and abs(rstd[0] - 1 / np.sqrt(1e-5)) < 1e-2


def test_gn_silu_staging_matches_double_precision():
    """GN + SiLU applied while staging: staged values are the quantised double-precision silu(a x + b) (gn_silu, tests/test_mx4_wide.c:118-121)."""
    rng = np.random.default_rng(9)
    N, C, D, H, W, G = 1, 32, 2, 3, 4, 8
    S = D * H * W
    x = rng.standard_normal((N, C, S)).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, C).astype(np.float32); bet = rng.uniform(-0.5, 0.5, C).astype(np.float32)
    mean = rng.uniform(-0.2, 0.2, N * G).astype(np.float32); rstd = rng.uniform(0.8, 1.2, N * G).astype(np.float32)
    xq = orc.f32_to_mx(8, x, N, C, S)
    c = orc.orc_conv_t()
    c.x, c.xdt, c.N, c.Ci, c.D, c.H, c.W, c.cbits, c.stride = orc.ptr(xq), 3, N, C, D, H, W, 8, 1
    c.gp = orc.gn(gam, bet, mean, rstd, G)
    st = np.zeros((N, 1, S, 32), np.float32)
    assert orc.lib().orc_conv3_staged(c, orc.ptr(st)) == 32
    xd = mx_dec(8, xq, N, C, S).astype(np.float64)
    a = (rstd[np.arange(C) // (C // G)] * gam).astype(np.float32)
    b = (bet.astype(np.float64) - mean[np.arange(C) // (C // G)].astype(np.float64) * a).astype(np.float32)
    u = (xd[0] * a[:, None].astype(np.float64) + b[:, None]).astype(np.float32).astype(np.float64)
    act = (u / (1 + np.exp(-u))).astype(np.float32)
    want, _ = refnp.quantize_block(act.T, 8)
    # floor / ceil neighbour acceptance as the reference (rn_near_ok): the affine is one fp32 FMA in the oracle, two roundings here
    got = st[0, 0]
    step = np.abs(want) * 2.0 ** -3 + 2.0 ** -20
    assert (np.abs(got - want) <= step).all()
    assert (got == want).mean() > 0.99


def test_up2_closed_form_on_grid_data():
    rng = np.random.default_rng(10)
    N, C, D, H, W = 1, 32, 3, 4, 5
    x = refnp.gen_exact(rng, (N, C, D * H * W))
    x[:, 5, :] = 6.0                                            # every blend's amax is 6 (gen_x6, tests/test_mx4_wide.c:87-91)
    xq = orc.f32_to_mx(8, x, N, C, D * H * W)
    y = np.zeros(orc.mx_bytes(8, N, C, 8 * D * H * W), np.uint8)
    orc.lib().orc_up2_mx(8, orc.ptr(xq), N, C, D, H, W, orc.gn(), orc.ptr(y), 8)
    got = mx_dec(8, y, N, C, 8 * D * H * W)
    want = refnp.up2_f64(x.reshape(N, C, D, H, W)).reshape(N, C, -1)
    # blends of grid values are multiples of 2^-7 below 6: exact in fp32 and within e4m3's range only after rounding -> compare with the quantiser
    assert np.array_equal(got, refnp.mx_quant_tensor(want.astype(np.float32), 8))
    # interior point closed form and the edge clamp
    xv = x.reshape(N, C, D, H, W).astype(np.float64)
    assert want.reshape(N, C, 2 * D, 2 * H, 2 * W)[0, 0, 0, 0, 0] == xv[0, 0, 0, 0, 0]
    assert want.reshape(N, C, 2 * D, 2 * H, 2 * W)[0, 0, 1, 0, 0] == 0.75 * xv[0, 0, 0, 0, 0] + 0.25 * xv[0, 0, 1, 0, 0]


def test_head_is_a_dot_product():
    rng = np.random.default_rng(11)
    N, Ci, Co, S = 2, 48, 8, 100
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = rng.standard_normal((Co, Ci)).astype(np.float32); b = rng.standard_normal(Co).astype(np.float32)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    y = np.zeros((N, Co, S), np.float32)
    orc.lib().orc_conv1_mx(8, orc.ptr(xq), N, Ci, S, orc.ptr(w), orc.ptr(b), Co, orc.gn(), orc.ptr(y))
    want = np.einsum("oc,ncs->nos", w.astype(np.float64), mx_dec(8, xq, N, Ci, S).astype(np.float64)) + b[None, :, None]
    assert np.abs(y - want).max() / np.abs(want).max() < 1e-5             # tests/test_mx.c:209


def test_fused_upsample_staging_exact_on_grid():
    """Decoder conv1 reading [up2(coarse) | skip]: on grid data with a 6 in every block the blend is exact, so the conv of the fused
    staging equals the conv of the materialised concatenation (tests/test_mx4_wide.c:392-427)."""
    rng = np.random.default_rng(12)
    N, Cu, Cs, Co, D, H, W = 1, 32, 32, 32, 4, 4, 6
    S, Sc = D * H * W, (D // 2) * (H // 2) * (W // 2)
    xc = refnp.gen_exact(rng, (N, Cu, Sc)); xc[:, 5, :] = 6.0
    sk = refnp.gen_exact(rng, (N, Cs, S))
    w = refnp.gen_exact(rng, (Co, Cu + Cs, 27))
    xcq = orc.f32_to_mx(8, xc, N, Cu, Sc); skq = orc.f32_to_mx(8, sk, N, Cs, S)
    y, _ = orc.conv3(xcq, 3, N, Cu + Cs, D, H, W, w, None, Co, 0, cbits=8, x2=skq, c_split=Cu, up=1)
    up = refnp.up2_f64(xc.reshape(N, Cu, D // 2, H // 2, W // 2)).reshape(N, Cu, S).astype(np.float32)
    upq = refnp.mx_quant_tensor(up, 8)                          # staged operand: the blend re-quantised to e4m3 per (voxel, 32 channels)
    cat = np.concatenate([upq, sk], axis=1).reshape(N, Cu + Cs, D, H, W)
    # weights are exact, the staged operand is on the e4m3 grid: the fp64 conv is the reference; fp32 accumulation error only
    want = refnp.conv3d_f64(cat, w)
    assert np.abs(y.reshape(want.shape) - want).max() <= 1e-6 * np.abs(want).max()
