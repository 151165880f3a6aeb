"""CPU tests (no GPU) that pin the oracle's elementwise functions the GPU tests use as their checker: the 16-bit -> MX converter, the
network input rows and the materialising GroupNorm + SiLU. Each is compared with a numpy statement written from the formulas the
reference states (src/lp_mx_cvt.cu:20-41, src/lp_mx_gn.cu:5-21), quantised by the independent block quantiser of refnp: a dropped
term, a wrong channel slot, a missing 16-bit rounding or a sign mistake fails one of them."""
import numpy as np
import pytest

import orc
import refnp


def decoded(bits, q, N, C, S):
    return orc.mx_to_f32(bits, q, N, C, S)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("C", [4, 12, 48, 70])
def test_h16_to_mx_equals_numpy_half_then_block_quantiser(bits, C):
    """orc_h16_to_mx = (fp16 bits -> the value numpy's float16 holds) -> the format's block quantiser, for every block width and a ragged
    last block; decoded values are compared, and the scale bytes against the independent scale rule."""
    rng = np.random.default_rng(100 + C)
    N, S = 2, 257
    xh = (rng.standard_normal((N, C, S)) * np.exp(rng.uniform(-6, 6, (N, 1, S)))).astype(np.float16)
    xh[0, 0, :7] = np.array([0.0, -0.0, 6e-8, -6e-8, 65504.0, -65504.0, 2.0 ** -14], np.float16)      # zeros, subnormals, the largest value
    want = refnp.mx_quant_tensor(xh.astype(np.float32), bits)
    got = np.zeros(orc.mx_bytes(bits, N, C, S), np.uint8)
    orc.lib().orc_h16_to_mx(bits, orc.ptr(np.ascontiguousarray(xh.view(np.uint16))), N, C, S, orc.ptr(got))
    assert np.array_equal(decoded(bits, got, N, C, S), want)
    # ... and it is the fp32 converter applied to the widened values, byte for byte (signed zeros and scale bytes included)
    assert np.array_equal(got, orc.f32_to_mx(bits, xh.astype(np.float32), N, C, S))
    bw = 8 if C <= 8 else 16 if C <= 16 else 32
    nb = (C + bw - 1) // bw
    sc = got[N * nb * S * (bw * bits // 8):].reshape(N, nb, S)
    pad = np.zeros((N, nb * bw, S), np.float32); pad[:, :C] = np.abs(xh.astype(np.float32))
    assert np.array_equal(sc.astype(np.int64) - 127, refnp.scale_exp(pad.reshape(N, nb, bw, S).max(axis=2), 448.0 if bits == 8 else 6.0))


def np_pred_input(ct, W, mean, isd, dyo, dxo, axis, z0, nz, hd):
    """The network input of src/lp_mx_cvt.cu:29-41 in numpy fp32: channel 0 the z-scored CT, 1 zero, 2 / 3 the unit direction away from the
    axis, d * axis / (sqrt(dy^2 + dx^2) + 1e-6) (the sum of squares with one fused multiply-add, evaluated exactly in float64 and rounded
    once), every value rounded to the 16-bit input type; channels 4-7 of the 8-wide row are zero."""
    f32 = np.float32
    z = np.arange(z0, z0 + nz)
    dy = (dyo[z][:, None, None] + np.arange(W, dtype=f32)[None, :, None]).astype(f32) + np.zeros((1, 1, W), f32)
    dx = (dxo[z][:, None, None] + np.arange(W, dtype=f32)[None, None, :]).astype(f32) + np.zeros((1, W, 1), f32)
    r = np.zeros((8, nz, W, W), f32)
    r[0] = ((ct[z0:z0 + nz].astype(f32) - f32(mean)) * f32(isd)).astype(f32)
    if axis:
        dxx = (dx * dx).astype(f32)
        ss = (dy.astype(np.float64) * dy.astype(np.float64) + dxx.astype(np.float64)).astype(f32)       # fma(dy, dy, dx * dx): one rounding
        inv = (f32(axis) / (np.sqrt(ss).astype(f32) + f32(1e-6))).astype(f32)
    else:
        inv = np.zeros_like(dy)
    r[2] = dy * inv; r[3] = dx * inv
    if hd == 2:
        r = r.astype(np.float16).astype(f32)
    elif hd == 1:
        u = r.view(np.uint32).astype(np.uint64)
        r = (((u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000).astype(np.uint32)).view(f32)
    return r.reshape(1, 8, nz * W * W)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("z0,nz,hd,axis", [(0, 5, 2, 1), (1, 3, 0, -1), (0, 5, 2, 0), (2, 2, 0, 0), (0, 4, 1, 1)])
def test_pred_input_equals_numpy_formula(bits, z0, nz, hd, axis):
    rng = np.random.default_rng(7 + hd + axis)
    W, D = 20, 5
    ct = np.clip(np.where(rng.random((D, W, W)) < 0.5, rng.normal(60, 20, (D, W, W)), rng.normal(170, 20, (D, W, W))), 0, 255).astype(np.uint8)
    dyo = rng.uniform(-15, 5, D).astype(np.float32); dxo = rng.uniform(-15, 5, D).astype(np.float32)     # the axis crosses the window: both signs
    dyo[0] = -3.0; dxo[0] = -4.0                                      # a voxel exactly on the axis (d = 0) in plane 0
    mean, isd = float(ct.mean()), float(1 / ct.std())
    S = nz * W * W
    got = np.zeros(orc.mx_bytes(bits, 1, 4, S), np.uint8)
    orc.lib().orc_pred_input_mx(bits, orc.ptr(ct), W, mean, isd, orc.ptr(dyo), orc.ptr(dxo), axis, z0, nz, orc.ptr(got), hd)
    r = np_pred_input(ct, W, mean, isd, dyo, dxo, axis, z0, nz, hd)
    want = refnp.mx_quant_tensor(r, bits)
    rows = np.zeros((S, 8), np.float32)
    rb = 8 * bits // 8
    L = orc.lib()
    for v in range(S):                                                # (rows of 8: decode through the row routine; a 4-channel tensor's accessor stops at channel 3)
        L.orc_load_row(bits, got[v * rb:].ctypes.data, int(got[S * rb + v]), 8, rows[v].ctypes.data)
    dec = np.ascontiguousarray(rows.T)[None]
    assert np.array_equal(dec[0, :, :], np.ascontiguousarray(want[0]).reshape(8, S))
    assert not dec[0, 1].any() and not dec[0, 4:].any()              # channel 1 and the padding channels are zero
    # signed zeros (src/lp_mx_cvt.cu:33-39): without an axis the direction channels are d * 0 = zeros carrying the sign of d, which the
    # 16-bit rounding and the element encoders keep; channel 1 and the padding are +0
    codes = got[:S * rb].reshape(S, rb)
    def code(ch):
        return codes[:, ch] if bits == 8 else (codes[:, ch // 2] >> (4 * (ch & 1))) & 15
    sign = 0x80 if bits == 8 else 8
    assert not (code(1) & sign).any() and not (code(5) & sign).any()
    if axis == 0:
        dyv = r[0, 2]; dy_neg = np.signbit(dyv)
        assert np.array_equal((code(2) & sign) != 0, dy_neg) and np.array_equal((code(3) & sign) != 0, np.signbit(r[0, 3]))
        assert dy_neg.any() and (~dy_neg).any()
        assert not (code(2) & ~np.uint8(sign) & 0xff).any()
    else:
        n2 = dec[0, 2].astype(np.float64) ** 2 + dec[0, 3].astype(np.float64) ** 2
        on_axis = (r[0, 2] == 0) & (r[0, 3] == 0)
        assert np.all(np.abs(np.sqrt(n2[~on_axis]) - 1) < (0.07 if bits == 8 else 0.35))      # unit vectors up to the quantisation
        if z0 == 0:
            assert on_axis.sum() == 1                                 # the voxel on the axis: 0 / 1e-6 = 0


def np_silu_gn(x, N, C, S, G, gam, bet, mean, rstd):
    cpg = C // G
    m = np.repeat(mean.reshape(N, G), cpg, axis=1)[:, :, None].astype(np.float32)
    r = np.repeat(rstd.reshape(N, G), cpg, axis=1)[:, :, None].astype(np.float32)
    t = ((x - m).astype(np.float32) * r).astype(np.float32)
    v = (t.astype(np.float64) * gam[None, :, None].astype(np.float64) + bet[None, :, None].astype(np.float64)).astype(np.float32)   # one fused multiply-add
    return v, (v.astype(np.float64) / (1.0 + np.exp(-v.astype(np.float64))))


@pytest.mark.parametrize("xdt,ybits,C", [(3, 8, 64), (4, 4, 64), (3, 4, 48), (0, 8, 12), (4, 8, 8)])
def test_gn_silu_apply_equals_fp64_silu_then_block_quantiser(xdt, ybits, C):
    """orc_gn_silu_apply_mx = decode -> (x - mean) rstd gamma + beta -> v / (1 + exp(-v)) in fp64 -> the block quantiser. Codes are the
    independent quantiser's or (where the fp32 rounding of the activation sits on a rounding boundary) its floor / ceil neighbour: the
    reference's own acceptance (rn_near_ok, tests/test_mx4_wide.c:165-175); closed-form checks pin the transform itself."""
    rng = np.random.default_rng(200 + C + ybits)
    N, S, G = 2, 300, 4
    x = (rng.standard_normal((N, C, S)) * 2).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, C).astype(np.float32); bet = rng.uniform(-.5, .5, C).astype(np.float32)
    mean = rng.uniform(-.3, .3, N * G).astype(np.float32); rstd = rng.uniform(.7, 1.3, N * G).astype(np.float32)
    if xdt >= 3:
        xin = orc.f32_to_mx(8 if xdt == 3 else 4, x, N, C, S)
        xv = orc.mx_to_f32(8 if xdt == 3 else 4, xin, N, C, S)
    else:
        xin, xv = x, x
    got = np.zeros(orc.mx_bytes(ybits, N, C, S), np.uint8)
    orc.lib().orc_gn_silu_apply_mx(orc.ptr(xin), xdt, N, C, S, orc.gn(gam, bet, mean, rstd, G), orc.ptr(got), ybits)
    gd = decoded(ybits, got, N, C, S)
    v, act = np_silu_gn(xv, N, C, S, G, gam, bet, mean, rstd)
    want = refnp.mx_quant_tensor(act.astype(np.float32), ybits)
    assert (gd != want).mean() < 1e-3                                # only where float32(act) is a rounding boundary case
    step = 0.26 if ybits == 8 else 0.67
    assert np.all(np.abs(gd - want) <= step * np.maximum(np.abs(want), np.abs(gd)) + 1e-30)


def test_gn_silu_apply_closed_forms():
    """Invariants no quantiser detail can hide: a constant group under its own statistics gives silu(beta) everywhere; gamma = 0 likewise;
    large positive inputs pass through (silu(v) -> v), large negative ones vanish; the group -> channel mapping is per sample."""
    N, C, S, G = 2, 32, 64, 8
    x = np.zeros((N, C, S), np.float32)
    for n in range(N):
        for g in range(G):
            x[n, 4 * g:4 * g + 4] = 1.5 * (g + 1) * (1 if n == 0 else -1)
    mean = np.array([x[n, 4 * g, 0] for n in range(N) for g in range(G)], np.float32)        # every group's own mean: (x - mean) = 0
    rstd = np.full(N * G, 316.22777, np.float32)                                             # 1 / sqrt(eps)
    gam = np.linspace(0.5, 2, C).astype(np.float32); bet = np.linspace(-4, 4, C).astype(np.float32)
    got = np.zeros(orc.mx_bytes(8, N, C, S), np.uint8)
    orc.lib().orc_gn_silu_apply_mx(orc.ptr(x), 0, N, C, S, orc.gn(gam, bet, mean, rstd, G), orc.ptr(got), 8)
    want = bet.astype(np.float64) / (1 + np.exp(-bet.astype(np.float64)))
    gd = decoded(8, got, N, C, S)
    assert np.all(np.abs(gd - want[None, :, None]) <= 2.0 ** -4 * np.abs(want[None, :, None]) + np.abs(want).max() * 2.0 ** -9)
    # swapping the samples' statistics must change the result (per-sample groups): with sample 1's means sample 0 is no longer centred
    got2 = np.zeros_like(got)
    orc.lib().orc_gn_silu_apply_mx(orc.ptr(x), 0, N, C, S, orc.gn(gam, bet, np.ascontiguousarray(mean.reshape(N, G)[::-1]).reshape(-1), rstd, G), orc.ptr(got2), 8)
    assert not np.array_equal(got, got2)
    # pass-through and vanishing tails
    big = np.full((1, 32, 8), 40.0, np.float32); big[0, 16:] = -40.0
    one = np.ones(32, np.float32); zero = np.zeros(32, np.float32)
    got3 = np.zeros(orc.mx_bytes(8, 1, 32, 8), np.uint8)
    orc.lib().orc_gn_silu_apply_mx(orc.ptr(big), 0, 1, 32, 8, orc.gn(one, zero, np.zeros(1, np.float32), np.ones(1, np.float32), 1), orc.ptr(got3), 8)
    d3 = decoded(8, got3, 1, 32, 8)
    assert np.all(d3[0, :16] == 40.0) and np.all(d3[0, 16:] == 0.0) and np.all(np.signbit(d3[0, 16:]))      # silu(-40) = -1.7e-16: rounds to -0
