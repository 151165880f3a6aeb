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


# ---- the binary16 upsample blend of the fp4 decoder conv (stage_up_smem_h2, src/lp_common.cuh:674-712) ----
from bisect import bisect_left
from fractions import Fraction

_H16 = None


def _half_values():
    """Every finite non-negative binary16 value as an exact fraction, ascending, with its bit pattern's parity (for ties)."""
    global _H16
    if _H16 is None:
        bits = np.arange(0, 0x7c00, dtype=np.uint16)
        _H16 = [Fraction(float(v)) for v in bits.view(np.float16).astype(np.float64)]
    return _H16


def half_round(x):
    """Exact rational -> nearest binary16 value (ties to the even bit pattern), as a float; overflow past 65520 -> inf."""
    vals = _half_values()
    s = -1.0 if x < 0 else 1.0
    a = abs(x)
    if a >= Fraction(65520):
        return s * float("inf")
    i = bisect_left(vals, a)
    if i < len(vals) and vals[i] == a:
        return s * float(vals[i])
    lo, hi = i - 1, i
    if hi >= len(vals):
        return s * float(vals[lo])                      # between 65504 and 65520
    dl, dh = a - vals[lo], vals[hi] - a
    k = lo if dl < dh else hi if dh < dl else (lo if lo % 2 == 0 else hi)
    return s * float(vals[k])


def test_h16_fma_is_one_rounding_of_the_exact_result():
    """orc_h16_fma against exact rational arithmetic rounded once: random operands over the whole exponent range, subnormals, exact ties
    (a product plus an addend that lands halfway between two binary16 values, with and without a sticky term), overflow to inf."""
    rng = np.random.default_rng(7)
    L = orc.lib()
    L.orc_h16_fma.restype = np.ctypeslib.ctypes.c_uint16
    L.orc_h16_fma.argtypes = [np.ctypeslib.ctypes.c_uint16] * 3
    cases = []
    r = rng.integers(0, 0x7c00, size=(4000, 3)).astype(np.uint16) | (rng.integers(0, 2, size=(4000, 3)).astype(np.uint16) << 15)
    cases += [tuple(int(v) for v in row) for row in r]
    sub = rng.integers(0, 0x0400, size=(500, 3)).astype(np.uint16)                      # subnormal operands and results
    cases += [(int(a) | 0x3c00 & 0, int(b) + 0x3800, int(c)) for a, b, c in sub]
    h = lambda f: int(np.float16(f).view(np.uint16))
    # ties: 1 + 2^-11 is halfway between 1 and 1 + 2^-10: (2^-11 x 1) + 1; with a sticky product term just above / below the tie
    cases += [(h(2.0 ** -11), h(1.0), h(1.0)), (h(2.0 ** -11), h(1.0 + 2.0 ** -10), h(1.0)), (h(2.0 ** -11), h(1.0), h(1.0 + 2.0 ** -10)),
              (h(2.0 ** -12), h(1.0 + 2.0 ** -9), h(1.0)), (h(-(2.0 ** -11)), h(1.0), h(1.0 + 2.0 ** -10)), (h(3.0), h(2.0 ** -24), h(2.0 ** -24)),
              (h(2.0 ** -14), h(2.0 ** -11), h(2.0 ** -24)), (h(65504.0), h(1.0), h(16.0)), (h(65504.0), h(1.0), h(15.0)), (h(256.0), h(256.0), h(-1.0))]
    for a, b, c in cases:
        fa, fb, fc = (float(np.uint16(v).view(np.float16)) for v in (a, b, c))
        want = half_round(Fraction(fa) * Fraction(fb) + Fraction(fc))
        got = float(np.uint16(L.orc_h16_fma(a, b, c)).view(np.float16))
        assert got == want and (want != 0 or True), (hex(a), hex(b), hex(c), got, want)


def _staged_up(x, N, C, Dc, Hc, Wc, cbits, up):
    D, H, W = 2 * Dc, 2 * Hc, 2 * Wc
    xq = orc.f32_to_mx(8, x, N, C, Dc * Hc * Wc)
    c = orc.orc_conv_t()
    c.x, c.xdt, c.N, c.Ci, c.D, c.H, c.W, c.cbits, c.stride, c.up = orc.ptr(xq), 3, N, C, D, H, W, cbits, 1, up
    st = np.zeros((N, (C + 31) // 32, D * H * W, 32), np.float32)
    assert orc.lib().orc_conv3_staged(c, orc.ptr(st)) == (C + 31) // 32 * 32
    return st, decoded(8, xq, N, C, Dc * Hc * Wc)


def test_fp16_upsample_blend_equals_rational_arithmetic_rounded_per_step():
    """The fp4 entry's fused-upsample staging: per fine voxel, the 8 coarse rows (e4m3 codes, one scale byte each) are blended in binary16
    with weights .75 / .25 per axis times 2^(e_row - e_max), in the order z, y, x, one fused rounding per step; the sum times 2^e_max is
    then quantised to e2m1. Restated here with exact rationals and the table-search rounding above, the rows' scale bytes from the
    independent scale rule; a wrong tap order, a weight rounded at the wrong place, an fp32 accumulator or a missing relative scale fails.
    Also: up = 1 of the fp4 entry IS this blend, of the fp8 entry the fp32 chain; up = 2 / 3 force one."""
    rng = np.random.default_rng(21)
    N, C, Dc, Hc, Wc = 1, 32, 2, 3, 2
    x = (rng.standard_normal((N, C, Dc * Hc * Wc)) * np.exp(rng.uniform(-4, 4, (N, 1, Dc * Hc * Wc)))).astype(np.float32)   # row scales spread over ~2^12
    st, xd = _staged_up(x, N, C, Dc, Hc, Wc, 4, 1)
    D, H, W = 2 * Dc, 2 * Hc, 2 * Wc
    rows = np.moveaxis(xd[0], 0, -1).reshape(Dc, Hc, Wc, 32).astype(np.float64)             # decoded coarse rows (each an e4m3 code times its scale)
    es = refnp.scale_exp(np.abs(rows).max(-1), 448.0)                                       # their scale exponents (the blend re-derives them)
    want = np.zeros((D, H, W, 32), np.float32)
    for gz in range(D):
        for gy in range(H):
            for gx in range(W):
                m = [(g >> 1, min(max((g >> 1) + (1 if g & 1 else -1), 0), n - 1)) for g, n in ((gz, Dc), (gy, Hc), (gx, Wc))]
                taps = [(a, b, c) for a in range(2) for b in range(2) for c in range(2)]
                em = max(int(es[m[0][a], m[1][b], m[2][c]]) for a, b, c in taps)
                acc = [Fraction(0)] * 32
                for a, b, c in taps:
                    iz, iy, ix = m[0][a], m[1][b], m[2][c]
                    e = int(es[iz, iy, ix])
                    w3 = half_round(Fraction([3, 1][a] * [3, 1][b] * [3, 1][c], 64) * Fraction(2) ** (e - em))
                    codes = [Fraction(float(v)) / Fraction(2) ** e for v in rows[iz, iy, ix]]           # the e4m3 values: exact in binary16
                    acc = [Fraction(half_round(Fraction(w3) * q + s)) for q, s in zip(codes, acc)]
                want[gz, gy, gx] = [float(s * Fraction(2) ** em) for s in acc]
    wq, _ = refnp.quantize_block(want.reshape(-1, 32), 4)
    assert np.array_equal(st[0, 0], wq)
    # the entry's default and the forced modes
    assert np.array_equal(_staged_up(x, N, C, Dc, Hc, Wc, 4, 2)[0], st)
    # (after the e2m1 rounding the fp32 chain rarely differs; under e4m3 compute, forced either way, the two blends are told apart)
    assert np.array_equal(_staged_up(x, N, C, Dc, Hc, Wc, 8, 1)[0], _staged_up(x, N, C, Dc, Hc, Wc, 8, 3)[0])
    assert not np.array_equal(_staged_up(x, N, C, Dc, Hc, Wc, 8, 2)[0], _staged_up(x, N, C, Dc, Hc, Wc, 8, 3)[0])


def test_fp16_upsample_blend_closed_forms():
    """Grid data (every row's amax 6, values on the e2m1 grid): all partial sums are multiples of 2^-7 below 6 and exact in binary16, so the
    binary16 blend equals the fp64 trilinear interpolation, and where the 8 rows coincide (a constant tensor) it returns the row itself."""
    rng = np.random.default_rng(22)
    N, C, Dc, Hc, Wc = 1, 32, 2, 2, 3
    x = refnp.gen_exact(rng, (N, C, Dc * Hc * Wc))
    x[:, 5, :] = 6.0
    st, _ = _staged_up(x, N, C, Dc, Hc, Wc, 4, 2)
    want = refnp.up2_f64(x.reshape(N, C, Dc, Hc, Wc)).reshape(N, C, -1)
    wq, _ = refnp.quantize_block(np.moveaxis(want[0], 0, -1).astype(np.float32), 4)
    assert np.array_equal(st[0, 0], wq)
    xc = np.repeat(x[:, :, :1], Dc * Hc * Wc, axis=2)
    st, _ = _staged_up(xc, N, C, Dc, Hc, Wc, 4, 2)
    assert np.array_equal(st[0, 0], np.repeat(xc[0, :, :1].T, 8 * Dc * Hc * Wc, axis=0))
