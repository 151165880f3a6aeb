"""GPU parity: MX converters and elementwise ops through the C ABI against the oracle. Bit-exact for everything that stores codes."""
import numpy as np
import pytest

import orc
import refnp
from gpuutil import DevBuf, LP, lib, mx_bytes, to_mx, dev_gn, shape5, gnp_t

pytestmark = pytest.mark.gpu


def wild(rng, shape):
    return (rng.standard_normal(shape) * np.exp(rng.standard_normal(shape[:1] + (1,) + shape[2:]) * 6)).astype(np.float32)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("N,Cc,S", [(2, 32, 8 * 8 * 8), (1, 4, 1000), (3, 12, 333), (2, 16, 512), (1, 40, 777), (1, 128, 4096), (2, 129, 65)])
def test_f32_to_mx_bit_exact(gpu, bits, N, Cc, S):
    rng = np.random.default_rng(bits + Cc + S)
    x = wild(rng, (N, Cc, S))
    x[0, 0, 0] = np.nan; x[0, min(1, Cc - 1), 1] = np.inf; x[-1, -1, -1] = 0; x[0, :, 2] = 0; x[0, 0, 3] = -0.0
    x[0, 0, 4] = 3.0e38; x[0, 0, 5] = 1e-45; x[0, 0, 6] = 448.0; x[0, 0, 7] = 6.0
    dq = to_mx(bits, x)
    got = dq.to_numpy(np.uint8)
    want = orc.f32_to_mx(bits, x, N, Cc, S)
    assert np.array_equal(got, want)
    # decode on the device == decode of the oracle, bit for bit (signed zeros and infinities included)
    dz = DevBuf(x.nbytes)
    (lib.lp_mx8_to_f32 if bits == 8 else lib.lp_mx4_to_f32)(dq.ptr, N, Cc, S, dz.ptr)
    back = dz.to_numpy(np.float32, x.shape)
    ref = orc.mx_to_f32(bits, want, N, Cc, S)
    assert ((back.view(np.uint32) == ref.view(np.uint32)) | (np.isnan(back) & np.isnan(ref))).all()     # (NaN payloads are not part of the format)


@pytest.mark.parametrize("bits", [8, 4])
def test_every_rounding_boundary_through_the_converter(gpu, bits):
    """Blocks whose first element pins the scale to 1 (448 or 6): the other 31 codes are the raw element encoder's output. Feeds every
    grid value, every midpoint and their 8 fp32 neighbours on both sides, both signs: the device encoder == the pinned oracle encoder."""
    grid = refnp.E4M3 if bits == 8 else refnp.E2M1
    pts = np.concatenate([grid, 0.5 * (grid[:-1] + grid[1:])]).astype(np.float32)
    vals = []
    for k in range(-8, 9):
        vals.append((pts.view(np.uint32).astype(np.int64) + k).clip(0, 0x7F7FFFFF).astype(np.uint32).view(np.float32))
    v = np.concatenate(vals); v = np.concatenate([v, -v])
    n = (len(v) + 30) // 31
    x = np.zeros((1, 32, n), np.float32)
    x[0, 0, :] = 448.0 if bits == 8 else 6.0
    x[0, 1:, :].T.reshape(-1)[:len(v)] = v
    x = np.ascontiguousarray(x)
    got = to_mx(bits, x).to_numpy(np.uint8)
    assert np.array_equal(got, orc.f32_to_mx(bits, x, 1, 32, n))
    L = orc.lib()
    rb = 32 * bits // 8
    codes = got[:n * rb].reshape(n, rb)
    for i in range(0, len(v), 97):                               # spot check against the scalar encoder itself
        vox, k = divmod(i, 31)
        xv = float(x[0, 1 + k, vox])
        c = int(codes[vox, 1 + k]) if bits == 8 else (int(codes[vox, (1 + k) // 2]) >> (4 * ((1 + k) & 1))) & 15
        assert c == (L.orc_enc_e4m3(xv) if bits == 8 else L.orc_enc_e2m1(xv))


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("e", [0, -7, 9])
def test_hardware_encoders_over_all_fp32_inputs(gpu, bits, e):
    """All 2^32 fp32 bit patterns through the hardware encoders the kernels use (v_cvt_scalef32_pk_fp8_f32 / _fp4_f32) at block exponents 0, -7
    and +9, against the device's software encoders of x 2^-e, which are the pinned oracle encoders (the test above and the CPU suite's sweep):
    no mismatch inside the domain the kernels use the instructions on. The reference does the same for its conversion instruction
    (src/lp_mxsw.cu:45-61). Outside the domain (e4m3 beyond 464 after scaling, NaN) the kernels take the software encoders; the counts there
    are printed, not asserted."""
    import ctypes as C
    out = (C.c_ulonglong * 4)()
    assert lib.mi_cvt_sweep(bits, e, out) == 0
    LP.check()
    n_in, bad_in, n_out, bad_out = (int(v) for v in out)
    print("bits %d e %d: in-domain %d (mismatches %d), outside %d (mismatches %d)" % (bits, e, n_in, bad_in, n_out, bad_out))
    assert n_in + n_out == 1 << 32
    assert n_in > (1 << 31) and bad_in == 0
    if bits == 4:
        assert n_out == 2 * ((1 << 23) - 1)                      # the NaN patterns of both signs


@pytest.mark.parametrize("bits", [8, 4])
def test_h16_to_mx(gpu, bits):
    rng = np.random.default_rng(3)
    N, Cc, S = 2, 48, 500
    xh = (rng.standard_normal((N, Cc, S)) * 10).astype(np.float16)
    dx = DevBuf.from_numpy(xh)
    dq = DevBuf(mx_bytes(bits, N, Cc, S))
    (lib.lp_h16_to_mx8 if bits == 8 else lib.lp_h16_to_mx4)(dx.ptr, 2, N, Cc, S, dq.ptr)
    LP.check()
    want = np.zeros(orc.mx_bytes(bits, N, Cc, S), np.uint8)
    orc.lib().orc_h16_to_mx(bits, orc.ptr(np.ascontiguousarray(xh.view(np.uint16))), N, Cc, S, orc.ptr(want))
    assert np.array_equal(dq.to_numpy(np.uint8), want)


def test_empty_tensors(gpu):
    lib.lp_f32_to_mx8(None, 0, 32, 0, None); lib.lp_mx8_to_f32(None, 0, 32, 0, None)
    LP.check()


@pytest.mark.parametrize("bits", [8, 4])
def test_pred_input(gpu, bits):
    _pred_input_case(bits, 24)
    _pred_input_case(bits, 18)                                   # a width that is not a multiple of 4: the one-voxel-per-thread form


def _pred_input_case(bits, W):
    rng = np.random.default_rng(4)
    D = 6
    ct = np.clip(np.where(rng.random((D, W, W)) < 0.5, rng.normal(60, 20, (D, W, W)), rng.normal(170, 20, (D, W, W))), 0, 255).astype(np.uint8)
    dyo = rng.uniform(-30, 30, D).astype(np.float32); dxo = rng.uniform(-30, 30, D).astype(np.float32)
    mean, isd = float(ct.mean()), float(1 / ct.std())
    dct, ddy, ddx = DevBuf.from_numpy(ct), DevBuf.from_numpy(dyo), DevBuf.from_numpy(dxo)
    for (z0, nz, hd, axis) in [(0, D, 2, 1), (2, 3, 0, -1), (1, 4, 2, 0), (0, D, 1, 1), (0, 2, 0, 0)]:
        S = nz * W * W
        dy = DevBuf(mx_bytes(bits, 1, 4, S))
        lib.lp_pred_input_mx(dct.ptr, W, mean, isd, ddy.ptr, ddx.ptr, axis, z0, nz, dy.ptr, hd, bits)
        LP.check()
        want = np.zeros(orc.mx_bytes(bits, 1, 4, S), np.uint8)
        orc.lib().orc_pred_input_mx(bits, orc.ptr(ct), W, mean, isd, orc.ptr(dyo), orc.ptr(dxo), axis, z0, nz, orc.ptr(want), hd)
        got = dy.to_numpy(np.uint8)
        # square root, division and the fused multiply-add are correctly rounded on both sides, zeros keep their signs: bit for bit
        assert np.array_equal(got, want), (z0, nz, hd, axis, (got != want).mean())


@pytest.mark.parametrize("bits,W", [(8, 16), (4, 16), (8, 10)])
def test_pred_input_batch_equals_the_windows_one_by_one(gpu, bits, W):
    """Eighteen windows (more than one launch carries) into samples 1 .. 18 of a 20-sample tensor: the bytes mi_pred_input_mx_n writes window by window."""
    import ctypes as C
    rng = np.random.default_rng(6)
    N, n0, nw, D = 20, 1, 18, W
    S = D * W * W
    ct = rng.integers(0, 256, (nw, D, W, W)).astype(np.uint8)
    dyo = rng.uniform(-30, 30, (nw, D)).astype(np.float32); dxo = rng.uniform(-30, 30, (nw, D)).astype(np.float32)
    dct, ddy, ddx = DevBuf.from_numpy(ct), DevBuf.from_numpy(dyo), DevBuf.from_numpy(dxo)
    nbytes = mx_bytes(bits, N, 4, S)
    dy = DevBuf(nbytes); d1 = DevBuf(nbytes)
    lib.mi_zero(dy.ptr, nbytes); lib.mi_zero(d1.ptr, nbytes)
    order = rng.permutation(nw)                                # window k of the call is window order[k] of the arrays
    cts = (C.c_void_p * nw)(*[dct.ptr + int(j) * S for j in order])
    dys = (C.c_void_p * nw)(*[ddy.ptr + int(j) * 4 * D for j in order]); dxs = (C.c_void_p * nw)(*[ddx.ptr + int(j) * 4 * D for j in order])
    lib.mi_pred_input_mx_batch(cts, W, 120.0, 1 / 50.0, dys, dxs, 1, 0, D, dy.ptr, 2, bits, N, n0, nw)
    for k, j in enumerate(order):
        lib.mi_pred_input_mx_n(dct.ptr + int(j) * S, W, 120.0, 1 / 50.0, ddy.ptr + int(j) * 4 * D, ddx.ptr + int(j) * 4 * D, 1, 0, D, d1.ptr, 2, bits, N, n0 + k)
    LP.check()
    got = dy.to_numpy(np.uint8)
    assert np.array_equal(got, d1.to_numpy(np.uint8)) and got.any()


@pytest.mark.parametrize("xdt,yb,Cc", [(3, 8, 64), (4, 4, 64), (3, 4, 64), (4, 8, 64), (3, 8, 48), (4, 4, 80), (3, 8, 16), (4, 4, 12), (3, 4, 8), (0, 8, 64), (2, 8, 40), (1, 4, 16), (0, 4, 5)])
def test_gn_silu_apply(gpu, xdt, yb, Cc):
    """MX rows of every block width and fp32 / fp16 / bf16 planes in, either MX format out, ragged last blocks."""
    rng = np.random.default_rng(5 + Cc)
    N, S = 2, 600
    G = 8 if Cc % 8 == 0 else 4 if Cc % 4 == 0 else 1
    x = rng.standard_normal((N, Cc, S)).astype(np.float32) * 2
    gam = rng.uniform(0.5, 1.5, Cc).astype(np.float32); bet = rng.uniform(-.5, .5, Cc).astype(np.float32)
    mean = rng.uniform(-.2, .2, N * G).astype(np.float32); rstd = rng.uniform(.8, 1.2, N * G).astype(np.float32)
    if xdt >= 3:
        xb = 8 if xdt == 3 else 4
        dq = to_mx(xb, x); xin = orc.f32_to_mx(xb, x, N, Cc, S)
    elif xdt == 2:
        xin = np.ascontiguousarray(x.astype(np.float16).view(np.uint16)); dq = DevBuf.from_numpy(xin)
        xo = x.astype(np.float16).astype(np.float32)
    elif xdt == 1:
        xin = np.ascontiguousarray((x.view(np.uint32) >> 16).astype(np.uint16)); dq = DevBuf.from_numpy(xin)     # bf16 by truncation: exact widening on both sides
        xo = (xin.astype(np.uint32) << 16).view(np.float32)
    else:
        xin = x; dq = DevBuf.from_numpy(x); xo = x
    g = dev_gn(gam, bet, mean, rstd, G)
    dy = DevBuf(mx_bytes(yb, N, Cc, S))
    lib.lp_gn_silu_apply_mx(dq.ptr, xdt, shape5(N, Cc, S, 1, 1), G, g.gamma, g.beta, g.mean, g.rstd, dy.ptr, 3 if yb == 8 else 4)
    LP.check()
    want = np.zeros(orc.mx_bytes(yb, N, Cc, S), np.uint8)
    src = xin if xdt >= 3 else np.ascontiguousarray(xo)                # (the oracle takes MX rows or fp32 planes: 16-bit planes widen exactly)
    orc.lib().orc_gn_silu_apply_mx(orc.ptr(src), xdt if xdt >= 3 else 0, N, Cc, S, orc.gn(gam, bet, mean, rstd, G), orc.ptr(want), yb)
    got = dy.to_numpy(np.uint8)
    gd, wd = orc.mx_to_f32(yb, got, N, Cc, S), orc.mx_to_f32(yb, want, N, Cc, S)
    # exp is evaluated by the hardware's fast exponential: codes may flip to the neighbour, never further (rn_near_ok, tests/test_mx4_wide.c:165-175)
    assert (gd != wd).mean() < 1e-3
    assert (np.abs(gd - wd) <= np.maximum(np.abs(wd), np.abs(gd)) * (0.26 if yb == 8 else 0.67) + 1e-30).all()


@pytest.mark.parametrize("xb", [8, 4])
def test_row_decode_at_the_extreme_scale_bytes(gpu, xb):
    """Stored rows whose scale byte is 0, 1, 254 or 255 next to ordinary ones: the device decodes a row by the converting instruction with the
    scale as its operand unless a wavefront holds byte 0 (the format's scale there is 0.0, the instruction's 2^-127) or 255 (inf against NaN),
    which take decode x scale. MX -> fp32 planes (bit for bit, NaN for NaN) and the GroupNorm + SiLU apply of the same tensor (statistics that
    keep the transformed values in range) against the oracle."""
    rng = np.random.default_rng(40 + xb)
    N, C, S = 1, 32, 4096
    rb = 32 if xb == 8 else 16
    codes = rng.integers(0, 256, (N, 1, S, rb), dtype=np.uint8)
    if xb == 8:
        codes[(codes & 0x7f) == 0x7f] = 0x3c                            # (no NaN codes: the rows' values are then finite wherever the scale is)
    sc = rng.integers(110, 140, (N, 1, S), dtype=np.uint8)
    sc[0, 0, 5::64] = 0; sc[0, 0, 70::64] = 1; sc[0, 0, 135::64] = 254   # each extreme byte in wavefronts of its own and ordinary wavefronts between
    sc[0, 0, 200::128] = 255
    xin = np.concatenate([codes.reshape(-1), sc.reshape(-1)])
    assert xin.size == orc.mx_bytes(xb, N, C, S)
    dq = DevBuf.from_numpy(xin)
    df = DevBuf(N * C * S * 4)
    (lib.lp_mx8_to_f32 if xb == 8 else lib.lp_mx4_to_f32)(dq.ptr, N, C, S, df.ptr); LP.check()
    got, want = df.to_numpy(np.float32).reshape(N, C, S), orc.mx_to_f32(xb, xin, N, C, S)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)].view(np.uint32), want[~np.isnan(want)].view(np.uint32))
    assert np.isnan(want).any() and (want[0, :, 5] == 0).all() and np.isinf(want).any()
    G = 8
    gam = rng.uniform(0.5, 1.5, C).astype(np.float32); bet = rng.uniform(-.5, .5, C).astype(np.float32)
    mean = rng.uniform(-.2, .2, N * G).astype(np.float32); rstd = rng.uniform(.8, 1.2, N * G).astype(np.float32) * 1e-3
    g = dev_gn(gam, bet, mean, rstd, G)
    dy = DevBuf(mx_bytes(8, N, C, S))
    lib.lp_gn_silu_apply_mx(dq.ptr, 3 if xb == 8 else 4, shape5(N, C, S, 1, 1), G, g.gamma, g.beta, g.mean, g.rstd, dy.ptr, 3); LP.check()
    wy = np.zeros(orc.mx_bytes(8, N, C, S), np.uint8)
    orc.lib().orc_gn_silu_apply_mx(orc.ptr(xin), 3 if xb == 8 else 4, N, C, S, orc.gn(gam, bet, mean, rstd, G), orc.ptr(wy), 8)
    gd, wd = orc.mx_to_f32(8, dy.to_numpy(np.uint8), N, C, S), orc.mx_to_f32(8, wy, N, C, S)
    fin = np.isfinite(wd) & np.isfinite(gd)
    assert np.array_equal(np.isfinite(gd).all(axis=1), np.isfinite(wd).all(axis=1))          # the same rows are non-finite
    assert (gd[fin] != wd[fin]).mean() < 1e-3
    assert (np.abs(gd[fin] - wd[fin]) <= np.maximum(np.abs(wd[fin]), np.abs(gd[fin])) * 0.26 + 1e-30).all()


@pytest.mark.parametrize("xb,yb,gn,Cc,dims", [(8, 8, False, 32, (6, 6, 6)), (4, 4, False, 32, (6, 6, 6)), (8, 8, True, 32, (6, 6, 6)), (4, 8, True, 32, (6, 6, 6)),
                                              (8, 8, False, 64, (5, 7, 9)), (8, 4, False, 48, (3, 4, 11)), (8, 8, False, 16, (4, 5, 6)), (4, 4, False, 12, (3, 5, 4)), (8, 8, False, 8, (2, 3, 5)),
                                              (8, 8, True, 16, (4, 4, 6)), (4, 4, True, 8, (3, 3, 3)), (8, 8, False, 32, (1, 1, 1)), (8, 8, True, 80, (4, 6, 5))])
def test_up2(gpu, xb, yb, gn, Cc, dims):
    rng = np.random.default_rng(6 + Cc)
    D, H, W = dims
    N, G = 2, (8 if Cc % 8 == 0 else 4)
    S = D * H * W
    x = rng.standard_normal((N, Cc, S)).astype(np.float32) * (1 if gn else 3)      # (random values: the blend is fp32 arithmetic in a fixed order on both sides)
    gam = rng.uniform(0.5, 1.5, Cc).astype(np.float32); bet = rng.uniform(-.5, .5, Cc).astype(np.float32)
    mean = rng.uniform(-.2, .2, N * G).astype(np.float32); rstd = rng.uniform(.8, 1.2, N * G).astype(np.float32)
    dq = to_mx(xb, x)
    g = dev_gn(gam, bet, mean, rstd, G) if gn else gnp_t()
    dy = DevBuf(mx_bytes(yb, N, Cc, 8 * S))
    lib.lp_up2_fwd_mx(dq.ptr, 3 if xb == 8 else 4, shape5(N, Cc, D, H, W), dy.ptr, 3 if yb == 8 else 4, g)
    LP.check()
    xq = orc.f32_to_mx(xb, x, N, Cc, S)
    want = np.zeros(orc.mx_bytes(yb, N, Cc, 8 * S), np.uint8)
    orc.lib().orc_up2_mx(xb, orc.ptr(xq), N, Cc, D, H, W, orc.gn(gam, bet, mean, rstd, G) if gn else orc.gn(), orc.ptr(want), yb)
    got = dy.to_numpy(np.uint8)
    if not gn:
        assert np.array_equal(got, want)                         # no transcendental: bit-exact
    else:
        assert (orc.mx_to_f32(yb, got, N, Cc, 8 * S) != orc.mx_to_f32(yb, want, N, Cc, 8 * S)).mean() < 1e-3


def test_up2_blocks_and_add(gpu):
    rng = np.random.default_rng(7)
    N, Cc, D, H, W = 1, 96, 4, 4, 4
    S = D * H * W
    x = refnp.gen_exact(rng, (N, Cc, S))
    dq = to_mx(8, x)
    dy = DevBuf(mx_bytes(8, N, 64, 8 * S))
    lib.lp_up2_fwd_mx_blocks(dq.ptr, 3, shape5(N, Cc, D, H, W), 1, 2, dy.ptr, 3)
    LP.check()
    sub = np.ascontiguousarray(x[:, 32:96])
    want = np.zeros(orc.mx_bytes(8, N, 64, 8 * S), np.uint8)
    subq = orc.f32_to_mx(8, sub, N, 64, S)
    orc.lib().orc_up2_mx(8, orc.ptr(subq), N, 64, D, H, W, orc.gn(), orc.ptr(want), 8)
    assert np.array_equal(dy.to_numpy(np.uint8), want)
    # y += x on MX tensors: decode, add in fp32, re-quantise with the NaN-propagating amax
    a = rng.standard_normal((N, 32, S)).astype(np.float32); b = rng.standard_normal((N, 32, S)).astype(np.float32)
    da, db = to_mx(8, a), to_mx(8, b)
    lib.lp_add_mx(da.ptr, db.ptr, shape5(N, 32, S, 1, 1), 8, 0)
    LP.check()
    sa = orc.mx_to_f32(8, orc.f32_to_mx(8, a, N, 32, S), N, 32, S) + orc.mx_to_f32(8, orc.f32_to_mx(8, b, N, 32, S), N, 32, S)
    assert np.array_equal(da.to_numpy(np.uint8), orc.f32_to_mx(8, sa, N, 32, S))
    for bits, Cn, Sn in [(4, 64, 1000), (8, 96, 515), (8, 16, 300), (4, 12, 77), (8, 5, 130), (4, 8, 64)]:      # either format, wide and narrow rows, ragged row counts
        a = (rng.standard_normal((2, Cn, Sn)) * np.exp(rng.uniform(-3, 3, (2, 1, Sn)))).astype(np.float32); b = rng.standard_normal((2, Cn, Sn)).astype(np.float32)
        if Cn % (8 if Cn <= 8 else 16 if Cn <= 16 else 32) == 0:                                              # (whole blocks: the padding channels of a non-finite row are not defined by the format)
            a[0, 0, 0] = np.nan; b[1, Cn - 1, 3] = np.inf                                                       # non-finite rows propagate (NaN-propagating amax)
        da, db = to_mx(bits, a), to_mx(bits, b)
        lib.lp_add_mx(da.ptr, db.ptr, shape5(2, Cn, Sn, 1, 1), 3 if bits == 8 else 4, 0)
        LP.check()
        with np.errstate(invalid="ignore"):
            sa = orc.mx_to_f32(bits, orc.f32_to_mx(bits, a, 2, Cn, Sn), 2, Cn, Sn) + orc.mx_to_f32(bits, orc.f32_to_mx(bits, b, 2, Cn, Sn), 2, Cn, Sn)
        assert np.array_equal(da.to_numpy(np.uint8), orc.f32_to_mx(bits, sa, 2, Cn, Sn)), (bits, Cn)


@pytest.mark.parametrize("bits,Cc,G", [(8, 16, 8), (8, 64, 8), (4, 32, 4)])
def test_gn_sums_and_finalize(gpu, bits, Cc, G):
    rng = np.random.default_rng(8)
    N, S = 2, 1000
    x = (rng.standard_normal((N, Cc, S)) + 3).astype(np.float32)
    dq = to_mx(bits, x)
    dsum = DevBuf(N * G * 2 * 24)
    assert lib.lp_gn_sums_mx(dq.ptr, 3 if bits == 8 else 4, N, Cc, G, S, dsum.ptr, 0, S) == 0
    dd = DevBuf(N * G * 2 * 8)
    lib.mi_gn_sums_get(dsum.ptr, N * G * 2, dd.ptr)
    got = dd.to_numpy(np.float64, (N * G, 2))
    dec = orc.mx_to_f32(bits, orc.f32_to_mx(bits, x, N, Cc, S), N, Cc, S).astype(np.float64).reshape(N * G, -1)
    assert np.allclose(got[:, 0], dec.sum(-1), rtol=1e-12) and np.allclose(got[:, 1], (dec * dec).sum(-1), rtol=1e-12)   # exact fixed point
    dm, dr = DevBuf(N * G * 4), DevBuf(N * G * 4)
    lib.mi_gn_finalize(dsum.ptr, N * G, (Cc // G) * S, 1e-5, dm.ptr, dr.ptr)
    assert np.allclose(dm.to_numpy(np.float32), dec.mean(-1), rtol=1e-6)
    assert np.allclose(dr.to_numpy(np.float32), 1 / np.sqrt(dec.var(-1) + 1e-5), rtol=1e-5)
    # a second accumulation doubles the sums (slots accumulate), clearing resets them
    lib.lp_gn_sums_mx(dq.ptr, 3 if bits == 8 else 4, N, Cc, G, S, dsum.ptr, 0, S)
    lib.mi_gn_sums_get(dsum.ptr, N * G * 2, dd.ptr)
    assert np.allclose(dd.to_numpy(np.float64, (N * G, 2)), 2 * got, rtol=1e-12)
    lib.mi_gn_sums_zero(dsum.ptr, N * G * 2)
    lib.mi_gn_sums_get(dsum.ptr, N * G * 2, dd.ptr)
    assert (dd.to_numpy(np.float64) == 0).all()


def test_head_matrix_pipe_gives_the_vector_form_s_bits(gpu):
    """The head's products through the matrix pipe (v_mfma_f32_4x4x1: one product per accumulator and step, in channel order) against the same
    products as fused multiply-adds on the vector ALUs: equal bit for bit, with GroupNorm + SiLU on the input, two channel blocks, denormal
    products, a voxel count that leaves lanes of the last wavefront without a voxel, fp32 and fp16 outputs, MX-fp8 and MX-fp4 inputs."""
    rng = np.random.default_rng(77)
    N, Ci, Co, D, H, W, G = 2, 64, 8, 7, 9, 11, 8
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    x[0, :, :40] *= 1e-30
    w = rng.standard_normal((Co, Ci)).astype(np.float32) * 0.3; b = rng.standard_normal(Co).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-.5, .5, Ci).astype(np.float32)
    mean = rng.uniform(-.2, .2, N * G).astype(np.float32); rstd = rng.uniform(.8, 1.2, N * G).astype(np.float32)
    dw = DevBuf.from_numpy(w); db = DevBuf.from_numpy(b)
    xs = shape5(N, Ci, D, H, W)
    try:
        for bits in (8, 4):
            dq = to_mx(bits, x)
            for gn in (False, True):
                g = dev_gn(gam, bet, mean, rstd, G) if gn else gnp_t()
                for h16 in (False, True):
                    out = []
                    for mode in (0, 1):
                        lib.mi_conv1_matrix(mode)
                        dy = DevBuf(N * Co * S * (2 if h16 else 4))
                        (lib.lp_conv1_fwd_mx_h16 if h16 else lib.lp_conv1_fwd_mx)(dq.ptr, 3 if bits == 8 else 4, xs, dw.ptr, db.ptr, Co, dy.ptr, g)
                        out.append(dy.to_numpy(np.uint16 if h16 else np.uint32, (N, Co, S)))
                    assert np.array_equal(out[0], out[1]), (bits, gn, h16)
    finally:
        lib.mi_conv1_matrix(-1)
    LP.check()


# (34 and 70 input channels: a whole 32-channel block, which takes the kernel's straight-line form, followed by a ragged one, with channel counts that
# are not multiples of 4 and output groups of 2 and 1 channels)
@pytest.mark.parametrize("bits,Ci,Co,gn,h16", [(8, 16, 1, False, False), (8, 32, 8, True, False), (4, 32, 11, True, False), (8, 64, 8, False, True), (8, 32, 20, True, False),
                                              (8, 34, 3, False, False), (4, 70, 5, False, False)])
def test_head(gpu, bits, Ci, Co, gn, h16):
    rng = np.random.default_rng(9)
    N, D, H, W, G = 2, 5, 6, 7, 8
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = rng.standard_normal((Co, Ci)).astype(np.float32) * 0.3; b = rng.standard_normal(Co).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-.5, .5, Ci).astype(np.float32)
    mean = rng.uniform(-.2, .2, N * G).astype(np.float32); rstd = rng.uniform(.8, 1.2, N * G).astype(np.float32)
    dq = to_mx(bits, x); dw = DevBuf.from_numpy(w); db = DevBuf.from_numpy(b)
    g = dev_gn(gam, bet, mean, rstd, G) if gn else gnp_t()
    dy = DevBuf(N * Co * S * (2 if h16 else 4))
    xs = shape5(N, Ci, D, H, W)
    (lib.lp_conv1_fwd_mx_h16 if h16 else lib.lp_conv1_fwd_mx)(dq.ptr, 3 if bits == 8 else 4, xs, dw.ptr, db.ptr, Co, dy.ptr, g)
    LP.check()
    want = np.zeros((N, Co, S), np.float32)
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    orc.lib().orc_conv1_mx(bits, orc.ptr(xq), N, Ci, S, orc.ptr(w), orc.ptr(b), Co,
                           orc.gn(gam, bet, mean, rstd, G) if gn else orc.gn(), orc.ptr(want))
    got = dy.to_numpy(np.float16 if h16 else np.float32, (N, Co, S)).astype(np.float32)
    tol = 2e-3 if h16 else (1e-5 if not gn else 2e-5)            # tests/test_mx.c:209 (1e-5); the fast exponential of the GN + SiLU adds a little
    assert np.abs(got - want).max() / np.abs(want).max() < tol
    if not h16:                                                  # a voxel range == the same rows of the whole output (tests/test_headz.c:1-5)
        vb, nv = 37, 101
        dr = DevBuf(N * Co * nv * 4)
        assert lib.lp_conv1_fwd_mx_r(dq.ptr, 3 if bits == 8 else 4, xs, dw.ptr, db.ptr, Co, dr.ptr, g, vb, nv, nv) == 1
        assert np.array_equal(dr.to_numpy(np.float32, (N, Co, nv)), got[:, :, vb:vb + nv])
