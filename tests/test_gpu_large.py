"""Tensors past 4 GiB (byte offsets beyond 32 bits, sample indices in the hundreds) through the C ABI: every kernel family once. A tensor is one
sample's data replicated on the device, so every sample's result is the one-sample oracle result; the first and the last sample are fetched
and compared byte for byte (exact operands) - an offset that wraps at 2^31 or 2^32 anywhere in the addressing writes the wrong place or reads
the wrong rows. The reference's counterpart is its large-index case (256 -> 256 at 192^3 sampled at the tensor's end, tests/test_mx4_wide.c:674-735)."""
import numpy as np
import pytest

from ufsm_amd import lib, LP, shape5, gnp_t, split_t, DevBuf
from gpuutil import dev_gn
import orc
import refnp

pytestmark = pytest.mark.gpu
GIB4 = 1 << 32


def rb_of(bits, C):
    bw = 8 if C <= 8 else 16 if C <= 16 else 32
    return bw, (C + bw - 1) // bw, bw * bits // 8


def replicate_mx(q1, bits, N, C, S):
    """One sample's MX tensor (host bytes) -> a device tensor of N such samples."""
    _, nb, rb = rb_of(bits, C)
    dsz, ssz = nb * S * rb, nb * S
    assert q1.size == dsz + ssz
    d1 = DevBuf.from_numpy(q1)
    big = DevBuf(N * (dsz + ssz), zero=False)
    for n in range(N):
        lib.mi_d2d(big.ptr + n * dsz, d1.ptr, dsz)
        lib.mi_d2d(big.ptr + N * dsz + n * ssz, d1.ptr + dsz, ssz)
    lib.mi_sync()
    return big


def fetch_mx(big, bits, N, C, S, n):
    _, nb, rb = rb_of(bits, C)
    dsz, ssz = nb * S * rb, nb * S
    out = np.empty(dsz + ssz, np.uint8)
    lib.mi_sync()
    lib.mi_d2h(out.ctypes.data, big.ptr + n * dsz, dsz)
    lib.mi_d2h(out.ctypes.data + dsz, big.ptr + N * dsz + n * ssz, ssz)
    return out


def fetch_planes(big, N, C, S, n, itemsize=4):
    out = np.empty(C * S * itemsize, np.uint8)
    lib.mi_sync()
    lib.mi_d2h(out.ctypes.data, big.ptr + n * C * S * itemsize, out.size)
    return out


CONVS = [  # name, Ci, Co, dims, N, stride, bits, gn, kernel name part
    ("wide", 128, 128, (16, 32, 32), 2000, 1, 8, False, "conv3_wide_k"),
    ("row", 96, 32, (8, 32, 32), 5400, 1, 8, False, "conv3_row_k"),
    ("one-block row", 32, 32, (16, 32, 32), 8000, 1, 8, False, "conv3_row1_k"),
    ("small", 32, 32, (16, 32, 16), 16000, 1, 8, False, "conv3_small_k"),
    ("general fp4 stride 2", 64, 64, (16, 32, 32), 7800, 2, 4, False, "stride 2"),
    ("direct fp4 stride 2", 64, 64, (16, 32, 32), 7800, 2, 4, False, "conv3s2_mx_k"),
    ("restaged GroupNorm input", 64, 64, (16, 16, 32), 8000, 1, 8, True, "conv3_"),
]


@pytest.mark.parametrize("name,Ci,Co,dims,N,stride,bits,gn,kpart", CONVS, ids=[c[0] for c in CONVS])
def test_conv_past_4gib(gpu, name, Ci, Co, dims, N, stride, bits, gn, kpart):
    rng = np.random.default_rng(len(name))
    D, H, W = dims
    S, xdt = D * H * W, 3 if bits == 8 else 4
    x1 = refnp.gen_exact(rng, (1, Ci, S)); w = refnp.gen_exact(rng, (Co, Ci, 27)); b = rng.integers(-8, 9, Co).astype(np.float32) * 0.25
    q1 = orc.f32_to_mx(bits, x1, 1, Ci, S)
    G = 8
    p = [rng.uniform(.5, 1.5, Ci).astype(np.float32), rng.uniform(-.3, .3, Ci).astype(np.float32)]
    m1, r1 = rng.uniform(-.2, .2, G).astype(np.float32), rng.uniform(.7, 1.4, G).astype(np.float32)
    xin = replicate_mx(q1, bits, N, Ci, S)
    assert xin.nbytes > GIB4, xin.nbytes
    Do, Ho, Wo = ((D - 1) // 2 + 1, (H - 1) // 2 + 1, (W - 1) // 2 + 1) if stride == 2 else dims
    So = Do * Ho * Wo
    _, nbo, rbo = rb_of(bits, Co)
    y = DevBuf(N * nbo * So * (rbo + 1), zero=False)
    dw, db = DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    g = dev_gn(p[0], p[1], np.tile(m1, N), np.tile(r1, N), G) if gn else gnp_t()
    sums = DevBuf(N * G * 2 * 24)
    lib.mi_gn_sums_zero(sums.ptr, 2 * N * G)
    xs = shape5(N, Ci, D, H, W)
    if stride == 2:
        lib.mi_conv_s2_direct(1 if name.startswith("direct") else 0)     # both stride-2 kernels at this size (by default the launch size picks one)
        try:
            rc = lib.lp_conv_fwd_s2_f8(xin.ptr, xdt, xs, dw.ptr, db.ptr, Co, y.ptr, xdt, shape5(N, Co, Do, Ho, Wo), g)
        finally:
            lib.mi_conv_s2_direct(-1)
        assert rc in (0, 3)
    else:
        rc = (lib.lp_conv_fwd_f8 if bits == 8 else lib.lp_conv_fwd_f4)(xin.ptr, xdt, xs, dw.ptr, db.ptr, Co, y.ptr, xdt, g, sums.ptr, G, split_t())
        assert rc == 0
    LP.check()
    assert kpart in lib.mi_last_kernel().decode(), lib.mi_last_kernel().decode()
    want, wsum = orc.conv3(q1, xdt, 1, Ci, D, H, W, w, b, Co, xdt, cbits=bits, stride=stride, gp=orc.gn(p[0], p[1], m1, r1, G) if gn else None,
                           Go=G if stride == 1 else 0, want_stats=stride == 1, acc64=0 if gn else 1)
    for n in (0, N // 2, N - 1):
        got = fetch_mx(y, bits, N, Co, So, n)
        if gn:                                               # the device's SiLU against the oracle's: neighbouring codes on a few rows
            assert (got != want).mean() < 5e-3, (name, n)
        else:
            assert np.array_equal(got, want), (name, n)
    if stride == 1 and not gn:                               # every sample's statistics are the one sample's
        sl = np.zeros((N * G, 2)); out = DevBuf(N * G * 2 * 8)
        lib.mi_gn_sums_get(sums.ptr, 2 * N * G, out.ptr)
        sl = out.to_numpy(np.float64).reshape(N, G, 2)
        assert np.allclose(sl[0], wsum[0], rtol=1e-6) and np.array_equal(sl[0], sl[N - 1]) and np.array_equal(sl[0], sl[N // 2])


def test_elementwise_past_4gib(gpu):
    """Converters, GroupNorm + SiLU apply, add, the materialising upsample and the head on tensors past 4 GiB."""
    rng = np.random.default_rng(77)
    C, D = 32, 32
    S = D ** 3
    N = GIB4 // (C * S * 4) + 3                                                   # fp32 planes past 4 GiB: 4099 samples... of 4 MiB each
    x1 = (rng.standard_normal((1, C, S)) * np.exp(rng.uniform(-3, 3, (1, 1, S)))).astype(np.float32)
    d1 = DevBuf.from_numpy(x1)
    xf = DevBuf(N * C * S * 4, zero=False)
    for n in range(N):
        lib.mi_d2d(xf.ptr + n * C * S * 4, d1.ptr, C * S * 4)
    assert xf.nbytes > GIB4
    for bits in (8, 4):
        q = DevBuf((lib.lp_mx8_bytes if bits == 8 else lib.lp_mx4_bytes)(N, C, S), zero=False)
        (lib.lp_f32_to_mx8 if bits == 8 else lib.lp_f32_to_mx4)(xf.ptr, N, C, S, q.ptr); LP.check()
        want = orc.f32_to_mx(bits, x1, 1, C, S)
        for n in (0, N - 1):
            assert np.array_equal(fetch_mx(q, bits, N, C, S, n), want), (bits, n)
        back = DevBuf(N * C * S * 4, zero=False)
        (lib.lp_mx8_to_f32 if bits == 8 else lib.lp_mx4_to_f32)(q.ptr, N, C, S, back.ptr); LP.check()
        wf = orc.mx_to_f32(bits, want, 1, C, S)
        for n in (0, N - 1):
            assert np.array_equal(fetch_planes(back, N, C, S, n).view(np.float32), wf.reshape(-1)), (bits, n)
        del back, q
    # MX-fp8 tensors past 4 GiB: 32 channels x 32^3 x 33 B = 1.03 MiB per sample
    N = GIB4 // (S * 33) + 5
    q1 = orc.f32_to_mx(8, x1, 1, C, S)
    a = replicate_mx(q1, 8, N, C, S)
    assert a.nbytes > GIB4
    G = 8
    gam, bet = rng.uniform(.5, 1.5, C).astype(np.float32), rng.uniform(-.3, .3, C).astype(np.float32)
    m1, r1 = rng.uniform(-.2, .2, G).astype(np.float32), rng.uniform(.7, 1.4, G).astype(np.float32)
    g = dev_gn(gam, bet, np.tile(m1, N), np.tile(r1, N), G)
    y = DevBuf(a.nbytes, zero=False)
    lib.lp_gn_silu_apply_mx(a.ptr, 3, shape5(N, C, D, D, D), G, g.gamma, g.beta, g.mean, g.rstd, y.ptr, 3); LP.check()
    want = np.zeros(q1.size, np.uint8)
    orc.lib().orc_gn_silu_apply_mx(orc.ptr(q1), 3, 1, C, S, orc.gn(gam, bet, m1, r1, G), orc.ptr(want), 8)
    for n in (0, N - 1):
        assert (fetch_mx(y, 8, N, C, S, n) != want).mean() < 2e-3, n
    # add: y = a + a (exactly representable: every code doubles) -> the oracle's add on one sample
    lib.lp_add_mx(y.ptr, a.ptr, shape5(N, C, D, D, D), 3, 0)
    lib.lp_add_mx(y.ptr, a.ptr, shape5(N, C, D, D, D), 3, 0); LP.check()                 # y = (silu(..) + a) + a: any value; compare first and last sample only
    f0, fl = fetch_mx(y, 8, N, C, S, 0), fetch_mx(y, 8, N, C, S, N - 1)
    assert np.array_equal(f0, fl) and f0.any()
    # head: 32 -> 8 logits in fp32 planes
    w = (rng.standard_normal((8, C)) * 0.2).astype(np.float32); b = rng.standard_normal(8).astype(np.float32)
    dw, db = DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    lg = DevBuf(N * 8 * S * 4, zero=False)
    lib.lp_conv1_fwd_mx(a.ptr, 3, shape5(N, C, D, D, D), dw.ptr, db.ptr, 8, lg.ptr, g); LP.check()
    want = np.zeros((1, 8, S), np.float32)
    orc.lib().orc_conv1_mx(8, orc.ptr(q1), 1, C, S, orc.ptr(w), orc.ptr(b), 8, orc.gn(gam, bet, m1, r1, G), orc.ptr(want))
    for n in (0, N - 1):
        got = fetch_planes(lg, N, 8, S, n).view(np.float32).reshape(8, S)
        assert np.abs(got - want[0]).max() < 1e-4 * np.abs(want).max(), n
    del lg, y
    # materialising upsample: the OUTPUT is past 4 GiB (8 x the input)
    Nu = N // 8 + 2
    up = DevBuf(lib.lp_mx8_bytes(Nu, C, 8 * S), zero=False)
    assert up.nbytes > GIB4
    au = replicate_mx(q1, 8, Nu, C, S)
    lib.lp_up2_fwd_mx(au.ptr, 3, shape5(Nu, C, D, D, D), up.ptr, 3, gnp_t()); LP.check()
    want = np.zeros(orc.mx_bytes(8, 1, C, 8 * S), np.uint8)
    orc.lib().orc_up2_mx(8, orc.ptr(q1), 1, C, D, D, D, orc.gn(), orc.ptr(want), 8)
    for n in (0, Nu - 1):
        assert np.array_equal(fetch_mx(up, 8, Nu, C, 8 * S, n), want), n


def test_conv2_past_4gib(gpu):
    rng = np.random.default_rng(5)
    Ci, Co, D = 64, 64, 16
    S = D ** 3
    for up in (0, 1):
        x1 = refnp.gen_exact(rng, (1, Ci, S)); w = refnp.gen_exact(rng, (Ci, Co, 8), block_axis=0) if up else refnp.gen_exact(rng, (Co, Ci, 8))
        q1 = orc.f32_to_mx(8, x1, 1, Ci, S)
        So = 8 * S if up else S // 8
        N = GIB4 // ((So if up else S) * 2 * 33) + 7                                    # the larger of input / output past 4 GiB
        xin = replicate_mx(q1, 8, N, Ci, S)
        y = DevBuf(lib.lp_mx8_bytes(N, Co, So), zero=False)
        assert max(xin.nbytes, y.nbytes) > GIB4
        f = lib.mi_convt_up2_fwd if up else lib.mi_conv_down2_fwd
        assert f(8, xin.ptr, 3, shape5(N, Ci, D, D, D), DevBuf.from_numpy(w).ptr, None, Co, y.ptr, 3, gnp_t()) == 0
        LP.check()
        want = orc.conv2(q1, 3, 1, Ci, D, D, D, w, None, Co, 3, up, cbits=8, acc64=1)
        for n in (0, N - 1):
            assert np.array_equal(fetch_mx(y, 8, N, Co, So, n), want), (up, n)


def test_empty_tensors_are_no_ops(gpu):
    """Zero samples or zero voxels: every entry point returns without a launch error and writes nothing."""
    d = DevBuf(4096); w = DevBuf(1 << 20); y = DevBuf(4096)
    lib.mi_zero(y.ptr, 4096)
    g, sp = gnp_t(), split_t()
    gg = dev_gn(np.ones(32, np.float32), np.zeros(32, np.float32), np.zeros(8, np.float32), np.ones(8, np.float32), 8)
    for N, D in ((0, 8), (1, 0)):
        S = D ** 3
        xs = shape5(N, 32, D, D, D)
        lib.lp_f32_to_mx8(d.ptr, N, 32, S, y.ptr); lib.lp_f32_to_mx4(d.ptr, N, 32, S, y.ptr)
        lib.lp_mx8_to_f32(d.ptr, N, 32, S, y.ptr); lib.lp_mx4_to_f32(d.ptr, N, 32, S, y.ptr)
        assert lib.lp_conv_fwd_f8(d.ptr, 3, xs, w.ptr, None, 32, y.ptr, 3, g, None, 0, sp) == 0
        assert lib.lp_conv_fwd_f4(d.ptr, 4, xs, w.ptr, None, 64, y.ptr, 4, g, None, 0, sp) == 0
        Do = (D - 1) // 2 + 1 if D else 1                                   # (the entry's C formula: (0 - 1) / 2 + 1 = 1)
        lib.lp_conv_fwd_s2_f8(d.ptr, 3, xs, w.ptr, None, 32, y.ptr, 3, shape5(N, 32, Do, Do, Do), g)
        lib.lp_conv1_fwd_mx(d.ptr, 3, xs, w.ptr, None, 8, y.ptr, g)
        lib.lp_up2_fwd_mx(d.ptr, 3, xs, y.ptr, 3, g)
        lib.lp_add_mx(y.ptr, d.ptr, xs, 3, 0)
        lib.lp_gn_silu_apply_mx(d.ptr, 3, xs, 8, gg.gamma, gg.beta, gg.mean, gg.rstd, y.ptr, 3)
        LP.check()
    assert not y.to_numpy(np.uint8).any()
