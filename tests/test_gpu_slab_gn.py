"""Slab-local GroupNorm statistics on the device (gnp_t.ns > 0: src/nn_lp.h:15-18, src/lp_slab.cuh:7-12) through the C ABI: every reader of an
MX tensor takes each plane's slab row. Checked against the oracle (whose slab rows are pinned on the CPU, tests/test_oracle_slab_gn.py) to
the bar of the per-sample tests of the same entry points, and, exactly, against the device's own per-sample results: a slab's planes cut
out of the tensor and run with that slab's rows as per-sample statistics give the same bytes."""
import ctypes as C

import numpy as np
import pytest

import orc
from gpuutil import dev_gn, gpu_conv
from test_oracle_slab_gn import mx_planes, slab_ranges, stats
from ufsm_amd import DevBuf, LP, gnp_t, lib, shape5

pytestmark = pytest.mark.gpu


def mx_bytes(bits, N, C, S):
    return (lib.lp_mx8_bytes if bits == 8 else lib.lp_mx4_bytes)(N, C, S)


def dev_gn_slab(gam, bet, mean, rstd, G, slab):
    g = dev_gn(gam, bet, mean.reshape(-1), rstd.reshape(-1), G)
    g.zs, g.zo, g.ns, g.zhw = slab
    return g


def row(a, s):
    return np.ascontiguousarray(a[:, s])


@pytest.mark.parametrize("bits,yb,Cc,zs,zo,ns,D", [(8, 8, 32, 4, 0, 2, 8), (8, 4, 64, 3, 1, 3, 8), (4, 8, 32, 4, 2, 2, 7), (8, 8, 12, 2, 0, 3, 6), (4, 4, 96, 5, 0, 2, 10)])
def test_gn_silu_apply_registered_statistics(gpu, bits, yb, Cc, zs, zo, ns, D):
    """lp_gn_silu_apply_mx takes the four pointers: the geometry comes from the registry (lp_gn_slab_reg), keyed by the mean array."""
    rng = np.random.default_rng(Cc + zs + zo)
    N, H, W, G = 2, 6, 20, 4
    HW, S = H * W, D * H * W
    x = rng.standard_normal((N, Cc, S)).astype(np.float32) * 2
    xq = orc.f32_to_mx(bits, x, N, Cc, S)
    gam = rng.uniform(0.5, 1.5, Cc).astype(np.float32); bet = rng.uniform(-.5, .5, Cc).astype(np.float32)
    mean, rstd = stats(rng, N, ns, G)
    xdt, ydt = (3 if bits == 8 else 4), (3 if yb == 8 else 4)
    dq = DevBuf.from_numpy(xq); dy = DevBuf(mx_bytes(yb, N, Cc, S))
    g = dev_gn(gam, bet, mean.reshape(-1), rstd.reshape(-1), G)
    lib.lp_gn_slab_reg(g.mean, zs, zo, ns, HW)
    try:
        assert lib.lp_gn_slab_any() == 1
        lib.lp_gn_silu_apply_mx(dq.ptr, xdt, shape5(N, Cc, D, H, W), G, g.gamma, g.beta, g.mean, g.rstd, dy.ptr, ydt)
        LP.check()
    finally:
        lib.lp_gn_slab_reg(None, 0, 0, 0, 0)
    got = dy.to_numpy(np.uint8)
    want = np.zeros(orc.mx_bytes(yb, N, Cc, S), np.uint8)
    orc.lib().orc_gn_silu_apply_mx(orc.ptr(xq), xdt, N, Cc, S, orc.gn(gam, bet, mean, rstd, G, slab=(zs, zo, ns, HW)), orc.ptr(want), yb)
    gd, wd = orc.mx_to_f32(yb, got, N, Cc, S), orc.mx_to_f32(yb, want, N, Cc, S)
    assert (gd != wd).mean() < 1e-3                      # (the hardware's fast exponential: a code may flip to its neighbour, never further)
    assert (np.abs(gd - wd) <= np.maximum(np.abs(wd), np.abs(gd)) * (0.26 if yb == 8 else 0.67) + 1e-30).all()
    for s, z0, z1 in slab_ranges(zs, zo, ns, D):        # the device's per-sample op on the slab's planes: the same bytes
        xs = mx_planes(xq, bits, N, Cc, D, HW, z0, z1)
        ds = DevBuf.from_numpy(xs); dys = DevBuf(mx_bytes(yb, N, Cc, (z1 - z0) * HW))
        gs = dev_gn(gam, bet, row(mean, s), row(rstd, s), G)
        lib.lp_gn_silu_apply_mx(ds.ptr, xdt, shape5(N, Cc, z1 - z0, H, W), G, gs.gamma, gs.beta, gs.mean, gs.rstd, dys.ptr, ydt)
        LP.check()
        assert np.array_equal(mx_planes(got, yb, N, Cc, D, HW, z0, z1), dys.to_numpy(np.uint8)), s


@pytest.mark.parametrize("bits,Ci,zs,zo,ns,D", [(8, 32, 4, 0, 2, 8), (4, 64, 3, 2, 3, 8), (8, 16, 2, 0, 2, 5)])
def test_head_slab_statistics(gpu, bits, Ci, zs, zo, ns, D):
    rng = np.random.default_rng(Ci + zs)
    N, H, W, G, Co = 2, 12, 10, 4, 3
    HW, S = H * W, D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    w = rng.standard_normal((Co, Ci)).astype(np.float32); b = rng.standard_normal(Co).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-.5, .5, Ci).astype(np.float32)
    mean, rstd = stats(rng, N, ns, G)
    dq, dw, db = DevBuf.from_numpy(xq), DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    dy = DevBuf(N * Co * S * 4)
    xdt = 3 if bits == 8 else 4
    lib.lp_conv1_fwd_mx(dq.ptr, xdt, shape5(N, Ci, D, H, W), dw.ptr, db.ptr, Co, dy.ptr, dev_gn_slab(gam, bet, mean, rstd, G, (zs, zo, ns, HW)))
    LP.check()
    got = dy.to_numpy(np.float32, (N, Co, S))
    want = np.zeros((N, Co, S), np.float32)
    orc.lib().orc_conv1_mx(bits, orc.ptr(xq), N, Ci, S, orc.ptr(w), orc.ptr(b), Co, orc.gn(gam, bet, mean, rstd, G, slab=(zs, zo, ns, HW)), orc.ptr(want))
    assert np.abs(got - want).max() / np.abs(want).max() < 2e-5
    # a voxel range that starts and ends inside slabs == the same voxels of the whole output
    vb, nv = HW + 7, S - 2 * HW - 11
    dr = DevBuf(N * Co * nv * 4)
    assert lib.lp_conv1_fwd_mx_r(dq.ptr, xdt, shape5(N, Ci, D, H, W), dw.ptr, db.ptr, Co, dr.ptr, dev_gn_slab(gam, bet, mean, rstd, G, (zs, zo, ns, HW)), vb, nv, nv) == 1
    LP.check()
    assert np.array_equal(dr.to_numpy(np.float32, (N, Co, nv)), got[:, :, vb:vb + nv])
    for s, z0, z1 in slab_ranges(zs, zo, ns, D):
        ds = DevBuf.from_numpy(mx_planes(xq, bits, N, Ci, D, HW, z0, z1)); Ss = (z1 - z0) * HW
        dys = DevBuf(N * Co * Ss * 4)
        lib.lp_conv1_fwd_mx(ds.ptr, xdt, shape5(N, Ci, z1 - z0, H, W), dw.ptr, db.ptr, Co, dys.ptr, dev_gn(gam, bet, row(mean, s), row(rstd, s), G))
        LP.check()
        assert np.array_equal(got.reshape(N, Co, D, HW)[:, :, z0:z1].reshape(N, Co, Ss), dys.to_numpy(np.float32, (N, Co, Ss))), s


# (bits, N, Ci, Co, dims, stride, (zs, zo, ns)): the small, general, wide and row kernels' shapes, both strides, both compute formats
SLAB_CONVS = [(8, 2, 32, 32, (12, 8, 16), 1, (6, 1, 2)), (8, 1, 64, 64, (12, 8, 16), 1, (4, 0, 3)), (8, 1, 128, 128, (8, 8, 16), 1, (4, 0, 2)),
              (8, 1, 64, 32, (8, 8, 32), 1, (5, 2, 2)), (8, 2, 32, 32, (12, 16, 16), 2, (6, 1, 2)), (8, 1, 64, 64, (12, 8, 16), 2, (4, 0, 3)),
              (4, 1, 64, 64, (12, 8, 16), 1, (6, 0, 2)), (4, 2, 32, 64, (8, 8, 16), 1, (3, 1, 3))]


@pytest.mark.parametrize("bits,N,Ci,Co,dims,stride,slab", SLAB_CONVS)
def test_conv_input_slab_statistics(gpu, bits, N, Ci, Co, dims, stride, slab):
    """Output planes whose input planes lie in one slab are, byte for byte, the device's conv with that slab's rows as per-sample statistics;
    the whole output, boundary planes included, matches the oracle to the per-sample tests' bar."""
    if stride == 2 and bits == 4:
        pytest.skip("the stride-2 entry computes in e4m3")
    rng = np.random.default_rng(Ci + Co + stride + bits)
    D, H, W = dims
    zs, zo, ns = slab
    G, S = 4, D * H * W
    xdt = 3 if bits == 8 else 4
    xq = orc.f32_to_mx(bits, rng.standard_normal((N, Ci, S)).astype(np.float32), N, Ci, S)
    w = (rng.standard_normal((Co, Ci, 27)) * np.sqrt(2.0 / (Ci * 27))).astype(np.float32); b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-.3, .3, Ci).astype(np.float32)
    mean, rstd = stats(rng, N, ns, G)
    got, _ = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride, gp=dev_gn_slab(gam, bet, mean, rstd, G, (zs, zo, ns, H * W)))
    want, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride, gp=orc.gn(gam, bet, mean, rstd, G, slab=(zs, zo, ns, H * W)))
    assert np.abs(got - want).max() / np.abs(want).max() < (1e-3 if bits == 8 else 2e-2)
    per = [gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride, gp=dev_gn(gam, bet, row(mean, s), row(rstd, s), G))[0] for s in range(ns)]
    Do = (D - 1) // 2 + 1 if stride == 2 else D
    g4 = got.reshape(N, Co, Do, -1)
    ranges = slab_ranges(zs, zo, ns, D)
    inside = 0
    for z in range(Do):
        lo, hi = (2 * z - 1, 2 * z + 1) if stride == 2 else (z - 1, z + 1)
        lo, hi = max(lo, 0), min(hi, D - 1)
        home = [s for s, z0, z1 in ranges if z0 <= lo and hi < z1]
        if home:
            assert np.array_equal(g4[:, :, z], per[home[0]].reshape(N, Co, Do, -1)[:, :, z]), z
            inside += 1
        else:
            assert all(not np.array_equal(g4[:, :, z], p.reshape(N, Co, Do, -1)[:, :, z]) for p in per), z
    assert 0 < inside < Do


@pytest.mark.parametrize("bits", [8, 4])
def test_decoder_conv_skip_with_slab_statistics(gpu, bits):
    """[2x upsampled coarse | skip]: the coarse segment keeps per-sample statistics, the skip's are per slab (sp.gp2); also through the z-range,
    slab convs of 4 planes whose slabs do not line up with the statistics' slabs."""
    from ufsm_amd import split_t
    rng = np.random.default_rng(31 + bits)
    N, Cu, Cs, Co, (D, H, W), G = 1, 64, 32, 32, (12, 8, 32), 4
    zs, zo, ns = 5, 0, 3
    S, Sc = D * H * W, D * H * W // 8
    xdt = 3 if bits == 8 else 4
    qu = orc.f32_to_mx(bits, rng.standard_normal((N, Cu, Sc)).astype(np.float32), N, Cu, Sc)
    qs = orc.f32_to_mx(bits, rng.standard_normal((N, Cs, S)).astype(np.float32), N, Cs, S)
    w = (rng.standard_normal((Co, Cu + Cs, 27)) * np.sqrt(2.0 / ((Cu + Cs) * 27))).astype(np.float32); b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    g1 = [rng.uniform(0.5, 1.5, Cu).astype(np.float32), rng.uniform(-.3, .3, Cu).astype(np.float32), rng.uniform(-.2, .2, (N, G)).astype(np.float32), rng.uniform(.7, 1.4, (N, G)).astype(np.float32)]
    gam2, bet2 = rng.uniform(0.5, 1.5, Cs).astype(np.float32), rng.uniform(-.3, .3, Cs).astype(np.float32)
    mean2, rstd2 = stats(rng, N, ns, G)
    want, _ = orc.conv3(qu, xdt, N, Cu + Cs, D, H, W, w, b, Co, 0, cbits=bits, x2=qs, c_split=Cu, up=1, gp=orc.gn(*g1, G=G), gp2=orc.gn(gam2, bet2, mean2, rstd2, G, slab=(zs, zo, ns, H * W)))
    mk2 = lambda: dev_gn_slab(gam2, bet2, mean2, rstd2, G, (zs, zo, ns, H * W))
    got, _ = gpu_conv(qu, xdt, N, Cu + Cs, D, H, W, w, b, Co, 0, cbits=bits, x2=qs, c_split=Cu, up=1, gp=dev_gn(g1[0], g1[1], g1[2].reshape(-1), g1[3].reshape(-1), G), gp2=mk2())
    assert np.abs(got - want).max() / np.abs(want).max() < (1e-3 if bits == 8 else 3e-2)
    # the same conv in z-range slabs of 4 output planes into an MX tensor of the full depth == the whole conv's MX output
    f = lib.lp_conv_fwd_f8 if bits == 8 else lib.lp_conv_fwd_f4
    du, ds, dw, db = DevBuf.from_numpy(qu), DevBuf.from_numpy(qs), DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    gp = dev_gn(g1[0], g1[1], g1[2].reshape(-1), g1[3].reshape(-1), G)
    outs = []
    for slabbed in (0, 1):
        dy = DevBuf(mx_bytes(bits, N, Co, S))
        for z0 in (range(0, D, 4) if slabbed else [0]):
            sp = split_t(); sp.x2, sp.c_split, sp.up, sp.gp2 = ds.ptr, Cu, 1, mk2()
            sk = min(4, D - z0) if slabbed else D
            if slabbed:
                sp.zi0, sp.Di, sp.yzo, sp.yD = z0, D, z0, D
            assert f(du.ptr, xdt, shape5(N, Cu + Cs, sk, H, W), dw.ptr, db.ptr, Co, dy.ptr, xdt, gp, None, 0, sp) == 0
        LP.check()
        outs.append(dy.to_numpy(np.uint8))
    assert np.array_equal(outs[0], outs[1])


def test_prestage_slab_statistics(gpu):
    """mi_conv_prestage (the skip formed once for its two readers) with slab rows, then the conv on the result without a GroupNorm: the bytes
    of the conv that applies the slab statistics itself."""
    rng = np.random.default_rng(77)
    N, Ci, Co, (D, H, W), G = 2, 32, 32, (8, 8, 16), 4
    zs, zo, ns = 3, 1, 3
    S = D * H * W
    xq = orc.f32_to_mx(8, rng.standard_normal((N, Ci, S)).astype(np.float32), N, Ci, S)
    w = (rng.standard_normal((Co, Ci, 27)) * 0.1).astype(np.float32); b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-.3, .3, Ci).astype(np.float32)
    mean, rstd = stats(rng, N, ns, G)
    g = dev_gn_slab(gam, bet, mean, rstd, G, (zs, zo, ns, H * W))
    direct, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, b, Co, 3, gp=g)
    dq = DevBuf.from_numpy(xq); dst = DevBuf(mx_bytes(8, N, Ci, S))
    assert lib.mi_conv_prestage(dq.ptr, 3, shape5(N, Ci, D, H, W), g, dst.ptr, 8) == 0
    LP.check()
    staged, _ = gpu_conv(dst.to_numpy(np.uint8), 3, N, Ci, D, H, W, w, b, Co, 3)
    assert np.array_equal(staged, direct)


@pytest.mark.parametrize("Ci,tile,zs,zo,ns,kern", [(8, 1, 6, 0, 2, "conv3_stem_k"), (4, 1, 4, 1, 3, "conv3_stem_k"), (16, 2, 6, 0, 2, "conv3_p16_k"), (12, 2, 5, 2, 3, "conv3_p16_k")])
def test_few_channel_convs_slab_statistics(gpu, Ci, tile, zs, zo, ns, kern):
    """The tap-packed and the row-scale kernels (inputs of at most 16 channels) form one coefficient table per slab and take each staged
    position's plane (src/lp_f8fwd.cuh:497): against the oracle to the per-sample tests' bar, with output statistics, also through the z-range."""
    from ufsm_amd import split_t
    rng = np.random.default_rng(Ci + zs)
    N, Co, (D, H, W), G = 2, 32, (12, 12, 20), 4
    S = D * H * W
    xq = orc.f32_to_mx(8, rng.standard_normal((N, Ci, S)).astype(np.float32), N, Ci, S)
    w = (rng.standard_normal((Co, Ci, 27)) * np.sqrt(2.0 / (Ci * 27))).astype(np.float32); b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-.5, .5, Ci).astype(np.float32)
    mean, rstd = stats(rng, N, ns, G)
    slab = (zs, zo, ns, H * W)
    want, wsum = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 3, stem_tile=tile, Go=8, want_stats=True, stored_stats=1, gp=orc.gn(gam, bet, mean, rstd, G, slab=slab))
    got, gsum = gpu_conv(xq, 3, N, Ci, D, H, W, w, b, Co, 3, Go=8, stats=True, stored_stats=1, gp=dev_gn_slab(gam, bet, mean, rstd, G, slab))
    assert kern in lib.mi_last_kernel().decode()
    from gpuutil import code_mismatch_fraction
    frac, near = code_mismatch_fraction(8, got, want, N, Co, S)
    assert frac < 2e-2 and near
    dec = orc.mx_to_f32(8, got, N, Co, S).astype(np.float64).reshape(N, 8, -1)
    assert np.allclose(gsum[:, :, 0], dec.sum(-1), rtol=1e-5, atol=1e-3) and np.allclose(gsum[:, :, 1], (dec * dec).sum(-1), rtol=1e-5)
    # the slabs' rows matter (another tensor with the first slab's rows everywhere) ...
    flat, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, b, Co, 3, gp=dev_gn(gam, bet, row(mean, 0), row(rstd, 0), G))
    assert not np.array_equal(flat, got)
    # ... and z-range slabs of 4 output planes into the full-depth tensor give the whole conv's bytes
    dq, dw, db = DevBuf.from_numpy(xq), DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    dy = DevBuf(mx_bytes(8, N, Co, S))
    g = dev_gn_slab(gam, bet, mean, rstd, G, slab)
    for z0 in range(0, D, 4):
        sp = split_t(); sp.zi0, sp.Di, sp.yzo, sp.yD = z0, D, z0, D
        assert lib.lp_conv_fwd_f8(dq.ptr, 3, shape5(N, Ci, 4, H, W), dw.ptr, db.ptr, Co, dy.ptr, 3, g, None, 0, sp) == 0
    LP.check()
    assert np.array_equal(dy.to_numpy(np.uint8), got)
