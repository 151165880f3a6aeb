"""GPU parity of the sliding-window pieces through the C ABI: placement and feather blend against the oracle, and the window driver
against the same windows run one by one (the checks of the reference's tests/test_predict_feather.c on a small volume)."""
import ctypes as C

import numpy as np
import pytest

import orc
from gpuutil import DevBuf, LP, lib

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("o,e,shard", [((-4, -4, -4), (24, 24, 24), 24), ((0, 3, -6), (10, 20, 9), 24), ((-8, -8, -8), (40, 40, 40), 40)])
def test_pred_place_matches_oracle(gpu, o, e, shard):
    rng = np.random.default_rng(5)
    W, halo, iso = 32, 4, 64
    lg = (3 * rng.standard_normal((W, W, W))).astype(np.float32); ct = rng.integers(0, 256, (W, W, W)).astype(np.uint8)
    dl, dc = DevBuf.from_numpy(lg), DevBuf.from_numpy(ct)
    dd = DevBuf.from_numpy(np.full((shard,) * 3, 7, np.uint8))
    lib.nn_set_pred_iso(iso); assert lib.nn_get_pred_iso() == iso
    lib.nn_pred_place(dl.ptr, dc.ptr, W, halo, o[0], o[1], o[2], e[0], e[1], e[2], shard, dd.ptr)
    LP.check()
    got = dd.to_numpy(np.uint8, (shard,) * 3)
    want = orc.pred_place(lg, ct, W, W, halo, halo, o, e, shard, iso, dsh=np.full((shard,) * 3, 7, np.uint8))
    lib.nn_set_pred_iso(1)
    d = np.abs(got.astype(int) - want.astype(int))
    # the same voxels are written; the byte is 255 sigmoid rounded, with the device's and the host's expf differing in the last bit: a
    # step of one on the rare voxel that sits on a rounding boundary
    assert np.array_equal(got == 7, want == 7) and d.max() <= 1 and (d > 0).mean() < 1e-4
    # the slab form (D != W, hz != halo) through nn_pred_place_d
    D, hz = 16, 2
    dd2 = DevBuf.from_numpy(np.full((shard,) * 3, 7, np.uint8))
    lib.nn_pred_place_d(dl.ptr, dc.ptr, D, W, hz, halo, o[0], o[1], o[2], e[0], e[1], e[2], shard, dd2.ptr)
    LP.check()
    want2 = orc.pred_place(lg[:D], ct[:D], D, W, hz, halo, o, e, shard, 1, dsh=np.full((shard,) * 3, 7, np.uint8))
    d2 = np.abs(dd2.to_numpy(np.uint8, (shard,) * 3).astype(int) - want2.astype(int))
    assert d2.max() <= 1 and (d2 > 0).mean() < 1e-4


@pytest.mark.parametrize("S,B,nss,bn,absent", [(12, 4, (2, 2, 2), (24, 24, 24), []), (8, 8, (3, 1, 2), (22, 8, 13), [2]), (16, 5, (2, 3, 2), (30, 48, 17), [0, 7]),
                                                (16, 0, (1, 2, 2), (16, 32, 20), [])])
def test_feather_blend_is_bit_exact(gpu, S, B, nss, bn, absent):
    rng = np.random.default_rng(S + B)
    nw = int(np.prod(nss)); En = S + B
    E = rng.integers(0, 256, (nw, En, En, En)).astype(np.uint8)
    present = np.ones(nw, np.uint8); present[absent] = 0
    dE, dp = DevBuf.from_numpy(E), DevBuf.from_numpy(present)
    do = DevBuf.from_numpy(np.full(bn, 99, np.uint8))
    nss_a = (C.c_int64 * 3)(*nss); bn_a = (C.c_int64 * 3)(*bn)
    assert lib.mi_feather_blend(dE.ptr, dp.ptr, S, B, nss_a, bn_a, do.ptr) == 0
    LP.check()
    got = do.to_numpy(np.uint8, bn)
    if B:
        assert np.array_equal(got, orc.feather_blend(E, present, S, B, nss, bn))          # integer output, same fp32 operations in the same order
    else:                                                                                  # no blend: every voxel is its window's own byte
        for wid, (a, b, c) in enumerate(np.ndindex(*nss)):
            sl = tuple(slice(k * S, min((k + 1) * S, n)) for k, n in zip((a, b, c), bn))
            assert np.array_equal(got[sl], E[wid][:sl[0].stop - sl[0].start, :sl[1].stop - sl[1].start, :sl[2].stop - sl[2].start])
    assert lib.mi_feather_blend(dE.ptr, dp.ptr, S, S + 1, nss_a, bn_a, do.ptr) == -1     # B > S: refused


@pytest.mark.parametrize("W", [24, 32])          # rows of 24 voxels are stored byte by byte, rows of a multiple of 16 as 16-byte vectors
def test_ct_window_gather(gpu, W):
    rng = np.random.default_rng(9)
    Z, Y, X = 20, 33, 47
    vol = rng.integers(0, 256, (Z, Y, X)).astype(np.uint8)
    dv = DevBuf.from_numpy(vol)
    for (oz, oy, ox) in [(-5, -5, -5), (3, 12, 30), (10, 20, 40)]:
        dw = DevBuf(W ** 3); da = DevBuf(4)
        lib.mi_ct_window(dv.ptr, Z, Y, X, oz, oy, ox, W, dw.ptr, 1, 4, da.ptr)
        LP.check()
        want = np.zeros((W, W, W), np.uint8)
        z0, y0, x0 = max(oz, 0), max(oy, 0), max(ox, 0); z1, y1, x1 = min(oz + W, Z), min(oy + W, Y), min(ox + W, X)
        want[z0 - oz:z1 - oz, y0 - oy:y1 - oy, x0 - ox:x1 - ox] = vol[z0:z1, y0:y1, x0:x1]
        assert np.array_equal(dw.to_numpy(np.uint8, (W, W, W)), want)
        assert (da.to_numpy(np.uint32)[0] != 0) == bool((want[4:-4, 4:-4, 4:-4] >= 1).any())       # the flag looks at the interior only
    # an all-air window leaves the flag clear
    dz = DevBuf.from_numpy(np.zeros((8, 8, 8), np.uint8)); dw = DevBuf(W ** 3); da = DevBuf(4)
    lib.mi_ct_window(dz.ptr, 8, 8, 8, 0, 0, 0, W, dw.ptr, 1, 0, da.ptr)
    assert da.to_numpy(np.uint32)[0] == 0


@pytest.mark.parametrize("W,n", [(24, 3), (32, 18)])     # 18: more windows than one launch carries
def test_ct_windows_and_flags_equal_the_single_window_calls(gpu, W, n):
    rng = np.random.default_rng(19)
    Z, Y, X = 40, 33, 48
    vol = (rng.integers(0, 256, (Z, Y, X)) * (rng.random((Z, Y, X)) < 0.002)).astype(np.uint8)       # sparse material: some windows are air
    vol[:, :, :24] = 0; vol[:16] = 0                            # and whole cells of air
    dv = DevBuf.from_numpy(vol)
    halo = 4
    org = np.stack([rng.integers(-W, Z, n), rng.integers(-W, Y, n), rng.integers(-W, X, n)], 1).astype(np.int64)
    dw = DevBuf(n * W ** 3); da = DevBuf(4 * n); lib.mi_zero(da.ptr, 4 * n)
    lib.mi_ct_windows(dv.ptr, Z, Y, X, org.ctypes.data_as(C.POINTER(C.c_int64)), n, W, dw.ptr, 3, halo, da.ptr)
    LP.check()
    got = dw.to_numpy(np.uint8, (n, W, W, W)); flags = da.to_numpy(np.uint32)
    d1 = DevBuf(W ** 3); a1 = DevBuf(4)
    for j in range(n):
        lib.mi_zero(a1.ptr, 4)
        lib.mi_ct_window(dv.ptr, Z, Y, X, int(org[j, 0]), int(org[j, 1]), int(org[j, 2]), W, d1.ptr, 3, halo, a1.ptr)
        assert np.array_equal(got[j], d1.to_numpy(np.uint8, (W, W, W))) and (flags[j] != 0) == (a1.to_numpy(np.uint32)[0] != 0)
    assert 0 < (flags != 0).sum() < n
    # the flags of a whole sliding grid in one pass: cell (a, b, c) is the interior of the window at (a, b, c) S - halo
    for S, sub in [(W - 2 * halo, (Z, Y, X)), (16, (Z, Y, X)), (16, (37, 30, 41))]:      # 16-voxel cells on 48-voxel rows take the 16-byte loads
        sv = np.ascontiguousarray(vol[:sub[0], :sub[1], :sub[2]]); dsv = DevBuf.from_numpy(sv)
        nss = np.array([(d + S - 1) // S for d in sub], np.int64); tot = int(nss.prod())
        df = DevBuf(4 * tot); lib.mi_zero(df.ptr, 4 * tot)
        lib.mi_ct_flags(dsv.ptr, sub[0], sub[1], sub[2], S, nss.ctypes.data_as(C.POINTER(C.c_int64)), 3, df.ptr)
        LP.check()
        want = np.array([(sv[a * S:a * S + S, b * S:b * S + S, c * S:c * S + S] >= 3).any() for a, b, c in np.ndindex(*nss)])
        assert np.array_equal(df.to_numpy(np.uint32) != 0, want) and 0 < want.sum() < tot


def test_pred_place_n_equals_the_single_window_calls(gpu):
    rng = np.random.default_rng(23)
    W, halo, n, En = 24, 6, 18, 16
    lg = (rng.standard_normal((n, 2, W, W, W)) * 3).astype(np.float32)          # (a second, unused logit plane per window: lstride != W^3)
    ct = rng.integers(0, 4, (n, W, W, W)).astype(np.uint8)
    dl = DevBuf.from_numpy(lg); dc = DevBuf.from_numpy(ct)
    order = rng.permutation(n + 2)[:n].astype(np.int64) * En ** 3                # targets in any order, with gaps
    dE = DevBuf((n + 2) * En ** 3); lib.mi_zero(dE.ptr, (n + 2) * En ** 3)
    lib.mi_pred_place_n(dl.ptr, 2 * W ** 3, dc.ptr, W ** 3, n, order.ctypes.data_as(C.POINTER(C.c_int64)), W, W, halo - 4, halo - 4, -halo, -halo, -halo, En, En, En, En, dE.ptr)
    LP.check()
    got = dE.to_numpy(np.uint8, (n + 2, En, En, En))
    d1 = DevBuf(En ** 3)
    for j in range(n):
        lib.mi_zero(d1.ptr, En ** 3)
        lib.nn_pred_place(dl.ptr + j * 2 * W ** 3 * 4, dc.ptr + j * W ** 3, W, halo - 4, -halo, -halo, -halo, En, En, En, En, d1.ptr)
        assert np.array_equal(got[order[j] // En ** 3], d1.to_numpy(np.uint8, (En, En, En)))
    assert got.any() and not got[[k for k in range(n + 2) if k * En ** 3 not in set(order.tolist())]].any()


def test_predict_volume_equals_windows_run_one_by_one(gpu):
    """The driver against its own parts: every window gathered, run and placed separately through the C ABI, blended by the oracle.
    Also the reference's checks: core voxels and the first window equal the unfeathered run byte for byte; shells differ."""
    from ufsm_amd.unet import UNet, make_cfg
    rng = np.random.default_rng(4)
    W, halo, B = 32, 8, 8; S = W - 2 * halo
    dims = (40, 32, 24)                                                     # 3 x 2 x 2 windows, ragged ends
    z, y, x = np.meshgrid(np.arange(dims[0]), np.arange(dims[1]), np.arange(dims[2]), indexing="ij")
    vol = np.clip(60 + 0.8 * z + 0.5 * y + 40 * np.sin(0.3 * x + 0.2 * y) * np.cos(0.15 * z) + rng.integers(0, 16, dims), 0, 255).astype(np.uint8)
    vol[:S, :S, S:] = 0                                                     # window (0, 0, 1) is air: skipped
    net = UNet(make_cfg(4, [16, 32], G=8, head_out=1, act_dt=8), 1, W, W, W, seed=5)
    p = net.params(); p[-1] = 0.0; net.set_params(p)                      # head bias 0: probabilities centred on 0.5
    dv = DevBuf.from_numpy(vol); dout = DevBuf(vol.size); dplain = DevBuf(vol.size)
    mean, isd, axis, cy, cx = 100.0, 1 / 50.0, 1, 40.0, -20.0
    rc, nw, ndone = net.predict_volume(dv.ptr, dims, halo, B, mean, isd, axis, cy, cx, dout.ptr)
    assert rc == 0 and nw == 12 and ndone == 11
    rc2, _, _ = net.predict_volume(dv.ptr, dims, halo, 0, mean, isd, axis, cy, cx, dplain.ptr)
    assert rc2 == 0
    got = dout.to_numpy(np.uint8, dims); plain = dplain.to_numpy(np.uint8, dims)
    # ---- the windows one by one ----
    nss = tuple((d + S - 1) // S for d in dims); En = S + B
    E = np.zeros((12, En, En, En), np.uint8); present = np.zeros(12, np.uint8)
    dlg = DevBuf(W ** 3 * 4); dw = DevBuf(W ** 3); dE = DevBuf(En ** 3)
    for wid, (a, b, c) in enumerate(np.ndindex(*nss)):
        o = (a * S - halo, b * S - halo, c * S - halo)
        lib.mi_ct_window(dv.ptr, dims[0], dims[1], dims[2], o[0], o[1], o[2], W, dw.ptr, 1, halo, None)
        if not (dw.to_numpy(np.uint8, (W, W, W))[halo:-halo, halo:-halo, halo:-halo] >= 1).any():
            continue
        off = DevBuf.from_numpy(np.concatenate([np.full(W, o[1] - cy, np.float32), np.full(W, o[2] - cx, np.float32)]))
        assert net.forward_ct(dw.ptr, mean, isd, off.ptr, off.ptr + 4 * W, axis, dlg.ptr) == 0
        lib.mi_zero(dE.ptr, En ** 3)
        lib.nn_pred_place(dlg.ptr, dw.ptr, W, halo - B, -halo, -halo, -halo, En, En, En, En, dE.ptr)
        LP.check()
        E[wid] = dE.to_numpy(np.uint8, (En, En, En)); present[wid] = 1
    assert present.sum() == 11 and present[1] == 0
    want = orc.feather_blend(E, present, S, B, nss, dims)
    assert np.array_equal(got, want)                                         # the forward is deterministic: byte for byte
    # ---- the reference's checks (tests/test_predict_feather.c:108-121) ----
    insh = ((z % S) < B) | ((y % S) < B) | ((x % S) < B)
    assert np.array_equal(got[~insh], plain[~insh])                          # core voxels: the plain prediction
    assert np.array_equal(got[:S, :S, :S], plain[:S, :S, :S])                # first window: nothing to blend with
    shell = insh & ~((z < S) & (y < S) & (x < S)) & (plain > 0)
    assert (got[shell] != plain[shell]).mean() > 0.25                        # the blended shells moved (windows disagree: per-window GroupNorm)
    assert (got[:S, :S, S:] == 0).all() and got.std() > 5                    # the air window stays empty; the output is not constant
    net.close()


@pytest.mark.gpu
@pytest.mark.parametrize("attn", [0, 1])
def test_predict_volume_batched_windows_equal_single(gpu, attn):
    """A graph created for two (three, eight) samples runs up to that many windows per forward: samples are independent, so the prediction is
    the one-window graph's byte for byte, with an odd number of windows (11: the last batch is incomplete) and with an attention stage."""
    from ufsm_amd.unet import UNet, make_cfg
    rng = np.random.default_rng(9)
    W, halo, B = 32, 8, 8; S = W - 2 * halo
    dims = (40, 32, 24)
    z, y, x = np.meshgrid(np.arange(dims[0]), np.arange(dims[1]), np.arange(dims[2]), indexing="ij")
    vol = np.clip(70 + 0.6 * z + 0.7 * y + 35 * np.sin(0.25 * x + 0.3 * y) * np.cos(0.2 * z) + rng.integers(0, 16, dims), 0, 255).astype(np.uint8)
    vol[:S, :S, S:] = 0                                                     # one air window: 11 of 12 computed
    dv = DevBuf.from_numpy(vol)
    kw = dict(attn_blocks=1, attn_pe=1, attn_reg=2) if attn else {}
    widths = [16, 192] if attn else [16, 32]
    outs = []
    for nb in (1, 2, 3, 8):                                                 # 8: the driver evens 11 windows out over two forwards of 6 (and rebuilds the graph for 6)
        net = UNet(make_cfg(4, widths, G=8, head_out=1, act_dt=8, **kw), nb, W, W, W, seed=5)
        p = net.params(); p[-1] = 0.0; net.set_params(p)
        dout = DevBuf(vol.size)
        rc, nw, ndone = net.predict_volume(dv.ptr, dims, halo, B, 100.0, 1 / 50.0, 1, 40.0, -20.0, dout.ptr)
        assert rc == 0 and nw == 12 and ndone == 11
        outs.append(dout.to_numpy(np.uint8, dims))
        net.close()
    assert outs[0].max() > 0 and outs[0].std() > 0
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2]) and np.array_equal(outs[0], outs[3])


def test_predict_volume_of_air_computes_nothing(gpu):
    """No window holds a voxel >= iso: no forward runs (the graph is not rebuilt for zero samples), the output is zero, the counts say so;
    and a volume smaller than one window's interior in every axis is one window."""
    from ufsm_amd.unet import UNet, make_cfg
    W, halo, B = 32, 8, 8
    net = UNet(make_cfg(4, [16, 32], G=8, head_out=1, act_dt=8), 4, W, W, W, seed=5)
    dims = (40, 32, 24)
    dv = DevBuf.from_numpy(np.zeros(dims, np.uint8)); dout = DevBuf.from_numpy(np.full(dims, 7, np.uint8))
    rc, nw, ndone = net.predict_volume(dv.ptr, dims, halo, B, 100.0, 1 / 50.0, 1, 40.0, -20.0, dout.ptr)
    assert rc == 0 and nw == 12 and ndone == 0 and not dout.to_numpy(np.uint8, dims).any()
    small = (10, 12, 9)
    vol = np.random.default_rng(3).integers(60, 200, small).astype(np.uint8)
    dv = DevBuf.from_numpy(vol); dout = DevBuf(vol.size)
    rc, nw, ndone = net.predict_volume(dv.ptr, small, halo, B, 100.0, 1 / 50.0, 1, 40.0, -20.0, dout.ptr)
    assert rc == 0 and nw == 1 and ndone == 1
    net.close()


@pytest.mark.gpu
def test_config4_full_volume_prediction_properties(gpu):
    """The whole 512 x 1024 x 1024 volume of the sliding-window configuration (128^3 windows, halo 16, feather 16: 6 x 11 x 11 = 726 windows,
    up to 64 per forward, i.e. 12 forwards of 61; widths 32/64/128/192, MX-fp4 weights over MX-fp8 activations, two attention blocks) through the driver, checked by what
    does not depend on the size (tests/test_predict_feather.c:108-121): core voxels and the first window equal the unfeathered prediction byte
    for byte, blended shells differ; windows at the far corner and in the middle, gathered, run alone on a one-window graph and placed through
    the C ABI, equal the unfeathered prediction of their region (offsets past 2^29 voxels, the incomplete last batch); a second run is identical."""
    from ufsm_amd.unet import UNet, make_cfg
    dims, W, halo, B = (512, 1024, 1024), 128, 16, 16
    S = W - 2 * halo
    rng = np.random.default_rng(7)
    z = np.arange(dims[0], dtype=np.float32)[:, None, None]; y = np.arange(dims[1], dtype=np.float32)[None, :, None]; x = np.arange(dims[2], dtype=np.float32)[None, None, :]
    r = np.sqrt((y - 400.0) ** 2 + (x + 300.0) ** 2)
    vol = (115 + 55 * np.sin(r * 0.35 + 0.02 * z)).astype(np.float32)
    vol += rng.integers(-20, 21, (1, dims[1], dims[2])).astype(np.float32) + rng.integers(-10, 11, (dims[0], 1, 1)).astype(np.float32)
    vol = np.clip(vol, 1, 255).astype(np.uint8)
    del r
    cfgk = dict(G=8, head_out=1, act_dt=8, prec=3, attn_blocks=2, attn_pe=1, attn_reg=4)
    net = UNet(make_cfg(4, [32, 64, 128, 192], **cfgk), 64, W, W, W, seed=1)
    p = net.params()
    dv = DevBuf.from_numpy(vol); dout = DevBuf(vol.size); dplain = DevBuf(vol.size)
    args = (115.0, 1 / 40.0, 1, 400.0, -300.0)
    rc, nw, ndone = net.predict_volume(dv.ptr, dims, halo, B, *args, dout.ptr)
    LP.check()
    assert rc == 0 and nw == 6 * 11 * 11 and ndone == nw
    got = dout.to_numpy(np.uint8, dims)
    rc, _, _ = net.predict_volume(dv.ptr, dims, halo, B, *args, dout.ptr)
    LP.check()
    assert rc == 0 and np.array_equal(dout.to_numpy(np.uint8, dims), got)   # deterministic
    rc, _, _ = net.predict_volume(dv.ptr, dims, halo, 0, *args, dplain.ptr)
    LP.check()
    assert rc == 0
    plain = dplain.to_numpy(np.uint8, dims)
    assert got.std() > 5 and got.max() > 128                               # not constant, both sides of one half
    sh = [(np.arange(d) % S) < B for d in dims]
    insh = sh[0][:, None, None] | sh[1][None, :, None] | sh[2][None, None, :]
    assert np.array_equal(got[~insh], plain[~insh])                          # core voxels: the plain prediction
    assert np.array_equal(got[:S, :S, :S], plain[:S, :S, :S])                # first window: nothing to blend with
    first = (np.arange(dims[0]) < S)[:, None, None] & (np.arange(dims[1]) < S)[None, :, None] & (np.arange(dims[2]) < S)[None, None, :]
    shell = insh & ~first & (plain > 0)
    assert (got[shell] != plain[shell]).mean() > 0.25                        # the blended shells moved
    del insh, shell, first
    # ---- sampled windows run alone on a one-window graph: the plain prediction of their S^3 region ----
    one = UNet(make_cfg(4, [32, 64, 128, 192], **cfgk), 1, W, W, W, seed=2); one.set_params(p)
    dlg = DevBuf(W ** 3 * 4); dw = DevBuf(W ** 3); dE = DevBuf(S ** 3)
    for a, b, c in ((0, 0, 0), (3, 5, 6), (5, 10, 10), (5, 0, 10)):          # (the last ones: ragged ends 512 - 480 = 32 planes, 1024 - 960 = 64 rows)
        o = (a * S - halo, b * S - halo, c * S - halo)
        lib.mi_ct_window(dv.ptr, dims[0], dims[1], dims[2], o[0], o[1], o[2], W, dw.ptr, 1, halo, None)
        off = DevBuf.from_numpy(np.concatenate([np.full(W, o[1] - args[3], np.float32), np.full(W, o[2] - args[4], np.float32)]))
        assert one.forward_ct(dw.ptr, args[0], args[1], off.ptr, off.ptr + 4 * W, args[2], dlg.ptr) == 0
        lib.mi_zero(dE.ptr, S ** 3)
        lib.nn_pred_place(dlg.ptr, dw.ptr, W, halo, -halo, -halo, -halo, S, S, S, S, dE.ptr)
        LP.check()
        E = dE.to_numpy(np.uint8, (S, S, S))
        reg = plain[a * S:(a + 1) * S, b * S:(b + 1) * S, c * S:(c + 1) * S]
        assert np.array_equal(E[:reg.shape[0], :reg.shape[1], :reg.shape[2]], reg), (a, b, c)
    one.close(); net.close()
