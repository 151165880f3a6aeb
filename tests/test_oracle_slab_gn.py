"""Slab-local GroupNorm statistics in the oracle (gnp_t.ns > 0: src/nn_lp.h:15-18, src/lp_slab.cuh:7-12): the statistics hold one row per
(sample, z-slab); plane z reads row n * ns + clamp((z + zo) / zs, 0, ns - 1). Pinned against the per-sample paths (which have their own pins):
a slab's planes, cut out of the tensor byte for byte, go through the per-sample function with that slab's rows; the conv's planes away from a
slab boundary equal the per-sample conv's, the two planes at a boundary equal neither."""
import numpy as np
import pytest

import orc


def mx_planes(q, bits, N, C, D, HW, z0, z1):
    """Planes [z0, z1) of an MX tensor as an MX tensor of depth z1 - z0 (element rows and scales of every (sample, block))."""
    bw = 8 if C <= 8 else 16 if C <= 16 else 32
    nb = (C + bw - 1) // bw
    rb = bw if bits == 8 else bw // 2
    S = D * HW
    data = q[:N * nb * S * rb].reshape(N * nb, D, HW * rb)[:, z0:z1]
    sc = q[N * nb * S * rb:].reshape(N * nb, D, HW)[:, z0:z1]
    return np.concatenate([data.reshape(-1), sc.reshape(-1)])


def slab_ranges(zs, zo, ns, D):
    """[(slab, z0, z1)]: written from the definition, independently of the oracle's row function: slab boundaries sit at planes k zs - zo,
    the first slab starts at plane 0 and the last one takes everything behind it."""
    cuts = [0] + [min(max(k * zs - zo, 0), D) for k in range(1, ns)] + [D]
    return [(s, cuts[s], cuts[s + 1]) for s in range(ns) if cuts[s] < cuts[s + 1]]


def stats(rng, N, ns, G):
    mean = rng.uniform(-0.4, 0.4, (N, ns, G)).astype(np.float32)
    rstd = rng.uniform(0.5, 2.0, (N, ns, G)).astype(np.float32)
    return mean, rstd


@pytest.mark.parametrize("zs,zo,ns,D", [(4, 0, 3, 12), (4, 1, 3, 12), (5, 4, 2, 12), (3, 0, 2, 10), (8, 7, 4, 9), (1, 0, 5, 5)])
def test_row_of_plane(zs, zo, ns, D):
    g = orc.gn(np.ones(8, np.float32), np.ones(8, np.float32), np.ones(64, np.float32), np.ones(64, np.float32), 8, slab=(zs, zo, ns, 16))
    want = {}
    for s, z0, z1 in slab_ranges(zs, zo, ns, D):
        for z in range(z0, z1):
            want[z] = s
    assert sorted(want) == list(range(D))
    for n in (0, 3):
        assert [orc.lib().orc_gn_row(g, n, z) for z in range(D)] == [n * ns + want[z] for z in range(D)]
    plain = orc.gn(np.ones(8, np.float32), np.ones(8, np.float32), np.ones(64, np.float32), np.ones(64, np.float32), 8)
    assert [orc.lib().orc_gn_row(plain, 2, z) for z in range(D)] == [2] * D


@pytest.mark.parametrize("bits,C,zs,zo,ns,D", [(8, 32, 4, 0, 2, 8), (8, 64, 3, 1, 3, 8), (4, 32, 4, 2, 2, 7), (8, 12, 2, 0, 3, 6), (4, 96, 5, 0, 2, 10)])
def test_apply_equals_per_sample_apply_of_each_slab(bits, C, zs, zo, ns, D):
    rng = np.random.default_rng(C + zs + zo)
    N, H, W, G = 2, 3, 5, 4
    HW, S = H * W, D * H * W
    x = rng.standard_normal((N, C, S)).astype(np.float32)
    xq = orc.f32_to_mx(bits, x, N, C, S)
    gam = rng.uniform(0.5, 1.5, C).astype(np.float32); bet = rng.uniform(-0.5, 0.5, C).astype(np.float32)
    mean, rstd = stats(rng, N, ns, G)
    y = np.zeros(orc.mx_bytes(bits, N, C, S), np.uint8)
    orc.lib().orc_gn_silu_apply_mx(orc.ptr(xq), 3 if bits == 8 else 4, N, C, S, orc.gn(gam, bet, mean, rstd, G, slab=(zs, zo, ns, HW)), orc.ptr(y), bits)
    seen = 0
    for s, z0, z1 in slab_ranges(zs, zo, ns, D):
        xs = mx_planes(xq, bits, N, C, D, HW, z0, z1)
        Ss = (z1 - z0) * HW
        ys = np.zeros(orc.mx_bytes(bits, N, C, Ss), np.uint8)
        m, r = np.ascontiguousarray(mean[:, s]), np.ascontiguousarray(rstd[:, s])
        orc.lib().orc_gn_silu_apply_mx(orc.ptr(xs), 3 if bits == 8 else 4, N, C, Ss, orc.gn(gam, bet, m, r, G), orc.ptr(ys), bits)
        assert np.array_equal(mx_planes(y, bits, N, C, D, HW, z0, z1), ys), s
        seen += z1 - z0
    assert seen == D
    # and the rows matter: the first slab's statistics everywhere give another tensor
    y0 = np.zeros_like(y)
    orc.lib().orc_gn_silu_apply_mx(orc.ptr(xq), 3 if bits == 8 else 4, N, C, S, orc.gn(gam, bet, np.ascontiguousarray(mean[:, 0]), np.ascontiguousarray(rstd[:, 0]), G), orc.ptr(y0), bits)
    assert not np.array_equal(y0, y)
    assert np.array_equal(mx_planes(y0, bits, N, C, D, HW, 0, slab_ranges(zs, zo, ns, D)[0][2]), mx_planes(y, bits, N, C, D, HW, 0, slab_ranges(zs, zo, ns, D)[0][2]))


@pytest.mark.parametrize("bits,Ci,zs,zo,ns,D", [(8, 32, 4, 0, 2, 8), (4, 64, 3, 2, 3, 8), (8, 16, 2, 0, 2, 5)])
def test_head_equals_per_sample_head_of_each_slab(bits, Ci, zs, zo, ns, D):
    rng = np.random.default_rng(Ci + zs)
    N, H, W, G, Co = 2, 4, 3, 4, 3
    HW, S = H * W, D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    w = rng.standard_normal((Co, Ci)).astype(np.float32); b = rng.standard_normal(Co).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-0.5, 0.5, Ci).astype(np.float32)
    mean, rstd = stats(rng, N, ns, G)
    y = np.zeros((N, Co, S), np.float32)
    orc.lib().orc_conv1_mx(bits, orc.ptr(xq), N, Ci, S, orc.ptr(w), orc.ptr(b), Co, orc.gn(gam, bet, mean, rstd, G, slab=(zs, zo, ns, HW)), orc.ptr(y))
    for s, z0, z1 in slab_ranges(zs, zo, ns, D):
        xs = mx_planes(xq, bits, N, Ci, D, HW, z0, z1)
        Ss = (z1 - z0) * HW
        ys = np.zeros((N, Co, Ss), np.float32)
        orc.lib().orc_conv1_mx(bits, orc.ptr(xs), N, Ci, Ss, orc.ptr(w), orc.ptr(b), Co, orc.gn(gam, bet, np.ascontiguousarray(mean[:, s]), np.ascontiguousarray(rstd[:, s]), G), orc.ptr(ys))
        assert np.array_equal(y.reshape(N, Co, D, HW)[:, :, z0:z1].reshape(N, Co, Ss), ys), s


def staged(xq, xdt, N, Ci, D, H, W, cbits, gp, x2=None, c_split=0, gp2=None, stride=1):
    c = orc.orc_conv_t()
    c.x, c.xdt, c.N, c.Ci, c.D, c.H, c.W, c.cbits, c.stride = orc.ptr(xq), xdt, N, Ci, D, H, W, cbits, stride
    c.x2, c.c_split = orc.ptr(x2), c_split
    c.gp = gp; c.gp2 = gp2 if gp2 is not None else orc.orc_gn_t()
    Cx = c_split if x2 is not None else Ci
    nch = (Cx + 31) // 32 + ((Ci - Cx + 31) // 32 if x2 is not None else 0)
    st = np.zeros((N, nch, D * H * W, 32), np.float32)
    assert orc.lib().orc_conv3_staged(c, orc.ptr(st)) == nch * 32
    return st


@pytest.mark.parametrize("bits,zs,zo,ns", [(8, 4, 0, 2), (4, 3, 1, 3)])
def test_conv_staging_takes_each_plane_s_slab(bits, zs, zo, ns):
    """The conv's staged operand (GroupNorm + SiLU, then the compute format): a slab's planes equal the per-sample staging with that slab's rows,
    for a plain input and for the skip segment of a split input whose first segment keeps per-sample statistics."""
    rng = np.random.default_rng(bits + zs)
    N, D, H, W, G = 2, 8, 3, 4, 4
    HW, S = H * W, D * H * W
    xdt = 3 if bits == 8 else 4
    for Cx, C2 in ((64, 0), (32, 32)):
        Ci = Cx + C2
        x = rng.standard_normal((N, Cx, S)).astype(np.float32); xq = orc.f32_to_mx(bits, x, N, Cx, S)
        x2q = orc.f32_to_mx(bits, rng.standard_normal((N, C2, S)).astype(np.float32), N, C2, S) if C2 else None
        gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-0.5, 0.5, Ci).astype(np.float32)
        mean, rstd = stats(rng, N, ns, G)
        m1 = rng.uniform(-0.3, 0.3, (N, G)).astype(np.float32); r1 = rng.uniform(0.6, 1.6, (N, G)).astype(np.float32)
        if C2:
            gp = orc.gn(gam[:Cx], bet[:Cx], m1, r1, G)
            mk2 = lambda m, r, slab=None: orc.gn(gam[Cx:], bet[Cx:], m, r, G, slab=slab)
            full = staged(xq, xdt, N, Ci, D, H, W, bits, gp, x2q, Cx, mk2(mean, rstd, (zs, zo, ns, HW)))
            per = [staged(xq, xdt, N, Ci, D, H, W, bits, gp, x2q, Cx, mk2(np.ascontiguousarray(mean[:, s]), np.ascontiguousarray(rstd[:, s]))) for s in range(ns)]
        else:
            full = staged(xq, xdt, N, Ci, D, H, W, bits, orc.gn(gam, bet, mean, rstd, G, slab=(zs, zo, ns, HW)))
            per = [staged(xq, xdt, N, Ci, D, H, W, bits, orc.gn(gam, bet, np.ascontiguousarray(mean[:, s]), np.ascontiguousarray(rstd[:, s]), G)) for s in range(ns)]
        f5 = full.reshape(N, -1, D, HW, 32)
        for s, z0, z1 in slab_ranges(zs, zo, ns, D):
            assert np.array_equal(f5[:, :, z0:z1], per[s].reshape(N, -1, D, HW, 32)[:, :, z0:z1]), (Cx, C2, s)
        assert not np.array_equal(full, per[0])


@pytest.mark.parametrize("stride", [1, 2])
def test_conv_output_planes_around_a_slab_boundary(stride):
    """Output plane z reads input planes z - 1 .. z + 1 (stride 2: 2z - 1 .. 2z + 1). Planes whose inputs lie in one slab equal the conv with
    that slab's rows as per-sample statistics; planes whose inputs straddle the boundary equal neither: the boundary sits where zs and zo put it."""
    rng = np.random.default_rng(5 + stride)
    N, Ci, Co, D, H, W, G = 1, 32, 32, 12, 4, 4, 4
    zs, zo, ns = 6, 1, 2                                   # boundary: input planes 0 .. 4 | 5 .. 11
    zb = zs - zo
    S = D * H * W
    xq = orc.f32_to_mx(8, rng.standard_normal((N, Ci, S)).astype(np.float32), N, Ci, S)
    w = (rng.standard_normal((Co, Ci, 27)) * 0.1).astype(np.float32); b = rng.standard_normal(Co).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-0.5, 0.5, Ci).astype(np.float32)
    mean, rstd = stats(rng, N, ns, G)
    y, _ = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 0, stride=stride, gp=orc.gn(gam, bet, mean, rstd, G, slab=(zs, zo, ns, H * W)))
    per = [orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 0, stride=stride, gp=orc.gn(gam, bet, np.ascontiguousarray(mean[:, s]), np.ascontiguousarray(rstd[:, s]), G))[0] for s in range(ns)]
    Do = (D - 1) // 2 + 1 if stride == 2 else D
    y = y.reshape(N, Co, Do, -1); per = [p.reshape(N, Co, Do, -1) for p in per]
    for z in range(Do):
        lo, hi = (2 * z - 1, 2 * z + 1) if stride == 2 else (z - 1, z + 1)
        lo, hi = max(lo, 0), min(hi, D - 1)
        if hi < zb:
            assert np.array_equal(y[:, :, z], per[0][:, :, z]), z
        elif lo >= zb:
            assert np.array_equal(y[:, :, z], per[1][:, :, z]), z
        else:
            assert not np.array_equal(y[:, :, z], per[0][:, :, z]) and not np.array_equal(y[:, :, z], per[1][:, :, z]), z


@pytest.mark.parametrize("Ci,tile", [(8, 1), (4, 1), (16, 2), (12, 2)])
def test_few_channel_conv_output_planes_around_a_slab_boundary(Ci, tile):
    """The few-channel forms (one activation scale per staged tile, or per staged row; src/lp_f8fwd.cuh:497 takes the slab row per staged
    plane): output planes whose staged input planes lie in one slab equal the conv with that slab's rows as per-sample statistics. The
    tap-packed form's tile scale couples the planes of a two-plane tile, so whole tiles are compared there."""
    rng = np.random.default_rng(Ci + tile)
    N, Co, D, H, W, G = 1, 32, 12, 8, 16, 4
    zs, zo, ns = 6, 0, 2                                   # boundary between input planes 5 and 6
    S = D * H * W
    xq = orc.f32_to_mx(8, rng.standard_normal((N, Ci, S)).astype(np.float32), N, Ci, S)
    w = (rng.standard_normal((Co, Ci, 27)) * 0.1).astype(np.float32); b = rng.standard_normal(Co).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-0.5, 0.5, Ci).astype(np.float32)
    mean, rstd = stats(rng, N, ns, G)
    y, _ = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 0, stem_tile=tile, gp=orc.gn(gam, bet, mean, rstd, G, slab=(zs, zo, ns, H * W)))
    per = [orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 0, stem_tile=tile, gp=orc.gn(gam, bet, np.ascontiguousarray(mean[:, s]), np.ascontiguousarray(rstd[:, s]), G))[0] for s in range(ns)]
    y = y.reshape(N, Co, D, -1); per = [p.reshape(N, Co, D, -1) for p in per]
    for z in range(D):
        t0 = z & ~1                                        # the staged planes of the output plane's tile (tap-packed) or of the plane itself
        lo, hi = (t0 - 1, t0 + 2) if tile == 1 else (z - 1, z + 1)
        lo, hi = max(lo, 0), min(hi, D - 1)
        if hi < zs:
            assert np.array_equal(y[:, :, z], per[0][:, :, z]), z
        elif lo >= zs:
            assert np.array_equal(y[:, :, z], per[1][:, :, z]), z
        elif max(z - 1, 0) < zs <= min(z + 1, D - 1):      # the plane's own taps straddle the boundary (a straddling tile's other plane may
            assert not np.array_equal(y[:, :, z], per[0][:, :, z]) and not np.array_equal(y[:, :, z], per[1][:, :, z]), z      # share its scale with a per-sample run)
