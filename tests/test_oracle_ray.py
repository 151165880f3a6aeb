"""Pins of the radial-attention oracle (oracle/ray_oracle.py) by what the geometry and the algebra fix, and the product's host-side ray plan
(at_rays_dims / at_rays_plan of libufsm_lp.so: host code, no GPU) against it. The reference's own test of this path (tests/test_attn_ray.c)
holds no stored vectors: it checks these same facts and a double-precision block."""
import ctypes as C
import math
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import ray_oracle as ro  # noqa: E402
import orc  # noqa: E402
from test_oracle_block import make_block  # noqa: E402


def make_axr(n, D, Hh, W, ads, kinds):
    """the axis records of tests/test_attn_ray.c:96-108: kind 0 an axis inside the plane drifting with k, 1 one outside, 2 none"""
    P = max(D, Hh, W); a = np.zeros((n, ro.axr_len(P)), np.float32)
    for b in range(n):
        Np, Nu, Nv = ro.ray_plane(ads[b], D, Hh, W)
        a[b, 0] = ads[b]; a[b, 1] = kinds[b] != 2
        for k in range(Np):
            a[b, 2 + 2 * k], a[b, 3 + 2 * k] = (0.37 * Nu + 0.21 * k, 0.55 * Nv - 0.13 * k) if kinds[b] == 0 else (-2.3 - 0.1 * k, 1.4 * Nv + 0.6 + 0.05 * k)
    return a


GRIDS = [(6, 5, 7, 2.0), (4, 8, 8, 1.5), (8, 8, 8, 2.0)]


def clip_independent(cu, cv, du, dv, Nu, Nv):
    """where the half line from (cu, cv) along (du, dv) lies inside [-0.5, Nu - 0.5] x [-0.5, Nv - 0.5]: by dense sampling, not by slabs"""
    t = np.linspace(0, 4 * (Nu + Nv), 400001)
    pu, pv = cu + t * du, cv + t * dv
    m = (pu >= -0.5) & (pu <= Nu - 0.5) & (pv >= -0.5) & (pv <= Nv - 0.5)
    return (t[m].min(), t[m].max()) if m.any() else None


@pytest.mark.parametrize("D,Hh,W,mult", GRIDS)
def test_plan_geometry(D, Hh, W, mult):
    n, ads, kinds = 3, (0, 1, 2), (0, 1, 2)
    axr = make_axr(n, D, Hh, W, ads, kinds)
    Q, Nt, Nr = ro.rays_dims(D, Hh, W, mult); P = max(D, Hh, W)
    assert Nt == math.ceil(mult * P) and Q == P * Nt
    d2 = sorted((D, Hh, W))[1:]
    assert Nr - 1 == math.ceil(math.hypot(*d2))                                   # the longest plane diagonal over the axis choices
    ray, lens, ad, cen = ro.rays_plan(n, D, Hh, W, mult, axr)
    assert ray.shape == (n, Q, 8) and list(ad) == list(ads)
    rng = np.random.default_rng(0)
    for b in range(n):
        Np, Nu, Nv = ro.ray_plane(ads[b], D, Hh, W)
        for q in range(Q):
            rr = ray[b, q].astype(np.float64); k, j = q // Nt, q % Nt; L = int(rr[6])
            assert rr[7] == k and lens[b, q] == max(1, L) and L <= Nr
            if k >= Np:
                assert L == 0
                continue
            if kinds[b] == 2:                                                     # no axis: the grid rows along v
                assert (L == min(Nv, Nr) and tuple(rr[:6]) == (j, 0, 0, 1, 0, j)) if j < Nu else L == 0
                continue
            if L == 0:
                continue
            cu, cv = axr[b, 2 + 2 * k], axr[b, 3 + 2 * k]
            assert abs(math.hypot(rr[2], rr[3]) - 1) < 1e-6                       # unit steps
            i = np.arange(L); pu, pv = rr[0] + i * rr[2], rr[1] + i * rr[3]
            assert (pu >= -0.5 - 1e-4).all() and (pu <= Nu - 0.5 + 1e-4).all() and (pv >= -0.5 - 1e-4).all() and (pv <= Nv - 0.5 + 1e-4).all()
            assert abs(math.hypot(rr[0] - cu, rr[1] - cv) - rr[4]) < 1e-4         # r0 is sample 0's distance from the centre
            if rng.random() < 0.15:                                               # (the dense clipping is slow: a sample of the rays)
                lo, hi = clip_independent(cu, cv, rr[2], rr[3], Nu, Nv); chord = hi - lo
                assert L == min(Nr, max(1, int(math.floor(chord + 1e-3)))) or L == min(Nr, max(1, int(math.floor(chord - 1e-3))))
                assert abs((rr[4] - lo) - (hi - (rr[4] + L - 1))) < 2e-3          # centred on the chord: the same margin at both ends
            th = math.atan2(rr[3], rr[2]); rc = cen[b, k, 2]
            assert abs(math.remainder(rr[5] / rc - th, 2 * math.pi)) < 1e-5       # arc = angle x the plane's radius
        if kinds[b] == 0:                                                         # centre inside: the fan is the full circle, rays 2 pi / Nt apart
            a0 = ray[b, :Nt, 5].astype(np.float64) / cen[b, 0, 2]
            assert np.allclose(np.diff(a0), 2 * math.pi / Nt, atol=1e-5) and abs(a0[0] + math.pi - math.pi / Nt) < 1e-5
        if kinds[b] == 1:                                                         # centre outside: the fan spans exactly the rectangle's corners
            k = 1; cu, cv = axr[b, 2 + 2 * k], axr[b, 3 + 2 * k]; phim = cen[b, k, 3]
            ths = [phim + math.remainder(math.atan2(qv - cv, qu - cu) - phim, 2 * math.pi) for qu in (-0.5, Nu - 0.5) for qv in (-0.5, Nv - 0.5)]
            a1 = ray[b, k * Nt:(k + 1) * Nt, 5].astype(np.float64) / cen[b, k, 2]; step = (max(ths) - min(ths)) / Nt
            assert abs(a1[0] - (min(ths) + 0.5 * step)) < 1e-5 and abs(a1[-1] - (max(ths) - 0.5 * step)) < 1e-5
            assert abs(phim - math.atan2(0.5 * (Nv - 1) - cv, 0.5 * (Nu - 1) - cu)) < 1e-6
        assert (cen[b, :, 2] == -1).all() if kinds[b] == 2 else (cen[b, :Np, 2] >= 0.5 * max(Nu, Nv) - 1e-6).all()


@pytest.mark.parametrize("D,Hh,W,mult", GRIDS)
def test_library_plan_equals_the_oracle_plan(D, Hh, W, mult):
    from ufsm_amd import lp
    L = lp.load()
    n, ads, kinds = 4, (0, 1, 2, 2), (0, 1, 2, 1)
    axr = make_axr(n, D, Hh, W, ads, kinds)
    q, nt, nr = C.c_int(), C.c_int(), C.c_int()
    L.at_rays_dims(D, Hh, W, C.c_float(mult), C.byref(q), C.byref(nt), C.byref(nr))
    assert (q.value, nt.value, nr.value) == ro.rays_dims(D, Hh, W, mult)
    P = max(D, Hh, W)
    ray = np.full((n, q.value, 8), 7, np.float32); lens = np.full((n, q.value), -3, np.int32); ad = np.full(n, -3, np.int32); cen = np.full((n, P, 4), 7, np.float32)
    L.at_rays_plan(n, D, Hh, W, C.c_float(mult), axr.ctypes.data, ray.ctypes.data, lens.ctypes.data, ad.ctypes.data, cen.ctypes.data)
    wray, wlens, wad, wcen = ro.rays_plan(n, D, Hh, W, mult, axr)
    assert np.array_equal(lens, wlens) and np.array_equal(ad, wad)
    assert np.array_equal(ray[..., 6:], wray[..., 6:])                            # lengths and planes
    assert np.abs(ray - wray).max() < 1e-5 and np.abs(cen - wcen).max() < 1e-5   # (two libms: the last bit of a sine may differ)


def test_stencil_is_bilinear_and_the_maps_are_adjoint():
    D, Hh, W, mult = 6, 5, 7, 2.0; n = 3
    R = ro.make_rays(n, D, Hh, W, mult, make_axr(n, D, Hh, W, (0, 1, 2), (0, 1, 2)))
    rows, w = R["rows"], R["w"]; used = rows[:, 0] >= 0
    assert used.sum() == R["lens"].sum() - (R["ray"][..., 6] == 0).sum()          # one stencil per slot inside a ray's length (dummies: none)
    assert np.abs(w[used].sum(1) - 1).max() < 1e-6 and (w >= 0).all()
    # an affine field of the in-plane coordinates is reproduced at every sample (the samples lie inside the plane's rectangle, where clamping
    # only acts within half a voxel of the border: compare against the clamped sample position)
    Tg = n * D * Hh * W; zz, yy, xx = np.meshgrid(np.arange(D), np.arange(Hh), np.arange(W), indexing="ij")
    for b in range(n):
        ad = R["ad"][b]; Np, Nu, Nv = ro.ray_plane(ad, D, Hh, W)
        u = (yy if ad == 0 else zz).reshape(-1).astype(np.float64); v = (yy if ad == 2 else xx).reshape(-1).astype(np.float64)
        f = np.zeros((Tg, 2)); f[b * D * Hh * W:(b + 1) * D * Hh * W] = np.stack([u, v], 1)
        g = ro.gather(f, rows, w)
        for q in range(R["Q"]):
            rr = R["ray"][b, q].astype(np.float64)
            for i in range(int(rr[6])):
                s = (b * R["Q"] + q) * R["Nr"] + i
                want = (min(max(rr[0] + i * rr[2], 0), Nu - 1), min(max(rr[1] + i * rr[3], 0), Nv - 1))
                assert abs(g[s, 0] - want[0]) < 1e-4 and abs(g[s, 1] - want[1]) < 1e-4
    rng = np.random.default_rng(1); Cc = 5
    x = rng.standard_normal((Tg, Cc)); y = rng.standard_normal((rows.shape[0], Cc))
    for winv in (None, R["winv"]):
        a, b2 = (ro.gather(x, rows, w, winv) * y).sum(), (x * ro.scatter(y, rows, w, Tg, winv)).sum()
        assert abs(a - b2) < 1e-9 * np.abs(x).sum()
    # the normalised scatter of a gathered constant is that constant on every covered token, 0 elsewhere
    one = ro.scatter(ro.gather(np.ones((Tg, 1)), rows, w), rows, w, Tg, R["winv"])[:, 0]
    cov = R["winv"] > 0
    assert np.abs(one[cov] - 1).max() < 1e-6 and (one[~cov] == 0).all() and cov.mean() > 0.8
    # no axis: the rays are the grid rows, every token exactly once
    b = 2; sl = slice(b * D * Hh * W, (b + 1) * D * Hh * W)
    assert np.allclose(R["winv"][sl], 1)
    xs = np.zeros((Tg, 1)); xs[sl, 0] = np.arange(D * Hh * W)
    gs = ro.gather(xs, rows, w)[b * R["Q"] * R["Nr"]:(b + 1) * R["Q"] * R["Nr"], 0].reshape(R["Q"], R["Nr"])
    Np, Nu, Nv = ro.ray_plane(2, D, Hh, W)
    for k in range(Np):
        for j in range(Nu):
            assert np.array_equal(gs[k * R["Nt"] + j, :Nv], [ro.ray_token(2, k, j, vv, Hh, W) for vv in range(Nv)])


def test_scroll_positions():
    D, Hh, W = 5, 6, 4; n = 3
    ray, lens, ad, cen = ro.rays_plan(n, D, Hh, W, 2.0, make_axr(n, D, Hh, W, (1, 0, 2), (0, 1, 2)))
    nreg = 2; pos = ro.scroll_pos(n, nreg, D, Hh, W, ad, cen).reshape(n, -1, 3)
    assert (pos[:, :nreg] == 0).all()
    for b in range(n):
        for ts in range(D * Hh * W):
            z, y, x = ts // (Hh * W), ts // W % Hh, ts % W
            k, ua, vb = (z, y, x) if ad[b] == 0 else (y, z, x) if ad[b] == 1 else (x, z, y)
            p = pos[b, nreg + ts]
            if b == 2:
                assert tuple(p) == (vb, ua, k)                                    # no axis: the grid indices
                continue
            cu, cv, rc, phim = cen[b, k].astype(np.float64)
            assert p[2] == k and abs(p[0] - math.hypot(ua - cu, vb - cv)) < 1e-9
            th = p[1] / rc                                                        # the token sits at radius r and angle arc / rc from the centre
            assert abs(cu + p[0] * math.cos(th) - ua) < 1e-6 and abs(cv + p[0] * math.sin(th) - vb) < 1e-6 and abs(th - phim) <= math.pi + 1e-9


def test_rotary_coordinates():
    rng = np.random.default_rng(2)
    nseq, D, nreg, Cc, H = 2, 3, 2, 96, 2; S = nreg + D ** 3; T = nseq * S
    qkv = rng.standard_normal((T, 3 * Cc)).astype(np.float32); qg = (1 + 0.2 * rng.standard_normal(Cc)).astype(np.float32); kg = (1 + 0.2 * rng.standard_normal(Cc)).astype(np.float32)
    # with the grid indices as coordinates the rotation is the C oracle's grid-index pack (pinned by its own tests)
    wqh = orc.fa_pack(qkv, qg, kg, nseq, S, D, D, nreg, Cc, 1, 100.0)[0].view(np.float16).astype(np.float64).reshape(3, H, T + 64, 48)
    q = qkv[:, :Cc].astype(np.float64).reshape(T, H, 48)
    q = q / np.sqrt((q ** 2).mean(-1, keepdims=True) + 1e-6) * qg.astype(np.float64).reshape(H, 48)
    mask = (np.arange(T) % S) >= nreg
    qr = np.where(mask[:, None, None], ro.rope(q, ro.grid_pos(nseq, S, D, D, D, nreg), 100.0), q)
    assert np.abs(qr.transpose(1, 0, 2) - wqh[0, :, :T]).max() < 2e-3 * np.abs(qr).max()          # (fp16 storage of the C oracle's result)
    # rotary attention sees coordinate differences only: the same block output after a shift of every token's coordinates
    P, lay = make_block(rng, Cc, 128)
    x = rng.standard_normal((T, Cc)).astype(np.float32)
    pos = rng.uniform(0, 9, (T, 3)); pos[~mask] = 0
    y0 = ro.block(P, lay, x, nseq, S, H, Cc, 128, rope_mode=2, pos=pos, nreg=0)
    y1 = ro.block(P, lay, x, nseq, S, H, Cc, 128, rope_mode=2, pos=pos + np.array([3.25, -1.5, 7.0]), nreg=0)
    assert np.abs(y0 - y1).max() < 1e-9 and np.abs(y0 - ro.block(P, lay, x, nseq, S, H, Cc, 128, rope_mode=0)).max() > 1e-3


def test_radial_block_without_an_axis_is_attention_along_the_grid_rows():
    rng = np.random.default_rng(3)
    D, Hh, W, Cc, H, F = 3, 4, 5, 96, 2, 128; n = 2; S = D * Hh * W; T = n * S
    axr = make_axr(n, D, Hh, W, (0, 0), (2, 2))
    R = ro.make_rays(n, D, Hh, W, 2.0, axr)
    P, lay = make_block(rng, Cc, F)
    x = rng.standard_normal((T, Cc)).astype(np.float32)
    y = ro.block(P, lay, x, n, S, H, Cc, F, rope_mode=2, rays=R)
    # written directly: the tokens of a row (z, y, :) attend to each other; coordinates (r, arc, k) = (x index, y index, z)
    pos = np.zeros((T, 3)); ts = np.arange(S)
    pos[:, 0] = np.tile(ts % W, n); pos[:, 1] = np.tile(ts // W % Hh, n); pos[:, 2] = np.tile(ts // (Hh * W), n)
    yd = ro.block(P, lay, x, n * D * Hh, W, H, Cc, F, rope_mode=2, pos=pos)
    assert np.abs(y - yd).max() < 1e-9
    # and it differs from full attention over the grid
    assert np.abs(y - ro.block(P, lay, x, n, S, H, Cc, F, rope_mode=2, pos=pos)).max() > 1e-3
