"""CPU restatement (numpy, double precision) of the reference's radial attention and scroll coordinates. TEST INFRASTRUCTURE ONLY: the checker of
tests/ (and nothing else may import it); the product path is ufsm_amd/csrc/attn_ray.hip.

Follows, function by function:
  rays_dims, rays_plan   src/nn_attn_ray.cu:12-20, :22-41, :43-104 (the host plan: ray records u0, v0, du, dv, r0, arc, len, k; the scroll frame)
  stencil                src/attn.h:118-128 (bilinear corners of a ray slot, float arithmetic), :130-136 (plane / token mapping)
  ray_pos, scroll_pos    src/nn_attn_ray.cu:118-123, :174-188
  gather, scatter, wsum  src/nn_attn_ray.cu:124-173 (the maps and the normalising weight sums)
  rope                   src/nn_attn.cu:272-289 (rotary pairs on three coordinates, 16 head dims each)
  block                  src/nn_attn.cu:576-633 with the attention on rays (gather, QK-norm, RoPE, length-masked softmax per ray, normalised
                         scatter) or over the grid with per-token coordinates, everything in double: the role of tests/test_attn_ray.c's ref_block

Pinned by tests/test_oracle_ray.py: the geometric facts the plan must satisfy (samples inside the rectangle at unit spacing and centred on the
chord, which an independent clipping computes; fans that cover the rectangle), bilinear exactness on affine fields, the adjoint identities, rays
without an axis = grid rows (a radial block then equals row-wise attention written directly), rotary attention's invariance under a shift of all
coordinates and its equality with the grid-index form of the C oracle's pack when the coordinates are the grid indices."""
import math
import os

import numpy as np

RAY_F = 8


def axr_len(pmax):
    return 2 + 2 * pmax


def ray_plane(ad, D, Hh, W):
    """planes along the axis dim, then the plane's two dims (u, v: the other two of z, y, x in order)"""
    return (D, Hh, W)[ad], (Hh if ad == 0 else D), (Hh if ad == 2 else W)


def ray_token(ad, k, a, b, Hh, W):
    z, y, x = (k, a, b) if ad == 0 else (a, k, b) if ad == 1 else (a, b, k)
    return (z * Hh + y) * W + x


def rays_dims(D, Hh, W, mult):
    P = max(D, Hh, W)
    nt = max(1, int(math.ceil(np.float32(mult) * np.float32(P))))
    lo, mid, hi = sorted((D, Hh, W))
    return P * nt, nt, int(math.ceil(math.sqrt(float(mid) * mid + float(hi) * hi))) + 1       # Q, Nt, Nr


def _ray_record(cu, cv, th, rc, Nu, Nv, Nr, k):
    rr = np.zeros(RAY_F, np.float32); rr[7] = k
    du, dv = math.cos(th), math.sin(th)
    tlo, thi, miss = 0.0, 1e300, False
    for c, d, hi in ((cu, du, Nu - 0.5), (cv, dv, Nv - 0.5)):
        if abs(d) < 1e-12:
            miss = miss or c < -0.5 or c > hi
            continue
        t1, t2 = (-0.5 - c) / d, (hi - c) / d
        if t1 > t2:
            t1, t2 = t2, t1
        tlo, thi = max(tlo, t1), min(thi, t2)
    chord = thi - tlo
    if miss or not chord > 1e-6:
        return rr
    L = min(1 if chord < 1 else int(math.floor(chord)), Nr)
    t0 = tlo + 0.5 * (chord - (L - 1))
    rr[:7] = (cu + t0 * du, cv + t0 * dv, du, dv, t0, th * rc, L)
    return rr


def rays_plan(n, D, Hh, W, mult, axr):
    """axr [n][2 + 2 Pmax] float32 -> ray [n][Q][8] f32, lens [n][Q] i32, ad [n] i32, cen [n][Pmax][4] f32"""
    Q, Nt, Nr = rays_dims(D, Hh, W, mult); P = max(D, Hh, W)
    v2 = int(os.environ.get("UFSM_SCROLL_PE_V2", "0") or 0) > 0
    axr = np.asarray(axr, np.float32).reshape(n, axr_len(P))
    ray = np.zeros((n, Q, RAY_F), np.float32); cen = np.zeros((n, P, 4), np.float32); ads = np.zeros(n, np.int32)
    for b in range(n):
        a = axr[b].astype(np.float64); ad = int(a[0])
        if ad < 0 or ad > 2:
            ad = 0
        valid = a[1] != 0; Np, Nu, Nv = ray_plane(ad, D, Hh, W); ads[b] = ad
        mu, mv, rmin = 0.5 * (Nu - 1), 0.5 * (Nv - 1), 0.5 * max(Nu, Nv)
        rcr = phir = 0.0
        if v2 and valid:
            cs = a[2:2 + 2 * Np].reshape(Np, 2)
            sx, sy, sr = (mu - cs[:, 0]).sum(), (mv - cs[:, 1]).sum(), np.hypot(mu - cs[:, 0], mv - cs[:, 1]).sum()
            rcr = max(sr / Np, rmin); phir = math.atan2(sy, sx) if math.hypot(sx, sy) > 0.25 * Np else 0.0
        for k in range(P):
            for j in range(Nt):
                rr = ray[b, k * Nt + j]; rr[7] = k
                if k >= Np:
                    continue
                if not valid:
                    if j < Nu:
                        rr[0] = j; rr[3] = 1; rr[5] = j; rr[6] = min(Nv, Nr)
                    continue
                cu, cv = a[2 + 2 * k], a[3 + 2 * k]
                inside = -0.5 <= cu <= Nu - 0.5 and -0.5 <= cv <= Nv - 0.5
                rc = max(math.hypot(mu - cu, mv - cv), rmin); phim, th0, th1 = 0.0, -math.pi, math.pi
                if v2:
                    rc, phim, th0, th1 = rcr, phir, phir - math.pi, phir + math.pi
                if not inside:
                    if not v2:
                        phim = math.atan2(mv - cv, mu - cu)
                    ths = [phim + math.remainder(math.atan2(qv - cv, qu - cu) - phim, 2 * math.pi) for qu in (-0.5, Nu - 0.5) for qv in (-0.5, Nv - 0.5)]
                    th0, th1 = min(ths), max(ths)
                if j == 0:
                    cen[b, k] = (cu, cv, rc, phim)
                ray[b, k * Nt + j] = _ray_record(cu, cv, th0 + (j + 0.5) * (th1 - th0) / Nt, rc, Nu, Nv, Nr, k)
        if not valid:
            cen[b, :, 2] = -1
    lens = np.maximum(ray[:, :, 6].astype(np.int32), 1)
    return ray, lens, ads, cen


def stencil(ray, ads, Nr, D, Hh, W):
    """per ray slot [n Q Nr] up to four (grid row, weight): rows int64 (-1: none), w float64 of the float32 arithmetic of src/attn.h:118-128"""
    n, Q, _ = ray.shape; Sg = D * Hh * W
    rows = np.full((n * Q * Nr, 4), -1, np.int64); w = np.zeros((n * Q * Nr, 4))
    f = np.float32
    for b in range(n):
        ad = int(ads[b]); Np, Nu, Nv = ray_plane(ad, D, Hh, W)
        for q in range(Q):
            rr = ray[b, q]; k = int(rr[7])
            for i in range(min(int(rr[6]), Nr)):
                pu = min(max(f(rr[0] + f(i) * rr[2]), f(0)), f(Nu - 1)); pv = min(max(f(rr[1] + f(i) * rr[3]), f(0)), f(Nv - 1))
                a0 = max(min(int(pu), Nu - 2), 0); b0 = max(min(int(pv), Nv - 2), 0); a1 = min(a0 + 1, Nu - 1); b1 = min(b0 + 1, Nv - 1)
                fu, fv = f(pu - f(a0)), f(pv - f(b0)); s = (b * Q + q) * Nr + i
                rows[s] = [b * Sg + ray_token(ad, k, aa, bb, Hh, W) for aa, bb in ((a0, b0), (a1, b0), (a0, b1), (a1, b1))]
                w[s] = [f(f(1) - fu) * f(f(1) - fv), fu * f(f(1) - fv), f(f(1) - fu) * fv, fu * fv]
    return rows, w


def wsum_inv(rows, w, Tg):
    acc = np.zeros(Tg); m = rows >= 0
    np.add.at(acc, rows[m], w[m])
    return np.where(acc > 1e-6, 1 / np.where(acc > 1e-6, acc, 1), 0.0)


def gather(x, rows, w, winv=None):
    """grid rows x [Tg][C] -> ray rows [Tr][C]; winv: the normalised form (each corner's weight x the token's 1 / weight sum)"""
    y = np.zeros((rows.shape[0], x.shape[1]))
    for c in range(4):
        m = rows[:, c] >= 0; r = rows[m, c]
        y[m] += (w[m, c] * (winv[r] if winv is not None else 1.0))[:, None] * x[r]
    return y


def scatter(y, rows, w, Tg, winv=None):
    x = np.zeros((Tg, y.shape[1]))
    for c in range(4):
        m = rows[:, c] >= 0; r = rows[m, c]
        np.add.at(x, r, (w[m, c] * (winv[r] if winv is not None else 1.0))[:, None] * y[m])
    return x


def ray_pos(ray, Nr):
    n, Q, _ = ray.shape
    pos = np.zeros((n, Q, Nr, 3))
    pos[..., 0] = ray[:, :, None, 4].astype(np.float64) + np.arange(Nr)
    pos[..., 1] = ray[:, :, None, 5]; pos[..., 2] = ray[:, :, None, 7]
    return pos.reshape(-1, 3)


def scroll_pos(n, nreg, D, Hh, W, ads, cen):
    S = nreg + D * Hh * W; pos = np.zeros((n, S, 3))
    for b in range(n):
        ad = int(ads[b])
        for ts in range(D * Hh * W):
            z, y, x = ts // (Hh * W), ts // W % Hh, ts % W
            k, ua, vb = (z, y, x) if ad == 0 else (y, z, x) if ad == 1 else (x, z, y)
            c = cen[b, k].astype(np.float64)
            if c[2] < 0:
                pos[b, nreg + ts] = (vb, ua, k)
                continue
            du, dv = ua - c[0], vb - c[1]
            th = c[3] + math.remainder(math.atan2(dv, du) - c[3], 2 * math.pi)
            pos[b, nreg + ts] = (math.hypot(du, dv), th * c[2], k)
    return pos.reshape(-1, 3)


def rope(q, pos, base):
    """q [T][H][48] double, pos [T][3] (None rows never occur: pass zeros for registers and skip them with mask) -> rotated copy"""
    T = q.shape[0]; out = q.copy()
    fr = base ** (-np.arange(8) / 8.0)
    for ax in range(3):
        ang = pos[:, ax, None] * fr[None, :]                                   # [T][8]
        cs, sn = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
        a = q[:, :, 16 * ax:16 * ax + 16:2]; b = q[:, :, 16 * ax + 1:16 * ax + 16:2]
        out[:, :, 16 * ax:16 * ax + 16:2] = a * cs - b * sn
        out[:, :, 16 * ax + 1:16 * ax + 16:2] = a * sn + b * cs
    return out


def grid_pos(nseq, S, D, Hh, W, nreg):
    """the grid indices (z, y, x) per token, registers 0: the coordinates of rope 1"""
    pos = np.zeros((nseq, S, 3)); ts = np.arange(D * Hh * W)
    pos[:, nreg:, 0] = ts // (Hh * W); pos[:, nreg:, 1] = ts // W % Hh; pos[:, nreg:, 2] = ts % W
    return pos.reshape(-1, 3)


def _ln(x, g, b, eps=1e-5):
    m = x.mean(-1, keepdims=True); v = ((x - m) ** 2).mean(-1, keepdims=True)
    return (x - m) / np.sqrt(v + eps) * g + b


def attend(q, k, v, nseq, S, lens=None):
    """q, k, v [nseq S][H][48] -> o [nseq S][H 48]: softmax over the first lens[s] keys of each sequence (None: S); length 0: zeros"""
    T, H, _ = q.shape; o = np.zeros((T, H * 48))
    for s in range(nseq):
        L = S if lens is None else int(lens[s]); sl = slice(s * S, (s + 1) * S); kl = slice(s * S, s * S + L)
        if L <= 0:
            continue
        for h in range(H):
            lg = q[sl, h] @ k[kl, h].T / math.sqrt(48.0); e = np.exp(lg - lg.max(1, keepdims=True))
            o[sl, h * 48:(h + 1) * 48] = (e / e.sum(1, keepdims=True)) @ v[kl, h]
    return o


def attention(qkv, qg, kg, nseq, S, H, Cc, rope_mode=0, base=100.0, nreg=0, pos=None, grid=None, rays=None):
    """the attention branch between the two projections: qkv rows [T][3 C] -> o [T][C] (QK-norm with gains, RoPE, softmax per sequence; with rays:
    gathered onto the ray samples first, length-masked per ray, scattered back normalised)"""
    T = nseq * S; Ta, nsa, Sa, lens = T, nseq, S, None
    if rays is not None:
        qkv = gather(qkv, rays["rows"], rays["w"]); Ta = qkv.shape[0]; Sa = rays["Nr"]; nsa = Ta // Sa; lens = rays["lens"]
    q, k, v = (qkv[:, i * Cc:(i + 1) * Cc].reshape(Ta, H, 48) for i in range(3))
    q = q / np.sqrt((q ** 2).mean(-1, keepdims=True) + 1e-6) * qg.reshape(H, 48)
    k = k / np.sqrt((k ** 2).mean(-1, keepdims=True) + 1e-6) * kg.reshape(H, 48)
    if rope_mode:
        if rays is not None:
            pp = rays["pos"] if rope_mode == 2 else grid_pos(nsa, Sa, 1, 1, Sa, 0)
            mask = np.ones(Ta, bool)
        else:
            pp = pos if rope_mode == 2 else grid_pos(nseq, S, *grid, nreg)
            mask = (np.arange(T) % S) >= nreg
        q = np.where(mask[:, None, None], rope(q, pp, base), q); k = np.where(mask[:, None, None], rope(k, pp, base), k)
    o = attend(q, k, v, nsa, Sa, lens)
    return scatter(o, rays["rows"], rays["w"], T, rays["winv"]) if rays is not None else o


def block(P, lay, x, nseq, S, H, Cc, F, rope_mode=0, base=100.0, nreg=0, pos=None, grid=None, rays=None):
    """the pre-LN block in double. rope_mode 0 none, 1 grid indices (grid = (D, Hh, W)), 2 the coordinates pos [T][3] (rays: the rays' own).
    rays: the dict of make_rays -> radial attention"""
    P = P.astype(np.float64); x = x.astype(np.float64)
    g = lambda name, n: P[lay[name]:lay[name] + n]
    xn = _ln(x, g("ln1g", Cc), g("ln1b", Cc))
    qkv = xn @ g("wqkv", 3 * Cc * Cc).reshape(3 * Cc, Cc).T + g("bqkv", 3 * Cc)
    o = attention(qkv, g("qg", Cc), g("kg", Cc), nseq, S, H, Cc, rope_mode, base, nreg, pos, grid, rays)
    x1 = o @ g("wo", Cc * Cc).reshape(Cc, Cc).T + g("bo", Cc) + x
    xn2 = _ln(x1, g("ln2g", Cc), g("ln2b", Cc))
    hh = xn2 @ g("w1", 2 * F * Cc).reshape(2 * F, Cc).T + g("b1", 2 * F)
    gg = hh[:, :F] / (1 + np.exp(-hh[:, :F])) * hh[:, F:]
    return gg @ g("w2", Cc * F).reshape(Cc, F).T + g("b2", Cc) + x1


def make_rays(n, D, Hh, W, mult, axr):
    """the whole ray set of n samples as the dict block() takes (plus the plan's tables)"""
    ray, lens, ads, cen = rays_plan(n, D, Hh, W, mult, axr); Q, Nt, Nr = rays_dims(D, Hh, W, mult)
    rows, w = stencil(ray, ads, Nr, D, Hh, W); Tg = n * D * Hh * W
    return dict(ray=ray, lens=lens.reshape(-1), ad=ads, cen=cen, Q=Q, Nt=Nt, Nr=Nr, rows=rows, w=w, winv=wsum_inv(rows, w, Tg), pos=ray_pos(ray, Nr), nseq_r=n * Q)
