"""Radial attention and scroll RoPE on the device (include/mi_attn.h: at_rays_setup, at_ray_gather / _scatter, at_scroll_pos, at_fa_fwd, at_fa_pack
with coordinates, at_block_fwd with rays) against the double-precision oracle (oracle/ray_oracle.py), with the gates of the reference's
tests/test_attn_ray.c: max |gpu - ref| / rms(ref) < 2e-3 per tensor for the maps and the fp16 core (the block's MX linears: test_attn.c's MX gate)."""
import ctypes as C
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
import ray_oracle as ro  # noqa: E402
from gpuutil import DevBuf, LP, lib  # noqa: E402
from ufsm_amd import at_geom, at_dims, at_bp, at_ws, at_rays  # noqa: E402
from test_oracle_block import make_block  # noqa: E402
from test_oracle_ray import make_axr  # noqa: E402

pytestmark = pytest.mark.gpu


def rel(a, b):
    return np.abs(a - b).max() / max(np.sqrt((b.astype(np.float64) ** 2).mean()), 1e-30)


class DevRays:
    """a ray set on the device, planned by the library, with the oracle's tables beside it"""

    def __init__(self, n, D, Hh, W, mult, axr):
        self.o = ro.make_rays(n, D, Hh, W, mult, axr)
        q, nt, nr = C.c_int(), C.c_int(), C.c_int()
        lib.at_rays_dims(D, Hh, W, C.c_float(mult), C.byref(q), C.byref(nt), C.byref(nr))
        Q, Nt, Nr = q.value, nt.value, nr.value; P = max(D, Hh, W)
        assert (Q, Nt, Nr) == (self.o["Q"], self.o["Nt"], self.o["Nr"])
        ray = np.zeros((n, Q, 8), np.float32); lens = np.zeros((n, Q), np.int32); ad = np.zeros(n, np.int32); cen = np.zeros((n, P, 4), np.float32)
        lib.at_rays_plan(n, D, Hh, W, C.c_float(mult), axr.ctypes.data, ray.ctypes.data, lens.ctypes.data, ad.ctypes.data, cen.ctypes.data)
        self.ray_h, self.lens_h, self.cen_h = ray, lens, cen
        self.Tr, self.Tg = n * Q * Nr, n * D * Hh * W
        self.bufs = dict(ray=DevBuf.from_numpy(ray), lens=DevBuf.from_numpy(lens), ad=DevBuf.from_numpy(ad), cen=DevBuf.from_numpy(cen),
                         pos=DevBuf.from_numpy(np.full(self.Tr * 3, np.nan, np.float32)), wsum=DevBuf.from_numpy(np.full(self.Tg, np.nan, np.float32)))
        R = at_rays(); R.n, R.Q, R.Nt, R.Nr, R.D, R.Hh, R.W = n, Q, Nt, Nr, D, Hh, W
        R.ad, R.ray, R.lens, R.pos, R.wsum = (self.bufs[k].ptr for k in ("ad", "ray", "lens", "pos", "wsum"))
        self.R = R
        lib.at_rays_setup(C.byref(R)); LP.check()


@pytest.mark.parametrize("D,Hh,W,mult", [(6, 5, 7, 2.0), (8, 8, 8, 2.0)])
def test_ray_maps(gpu, D, Hh, W, mult):
    n = 3; axr = make_axr(n, D, Hh, W, (0, 1, 2), (0, 1, 2))
    t = DevRays(n, D, Hh, W, mult, axr); o = t.o
    pos = t.bufs["pos"].to_numpy(np.float32, (t.Tr, 3)); ws = t.bufs["wsum"].to_numpy(np.float32, (t.Tg,))
    assert np.abs(pos - o["pos"]).max() < 1e-5                                     # (r0 + i, arc, k) as the table says
    assert rel(ws, o["winv"]) < 1e-5 and ((ws > 0) == (o["winv"] > 0)).all()
    rng = np.random.default_rng(0); Cc = 8
    x = rng.standard_normal((t.Tg, Cc)).astype(np.float32); y = rng.standard_normal((t.Tr, Cc)).astype(np.float32)
    dx, dy, dg, ds = DevBuf.from_numpy(x), DevBuf.from_numpy(y), DevBuf.from_numpy(np.full((t.Tr, Cc), np.nan, np.float32)), DevBuf.from_numpy(np.full((t.Tg, Cc), np.nan, np.float32))
    for norm in (0, 1):
        lib.at_ray_gather(C.byref(t.R), dx.ptr, dg.ptr, Cc, norm); lib.at_ray_scatter(C.byref(t.R), dy.ptr, ds.ptr, Cc, norm); LP.check()
        G, S = dg.to_numpy(np.float32, (t.Tr, Cc)), ds.to_numpy(np.float32, (t.Tg, Cc))
        winv = o["winv"] if norm else None
        wg, wsx = ro.gather(x.astype(np.float64), o["rows"], o["w"], winv), ro.scatter(y.astype(np.float64), o["rows"], o["w"], t.Tg, winv)
        assert rel(G, wg) < 1e-5 and rel(S, wsx) < 1e-5
        a, b = (G.astype(np.float64) * y).sum(), (x * S.astype(np.float64)).sum()  # <G x, y> = <x, S y> on the device's own results
        assert abs(a - b) < 1e-5 * np.abs(G.astype(np.float64) * y).sum()
    # slots past a ray's length gather zero rows
    lens = np.repeat(t.ray_h[..., 6].reshape(-1).astype(np.int64), o["Nr"]); slot = np.tile(np.arange(o["Nr"]), n * o["Q"])
    assert (G[slot >= lens] == 0).all()


def test_scroll_pos_on_the_device(gpu):
    D, Hh, W, n, nreg = 5, 6, 4, 3, 2
    axr = make_axr(n, D, Hh, W, (1, 0, 2), (0, 1, 2))
    t = DevRays(n, D, Hh, W, 2.0, axr)
    S = nreg + D * Hh * W; dp = DevBuf.from_numpy(np.full((n * S, 3), np.nan, np.float32))
    lib.at_scroll_pos(n, nreg, D, Hh, W, t.bufs["ad"].ptr, t.bufs["cen"].ptr, dp.ptr); LP.check()
    want = ro.scroll_pos(n, nreg, D, Hh, W, t.o["ad"], t.cen_h)
    got = dp.to_numpy(np.float32, (n * S, 3))
    assert np.abs(got - want).max() < 1e-4


def pack(qkv, qg, kg, g, nreg, Cc, rope):
    T = g.nseq * g.S; H = Cc // 48
    dq, dqg, dkg = DevBuf.from_numpy(qkv), DevBuf.from_numpy(qg), DevBuf.from_numpy(kg)
    dqh = DevBuf.from_numpy(np.full(3 * H * (T + 64) * 48, 0x7e00, np.uint16)); drq, drk, damx = DevBuf(T * H * 4), DevBuf(T * H * 4), DevBuf(16)
    lib.at_fa_pack(dq.ptr, dqg.ptr, dkg.ptr, dqh.ptr, drq.ptr, drk.ptr, damx.ptr, C.byref(g), nreg, Cc, rope, 100.0); LP.check()
    return dqh


def test_pack_with_coordinates_and_the_length_masked_core(gpu):
    rng = np.random.default_rng(5)
    nseq, S, Cc, H = 37, 23, 96, 2; T = nseq * S
    qkv = rng.standard_normal((T, 3 * Cc)).astype(np.float32); qg = (1 + 0.2 * rng.standard_normal(Cc)).astype(np.float32); kg = (1 + 0.2 * rng.standard_normal(Cc)).astype(np.float32)
    pos = rng.uniform(-4, 12, (T, 3)).astype(np.float32); lens = rng.integers(0, S + 1, nseq).astype(np.int32); lens[:3] = (0, 1, S)
    dpos, dlens = DevBuf.from_numpy(pos), DevBuf.from_numpy(lens)
    g = at_geom(); g.nseq, g.S, g.D, g.Hh, g.W = nseq, S, 1, 1, S; g.pos = dpos.ptr
    dqh = pack(qkv, qg, kg, g, 0, Cc, 2)
    got = dqh.to_numpy(np.uint16, (3, H, T + 64, 48)).view(np.float16).astype(np.float64)
    q, k, v = (qkv[:, i * Cc:(i + 1) * Cc].astype(np.float64).reshape(T, H, 48) for i in range(3))
    q = q / np.sqrt((q ** 2).mean(-1, keepdims=True) + 1e-6) * qg.astype(np.float64).reshape(H, 48)
    k = k / np.sqrt((k ** 2).mean(-1, keepdims=True) + 1e-6) * kg.astype(np.float64).reshape(H, 48)
    qr, kr = ro.rope(q, pos.astype(np.float64), 100.0), ro.rope(k, pos.astype(np.float64), 100.0)
    for i, want in enumerate((qr, kr, v)):
        assert np.abs(got[i, :, :T].transpose(1, 0, 2) - want).max() < 1.5e-3 * np.abs(want).max()          # fp16 storage (and fp32 angles up to 12 x 1)
    assert (got[:, :, T:] == 0).all()
    # the core on exactly these fp16 rows, keys masked past each sequence's length
    g.lens = dlens.ptr
    do, dl = DevBuf.from_numpy(np.full((T, Cc), np.nan, np.float32)), DevBuf.from_numpy(np.full((nseq, H, S), np.nan, np.float32))
    lib.at_fa_fwd(dqh.ptr, do.ptr, dl.ptr, C.byref(g), H, Cc); LP.check()
    o = do.to_numpy(np.float32, (T, Cc)); lse = dl.to_numpy(np.float32, (nseq, H, S))
    qh, kh, vh = (got[i, :, :T].transpose(1, 0, 2) for i in range(3))
    want = ro.attend(qh, kh, vh, nseq, S, lens)
    assert rel(o, want) < 2e-3                                                     # (probabilities rounded to fp16 before they meet v)
    assert (o[:S] == 0).all() and (lse[0] == 0).all()                              # a length of 0: zero output
    assert np.abs(o[S:2 * S] - vh[S].reshape(-1)).max() < 1e-6                     # a length of 1: the one key's value for every query
    s = 2; lg = np.einsum("ihd,jhd->hij", qh[s * S:(s + 1) * S], kh[s * S:(s + 1) * S]) / np.sqrt(48.0)
    assert np.abs(lse[s] - np.log2(np.exp(lg).sum(-1))).max() < 1e-4
    # without lengths every key counts
    g.lens = None
    lib.at_fa_fwd(dqh.ptr, do.ptr, dl.ptr, C.byref(g), H, Cc); LP.check()
    assert rel(do.to_numpy(np.float32, (T, Cc)), ro.attend(qh, kh, vh, nseq, S, None)) < 2e-3


@pytest.mark.parametrize("nseq,S,lens", [(3, 150, (150, 97, 64)), (5, 17, (17, 3, 0, 9, 16)), (1, 32, (32,)), (7, 33, (33, 1, 32, 20, 0, 33, 7))])
def test_core_on_other_sequence_lengths(gpu, nseq, S, lens):
    """sequences longer than a wavefront's 64 queries, an odd number of half-wavefront units (the last wavefront's second half idles), the widths at
    which the kernel changes from two units per wavefront to one"""
    rng = np.random.default_rng(6 + S)
    Cc, H = 48, 1; T = nseq * S
    qkv = rng.standard_normal((T, 3 * Cc)).astype(np.float32); ones = np.ones(Cc, np.float32)
    lens = np.array(lens, np.int32); dlens = DevBuf.from_numpy(lens)
    g = at_geom(); g.nseq, g.S, g.D, g.Hh, g.W = nseq, S, 1, 1, S
    dqh = pack(qkv, ones, ones, g, 0, Cc, 0)
    got = dqh.to_numpy(np.uint16, (3, H, T + 64, 48)).view(np.float16).astype(np.float64)
    g.lens = dlens.ptr
    do, dl = DevBuf(T * Cc * 4), DevBuf(nseq * H * S * 4)
    lib.at_fa_fwd(dqh.ptr, do.ptr, dl.ptr, C.byref(g), H, Cc); LP.check()
    qh, kh, vh = (got[i, :, :T].transpose(1, 0, 2) for i in range(3))
    assert rel(do.to_numpy(np.float32, (T, Cc)), ro.attend(qh, kh, vh, nseq, S, lens)) < 2e-3


def run_block(P, lay, x, d, g, Tr=0):
    bp = at_bp(); assert lib.at_block_layout(C.byref(d), C.byref(bp), 0) == P.size
    T = x.shape[0]
    ws = at_ws(); wsb = DevBuf(lib.at_ws_bytes_r(C.byref(d), T, Tr)); lib.at_ws_carve_r(C.byref(ws), C.byref(d), T, Tr, wsb.ptr)
    assert (ws.qkvr is not None) == (Tr > 0) and lib.at_ws_bytes_r(C.byref(d), T, 0) == lib.at_ws_bytes(C.byref(d), T)
    dP, dx, dy = DevBuf.from_numpy(P), DevBuf.from_numpy(x), DevBuf.from_numpy(np.full(x.shape, np.nan, np.float32))
    rc = lib.at_block_fwd(C.byref(d), dP.ptr, C.byref(bp), dx.ptr, dy.ptr, C.byref(g), C.byref(ws)); LP.check()
    lib.mi_sync()
    qkv, o = np.empty((T, 3 * d.C), np.float32), np.empty((T, d.C), np.float32)    # the block's own projected rows and its attention output
    lib.mi_d2h(qkv.ctypes.data, ws.qkv, qkv.nbytes); lib.mi_d2h(o.ctypes.data, ws.o, o.nbytes)
    return rc, dy.to_numpy(np.float32, x.shape), qkv, o


def attention_of(P, lay, qkv, **kw):
    Cc = kw["Cc"]
    """the oracle's attention branch on the device's own qkv rows: what the block's attention output must be, without the MX linears' noise"""
    return ro.attention(qkv.astype(np.float64), P[lay["qg"]:lay["qg"] + Cc].astype(np.float64), P[lay["kg"]:lay["kg"] + Cc].astype(np.float64), **kw)


@pytest.mark.parametrize("rope", [2, 1, 0])
def test_block_with_radial_attention(gpu, rope):
    """samples with the axis inside the grid, outside it and without one (tests/test_attn_ray.c:340-372's cases), one block each way"""
    rng = np.random.default_rng(7 + rope)
    D, Hh, W, Cc, H, F, n = 6, 5, 7, 192, 4, 512, 3; S = D * Hh * W; T = n * S
    axr = make_axr(n, D, Hh, W, (0, 1, 2), (0, 1, 2))
    t = DevRays(n, D, Hh, W, 2.0, axr)
    P, lay = make_block(rng, Cc, F)
    x = rng.standard_normal((T, Cc)).astype(np.float32)
    d = at_dims(); d.C, d.H, d.F, d.rope, d.nreg, d.rope_base = Cc, H, F, rope, 0, 100.0
    g = at_geom(); g.nseq, g.S, g.D, g.Hh, g.W = n, S, D, Hh, W; g.rays = C.addressof(t.R)
    rc, y, qkv, o = run_block(P, lay, x, d, g, t.Tr)
    assert rc == 0 and np.isfinite(y).all()
    # gather, QK-norm, RoPE on the ray positions, length-masked attention per ray (fp16 q / k / v), normalised scatter: the reference's gate for
    # the fp16 core is 6e-3 of the tensor's rms (tests/test_attn_ray.c:13)
    assert rel(o, attention_of(P, lay, qkv, nseq=n, S=S, H=H, Cc=Cc, rope_mode=rope, rays=t.o)) < 6e-3
    want = ro.block(P, lay, x, n, S, H, Cc, F, rope_mode=rope, rays=t.o)
    # the linears are MX-fp8 GEMMs: the reference's gate for them against the exact block is 0.1 (tests/test_attn.c)
    assert np.linalg.norm(y - want) / np.linalg.norm(want) < 0.05
    # and the radial attention is what ran: full attention over the grid is further away
    full = ro.block(P, lay, x, n, S, H, Cc, F, rope_mode=0)
    assert np.linalg.norm(y - full) > 2 * np.linalg.norm(y - want)
    d.nreg = 1                                                                     # rays take no register tokens
    assert run_block(P, lay, x, d, g, t.Tr)[0] == -1


def test_block_with_scroll_rope_over_the_grid(gpu):
    rng = np.random.default_rng(11)
    D, Hh, W, Cc, H, F, n, nreg = 5, 6, 4, 192, 4, 512, 3, 2; S = nreg + D * Hh * W; T = n * S
    axr = make_axr(n, D, Hh, W, (1, 0, 2), (0, 1, 2))
    t = DevRays(n, D, Hh, W, 2.0, axr)
    dp = DevBuf(T * 12)
    lib.at_scroll_pos(n, nreg, D, Hh, W, t.bufs["ad"].ptr, t.bufs["cen"].ptr, dp.ptr); LP.check()
    pos = dp.to_numpy(np.float32, (T, 3)).astype(np.float64)                       # (the device's own coordinates: their parity is the test above)
    P, lay = make_block(rng, Cc, F)
    x = rng.standard_normal((T, Cc)).astype(np.float32)
    d = at_dims(); d.C, d.H, d.F, d.rope, d.nreg, d.rope_base = Cc, H, F, 2, nreg, 100.0
    g = at_geom(); g.nseq, g.S, g.D, g.Hh, g.W = n, S, D, Hh, W; g.pos = dp.ptr
    rc, y, qkv, o = run_block(P, lay, x, d, g)
    assert rc == 0
    # the MX-fp8 core with rotations by the scroll coordinates: the core's own gate (tests/test_gpu_gemm_attn.py) on the block's attention output
    wo = attention_of(P, lay, qkv, nseq=n, S=S, H=H, Cc=Cc, rope_mode=2, pos=pos, nreg=nreg)
    assert np.linalg.norm(o - wo) / np.linalg.norm(wo) < 0.05
    want = ro.block(P, lay, x, n, S, H, Cc, F, rope_mode=2, pos=pos, nreg=nreg)
    assert np.linalg.norm(y - want) / np.linalg.norm(want) < 0.05
    grid = ro.block(P, lay, x, n, S, H, Cc, F, rope_mode=1, grid=(D, Hh, W), nreg=nreg)
    assert np.linalg.norm(y - grid) > 2 * np.linalg.norm(y - want)                 # not the grid-index rotation
    g.pos = None                                                                   # scroll RoPE without coordinates is refused
    assert run_block(P, lay, x, d, g)[0] == -1


def window_axis_records(N, D, kinds):
    """unet_set_attn_axis records (window voxels, the axis along window z) and the same axes at the bottleneck of a two-level net (F = 2 window planes
    per grid plane; a voxel centre c of the window is (c + 0.5) / F - 0.5 on the grid): kind 0 inside the window, 1 outside, 2 none"""
    np_ = D; rec = np.zeros((N, 4 + 2 * np_), np.float32); F = 2; Dg = D // F; axr = np.zeros((N, ro.axr_len(Dg)), np.float32)
    for b in range(N):
        rec[b, :4] = (0, kinds[b] != 2, np_, 1)
        for z in range(np_):
            rec[b, 4 + 2 * z], rec[b, 5 + 2 * z] = (0.41 * D + 0.11 * z, 0.57 * D - 0.07 * z) if kinds[b] == 0 else (-3.2 - 0.05 * z, 1.3 * D + 0.04 * z)
        axr[b, :2] = (0, kinds[b] != 2)
        c = rec[b, 4:].astype(np.float64).reshape(Dg, F, 2).mean(1)
        axr[b, 2:] = ((c + 0.5) / F - 0.5).reshape(-1)
    return rec, axr


@pytest.mark.parametrize("radial", [1, 0])
def test_unet_attention_stage_on_the_scroll_geometry(gpu, tmp_path, radial):
    """cfg.attn_axis 1 (radial attention) and cfg.attn_pe 3 (scroll RoPE) in the graph: the axis records of unet_set_attn_axis reach the stage at the
    bottleneck's resolution, the stage's output follows the double-precision blocks on that geometry, no records = rays along the grid rows /
    grid-index coordinates, and the checkpoint header carries the two fields (src/unet.h:77-83, src/unet.c:2732-2782, :5570)."""
    import orc
    import unet_ref
    from gpuutil import to_mx
    from ufsm_amd.unet import UNet, make_cfg, load_host
    rng = np.random.default_rng(50 + radial)
    N, D = 2, 16; widths = [32, 96]; cin, head_out, nblk = 4, 2, 2; nreg = 0 if radial else 2
    S = D ** 3; Cb = widths[-1]; Hh = Cb // 48; F = (8 * Cb // 3 + 31) // 32 * 32; Dg = D // 2; Sg = Dg ** 3
    x = rng.standard_normal((N, cin, S)).astype(np.float32); dxq = to_mx(8, x)
    kw = dict(head_out=head_out, attn_blocks=nblk, attn_reg=nreg)
    net = UNet(make_cfg(cin, widths, attn_pe=3, attn_axis=radial, **kw), N, D, D, D, seed=7)
    plain = UNet(make_cfg(cin, widths, attn_pe=2, **kw), N, D, D, D, seed=7)
    pp = net.params()
    assert pp.size == plain.params().size                                          # neither field has parameters of its own
    n_conv = unet_ref.param_layout(cin, widths, head_out)[1]
    lays = []; o = n_conv + nreg * Cb
    for _ in range(nblk):
        bl, o = orc.block_layout(Cb, F, o); lays.append(bl)
    assert o == pp.size
    for lay in lays:
        for k, n in (("wo", Cb * Cb), ("w2", Cb * F), ("bo", Cb), ("b1", 2 * F), ("bqkv", 3 * Cb)):
            pp[lay[k]:lay[k] + n] = 0.05 * rng.standard_normal(n)
    net.set_params(pp)
    H0 = load_host()

    def run(rec):
        if rec is None:
            H0.unet_set_attn_axis(net.h, None, 0, 0)
        else:
            H0.unet_set_attn_axis(net.h, rec.ctypes.data, rec.shape[0], rec.shape[1])
        d = DevBuf(N * head_out * S * 4)
        assert net.forward_x(dxq.ptr, d.ptr) == 0
        LP.check()
        outs = {name: (ptr, shp) for name, ptr, shp in net.layer_outs()}

        def fetch(name):
            ptr, shp = outs[name]; nb = lib.lp_mx8_bytes(shp[0], shp[1], Sg)
            buf = np.empty(nb, np.uint8); lib.mi_d2h(buf.ctypes.data, ptr, nb)
            return orc.mx_to_f32(8, buf, N, Cb, Sg)
        return d.to_numpy(np.float32, (N, head_out, S)), fetch("enc1.c2"), fetch("attn")

    def stage(xb, axr):
        tok = np.zeros((N, Sg + nreg, Cb), np.float32)
        reg = np.ascontiguousarray(pp[n_conv:n_conv + nreg * Cb].reshape(nreg, Cb)) if nreg else np.zeros((1, Cb), np.float32)
        orc.lib().orc_cs_to_tok(orc.ptr(xb), orc.ptr(tok), orc.ptr(reg), N, Cb, Sg, nreg)
        t = tok.reshape(N * (Sg + nreg), Cb).astype(np.float64)
        R = ro.make_rays(N, Dg, Dg, Dg, 2.0, axr)
        geo = dict(rays=R) if radial else dict(pos=ro.scroll_pos(N, nreg, Dg, Dg, Dg, R["ad"], R["cen"]), nreg=nreg)
        for lay in lays:
            t = ro.block(pp, lay, t, N, Sg + nreg, Hh, Cb, F, rope_mode=2, **geo)
        t = np.ascontiguousarray(t, np.float32); want = np.zeros_like(xb)
        orc.lib().orc_tok_to_cs(orc.ptr(t), orc.ptr(want), N, Cb, Sg, nreg)
        return orc.mx_to_f32(8, orc.f32_to_mx(8, want, N, Cb, Sg), N, Cb, Sg)      # (the stage's output is stored as MX-fp8)

    rec, axr = window_axis_records(N, D, (0, 1))
    _, axr_none = window_axis_records(N, D, (2, 2))
    lg, xb, got = run(rec)
    want, other = stage(xb, axr), stage(xb, axr_none)
    # two blocks of MX-fp8 linears against exact ones, then the MX-fp8 storage of the result; the reference's gate for an MX block is 0.1
    # (measured 0.065: e4m3 storage of both results alone is 0.05; the other geometry is 7 x further away)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 0.1
    far = 3 if radial else 1.2                                                     # (rotations by other coordinates change the stage less than other rays do: 1.36 x measured)
    assert np.linalg.norm(got - other) > far * np.linalg.norm(got - want)          # the axis is what the stage used
    lg0, xb0, got0 = run(None)                                                      # no records: the grid rows / the grid indices
    assert np.array_equal(xb0, xb) and not np.array_equal(got0, got)
    assert np.linalg.norm(got0 - other) / np.linalg.norm(other) < 0.1 and np.linalg.norm(got0 - want) > far * np.linalg.norm(got0 - other)
    bad = rec.copy(); bad[:, 2] = D // 2                                            # records of another plane count do not describe this grid: no axis
    assert np.array_equal(run(bad[:, :4 + D])[2], got0)
    assert np.array_equal(run(rec)[0], lg)                                          # and the records again: the first result, bit for bit
    q, nr, cov = C.c_int(), C.c_int(), C.c_double()
    if radial:
        assert H0.unet_attn_rays(net.h, C.byref(q), C.byref(nr), C.byref(cov)) == 0
        assert (q.value, nr.value) == ro.rays_dims(Dg, Dg, Dg, 2.0)[::2] and 0.8 < cov.value <= 1
    else:
        assert H0.unet_attn_rays(net.h, C.byref(q), C.byref(nr), C.byref(cov)) == -1
    path = str(tmp_path / "scroll.ckpt")
    assert net.save(path, step=4, extra="{}") == 0
    head = open(path, "rb").readline()
    assert b'"attn_pe":3,' in head and (b',"attn_axis":1' in head) == bool(radial)
    c2 = type(net.cfg)(); st = C.c_int()
    assert H0.unet_peek(path.encode(), C.byref(c2), C.byref(st)) == 0 and (c2.attn_pe, c2.attn_axis, st.value) == (3, radial, 4)
    twin = UNet(make_cfg(cin, widths, attn_pe=3, attn_axis=radial, **kw), N, D, D, D, seed=1)
    assert twin.load(path) == 4
    H0.unet_set_attn_axis(twin.h, rec.ctypes.data, N, rec.shape[1])
    d = DevBuf(N * head_out * S * 4)
    assert twin.forward_x(dxq.ptr, d.ptr) == 0
    assert np.array_equal(d.to_numpy(np.float32, (N, head_out, S)), lg)
    assert plain.load(path) == -1                                                   # another positional encoding: another function
    net.close(); plain.close(); twin.close()


@pytest.mark.parametrize("radial", [1, 0])
def test_predict_volume_hands_every_window_its_axis(gpu, radial):
    """The sliding-window driver gives a net whose attention stage reads the scroll axis each window's record (pred_axis, src/predict.c:1128-1141):
    windows run alone on a one-window graph with the record written by hand give the bytes of their region; a prediction does not depend on the
    windows per forward (the ray sums are order-independent); and with another axis the prediction is another."""
    from ufsm_amd.unet import UNet, make_cfg, load_host
    rng = np.random.default_rng(9)
    W, halo = 32, 8; S = W - 2 * halo
    dims = (40, 32, 24)
    z, y, x = np.meshgrid(np.arange(dims[0]), np.arange(dims[1]), np.arange(dims[2]), indexing="ij")
    vol = np.clip(70 + 0.6 * z + 0.7 * y + 35 * np.sin(0.25 * x + 0.3 * y) * np.cos(0.2 * z) + rng.integers(0, 16, dims), 0, 255).astype(np.uint8)
    dv = DevBuf.from_numpy(vol)
    import orc
    import unet_ref
    nreg = 0 if radial else 2
    kw = dict(G=8, head_out=1, act_dt=8, attn_blocks=2, attn_pe=3, attn_axis=radial, attn_reg=nreg)
    args = (100.0, 1 / 50.0, 1, 11.5, 20.25)                                     # mean, 1 / sd, axis on, the axis at (y, x) = (11.5, 20.25): inside some windows, outside others
    outs = {}
    for nb in (1, 5):
        net = UNet(make_cfg(4, [16, 96], **kw), nb, W, W, W, seed=5)
        q = net.params(); r2 = np.random.default_rng(1)
        o = unet_ref.param_layout(4, [16, 96], 1)[1] + nreg * 96                  # (the zero-initialised out projections made trained-like: the stage acts)
        for _ in range(2):
            lay, o = orc.block_layout(96, 256, o)
            for k, n in (("wo", 96 * 96), ("w2", 96 * 256), ("bo", 96), ("b1", 512), ("bqkv", 288)):
                q[lay[k]:lay[k] + n] = 0.05 * r2.standard_normal(n)
        assert o == q.size
        net.set_params(q)
        dout = DevBuf(vol.size)
        rc, nw, ndone = net.predict_volume(dv.ptr, dims, halo, 0, *args, dout.ptr)
        assert rc == 0 and nw == 12 and ndone == 12
        outs[nb] = dout.to_numpy(np.uint8, dims)
        if nb == 5:
            rc, _, _ = net.predict_volume(dv.ptr, dims, halo, 0, args[0], args[1], 1, 300.0, -200.0, dout.ptr)
            assert rc == 0
            outs["far"] = dout.to_numpy(np.uint8, dims)
        net.close()
    assert outs[1].std() > 0 and np.array_equal(outs[1], outs[5])
    assert not np.array_equal(outs[5], outs["far"])
    one = UNet(make_cfg(4, [16, 96], **kw), 1, W, W, W, seed=2); one.set_params(q)
    H0 = load_host()
    dlg = DevBuf(W ** 3 * 4); dw = DevBuf(W ** 3); dE = DevBuf(S ** 3)
    for a, b, c in ((0, 0, 0), (1, 1, 1), (2, 0, 1)):
        o = (a * S - halo, b * S - halo, c * S - halo)
        lib.mi_ct_window(dv.ptr, dims[0], dims[1], dims[2], o[0], o[1], o[2], W, dw.ptr, 1, halo, None)
        off = DevBuf.from_numpy(np.concatenate([np.full(W, o[1] - args[3], np.float32), np.full(W, o[2] - args[4], np.float32)]))
        rec = np.zeros(4 + 2 * W, np.float32); rec[:4] = (0, 1, W, 1); rec[4::2] = args[3] - o[1]; rec[5::2] = args[4] - o[2]
        H0.unet_set_attn_axis(one.h, rec.ctypes.data, 1, rec.size)
        assert one.forward_ct(dw.ptr, args[0], args[1], off.ptr, off.ptr + 4 * W, args[2], dlg.ptr) == 0
        lib.mi_zero(dE.ptr, S ** 3)
        lib.nn_pred_place(dlg.ptr, dw.ptr, W, halo, -halo, -halo, -halo, S, S, S, S, dE.ptr)
        LP.check()
        E = dE.to_numpy(np.uint8, (S, S, S))
        reg = outs[1][a * S:(a + 1) * S, b * S:(b + 1) * S, c * S:(c + 1) * S]
        assert np.array_equal(E[:reg.shape[0], :reg.shape[1], :reg.shape[2]], reg), (a, b, c)
    one.close()
