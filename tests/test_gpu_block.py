"""GPU parity of the attention block's pieces and of the block forward, through the C ABI, against the oracle; and the reference's gate
against the exact fp64 block (tests/test_attn.c:398-424)."""
import ctypes as C

import numpy as np
import pytest

import orc
from gpuutil import DevBuf, LP, lib
from ufsm_amd import at_geom, at_dims, at_bp, at_ws
from test_oracle_block import exact_block, make_block

pytestmark = pytest.mark.gpu


def test_layernorm_glu_token_layout(gpu):
    rng = np.random.default_rng(0)
    T, Cc, F = 300, 192, 512
    x = (2 * rng.standard_normal((T, Cc)) + 1).astype(np.float32); g = rng.uniform(0.5, 1.5, Cc).astype(np.float32); b = rng.standard_normal(Cc).astype(np.float32)
    dx, dg, db = DevBuf.from_numpy(x), DevBuf.from_numpy(g), DevBuf.from_numpy(b); dy, dm, dr = DevBuf(x.nbytes), DevBuf(T * 4), DevBuf(T * 4)
    lib.at_ln_fwd(dx.ptr, dg.ptr, db.ptr, dy.ptr, dm.ptr, dr.ptr, T, Cc)
    LP.check()
    y = np.zeros_like(x); m = np.zeros(T, np.float32); r = np.zeros(T, np.float32)
    orc.lib().orc_ln_fwd(orc.ptr(x), orc.ptr(g), orc.ptr(b), orc.ptr(y), orc.ptr(m), orc.ptr(r), T, Cc)
    assert np.abs(dy.to_numpy(np.float32, (T, Cc)) - y).max() < 1e-5 * np.abs(y).max()
    assert np.abs(dm.to_numpy(np.float32) - m).max() < 1e-6 and np.abs(dr.to_numpy(np.float32) - r).max() < 1e-5 * r.max()
    h = rng.standard_normal((T, 2 * F)).astype(np.float32)
    dh, dgg = DevBuf.from_numpy(h), DevBuf(T * F * 4)
    lib.at_glu_fwd(dh.ptr, dgg.ptr, T, F)
    gg = np.zeros((T, F), np.float32); orc.lib().orc_glu_fwd(orc.ptr(h), orc.ptr(gg), T, F)
    assert np.abs(dgg.to_numpy(np.float32, (T, F)) - gg).max() < 2e-6 * max(1.0, np.abs(gg).max())      # (hardware exp2 and reciprocal: a few ulp of the largest values)
    n, Sg, nreg = 2, 125, 4
    xc = rng.standard_normal((n, Cc, Sg)).astype(np.float32); reg = rng.standard_normal((nreg, Cc)).astype(np.float32)
    dxc, dreg, dtok, dback = DevBuf.from_numpy(xc), DevBuf.from_numpy(reg), DevBuf(n * (Sg + nreg) * Cc * 4), DevBuf(xc.nbytes)
    lib.at_cs_to_tok(dxc.ptr, dtok.ptr, dreg.ptr, n, Cc, Sg, nreg)
    lib.at_tok_to_cs(dtok.ptr, dback.ptr, n, Cc, Sg, nreg)
    LP.check()
    tok = np.zeros((n, Sg + nreg, Cc), np.float32); orc.lib().orc_cs_to_tok(orc.ptr(xc), orc.ptr(tok), orc.ptr(reg), n, Cc, Sg, nreg)
    assert np.array_equal(dtok.to_numpy(np.float32, tok.shape), tok) and np.array_equal(dback.to_numpy(np.float32, xc.shape), xc)


@pytest.mark.parametrize("rope", [0, 1])
def test_pack_matches_oracle(gpu, rope):
    rng = np.random.default_rng(3 + rope)
    nseq, D, nreg, Cc = 2, 5, 3, 144; H = Cc // 48; S = nreg + D ** 3; T = nseq * S
    qkv = rng.standard_normal((T, 3 * Cc)).astype(np.float32); qg = (1 + 0.2 * rng.standard_normal(Cc)).astype(np.float32); kg = (1 + 0.2 * rng.standard_normal(Cc)).astype(np.float32)
    dq, dqg, dkg = DevBuf.from_numpy(qkv), DevBuf.from_numpy(qg), DevBuf.from_numpy(kg)
    dqh = DevBuf.from_numpy(np.full(3 * H * (T + 64) * 48, 0x7e00, np.uint16)); drq, drk, damx = DevBuf(T * H * 4), DevBuf(T * H * 4), DevBuf.from_numpy(np.full(4, 9.0, np.float32))
    g = at_geom(); g.nseq, g.S, g.D, g.Hh, g.W = nseq, S, D, D, D
    lib.at_fa_pack(dq.ptr, dqg.ptr, dkg.ptr, dqh.ptr, drq.ptr, drk.ptr, damx.ptr, C.byref(g), nreg, Cc, rope, 100.0)
    LP.check()
    wqh, wrq, wrk, wamx = orc.fa_pack(qkv, qg, kg, nseq, S, D, D, nreg, Cc, rope, 100.0)
    got = dqh.to_numpy(np.uint16, wqh.shape).view(np.float16).astype(np.float32); want = wqh.view(np.float16).astype(np.float32)
    # fp16 results of the same fp32 arithmetic; the rotary sin / cos of the device and the host differ in their last bits: one fp16 step at most
    assert np.abs(got - want).max() <= 2.0 ** -10 * np.abs(want).max() and (got != want).mean() < (0.02 if rope else 1e-3)
    assert np.abs(drq.to_numpy(np.float32, wrq.shape) - wrq).max() < 1e-5 * wrq.max() and np.abs(drk.to_numpy(np.float32, wrk.shape) - wrk).max() < 1e-5 * wrk.max()
    assert np.array_equal(damx.to_numpy(np.float32), wamx)


def run_block(bits, Cc, H, F, rope, nreg, P, lay, x, nseq, S, D):
    d = at_dims(); d.C, d.H, d.F, d.rope, d.nreg, d.rope_base = Cc, H, F, rope, nreg, 100.0
    bp = at_bp(); assert lib.at_block_layout(C.byref(d), C.byref(bp), 0) == P.size == lib.at_block_nparams(C.byref(d))
    for k, off in lay.items():
        assert getattr(bp, k) == off, k                                   # the reference's parameter order (src/nn_attn.cu:460-480)
    T = nseq * S
    ws = at_ws(); wsb = DevBuf(lib.at_ws_bytes(C.byref(d), T)); lib.at_ws_carve(C.byref(ws), C.byref(d), T, wsb.ptr)
    dP, dx, dy = DevBuf.from_numpy(P), DevBuf.from_numpy(x), DevBuf(x.nbytes)
    g = at_geom(); g.nseq, g.S, g.D, g.Hh, g.W = nseq, S, D, D, D
    lib.at_set_mx(bits); assert lib.at_get_mx() == bits
    rc = lib.at_block_fwd(C.byref(d), dP.ptr, C.byref(bp), dx.ptr, dy.ptr, C.byref(g), C.byref(ws))
    lib.at_set_mx(8)
    LP.check()
    return rc, dy.to_numpy(np.float32, x.shape)


@pytest.mark.parametrize("bits,rope,nreg,tol", [(8, 0, 0, 0.1), (8, 1, 4, 0.1), (4, 0, 0, 0.35)])
def test_block_forward(gpu, bits, rope, nreg, tol):
    rng = np.random.default_rng(bits + rope)
    Cc, H, F, nseq, D = 192, 4, 512, 2, 6; S = nreg + D ** 3
    P, lay = make_block(rng, Cc, F)
    x = rng.standard_normal((nseq * S, Cc)).astype(np.float32)
    rc, y = run_block(bits, Cc, H, F, rope, nreg, P, lay, x, nseq, S, D)
    assert rc == 0
    want = orc.block_fwd(bits, Cc, H, F, rope, nreg, 100.0, P, x, nseq, S, D, D)
    # the same arithmetic step by step; every MX re-quantisation (four GEMM operands, q / k / v, P) turns last-bit differences into
    # occasional code flips, so the two agree far inside the format's own noise but not bit for bit
    rel = np.linalg.norm(y - want) / np.linalg.norm(want - x)
    assert rel < (0.02 if bits == 8 else 0.08), rel
    if not rope:                                                                 # the reference's gate against the exact fp64 block
        ye = exact_block(P, lay, x, nseq, S, H, Cc, F)
        assert np.linalg.norm(y - ye) / np.linalg.norm(ye) < tol


def test_block_with_packed_operands_from_the_producers_has_the_same_bits(gpu):
    """The LayerNorms and the SwiGLU write the GEMMs' packed MX-fp8 operands themselves (default) or fp32 rows that the GEMMs pack: the same
    values quantised the same way, so the block's output is equal bit for bit (C 192 = three 64-channel groups per row, a token count that is not
    a multiple of the four rows of a workgroup)."""
    rng = np.random.default_rng(11)
    Cc, H, F, nseq, D, nreg = 192, 4, 512, 3, 5, 2; S = nreg + D ** 3
    P, lay = make_block(rng, Cc, F)
    x = (rng.standard_normal((nseq * S, Cc)) * np.exp(rng.uniform(-2, 2, (nseq * S, 1)))).astype(np.float32)
    ys = []
    try:
        for mode in (0, 1, 2):                                   # 2: the up projection also forms the SwiGLU and packs it for the down projection
            lib.at_fuse_pack(mode)
            rc, y = run_block(8, Cc, H, F, 1, nreg, P, lay, x, nseq, S, D)
            assert rc == 0 and np.isfinite(y).all()
            ys.append(y)
    finally:
        lib.at_fuse_pack(2)
    assert np.array_equal(ys[0], ys[1]) and np.array_equal(ys[0], ys[2])


@pytest.mark.parametrize("nseq,dims,nreg,Cc", [(2, (3, 4, 5), 2, 96), (1, (8, 8, 8), 0, 192), (3, (1, 1, 7), 4, 48), (1, (2, 2, 2), 1, 4)])
def test_peg_matches_oracle_bit_for_bit(gpu, nseq, dims, nreg, Cc):
    """at_peg_fwd (src/attn.h:141-144): x + b + depthwise 3^3 conv on the grid tokens, the taps in (dz, dy, dx) order as fused multiply-adds:
    the same bits as the oracle's loop; register rows are copies."""
    rng = np.random.default_rng(Cc + nreg)
    D, Hh, W = dims; S = nreg + D * Hh * W
    x = rng.standard_normal((nseq * S, Cc)).astype(np.float32); w = (0.3 * rng.standard_normal((Cc, 27))).astype(np.float32); b = rng.standard_normal(Cc).astype(np.float32)
    dx, dy, dw, db = DevBuf.from_numpy(x), DevBuf(x.nbytes), DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    g = at_geom(); g.nseq, g.S, g.D, g.Hh, g.W = nseq, S, D, Hh, W
    lib.at_peg_fwd(dx.ptr, dy.ptr, dw.ptr, db.ptr, C.byref(g), nreg, Cc); LP.check()
    y = dy.to_numpy(np.float32, x.shape)
    assert np.array_equal(y, orc.peg_fwd(x, w, b, nseq, S, D, Hh, W, nreg))
    assert np.array_equal(y.reshape(nseq, S, Cc)[:, :nreg], x.reshape(nseq, S, Cc)[:, :nreg]) and np.array_equal(dx.to_numpy(np.float32, x.shape), x)


def test_block_value_residual(gpu):
    """at_ws.vr (src/nn_attn.cu:535-542, :609-610): vr 1 keeps the block's V rows in v1 and changes nothing else; vr 2 mixes them into a
    later block's V by the per-head lerp; lam 0 is the plain block bit for bit."""
    rng = np.random.default_rng(5)
    Cc, H, F, nseq, D, nreg = 192, 4, 512, 2, 4, 3; S = nreg + D ** 3; T = nseq * S
    P1, lay = make_block(rng, Cc, F); P2, _ = make_block(rng, Cc, F)
    x = rng.standard_normal((T, Cc)).astype(np.float32)
    d = at_dims(); d.C, d.H, d.F, d.rope, d.nreg, d.rope_base = Cc, H, F, 1, nreg, 100.0
    bp = at_bp(); lib.at_block_layout(C.byref(d), C.byref(bp), 0)
    ws = at_ws(); wsb = DevBuf(lib.at_ws_bytes(C.byref(d), T)); lib.at_ws_carve(C.byref(ws), C.byref(d), T, wsb.ptr)
    g = at_geom(); g.nseq, g.S, g.D, g.Hh, g.W = nseq, S, D, D, D
    dv1, down = DevBuf(T * Cc * 4), DevBuf(T * Cc * 4)
    dx, dy = DevBuf.from_numpy(x), DevBuf(x.nbytes)
    lib.at_set_mx(8)

    def run(P, vr, lam=None, own=False):
        dP = DevBuf.from_numpy(P); dl = DevBuf.from_numpy(np.asarray(lam if lam is not None else np.zeros(H), np.float32))
        ws.vr = vr; ws.v1 = dv1.ptr; ws.lam = dl.ptr
        ws.own = down.ptr if own else None
        assert lib.at_block_fwd(C.byref(d), dP.ptr, C.byref(bp), dx.ptr, dy.ptr, C.byref(g), C.byref(ws)) == 0
        LP.check()
        return dy.to_numpy(np.float32, x.shape)

    plain1, plain2 = run(P1, 0), run(P2, 0)
    assert np.array_equal(run(P1, 1), plain1)                                    # keeping V changes nothing
    v1 = dv1.to_numpy(np.float32, (T, Cc))
    v1o = np.zeros((T, Cc), np.float32)
    orc.block_fwd(8, Cc, H, F, 1, nreg, 100.0, P1, x, nseq, S, D, D, vr=1, v1=v1o)
    # the value projection's rows: an MX GEMM of LayerNorm outputs both sides, last-bit differences flip an operand code now and then
    assert np.linalg.norm(v1 - v1o) / np.linalg.norm(v1o) < 2e-3 and np.abs(v1o).max() > 0.1
    assert np.array_equal(run(P2, 2, np.zeros(H)), plain2)                       # lam 0
    lam = np.array([0.3, 1.0, 0.0, 0.7], np.float32)
    got = run(P2, 2, lam, own=True)
    want = orc.block_fwd(8, Cc, H, F, 1, nreg, 100.0, P2, x, nseq, S, D, D, vr=2, v1=v1, lam=lam)     # (from the device's v1: the mix alone is compared)
    rel = np.linalg.norm(got - want) / np.linalg.norm(want - x)
    assert rel < 0.02, rel
    assert np.linalg.norm(got - plain2) / np.linalg.norm(plain2 - x) > 0.05
    own = down.to_numpy(np.float32, (T, Cc))                                     # the block's own V rows, kept when a buffer is given
    v2o = np.zeros((T, Cc), np.float32)
    orc.block_fwd(8, Cc, H, F, 1, nreg, 100.0, P2, x, nseq, S, D, D, vr=1, v1=v2o)
    assert np.linalg.norm(own - v2o) / np.linalg.norm(v2o) < 2e-3
    assert np.array_equal(run(P2, 2, lam), got)                                  # without the buffer: the same output
    ws.vr = 0


def test_block_refuses_what_it_does_not_run(gpu):
    d = at_dims(); d.C, d.H, d.F = 96, 2, 128
    bp = at_bp(); lib.at_block_layout(C.byref(d), C.byref(bp), 0)
    ws = at_ws(); g = at_geom(); g.nseq, g.S = 1, 8
    d.rope = 2                                                                   # scroll-coordinate RoPE needs per-token positions
    assert lib.at_block_fwd(C.byref(d), None, C.byref(bp), None, None, C.byref(g), C.byref(ws)) == -1
    d.rope = 0; ws.vr = 1                                                        # value residual without its buffer
    assert lib.at_block_fwd(C.byref(d), None, C.byref(bp), None, None, C.byref(g), C.byref(ws)) == -1
