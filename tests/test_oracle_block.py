"""Pins of the oracle's attention-block pieces (CPU only): textbook formulas in numpy fp64, and the reference's gate for the whole block
(tests/test_attn.c:398-424: MX linears and the MX-fp8 core against the exact block, relative L2)."""
import numpy as np
import pytest

import orc


def ln64(x, g, b, eps=1e-5):
    m = x.mean(-1, keepdims=True); v = ((x - m) ** 2).mean(-1, keepdims=True)
    return (x - m) / np.sqrt(v + eps) * g + b


def test_layernorm_glu_and_token_layout():
    rng = np.random.default_rng(0)
    T, Cc, F = 37, 96, 40
    x = (2 * rng.standard_normal((T, Cc)) + 1).astype(np.float32); g = rng.uniform(0.5, 1.5, Cc).astype(np.float32); b = rng.standard_normal(Cc).astype(np.float32)
    y = np.zeros_like(x); m = np.zeros(T, np.float32); r = np.zeros(T, np.float32)
    orc.lib().orc_ln_fwd(orc.ptr(x), orc.ptr(g), orc.ptr(b), orc.ptr(y), orc.ptr(m), orc.ptr(r), T, Cc)
    x64 = x.astype(np.float64)
    assert np.abs(y - ln64(x64, g, b)).max() < 1e-5 and np.abs(m - x64.mean(1)).max() < 1e-6
    assert np.abs(r - 1 / np.sqrt(x64.var(1) + 1e-5)).max() < 1e-5
    h = rng.standard_normal((T, 2 * F)).astype(np.float32); gg = np.zeros((T, F), np.float32)
    orc.lib().orc_glu_fwd(orc.ptr(h), orc.ptr(gg), T, F)
    a, bb = h[:, :F].astype(np.float64), h[:, F:].astype(np.float64)
    assert np.abs(gg - a / (1 + np.exp(-a)) * bb).max() < 1e-6
    n, Sg, nreg = 2, 27, 3
    xc = rng.standard_normal((n, Cc, Sg)).astype(np.float32); reg = rng.standard_normal((nreg, Cc)).astype(np.float32)
    tok = np.zeros((n, Sg + nreg, Cc), np.float32)
    orc.lib().orc_cs_to_tok(orc.ptr(xc), orc.ptr(tok), orc.ptr(reg), n, Cc, Sg, nreg)
    assert np.array_equal(tok[:, :nreg], np.broadcast_to(reg, (n, nreg, Cc))) and np.array_equal(tok[:, nreg:], xc.transpose(0, 2, 1))
    back = np.zeros_like(xc)
    orc.lib().orc_tok_to_cs(orc.ptr(tok), orc.ptr(back), n, Cc, Sg, nreg)
    assert np.array_equal(back, xc)                                   # registers dropped, the grid tokens back in place


@pytest.mark.parametrize("rope", [0, 1])
def test_pack_is_rms_norm_gains_rotary_and_fp16(rope):
    rng = np.random.default_rng(1 + rope)
    nseq, D, nreg, Cc = 2, 3, 2, 96; H = Cc // 48; S = nreg + D ** 3; T = nseq * S
    qkv = rng.standard_normal((T, 3, H, 48)); qg = 1 + 0.2 * rng.standard_normal((H, 48)); kg = 1 + 0.2 * rng.standard_normal((H, 48))
    qh, rq, rk, amx = orc.fa_pack(qkv.reshape(T, 3 * Cc), qg, kg, nseq, S, D, D, nreg, Cc, rope, 100.0)
    x = qkv.astype(np.float32).astype(np.float64)
    want = np.zeros((3, H, T, 48))
    for p, gains in ((0, qg), (1, kg)):
        r = 1 / np.sqrt((x[:, p] ** 2).mean(-1, keepdims=True) + 1e-6)
        v = x[:, p] * r * gains.astype(np.float32)[None]
        assert np.abs((rq if p == 0 else rk) - r[..., 0]).max() < 1e-5
        if rope:
            ts = np.arange(T) % S - nreg
            pos = np.stack([ts // (D * D), (ts // D) % D, ts % D], -1).astype(np.float64)           # z, y, x of the grid token
            for ax in range(3):
                ang = pos[:, ax, None] * 100.0 ** (-np.arange(8) / 8.0)[None]                      # [T][8]
                z = (v[..., 16 * ax:16 * ax + 16:2] + 1j * v[..., 16 * ax + 1:16 * ax + 16:2]) * np.exp(1j * ang)[:, None, :]
                rot = np.stack([z.real, z.imag], -1).reshape(T, H, 16)
                v[..., 16 * ax:16 * ax + 16] = np.where((ts >= 0)[:, None, None], rot, v[..., 16 * ax:16 * ax + 16])
        want[p] = v.transpose(1, 0, 2)
    want[2] = x[:, 2].transpose(1, 0, 2)
    got = qh.view(np.float16).astype(np.float64)
    assert (got[:, :, T:] == 0).all()                                  # the 64 padding rows
    err = np.abs(got[:, :, :T] - want)
    assert (err <= np.abs(want) * 2.0 ** -10 + 1e-6).all()             # fp16 rounding of the fp32 result (half an ulp of 11 bits, plus fp32 noise)
    assert abs(amx[1] - np.abs(x[:, 2]).max()) < 1e-6 and amx[0] == 0
    if rope:                                                           # rotations preserve the norm of every pair; registers are not rotated
        assert np.abs((got[0, :, :T] ** 2).sum(-1) - (want[0] ** 2).sum(-1)).max() < 0.05


def exact_block(P, lay, x, nseq, S, H, Cc, F, v1=None, lam=None):
    """v1 / lam: the value residual from its definition, V <- v + lam[head] (v1 - v)"""
    P = P.astype(np.float64); x = x.astype(np.float64)
    g = lambda k, n: P[lay[k]:lay[k] + n]
    xn = ln64(x, g("ln1g", Cc), g("ln1b", Cc))
    qkv = xn @ g("wqkv", 3 * Cc * Cc).reshape(3 * Cc, Cc).T + g("bqkv", 3 * Cc)
    T = nseq * S
    q, k, v = (qkv[:, i * Cc:(i + 1) * Cc].reshape(T, H, 48) for i in range(3))
    q = q / np.sqrt((q ** 2).mean(-1, keepdims=True) + 1e-6) * g("qg", Cc).reshape(H, 48)
    k = k / np.sqrt((k ** 2).mean(-1, keepdims=True) + 1e-6) * g("kg", Cc).reshape(H, 48)
    if v1 is not None:
        v = v + np.asarray(lam, np.float64)[None, :, None] * (v1.astype(np.float64).reshape(T, H, 48) - v)
    o = np.zeros((T, Cc))
    for s in range(nseq):
        sl = slice(s * S, (s + 1) * S)
        for h in range(H):
            lg = q[sl, h] @ k[sl, h].T / np.sqrt(48.0); e = np.exp(lg - lg.max(1, keepdims=True))
            o[sl, h * 48:(h + 1) * 48] = (e / e.sum(1, keepdims=True)) @ v[sl, h]
    x1 = o @ g("wo", Cc * Cc).reshape(Cc, Cc).T + g("bo", Cc) + x
    xn2 = ln64(x1, g("ln2g", Cc), g("ln2b", Cc))
    hh = xn2 @ g("w1", 2 * F * Cc).reshape(2 * F, Cc).T + g("b1", 2 * F)
    gg = hh[:, :F] / (1 + np.exp(-hh[:, :F])) * hh[:, F:]
    return gg @ g("w2", Cc * F).reshape(Cc, F).T + g("b2", Cc) + x1


def make_block(rng, Cc, F):
    lay, n = orc.block_layout(Cc, F)
    P = (0.05 * rng.standard_normal(n)).astype(np.float32)                   # as tests/test_attn.c:407-408
    for k in ("ln1g", "ln2g", "qg", "kg"):
        P[lay[k]:lay[k] + Cc] = 1
    return P, lay


@pytest.mark.parametrize("bits,tol", [(8, 0.1), (4, 0.35)])
def test_block_within_reference_gate_of_exact_block(bits, tol):
    rng = np.random.default_rng(bits)
    Cc, H, F, nseq, D = 96, 2, 128, 2, 4; S = D ** 3
    P, lay = make_block(rng, Cc, F)
    assert orc.block_layout(Cc, F)[1] == 2 * Cc + 3 * Cc * Cc + 3 * Cc + 2 * Cc + Cc * Cc + Cc + 2 * Cc + 2 * F * Cc + 2 * F + Cc * F + Cc      # src/nn_attn.cu:460-480
    x = rng.standard_normal((nseq * S, Cc)).astype(np.float32)
    y = orc.block_fwd(bits, Cc, H, F, 0, 0, 100.0, P, x, nseq, S, D, D)
    ye = exact_block(P, lay, x, nseq, S, H, Cc, F)
    rel = np.linalg.norm(y - ye) / np.linalg.norm(ye)
    assert rel < tol, rel
    # the residual stream dominates y; the gate must also hold on what the block adds
    rel_d = np.linalg.norm((y - x) - (ye - x)) / np.linalg.norm(ye - x)
    assert rel_d < 3 * tol, rel_d


def test_value_residual_special_cases_and_exact_block():
    """orc_block_fwd_vr (src/nn_attn.cu:535-542, :609-610): lam 0 is the plain block bit for bit; lam 1 on one head gives that head the V rows of
    another value projection and leaves the other heads alone (so the rows mixed are V's, head by head); a general lam stays within the
    reference's gate of the exact fp64 block with V mixed from the definition."""
    rng = np.random.default_rng(21)
    Cc, H, F, nseq, D, nreg = 96, 2, 128, 2, 4, 2; S = nreg + D ** 3; T = nseq * S
    P, lay = make_block(rng, Cc, F)
    x = rng.standard_normal((T, Cc)).astype(np.float32)
    run = lambda Pm, **kw: orc.block_fwd(8, Cc, H, F, 1, nreg, 100.0, Pm, x, nseq, S, D, D, **kw)
    plain = run(P)
    P2 = P.copy()                                                    # another value projection: the V third of wqkv / bqkv
    P2[lay["wqkv"] + 2 * Cc * Cc:lay["wqkv"] + 3 * Cc * Cc] = 0.05 * rng.standard_normal(Cc * Cc)
    P2[lay["bqkv"] + 2 * Cc:lay["bqkv"] + 3 * Cc] = 0.05 * rng.standard_normal(Cc)
    v1 = np.zeros((T, Cc), np.float32)
    assert np.array_equal(run(P2, vr=1, v1=v1), run(P2)) and np.abs(v1).max() > 0                    # keeping V changes nothing
    v1_0 = v1.copy()
    assert np.array_equal(run(P, vr=2, v1=v1, lam=[0, 0]), plain) and np.array_equal(v1, v1_0)
    for head in range(H):
        lam = np.zeros(H, np.float32); lam[head] = 1
        P3 = P.copy()                                                # the block whose value projection of that head is P2's
        for h_ in (head,):
            r0 = lay["wqkv"] + (2 * Cc + h_ * 48) * Cc
            P3[r0:r0 + 48 * Cc] = P2[r0:r0 + 48 * Cc]
            b0 = lay["bqkv"] + 2 * Cc + h_ * 48
            P3[b0:b0 + 48] = P2[b0:b0 + 48]
        got, want = run(P, vr=2, v1=v1, lam=lam), run(P3)
        assert np.linalg.norm(got - want) / np.linalg.norm(want - x) < 2e-3                           # v + (v1 - v) is v1 up to an ulp: a rare code flip downstream
        assert np.linalg.norm(got - plain) / np.linalg.norm(plain - x) > 0.05
    lam = np.array([0.3, 0.8], np.float32)
    # (the exact block above has no rotary embedding and no registers: the gate is taken without them, S = D^3)
    S0 = D ** 3; x0 = np.ascontiguousarray(x[:nseq * S0])
    run0 = lambda Pm, **kw: orc.block_fwd(8, Cc, H, F, 0, 0, 100.0, Pm, x0, nseq, S0, D, D, **kw)
    v1n = np.zeros((nseq * S0, Cc), np.float32); run0(P2, vr=1, v1=v1n)
    got = run0(P, vr=2, v1=v1n, lam=lam)
    ye = exact_block(P, lay, x0, nseq, S0, H, Cc, F, v1=v1n, lam=lam)
    assert np.linalg.norm(got - ye) / np.linalg.norm(ye) < 0.1 and np.linalg.norm((got - x0) - (ye - x0)) / np.linalg.norm(ye - x0) < 0.3
    ye_plain = exact_block(P, lay, x0, nseq, S0, H, Cc, F)
    assert np.linalg.norm(got - ye_plain) > 2 * np.linalg.norm(got - ye)         # and the mix is what moved it


def test_peg_is_depthwise_conv_plus_bias_plus_identity():
    """orc_peg_fwd (src/attn.h:141-144): against scipy's zero-padded correlation per channel in fp64; a single unit tap shifts the grid."""
    from scipy.ndimage import correlate
    rng = np.random.default_rng(4)
    nseq, (D, Hh, W), nreg, Cc = 2, (3, 4, 5), 2, 8
    Sg = D * Hh * W; S = nreg + Sg
    x = rng.standard_normal((nseq, S, Cc)).astype(np.float32); w = (0.3 * rng.standard_normal((Cc, 27))).astype(np.float32); b = rng.standard_normal(Cc).astype(np.float32)
    y = orc.peg_fwd(x.reshape(nseq * S, Cc), w, b, nseq, S, D, Hh, W, nreg).reshape(nseq, S, Cc)
    assert np.array_equal(y[:, :nreg], x[:, :nreg])
    for s in range(nseq):
        for c in range(Cc):
            g = x[s, nreg:, c].astype(np.float64).reshape(D, Hh, W)
            want = g + float(b[c]) + correlate(g, w[c].astype(np.float64).reshape(3, 3, 3), mode="constant", cval=0.0)
            assert np.abs(y[s, nreg:, c].reshape(D, Hh, W) - want).max() < 1e-5
    w1 = np.zeros((Cc, 27), np.float32); w1[:, 2 * 9 + 0 * 3 + 1] = 1      # the tap (dz, dy, dx) = (+1, -1, 0)
    y1 = orc.peg_fwd(x.reshape(nseq * S, Cc), w1, np.zeros(Cc), nseq, S, D, Hh, W, nreg).reshape(nseq, S, Cc)
    g = x[:, nreg:].reshape(nseq, D, Hh, W, Cc); sh = np.zeros_like(g); sh[:, :-1, 1:] = g[:, 1:, :-1]
    assert np.array_equal(y1[:, nreg:].reshape(g.shape), g + sh)
