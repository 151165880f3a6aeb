"""Pins of the oracle's MX GEMM and MX-fp8 attention forward (CPU only).

GEMM: the reference's own check (tests/test_attn.c:375-396): operands quantised by an independent block quantiser (here the numpy one
written from the format), multiplied in fp64. Attention: closed forms the mathematics fixes, plus the reference's gate against exact
fp64 attention (tests/test_attn.c:445-446: relative L2 < 0.1 for the fp8 core)."""
import numpy as np
import pytest

import orc
import refnp


def quant_rows(X, bits):
    """X [rows][K] float32 -> decoded MX values, one scale per 32 K (zero padding past K)."""
    rows, K = X.shape
    Kp = (K + 31) // 32 * 32
    Xp = np.zeros((rows, Kp), np.float32); Xp[:, :K] = X
    q, _ = refnp.quantize_block(Xp.reshape(rows, Kp // 32, 32), bits)
    return q.reshape(rows, Kp)[:, :K].astype(np.float64)


def stored(A, B, ta, tb):
    """logical A [M][K], B [N][K] -> the layouts the transpose flags name (A [K][M] for ta, B [K][N] unless tb)."""
    return (np.ascontiguousarray(A.T) if ta else A), (B if tb else np.ascontiguousarray(B.T))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", [(70, 45, 100), (33, 64, 64), (5, 3, 31)])
def test_gemm_equals_fp64_product_of_quantised_operands(bits, ta, tb, M, N, K):
    rng = np.random.default_rng(M * 7 + N + K + bits + 2 * ta + tb)
    A = rng.standard_normal((M, K)).astype(np.float32); B = (0.1 * rng.standard_normal((N, K))).astype(np.float32)
    ref = quant_rows(A, bits) @ quant_rows(B, bits).T
    As, Bs = stored(A, B, ta, tb)
    got = orc.mx_gemm(bits, ta, tb, M, N, K, As, Bs)
    assert np.abs(got - ref).max() <= 2e-6 * np.abs(ref).max() + 1e-7          # fp32 accumulation of exact block sums
    # the quantisation itself is visible: the unquantised product differs by the format's noise, not by rounding of the sums
    rel = np.linalg.norm(got - A.astype(np.float64) @ B.astype(np.float64).T) / np.linalg.norm(ref)
    assert (0.005 if bits == 8 else 0.05) < rel < (0.08 if bits == 8 else 0.35)


@pytest.mark.parametrize("bits", [4, 8])
def test_gemm_exact_operands_and_epilogue(bits):
    """Grid-valued operands with power-of-two block maxima quantise exactly: the GEMM must equal the integer product, and the
    epilogue terms (bias per column, residual, beta C) add on top (src/lp_mxgemm.cu:82-86)."""
    rng = np.random.default_rng(bits)
    M, N, K = 37, 29, 96
    grid = np.array([0, .5, 1, 1.5, 2, 3, 4, 6]) if bits == 4 else np.arange(0, 17) / 2.0
    A = (rng.choice(grid, (M, K)) * rng.choice([-1, 1], (M, K))).astype(np.float32); A[:, ::32] = grid[-1]      # amax = qmax-representable
    B = (rng.choice(grid, (N, K)) * rng.choice([-1, 1], (N, K))).astype(np.float32); B[:, 5::32] = -grid[-1]
    assert np.array_equal(quant_rows(A, bits), A) and np.array_equal(quant_rows(B, bits), B)
    bias = rng.standard_normal(N).astype(np.float32); res = rng.standard_normal((M, N)).astype(np.float32); C0 = rng.standard_normal((M, N)).astype(np.float32)
    As, Bs = stored(A, B, 1, 0)
    exact = A.astype(np.float64) @ B.astype(np.float64).T
    assert np.array_equal(orc.mx_gemm(bits, 1, 0, M, N, K, As, Bs), exact.astype(np.float32))
    got = orc.mx_gemm(bits, 1, 0, M, N, K, As, Bs, C0=C0, beta=0.5, bias=bias, res=res)
    want = exact + bias[None, :] + res + 0.5 * C0
    assert np.abs(got - want).max() < 1e-4
    assert orc.lib().orc_mx_gemm(6, 0, 0, 1, 1, 1, None, None, None, 0.0, None, None) == -1                       # unsupported width


def pack(q, k, v, nseq, S, H):
    """q, k, v float [nseq * S][H][48] -> fp16 head-major pack [3][H][nseq * S + 64][48] (rows past T unused)."""
    T = nseq * S
    out = np.zeros((3, H, T + 64, 48), np.float16)
    for p, x in enumerate((q, k, v)):
        out[p, :, :T] = np.moveaxis(x, 1, 0)
    return out.view(np.uint16)


def exact_attention(qkvh, nseq, S, H):
    x = qkvh.view(np.float16).astype(np.float64)
    o = np.zeros((nseq * S, H * 48)); lse = np.zeros((nseq, H, S))
    for s in range(nseq):
        for h in range(H):
            q, k, v = (x[p, h, s * S:(s + 1) * S] for p in range(3))
            lg = q @ k.T / np.sqrt(48.0)
            m = lg.max(1, keepdims=True); e = np.exp(lg - m)
            o[s * S:(s + 1) * S, h * 48:(h + 1) * 48] = (e / e.sum(1, keepdims=True)) @ v
            lse[s, h] = (m[:, 0] + np.log(e.sum(1))) * np.log2(np.e)
    return o, lse


def quant_v(v, S):
    """v [S][48] -> the values the attention multiplies with: one scale per (dim, 32 tokens of the sequence)."""
    Sp = (S + 63) // 64 * 64
    vp = np.zeros((Sp, 48), np.float32); vp[:S] = v
    q, _ = refnp.quantize_block(np.ascontiguousarray(vp.T).reshape(48, Sp // 32, 32), 8)
    return q.reshape(48, Sp).T[:S].astype(np.float64)


@pytest.mark.parametrize("S", [64, 100, 191])
def test_attention_uniform_logits_is_mean_of_quantised_v(S):
    """q = 0: every logit is 0, P = 1 exactly, so o = mean over the S keys of the quantised V and lse = log2(S); masked keys past S
    and zero rows of the padded tiles must not enter (S not a multiple of 64)."""
    rng = np.random.default_rng(S)
    nseq, H = 2, 2
    T = nseq * S
    q = np.zeros((T, H, 48)); k = rng.standard_normal((T, H, 48)); v = rng.standard_normal((T, H, 48))
    qk = pack(q, k, v, nseq, S, H)
    o, lse = orc.fa8_fwd(qk, nseq, S, H)
    vh = qk.view(np.float16)[2].astype(np.float32)
    for s in range(nseq):
        for h in range(H):
            want = quant_v(vh[h, s * S:(s + 1) * S], S).mean(0)
            assert np.abs(o[s * S:(s + 1) * S, h * 48:(h + 1) * 48] - want[None]).max() < 2e-6 * S
    assert np.abs(lse - np.log2(S)).max() < 1e-5


def test_attention_dominant_key_selects_its_quantised_v_row():
    """One key per query outweighs the rest by > 2^30: P is 1 there and underflows the e4m3 grid elsewhere, so o is that key's
    quantised V row: checks the token order of the transposed V, the running maximum moving to a later key tile (the accumulated
    earlier tiles are rescaled to nothing) and staying on an earlier one."""
    rng = np.random.default_rng(5)
    nseq, S, H = 1, 200, 1
    sel = rng.integers(0, S, S); sel[:4] = [0, 63, 64, 199]
    k = np.zeros((S, H, 48)); q = np.zeros((S, H, 48))
    # key j = e_(j % 48) * (1 + j // 48); query i points at key sel[i] alone: dims are shared by keys 48 apart, told apart by sign pattern
    code = rng.choice([-1.0, 1.0], (S, 48))
    k[:, 0] = code * 8.0
    q[:, 0] = code[sel] * 8.0                                      # q.k = 64 * (agreeing - disagreeing signs): 3072 for the selected key
    lg = (q[:, 0] @ k[:, 0].T) / np.sqrt(48.0) * np.log2(np.e)
    second = np.sort(lg, 1)[:, -2]
    assert ((lg[np.arange(S), sel] - second) > 40).all()           # every other key is below 2^-40 of the maximum
    v = rng.standard_normal((S, H, 48))
    qk = pack(q, k, v, nseq, S, H)
    o, lse = orc.fa8_fwd(qk, nseq, S, H)
    vq = quant_v(qk.view(np.float16)[2, 0, :S].astype(np.float32), S)
    assert np.abs(o - vq[sel]).max() < 1e-6
    assert np.abs(lse[0, 0] - lg[np.arange(S), sel]).max() < 1e-3 * np.abs(lg).max()


@pytest.mark.parametrize("nseq,S,H", [(2, 130, 2), (1, 1003 // 4, 3)])
def test_attention_within_reference_gate_of_exact_attention(nseq, S, H):
    """The reference's acceptance test of its fp8 core (tests/test_attn.c:445-446): relative L2 < 0.1 against exact attention on
    QK-normalised rows (unit RMS times gains near 1) and N(0, 0.6^2) values; the same gate for lse."""
    rng = np.random.default_rng(nseq * S + H)
    T = nseq * S
    qkv = 0.6 * rng.standard_normal((3, T, H, 48))
    for p in range(2):
        qkv[p] *= (1 + 0.2 * rng.standard_normal((1, H, 48))) / np.sqrt((qkv[p] ** 2).mean(-1, keepdims=True) + 1e-6)
    qk = pack(qkv[0], qkv[1], qkv[2], nseq, S, H)
    o, lse = orc.fa8_fwd(qk, nseq, S, H)
    oe, le = exact_attention(qk, nseq, S, H)
    assert np.linalg.norm(o - oe) / np.linalg.norm(oe) < 0.1
    assert np.linalg.norm(lse - le) / np.linalg.norm(le) < 0.1 and np.abs(lse - le).max() < 0.1       # (logits carry e4m3 noise)
