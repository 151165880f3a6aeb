"""GPU parity of the MX GEMM and the MX-fp8 attention forward, through the C ABI, against the CPU oracle.

Shapes are the reference's own test matrix (tests/test_attn.c:442-449): GEMMs 70x45x100 and 300x520x100 for every transpose flag, the
split-K weight-gradient shape 300x96x4100; attention with 2 x (4 + 16^3) tokens at C 96 and 1 x (3 + 10^3) tokens at C 144."""
import ctypes as C

import numpy as np
import pytest

import orc
from gpuutil import DevBuf, LP, lib
from ufsm_amd import at_geom
from test_oracle_gemm_attn import stored, pack, exact_attention, quant_rows

pytestmark = pytest.mark.gpu


def gpu_gemm(bits, ta, tb, M, N, K, As, Bs, C0=None, beta=0.0, bias=None, res=None, ex=True):
    dA, dB = DevBuf.from_numpy(As.astype(np.float32)), DevBuf.from_numpy(Bs.astype(np.float32))
    dC = DevBuf.from_numpy(C0.astype(np.float32)) if C0 is not None else DevBuf.from_numpy(np.full((M, N), np.nan, np.float32))
    db = DevBuf.from_numpy(bias.astype(np.float32)) if bias is not None else None
    dr = DevBuf.from_numpy(res.astype(np.float32)) if res is not None else None
    if ex:
        rc = lib.lp_mx_gemm_ex(bits, ta, tb, M, N, K, dA.ptr, dB.ptr, dC.ptr, beta, db.ptr if db else None, dr.ptr if dr else None)
    else:
        rc = lib.lp_mx_gemm(bits, ta, tb, M, N, K, dA.ptr, dB.ptr, dC.ptr, beta)
    assert rc == 0
    LP.check()
    return dC.to_numpy(np.float32, (M, N))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("M,N,K", [(70, 45, 100), (300, 520, 100)])
def test_gemm_matches_oracle(gpu, bits, ta, tb, M, N, K):
    rng = np.random.default_rng(M + N + K + bits + 2 * ta + tb)
    A = rng.standard_normal((M, K)).astype(np.float32); B = (0.1 * rng.standard_normal((N, K))).astype(np.float32)
    As, Bs = stored(A, B, ta, tb)
    got = gpu_gemm(bits, ta, tb, M, N, K, As, Bs, ex=False)
    want = orc.mx_gemm(bits, ta, tb, M, N, K, As, Bs)
    # same operands bit for bit. e2m1 products are summed exactly by the MFMA; with e4m3 its internal alignment of the 64 products of
    # a step drops low bits (measured <= 4e-5 of the largest output): bound at 1e-4, a tenth of the conv's 1e-3 bar
    assert np.abs(got - want).max() <= (1e-4 if bits == 8 else 1e-6) * np.abs(want).max()
    ref = quant_rows(A, bits) @ quant_rows(B, bits).T                           # the reference's check (tests/test_attn.c:383, :394)
    assert np.abs(got - ref).max() <= 2e-3 * np.abs(ref).max()


@pytest.mark.parametrize("bits", [4, 8])
def test_gemm_epilogue_exact_operands(gpu, bits):
    """Grid-valued operands: products and sums are exact, so the GPU must EQUAL the integer product; then bias + residual + beta C."""
    rng = np.random.default_rng(bits)
    M, N, K = 150, 200, 96
    grid = np.array([0, .5, 1, 1.5, 2, 3, 4, 6]) if bits == 4 else np.arange(0, 17) / 2.0
    A = (rng.choice(grid, (M, K)) * rng.choice([-1, 1], (M, K))).astype(np.float32); A[:, ::32] = grid[-1]
    B = (rng.choice(grid, (N, K)) * rng.choice([-1, 1], (N, K))).astype(np.float32); B[:, 5::32] = -grid[-1]
    exact = (A.astype(np.float64) @ B.astype(np.float64).T).astype(np.float32)
    As, Bs = stored(A, B, 0, 1)
    assert np.array_equal(gpu_gemm(bits, 0, 1, M, N, K, As, Bs), exact)
    bias = rng.standard_normal(N).astype(np.float32); res = rng.standard_normal((M, N)).astype(np.float32); C0 = rng.standard_normal((M, N)).astype(np.float32)
    got = gpu_gemm(bits, 0, 1, M, N, K, As, Bs, C0=C0, beta=0.5, bias=bias, res=res)
    want = orc.mx_gemm(bits, 0, 1, M, N, K, As, Bs, C0=C0, beta=0.5, bias=bias, res=res)
    assert np.abs(got - want).max() < 1e-4
    assert lib.lp_mx_gemm(6, 0, 0, 4, 4, 4, None, None, None, 0.0) == -1         # unsupported width: the reference's return code
    assert lib.lp_mx_gemm(8, 0, 0, 0, 4, 4, None, None, None, 0.0) == 0          # empty output: nothing to do


@pytest.mark.parametrize("bits,beta", [(4, 0.0), (8, 0.0), (8, 1.0)])
def test_gemm_split_k(gpu, bits, beta):
    """The weight-gradient shape: few output tiles, K = tokens (tests/test_attn.c:447): K is split over workgroups that add atomically."""
    rng = np.random.default_rng(11 + bits)
    M, N, K = 300, 96, 4100
    A = rng.standard_normal((M, K)).astype(np.float32); B = (0.1 * rng.standard_normal((N, K))).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    As, Bs = stored(A, B, 1, 0)
    got = gpu_gemm(bits, 1, 0, M, N, K, As, Bs, C0=C0, beta=beta)
    want = orc.mx_gemm(bits, 1, 0, M, N, K, As, Bs, C0=C0, beta=beta)
    assert np.abs(got - want).max() <= (1e-4 if bits == 8 else 2e-5) * np.abs(want).max()    # (atomic sum order; e4m3 as above)


def gpu_attention(qk, nseq, S, H):
    T, Cc = nseq * S, H * 48
    dq = DevBuf.from_numpy(qk)
    do = DevBuf.from_numpy(np.full((T, Cc), np.nan, np.float32)); dl = DevBuf.from_numpy(np.full((nseq, H, S), np.nan, np.float32))
    g = at_geom(); g.nseq, g.S, g.D, g.Hh, g.W = nseq, S, 0, 0, 0
    assert lib.at_fa8_fwd(dq.ptr, do.ptr, dl.ptr, C.byref(g), H, Cc) == 0
    LP.check()
    return do.to_numpy(np.float32, (T, Cc)), dl.to_numpy(np.float32, (nseq, H, S))


def normed_qkv(rng, nseq, S, H):
    T = nseq * S
    qkv = 0.6 * rng.standard_normal((3, T, H, 48))
    for p in range(2):
        qkv[p] *= (1 + 0.2 * rng.standard_normal((1, H, 48))) / np.sqrt((qkv[p] ** 2).mean(-1, keepdims=True) + 1e-6)
    return pack(qkv[0], qkv[1], qkv[2], nseq, S, H)


@pytest.mark.parametrize("nseq,S,H", [(2, 4 + 8 ** 3, 2), (1, 3 + 10 ** 3, 3), (3, 37, 1), (1, 128, 4)])
def test_attention_matches_oracle(gpu, nseq, S, H):
    rng = np.random.default_rng(nseq * S + H)
    qk = normed_qkv(rng, nseq, S, H)
    o, lse = gpu_attention(qk, nseq, S, H)
    wo, wl = orc.fa8_fwd(qk, nseq, S, H)
    # The same quantised operands. The logits differ in their last bits (MFMA sum vs the oracle's exact block sums, <= 4e-5 relative),
    # so about one P code in 300 rounds to the neighbouring e4m3 value (a 2^-4 step of that key's weight): most query rows agree to
    # 1e-4, a few percent carry one such step, the largest being one step of a row's heaviest key. All far below the format's own
    # noise against exact attention (last assertion).
    rows = np.abs(o - wo).max(1) / np.abs(wo).max()
    assert np.median(rows) < 1e-4 and rows.max() < 2e-2 and np.linalg.norm(o - wo) <= 3e-3 * np.linalg.norm(wo)
    assert np.abs(lse - wl).max() < 1e-4 * max(1.0, np.abs(wl).max())
    oe, le = exact_attention(qk, nseq, S, H)                                       # the reference's gate (tests/test_attn.c:445-446)
    assert np.linalg.norm(o - oe) / np.linalg.norm(oe) < 0.1 and np.linalg.norm(lse - le) / np.linalg.norm(le) < 0.1


def test_attention_full_size_of_the_window_bottleneck(gpu):
    """The configs[4] shape: one sequence of 4 registers + 16^3 grid tokens, 4 heads (C 192). Against the oracle on sampled query rows'
    worth of checks (the whole oracle run is a few seconds on the host cores), and two size-independent properties: every output row lies
    in the convex hull of the quantised V (|o| <= max |v| per dim), and lse >= the largest logit of a row (checked through its bound
    log2 S + max - ... >= 0 on the softmax denominator: 2^(lse - m) in [1, S])."""
    rng = np.random.default_rng(77)
    nseq, S, H = 1, 4 + 16 ** 3, 4
    qk = normed_qkv(rng, nseq, S, H)
    o, lse = gpu_attention(qk, nseq, S, H)
    wo, wl = orc.fa8_fwd(qk, nseq, S, H)
    # with 4100 keys every query row carries a dozen of the one-in-300 P code steps (each 2^-4 of one key's ~1/4100 weight), and the
    # outputs themselves are small averages: the row errors rise to ~1e-3 of max |o| but stay steps of single keys
    rows = np.abs(o - wo).max(1) / np.abs(wo).max()
    assert np.median(rows) < 2e-3 and rows.max() < 3e-2 and np.linalg.norm(o - wo) <= 1e-2 * np.linalg.norm(wo)
    assert np.abs(lse - wl).max() < 1e-4 * np.abs(wl).max()
    v = qk.view(np.float16)[2].astype(np.float32)[:, :S]                              # [H][S][48]
    for h in range(H):
        assert (np.abs(o[:, h * 48:(h + 1) * 48]) <= np.abs(v[h]).max(0)[None] * (1 + 2.0 ** -3)).all()      # (e4m3 rounding of V can exceed |v| by 1/16)
    assert np.isfinite(o).all() and np.isfinite(lse).all()


@pytest.mark.parametrize("nseq,S,H", [(2, 4 + 8 ** 3, 2), (1, 128 * 3 + 1, 1), (3, 5, 1), (1, 250, 2)])
def test_attention_four_wavefront_workgroups_and_the_shared_last_tile(gpu, nseq, S, H):
    """Workgroups of four wavefronts (the launch the window bottleneck's eight sequences get). 4 + 8^3 and 385 tokens leave a last 32-query tile
    alone in its workgroup: its keys are shared among the four wavefronts and merged. Those rows are the same probabilities summed in another
    order (the other rows' bits do not change); 5 tokens: the only tile is such a tile and three wavefronts hold no keys; 250: no shared tile."""
    rng = np.random.default_rng(nseq * S + H + 1)
    qk = normed_qkv(rng, nseq, S, H)
    lib.at_fa8_waves(1)
    o1, l1 = gpu_attention(qk, nseq, S, H)
    lib.at_fa8_waves(4)
    try:
        o4, l4 = gpu_attention(qk, nseq, S, H)
    finally:
        lib.at_fa8_waves(0)
    shared = ((S + 31) // 32) % 4 == 1
    first = (S - 1) // 32 * 32 if shared else S                  # first token of the shared tile
    o1s, o4s = o1.reshape(nseq, S, -1), o4.reshape(nseq, S, -1)
    assert np.array_equal(o1s[:, :first], o4s[:, :first]) and np.array_equal(l1[:, :, :first], l4[:, :, :first])
    wo, wl = orc.fa8_fwd(qk, nseq, S, H)
    rows = np.abs(o4 - wo).max(1) / np.abs(wo).max()
    assert np.median(rows) < 1e-4 and rows.max() < 2e-2 and np.linalg.norm(o4 - wo) <= 3e-3 * np.linalg.norm(wo)
    assert np.abs(l4 - wl).max() < 1e-4 * max(1.0, np.abs(wl).max())
    if shared:                                                    # the same probabilities and codes, summed in another order
        d = np.abs(o4s[:, first:] - o1s[:, first:]).max() / np.abs(wo).max()
        assert d < 1e-5 and np.abs(l4[:, :, first:] - l1[:, :, first:]).max() < 1e-5 and np.isfinite(o4).all() and np.isfinite(l4).all()


def test_attention_closed_forms(gpu):
    """q = 0: o is the mean of the quantised V over the S valid keys and lse = log2 S, exactly as on the oracle; rows of another
    sequence or of the padding must not leak in."""
    rng = np.random.default_rng(2)
    nseq, S, H = 2, 100, 2
    T = nseq * S
    q = np.zeros((T, H, 48)); k = rng.standard_normal((T, H, 48)); v = rng.standard_normal((T, H, 48)); v[S:] += 10.0   # sequence 1 stands apart
    qk = pack(q, k, v, nseq, S, H)
    o, lse = gpu_attention(qk, nseq, S, H)
    wo, wl = orc.fa8_fwd(qk, nseq, S, H)
    assert np.abs(o - wo).max() < 1e-5 and np.abs(lse - np.log2(S)).max() < 1e-5
    assert o[:S].mean() < 1.0 and o[S:].mean() > 9.0
