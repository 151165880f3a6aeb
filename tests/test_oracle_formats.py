"""CPU tests that pin the oracle's format arithmetic (no GPU): encoders against an independent nearest-grid search and the known
answers the reference documents, the scale rule against its ceil(log2) form, the block quantiser against a numpy statement of the format."""
import ctypes as C
import os

import numpy as np
import pytest

import orc
import refnp


def f32(u):
    return np.array([u], dtype=np.uint32).view(np.float32)[0]


def test_e2m1_known_answers():
    L = orc.lib()
    # ties go to the even code (src/mx_sw.cuh:8-9; tests/test_mx4_wide.c:129-135): 0.25->0, 0.75->1.0, 1.25->1.0, 1.75->2.0, 2.5->2.0, 3.5->4.0, 5.0->4.0
    for x, val in [(0.25, 0.0), (0.75, 1.0), (1.25, 1.0), (1.75, 2.0), (2.5, 2.0), (3.5, 4.0), (5.0, 4.0), (5.0001, 6.0), (6.0, 6.0), (7.0, 6.0), (1e30, 6.0),
                   (0.26, 0.5), (0.74, 0.5), (2.51, 3.0), (3.49, 3.0), (4.99, 4.0)]:
        assert L.orc_dec_e2m1(L.orc_enc_e2m1(x)) == val, x
        assert L.orc_dec_e2m1(L.orc_enc_e2m1(-x)) == -val, x
    assert L.orc_enc_e2m1(float("nan")) == 7 and L.orc_enc_e2m1(-float("nan")) == 7       # NaN -> +6
    assert L.orc_enc_e2m1(float("inf")) == 7 and L.orc_enc_e2m1(-float("inf")) == 15
    assert L.orc_enc_e2m1(-0.0) == 8                                                        # -0 keeps its sign


def test_e4m3_known_answers():
    L = orc.lib()
    assert L.orc_enc_e4m3(448.0) == 0x7E and L.orc_enc_e4m3(464.0) == 0x7E and L.orc_enc_e4m3(1e9) == 0x7E     # src/mx_sw.cuh:5
    assert L.orc_enc_e4m3(-500.0) == 0xFE and L.orc_enc_e4m3(float("inf")) == 0x7E and L.orc_enc_e4m3(-float("inf")) == 0xFE
    assert L.orc_enc_e4m3(float("nan")) == 0x7F and L.orc_enc_e4m3(-float("nan")) == 0x7F                       # NaN of either sign
    assert L.orc_enc_e4m3(447.9) == 0x7E and L.orc_enc_e4m3(432.0) == 0x7E and L.orc_enc_e4m3(431.9) == 0x7D   # tie 432 = (416+448)/2 -> even code 0x7E
    assert L.orc_enc_e4m3(2.0 ** -9) == 1 and L.orc_enc_e4m3(2.0 ** -10) == 0 and L.orc_enc_e4m3(1.5 * 2.0 ** -9) == 2   # subnormal step, ties to even
    assert L.orc_enc_e4m3(2.0 ** -6) == 8 and L.orc_enc_e4m3(1.0) == 0x38 and L.orc_enc_e4m3(-1.0) == 0xB8 and L.orc_enc_e4m3(-0.0) == 0x80
    # every code decodes and re-encodes to itself
    for c in range(256):
        if (c & 0x7F) == 0x7F:
            assert np.isnan(L.orc_dec_e4m3(c))
        else:
            assert L.orc_enc_e4m3(L.orc_dec_e4m3(c)) == c, c
    for c in range(16):
        assert L.orc_enc_e2m1(L.orc_dec_e2m1(c)) == c


def test_decode_tables_match_format_definition():
    L = orc.lib()
    for c in range(127):
        assert L.orc_dec_e4m3(c) == np.float32(refnp.E4M3[c])
        assert L.orc_dec_e4m3(c | 0x80) == -np.float32(refnp.E4M3[c]) or c == 0
    for c in range(8):
        assert L.orc_dec_e2m1(c) == np.float32(refnp.E2M1[c])


def test_encoders_equal_nearest_grid_search():
    """The pin of the encoders: equality with the exhaustive nearest-code search on (a) a stride through all 2^32 bit patterns,
    (b) every bit pattern within 64 ulps of each grid value and each midpoint of both formats, (c) every exponent's first / last values.
    The whole 2^32 sweep (about 15 core-minutes) runs with UFSM_FULL_SWEEP=1; it passed when the oracle was written."""
    L = orc.lib()
    bad = C.c_uint32(0)
    assert L.orc_enc_sweep(0, 1 << 32, 4093, C.byref(bad)) == 0, hex(bad.value)
    pts = list(refnp.E4M3) + list(refnp.E2M1)
    pts += [0.5 * (a + b) for a, b in zip(refnp.E4M3[:-1], refnp.E4M3[1:])] + [0.5 * (a + b) for a, b in zip(refnp.E2M1[:-1], refnp.E2M1[1:])]
    pts += [448.0, 464.0, 480.0, 6.0, 5.0, 2.0 ** -10, 2.0 ** -11]
    for p in pts:
        u = int(np.array([p], dtype=np.float32).view(np.uint32)[0])
        lo = max(u - 64, 0)
        assert L.orc_enc_sweep(lo, 129, 1, C.byref(bad)) == 0, hex(bad.value)
        assert L.orc_enc_sweep(lo | 0x80000000, 129, 1, C.byref(bad)) == 0, hex(bad.value)
    for ex in range(256):
        assert L.orc_enc_sweep(ex << 23, 64, 1, C.byref(bad)) == 0
        assert L.orc_enc_sweep(((ex + 1) << 23) - 64, 64, 1, C.byref(bad)) == 0


@pytest.mark.skipif(not os.environ.get("UFSM_FULL_SWEEP"), reason="15 core-minutes; set UFSM_FULL_SWEEP=1")
def test_encoders_full_sweep():
    bad = C.c_uint32(0)
    assert orc.lib().orc_enc_sweep(0, 1 << 32, 1, C.byref(bad)) == 0, hex(bad.value)


def test_mx_exp_closed_form_and_specials():
    L = orc.lib()
    rng = np.random.default_rng(1)
    for qmax in (448.0, 6.0):
        inv = float(np.float32(1.0) / np.float32(qmax))
        am = np.concatenate([np.exp(rng.uniform(-80, 80, 20000)).astype(np.float32), qmax * np.ldexp(1.0, rng.integers(-100, 100, 2000)).astype(np.float32),
                             np.nextafter((qmax * np.ldexp(1.0, rng.integers(-100, 100, 2000))).astype(np.float32), np.float32(np.inf))])
        want = refnp.scale_exp(am, qmax)
        got = np.array([L.orc_mx_exp(float(a), inv) for a in am])
        assert (got == want).all()
        # the defining property on the fp32 product the reference forms: fl(amax * fl(1 / qmax)) <= 2^e, and e is the smallest such
        # exponent inside the clamp
        p32 = (am * np.float32(inv)).astype(np.float64)
        inside = (got > -126) & (got < 126)
        assert (p32 <= np.ldexp(1.0, got))[got < 126].all()
        assert (p32 > np.ldexp(1.0, got - 1))[inside].all()
        assert L.orc_mx_exp(0.0, inv) == -126                  # zero block -> scale byte 1 (never 0)
        assert L.orc_mx_exp(float("inf"), inv) == 128 and L.orc_mx_exp(float("nan"), inv) == 128      # scale byte 0xFF
        assert L.orc_mx_exp(3.0e38, inv) <= 126
    assert L.orc_mx_exp(448.0, float(np.float32(1) / np.float32(448))) == 0 and L.orc_mx_exp(6.0, float(np.float32(1) / np.float32(6))) in (0, 1)
    assert L.orc_mx_scale(127) == 1.0 and L.orc_mx_scale(1) == 2.0 ** -126 and np.isinf(L.orc_mx_scale(255))


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("Cc", [4, 12, 16, 32, 48, 80])
def test_tensor_quantiser_equals_format_definition(bits, Cc):
    rng = np.random.default_rng(bits * 100 + Cc)
    N, S = 2, 321
    x = (rng.standard_normal((N, Cc, S)) * np.exp(rng.standard_normal((N, 1, S)) * 4)).astype(np.float32)
    x[0, :, 5] = 0.0                                           # an all-zero block
    x[1, 0, 7] = 448.0 if bits == 8 else 6.0
    q = orc.f32_to_mx(bits, x, N, Cc, S)
    assert q.size == orc.mx_bytes(bits, N, Cc, S)
    dec = orc.mx_to_f32(bits, q, N, Cc, S)
    want = refnp.mx_quant_tensor(x, bits)
    assert (dec.view(np.uint32) == want.view(np.uint32)).all() or np.array_equal(dec, want)
    # scale bytes stay in 1..253 for finite data; padding channels are zero codes
    bw = 8 if Cc <= 8 else 16 if Cc <= 16 else 32
    nb = (Cc + bw - 1) // bw
    rb = bw * bits // 8
    sc = q[N * nb * S * rb:]
    assert sc.min() >= 1 and sc.max() <= 253
    # a second quantisation of the decoded tensor is lossless (dmx4_exact, tests/test_mx4_wide.c:70-75)
    assert np.array_equal(orc.mx_to_f32(bits, orc.f32_to_mx(bits, dec, N, Cc, S), N, Cc, S), dec)


@pytest.mark.parametrize("bits", [8, 4])
def test_nonfinite_block_policy(bits):
    """A NaN / inf in a block gives scale byte 0xFF and the block decodes non-finite (tests/test_mx4.c:139-168)."""
    N, Cc, S = 1, 32, 8
    x = np.ones((N, Cc, S), dtype=np.float32)
    x[0, 3, 1] = np.nan
    x[0, 4, 2] = np.inf
    x[0, 5, 3] = -np.inf
    q = orc.f32_to_mx(bits, x, N, Cc, S)
    rb = 32 * bits // 8
    sc = q[S * rb:]
    assert sc[1] == 0xFF and sc[2] == 0xFF and sc[3] == 0xFF and sc[0] != 0xFF
    dec = orc.mx_to_f32(bits, q, N, Cc, S)
    for v in (1, 2, 3):
        assert not np.isfinite(dec[0, :, v]).any()
    assert np.isfinite(dec[0, :, 0]).all()


def test_h16_roundtrip():
    L = orc.lib()
    for h in list(range(0, 0x7C00, 7)) + [0x7BFF, 0x0001, 0x03FF, 0x0400]:
        f = L.orc_h16_to_f32(h)
        assert L.orc_f32_to_h16(f) == h
        assert np.float16(f).view(np.uint16) == h
    rng = np.random.default_rng(3)
    for v in (rng.standard_normal(2000) * np.exp(rng.uniform(-12, 12, 2000))).astype(np.float32):
        assert L.orc_f32_to_h16(float(v)) == int(np.float16(v).view(np.uint16))
