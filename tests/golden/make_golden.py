#!/usr/bin/env python3
"""Writes tests/golden/mx_golden.npz: small input / expected-output vectors of the MX path.

The reference holds no golden files for this path (its tests draw data from xorshift seeds), so these are made by this repository's CPU
oracle once its pins pass (tests/test_oracle_*.py), plus a hand-derived known-answer table of the element encoders taken from the format
definitions (OCP e4m3 "FN" and e2m1 grids, round to nearest even, saturating). Two uses: the oracle is held to them on the CPU
(a regression guard: an edit to the oracle that changes any byte fails), and the device is held to them on the GPU without the
oracle in the loop. Re-run only when a format rule changes:  python3 tests/golden/make_golden.py"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import orc      # noqa: E402
import refnp    # noqa: E402

# value -> (e4m3 code, e2m1 code), derived by hand from the grids: ties go to the even code, overflow saturates, NaN -> 0x7f / 0x7
KNOWN = [
    (0.0, 0x00, 0x0), (-0.0, 0x80, 0x8), (1.0, 0x38, 0x2), (-1.0, 0xb8, 0xa), (0.5, 0x30, 0x1), (1.5, 0x3c, 0x3), (2.0, 0x40, 0x4), (3.0, 0x44, 0x5),
    (4.0, 0x48, 0x6), (6.0, 0x4c, 0x7), (448.0, 0x7e, 0x7), (464.0, 0x7e, 0x7), (1e9, 0x7e, 0x7), (-1e9, 0xfe, 0xf),
    (0.25, 0x28, 0x0),         # e2m1: tie between 0 and 0.5 -> even code 0
    (0.75, 0x34, 0x2),         # e2m1: tie between 0.5 (code 1) and 1.0 (code 2) -> even code 2
    (1.25, 0x3a, 0x2),         # e2m1: tie 1.0 / 1.5 -> code 2
    (2.5, 0x42, 0x4),          # e2m1: tie 2 / 3 -> code 4
    (5.0, 0x4a, 0x6),          # e2m1: tie 4 / 6 -> code 6 (4.0)
    (5.0001, 0x4a, 0x7), (1.0625, 0x38, 0x2),   # e4m3: tie 1.0 / 1.125 -> even mantissa (1.0)
    (1.1875, 0x3a, 0x2),       # e4m3: tie 1.125 (0x39) / 1.25 (0x3a) -> even 0x3a
    (2.0 ** -9, 0x01, 0x0), (2.0 ** -10, 0x00, 0x0),   # e4m3 smallest subnormal; half of it ties to even 0
    (3 * 2.0 ** -10, 0x02, 0x0),                         # tie between subnormals 1 and 2 -> 2
    (float("inf"), 0x7e, 0x7), (float("-inf"), 0xfe, 0xf), (float("nan"), 0x7f, 0x7),
]


def main():
    L = orc.lib()
    out = {}
    kv = np.array([k[0] for k in KNOWN], np.float32)
    out["known_x"] = kv
    out["known_e4m3"] = np.array([k[1] for k in KNOWN], np.uint8)
    out["known_e2m1"] = np.array([k[2] for k in KNOWN], np.uint8)
    for x, c8, c4 in KNOWN:                      # the table must hold for the oracle before anything is written
        g8, g4 = L.orc_enc_e4m3(x), L.orc_enc_e2m1(x)
        if x != x:
            assert (g8 & 0x7f) == 0x7f and (g4 & 7) == 7, (x, g8, g4)
        else:
            assert (g8, g4) == (c8, c4), (x, hex(g8), hex(g4), hex(c8), hex(c4))
    rng = np.random.default_rng(20240607)
    # converters: ragged channel counts (block widths 8, 16, 32 and a partial last block), values over many binades
    for name, (N, C, S) in {"cvt_a": (1, 4, 37), "cvt_b": (2, 12, 29), "cvt_c": (1, 40, 50), "cvt_d": (1, 64, 33)}.items():
        x = (rng.standard_normal((N, C, S)) * np.exp2(rng.integers(-12, 12, (N, 1, S)))).astype(np.float32)
        x[0, 0, :4] = [0.0, -0.0, 3e38, -1e-40]
        out[name + "_x"] = x
        for bits in (8, 4):
            out["%s_mx%d" % (name, bits)] = orc.f32_to_mx(bits, x, N, C, S)
    # convs with exact operands (every partial sum exact in fp32: the expected bytes do not depend on a summation order)
    for name, (bits, N, Ci, Co, D, H, W, stride) in {"conv_f8": (8, 1, 32, 32, 3, 5, 9, 1), "conv_f4": (4, 1, 64, 32, 2, 6, 7, 1),
                                                     "conv_f8_wide": (8, 1, 96, 64, 2, 4, 18, 1), "conv_f8_s2": (8, 1, 32, 32, 5, 6, 7, 2)}.items():
        S = D * H * W
        xdt = 3 if bits == 8 else 4
        x = refnp.gen_exact(rng, (N, Ci, S)); w = refnp.gen_exact(rng, (Co, Ci, 27))
        b = (np.array([0, .5, 1, 1.5, 2, 3, 4, 6], np.float32)[rng.integers(0, 8, Co)] * 0.25).astype(np.float32)
        xq = orc.f32_to_mx(bits, x, N, Ci, S)
        yq, sums = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, stride=stride, acc64=1, Go=4, want_stats=True)
        yf, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride, acc64=1)
        out[name + "_shape"] = np.array([bits, N, Ci, Co, D, H, W, stride], np.int32)
        out[name + "_xq"] = xq; out[name + "_w"] = w; out[name + "_b"] = b
        out[name + "_yq"] = yq; out[name + "_yf"] = yf; out[name + "_sums"] = sums
    # trilinear 2x on grid data with a +6 in every block (the blend is exact: tests/test_mx4_wide.c:18-19)
    N, C, D, H, W = 1, 32, 2, 3, 4
    x = refnp.gen_exact(rng, (N, C, D * H * W)); x[:, 0, :] = 6.0
    xq = orc.f32_to_mx(8, x, N, C, D * H * W)
    y = np.zeros(orc.mx_bytes(8, N, C, 8 * D * H * W), np.uint8)
    L.orc_up2_mx(8, orc.ptr(xq), N, C, D, H, W, orc.gn(), orc.ptr(y), 8)
    out["up2_shape"] = np.array([N, C, D, H, W], np.int32); out["up2_xq"] = xq; out["up2_yq"] = y
    np.savez_compressed(os.path.join(HERE, "mx_golden.npz"), **out)
    print("wrote mx_golden.npz:", len(out), "arrays,", os.path.getsize(os.path.join(HERE, "mx_golden.npz")), "bytes")


if __name__ == "__main__":
    main()
