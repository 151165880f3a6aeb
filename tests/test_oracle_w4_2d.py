"""CPU pins (no GPU) of the oracle's 2-D fp4 weight scales (lp_set_w4_2d, src/lp_f4fwd.cu:67-83) and in-place fake quantisation
(lp_fakeq_w4, src/lp_mx_cvt.cu:369-395) against the independent numpy block quantiser, and of the invariant the reference builds on them:
values fake-quantised per 32 x 32 block are re-quantised exactly by the forward's per-output-channel blocks."""
import ctypes as C

import numpy as np
import pytest

import orc
import refnp


def np_fakeq(w, Bo, Bi):
    """w [Co][Ci][T] -> MX-fp4 values with one scale per Bo x Bi block and tap: amax over the block, the format's scale rule, nearest-even e2m1."""
    Co, Ci, T = w.shape
    out = np.zeros_like(w)
    for o0 in range(0, Co, Bo):
        for i0 in range(0, Ci, Bi):
            for t in range(T):
                blk = w[o0:o0 + Bo, i0:i0 + Bi, t]
                q, _ = refnp.quantize_block(blk.reshape(1, -1), 4)            # one block holding the whole tile
                out[o0:o0 + Bo, i0:i0 + Bi, t] = q.reshape(blk.shape)
    return out


@pytest.mark.parametrize("Co,Ci,T,Bo,Bi", [(64, 64, 27, 32, 32), (48, 80, 27, 32, 32), (20, 40, 8, 32, 32), (32, 64, 27, 1, 32), (64, 32, 3, 16, 1)])
def test_fakeq_equals_numpy_block_quantiser(Co, Ci, T, Bo, Bi):
    rng = np.random.default_rng(Co + Ci)
    w = (rng.standard_normal((Co, Ci, T)) * np.exp(rng.uniform(-3, 3, (Co, 1, 1)))).astype(np.float32)
    got = w.copy()
    orc.lib().orc_fakeq_w4(orc.ptr(got), Co, Ci, T, Bo, Bi)
    assert np.array_equal(got, np_fakeq(w, Bo, Bi))
    again = got.copy()
    orc.lib().orc_fakeq_w4(orc.ptr(again), Co, Ci, T, Bo, Bi)
    assert np.array_equal(again, got)                                          # idempotent


def prep(w, Co, Ci, on):
    Cip = (Ci + 31) // 32 * 32
    wv = np.zeros((27, Co, Cip), np.float32); ws = np.zeros((27, Co, Cip // 32), np.uint8)
    orc.lib().orc_set_w4_2d(on)
    try:
        orc.lib().orc_prep_w(4, orc.ptr(w), Co, Ci, Ci, Cip, Cip, orc.ptr(wv), orc.ptr(ws), None)
    finally:
        orc.lib().orc_set_w4_2d(0)
    return wv * np.repeat(np.ldexp(1.0, ws.astype(np.int64) - 127), 32, axis=2).astype(np.float32)      # decoded weights [tap][co][ci]


@pytest.mark.parametrize("Co,Ci", [(64, 64), (48, 96), (32, 40)])
def test_2d_prep_equals_the_fake_quantised_weights_and_1d_prep_keeps_them(Co, Ci):
    rng = np.random.default_rng(3 * Co + Ci)
    w = (rng.standard_normal((Co, Ci, 27)) * np.exp(rng.uniform(-2, 2, (Co, 1, 1))) * 0.1).astype(np.float32)
    want = np.transpose(np_fakeq(w, 32, 32), (2, 0, 1))                         # [tap][co][ci]
    got2d = prep(w, Co, Ci, 1)[:, :, :Ci]
    assert np.array_equal(got2d, want)
    # the invariant: per-output-channel blocks (1-D prep) of the fake-quantised values reproduce them
    fq = np.ascontiguousarray(np.transpose(want, (1, 2, 0)))
    assert np.array_equal(prep(fq, Co, Ci, 0)[:, :, :Ci], want)
    # ... and on raw weights the two preps differ (rows well below their tile's maximum lose resolution under the shared scale)
    assert not np.array_equal(prep(w, Co, Ci, 0)[:, :, :Ci], want)


def test_conv_with_2d_scales_is_the_conv_of_the_fake_quantised_weights():
    rng = np.random.default_rng(11)
    N, Ci, Co, D, H, W = 1, 64, 48, 3, 4, 5
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci, 27)) * np.exp(rng.uniform(-2, 2, (Co, 1, 1))) * 0.05).astype(np.float32)
    xq = orc.f32_to_mx(4, x, N, Ci, S)
    orc.lib().orc_set_w4_2d(1)
    try:
        a, _ = orc.conv3(xq, 4, N, Ci, D, H, W, w, None, Co, 0, cbits=4)
        s2, _ = orc.conv3(xq, 4, N, Ci, D, H, W, w, None, Co, 0, cbits=4, stride=2)
    finally:
        orc.lib().orc_set_w4_2d(0)
    fq = w.copy(); orc.lib().orc_fakeq_w4(orc.ptr(fq), Co, Ci, 27, 32, 32)
    b, _ = orc.conv3(xq, 4, N, Ci, D, H, W, fq, None, Co, 0, cbits=4)
    assert np.array_equal(a, b)
    s2_1d, _ = orc.conv3(xq, 4, N, Ci, D, H, W, w, None, Co, 0, cbits=4, stride=2)
    assert np.array_equal(s2, s2_1d)                                            # the stride-2 prep keeps its per-channel scales (src/lp_f4fwd.cuh:1163)
