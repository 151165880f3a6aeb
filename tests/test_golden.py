"""Committed golden vectors (tests/golden/mx_golden.npz, made by tests/golden/make_golden.py): the oracle and an independent numpy
quantiser are held to them on the CPU, the device is held to them on the GPU with no oracle in the loop."""
import os

import numpy as np
import pytest

import orc
import refnp

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mx_golden.npz"), allow_pickle=False)
CVT = ["cvt_a", "cvt_b", "cvt_c", "cvt_d"]
CONV = ["conv_f8", "conv_f4", "conv_f8_wide", "conv_f8_s2"]


def test_known_answer_table_of_the_encoders():
    L = orc.lib()
    for x, c8, c4 in zip(G["known_x"], G["known_e4m3"], G["known_e2m1"]):
        g8, g4 = L.orc_enc_e4m3(float(x)), L.orc_enc_e2m1(float(x))
        if np.isnan(x):
            assert (g8 & 0x7f) == 0x7f and (g4 & 7) == 7
        else:
            assert (g8, g4) == (int(c8), int(c4)), (float(x), hex(g8), hex(g4))
            assert L.orc_ref_e4m3(float(x)) == int(c8) and L.orc_ref_e2m1(float(x)) == int(c4)


@pytest.mark.parametrize("name", CVT)
@pytest.mark.parametrize("bits", [8, 4])
def test_converter_vectors(name, bits):
    x = G[name + "_x"]
    N, C, S = x.shape
    want = G["%s_mx%d" % (name, bits)]
    assert np.array_equal(orc.f32_to_mx(bits, x, N, C, S), want)
    # the independent numpy quantiser decodes to the same values (it does not share code with the oracle)
    assert np.array_equal(orc.mx_to_f32(bits, want, N, C, S), refnp.mx_quant_tensor(x, bits))


@pytest.mark.parametrize("name", CONV)
def test_conv_vectors(name):
    bits, N, Ci, Co, D, H, W, stride = [int(v) for v in G[name + "_shape"]]
    xdt = 3 if bits == 8 else 4
    xq, w, b = G[name + "_xq"], G[name + "_w"], G[name + "_b"]
    yq, sums = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, stride=stride, Go=4, want_stats=True)   # fp32 accumulation: exact operands
    assert np.array_equal(yq, G[name + "_yq"])
    assert np.allclose(sums, G[name + "_sums"], rtol=1e-12)
    # and the fp32 output equals a direct fp64 convolution of the decoded operands done in numpy
    # (weights on the e2m1 grid with a 6 in every block quantise losslessly, so w itself is the decoded operand)
    x = orc.mx_to_f32(bits, xq, N, Ci, D * H * W).reshape(N, Ci, D, H, W)
    ref = refnp.conv3d_f64(x, w, b, stride)
    assert np.array_equal(ref.astype(np.float32).reshape(N, Co, -1), G[name + "_yf"])


def test_up2_vector():
    N, C, D, H, W = [int(v) for v in G["up2_shape"]]
    y = np.zeros(orc.mx_bytes(8, N, C, 8 * D * H * W), np.uint8)
    xq = G["up2_xq"]
    orc.lib().orc_up2_mx(8, orc.ptr(xq), N, C, D, H, W, orc.gn(), orc.ptr(y), 8)
    assert np.array_equal(y, G["up2_yq"])


# ---------------- device against the fixtures ----------------
@pytest.mark.gpu
@pytest.mark.parametrize("name", CVT)
@pytest.mark.parametrize("bits", [8, 4])
def test_gpu_converter_vectors(gpu, name, bits):
    from gpuutil import to_mx
    assert np.array_equal(to_mx(bits, G[name + "_x"]).to_numpy(np.uint8), G["%s_mx%d" % (name, bits)])


@pytest.mark.gpu
@pytest.mark.parametrize("name", CONV)
def test_gpu_conv_vectors(gpu, name):
    from gpuutil import gpu_conv
    bits, N, Ci, Co, D, H, W, stride = [int(v) for v in G[name + "_shape"]]
    xdt = 3 if bits == 8 else 4
    xq, w, b = G[name + "_xq"], G[name + "_w"], G[name + "_b"]
    st = stride == 1                                                # lp_conv_fwd_s2_f8 has no statistics argument (src/nn_lp.h:104)
    yq, sums = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, stride=stride, Go=4 if st else 0, stats=st)
    assert np.array_equal(yq, G[name + "_yq"])
    assert not st or np.allclose(sums, G[name + "_sums"], rtol=1e-6)
    yf, _ = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride)
    assert np.array_equal(yf, G[name + "_yf"])


@pytest.mark.gpu
def test_gpu_up2_vector(gpu):
    from gpuutil import DevBuf, LP, lib, shape5, gnp_t
    N, C, D, H, W = [int(v) for v in G["up2_shape"]]
    dx = DevBuf.from_numpy(G["up2_xq"]); dy = DevBuf(G["up2_yq"].size)
    lib.lp_up2_fwd_mx(dx.ptr, 3, shape5(N, C, D, H, W), dy.ptr, 3, gnp_t())
    LP.check()
    assert np.array_equal(dy.to_numpy(np.uint8), G["up2_yq"])
