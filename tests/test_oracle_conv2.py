"""CPU pins (no GPU) of the oracle's 2x2x2 stride-2 conv and transposed conv, the two stride-2 layers the reference does not have (its down conv
is 3x3x3 stride 2, its upsample trilinear: src/lp_s2.cu:4-9, src/lp_mx_gn.cu:32-33). Pinned by what the mathematics fixes: fp64 closed forms on
operands that are exact in the formats, the 3x3x3 stride-2 oracle conv with the eight taps embedded in its kernel (a path already pinned by
the reference's own checkers), adjointness of the two ops, and the independent numpy block quantiser for inexact operands."""
import numpy as np
import pytest

import orc
import refnp


def down_f64(x, w, b):
    """x [N][Ci][D][H][W], w [Co][Ci][2][2][2] -> [N][Co][D/2][H/2][W/2] in float64."""
    N, Ci, D, H, W = x.shape
    xr = x.reshape(N, Ci, D // 2, 2, H // 2, 2, W // 2, 2).astype(np.float64)
    y = np.einsum("niazbydx,oizyx->noabd", xr, w.astype(np.float64))
    return y + (b.astype(np.float64)[None, :, None, None, None] if b is not None else 0)


def up_f64(x, w, b):
    """x [N][Ci][D][H][W], w [Ci][Co][2][2][2] -> [N][Co][2D][2H][2W] in float64 (torch ConvTranspose3d, stride 2)."""
    N, Ci, D, H, W = x.shape
    Co = w.shape[1]
    y = np.einsum("niabd,iozyx->noazbydx", x.astype(np.float64), w.astype(np.float64)).reshape(N, Co, 2 * D, 2 * H, 2 * W)
    return y + (b.astype(np.float64)[None, :, None, None, None] if b is not None else 0)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("Ci,Co,dims", [(32, 32, (4, 4, 6)), (64, 48, (2, 6, 4)), (40, 16, (4, 2, 2))])
def test_down_exact_operands_equal_fp64_and_the_embedded_3x3x3(bits, Ci, Co, dims):
    rng = np.random.default_rng(bits * 100 + Ci)
    D, H, W = dims
    N, S = 2, D * H * W
    x = refnp.gen_exact(rng, (N, Ci, S)); w = refnp.gen_exact(rng, (Co, Ci, 8)); b = rng.integers(-8, 9, Co).astype(np.float32) * 0.25
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    got = orc.conv2(xq, 3 if bits == 8 else 4, N, Ci, D, H, W, w, b, Co, 0, 0, cbits=bits, acc64=1)
    want = down_f64(x.reshape(N, Ci, D, H, W), w.reshape(Co, Ci, 2, 2, 2), b).reshape(N, Co, -1)
    assert np.array_equal(got, want.astype(np.float32))
    # the same numbers from the 3x3x3 stride-2 pad-1 conv whose taps (1 + dz, 1 + dy, 1 + dx) hold the kernel and whose other taps are zero
    w3 = np.zeros((Co, Ci, 3, 3, 3), np.float32); w3[:, :, 1:, 1:, 1:] = w.reshape(Co, Ci, 2, 2, 2)
    y3, _ = orc.conv3(xq, 3 if bits == 8 else 4, N, Ci, D, H, W, np.ascontiguousarray(w3.reshape(Co, Ci, 27)), b, Co, 0, cbits=bits, stride=2, acc64=1)
    assert np.array_equal(got, y3)
    # ... also on random operands, where both quantise weights per (tap, output channel, 32 input channels) and rows per voxel: equal in fp64 accumulation
    xr = rng.standard_normal((N, Ci, S)).astype(np.float32); wr = (rng.standard_normal((Co, Ci, 8)) * 0.2).astype(np.float32)
    xq = orc.f32_to_mx(bits, xr, N, Ci, S)
    w3[:, :, 1:, 1:, 1:] = wr.reshape(Co, Ci, 2, 2, 2)
    for ydt in (0, 3, 4):
        g = orc.conv2(xq, 3 if bits == 8 else 4, N, Ci, D, H, W, wr, b, Co, ydt, 0, cbits=bits, acc64=1)
        y3, _ = orc.conv3(xq, 3 if bits == 8 else 4, N, Ci, D, H, W, np.ascontiguousarray(w3.reshape(Co, Ci, 27)), b, Co, ydt, cbits=bits, stride=2, acc64=1)
        assert np.array_equal(g, y3)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("Ci,Co,dims", [(32, 32, (2, 3, 4)), (64, 48, (1, 2, 5)), (40, 16, (2, 2, 2))])
def test_up_exact_operands_equal_fp64(bits, Ci, Co, dims):
    rng = np.random.default_rng(bits * 100 + Ci + 1)
    D, H, W = dims
    N, S = 2, D * H * W
    x = refnp.gen_exact(rng, (N, Ci, S)); w = refnp.gen_exact(rng, (Ci, Co, 8), block_axis=0); b = rng.integers(-8, 9, Co).astype(np.float32) * 0.25
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    got = orc.conv2(xq, 3 if bits == 8 else 4, N, Ci, D, H, W, w, b, Co, 0, 1, cbits=bits, acc64=1)
    want = up_f64(x.reshape(N, Ci, D, H, W), w.reshape(Ci, Co, 2, 2, 2), b).reshape(N, Co, -1)
    assert np.array_equal(got, want.astype(np.float32))
    # MX outputs: the fp64 result through the independent block quantiser
    for ydt, ob in ((3, 8), (4, 4)):
        q = orc.conv2(xq, 3 if bits == 8 else 4, N, Ci, D, H, W, w, b, Co, ydt, 1, cbits=bits, acc64=1)
        assert np.array_equal(orc.mx_to_f32(ob, q, N, Co, 8 * S), refnp.mx_quant_tensor(want.astype(np.float32), ob))


@pytest.mark.parametrize("bits", [8, 4])
def test_random_operands_follow_the_block_quantisers_and_the_ops_are_adjoint(bits):
    """Inexact operands: the result is the fp64 op applied to independently quantised operands (rows per voxel and 32 channels, weights per
    tap, output channel and 32 input channels); with the same quantised operands <down(x), u> = <x, up(u)> when the up weights are the
    down weights transposed (the scales then sit on the same 32-channel groups only for Co = Ci = 32, which is the case taken)."""
    rng = np.random.default_rng(77 + bits)
    N, C, D, H, W = 1, 32, 4, 4, 4
    S = D * H * W
    x = rng.standard_normal((N, C, S)).astype(np.float32); w = (rng.standard_normal((C, C, 8)) * 0.3).astype(np.float32)
    xq = orc.f32_to_mx(bits, x, N, C, S)
    xd = refnp.mx_quant_tensor(x, bits)
    wd = np.zeros_like(w)
    for t in range(8):
        wd[:, :, t], _ = refnp.quantize_block(w[:, :, t], bits)              # [co][32 ci] blocks
    got = orc.conv2(xq, 3 if bits == 8 else 4, N, C, D, H, W, w, None, C, 0, 0, cbits=bits, acc64=1)
    want = down_f64(xd.reshape(N, C, D, H, W), wd.reshape(C, C, 2, 2, 2), None).reshape(N, C, -1)
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    # fp32 accumulation stays within a few ulp of the running sums
    got32 = orc.conv2(xq, 3 if bits == 8 else 4, N, C, D, H, W, w, None, C, 0, 0, cbits=bits, acc64=0)
    assert np.abs(got32 - want).max() <= 1e-5 * np.abs(want).max()
    # transposed conv with the transposed kernel: weights [ci][co][tap] quantised along ci for each (tap, co): blocks along axis 0
    wt = np.ascontiguousarray(np.transpose(w, (1, 0, 2)))                       # [ci'][co'][tap] = w[co'][ci'][tap]
    wtd = np.zeros_like(wt)
    for t in range(8):
        q, _ = refnp.quantize_block(np.ascontiguousarray(wt[:, :, t].T), bits)  # rows co', blocks over ci'
        wtd[:, :, t] = q.T
    Sc = S // 8
    u = rng.standard_normal((N, C, Sc)).astype(np.float32)
    uq = orc.f32_to_mx(bits, u, N, C, Sc); ud = refnp.mx_quant_tensor(u, bits)
    upv = orc.conv2(uq, 3 if bits == 8 else 4, N, C, D // 2, H // 2, W // 2, wt, None, C, 0, 1, cbits=bits, acc64=1)
    wantu = up_f64(ud.reshape(N, C, D // 2, H // 2, W // 2), wtd.reshape(C, C, 2, 2, 2), None).reshape(N, C, -1)
    assert np.allclose(upv, wantu, rtol=1e-6, atol=1e-6)
    # adjointness in exact arithmetic on one set of dequantised weights
    dn = down_f64(xd.reshape(N, C, D, H, W), wd.reshape(C, C, 2, 2, 2), None)
    upw = up_f64(ud.reshape(N, C, D // 2, H // 2, W // 2), wd.reshape(C, C, 2, 2, 2), None)      # (the adjoint's [in][out] kernel is the down conv's [out][in] as it lies)
    assert np.isclose((dn * ud.reshape(dn.shape)).sum(), (xd.reshape(upw.shape) * upw).sum(), rtol=1e-12)


def test_gn_silu_input_goes_through_the_staging():
    """A GroupNorm + SiLU input is activated and re-quantised per voxel and 32 channels before the taps, as in the 3x3x3 convs: the embedded
    3x3x3 stride-2 conv of the same input agrees value for value."""
    rng = np.random.default_rng(5)
    N, Ci, Co, D, H, W, G = 1, 64, 32, 4, 4, 4, 8
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32); w = (rng.standard_normal((Co, Ci, 8)) * 0.2).astype(np.float32)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    g = orc.gn(rng.uniform(.5, 1.5, Ci).astype(np.float32), rng.uniform(-.3, .3, Ci).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.7, 1.4, N * G).astype(np.float32), G)
    got = orc.conv2(xq, 3, N, Ci, D, H, W, w, None, Co, 3, 0, cbits=8, gp=g, acc64=1)
    w3 = np.zeros((Co, Ci, 3, 3, 3), np.float32); w3[:, :, 1:, 1:, 1:] = w.reshape(Co, Ci, 2, 2, 2)
    y3, _ = orc.conv3(xq, 3, N, Ci, D, H, W, np.ascontiguousarray(w3.reshape(Co, Ci, 27)), None, Co, 3, cbits=8, stride=2, gp=g, acc64=1)
    assert np.array_equal(got, y3)
