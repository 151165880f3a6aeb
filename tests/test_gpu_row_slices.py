"""The row kernels with two channel slices (33 .. 64 output channels from one to three input blocks: one slice per workgroup, the one-block
kernel for a single input block): exact operands equal the oracle in every output type, random operands meet the conv tolerance, the statistics
are the oracle's and identical run to run."""
import numpy as np
import pytest

from ufsm_amd import lib
import orc
from test_gpu_conv import exact_case, rand_case, gpu_conv, code_mismatch_fraction

pytestmark = pytest.mark.gpu

ROW_CS_SHAPES = [(8, 2, 32, 128, 16, 32, 64), (4, 1, 32, 96, 6, 9, 40),      # four (three) slices: the one-block kernel
                 (8, 2, 32, 64, 8, 16, 32), (8, 1, 32, 48, 5, 9, 40), (4, 1, 32, 64, 8, 12, 48), (8, 2, 32, 64, 64, 64, 64), (8, 3, 32, 64, 12, 64, 128), (4, 2, 20, 40, 6, 9, 34),
                 (8, 1, 64, 64, 8, 12, 20), (8, 2, 64, 64, 16, 16, 64), (8, 1, 96, 48, 5, 9, 40), (4, 1, 64, 64, 8, 12, 48), (4, 2, 96, 64, 6, 9, 34),
                 (8, 2, 64, 64, 64, 64, 64), (4, 3, 64, 40, 12, 64, 128)]


@pytest.mark.parametrize("bits,N,Ci,Co,D,H,W", ROW_CS_SHAPES)
def test_row_kernel_two_channel_slices(gpu, bits, N, Ci, Co, D, H, W):
    rng = np.random.default_rng(Ci * 5 + Co + D + W)
    S = D * H * W
    xdt = 3 if bits == 8 else 4
    x, w, b = exact_case(rng, N, Ci, Co, S)
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    want, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, acc64=1)
    got, _ = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits)
    assert "channel slices" in lib.mi_last_kernel().decode(), lib.mi_last_kernel().decode()
    assert np.array_equal(got, want)
    for ydt in (2, 3, 4):
        wq, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, ydt, cbits=bits, acc64=1)
        gq, _ = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, ydt, cbits=bits)
        assert np.array_equal(gq, wq), ydt
    if S * N > 600000:                                            # (the large cases: exact operands only)
        return
    x, w, b = rand_case(rng, N, Ci, Co, S)
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    G = 8 if Co % 32 == 0 else 2                                  # (channels per group a multiple of 4, or the launch leaves this kernel)
    want, ws = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, Go=G, want_stats=True)
    got, gs = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, Go=G, stats=True)
    assert "channel slices" in lib.mi_last_kernel().decode()
    assert np.abs(got - want).max() / np.abs(want).max() < 2e-4
    assert np.abs(gs - ws).max() / np.abs(ws).max() < 1e-5
    got2, gs2 = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, Go=G, stats=True)
    assert np.array_equal(got, got2) and np.array_equal(gs, gs2)


@pytest.mark.parametrize("Ci", [32, 64])
def test_fused_activation_epilogue_on_the_sliced_kernels(gpu, Ci):
    """mi_conv_fwd_fused on 64 output channels: each slice's workgroups take their own 32 affine pairs and biases."""
    rng = np.random.default_rng(61 + Ci)
    N, Co, D, H, W = 2, 64, 8, 16, 32
    S = D * H * W
    x, w, b = rand_case(rng, N, Ci, Co, S)
    ea = rng.uniform(0.5, 1.5, Co).astype(np.float32); eb = rng.uniform(-.5, .5, Co).astype(np.float32)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    for act in (1, 2, 3):
        want, _ = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 0, fused_act=act, ep_a=ea, ep_b=eb)
        got, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, b, Co, 0, fused=(act, ea, eb))
        assert "two channel slices" in lib.mi_last_kernel().decode(), lib.mi_last_kernel().decode()
        assert np.abs(got - want).max() / np.abs(want).max() < 1e-4
        wq, _ = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 3, fused_act=act, ep_a=ea, ep_b=eb)
        gq, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, b, Co, 3, fused=(act, ea, eb))
        frac, near = code_mismatch_fraction(8, gq, wq, N, Co, S)
        assert frac < 5e-3 and near


@pytest.mark.parametrize("gn", [False, True])
def test_decoder_conv_with_split_input_on_the_sliced_kernel(gpu, gn):
    """A decoder conv1 with 64 output channels, [up2(silu(gn(coarse 32))) | silu(gn(skip 64))] -> 64: three input blocks in two segments, the upsampled
    one blended by the pre-pass, each channel slice on its own workgroups (exact operands without the GroupNorm, the conv tolerance with it)."""
    import refnp
    from gpuutil import dev_gn
    rng = np.random.default_rng(77)
    Cu, Cs, Co, D, H, W = 32, 64, 64, 8, 16, 32
    N, S, Sc, G = 2, D * H * W, (D // 2) * (H // 2) * (W // 2), 8
    exact = not gn
    xa = refnp.gen_exact(rng, (N, Cu, Sc)) if exact else rng.standard_normal((N, Cu, Sc)).astype(np.float32)
    xb = refnp.gen_exact(rng, (N, Cs, S)) if exact else rng.standard_normal((N, Cs, S)).astype(np.float32)
    w = refnp.gen_exact(rng, (Co, Cu + Cs, 27)) if exact else (rng.standard_normal((Co, Cu + Cs, 27)) * 0.05).astype(np.float32)
    qa, qb = orc.f32_to_mx(8, xa, N, Cu, Sc), orc.f32_to_mx(8, xb, N, Cs, S)
    p = [rng.uniform(0.5, 1.5, Cu).astype(np.float32), rng.uniform(-.5, .5, Cu).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    p2 = [rng.uniform(0.5, 1.5, Cs).astype(np.float32), rng.uniform(-.5, .5, Cs).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    want, _ = orc.conv3(qa, 3, N, Cu + Cs, D, H, W, w, None, Co, 0, x2=qb, c_split=Cu, up=1, gp=orc.gn(*p, G) if gn else None, gp2=orc.gn(*p2, G) if gn else None)
    got, _ = gpu_conv(qa, 3, N, Cu + Cs, D, H, W, w, None, Co, 0, x2=qb, c_split=Cu, up=1, gp=dev_gn(*p, G) if gn else None, gp2=dev_gn(*p2, G) if gn else None)
    assert "conv3_row_k" in lib.mi_last_kernel().decode() and "two channel slices" in lib.mi_last_kernel().decode(), lib.mi_last_kernel().decode()
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < (1e-5 if exact else 3e-3)
