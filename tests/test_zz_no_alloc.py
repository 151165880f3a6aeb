"""The conv entry point that allocates nothing (mi_conv_fwd_static) against the allocating one (lp_conv_fwd_f8 / _f4) through the C ABI:
byte-identical outputs and statistics on calls in a row that share the fixed scratch, each smaller or differently shaped than the one before."""
import numpy as np
import pytest

import orc
from gpuutil import dev_gn, lib, LP, DevBuf, shape5, gnp_t, split_t

pytestmark = pytest.mark.gpu


def run_both(rng, bits, N, Ci, Co, D, H, W, gn=False, up=0, Cu=0, G=8):
    S = D * H * W
    dt = 3 if bits == 8 else 4
    w = (rng.standard_normal((Co, Ci, 27)) * np.sqrt(2.0 / (Ci * 27))).astype(np.float32)
    b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    dw, db = DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    sp = split_t(); keep = []
    if up:
        Cs = Ci - Cu
        dx = DevBuf.from_numpy(orc.f32_to_mx(bits, rng.standard_normal((N, Cu, S // 8)).astype(np.float32), N, Cu, S // 8))
        dx2 = DevBuf.from_numpy(orc.f32_to_mx(bits, rng.standard_normal((N, Cs, S)).astype(np.float32), N, Cs, S))
        sp.x2, sp.c_split, sp.up = dx2.ptr, Cu, 1
        g1 = dev_gn(rng.uniform(.5, 1.5, Cu).astype(np.float32), rng.uniform(-.3, .3, Cu).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.7, 1.4, N * G).astype(np.float32), G)
        g2 = dev_gn(rng.uniform(.5, 1.5, Cs).astype(np.float32), rng.uniform(-.3, .3, Cs).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.7, 1.4, N * G).astype(np.float32), G)
        sp.gp2 = g2; keep += [dx2, g2]
    else:
        dx = DevBuf.from_numpy(orc.f32_to_mx(bits, rng.standard_normal((N, Ci, S)).astype(np.float32), N, Ci, S))
        g1 = dev_gn(rng.uniform(.5, 1.5, Ci).astype(np.float32), rng.uniform(-.3, .3, Ci).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.7, 1.4, N * G).astype(np.float32), G) if gn else gnp_t()
    ybytes = orc.mx_bytes(bits, N, Co, S)
    xs = shape5(N, Ci, D, H, W)
    ya, sa = DevBuf(ybytes), DevBuf(N * G * 2 * 24)
    lib.mi_gn_sums_zero(sa.ptr, 2 * N * G)
    f = lib.lp_conv_fwd_f8 if bits == 8 else lib.lp_conv_fwd_f4
    assert f(dx.ptr, dt, xs, dw.ptr, db.ptr, Co, ya.ptr, dt, g1, sa.ptr, G, sp) == 0
    ka = lib.mi_last_kernel().decode()
    LP.check()
    yb, sb = DevBuf(ybytes), DevBuf(N * G * 2 * 24)
    lib.mi_gn_sums_zero(sb.ptr, 2 * N * G)
    lib.mi_sync()
    n0 = lib.mi_alloc_count()
    assert lib.mi_conv_fwd_static(bits, dx.ptr, dt, xs, dw.ptr, db.ptr, Co, yb.ptr, dt, g1, sb.ptr, G, sp) == 0
    assert lib.mi_alloc_count() == n0, "the entry point allocated device memory"
    kb = lib.mi_last_kernel().decode()
    LP.check()
    assert ka == kb
    assert np.array_equal(ya.to_numpy(np.uint8), yb.to_numpy(np.uint8)), ka
    assert np.array_equal(sa.to_numpy(np.uint8), sb.to_numpy(np.uint8)), ka
    return ka


def test_static_scratch_conv_equals_the_allocating_entry(gpu):
    rng = np.random.default_rng(2024)
    assert lib.mi_conv_static_scratch_bytes() == 64 << 20
    names = []
    # calls in a row on the shared array, every one smaller than or unlike the one before: wide kernel with a re-staged GroupNorm input,
    # then a smaller direct input, a fused-upsample split input (coarse rows + two staged segments), the same on rows of 32 voxels and a
    # 32 -> 32 conv (the row kernels), the small-channel kernel, the tap-packed stem, an MX-fp4 conv, and the first shape again
    names.append(run_both(rng, 8, 2, 128, 128, 16, 32, 32, gn=True))
    names.append(run_both(rng, 8, 1, 128, 128, 8, 16, 32))
    names.append(run_both(rng, 8, 1, 96, 32, 8, 16, 16, up=1, Cu=64))
    names.append(run_both(rng, 8, 1, 96, 32, 8, 16, 32, up=1, Cu=64))
    names.append(run_both(rng, 8, 2, 32, 32, 8, 16, 32, gn=True))
    names.append(run_both(rng, 8, 1, 32, 32, 8, 16, 16, gn=True))
    names.append(run_both(rng, 8, 2, 4, 32, 6, 16, 16, G=8))
    names.append(run_both(rng, 4, 1, 64, 64, 4, 8, 16, gn=True))
    names.append(run_both(rng, 8, 2, 128, 128, 16, 32, 32, gn=True))
    assert any("conv3_wide_k" in n for n in names) and any("conv3_row_k" in n for n in names) and any("conv3_row1_k" in n for n in names) and any("conv3_small_k" in n for n in names) and any("conv3_stem_k" in n for n in names)


def test_static_scratch_conv_refuses_what_does_not_fit(gpu):
    """A GroupNorm input of 138 MB needs a re-staged copy larger than the fixed scratch: refused with -1, nothing launched, nothing allocated;
    the same tensor without GroupNorm (read as stored) needs only its weights and runs."""
    rng = np.random.default_rng(7)
    N, C, D = 2, 32, 128
    S = D ** 3
    dx = DevBuf(lib.lp_mx8_bytes(N, C, S)); dy = DevBuf(lib.lp_mx8_bytes(N, C, S))
    w = (rng.standard_normal((C, C, 27)) * 0.05).astype(np.float32)
    dw = DevBuf.from_numpy(w)
    G = 8
    g = dev_gn(np.ones(C, np.float32), np.zeros(C, np.float32), np.zeros(N * G, np.float32), np.ones(N * G, np.float32), G)
    n0 = lib.mi_alloc_count()
    assert lib.mi_conv_fwd_static(8, dx.ptr, 3, shape5(N, C, D, D, D), dw.ptr, None, C, dy.ptr, 3, g, None, 0, split_t()) == -1
    assert lib.mi_conv_fwd_static(8, dx.ptr, 3, shape5(N, C, D, D, D), dw.ptr, None, C, dy.ptr, 3, gnp_t(), None, 0, split_t()) == 0
    LP.check()
    assert lib.mi_alloc_count() == n0
    # a few-channel fp32 network input goes to the tap-packed kernel, which reads it as stored and stages nothing: a whole 2 x 128^3 window fits
    dx4 = DevBuf(N * 4 * S * 4); w4 = DevBuf.from_numpy((rng.standard_normal((C, 4, 27)) * 0.1).astype(np.float32))
    n1 = lib.mi_alloc_count()
    assert lib.mi_conv_fwd_static(8, dx4.ptr, 0, shape5(N, 4, D, D, D), w4.ptr, None, C, dy.ptr, 3, gnp_t(), None, 0, split_t()) == 0
    LP.check()
    assert lib.mi_alloc_count() == n1 and "conv3_stem_k" in lib.mi_last_kernel().decode()
    assert lib.mi_conv_fwd_static(5, dx.ptr, 3, shape5(N, C, D, D, D), dw.ptr, None, C, dy.ptr, 3, gnp_t(), None, 0, split_t()) == -1
