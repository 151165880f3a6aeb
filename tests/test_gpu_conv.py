"""GPU parity of the 3x3x3 MX convolutions through the C ABI (lp_conv_fwd_f8 / _f4 / _s2_f8) against the oracle.

Bars: exact-operand cases (tests/test_mx4_wide.c:81-98) are bit-exact / byte-identical; random data within 1e-3 max-abs-rel of the
oracle's fp32-accumulated result (the north-star tolerance; measured about 2e-5), MX outputs byte-identical except rounding flips to a
neighbouring code caused by the last bits of the fp32 sum; GroupNorm sums within 1e-5 relative (the reference accepts 1e-4,
tests/test_mx4.c:293-318). Shapes follow the reference's own test matrix (tests/test_mx.c, tests/test_mx4.c, tests/test_mx4_wide.c)."""
import numpy as np
import pytest

import orc
import refnp
from gpuutil import gpu_conv, dev_gn, code_mismatch_fraction, out_dims, lib, LP, DevBuf, to_mx, shape5, gnp_t, split_t

pytestmark = pytest.mark.gpu
GRID = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], np.float32)


def rand_case(rng, N, Ci, Co, S):
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci, 27)) * np.sqrt(2.0 / (Ci * 27))).astype(np.float32)       # Kaiming normal (src/unet.c:588-607)
    b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    return x, w, b


def exact_case(rng, N, Ci, Co, S):
    return refnp.gen_exact(rng, (N, Ci, S)), refnp.gen_exact(rng, (Co, Ci, 27)), (GRID[rng.integers(0, 8, Co)] * 0.25).astype(np.float32)


# (bits, N, Ci, Co, D, H, W, stride): ragged W = 20 (tests/test_mx.c:34-45), partial tiles (tests/test_mx4.c:727-760), wide channel
# counts with odd block counts (tests/test_mx4_wide.c:741-745), stride-2 odd dims (tests/test_mx.c:159-199)
# the wide kernel (128-channel output slices, stride 1): odd and even block counts, several output slices, ragged tiles, depths that
# are not a multiple of its 4-deep tile, more tiles than workgroups (persistent walk), fp4
WIDE_SHAPES = [(8, 1, 96, 128, 5, 9, 18), (8, 1, 32, 128, 3, 8, 16), (8, 2, 128, 256, 6, 10, 33), (8, 1, 384, 128, 4, 8, 16), (8, 3, 64, 128, 9, 17, 40),
               (4, 1, 160, 128, 7, 8, 16), (4, 2, 64, 256, 4, 16, 16)]


@pytest.fixture(params=[0, 1 << 30], ids=["slices128", "slices64"])
def slice_split(request):
    """Launches of few tiles run as slices of 64 channels (two channel tiles per workgroup) when the tile count is under the split; 0 keeps the
    slices of 128 (four channel tiles, the form the large layers run in): both forms of the wide kernel see every shape."""
    lib.mi_conv_split(request.param)
    yield request.param
    lib.mi_conv_split(-1)


@pytest.mark.parametrize("bits,N,Ci,Co,D,H,W", WIDE_SHAPES)
def test_wide_kernel_exact(gpu, slice_split, bits, N, Ci, Co, D, H, W):
    rng = np.random.default_rng(Ci * 17 + Co + D * 3 + bits)
    S = D * H * W
    x, w, b = exact_case(rng, N, Ci, Co, S)
    xdt = 3 if bits == 8 else 4
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    want, wsum = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, acc64=1, Go=8, want_stats=True)
    got, gsum = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, Go=8, stats=True)
    name = lib.mi_last_kernel().decode()
    assert "conv3_wide_k" in name and ("MT 2" in name) == (slice_split != 0)
    assert np.array_equal(got, want)
    assert np.allclose(gsum, wsum, rtol=1e-6)
    wf, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, acc64=1)
    gf, _ = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits)
    assert np.array_equal(gf, wf)


@pytest.mark.parametrize("bits,N,Ci,Co,D,H,W", WIDE_SHAPES[:3] + WIDE_SHAPES[5:])
def test_few_tiles_default_dispatch(gpu, bits, N, Ci, Co, D, H, W):
    """The default rule for launches of very few tiles (the coarsest levels): one channel tile and two planes per workgroup on the general
    kernel instead of the wide kernel's slices."""
    rng = np.random.default_rng(Ci * 19 + Co + D * 5 + bits)
    S = D * H * W
    x, w, b = exact_case(rng, N, Ci, Co, S)
    xdt = 3 if bits == 8 else 4
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    want, wsum = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, acc64=1, Go=8, want_stats=True)
    got, gsum = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, Go=8, stats=True)
    name = lib.mi_last_kernel().decode()
    assert "conv3_mx_k" in name and "MT 1, NT 2" in name, name
    assert np.array_equal(got, want)
    assert np.allclose(gsum, wsum, rtol=1e-6)


@pytest.mark.parametrize("Ci,Co,split", [(32, 128, 0), (64, 128, 0), (32, 128, 1 << 30)])
def test_wide_kernel_persistent_walk_few_blocks(gpu, Ci, Co, split):
    """More tiles than workgroups (every workgroup walks two or four tiles) on inputs of one and two blocks, slices of 128 and of 64 channels:
    the blocks of a workgroup's next tile are requested while the current one is multiplied, whatever the block count (a one-block input
    has only the next tile's block to request)."""
    rng = np.random.default_rng(Ci + Co)
    N, D, H, W = 2, 32, 64, 64
    S = D * H * W
    x, w, b = exact_case(rng, N, Ci, Co, S)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    lib.mi_conv_split(split)
    try:
        got, gsum = gpu_conv(xq, 3, N, Ci, D, H, W, w, b, Co, 3, cbits=8, Go=8, stats=True)
    finally:
        lib.mi_conv_split(-1)
    name = lib.mi_last_kernel().decode()
    assert "conv3_wide_k" in name and ("tiles 1024 wgs 256" if split else "tiles 512 wgs 256") in name and ("MT 2" in name) == (split != 0)
    want, wsum = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 3, cbits=8, acc64=1, Go=8, want_stats=True)
    assert np.array_equal(got, want)
    assert np.allclose(gsum, wsum, rtol=1e-6)


def test_wide_kernel_decoder_conv(gpu):
    """[2x upsampled coarse | skip] -> 128 channels with both GroupNorms: the wide kernel on a split, restaged input (12 blocks)."""
    rng = np.random.default_rng(77)
    Cu, Cs, Co, (D, H, W) = 256, 128, 128, (4, 8, 16)
    S, Sc = D * H * W, D * H * W // 8
    xu = rng.standard_normal((1, Cu, Sc)).astype(np.float32); xs = rng.standard_normal((1, Cs, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Cu + Cs, 27)) * np.sqrt(2.0 / ((Cu + Cs) * 27))).astype(np.float32)
    b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    qu, qs = orc.f32_to_mx(8, xu, 1, Cu, Sc), orc.f32_to_mx(8, xs, 1, Cs, S)
    G = 8
    g1 = [rng.uniform(0.5, 1.5, Cu).astype(np.float32), rng.uniform(-0.3, 0.3, Cu).astype(np.float32), rng.uniform(-0.2, 0.2, G).astype(np.float32), rng.uniform(0.7, 1.4, G).astype(np.float32)]
    g2 = [rng.uniform(0.5, 1.5, Cs).astype(np.float32), rng.uniform(-0.3, 0.3, Cs).astype(np.float32), rng.uniform(-0.2, 0.2, G).astype(np.float32), rng.uniform(0.7, 1.4, G).astype(np.float32)]
    want, _ = orc.conv3(qu, 3, 1, Cu + Cs, D, H, W, w, b, Co, 0, x2=qs, c_split=Cu, up=1, gp=orc.gn(*g1, G=G), gp2=orc.gn(*g2, G=G))
    for split, kern in ((1 << 30, "conv3_wide_k"), (-1, "conv3_mx_k")):       # forced slices of 64 on the wide kernel; the default for so few tiles
        lib.mi_conv_split(split)
        try:
            got, _ = gpu_conv(qu, 3, 1, Cu + Cs, D, H, W, w, b, Co, 0, x2=qs, c_split=Cu, up=1, gp=dev_gn(*g1, G), gp2=dev_gn(*g2, G))
        finally:
            lib.mi_conv_split(-1)
        assert kern in lib.mi_last_kernel().decode()
        assert np.abs(got - want).max() / np.abs(want).max() < 1e-3


EXACT_SHAPES = [
    (8, 1, 32, 32, 2, 8, 16, 1), (8, 2, 32, 32, 5, 9, 18, 1), (8, 1, 64, 64, 8, 12, 20, 1), (8, 2, 128, 128, 4, 12, 20, 1), (8, 1, 96, 32, 6, 12, 20, 1),
    (8, 1, 160, 96, 3, 8, 16, 1), (8, 1, 256, 320, 4, 8, 16, 1), (8, 1, 32, 16, 5, 9, 18, 1), (8, 1, 48, 40, 4, 7, 9, 1),
    (4, 1, 32, 32, 16, 12, 16, 1), (4, 1, 32, 64, 8, 12, 16, 1), (4, 1, 256, 256, 6, 10, 14, 1), (4, 1, 288, 288, 6, 6, 6, 1), (4, 2, 64, 64, 4, 8, 16, 1),
    (8, 1, 32, 32, 16, 16, 16, 2), (8, 1, 64, 64, 13, 10, 17, 2), (8, 2, 128, 128, 8, 16, 32, 2), (4, 1, 32, 32, 16, 16, 16, 2), (8, 1, 96, 96, 12, 10, 14, 2),
]


# the stride-2 kernel that reads the taps' rows from the stored tensor (large launches take it by default): odd and even dims, one to five
# input blocks, 32 / 64 / 128 / 96 output channels, both formats (fp4 compute only for 32 -> <= 32 on even dims, src/lp_s2.cu:647-754)
S2_DIRECT_SHAPES = [(8, 1, 32, 32, 16, 16, 16), (8, 1, 64, 64, 13, 10, 17), (8, 2, 128, 128, 8, 16, 32), (4, 1, 32, 32, 16, 16, 16), (8, 1, 96, 96, 12, 10, 14),
                    (8, 2, 160, 64, 5, 7, 33), (4, 1, 64, 128, 6, 12, 20), (8, 1, 32, 40, 3, 5, 7)]


@pytest.mark.parametrize("mode", [0, 1], ids=["general", "direct"])
@pytest.mark.parametrize("bits,N,Ci,Co,D,H,W", S2_DIRECT_SHAPES)
def test_stride2_kernels_exact(gpu, mode, bits, N, Ci, Co, D, H, W):
    rng = np.random.default_rng(Ci * 31 + Co * 5 + D)
    S = D * H * W
    x, w, b = exact_case(rng, N, Ci, Co, S)
    xdt = 3 if bits == 8 else 4
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    cb = 4 if bits == 4 and Ci == 32 and Co <= 32 and not (D | H | W) & 1 else 8      # the compute format the entry point picks
    lib.mi_conv_s2_direct(mode)
    try:
        for ydt in (0, 2, xdt):                                   # fp32 / fp16 planes == the exact host conv; the MX output byte-identical
            want, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, ydt, cbits=cb, stride=2, acc64=1)
            got, _ = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, ydt, cbits=cb, stride=2)
            assert ("conv3s2_mx_k" in lib.mi_last_kernel().decode()) == (mode == 1), lib.mi_last_kernel().decode()
            assert np.array_equal(got, want), ydt
    finally:
        lib.mi_conv_s2_direct(-1)


def test_stride2_direct_kernel_groupnorm_input(gpu):
    """The direct kernel behind lp_conv_fwd_s2_f8 with a GroupNorm + SiLU input (re-staged once); random data against the oracle's fp32 result."""
    rng = np.random.default_rng(91)
    N, Ci, Co, D, H, W, G = 2, 64, 64, 32, 32, 64, 8
    S = D * H * W
    x, w, b = rand_case(rng, N, Ci, Co, S)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    p = [rng.uniform(.5, 1.5, Ci).astype(np.float32), rng.uniform(-.3, .3, Ci).astype(np.float32)]
    mean, rstd = rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.7, 1.4, N * G).astype(np.float32)
    want, _ = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 0, cbits=8, stride=2, gp=orc.gn(p[0], p[1], mean, rstd, G), acc64=0)
    lib.mi_conv_s2_direct(1)
    try:
        got, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, b, Co, 0, cbits=8, stride=2, gp=dev_gn(p[0], p[1], mean, rstd, G))
    finally:
        lib.mi_conv_s2_direct(-1)
    assert "conv3s2_mx_k" in lib.mi_last_kernel().decode()
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-2


@pytest.mark.parametrize("bits,N,Ci,Co,D,H,W,stride", EXACT_SHAPES)
def test_exact_operand_conv(gpu, bits, N, Ci, Co, D, H, W, stride):
    rng = np.random.default_rng(Ci * 131 + Co * 7 + D + stride)
    S = D * H * W
    x, w, b = exact_case(rng, N, Ci, Co, S)
    xdt = 3 if bits == 8 else 4
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    want, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride, acc64=1)
    got, _ = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride)
    assert np.array_equal(got, want)                              # fp32 output == exact host conv, whatever the MFMA's summation order
    got16, _ = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 2, cbits=bits, stride=stride)
    want16, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, 2, cbits=bits, stride=stride, acc64=1)
    assert np.array_equal(got16, want16)
    for ydt in (3, 4):                                            # MX outputs of either format: byte-identical to the host quantiser
        if stride == 2 and ydt != xdt:
            continue
        wq, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, ydt, cbits=bits, stride=stride, acc64=1)
        gq, _ = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, ydt, cbits=bits, stride=stride)
        assert np.array_equal(gq, wq)


# (the last two: columns of three z tiles and four tiles per workgroup, so a workgroup's walk crosses column ends - the halo ring restarts -
# and the XCDs' ranges start and end inside columns; six tiles per workgroup on columns of five with a ragged last plane)
ROW1_SHAPES = [(8, 2, 32, 32, 8, 16, 32), (8, 1, 32, 32, 5, 9, 40), (8, 1, 20, 24, 7, 10, 33), (8, 2, 32, 32, 64, 64, 64),
               (4, 1, 32, 32, 8, 12, 48), (4, 2, 32, 24, 6, 9, 34), (4, 1, 32, 32, 32, 64, 128),
               (8, 3, 32, 32, 12, 64, 128), (4, 3, 32, 24, 12, 64, 128), (8, 6, 32, 32, 19, 72, 160)]


@pytest.mark.parametrize("bits,N,Ci,Co,D,H,W", ROW1_SHAPES)
def test_one_block_row_kernel(gpu, bits, N, Ci, Co, D, H, W):
    """The one-input-block row kernel (17 .. 32 output channels from <= 32 input channels on volumes wider than 16 voxels; the two halves of
    its workgroups run half a tile apart and keep their statistics per wavefront): exact operands equal the oracle in every output type, ragged
    tiles and more tiles than workgroups included (the persistent walk's double buffer); random operands meet the conv tolerance, the statistics
    are those of the oracle and identical run to run."""
    rng = np.random.default_rng(Ci * 5 + Co + D + W)
    S = D * H * W
    xdt = 3 if bits == 8 else 4
    x, w, b = exact_case(rng, N, Ci, Co, S)
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    want, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, acc64=1)
    got, _ = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits)
    assert "conv3_row1_k" in lib.mi_last_kernel().decode(), lib.mi_last_kernel().decode()
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
    assert "conv3_row1_k" in lib.mi_last_kernel().decode()
    assert np.abs(got - want).max() / np.abs(want).max() < 2e-4
    assert np.abs(gs - ws).max() / np.abs(ws).max() < 1e-5
    gq, gs2 = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, Go=G, stats=True, stored_stats=1)
    dec = orc.mx_to_f32(bits, gq, N, Co, S).astype(np.float64).reshape(N, G, -1)
    assert np.allclose(gs2[:, :, 0], dec.sum(-1), rtol=1e-5, atol=1e-3) and np.allclose(gs2[:, :, 1], (dec * dec).sum(-1), rtol=1e-5)
    gq2, gs3 = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, Go=G, stats=True, stored_stats=1)
    assert np.array_equal(gq, gq2) and np.array_equal(gs2, gs3)


RANDOM_SHAPES = [(8, 2, 32, 16, 8, 16, 16, 1), (8, 1, 16, 24, 4, 8, 16, 1), (8, 2, 32, 32, 8, 16, 16, 1), (8, 1, 128, 128, 6, 12, 20, 1), (8, 1, 64, 64, 8, 8, 24, 1), (4, 1, 256, 256, 4, 8, 16, 1), (4, 1, 32, 32, 8, 16, 16, 1),
                 (8, 1, 64, 64, 12, 10, 14, 2), (8, 1, 80, 48, 5, 9, 18, 1),
                 # channels per group that are not a multiple of 4 on more than one channel tile: 80 / 8 = 10 (the reference's 16/32/64/80 nets)
                 (8, 2, 64, 80, 5, 9, 18, 1), (4, 1, 80, 80, 4, 8, 16, 1), (8, 1, 160, 200, 3, 8, 16, 1)]


@pytest.mark.parametrize("bits,N,Ci,Co,D,H,W,stride", RANDOM_SHAPES)
def test_random_conv_tolerance_and_stats(gpu, bits, N, Ci, Co, D, H, W, stride):
    rng = np.random.default_rng(Ci + Co * 3 + bits)
    S = D * H * W
    x, w, b = rand_case(rng, N, Ci, Co, S)
    xdt = 3 if bits == 8 else 4
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    G = 8
    stats = stride == 1                                            # (any group size: channels per group that are not a multiple of 4 take per-channel records)
    want, ws = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride, Go=G, want_stats=stats)
    got, gs = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, stride=stride, Go=G, stats=stats)
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-3          # north-star tolerance on the fp32-accumulated result
    assert np.abs(got - want).max() / np.abs(want).max() < 2e-4          # what the block-scaled MFMA actually delivers
    if stats:
        assert np.abs(gs - ws).max() / np.abs(ws).max() < 1e-5
    Do, Ho, Wo = out_dims(D, H, W, stride)
    wq, ws2 = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, stride=stride, Go=G, want_stats=stats, stored_stats=1)
    gq, gs2 = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, stride=stride, Go=G, stats=stats, stored_stats=1)
    frac, near = code_mismatch_fraction(bits, gq, wq, N, Co, Do * Ho * Wo)
    assert frac < 5e-3 and near
    if stats:                                                     # statistics of the decoded stored tensor (tests/test_gn_contract.c)
        dec = orc.mx_to_f32(bits, gq, N, Co, Do * Ho * Wo).astype(np.float64).reshape(N, G, -1)
        assert np.allclose(gs2[:, :, 0], dec.sum(-1), rtol=1e-5, atol=1e-3) and np.allclose(gs2[:, :, 1], (dec * dec).sum(-1), rtol=1e-5)
    # run to run: byte-identical outputs and identical statistics (deterministic reduction order)
    gq2, gs3 = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, stride=stride, Go=G, stats=stats, stored_stats=1)
    assert np.array_equal(gq, gq2) and (not stats or np.array_equal(gs2, gs3))


@pytest.mark.parametrize("bits,xdt", [(8, 3), (4, 4), (4, 3), (8, 4), (8, 0), (8, 2)])
def test_gn_silu_input_staging(gpu, bits, xdt):
    """The consumer applies GroupNorm + SiLU while staging (src/lp_common.cuh:413-431); any stored format feeds either compute format."""
    rng = np.random.default_rng(20 + bits + xdt)
    N, Ci, Co, D, H, W, G = 2, 64, 32, 4, 8, 16, 8
    S = D * H * W
    x, w, b = rand_case(rng, N, Ci, Co, S)
    gam = rng.uniform(0.5, 1.5, Ci).astype(np.float32); bet = rng.uniform(-.5, .5, Ci).astype(np.float32)
    mean = rng.uniform(-.2, .2, N * G).astype(np.float32); rstd = rng.uniform(.8, 1.2, N * G).astype(np.float32)
    if xdt >= 3:
        xin = orc.f32_to_mx(8 if xdt == 3 else 4, x, N, Ci, S)
    elif xdt == 2:
        xin = np.ascontiguousarray(x.astype(np.float16).view(np.uint16))
    else:
        xin = x
    want, _ = orc.conv3(xin, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, gp=orc.gn(gam, bet, mean, rstd, G))
    got, _ = gpu_conv(xin, xdt, N, Ci, D, H, W, w, b, Co, 0, cbits=bits, gp=dev_gn(gam, bet, mean, rstd, G))
    # the sigmoid runs on the hardware's fast exponential: a few staged codes land on the neighbour (the reference's own acceptance,
    # tests/test_mx4_wide.c:165-175); measured at the conv output that is a small relative error, larger for the 8-value fp4 grid
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < (3e-3 if bits == 8 else 3e-2)


def test_plain_input_without_gn_is_bit_exact_vs_converter(gpu):
    rng = np.random.default_rng(31)
    N, Ci, Co, D, H, W = 1, 64, 32, 4, 8, 16
    S = D * H * W
    x, w, b = rand_case(rng, N, Ci, Co, S)
    g0, _ = gpu_conv(x, 0, N, Ci, D, H, W, w, b, Co, 3)
    g1, _ = gpu_conv(orc.f32_to_mx(8, x, N, Ci, S), 3, N, Ci, D, H, W, w, b, Co, 3)
    assert np.array_equal(g0, g1)


@pytest.mark.parametrize("bits,Cu,Cs,Co,dims,gn", [(8, 32, 32, 32, (4, 8, 16), False), (8, 64, 32, 32, (4, 8, 16), True), (8, 80, 64, 64, (8, 8, 12), True),
                                                   (4, 64, 32, 32, (4, 8, 16), False), (8, 32, 16, 16, (12, 12, 16), True)])
def test_decoder_conv_split_input(gpu, bits, Cu, Cs, Co, dims, gn):
    """Decoder conv1: channels [0, Cu) from x, the rest from x2, each with its own GroupNorm (tests/test_mx.c:138-156)."""
    rng = np.random.default_rng(40 + Cu + Cs)
    D, H, W = dims
    N, S, G = 1, D * H * W, 8
    xa = rng.standard_normal((N, Cu, S)).astype(np.float32); xb = rng.standard_normal((N, Cs, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Cu + Cs, 27)) * np.sqrt(2.0 / ((Cu + Cs) * 27))).astype(np.float32); b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    xdt = 3 if bits == 8 else 4
    qa, qb = orc.f32_to_mx(bits, xa, N, Cu, S), orc.f32_to_mx(bits, xb, N, Cs, S)
    p = [rng.uniform(0.5, 1.5, Cu).astype(np.float32), rng.uniform(-.5, .5, Cu).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    p2 = [rng.uniform(0.5, 1.5, Cs).astype(np.float32), rng.uniform(-.5, .5, Cs).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    want, _ = orc.conv3(qa, xdt, N, Cu + Cs, D, H, W, w, b, Co, 0, cbits=bits, x2=qb, c_split=Cu, gp=orc.gn(*p, G) if gn else None, gp2=orc.gn(*p2, G) if gn else None)
    got, _ = gpu_conv(qa, xdt, N, Cu + Cs, D, H, W, w, b, Co, 0, cbits=bits, x2=qb, c_split=Cu, gp=dev_gn(*p, G) if gn else None, gp2=dev_gn(*p2, G) if gn else None)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < (2e-4 if not gn else 3e-3 if bits == 8 else 3e-2)


@pytest.mark.parametrize("Cu,Cs,Co,dims,gn", [(32, 32, 32, (4, 8, 16), False), (64, 32, 32, (8, 8, 16), True), (32, 16, 16, (12, 12, 16), True)])
def test_decoder_conv_fused_upsample(gpu, Cu, Cs, Co, dims, gn):
    """Decoder conv1 reading [up2(silu(gn(coarse))) | silu(gn(skip))] without materialising the upsample (tests/test_mx.c:319+)."""
    rng = np.random.default_rng(50 + Cu)
    D, H, W = dims
    N, S, Sc, G = 1, D * H * W, (D // 2) * (H // 2) * (W // 2), 8
    exact = not gn
    xa = refnp.gen_exact(rng, (N, Cu, Sc)) if exact else rng.standard_normal((N, Cu, Sc)).astype(np.float32)
    if exact:
        xa[:, 5, :] = 6.0
    xb = refnp.gen_exact(rng, (N, Cs, S)) if exact else rng.standard_normal((N, Cs, S)).astype(np.float32)
    w = refnp.gen_exact(rng, (Co, Cu + Cs, 27)) if exact else (rng.standard_normal((Co, Cu + Cs, 27)) * 0.05).astype(np.float32)
    qa, qb = orc.f32_to_mx(8, xa, N, Cu, Sc), orc.f32_to_mx(8, xb, N, Cs, S)
    p = [rng.uniform(0.5, 1.5, Cu).astype(np.float32), rng.uniform(-.5, .5, Cu).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    p2 = [rng.uniform(0.5, 1.5, Cs).astype(np.float32), rng.uniform(-.5, .5, Cs).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    want, _ = orc.conv3(qa, 3, N, Cu + Cs, D, H, W, w, None, Co, 0, x2=qb, c_split=Cu, up=1, gp=orc.gn(*p, G) if gn else None, gp2=orc.gn(*p2, G) if gn else None)
    got, _ = gpu_conv(qa, 3, N, Cu + Cs, D, H, W, w, None, Co, 0, x2=qb, c_split=Cu, up=1, gp=dev_gn(*p, G) if gn else None, gp2=dev_gn(*p2, G) if gn else None)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < (1e-5 if exact else 3e-3)


def test_fused_activation_epilogue(gpu):
    """Extension (no reference counterpart): per-channel affine + SiLU / GELU / ReLU before the MX re-quantisation, pinned by fp64 closed forms."""
    rng = np.random.default_rng(60)
    N, Ci, Co, D, H, W = 1, 64, 64, 4, 8, 16
    S = D * H * W
    x, w, b = rand_case(rng, N, Ci, Co, S)
    ea = rng.uniform(0.5, 1.5, Co).astype(np.float32); eb = rng.uniform(-.5, .5, Co).astype(np.float32)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    lin, _ = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 0)
    for act in (1, 2, 3):
        want, _ = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 0, fused_act=act, ep_a=ea, ep_b=eb)
        got, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, b, Co, 0, fused=(act, ea, eb))
        assert np.abs(got - want).max() / np.abs(want).max() < 1e-4
        u = lin.astype(np.float64) * ea[None, :, None] + eb[None, :, None]
        from math import erf
        closed = {1: u / (1 + np.exp(-u)), 2: 0.5 * u * (1 + np.vectorize(erf)(u / np.sqrt(2))), 3: np.maximum(u, 0)}[act]
        assert np.abs(want - closed).max() / np.abs(closed).max() < 1e-5
        wq, _ = orc.conv3(xq, 3, N, Ci, D, H, W, w, b, Co, 3, fused_act=act, ep_a=ea, ep_b=eb)
        gq, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, b, Co, 3, fused=(act, ea, eb))
        frac, near = code_mismatch_fraction(8, gq, wq, N, Co, S)
        assert frac < 5e-3 and near


def test_weight_memo(gpu):
    rng = np.random.default_rng(70)
    N, Ci, Co, D, H, W = 1, 32, 32, 4, 8, 16
    S = D * H * W
    x, w, b = rand_case(rng, N, Ci, Co, S)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    dxq, dw, db = DevBuf.from_numpy(xq), DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    dy = DevBuf(lib.lp_mx8_bytes(N, Co, S))
    sp = split_t(); sp.wkey = 1234
    outs = []
    w2 = np.ascontiguousarray(2 * w)
    for step in (0, 0, 1):
        if step:                                                  # weights changed: a new step drops the memo (src/nn_lp.h:56)
            lib.mi_h2d(dw.ptr, w2.ctypes.data, w2.nbytes); lib.lp_wmemo_step(1)
        lib.lp_conv_fwd_f8(dxq.ptr, 3, shape5(N, Ci, D, H, W), dw.ptr, db.ptr, Co, dy.ptr, 3, gnp_t(), None, 0, sp)
        LP.check()
        outs.append(dy.to_numpy(np.uint8))
    assert np.array_equal(outs[0], outs[1]) and not np.array_equal(outs[0], outs[2])
    want, _ = orc.conv3(xq, 3, N, Ci, D, H, W, w2, b, Co, 3)
    assert code_mismatch_fraction(8, outs[2], want, N, Co, S)[0] < 5e-3
    lib.lp_wmemo_clear()


def test_weight_memo_keeps_layouts_apart(gpu):
    """One memoised 128 -> 128 conv (same weights, same wkey) at tile counts on either side of the slice-split threshold, and with the
    per-thread split knob toggled between calls: the wide kernel's weight image differs between its two forms (four or two channel tiles
    per workgroup), so each form must find its own prepared weights. Exact operands: every result equals the oracle."""
    rng = np.random.default_rng(71)
    Ci = Co = 128
    D, H, W = 16, 32, 64
    S = D * H * W
    w = refnp.gen_exact(rng, (Co, Ci, 27)); b = (GRID[rng.integers(0, 8, Co)] * 0.25).astype(np.float32)
    dw, db = DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    sp = split_t(); sp.wkey = 4321
    lib.lp_wmemo_clear()

    def run(N, xq):
        dxq = DevBuf.from_numpy(xq); dy = DevBuf(lib.lp_mx8_bytes(N, Co, S))
        assert lib.lp_conv_fwd_f8(dxq.ptr, 3, shape5(N, Ci, D, H, W), dw.ptr, db.ptr, Co, dy.ptr, 3, gnp_t(), None, 0, sp) == 0
        LP.check()
        return dy.to_numpy(np.uint8), lib.mi_last_kernel().decode()

    xq = {N: orc.f32_to_mx(8, refnp.gen_exact(rng, (N, Ci, S)), N, Ci, S) for N in (2, 3)}
    want = {N: orc.conv3(xq[N], 3, N, Ci, D, H, W, w, b, Co, 3, acc64=1)[0] for N in (2, 3)}
    seen = set()
    for N, split in [(2, -1), (3, -1), (2, -1), (2, 0), (3, 1 << 20), (2, -1), (3, -1)]:      # 128 tiles: halved by default; 192: not
        lib.mi_conv_split(split)
        got, name = run(N, xq[N])
        seen.add("MT 2" in name)
        assert "conv3_wide_k" in name and np.array_equal(got, want[N]), (N, split, name)
    lib.mi_conv_split(-1)
    assert seen == {True, False}
    lib.lp_wmemo_clear()


def test_nonfinite_input_propagates(gpu):
    """A NaN block (scale byte 0xFF) reaches every output voxel whose taps touch it and nothing else (tests/test_mx4.c:139-168)."""
    rng = np.random.default_rng(80)
    N, Ci, Co, D, H, W = 1, 32, 32, 4, 8, 16
    S = D * H * W
    x, w, b = rand_case(rng, N, Ci, Co, S)
    x[0, 3, (2 * H + 4) * W + 8] = np.nan
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    got, _ = gpu_conv(xq, 3, N, Ci, D, H, W, w, b, Co, 0)
    bad = ~np.isfinite(got[0, 0].reshape(D, H, W))
    exp = np.zeros((D, H, W), bool); exp[1:4, 3:6, 7:10] = True
    assert np.array_equal(bad, exp)


def test_config0_full_size_against_oracle(gpu):
    """The reference's CPU-runnable case at its full size: one 3x3x3 conv 32 -> 32, N 1, 64^3, seed 0, activations N(0, 1) as fp32 planes
    (quantised to MX-fp8 per 32 channels while staging), Kaiming weights, no bias, fp16 planes out, through lp_conv_fwd_f8 - the call the
    benchmark's c0 record times. Against the oracle's fp32-accumulated conv of the same operands: the north-star tolerance of 1e-3 max-abs-rel
    on the binary16 result (whose own rounding is 4.9e-4 relative per value), and at most one binary16 step between any two values that are not
    small against the largest (the fp32 sums differ by about 1e-5 of the largest output, which is many steps of a value near zero)."""
    N, Cc, D = 1, 32, 64
    S = D ** 3
    rng = np.random.default_rng(0)
    x = rng.standard_normal((N, Cc, S)).astype(np.float32)
    w = (rng.standard_normal((Cc, Cc, 27)) * np.sqrt(2.0 / (Cc * 27))).astype(np.float32)
    want, _ = orc.conv3(x, 0, N, Cc, D, D, D, w, None, Cc, 2, cbits=8)
    got, _ = gpu_conv(x, 0, N, Cc, D, D, D, w, None, Cc, 2, cbits=8)
    assert "conv3_row1_k<fmt 8, out 0" in lib.mi_last_kernel().decode(), lib.mi_last_kernel().decode()
    g = got.view(np.float16).astype(np.float32).reshape(N, Cc, S); q = want.view(np.float16).astype(np.float32).reshape(N, Cc, S)
    assert np.isfinite(g).all()
    assert np.abs(g - q).max() / np.abs(q).max() < 1e-3
    # two roundings of nearly equal fp32 sums: the same binary16 value or its neighbour, and the neighbour rarely
    gi = got.view(np.int16).astype(np.int32).ravel(); qi = want.view(np.int16).astype(np.int32).ravel()
    ordg = np.where(gi < 0, -(gi & 0x7fff), gi); ordq = np.where(qi < 0, -(qi & 0x7fff), qi)
    step = np.abs(ordg - ordq)
    big = np.abs(q.ravel()) >= np.abs(q).max() / 16
    assert big.sum() > 100000 and step[big].max() <= 1 and (step[big] != 0).mean() < 0.05, (step[big].max(), (step[big] != 0).mean())
    assert (step != 0).mean() < 0.15
    # the same operands as stored MX-fp8 give the same bytes: the staging pass quantises exactly as lp_f32_to_mx8 does
    got2, _ = gpu_conv(orc.f32_to_mx(8, x, N, Cc, S), 3, N, Cc, D, D, D, w, None, Cc, 2, cbits=8)
    assert np.array_equal(got, got2)


@pytest.mark.parametrize("bits", [8, 4])
def test_full_size_properties(gpu, bits):
    """BASELINE-size layer (128 -> 128, 64^3, N 2; fp4: 256 -> 256, 32^3, N 2): exact-operand output compared on sampled planes with the
    oracle restricted to those planes, and byte-equal reruns."""
    rng = np.random.default_rng(90 + bits)
    N, Ci, Co, D = (2, 128, 128, 64) if bits == 8 else (2, 256, 256, 32)
    H = W = D
    S = D * H * W
    xdt = 3 if bits == 8 else 4
    x, w, b = exact_case(rng, N, Ci, Co, S)
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    gq, gs = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, Go=8, stats=True)
    gq2, gs2 = gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, Go=8, stats=True, wkey=99)
    assert np.array_equal(gq, gq2) and np.array_equal(gs, gs2)
    lib.lp_wmemo_clear()
    dec = orc.mx_to_f32(bits, gq, N, Co, S).reshape(N, Co, D, H, W)
    for (z0, z1) in [(0, 1), (D // 2, D // 2 + 1), (D - 1, D)]:
        want, _ = orc.conv3(xq, xdt, N, Ci, D, H, W, w, b, Co, xdt, cbits=bits, z0=z0, z1=z1, acc64=1)
        wdec = orc.mx_to_f32(bits, want, N, Co, S).reshape(N, Co, D, H, W)
        assert np.array_equal(dec[:, :, z0:z1], wdec[:, :, z0:z1])
    # statistics == fp64 sums of the exact pre-quantisation values is checked at small sizes; here: sum of the sums is finite and stable
    assert np.isfinite(gs).all()


@pytest.mark.parametrize("bits,Ci,Co,dims", [(8, 128, 128, (4, 8, 16)), (8, 32, 32, (5, 9, 18)), (4, 64, 64, (4, 8, 16)), (8, 32, 16, (4, 8, 16))])
def test_fused_statistics_finalize(gpu, bits, Ci, Co, dims):
    """mi_conv_fwd_gn == mi_gn_sums_zero + lp_conv_fwd_* + mi_gn_finalize, bit for bit (mean, rstd, slots), with uncleared slots on entry."""
    rng = np.random.default_rng(Ci + Co + bits)
    D, H, W = dims
    N, S, G = 2, D * H * W, 8
    x, w, b = rand_case(rng, N, Ci, Co, S)
    dq = to_mx(bits, x)
    dt = 3 if bits == 8 else 4
    dw, db = DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    ybytes = (lib.lp_mx8_bytes if bits == 8 else lib.lp_mx4_bytes)(N, Co, S)
    xs = shape5(N, Ci, D, H, W)
    res = []
    for fused in (False, True):
        dy = DevBuf(ybytes); dsum = DevBuf.from_numpy(rng.integers(0, 255, N * G * 2 * 24).astype(np.uint8))     # garbage in the slots
        dm, dr = DevBuf(N * G * 4), DevBuf(N * G * 4)
        if fused:
            assert lib.mi_conv_fwd_gn(bits, dq.ptr, dt, xs, dw.ptr, db.ptr, Co, dy.ptr, dt, gnp_t(), dsum.ptr, G, split_t(), 1e-5, dm.ptr, dr.ptr) == 0
        else:
            lib.mi_gn_sums_zero(dsum.ptr, N * G * 2)
            f = lib.lp_conv_fwd_f8 if bits == 8 else lib.lp_conv_fwd_f4
            assert f(dq.ptr, dt, xs, dw.ptr, db.ptr, Co, dy.ptr, dt, gnp_t(), dsum.ptr, G, split_t()) == 0
            lib.mi_gn_finalize(dsum.ptr, N * G, (Co // G) * S, 1e-5, dm.ptr, dr.ptr)
        LP.check()
        res.append((dy.to_numpy(np.uint8), dsum.to_numpy(np.uint8), dm.to_numpy(np.float32), dr.to_numpy(np.float32)))
    for u, v in zip(*res):
        assert np.array_equal(u, v)


@pytest.mark.parametrize("case", ["general32", "wide128", "stem4", "decoder_up", "fp4_64", "gn_input", "row_slices64", "row1_slices64", "row_slices_fp4"])
def test_z_range_slabs_equal_whole(gpu, case):
    """split_t's z-range (zi0 / Di: output plane z reads input plane z + zi0 of a depth-Di input) with direct slab outputs (yzo / yD), the
    reference's in-place slab inference (src/nn_lp.h:36-40, src/nn_bwd.cu:33-46): the conv computed slab by slab into the full-depth output,
    statistics accumulating over the calls, is byte-identical to one call over the whole tensor (tests/test_infer_mem.c's contract)."""
    rng = np.random.default_rng(hash(case) % 1000)
    bits, xdt, up, gn = 8, 3, 0, False
    Cu = 0
    if case == "general32": N, Ci, Co, D, H, W, slabs = 2, 32, 32, 12, 16, 32, (4, 8)
    elif case == "wide128": N, Ci, Co, D, H, W, slabs = 1, 64, 128, 16, 8, 32, (8, 4, 4)
    elif case == "stem4": N, Ci, Co, D, H, W, slabs = 2, 4, 32, 10, 16, 16, (4, 6)
    elif case == "decoder_up": N, Ci, Co, D, H, W, slabs, up, gn, Cu = 1, 96, 32, 16, 16, 16, (4, 4, 8), 1, True, 64
    elif case == "fp4_64": N, Ci, Co, D, H, W, slabs, bits, xdt = 1, 64, 64, 12, 8, 16, (8, 4), 4, 4
    elif case == "row_slices64": N, Ci, Co, D, H, W, slabs, gn = 2, 64, 64, 12, 16, 32, (4, 8), True          # the row kernels' two channel slices
    elif case == "row1_slices64": N, Ci, Co, D, H, W, slabs = 2, 32, 64, 12, 16, 64, (8, 4)
    elif case == "row_slices_fp4": N, Ci, Co, D, H, W, slabs, bits, xdt = 1, 96, 64, 12, 8, 32, (4, 4, 4), 4, 4
    else: N, Ci, Co, D, H, W, slabs, gn = 2, 64, 64, 8, 16, 16, (4, 4), True
    S = D * H * W
    G = 8
    w = (rng.standard_normal((Co, Ci, 27)) * np.sqrt(2.0 / (Ci * 27))).astype(np.float32)
    b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    dw, db = DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    sp = split_t(); keep = []
    if up:
        Cs = Ci - Cu
        xu = rng.standard_normal((N, Cu, S // 8)).astype(np.float32); xs_ = rng.standard_normal((N, Cs, S)).astype(np.float32)
        dx, dx2 = DevBuf.from_numpy(orc.f32_to_mx(bits, xu, N, Cu, S // 8)), DevBuf.from_numpy(orc.f32_to_mx(bits, xs_, N, Cs, S))
        sp.x2, sp.c_split, sp.up = dx2.ptr, Cu, 1
        g1 = dev_gn(rng.uniform(.5, 1.5, Cu).astype(np.float32), rng.uniform(-.3, .3, Cu).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.7, 1.4, N * G).astype(np.float32), G)
        g2 = dev_gn(rng.uniform(.5, 1.5, Cs).astype(np.float32), rng.uniform(-.3, .3, Cs).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.7, 1.4, N * G).astype(np.float32), G)
        sp.gp2 = g2                                     # (a copy of the struct: g2 itself keeps the device buffers alive)
        keep += [dx2, g2]
    else:
        x = rng.standard_normal((N, Ci, S)).astype(np.float32)
        dx = DevBuf.from_numpy(orc.f32_to_mx(bits, x, N, Ci, S))
        g1 = dev_gn(rng.uniform(.5, 1.5, Ci).astype(np.float32), rng.uniform(-.3, .3, Ci).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.7, 1.4, N * G).astype(np.float32), G) if gn else gnp_t()
    f = lib.lp_conv_fwd_f8 if bits == 8 else lib.lp_conv_fwd_f4
    ybytes = orc.mx_bytes(bits, N, Co, S)
    ywhole, yslab = DevBuf(ybytes), DevBuf(ybytes)
    sw, ss = DevBuf(N * G * 2 * 24), DevBuf(N * G * 2 * 24)
    lib.mi_gn_sums_zero(sw.ptr, 2 * N * G); lib.mi_gn_sums_zero(ss.ptr, 2 * N * G)
    sp.stored_stats = 1
    assert f(dx.ptr, xdt, shape5(N, Ci, D, H, W), dw.ptr, db.ptr, Co, ywhole.ptr, xdt, g1, sw.ptr, G, sp) == 0
    kernel = lib.mi_last_kernel().decode()
    z0 = 0
    for sk in slabs:
        sp.zi0, sp.Di, sp.yzo, sp.yD = z0, D, z0, D
        assert f(dx.ptr, xdt, shape5(N, Ci, sk, H, W), dw.ptr, db.ptr, Co, yslab.ptr, xdt, g1, ss.ptr, G, sp) == 0
        z0 += sk
    assert z0 == D
    LP.check()
    assert ("two channel slices" in kernel) == case.startswith("row"), kernel
    assert np.array_equal(ywhole.to_numpy(np.uint8), yslab.to_numpy(np.uint8)), kernel
    a, c = np.zeros((N, G, 2), np.float64), np.zeros((N, G, 2), np.float64)
    da, dc = DevBuf(a.nbytes), DevBuf(c.nbytes)
    lib.mi_gn_sums_get(sw.ptr, 2 * N * G, da.ptr); lib.mi_gn_sums_get(ss.ptr, 2 * N * G, dc.ptr)
    a, c = da.to_numpy(np.float64), dc.to_numpy(np.float64)
    assert np.allclose(a, c, rtol=1e-12, atol=1e-9), kernel
    # a slab into its own depth-sk output (the temp of the reference's in-place form): the same planes
    sk = slabs[0]
    sp.zi0, sp.Di, sp.yzo, sp.yD = slabs[0] if len(slabs) > 1 else 0, D, 0, 0
    sk2 = slabs[1] if len(slabs) > 1 else sk
    ytmp = DevBuf(orc.mx_bytes(bits, N, Co, sk2 * H * W))
    assert f(dx.ptr, xdt, shape5(N, Ci, sk2, H, W), dw.ptr, db.ptr, Co, ytmp.ptr, xdt, g1, None, 0, sp) == 0
    LP.check()
    full = orc.mx_to_f32(bits, ywhole.to_numpy(np.uint8), N, Co, S).reshape(N, Co, D, H * W)
    part = orc.mx_to_f32(bits, ytmp.to_numpy(np.uint8), N, Co, sk2 * H * W).reshape(N, Co, sk2, H * W)
    zz = slabs[0] if len(slabs) > 1 else 0
    assert np.array_equal(part, full[:, :, zz:zz + sk2])


# ---- the fp4-storage shapes of the BASELINE's third configuration and the fp4 entry's small-channel rows ----
@pytest.mark.parametrize("Ci,Co,dims,gn", [(128, 128, (16, 16, 16), False), (128, 256, (12, 10, 14), False), (128, 256, (16, 16, 32), True), (96, 96, (13, 10, 17), True)])
def test_stride2_wide_mx4_input_computes_in_e4m3(gpu, Ci, Co, dims, gn):
    """A wide MX-fp4 tensor through the stride-2 entry: the reference keeps fp4 compute for exactly 32 -> <= 32 channels and runs every other
    MX-fp4 input on the e4m3 kernel, the stored rows decoded, (GroupNorm + SiLU,) re-quantised to e4m3 per (voxel, 32 channels), the weights
    e4m3 blocks (src/lp_s2.cu:653-671, :729-749); the call returns 0, not 3. Exact operands equal the oracle byte for byte."""
    rng = np.random.default_rng(Ci + Co + dims[0])
    D, H, W = dims
    N, S, G = 2, D * H * W, 8
    if gn:
        x, w, b = rand_case(rng, N, Ci, Co, S)
        p = [rng.uniform(0.5, 1.5, Ci).astype(np.float32), rng.uniform(-.5, .5, Ci).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    else:
        x, w, b = exact_case(rng, N, Ci, Co, S)
    xq = orc.f32_to_mx(4, x, N, Ci, S)
    dxq, dw, db = DevBuf.from_numpy(xq), DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    Do, Ho, Wo = out_dims(D, H, W, 2)
    So = Do * Ho * Wo
    dy = DevBuf(lib.lp_mx4_bytes(N, Co, So))
    g = dev_gn(*p, G) if gn else gnp_t()
    rc = lib.lp_conv_fwd_s2_f8(dxq.ptr, 4, shape5(N, Ci, D, H, W), dw.ptr, db.ptr, Co, dy.ptr, 4, shape5(N, Co, Do, Ho, Wo), g)
    LP.check()
    assert rc == 0 and "fmt 8, stride 2" in lib.mi_last_kernel().decode()
    got = dy.to_numpy(np.uint8)
    want, _ = orc.conv3(xq, 4, N, Ci, D, H, W, w, b, Co, 4, cbits=8, stride=2, gp=orc.gn(*p, G) if gn else None, acc64=0 if gn else 1)
    if gn:
        frac, near = code_mismatch_fraction(4, got, want, N, Co, So)
        assert frac < 5e-3 and near
    else:
        assert np.array_equal(got, want)
    # ... while 32 -> 32 on even dims of an MX-fp4 tensor does compute in e2m1 and says so
    x2, w2, b2 = exact_case(rng, 1, 32, 32, 16 * 16 * 16)
    q2 = orc.f32_to_mx(4, x2, 1, 32, 4096)
    d2, dw2, db2, dy2 = DevBuf.from_numpy(q2), DevBuf.from_numpy(w2), DevBuf.from_numpy(b2), DevBuf(lib.lp_mx4_bytes(1, 32, 512))
    assert lib.lp_conv_fwd_s2_f8(d2.ptr, 4, shape5(1, 32, 16, 16, 16), dw2.ptr, db2.ptr, 32, dy2.ptr, 4, shape5(1, 32, 8, 8, 8), gnp_t()) == 3
    LP.check()
    assert np.array_equal(dy2.to_numpy(np.uint8), orc.conv3(q2, 4, 1, 32, 16, 16, 16, w2, b2, 32, 4, cbits=4, stride=2, acc64=1)[0])


@pytest.mark.parametrize("Cu,Cs,Co,dims,gn", [(256, 128, 128, (4, 8, 16), False), (256, 128, 128, (8, 8, 16), True), (320, 256, 256, (4, 8, 16), False), (64, 32, 32, (8, 16, 16), True)])
def test_fp4_decoder_conv_fused_upsample(gpu, Cu, Cs, Co, dims, gn):
    """The MX-fp4 decoder conv1 over [2x trilinear up(coarse) | skip] (256 + 128 -> 128: the BASELINE's fp4 up path; 320 + 256 -> 256:
    tests/test_mx4_wide.c:749-751). Grid-valued coarse data with a +6 in every block blend exactly in any arithmetic (tests/test_mx4_wide.c:18-19):
    the fp32 output equals the oracle; with GroupNorm + SiLU on both segments the e2m1 operands agree up to neighbouring codes of the staged rows."""
    rng = np.random.default_rng(60 + Cu + Cs)
    D, H, W = dims
    N, S, Sc, G = 1, D * H * W, (D // 2) * (H // 2) * (W // 2), 8
    if gn:
        xa = rng.standard_normal((N, Cu, Sc)).astype(np.float32); xb = rng.standard_normal((N, Cs, S)).astype(np.float32)
        w = (rng.standard_normal((Co, Cu + Cs, 27)) * np.sqrt(2.0 / ((Cu + Cs) * 27))).astype(np.float32)
    else:
        xa = refnp.gen_exact(rng, (N, Cu, Sc)); xa[np.abs(xa) == 6] = 6.0      # (+6, not -6: the blend of equal-sign maxima stays the block maximum)
        xb = refnp.gen_exact(rng, (N, Cs, S)); w = refnp.gen_exact(rng, (Co, Cu + Cs, 27))
    qa, qb = orc.f32_to_mx(4, xa, N, Cu, Sc), orc.f32_to_mx(4, xb, N, Cs, S)
    p = [rng.uniform(0.5, 1.5, Cu).astype(np.float32), rng.uniform(-.5, .5, Cu).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    p2 = [rng.uniform(0.5, 1.5, Cs).astype(np.float32), rng.uniform(-.5, .5, Cs).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    want, _ = orc.conv3(qa, 4, N, Cu + Cs, D, H, W, w, None, Co, 0, cbits=4, x2=qb, c_split=Cu, up=1, gp=orc.gn(*p, G) if gn else None, gp2=orc.gn(*p2, G) if gn else None)
    got, _ = gpu_conv(qa, 4, N, Cu + Cs, D, H, W, w, None, Co, 0, cbits=4, x2=qb, c_split=Cu, up=1, gp=dev_gn(*p, G) if gn else None, gp2=dev_gn(*p2, G) if gn else None)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < (3e-2 if gn else 1e-5), err
    if not gn:                                                     # the blend of grid values is a multiple of 1/64 of at most 6: re-quantised to e2m1 it is not exact,
        wq, _ = orc.conv3(qa, 4, N, Cu + Cs, D, H, W, w, None, Co, 4, cbits=4, x2=qb, c_split=Cu, up=1)   # but both sides round the same values: identical output codes
        gq, _ = gpu_conv(qa, 4, N, Cu + Cs, D, H, W, w, None, Co, 4, cbits=4, x2=qb, c_split=Cu, up=1)
        assert np.array_equal(gq, wq)


@pytest.mark.parametrize("Ci,Co,dims", [(16, 16, (12, 12, 16)), (12, 32, (6, 12, 20)), (9, 16, (5, 9, 18)), (16, 64, (4, 8, 16))])
def test_fp4_entry_9_to_16_channels(gpu, Ci, Co, dims):
    """lp_conv_fwd_f4 on 9 - 16 input channels (one 16-wide stored block). The reference's packed kernel scales each 16-channel group of a position
    and each (tap, output channel) group of 16 weights on its own (src/lp_f4fwd.cuh:786-800, src/lp_f4fwd.cu:85-100): the operands of a
    32-block holding the 16 channels and 16 zeros. Exact operands: every output type equals the oracle."""
    rng = np.random.default_rng(Ci * 3 + Co)
    D, H, W = dims
    N, S = 2, D * H * W
    x = refnp.gen_exact(rng, (N, Ci, S), block=16); w = refnp.gen_exact(rng, (Co, Ci, 27), block=16)
    b = (GRID[rng.integers(0, 8, Co)] * 0.25).astype(np.float32)
    xq = orc.f32_to_mx(4, x, N, Ci, S)
    for ydt in (0, 4, 3):
        want, ws = orc.conv3(xq, 4, N, Ci, D, H, W, w, b, Co, ydt, cbits=4, acc64=1, Go=min(8, Co), want_stats=True)
        got, gs = gpu_conv(xq, 4, N, Ci, D, H, W, w, b, Co, ydt, cbits=4, Go=min(8, Co), stats=True)
        assert np.array_equal(got, want), (ydt, lib.mi_last_kernel().decode())
        assert np.allclose(gs, ws, rtol=1e-6)
    xr, wr, br = rand_case(rng, N, Ci, Co, S)                      # random data with GroupNorm on the input (tests/test_mx4.c:224-270: 16 -> 32 with GN)
    G = 1 if Ci % 4 else 4
    p = [rng.uniform(0.5, 1.5, Ci).astype(np.float32), rng.uniform(-.5, .5, Ci).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    xrq = orc.f32_to_mx(4, xr, N, Ci, S)
    want, _ = orc.conv3(xrq, 4, N, Ci, D, H, W, wr, br, Co, 0, cbits=4, gp=orc.gn(*p, G))
    got, _ = gpu_conv(xrq, 4, N, Ci, D, H, W, wr, br, Co, 0, cbits=4, gp=dev_gn(*p, G))
    assert np.abs(got - want).max() / np.abs(want).max() < 3e-2


@pytest.mark.parametrize("Cu,Cs,Co,dims", [(16, 16, 16, (12, 12, 16)), (12, 16, 16, (4, 8, 16)), (16, 8, 8, (8, 8, 16))])
def test_fp4_fused_upsample_small_channels(gpu, Cu, Cs, Co, dims):
    """The level-0 decoder conv of a narrow net: <= 16 coarse + <= 16 skip channels -> <= 16, MX-fp4, the coarse segment read through the fused
    trilinear 2x (src/lp_f4up.cu:141-291). Grid data with a +6 per block: the blend is exact, outputs equal the oracle; random data with both
    GroupNorms within the e2m1 staging tolerance."""
    rng = np.random.default_rng(Cu + Cs * 5 + Co)
    D, H, W = dims
    N, S, Sc, G = 2, D * H * W, (D // 2) * (H // 2) * (W // 2), 4
    xa = refnp.gen_exact(rng, (N, Cu, Sc), block=16); xa[np.abs(xa) == 6] = 6.0
    xb = refnp.gen_exact(rng, (N, Cs, S), block=16 if Cs > 8 else 8); w = refnp.gen_exact(rng, (Co, Cu + Cs, 27), block=16)
    qa, qb = orc.f32_to_mx(4, xa, N, Cu, Sc), orc.f32_to_mx(4, xb, N, Cs, S)
    want, _ = orc.conv3(qa, 4, N, Cu + Cs, D, H, W, w, None, Co, 0, cbits=4, x2=qb, c_split=Cu, up=1)
    got, _ = gpu_conv(qa, 4, N, Cu + Cs, D, H, W, w, None, Co, 0, cbits=4, x2=qb, c_split=Cu, up=1)
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-5
    wq, _ = orc.conv3(qa, 4, N, Cu + Cs, D, H, W, w, None, Co, 4, cbits=4, x2=qb, c_split=Cu, up=1)
    gq, _ = gpu_conv(qa, 4, N, Cu + Cs, D, H, W, w, None, Co, 4, cbits=4, x2=qb, c_split=Cu, up=1)
    assert np.array_equal(gq, wq)
    xa = rng.standard_normal((N, Cu, Sc)).astype(np.float32); xb = rng.standard_normal((N, Cs, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Cu + Cs, 27)) * np.sqrt(2.0 / ((Cu + Cs) * 27))).astype(np.float32)
    qa, qb = orc.f32_to_mx(4, xa, N, Cu, Sc), orc.f32_to_mx(4, xb, N, Cs, S)
    p = [rng.uniform(0.5, 1.5, Cu).astype(np.float32), rng.uniform(-.5, .5, Cu).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    p2 = [rng.uniform(0.5, 1.5, Cs).astype(np.float32), rng.uniform(-.5, .5, Cs).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.8, 1.2, N * G).astype(np.float32)]
    want, _ = orc.conv3(qa, 4, N, Cu + Cs, D, H, W, w, None, Co, 0, cbits=4, x2=qb, c_split=Cu, up=1, gp=orc.gn(*p, G), gp2=orc.gn(*p2, G))
    got, _ = gpu_conv(qa, 4, N, Cu + Cs, D, H, W, w, None, Co, 0, cbits=4, x2=qb, c_split=Cu, up=1, gp=dev_gn(*p, G), gp2=dev_gn(*p2, G))
    assert np.abs(got - want).max() / np.abs(want).max() < 3e-2


def test_config2_full_size_down_and_decoder(gpu):
    """The BASELINE's fp4 configuration at its stated sizes, exact operands, compared on sampled output planes with the oracle restricted to
    them: the stride-2 down conv 128 -> 256 from 64^3, N 2 (MX-fp4 storage, e4m3 compute), and the decoder conv over [up(256 @ 32^3) | skip
    (128 @ 64^3)] -> 128 (e2m1 compute); reruns byte-identical."""
    rng = np.random.default_rng(222)
    N, D = 2, 64
    S, Sc = D ** 3, (D // 2) ** 3
    x, w, b = exact_case(rng, N, 128, 256, S)
    xq = orc.f32_to_mx(4, x, N, 128, S)
    got, _ = gpu_conv(xq, 4, N, 128, D, D, D, w, b, 256, 4, stride=2)
    got2, _ = gpu_conv(xq, 4, N, 128, D, D, D, w, b, 256, 4, stride=2)
    assert np.array_equal(got, got2)
    dec = orc.mx_to_f32(4, got, N, 256, Sc).reshape(N, 256, D // 2, D // 2, D // 2)
    for z in (0, D // 4, D // 2 - 1):
        want, _ = orc.conv3(xq, 4, N, 128, D, D, D, w, b, 256, 4, cbits=8, stride=2, z0=z, z1=z + 1, acc64=1)
        wd = orc.mx_to_f32(4, want, N, 256, Sc).reshape(N, 256, D // 2, D // 2, D // 2)
        assert np.array_equal(dec[:, :, z], wd[:, :, z]), z
    del x, xq, got, got2, dec
    xa = refnp.gen_exact(rng, (N, 256, Sc)); xa[np.abs(xa) == 6] = 6.0
    xb = refnp.gen_exact(rng, (N, 128, S)); w = refnp.gen_exact(rng, (128, 384, 27))
    qa, qb = orc.f32_to_mx(4, xa, N, 256, Sc), orc.f32_to_mx(4, xb, N, 128, S)
    got, _ = gpu_conv(qa, 4, N, 384, D, D, D, w, None, 128, 4, cbits=4, x2=qb, c_split=256, up=1)
    assert "conv3_wide_k" in lib.mi_last_kernel().decode()
    dec = orc.mx_to_f32(4, got, N, 128, S).reshape(N, 128, D, D, D)
    for z in (0, 31, D - 1):
        want, _ = orc.conv3(qa, 4, N, 384, D, D, D, w, None, 128, 4, cbits=4, x2=qb, c_split=256, up=1, z0=z, z1=z + 1)
        wd = orc.mx_to_f32(4, want, N, 128, S).reshape(N, 128, D, D, D)
        assert np.array_equal(dec[:, :, z], wd[:, :, z]), z


@pytest.mark.parametrize("cbits,up", [(4, 1), (4, 2), (4, 3), (8, 1), (8, 2)])
def test_fused_upsample_blend_modes(gpu, cbits, up):
    """The fused-upsample staging's two blends on non-grid data with row scales spread over 2^12: the fp4 entry's default (up 1) is the binary16
    blend (src/lp_common.cuh:674-712, chosen at src/lp_f4fwd.cuh:1135-1136), the fp8 entry's the fp32 chain; up 2 / 3 force one. The e2m1 products
    of the matrix cores are summed exactly, so under e2m1 compute the fp32 output agrees with the oracle's fp64 accumulation to 1e-5 only if
    every staged code is the same: one differing code of a row shows as ~1e-2."""
    rng = np.random.default_rng(300 + 10 * cbits + up)
    N, Cu, Cs, Co, D, H, W = 1, 64, 32, 32, 8, 8, 16
    S, Sc = D * H * W, (D // 2) * (H // 2) * (W // 2)
    xa = (rng.standard_normal((N, Cu, Sc)) * np.exp(rng.uniform(-4, 4, (N, 1, Sc)))).astype(np.float32)
    xb = rng.standard_normal((N, Cs, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Cu + Cs, 27)) * np.sqrt(2.0 / ((Cu + Cs) * 27))).astype(np.float32)
    qa, qb = orc.f32_to_mx(8, xa, N, Cu, Sc), orc.f32_to_mx(8, xb, N, Cs, S)
    want, _ = orc.conv3(qa, 3, N, Cu + Cs, D, H, W, w, None, Co, 0, cbits=cbits, x2=qb, c_split=Cu, up=up, acc64=1)
    got, _ = gpu_conv(qa, 3, N, Cu + Cs, D, H, W, w, None, Co, 0, cbits=cbits, x2=qb, c_split=Cu, up=up)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < (1e-5 if cbits == 4 else 2e-3), err
    if cbits == 4 and up != 1:                                      # the entry's default is the binary16 blend, and the two blends are different operands
        other, _ = orc.conv3(qa, 3, N, Cu + Cs, D, H, W, w, None, Co, 0, cbits=4, x2=qb, c_split=Cu, up=5 - up, acc64=1)
        d = np.abs(got - other).max() / np.abs(want).max()
        assert d > 1e-4, d


@pytest.mark.gpu
def test_prestage_in_both_formats_and_a_split_conv_on_the_fp4_rows(gpu):
    """mi_conv_prestage2: one read and one evaluation write the MX-fp8 and the MX-fp4 form of silu(gn(x)), the bytes of the two single calls; an
    MX-fp4 conv whose second segment is those fp4 rows (mi_conv_x2_dt(4), no GroupNorm left on it) beside an upsampled MX-fp8 first segment gives
    the bytes of the conv that transforms the MX-fp8 skip itself."""
    from ufsm_amd import gnp_t
    rng = np.random.default_rng(91)
    N, Cu, Cs, Co, (D, H, W), G = 2, 64, 32, 32, (8, 16, 32), 8
    S = D * H * W
    xs_ = rng.standard_normal((N, Cs, S)).astype(np.float32); xu = rng.standard_normal((N, Cu, S // 8)).astype(np.float32)
    qs, qu = orc.f32_to_mx(8, xs_, N, Cs, S), orc.f32_to_mx(8, xu, N, Cu, S // 8)
    par = lambda C: (rng.uniform(.5, 1.5, C).astype(np.float32), rng.uniform(-.3, .3, C).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.7, 1.4, N * G).astype(np.float32))
    p1, p2 = par(Cu), par(Cs)
    g2 = dev_gn(*p2, G)
    dq = DevBuf.from_numpy(qs); y8, y4, s8, s4 = (DevBuf(orc.mx_bytes(b, N, Cs, S)) for b in (8, 4, 8, 4))
    assert lib.mi_conv_prestage2(dq.ptr, shape5(N, Cs, D, H, W), g2, y8.ptr, y4.ptr) == 0
    assert lib.mi_conv_prestage(dq.ptr, 3, shape5(N, Cs, D, H, W), g2, s8.ptr, 8) == 0 and lib.mi_conv_prestage(dq.ptr, 3, shape5(N, Cs, D, H, W), g2, s4.ptr, 4) == 0
    LP.check()
    assert np.array_equal(y8.to_numpy(np.uint8), s8.to_numpy(np.uint8)) and np.array_equal(y4.to_numpy(np.uint8), s4.to_numpy(np.uint8))
    w = (rng.standard_normal((Co, Cu + Cs, 27)) * np.sqrt(2.0 / ((Cu + Cs) * 27))).astype(np.float32)
    own, _ = gpu_conv(qu, 3, N, Cu + Cs, D, H, W, w, None, Co, 3, cbits=4, x2=qs, c_split=Cu, up=1, gp=dev_gn(*p1, G), gp2=g2)
    none = gnp_t(); none.G = -1
    lib.mi_conv_x2_dt(4)
    pre, _ = gpu_conv(qu, 3, N, Cu + Cs, D, H, W, w, None, Co, 3, cbits=4, x2=y4.to_numpy(np.uint8), c_split=Cu, up=1, gp=dev_gn(*p1, G), gp2=none)
    assert np.array_equal(pre, own)
    again, _ = gpu_conv(qu, 3, N, Cu + Cs, D, H, W, w, None, Co, 3, cbits=4, x2=qs, c_split=Cu, up=1, gp=dev_gn(*p1, G), gp2=g2)      # the setting held for one call
    assert np.array_equal(again, own)
