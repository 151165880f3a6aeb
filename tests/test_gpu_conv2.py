"""GPU parity of the 2x2x2 stride-2 conv and transposed conv (mi_conv_down2_fwd, mi_convt_up2_fwd) against the oracle's restatement, through the C ABI.
The reference has neither layer (src/lp_s2.cu:4-9, src/lp_mx_gn.cu:32-33); the oracle is pinned by fp64 closed forms in tests/test_oracle_conv2.py."""
import numpy as np
import pytest

from ufsm_amd import lib, LP, shape5, gnp_t, DevBuf
from gpuutil import dev_gn, mx_bytes
import orc
import refnp

pytestmark = pytest.mark.gpu


def gpu_conv2(up, xq, xdt, N, Ci, D, H, W, w, b, Co, ydt, cbits, gp=None):
    So = 8 * D * H * W if up else (D // 2) * (H // 2) * (W // 2)
    dx, dw = DevBuf.from_numpy(xq), DevBuf.from_numpy(w.astype(np.float32))
    db = DevBuf.from_numpy(b.astype(np.float32)) if b is not None else None
    if ydt >= 3:
        nbytes, dtype = mx_bytes(8 if ydt == 3 else 4, N, Co, So), np.uint8
    else:
        nbytes, dtype = N * Co * So * (2 if ydt == 2 else 4), (np.uint16 if ydt == 2 else np.float32)
    dy = DevBuf(nbytes)
    f = lib.mi_convt_up2_fwd if up else lib.mi_conv_down2_fwd
    rc = f(cbits, dx.ptr, xdt, shape5(N, Ci, D, H, W), dw.ptr, db.ptr if db is not None else None, Co, dy.ptr, ydt, gp if gp is not None else gnp_t())
    LP.check()
    assert rc == 0 and "conv2_mx_k" in lib.mi_last_kernel().decode()
    y = dy.to_numpy(dtype)
    return y.reshape(N, Co, So) if ydt < 3 else y


SHAPES = [(32, 32, (4, 8, 16)), (64, 48, (6, 10, 14)), (128, 256, (8, 8, 8)), (40, 16, (2, 6, 10)), (16, 64, (4, 4, 6)), (256, 128, (4, 4, 8)), (96, 8, (2, 2, 18))]


@pytest.mark.parametrize("up", [0, 1])
@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("Ci,Co,dims", SHAPES)
def test_exact_operands_equal_the_oracle(gpu, up, bits, Ci, Co, dims):
    """Operands exact in the formats: fp32 planes equal the oracle's fp64 accumulation bit for bit, MX-fp8 / MX-fp4 outputs byte for byte (every row
    width 8 / 16 / 32 of the output, ragged channel blocks, column counts that are no multiple of the 64-column wavefront tile, N 2)."""
    rng = np.random.default_rng(1000 * up + 100 * bits + Ci + Co)
    D, H, W = dims
    N, S = 2, D * H * W
    x = refnp.gen_exact(rng, (N, Ci, S))
    w = refnp.gen_exact(rng, (Ci, Co, 8), block_axis=0) if up else refnp.gen_exact(rng, (Co, Ci, 8))
    b = rng.integers(-8, 9, Co).astype(np.float32) * 0.25
    xdt = 3 if bits == 8 else 4
    xq = orc.f32_to_mx(bits, x, N, Ci, S)
    for ydt in (0, 3, 4):
        want = orc.conv2(xq, xdt, N, Ci, D, H, W, w, b, Co, ydt, up, cbits=bits, acc64=1)
        got = gpu_conv2(up, xq, xdt, N, Ci, D, H, W, w, b, Co, ydt, bits)
        assert np.array_equal(got, want), (ydt, np.abs(got.astype(np.float64) - want.astype(np.float64)).max())


@pytest.mark.parametrize("up", [0, 1])
@pytest.mark.parametrize("bits,xbits,gn", [(8, 8, False), (4, 4, False), (4, 8, False), (8, 4, False), (8, 8, True), (4, 8, True)])
def test_random_operands_within_tolerance(gpu, up, bits, xbits, gn):
    """N(0,1) data and Kaiming weights, a stored format that differs from the compute format, GroupNorm + SiLU on the input: conv outputs within 1e-3
    max-abs-rel of the fp64-accumulated oracle under e4m3 compute; under e2m1 compute the matrix cores add the products exactly, so without the
    device's SiLU in the way the bound is 1e-5 (one differing staged code would show as ~1e-2)."""
    rng = np.random.default_rng(50 + 10 * up + bits + xbits + gn)
    N, Ci, Co, D, H, W, G = 1, 96, 64, 4, 6, 8, 8
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = (rng.standard_normal((Ci, Co, 8) if up else (Co, Ci, 8)) * np.sqrt(2.0 / (Ci * (1 if up else 8)))).astype(np.float32)
    b = (rng.standard_normal(Co) * 0.1).astype(np.float32)
    xdt = 3 if xbits == 8 else 4
    xq = orc.f32_to_mx(xbits, x, N, Ci, S)
    p = [rng.uniform(.5, 1.5, Ci).astype(np.float32), rng.uniform(-.3, .3, Ci).astype(np.float32), rng.uniform(-.2, .2, N * G).astype(np.float32), rng.uniform(.7, 1.4, N * G).astype(np.float32)]
    want = orc.conv2(xq, xdt, N, Ci, D, H, W, w, b, Co, 0, up, cbits=bits, gp=orc.gn(*p, G) if gn else None, acc64=1)
    got = gpu_conv2(up, xq, xdt, N, Ci, D, H, W, w, b, Co, 0, bits, gp=dev_gn(*p, G) if gn else None)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < (3e-2 if gn and bits == 4 else 1e-3 if bits == 8 else 1e-5), err


def test_config2_layers_at_full_size(gpu):
    """BASELINE configs[2]'s stride-2 layers in MX-fp4: the 2x2x2 down conv 128 -> 256 on 64^3 (N 2) and the 2x2x2 transposed conv 256 -> 128 on
    32^3 (N 2), inputs uniform[-3, 3], Kaiming weights, MX-fp4 in and out, against the oracle (fp64 accumulation of the same e2m1 operands: fp32
    planes within 1e-5, and the stored MX-fp4 codes byte for byte up to rows whose pre-rounding value sits on a code boundary: < 1e-4 of them)."""
    rng = np.random.default_rng(2)
    for up, Ci, Co, D in ((0, 128, 256, 64), (1, 256, 128, 32)):
        N, S = 2, D ** 3
        x = rng.uniform(-3, 3, (N, Ci, S)).astype(np.float32)
        w = (rng.standard_normal((Ci, Co, 8) if up else (Co, Ci, 8)) * np.sqrt(2.0 / (Ci * (1 if up else 8)))).astype(np.float32)
        xq = orc.f32_to_mx(4, x, N, Ci, S)
        want = orc.conv2(xq, 4, N, Ci, D, D, D, w, None, Co, 0, up, cbits=4, acc64=1)
        got = gpu_conv2(up, xq, 4, N, Ci, D, D, D, w, None, Co, 0, 4)
        err = np.abs(got - want).max() / np.abs(want).max()
        assert err < 1e-5, (up, err)
        wq = orc.conv2(xq, 4, N, Ci, D, D, D, w, None, Co, 4, up, cbits=4, acc64=1)
        gq = gpu_conv2(up, xq, 4, N, Ci, D, D, D, w, None, Co, 4, 4)
        assert (gq != wq).mean() < 1e-4, (up, (gq != wq).mean())


@pytest.mark.parametrize("up", [0, 1])
def test_weight_memo(gpu, up):
    """mi_conv_s2_wkey: the prepared weights are kept under the caller's id (no second preparation, no further allocation), give the bytes of the
    per-call preparation, are told apart by direction, and are dropped by a new weight step."""
    rng = np.random.default_rng(81 + up)
    N, Ci, Co, D, H, W = 1, 64, 64, 4, 4, 8
    S = D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = (rng.standard_normal((Ci, Co, 8) if up else (Co, Ci, 8)) * 0.1).astype(np.float32)
    xq = orc.f32_to_mx(8, x, N, Ci, S)
    So = 8 * S if up else S // 8
    dx, dw, dy = DevBuf.from_numpy(xq), DevBuf.from_numpy(w), DevBuf(mx_bytes(8, N, Co, So))
    f = lib.mi_convt_up2_fwd if up else lib.mi_conv_down2_fwd

    def run(key):
        if key:
            lib.mi_conv_s2_wkey(key)
        assert f(8, dx.ptr, 3, shape5(N, Ci, D, H, W), dw.ptr, None, Co, dy.ptr, 3, gnp_t()) == 0
        LP.check()
        return dy.to_numpy(np.uint8).copy()

    lib.lp_wmemo_clear()
    plain = run(0)
    first = run(777)
    allocs = lib.mi_alloc_count()
    second = run(777)
    assert lib.mi_alloc_count() == allocs
    assert np.array_equal(plain, first) and np.array_equal(plain, second)
    w2 = np.ascontiguousarray(-2 * w)
    lib.mi_h2d(dw.ptr, w2.ctypes.data, w2.nbytes)
    assert np.array_equal(run(777), plain)                        # (the kept image: the caller said the weights are constant)
    assert np.array_equal(run(0), run(0)) and not np.array_equal(run(0), plain)      # the id was consumed by its call: these prepare per call
    lib.lp_wmemo_step(12345)                                      # weights changed: a new step drops the memo (src/nn_lp.h:56)
    assert np.array_equal(run(777), run(0))
    lib.lp_wmemo_clear(); lib.lp_wmemo_step(0)


def test_refusals(gpu):
    x = DevBuf(1 << 16); w = DevBuf(1 << 16); y = DevBuf(1 << 20)
    assert lib.mi_conv_down2_fwd(8, x.ptr, 3, shape5(1, 32, 3, 4, 4), w.ptr, None, 32, y.ptr, 3, gnp_t()) == -1      # odd depth
    assert lib.mi_conv_down2_fwd(6, x.ptr, 3, shape5(1, 32, 4, 4, 4), w.ptr, None, 32, y.ptr, 3, gnp_t()) == -1      # compute format
    assert lib.mi_convt_up2_fwd(8, x.ptr, 0, shape5(1, 32, 4, 4, 4), w.ptr, None, 32, y.ptr, 3, gnp_t()) == -1       # fp32 planes in
    LP.check()
