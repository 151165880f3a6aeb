"""The op layer's conv entries with the reference's names (src/nn.h:399-400, :416, :423, :442) through the host library's C ABI, called the way
the reference's own tests call them (tests/test_mx.c:32-45, :96-156, :159-212; tests/test_mx4.c:170-270): tensors are device pointers whose
storage is registered with nn_set_storage, the precision policy is nn_set_prec, and the entry picks the kernel family. Checked here: the
dispatch rule (MX in gives MX out of the same format; MX-fp4 storage or precision 3 gives the fp4 kernels; <= 8 input channels give the
tap-packed fp8 stem), that every entry's result is the bytes of the lp_* entry it must reach, and the reference's own tolerances against an
fp64 convolution of the decoded operands."""
import ctypes as C

import numpy as np
import pytest

from ufsm_amd import lib, LP, shape5, DevBuf
import orc
import refnp
from gpuutil import gpu_conv, to_mx, mx_bytes

pytestmark = pytest.mark.gpu


def _host():
    from ufsm_amd.unet import load_host
    return load_host()


def _reg(H_, buf, dt):
    H_.nn_set_storage(buf.ptr, buf.nbytes, dt)


def _rel_l2(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b) / max(np.linalg.norm(b), 1e-300))


def test_fp8_conv_on_fp32_planes_under_precision_2(gpu):
    """tests/test_mx.c:32-45: fp32 tensors, precision 2: the fp8 entry quantises while staging; rel. L2 < 0.06 against the fp32 conv; the
    result is lp_conv_fwd_f8's on the same planes."""
    H_ = _host()
    rng = np.random.default_rng(1)
    N = 2
    for ci, co, d in ((16, 16, 16), (12, 16, 12), (16, 64, 8)):
        xs = shape5(N, ci, d, 12, 20)
        S = d * 12 * 20
        x = rng.standard_normal((N, ci, S)).astype(np.float32)
        w = (rng.standard_normal((co, ci, 27)) * 0.1).astype(np.float32); b = (rng.standard_normal(co) * 0.1).astype(np.float32)
        dx, dw, db, dy = DevBuf.from_numpy(x), DevBuf.from_numpy(w), DevBuf.from_numpy(b), DevBuf(N * co * S * 4)
        H_.nn_set_prec(2)
        try:
            H_.nn_conv3d_fwd(dx.ptr, xs, dw.ptr, db.ptr, co, 3, 1, dy.ptr)
        finally:
            H_.nn_set_prec(0)
        LP.check()
        got = dy.to_numpy(np.float32, (N, co, S))
        direct, _ = gpu_conv(x, 0, N, ci, d, 12, 20, w, b, co, 0)
        assert np.array_equal(got, direct)
        ref = refnp.conv3d_f64(x.reshape(N, ci, d, 12, 20), w, b).reshape(N, co, S)
        assert _rel_l2(got, ref) < 0.06
        os_ = H_.nn_conv3d_out_shape(xs, co, 3, 2)
        assert (os_.n, os_.c, os_.d, os_.h, os_.w) == (N, co, (d - 1) // 2 + 1, 6, 10)


@pytest.mark.parametrize("dt,prec,ci,want_kernel", [(8, 0, 32, "fmt 8"), (4, 0, 32, "fmt 4"), (8, 3, 32, "fmt 4"), (8, 0, 4, "conv3_stem_k"), (4, 0, 8, "conv3_stem_k"), (8, 3, 8, "conv3_stem_k")])
def test_dispatch_rule_of_the_plain_conv(gpu, dt, prec, ci, want_kernel):
    """src/nn_bwd.cu:97-112, src/lp_f4fwd.cu:37: MX in gives MX out of the same format; MX-fp4 storage or precision 3 gives the fp4 kernels;
    an input of <= 8 channels gives the fp8 stem whatever the format."""
    H_ = _host()
    rng = np.random.default_rng(2)
    N, co, D, Hh, W = 2, 32, 8, 12, 16
    S = D * Hh * W
    x = rng.standard_normal((N, ci, S)).astype(np.float32)
    w = (rng.standard_normal((co, ci, 27)) * 0.1).astype(np.float32); b = (rng.standard_normal(co) * 0.1).astype(np.float32)
    dq = to_mx(dt, x); dw, db = DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    dy = DevBuf(mx_bytes(dt, N, co, S))
    _reg(H_, dq, dt); _reg(H_, dy, dt)
    H_.nn_set_prec(prec)
    try:
        H_.nn_conv3d_fwd(dq.ptr, shape5(N, ci, D, Hh, W), dw.ptr, db.ptr, co, 3, 1, dy.ptr)
    finally:
        H_.nn_set_prec(0); H_.nn_storage_forget(dq.ptr); H_.nn_storage_forget(dy.ptr)
    LP.check()
    assert want_kernel in lib.mi_last_kernel().decode(), lib.mi_last_kernel().decode()
    ldt = 3 if dt == 8 else 4
    direct, _ = gpu_conv(dq.to_numpy(np.uint8), ldt, N, ci, D, Hh, W, w, b, co, ldt, cbits=4 if (dt == 4 or prec == 3) else 8)
    assert np.array_equal(dy.to_numpy(np.uint8), direct)


def test_mx4_input_with_fp32_planes_out_runs_the_fp4_entry(gpu):
    """src/nn_bwd.cu:104 (the reference's fp4 tests, tests/test_mx4.c:183-198): MX-fp4 in, unregistered fp32 out."""
    H_ = _host()
    rng = np.random.default_rng(3)
    N, ci, co, D, Hh, W = 2, 32, 64, 8, 12, 16
    S = D * Hh * W
    x = rng.standard_normal((N, ci, S)).astype(np.float32)
    w = (rng.standard_normal((co, ci, 27)) * 0.1).astype(np.float32)
    dq = to_mx(4, x); dw = DevBuf.from_numpy(w); dy = DevBuf(N * co * S * 4)
    _reg(H_, dq, 4)
    try:
        H_.nn_conv3d_fwd(dq.ptr, shape5(N, ci, D, Hh, W), dw.ptr, None, co, 3, 1, dy.ptr)
    finally:
        H_.nn_storage_forget(dq.ptr)
    LP.check()
    assert "fmt 4" in lib.mi_last_kernel().decode()
    xq = dq.to_numpy(np.uint8)
    want, _ = orc.conv3(xq, 4, N, ci, D, Hh, W, w, None, co, 0, cbits=4)
    got = dy.to_numpy(np.float32, (N, co, S))
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-3
    ref = refnp.conv3d_f64(orc.mx_to_f32(4, xq, N, ci, S).reshape(N, ci, D, Hh, W), w).reshape(N, co, S)
    assert _rel_l2(got, ref) < 0.25                                   # tests/test_mx4.c:99 (the weights are quantised to e2m1 too)


def test_stride2_and_head_through_the_plain_conv(gpu):
    """tests/test_mx.c:159-166 (32 -> 32, 16^3 -> 8^3) and :202-212 (the 1^3 head 16 -> 1 at 10^3, 1e-5)."""
    H_ = _host()
    rng = np.random.default_rng(4)
    N, c, D = 2, 32, 16
    S, So = D ** 3, (D // 2) ** 3
    x = rng.standard_normal((N, c, S)).astype(np.float32)
    w = (rng.standard_normal((c, c, 27)) * 0.1).astype(np.float32); b = (rng.standard_normal(c) * 0.1).astype(np.float32)
    dq = to_mx(8, x); dw, db = DevBuf.from_numpy(w), DevBuf.from_numpy(b); dy = DevBuf(mx_bytes(8, N, c, So))
    _reg(H_, dq, 8); _reg(H_, dy, 8)
    try:
        H_.nn_conv3d_fwd(dq.ptr, shape5(N, c, D, D, D), dw.ptr, db.ptr, c, 3, 2, dy.ptr)
    finally:
        H_.nn_storage_forget(dq.ptr); H_.nn_storage_forget(dy.ptr)
    LP.check()
    direct, _ = gpu_conv(dq.to_numpy(np.uint8), 3, N, c, D, D, D, w, b, c, 3, stride=2)
    assert np.array_equal(dy.to_numpy(np.uint8), direct)
    ref = refnp.conv3d_f64(orc.mx_to_f32(8, dq.to_numpy(np.uint8), N, c, S).reshape(N, c, D, D, D), w, b, stride=2).reshape(N, c, So)
    assert _rel_l2(orc.mx_to_f32(8, direct, N, c, So), ref) < 0.08
    # the head
    ci, D = 16, 10
    S = D ** 3
    x = rng.standard_normal((N, ci, S)).astype(np.float32)
    w1 = rng.standard_normal((1, ci)).astype(np.float32) * 0.3; b1 = rng.standard_normal(1).astype(np.float32)
    dq = to_mx(8, x); dw, db = DevBuf.from_numpy(w1), DevBuf.from_numpy(b1); dl = DevBuf(N * S * 4)
    _reg(H_, dq, 8)
    try:
        H_.nn_conv3d_fwd(dq.ptr, shape5(N, ci, D, D, D), dw.ptr, db.ptr, 1, 1, 1, dl.ptr)
    finally:
        H_.nn_storage_forget(dq.ptr)
    LP.check()
    xd = orc.mx_to_f32(8, dq.to_numpy(np.uint8), N, ci, S).astype(np.float64)
    want = np.einsum("oc,ncs->nos", w1.astype(np.float64), xd) + b1[0]
    assert np.abs(dl.to_numpy(np.float32, (N, 1, S)) - want).max() / np.abs(want).max() < 1e-5


@pytest.mark.parametrize("dt", [8, 4])
def test_conv_of_silu_gn_and_its_statistics(gpu, dt):
    """tests/test_mx.c:96-135, tests/test_mx4.c:170-182: 16 -> 32 at 12 x 12 x 16 with GroupNorm + SiLU on the input (nn_conv3d_fwd_gn) and the
    output's statistics (nn_conv3d_fwd_gn_stats); more groups than channels clamp to the channel count."""
    H_ = _host()
    rng = np.random.default_rng(5)
    N, ci, co, D, Hh, W, G = 2, 16, 32, 12, 12, 16, 8
    S = D * Hh * W
    x = rng.standard_normal((N, ci, S)).astype(np.float32)
    w = (rng.standard_normal((co, ci, 27)) * 0.1).astype(np.float32); b = (rng.standard_normal(co) * 0.1).astype(np.float32)
    gam = rng.uniform(0.5, 1.5, ci).astype(np.float32); bet = rng.uniform(-.5, .5, ci).astype(np.float32)
    mean = rng.uniform(-.2, .2, N * G).astype(np.float32); rstd = rng.uniform(.8, 1.2, N * G).astype(np.float32)
    ldt = 3 if dt == 8 else 4
    dq = to_mx(dt, x); dw, db = DevBuf.from_numpy(w), DevBuf.from_numpy(b)
    dg = [DevBuf.from_numpy(a) for a in (gam, bet, mean, rstd)]
    dy, dy2 = DevBuf(mx_bytes(dt, N, co, S)), DevBuf(mx_bytes(dt, N, co, S))
    dm, dr = DevBuf(N * G * 4), DevBuf(N * G * 4)
    xs = shape5(N, ci, D, Hh, W)
    for t in (dq, dy, dy2):
        _reg(H_, t, dt)
    try:
        assert H_.nn_conv3d_fwd_gn(dq.ptr, xs, G, dg[0].ptr, dg[1].ptr, dg[2].ptr, dg[3].ptr, dw.ptr, db.ptr, co, dy.ptr) == 0
        assert H_.nn_conv3d_fwd_gn_stats(dq.ptr, xs, G, dg[0].ptr, dg[1].ptr, dg[2].ptr, dg[3].ptr, dw.ptr, db.ptr, co, dy2.ptr, G, 1e-5, dm.ptr, dr.ptr) == 0
    finally:
        for t in (dq, dy, dy2):
            H_.nn_storage_forget(t.ptr)
    LP.check()
    from gpuutil import dev_gn
    direct, sums = gpu_conv(dq.to_numpy(np.uint8), ldt, N, ci, D, Hh, W, w, b, co, ldt, cbits=dt, gp=dev_gn(gam, bet, mean, rstd, G), Go=G, stats=True)
    assert np.array_equal(dy.to_numpy(np.uint8), direct) and np.array_equal(dy2.to_numpy(np.uint8), direct)
    ln = (co // G) * S
    m = sums[:, :, 0] / ln; var = np.maximum(sums[:, :, 1] / ln - m * m, 0)
    assert np.allclose(dm.to_numpy(np.float32, (N, G)), m, rtol=1e-5, atol=1e-6) and np.allclose(dr.to_numpy(np.float32, (N, G)), 1 / np.sqrt(var + 1e-5), rtol=1e-5)
    # against the fp64 conv of silu(gn(decoded x)): the reference's bound 0.08 (fp8) / 0.25 (fp4)
    xd = orc.mx_to_f32(dt, dq.to_numpy(np.uint8), N, ci, S).astype(np.float64).reshape(N, G, ci // G, S)
    a = (rstd.reshape(N, G, 1, 1) * gam.reshape(1, G, ci // G, 1)).astype(np.float64)
    u = xd * a + (bet.reshape(1, G, ci // G, 1) - mean.reshape(N, G, 1, 1) * a)
    act = (u / (1 + np.exp(-u))).reshape(N, ci, D, Hh, W)
    ref = refnp.conv3d_f64(act, w, b).reshape(N, co, S)
    assert _rel_l2(orc.mx_to_f32(dt, direct, N, co, S), ref) < (0.08 if dt == 8 else 0.25)


@pytest.mark.parametrize("dt", [8, 4])
def test_split_input_conv(gpu, dt):
    """tests/test_mx.c:138-156, tests/test_mx4.c:252-262: the decoder's concat conv 80 + 64 -> 64 at 8 x 8 x 12 without GroupNorm, and 32 + 16 -> 16
    with one GroupNorm over all 48 channels and the output's statistics."""
    H_ = _host()
    rng = np.random.default_rng(6)
    N, D, Hh, W = 2, 8, 8, 12
    S = D * Hh * W
    ldt = 3 if dt == 8 else 4
    for ca, cb, co, G in ((80, 64, 64, 0), (32, 16, 16, 8)):
        xa = rng.standard_normal((N, ca, S)).astype(np.float32); xb = rng.standard_normal((N, cb, S)).astype(np.float32)
        w = (rng.standard_normal((co, ca + cb, 27)) * 0.05).astype(np.float32)
        da, db_ = to_mx(dt, xa), to_mx(dt, xb); dw = DevBuf.from_numpy(w); dy = DevBuf(mx_bytes(dt, N, co, S))
        gam = rng.uniform(0.5, 1.5, ca + cb).astype(np.float32); bet = rng.uniform(-.5, .5, ca + cb).astype(np.float32)
        mean = rng.uniform(-.2, .2, N * max(G, 1)).astype(np.float32); rstd = rng.uniform(.8, 1.2, N * max(G, 1)).astype(np.float32)
        dg = [DevBuf.from_numpy(a) for a in (gam, bet, mean, rstd)]
        dm, dr = DevBuf(N * 8 * 4), DevBuf(N * 8 * 4)
        for t in (da, db_, dy):
            _reg(H_, t, dt)
        try:
            if G:
                rc = H_.nn_conv3d_fwd_split(da.ptr, db_.ptr, ca, shape5(N, ca + cb, D, Hh, W), G, dg[0].ptr, dg[1].ptr, dg[2].ptr, dg[3].ptr, dw.ptr, None, co, dy.ptr, 8, 1e-5, dm.ptr, dr.ptr)
            else:
                rc = H_.nn_conv3d_fwd_split(da.ptr, db_.ptr, ca, shape5(N, ca + cb, D, Hh, W), 0, None, None, None, None, dw.ptr, None, co, dy.ptr, 0, 1e-5, None, None)
            assert rc == 0
        finally:
            for t in (da, db_, dy):
                H_.nn_storage_forget(t.ptr)
        LP.check()
        from gpuutil import dev_gn
        direct, sums = gpu_conv(da.to_numpy(np.uint8), ldt, N, ca + cb, D, Hh, W, w, None, co, ldt, cbits=dt, x2=db_.to_numpy(np.uint8), c_split=ca,
                                gp=dev_gn(gam, bet, mean, rstd, G) if G else None, Go=8 if G else 0, stats=bool(G))
        assert np.array_equal(dy.to_numpy(np.uint8), direct)
        want, _ = orc.conv3(da.to_numpy(np.uint8), ldt, N, ca + cb, D, Hh, W, w, None, co, 0, cbits=dt, x2=db_.to_numpy(np.uint8), c_split=ca,
                            gp=orc.gn(gam, bet, mean, rstd, G) if G else None)
        assert _rel_l2(orc.mx_to_f32(dt, direct, N, co, S), want.astype(np.float64)) < (0.05 if dt == 8 else 0.2)      # one output quantisation from the fp32-accumulated result
        if G:
            ln = (co // 8) * S
            m = sums[:, :, 0] / ln
            assert np.allclose(dm.to_numpy(np.float32, (N, 8)), m, rtol=1e-5, atol=1e-6)
