"""GPU parity of the 2-D fp4 weight scales (lp_set_w4_2d, src/lp_f4fwd.cu:67-83), the in-place fake quantisation (lp_fakeq_w4, src/lp_mx_cvt.cu:369-395)
and the U-Net's cfg.w4_2d forward copy (src/unet.c:5292-5326) against the oracle (pinned in tests/test_oracle_w4_2d.py)."""
import numpy as np
import pytest

from ufsm_amd import lib, LP, DevBuf
from gpuutil import gpu_conv
import orc

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("Co,Ci,T,Bo,Bi", [(64, 64, 27, 32, 32), (48, 80, 27, 32, 32), (20, 40, 8, 32, 32), (32, 64, 27, 1, 32), (64, 32, 3, 16, 1), (256, 384, 27, 32, 32)])
def test_fakeq_bit_exact(gpu, Co, Ci, T, Bo, Bi):
    rng = np.random.default_rng(Co * 7 + Ci)
    w = (rng.standard_normal((Co, Ci, T)) * np.exp(rng.uniform(-3, 3, (Co, 1, 1)))).astype(np.float32)
    want = w.copy(); orc.lib().orc_fakeq_w4(orc.ptr(want), Co, Ci, T, Bo, Bi)
    d = DevBuf.from_numpy(w)
    lib.lp_fakeq_w4(d.ptr, Co, Ci, T, Bo, Bi); LP.check()
    assert np.array_equal(d.to_numpy(np.float32).reshape(w.shape), want)
    if Bo == Bi:
        d = DevBuf.from_numpy(w); lib.nn_fakeq_w4_2d(d.ptr, Co, Ci, T, Bo); LP.check()
        assert np.array_equal(d.to_numpy(np.float32).reshape(w.shape), want)


@pytest.mark.parametrize("Ci,Co,dims,split", [(64, 48, (4, 8, 16), 0), (128, 128, (4, 8, 16), 0), (96, 32, (8, 8, 32), 64), (40, 64, (2, 6, 10), 0)])
def test_conv_with_2d_scales(gpu, Ci, Co, dims, split):
    """lp_conv_fwd_f4 under lp_set_w4_2d(1) against the oracle under the same setting (e2m1 products add exactly in the matrix cores: 1e-5 of the
    fp64 accumulation only if every weight code and scale agrees), on every fp4 kernel family: general, wide, the row kernel with a split input.
    And the reference's invariant on the device: raw weights under 2-D scales = fake-quantised weights under per-channel scales, byte for byte."""
    rng = np.random.default_rng(Ci + Co)
    D, H, W = dims
    N, S = 1, D * H * W
    x = rng.standard_normal((N, Ci, S)).astype(np.float32)
    w = (rng.standard_normal((Co, Ci, 27)) * np.exp(rng.uniform(-2, 2, (Co, 1, 1))) * 0.05).astype(np.float32)
    if split:
        qa, qb = orc.f32_to_mx(4, x[:, :split], N, split, S), orc.f32_to_mx(4, x[:, split:], N, Ci - split, S)
        kw = dict(x2=qb, c_split=split)
    else:
        qa, kw = orc.f32_to_mx(4, x, N, Ci, S), {}
    lib.lp_set_w4_2d(1); orc.lib().orc_set_w4_2d(1)
    try:
        want, _ = orc.conv3(qa, 4, N, Ci, D, H, W, w, None, Co, 0, cbits=4, acc64=1, **kw)
        got, _ = gpu_conv(qa, 4, N, Ci, D, H, W, w, None, Co, 0, cbits=4, **kw)
        gq, _ = gpu_conv(qa, 4, N, Ci, D, H, W, w, None, Co, 4, cbits=4, **kw)
    finally:
        lib.lp_set_w4_2d(0); orc.lib().orc_set_w4_2d(0)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err < 1e-5, err
    fq = w.copy(); orc.lib().orc_fakeq_w4(orc.ptr(fq), Co, Ci, 27, 32, 32)
    if not split:                                                   # (a split input pads each segment to 32: its blocks are not the flat tensor's)
        g1, _ = gpu_conv(qa, 4, N, Ci, D, H, W, fq, None, Co, 4, cbits=4, **kw)
        assert np.array_equal(g1, gq)
    raw, _ = gpu_conv(qa, 4, N, Ci, D, H, W, w, None, Co, 0, cbits=4, **kw)
    assert np.abs(raw - got).max() > 1e-4 * np.abs(want).max()      # the setting is off again and the per-channel scales give other numbers


def test_unet_w4_2d_forward_copy(gpu, tmp_path):
    """A cfg.w4_2d net forwards with its stride-1 3^3 conv weights (not the network input conv, not the down convs) rounded per 32 x 32 block: the
    same logits, byte for byte, as a plain net holding the oracle's fake-quantised weights; the copy follows set_params, the EMA switch and a
    checkpoint round trip (whose header carries the key)."""
    from ufsm_amd.unet import UNet, make_cfg
    widths, N, D = [32, 64], 1, 16
    rng = np.random.default_rng(4)
    x = rng.standard_normal((N, 4, D ** 3)).astype(np.float32)
    xq = DevBuf.from_numpy(orc.f32_to_mx(8, x, N, 4, D ** 3))
    a = UNet(make_cfg(4, widths, head_out=2, act_dt=4, w4_2d=1), N, D, D, D, seed=3)
    b = UNet(make_cfg(4, widths, head_out=2, act_dt=4), N, D, D, D, seed=3)
    p = a.params()
    p[:200000] *= np.exp(rng.uniform(-1.5, 1.5, 200000)).astype(np.float32)      # spread the rows' magnitudes so the two scale rules differ
    a.set_params(p)
    # the plain net's weights: the oracle's fake quantisation of the convs the reference rounds (parameter order: encoder blocks, downs, decoder blocks, head)
    q = p.copy(); off = 0
    def conv(ci, co, fq):
        nonlocal off
        n = co * ci * 27
        if fq:
            blk = np.ascontiguousarray(q[off:off + n]); orc.lib().orc_fakeq_w4(orc.ptr(blk), co, ci, 27, 32, 32); q[off:off + n] = blk
        off += n + co
    for i, wd in enumerate(widths):
        conv(widths[i - 1] if i else 4, wd, i > 0); off += 2 * wd; conv(wd, wd, True); off += 2 * wd
    for i in range(len(widths) - 1):
        conv(widths[i], widths[i], False)
    for i in range(len(widths) - 1):
        conv(widths[i + 1] + widths[i], widths[i], True); off += 2 * widths[i]; conv(widths[i], widths[i], True); off += 2 * widths[i]
    b.set_params(q)
    nb = a.logits_bytes()
    la, lb, lc = DevBuf(nb), DevBuf(nb), DevBuf(nb)
    assert a.forward_x(xq.ptr, la.ptr) == 0 and b.forward_x(xq.ptr, lb.ptr) == 0
    LP.check()
    assert np.array_equal(la.to_numpy(np.uint8), lb.to_numpy(np.uint8))
    b.set_params(p)
    assert b.forward_x(xq.ptr, lc.ptr) == 0
    assert not np.array_equal(lc.to_numpy(np.uint8), lb.to_numpy(np.uint8))      # (the unrounded weights give other logits: the copy matters)
    # checkpoint round trip into a fresh w4_2d net; a plain net refuses the file
    path = str(tmp_path / "w.ckpt")
    assert a.save(path, step=5) == 0
    c = UNet(make_cfg(4, widths, head_out=2, act_dt=4, w4_2d=1), N, D, D, D, seed=9)
    assert c.load(path) == 5
    assert c.forward_x(xq.ptr, lc.ptr) == 0
    assert np.array_equal(lc.to_numpy(np.uint8), la.to_numpy(np.uint8))
    assert b.load(path) == -1
    LP.check()
