"""Helpers of the GPU parity tests: run an lp_* entry point through the C ABI on device buffers and fetch the result."""
import numpy as np

from ufsm_amd import lib, LP, shape5, gnp_t, split_t, DevBuf
import orc


def mx_bytes(bits, N, C, S):
    return (lib.lp_mx8_bytes if bits == 8 else lib.lp_mx4_bytes)(N, C, S)


def to_mx(bits, x):
    """fp32 [N][C][S] on the host -> device MX tensor through lp_f32_to_mx8 / 4."""
    N, C, S = x.shape
    dx = DevBuf.from_numpy(x.astype(np.float32))
    dq = DevBuf(mx_bytes(bits, N, C, S))
    (lib.lp_f32_to_mx8 if bits == 8 else lib.lp_f32_to_mx4)(dx.ptr, N, C, S, dq.ptr)
    LP.check()
    return dq


def dev_gn(gam, bet, mean, rstd, G):
    bufs = [DevBuf.from_numpy(np.asarray(a, np.float32)) for a in (gam, bet, mean, rstd)]
    g = LP.gn(*bufs, G=G)
    g._keep = bufs
    return g


def out_dims(D, H, W, stride):
    return ((D - 1) // 2 + 1, (H - 1) // 2 + 1, (W - 1) // 2 + 1) if stride == 2 else (D, H, W)


def gpu_conv(xq, xdt, N, Ci, D, H, W, w, b, Co, ydt, cbits=8, stride=1, x2=None, c_split=0, up=0, gp=None, gp2=None, Go=0, stats=False,
             stored_stats=0, wkey=0, fused=None):
    """xq / x2: host arrays holding the input as stored (MX bytes, fp32 or fp16 planes). Returns (y host array, sums [N][Go][2] or None)."""
    dxq = DevBuf.from_numpy(xq)
    dx2 = DevBuf.from_numpy(x2) if x2 is not None else None
    dw = DevBuf.from_numpy(w.astype(np.float32))
    db = DevBuf.from_numpy(b.astype(np.float32)) if b is not None else None
    Do, Ho, Wo = out_dims(D, H, W, stride)
    So = Do * Ho * Wo
    if ydt >= 3:
        ybytes, ydtype = mx_bytes(8 if ydt == 3 else 4, N, Co, So), np.uint8
    else:
        ybytes, ydtype = N * Co * So * (2 if ydt == 2 else 4), (np.uint16 if ydt == 2 else np.float32)
    dy = DevBuf(ybytes)
    dsum = DevBuf(N * max(Go, 1) * 2 * 24) if stats else None
    sp = split_t()
    if dx2 is not None:
        sp.x2, sp.c_split, sp.up = dx2.ptr, c_split, up
    if gp2 is not None:
        sp.gp2 = gp2
    sp.stored_stats, sp.wkey = stored_stats, wkey
    g = gp if gp is not None else gnp_t()
    xs = shape5(N, Ci, D, H, W)
    bp = db.ptr if db is not None else None
    sm = dsum.ptr if stats else None
    if fused is not None:
        act, ea, eb = fused
        dea = DevBuf.from_numpy(ea.astype(np.float32)) if ea is not None else None
        deb = DevBuf.from_numpy(eb.astype(np.float32)) if eb is not None else None
        lib.mi_conv_fwd_fused(cbits, dxq.ptr, xdt, xs, dw.ptr, bp, Co, dy.ptr, ydt, dea.ptr if dea else None, deb.ptr if deb else None, act, g, sm, Go if stats else 0, sp)
    elif stride == 2:
        rc = lib.lp_conv_fwd_s2_f8(dxq.ptr, xdt, xs, dw.ptr, bp, Co, dy.ptr, ydt, shape5(N, Co, Do, Ho, Wo), g)
        assert rc in (0, 3)
    else:
        f = lib.lp_conv_fwd_f8 if cbits == 8 else lib.lp_conv_fwd_f4
        assert f(dxq.ptr, xdt, xs, dw.ptr, bp, Co, dy.ptr, ydt, g, sm, Go if stats else 0, sp) == 0
    LP.check()
    y = dy.to_numpy(ydtype)
    if ydt < 3:
        y = y.reshape(N, Co, So)
    sums = None
    if stats:
        ds = DevBuf(N * Go * 2 * 8)
        lib.mi_gn_sums_get(dsum.ptr, N * Go * 2, ds.ptr)
        sums = ds.to_numpy(np.float64, (N, Go, 2))
    return y, sums


def mx_decode_host(bits, q, N, C, S):
    return orc.mx_to_f32(bits, q, N, C, S)


def code_mismatch_fraction(bits, got, want, N, C, S):
    """Fraction of elements whose decoded values differ, and whether every differing element is a neighbouring code of the oracle's.
    A last-bit difference of the fp32 accumulation can flip one rounding, or the block's exponent when the block amax sits on a power of
    two: then every element of the block moves by at most one step of the coarser grid. Anything larger is a bug."""
    g = mx_decode_host(bits, got, N, C, S); w = mx_decode_host(bits, want, N, C, S)
    diff = g != w
    if not diff.any():
        return 0.0, True
    bw = 8 if C <= 8 else 16 if C <= 16 else 32
    nb = (C + bw - 1) // bw
    pad = nb * bw - C
    wp = np.pad(np.abs(w), ((0, 0), (0, pad), (0, 0))).reshape(N, nb, bw, S)
    amax = np.repeat(wp.max(axis=2), bw, axis=1)[:, :C, :]              # the block amax at every element
    rel, floor = (0.26, 2.0 ** -7) if bits == 8 else (0.67, 0.18)       # one code step relative to the value / to the block maximum
    ok = np.abs(g - w) <= rel * np.maximum(np.abs(w), np.abs(g)) + floor * amax
    return float(diff.mean()), bool(ok[diff].all())
