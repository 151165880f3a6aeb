"""Independent numpy statements of the MX format, written from the format's definition (not from the oracle's code):
nearest-grid rounding with ties to the even code, the ceil(log2) scale rule with its fix-up, a direct fp64 convolution.
They pin the oracle the way the reference's host checkers (tests/test_mx4.c:36-54, tests/test_mx4_wide.c:122-148, :179-204) pin its kernels."""
import numpy as np

E2M1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], dtype=np.float64)
E4M3 = np.array([(m * 2.0 ** -9) if e == 0 else (8 + m) * 2.0 ** (e - 10) for e in range(16) for m in range(8)][:127], dtype=np.float64)  # codes 0..126


def round_to_grid(a, grid):
    """|a| (float64 array) -> index of the nearest grid value, exact ties to the even index; beyond the last value saturates."""
    a = np.asarray(a, dtype=np.float64)
    idx = np.searchsorted(grid, a, side="right") - 1          # largest i with grid[i] <= a
    idx = np.clip(idx, 0, len(grid) - 1)
    hi = np.clip(idx + 1, 0, len(grid) - 1)
    dlo, dhi = a - grid[idx], grid[hi] - a
    up = (dhi < dlo) | ((dhi == dlo) & (idx % 2 == 1))
    out = np.where(up & (hi != idx), hi, idx)
    return np.where(a >= grid[-1], len(grid) - 1, out)


def scale_exp(amax, qmax):
    """e = ceil(log2(amax / qmax)) with the fix-up of tests/test_mx4.c:51, clamped to [-126, 126]; amax == 0 -> -126.
    Evaluated in float64 on amax * float32(1 / qmax), the product the reference forms (src/lp_common.cuh:492-500)."""
    inv = np.float32(1.0) / np.float32(qmax)
    p = (np.asarray(amax, dtype=np.float32) * inv).astype(np.float64)
    e = np.full(p.shape, -126, dtype=np.int64)
    nz = p > 0
    with np.errstate(divide="ignore"):
        e[nz] = np.ceil(np.log2(p[nz])).astype(np.int64)
    # log2 rounding fix-up: the smallest e with p <= 2^e
    e = np.where(nz & (np.ldexp(1.0, np.clip(e, -1000, 1000)) < p), e + 1, e)
    e = np.where(nz & (np.ldexp(1.0, np.clip(e - 1, -1000, 1000)) >= p), e - 1, e)
    return np.clip(e, -126, 126)


def quantize_block(v, bits):
    """v: [..., bw] float32 finite -> (decoded float32 values, scale exponent e) of the MX block (round to nearest)."""
    v = np.asarray(v, dtype=np.float32)
    amax = np.abs(v).max(axis=-1)
    qmax = 448.0 if bits == 8 else 6.0
    e = scale_exp(amax, qmax)
    grid = E4M3 if bits == 8 else E2M1
    scaled = np.abs(v.astype(np.float64)) * np.ldexp(1.0, -e)[..., None]       # exact power-of-two scaling
    q = grid[round_to_grid(scaled, grid)] * np.ldexp(1.0, e)[..., None]
    return (np.sign(v) * q).astype(np.float32), e


def mx_quant_tensor(x, bits):
    """x: [N][C][S] -> decoded MX tensor (the host_mx4 of tests/test_mx4.c:46-54 for either format)."""
    N, C, S = x.shape
    bw = 8 if C <= 8 else 16 if C <= 16 else 32
    y = np.zeros_like(x)
    for b0 in range(0, C, bw):
        blk = np.moveaxis(x[:, b0:b0 + bw, :], 1, -1)          # [N][S][bw']
        q, _ = quantize_block(blk, bits)
        y[:, b0:b0 + bw, :] = np.moveaxis(q, -1, 1)
    return y


def conv3d_f64(x, w, b=None, stride=1):
    """x: [N][Ci][D][H][W], w: [Co][Ci][27] (tap = kz*9+ky*3+kx), pad 1 -> float64 [N][Co][Do][Ho][Wo] (tests/test_nn.c:20-32)."""
    N, Ci, D, H, W = x.shape
    Co = w.shape[0]
    xp = np.zeros((N, Ci, D + 2, H + 2, W + 2), dtype=np.float64)
    xp[:, :, 1:-1, 1:-1, 1:-1] = x
    Do, Ho, Wo = ((D - 1) // stride + 1, (H - 1) // stride + 1, (W - 1) // stride + 1)
    y = np.zeros((N, Co, Do, Ho, Wo), dtype=np.float64)
    wd = w.astype(np.float64).reshape(Co, Ci, 3, 3, 3)
    for kz in range(3):
        for ky in range(3):
            for kx in range(3):
                sl = xp[:, :, kz:kz + stride * (Do - 1) + 1:stride, ky:ky + stride * (Ho - 1) + 1:stride, kx:kx + stride * (Wo - 1) + 1:stride]
                y += np.einsum("oc,ncdhw->nodhw", wd[:, :, kz, ky, kx], sl)
    if b is not None:
        y += np.asarray(b, dtype=np.float64)[None, :, None, None, None]
    return y


def up2_f64(x):
    """x: [N][C][D][H][W] -> trilinear 2x, align_corners=false, edge clamp: out[o] = .75 in[o/2] + .25 in[o/2 -+ 1] per axis."""
    y = x.astype(np.float64)
    for ax in (2, 3, 4):
        n = y.shape[ax]
        o = np.arange(2 * n)
        near = o // 2
        far = np.clip(near + np.where(o % 2 == 1, 1, -1), 0, n - 1)
        y = 0.75 * np.take(y, near, axis=ax) + 0.25 * np.take(y, far, axis=ax)
    return y


def gen_exact(rng, shape, block_axis=1, block=32, force6=True):
    """Values on the signed e2m1 grid with a +-6 in every 32-channel block (tests/test_mx4_wide.c:81-98): all block scales are 1 and
    every partial sum of a conv is exact in fp32."""
    g = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], dtype=np.float32)
    x = g[rng.integers(0, 8, shape)] * rng.choice(np.array([-1, 1], dtype=np.float32), shape)
    if force6:
        x = np.moveaxis(x, block_axis, -1)
        C = x.shape[-1]
        flat = x.reshape(-1, C)
        for c0 in range(0, C, block):
            n = min(block, C - c0)
            idx = rng.integers(0, n, flat.shape[0])
            flat[np.arange(flat.shape[0]), c0 + idx] = rng.choice(np.array([-6, 6], dtype=np.float32), flat.shape[0])
        x = np.moveaxis(flat.reshape(x.shape), -1, block_axis)
    return np.ascontiguousarray(x, dtype=np.float32)
