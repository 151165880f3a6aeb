"""ctypes binding of the CPU oracle (oracle/liboracle.so). Test infrastructure only."""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(ROOT, "oracle", "liboracle.so")


class orc_gn_t(C.Structure):
    _fields_ = [("gamma", C.c_void_p), ("beta", C.c_void_p), ("mean", C.c_void_p), ("rstd", C.c_void_p), ("G", C.c_int),
                ("zs", C.c_int), ("zo", C.c_int), ("ns", C.c_int), ("zhw", C.c_int)]


class orc_conv_t(C.Structure):
    _fields_ = [("x", C.c_void_p), ("xdt", C.c_int), ("N", C.c_int), ("Ci", C.c_int), ("D", C.c_int), ("H", C.c_int), ("W", C.c_int),
                ("x2", C.c_void_p), ("c_split", C.c_int), ("up", C.c_int), ("gp", orc_gn_t), ("gp2", orc_gn_t),
                ("w", C.c_void_p), ("b", C.c_void_p), ("Co", C.c_int), ("stride", C.c_int), ("cbits", C.c_int),
                ("y", C.c_void_p), ("ydt", C.c_int), ("osum", C.c_void_p), ("Go", C.c_int), ("stored_stats", C.c_int),
                ("acc64", C.c_int), ("fused_act", C.c_int), ("ep_a", C.c_void_p), ("ep_b", C.c_void_p),
                ("z0", C.c_int), ("z1", C.c_int), ("stem_tile", C.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            import subprocess
            subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "liboracle.so"])
        L = C.CDLL(LIB_PATH)
        L.orc_mx_exp.restype = C.c_int; L.orc_mx_exp.argtypes = [C.c_float, C.c_float]
        L.orc_exp2i.restype = C.c_float; L.orc_exp2i.argtypes = [C.c_int]
        L.orc_mx_scale.restype = C.c_float; L.orc_mx_scale.argtypes = [C.c_uint]
        for n in ("orc_enc_e4m3", "orc_enc_e2m1", "orc_ref_e4m3", "orc_ref_e2m1"):
            getattr(L, n).restype = C.c_uint; getattr(L, n).argtypes = [C.c_float]
        for n in ("orc_dec_e4m3", "orc_dec_e2m1"):
            getattr(L, n).restype = C.c_float; getattr(L, n).argtypes = [C.c_uint]
        L.orc_enc_sweep.restype = C.c_uint64; L.orc_enc_sweep.argtypes = [C.c_uint32, C.c_uint64, C.c_uint32, C.POINTER(C.c_uint32)]
        L.orc_mx_bytes.restype = C.c_size_t; L.orc_mx_bytes.argtypes = [C.c_int, C.c_int, C.c_int, C.c_size_t]
        L.orc_store_row.restype = C.c_uint8; L.orc_store_row.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_int]
        L.orc_load_row.restype = None; L.orc_load_row.argtypes = [C.c_int, C.c_void_p, C.c_uint8, C.c_int, C.c_void_p]
        L.orc_f32_to_mx.restype = None; L.orc_f32_to_mx.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_size_t, C.c_void_p]
        L.orc_h16_to_mx.restype = None; L.orc_h16_to_mx.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_size_t, C.c_void_p]
        L.orc_mx_to_f32.restype = None; L.orc_mx_to_f32.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_size_t, C.c_void_p]
        L.orc_pred_input_mx.restype = None
        L.orc_pred_input_mx.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_float, C.c_float, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int]
        L.orc_prep_w.restype = None
        L.orc_prep_w.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_conv3.restype = C.c_int; L.orc_conv3.argtypes = [C.POINTER(orc_conv_t)]
        L.orc_conv3_staged.restype = C.c_int; L.orc_conv3_staged.argtypes = [C.POINTER(orc_conv_t), C.c_void_p]
        L.orc_gn_row.restype = C.c_int; L.orc_gn_row.argtypes = [C.POINTER(orc_gn_t), C.c_int, C.c_int]
        L.orc_set_w4_2d.restype = None; L.orc_set_w4_2d.argtypes = [C.c_int]
        L.orc_fakeq_w4.restype = None; L.orc_fakeq_w4.argtypes = [C.c_void_p] + [C.c_int] * 5
        L.orc_conv2.restype = C.c_int; L.orc_conv2.argtypes = [C.POINTER(orc_conv_t), C.c_int]
        L.orc_gn_finalize.restype = None; L.orc_gn_finalize.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.c_float, C.c_void_p, C.c_void_p]
        L.orc_gn_sums_mx.restype = None; L.orc_gn_sums_mx.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t]
        L.orc_gn_silu_apply_mx.restype = None; L.orc_gn_silu_apply_mx.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_size_t, orc_gn_t, C.c_void_p, C.c_int]
        L.orc_up2_mx.restype = None; L.orc_up2_mx.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, orc_gn_t, C.c_void_p, C.c_int]
        L.orc_conv1_mx.restype = None; L.orc_conv1_mx.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_size_t, C.c_void_p, C.c_void_p, C.c_int, orc_gn_t, C.c_void_p]
        L.orc_act_ab.restype = C.c_float; L.orc_act_ab.argtypes = [C.c_float, C.c_float, C.c_float]
        L.orc_f32_to_h16.restype = C.c_uint16; L.orc_f32_to_h16.argtypes = [C.c_float]
        L.orc_h16_to_f32.restype = C.c_float; L.orc_h16_to_f32.argtypes = [C.c_uint16]
        L.orc_threads.restype = C.c_int
        L.orc_set_align_bits.restype = None; L.orc_set_align_bits.argtypes = [C.c_int]
        L.orc_set_act_mode.restype = None; L.orc_set_act_mode.argtypes = [C.c_int]
        L.orc_mx_gemm.restype = C.c_int
        L.orc_mx_gemm.argtypes = [C.c_int] * 6 + [C.c_void_p, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_void_p]
        L.orc_pred_place.restype = None; L.orc_pred_place.argtypes = [C.c_void_p, C.c_void_p] + [C.c_int] * 12 + [C.c_void_p]
        L.orc_feather_blend.restype = None; L.orc_feather_blend.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
        L.orc_ln_fwd.restype = None; L.orc_ln_fwd.argtypes = [C.c_void_p] * 6 + [C.c_long, C.c_int]
        L.orc_glu_fwd.restype = None; L.orc_glu_fwd.argtypes = [C.c_void_p, C.c_void_p, C.c_long, C.c_int]
        L.orc_cs_to_tok.restype = None; L.orc_cs_to_tok.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_long, C.c_int]
        L.orc_tok_to_cs.restype = None; L.orc_tok_to_cs.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_long, C.c_int]
        L.orc_fa_pack.restype = None; L.orc_fa_pack.argtypes = [C.c_void_p] * 7 + [C.c_int] * 7 + [C.c_float]
        L.orc_block_layout.restype = C.c_size_t; L.orc_block_layout.argtypes = [C.c_int, C.c_int, C.c_size_t, C.c_void_p]
        L.orc_block_fwd.restype = C.c_int; L.orc_block_fwd.argtypes = [C.c_int] * 6 + [C.c_float, C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int] * 4
        L.orc_peg_fwd.restype = None; L.orc_peg_fwd.argtypes = [C.c_void_p] * 4 + [C.c_int] * 7
        L.orc_block_fwd_vr.restype = C.c_int; L.orc_block_fwd_vr.argtypes = [C.c_int] * 6 + [C.c_float, C.c_void_p, C.c_void_p, C.c_void_p] + [C.c_int] * 5 + [C.c_void_p, C.c_void_p]
        L.orc_fa8_fwd.restype = None; L.orc_fa8_fwd.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int]
        _lib = L
    return _lib


def ptr(a):
    return a.ctypes.data if a is not None else None


def gn(gamma=None, beta=None, mean=None, rstd=None, G=0, slab=None):
    """slab = (zs, zo, ns, zhw): mean / rstd hold one row per (sample, z-slab), [n][ns][G] (src/nn_lp.h:15-18)."""
    g = orc_gn_t()
    if G:
        g.gamma, g.beta, g.mean, g.rstd, g.G = ptr(gamma), ptr(beta), ptr(mean), ptr(rstd), G
        if slab:
            g.zs, g.zo, g.ns, g.zhw = slab
    return g


def mx_bytes(bits, N, C, S):
    return lib().orc_mx_bytes(bits, N, C, S)


def f32_to_mx(bits, x, N, C, S):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.zeros(mx_bytes(bits, N, C, S), dtype=np.uint8)
    lib().orc_f32_to_mx(bits, ptr(x), N, C, S, ptr(y))
    return y


def mx_to_f32(bits, q, N, C, S):
    q = np.ascontiguousarray(q, dtype=np.uint8)
    y = np.zeros((N, C, S), dtype=np.float32)
    lib().orc_mx_to_f32(bits, ptr(q), N, C, S, ptr(y))
    return y


def conv3(x, xdt, N, Ci, D, H, W, w, b, Co, ydt, cbits=8, stride=1, x2=None, c_split=0, up=0, gp=None, gp2=None, Go=0, want_stats=False,
          stored_stats=0, acc64=0, fused_act=0, ep_a=None, ep_b=None, z0=0, z1=0, stem_tile=0):
    """Runs the oracle conv; returns (y, sums or None). y: uint8 MX bytes, float32 or uint16 (fp16 bits) planes [N][Co][So]."""
    c = orc_conv_t()
    keep = [x, x2, w, b, ep_a, ep_b]
    c.x, c.xdt, c.N, c.Ci, c.D, c.H, c.W = ptr(x), xdt, N, Ci, D, H, W
    c.x2, c.c_split, c.up = ptr(x2), c_split, up
    c.gp = gp if gp is not None else orc_gn_t(); c.gp2 = gp2 if gp2 is not None else orc_gn_t()
    c.w, c.b, c.Co, c.stride, c.cbits = ptr(w), ptr(b), Co, stride, cbits
    Do, Ho, Wo = ((D - 1) // 2 + 1, (H - 1) // 2 + 1, (W - 1) // 2 + 1) if stride == 2 else (D, H, W)
    So = Do * Ho * Wo
    if ydt >= 3:
        y = np.zeros(mx_bytes(8 if ydt == 3 else 4, N, Co, So), dtype=np.uint8)
    elif ydt == 2:
        y = np.zeros((N, Co, So), dtype=np.uint16)
    else:
        y = np.zeros((N, Co, So), dtype=np.float32)
    sums = np.zeros((N, max(Go, 1), 2), dtype=np.float64) if want_stats else None
    c.y, c.ydt, c.osum, c.Go, c.stored_stats = ptr(y), ydt, ptr(sums), Go, stored_stats
    c.acc64, c.fused_act, c.ep_a, c.ep_b, c.z0, c.z1, c.stem_tile = acc64, fused_act, ptr(ep_a), ptr(ep_b), z0, z1, stem_tile
    rc = lib().orc_conv3(C.byref(c))
    assert rc == 0, rc
    del keep
    return y, sums


def conv2(x, xdt, N, Ci, D, H, W, w, b, Co, ydt, up, cbits=8, gp=None, acc64=0):
    """The oracle's 2x2x2 stride-2 conv (up 0, w [Co][Ci][8]) or transposed conv (up 1, w [Ci][Co][8]) of an MX tensor; y as conv3."""
    c = orc_conv_t()
    c.x, c.xdt, c.N, c.Ci, c.D, c.H, c.W = ptr(x), xdt, N, Ci, D, H, W
    c.gp = gp if gp is not None else orc_gn_t(); c.gp2 = orc_gn_t()
    c.w, c.b, c.Co, c.stride, c.cbits, c.acc64 = ptr(w), ptr(b), Co, 1, cbits, acc64
    So = (8 * D * H * W) if up else (D // 2) * (H // 2) * (W // 2)
    y = np.zeros(mx_bytes(8 if ydt == 3 else 4, N, Co, So), dtype=np.uint8) if ydt >= 3 else np.zeros((N, Co, So), dtype=np.uint16 if ydt == 2 else np.float32)
    c.y, c.ydt = ptr(y), ydt
    rc = lib().orc_conv2(C.byref(c), up)
    assert rc == 0, rc
    return y


def mx_gemm(bits, ta, tb, M, N, K, A, B, C0=None, beta=0.0, bias=None, res=None):
    """C = op(A) op(B) + bias + res + beta C0 with MX-quantised operands; A, B float32 in their stored (possibly transposed) layout."""
    A = np.ascontiguousarray(A, dtype=np.float32); B = np.ascontiguousarray(B, dtype=np.float32)
    out = np.zeros((M, N), np.float32) if C0 is None else np.array(C0, dtype=np.float32, copy=True)
    rc = lib().orc_mx_gemm(bits, ta, tb, M, N, K, ptr(A), ptr(B), ptr(out), beta, ptr(bias), ptr(res))
    assert rc == 0
    return out


def fa8_fwd(qkvh, nseq, S, H):
    """qkvh: uint16 (fp16 bits) [3][H][nseq * S + 64][48] -> (o [nseq * S][H * 48], lse [nseq][H][S]) float32."""
    qkvh = np.ascontiguousarray(qkvh, dtype=np.uint16)
    assert qkvh.shape == (3, H, nseq * S + 64, 48)
    o = np.zeros((nseq * S, H * 48), np.float32); lse = np.zeros((nseq, H, S), np.float32)
    lib().orc_fa8_fwd(ptr(qkvh), ptr(o), ptr(lse), nseq, S, H, H * 48)
    return o, lse


def pred_place(lg, ct, D, W, hz, halo, o, e, shard, iso=1, dsh=None):
    lg = np.ascontiguousarray(lg, np.float32); ct = np.ascontiguousarray(ct, np.uint8)
    out = np.zeros((shard, shard, shard), np.uint8) if dsh is None else dsh
    lib().orc_pred_place(ptr(lg), ptr(ct), D, W, hz, halo, o[0], o[1], o[2], e[0], e[1], e[2], shard, iso, ptr(out))
    return out


def feather_blend(E, present, S, B, nss, bn):
    E = np.ascontiguousarray(E, np.uint8); present = np.ascontiguousarray(present, np.uint8)
    nss_a = np.asarray(nss, np.int64); bn_a = np.asarray(bn, np.int64)
    out = np.zeros(tuple(int(v) for v in bn), np.uint8)
    lib().orc_feather_blend(ptr(E), ptr(present), S, B, ptr(nss_a), ptr(bn_a), ptr(out))
    return out


BLOCK_FIELDS = ("ln1g", "ln1b", "wqkv", "bqkv", "qg", "kg", "wo", "bo", "ln2g", "ln2b", "w1", "b1", "w2", "b2")


def block_layout(Cc, F, off=0):
    o = np.zeros(14, np.uint64)
    end = lib().orc_block_layout(Cc, F, off, ptr(o))
    return dict(zip(BLOCK_FIELDS, (int(v) for v in o))), int(end)


def fa_pack(qkv, qg, kg, nseq, S, Hh, W, nreg, Cc, rope, base=100.0):
    H = Cc // 48; T = nseq * S
    qkv = np.ascontiguousarray(qkv, np.float32); qg = np.ascontiguousarray(qg, np.float32); kg = np.ascontiguousarray(kg, np.float32)
    qh = np.zeros((3, H, T + 64, 48), np.uint16); rq = np.zeros((T, H), np.float32); rk = np.zeros((T, H), np.float32); amx = np.zeros(4, np.float32)
    lib().orc_fa_pack(ptr(qkv), ptr(qg), ptr(kg), ptr(qh), ptr(rq), ptr(rk), ptr(amx), nseq, S, Hh, W, nreg, Cc, rope, base)
    return qh, rq, rk, amx


def peg_fwd(x, w, b, nseq, S, D, Hh, W, nreg):
    """token rows x [nseq * S][C] -> x + b + depthwise 3^3 conv on the grid tokens; w [C][27], b [C]"""
    x = np.ascontiguousarray(x, np.float32); w = np.ascontiguousarray(w, np.float32); b = np.ascontiguousarray(b, np.float32)
    y = np.zeros_like(x)
    lib().orc_peg_fwd(ptr(x), ptr(y), ptr(w), ptr(b), nseq, S, D, Hh, W, nreg, x.shape[-1])
    return y


def block_fwd(bits, Cc, H, F, rope, nreg, base, P, x, nseq, S, Hh, W, vr=0, v1=None, lam=None):
    """vr 1: the block's V rows are written into v1 ([T][C] float32, in place); vr 2: V <- v + lam[head] (v1 - v) (src/nn_attn.cu:535-542)"""
    P = np.ascontiguousarray(P, np.float32); x = np.ascontiguousarray(x, np.float32)
    y = np.zeros_like(x)
    if not vr:
        assert lib().orc_block_fwd(bits, Cc, H, F, rope, nreg, base, ptr(P), ptr(x), ptr(y), nseq, S, Hh, W) == 0
        return y
    assert v1.dtype == np.float32 and v1.flags.c_contiguous and v1.size == x.size
    lam = np.ascontiguousarray(lam if lam is not None else np.zeros(H), np.float32)
    assert lib().orc_block_fwd_vr(bits, Cc, H, F, rope, nreg, base, ptr(P), ptr(x), ptr(y), nseq, S, Hh, W, vr, ptr(v1), ptr(lam)) == 0
    return y
