"""ctypes mirror of include/mi_lp.h (the forward subset of the reference's src/nn_lp.h).

Everything here is plumbing: argument marshalling and device-buffer helpers. All arithmetic happens in the HIP library.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libufsm_lp.so")
MI_GN_SLOT_BYTES = 24


class shape5(C.Structure):  # src/nn.h:21
    _fields_ = [("n", C.c_int), ("c", C.c_int), ("d", C.c_int), ("h", C.c_int), ("w", C.c_int)]


class gnp_t(C.Structure):  # src/nn_lp.h:15
    _fields_ = [("gamma", C.c_void_p), ("beta", C.c_void_p), ("mean", C.c_void_p), ("rstd", C.c_void_p),
                ("G", C.c_int), ("zs", C.c_int), ("zo", C.c_int), ("ns", C.c_int), ("zhw", C.c_int)]


class split_t(C.Structure):  # src/nn_lp.h:32
    _fields_ = [("x2", C.c_void_p), ("c_split", C.c_int), ("y2", C.c_void_p), ("o_split", C.c_int), ("accum", C.c_int),
                ("gp2", gnp_t), ("up", C.c_int16), ("yD", C.c_int16), ("sr", C.c_uint), ("wkey", C.c_uint),
                ("zlo", C.c_int), ("zhi", C.c_int), ("stored_stats", C.c_int), ("osr", C.c_uint),
                ("zi0", C.c_int16), ("Di", C.c_int16), ("o_pad", C.c_int16), ("zw0", C.c_int16), ("zw1", C.c_int16), ("yzo", C.c_int16)]


assert C.sizeof(split_t) <= 128  # src/nn_lp.h:41


class skipm_t(C.Structure):  # src/nn_lp.h:44
    _fields_ = [("m", C.c_void_p), ("mi", C.c_void_p), ("my", C.c_int), ("mx", C.c_int), ("zoff", C.c_int)]


_P, _I, _Z, _F = C.c_void_p, C.c_int, C.c_size_t, C.c_float
_PROTOS = {
    "lp_conv_fwd_f8": (_I, [_P, _I, shape5, _P, _P, _I, _P, _I, gnp_t, _P, _I, split_t]),
    "lp_conv_fwd_f4": (_I, [_P, _I, shape5, _P, _P, _I, _P, _I, gnp_t, _P, _I, split_t]),
    "lp_conv_fwd_s2_f8": (_I, [_P, _I, shape5, _P, _P, _I, _P, _I, shape5, gnp_t]),
    "lp_wmemo_step": (None, [C.c_uint]),
    "lp_wmemo_clear": (None, []),
    "mi_conv_s2_wkey": (None, [C.c_uint]),
    "mi_conv_stem_zc": (None, [C.c_int]),
    "mi_conv_split": (None, [C.c_int]),
    "mi_conv_s2_direct": (None, [C.c_int]),
    "mi_conv1_matrix": (None, [C.c_int]),
    "mi_conv_prestage": (_I, [_P, _I, shape5, gnp_t, _P, _I]),
    "mi_conv_prestage2": (_I, [_P, shape5, gnp_t, _P, _P]),
    "mi_conv_x2_dt": (None, [_I]),
    "gnp_mk": (gnp_t, [_P, _P, _P, _P, _I]),
    "lp_gn_slab_any": (_I, []),
    "lp_gn_slab_reg": (None, [_P, _I, _I, _I, _I]),
    "lp_skip_get": (skipm_t, [shape5, split_t, _I]),
    "nn_skip_fwd_level": (_I, [shape5, split_t]),
    "nn_skip_masks": (_I, [shape5, split_t]),
    "zw_win": (_I, [_I, _P, _P]),
    "lp_mx8_bytes": (_Z, [_I, _I, _Z]),
    "lp_mx4_bytes": (_Z, [_I, _I, _Z]),
    "lp_f32_to_mx8": (None, [_P, _I, _I, _Z, _P]),
    "lp_f32_to_mx4": (None, [_P, _I, _I, _Z, _P]),
    "lp_h16_to_mx8": (None, [_P, _I, _I, _I, _Z, _P]),
    "lp_h16_to_mx4": (None, [_P, _I, _I, _I, _Z, _P]),
    "lp_mx8_to_f32": (None, [_P, _I, _I, _Z, _P]),
    "lp_mx4_to_f32": (None, [_P, _I, _I, _Z, _P]),
    "lp_pred_input_mx": (None, [_P, _I, _F, _F, _P, _P, _I, _I, _I, _P, _I, _I]),
    "lp_pred_input_mx8": (None, [_P, _I, _F, _F, _P, _P, _I, _I, _I, _P, _I]),
    "mi_pred_input_mx_n": (None, [_P, _I, _F, _F, _P, _P, _I, _I, _I, _P, _I, _I, _I, _I]),
    "mi_pred_input_mx_batch": (None, [_P, _I, _F, _F, _P, _P, _I, _I, _I, _P, _I, _I, _I, _I, _I]),
    "lp_gn_silu_apply_mx": (None, [_P, _I, shape5, _I, _P, _P, _P, _P, _P, _I]),
    "lp_add_mx": (None, [_P, _P, shape5, _I, C.c_uint]),
    "lp_up2_fwd_mx": (None, [_P, _I, shape5, _P, _I, gnp_t]),
    "lp_up2_fwd_mx_blocks": (None, [_P, _I, shape5, _I, _I, _P, _I]),
    "lp_gn_sums_mx": (_I, [_P, _I, _I, _I, _I, _Z, _P, _Z, _Z]),
    "lp_gn_sums_mx_n": (_I, [_P, _I, _I, _I, _I, _Z, _P, _Z, _Z, _I, _I]),
    "lp_conv1_fwd_mx": (None, [_P, _I, shape5, _P, _P, _I, _P, gnp_t]),
    "lp_conv1_fwd_mx_h16": (None, [_P, _I, shape5, _P, _P, _I, _P, gnp_t]),
    "lp_conv1_fwd_mx_h16_r": (None, [_P, _I, shape5, _P, _P, _I, _P, gnp_t, _Z, _Z]),
    "lp_conv1_fwd_mx_r": (_I, [_P, _I, shape5, _P, _P, _I, _P, gnp_t, _Z, _Z, _Z]),
    "lp_check": (C.c_char_p, []),
    "mi_init": (_I, [_I]),
    "mi_device_count": (_I, []),
    "mi_malloc": (_P, [_Z]),
    "mi_free": (None, [_P]),
    "mi_zero": (None, [_P, _Z]),
    "mi_h2d": (None, [_P, _P, _Z]),
    "mi_host_alloc": (_P, [_Z]),
    "mi_host_free": (None, [_P]),
    "mi_h2d_async": (None, [_P, _P, _Z]),
    "mi_fence_new": (_P, []),
    "mi_fence_set": (None, [_P]),
    "mi_fence_wait": (None, [_P]),
    "mi_fence_free": (None, [_P]),
    "mi_d2h": (None, [_P, _P, _Z]),
    "mi_d2d": (None, [_P, _P, _Z]),
    "mi_d2d_rows": (None, [_P, _Z, _P, _Z, _Z, _Z]),
    "mi_sync": (None, []),
    "mi_ws_release": (None, []),
    "mi_gn_finalize": (None, [_P, _I, _Z, _F, _P, _P]),
    "mi_gn_sums_zero": (None, [_P, _I]),
    "mi_gn_sums_get": (None, [_P, _I, _P]),
    "mi_event_create": (_P, []),
    "mi_event_record": (None, [_P]),
    "mi_event_elapsed_ms": (_F, [_P, _P]),
    "mi_event_destroy": (None, [_P]),
    "mi_conv_fwd_fused": (_I, [_I, _P, _I, shape5, _P, _P, _I, _P, _I, _P, _P, _I, gnp_t, _P, _I, split_t]),
    "lp_set_w4_2d": (None, [_I]),
    "lp_fakeq_w4": (None, [_P, _I, _I, _I, _I, _I]),
    "nn_fakeq_w4_2d": (None, [_P, _I, _I, _I, _I]),
    "nn_gn_const_fill": (None, [_P, _P, _P, _I, _I, _F]),
    "nn_ws_fwd": (None, [_P, _P, _I, _I, _F, _F]),
    "nn_axpy": (None, [_P, _F, _P, _Z]),
    "nn_film_fwd": (None, [_P, _P, _Z, _Z, _Z, _I, _I, _P]),
    "nn_gfilm_pool": (None, [_P, _I, C.c_long, _P]),
    "nn_gfilm_fwd": (None, [_P, _P, _Z, _Z, _Z, _I, _I, _P, _P]),
    "mi_conv_down2_fwd": (_I, [_I, _P, _I, shape5, _P, _P, _I, _P, _I, gnp_t]),
    "mi_convt_up2_fwd": (_I, [_I, _P, _I, shape5, _P, _P, _I, _P, _I, gnp_t]),
    "mi_conv_fwd_gn": (_I, [_I, _P, _I, shape5, _P, _P, _I, _P, _I, gnp_t, _P, _I, split_t, C.c_float, _P, _P]),
    "mi_conv_fwd_static": (_I, [_I, _P, _I, shape5, _P, _P, _I, _P, _I, gnp_t, _P, _I, split_t]),
    "mi_conv_static_scratch_bytes": (_Z, []),
    "mi_alloc_count": (C.c_long, []),
    "mi_cvt_sweep": (_I, [_I, _I, C.POINTER(C.c_ulonglong)]),
    "mi_kernel_timing": (None, [_I]),
    "mi_kernel_timing_read": (C.c_double, [C.POINTER(C.c_long)]),
    "mi_kernel_timing_launch": (C.c_long, [C.c_long, C.POINTER(C.c_float), C.POINTER(C.c_double), C.c_char_p, _Z]),
    "mi_last_kernel": (C.c_char_p, []),
}
EXPORTS = tuple(_PROTOS)


class at_geom(C.Structure):  # src/attn.h:81
    _fields_ = [("nseq", C.c_int), ("S", C.c_int), ("D", C.c_int), ("Hh", C.c_int), ("W", C.c_int),
                ("lens", C.c_void_p), ("pos", C.c_void_p), ("rays", C.c_void_p), ("dfx", C.c_void_p * 3), ("dfr", C.c_void_p)]


class at_rays(C.Structure):  # src/attn.h:93-100
    _fields_ = [(n, C.c_int) for n in ("n", "Q", "Nt", "Nr", "D", "Hh", "W")] + [(n, C.c_void_p) for n in ("ad", "ray", "lens", "pos", "wsum")]


class at_dims(C.Structure):  # src/attn.h:33
    _fields_ = [("C", C.c_int), ("H", C.c_int), ("F", C.c_int), ("rope", C.c_int), ("nreg", C.c_int), ("rope_base", C.c_float),
                ("dK", C.c_int), ("dL", C.c_int), ("dC", C.c_int * 3), ("dCo", C.c_int), ("dInit", C.c_int)]


class at_bp(C.Structure):  # src/attn.h:39
    _fields_ = [(n, C.c_size_t) for n in ("ln1g", "ln1b", "wqkv", "bqkv", "qg", "kg", "wo", "bo", "ln2g", "ln2b", "w1", "b1", "w2", "b2", "woa", "boa")] + \
               [("wvl", C.c_size_t * 3), ("bvl", C.c_size_t * 3)]


class at_ws(C.Structure):  # src/attn.h:47-60
    _fields_ = [(n, C.c_void_p) for n in ("xn", "qkv", "qkn", "o", "x1", "xn2", "h", "gg", "m1", "r1", "m2", "r2", "rq", "rk", "lse", "dv",
                                          "bA", "bB", "bC", "dx1", "qkvh", "doh", "amx", "qkvr", "orr", "dor", "dqr", "dqr2")] + \
               [("vl", C.c_void_p * 4), ("oa", C.c_void_p), ("aw", C.c_void_p), ("dvl", C.c_void_p * 4), ("doa", C.c_void_p), ("kept", C.c_int), ("vr", C.c_int),
                ("v1", C.c_void_p), ("own", C.c_void_p), ("dv1", C.c_void_p), ("lam", C.c_void_p), ("glam", C.c_void_p)]


# include/mi_attn.h
_ATTN_PROTOS = {
    "at_block_nparams": (_Z, [C.POINTER(at_dims)]),
    "at_block_layout": (_Z, [C.POINTER(at_dims), C.POINTER(at_bp), _Z]),
    "at_ws_bytes": (_Z, [C.POINTER(at_dims), C.c_long]),
    "at_ws_carve": (None, [C.POINTER(at_ws), C.POINTER(at_dims), C.c_long, _P]),
    "at_set_mx": (None, [_I]),
    "at_get_mx": (_I, []),
    "at_gemm_ex": (_I, [_I, _I, _I, _I, _I, _P, _P, _P, _F, _P, _P]),
    "at_ln_fwd": (None, [_P, _P, _P, _P, _P, _P, C.c_long, _I]),
    "at_glu_fwd": (None, [_P, _P, C.c_long, _I]),
    "at_fa_pack": (None, [_P, _P, _P, _P, _P, _P, _P, C.POINTER(at_geom), _I, _I, _I, _F]),
    "at_cs_to_tok": (None, [_P, _P, _P, _I, _I, C.c_long, _I]),
    "at_peg_fwd": (None, [_P, _P, _P, _P, C.POINTER(at_geom), _I, _I]),
    "at_tok_to_cs": (None, [_P, _P, _I, _I, C.c_long, _I]),
    "at_block_fwd": (_I, [C.POINTER(at_dims), _P, C.POINTER(at_bp), _P, _P, C.POINTER(at_geom), C.POINTER(at_ws)]),
    "lp_mx_gemm": (_I, [_I, _I, _I, _I, _I, _I, _P, _P, _P, _F]),
    "lp_mx_gemm_bmemo": (None, [_I]),
    "lp_mx_gemm_ex": (_I, [_I, _I, _I, _I, _I, _I, _P, _P, _P, _F, _P, _P]),
    "at_fa8_fwd": (_I, [_P, _P, _P, C.POINTER(at_geom), _I, _I]),
    "at_fa8_waves": (None, [_I]),
    "at_fuse_pack": (None, [_I]),
    "at_ws_bytes_r": (_Z, [C.POINTER(at_dims), C.c_long, C.c_long]),
    "at_ws_carve_r": (None, [C.POINTER(at_ws), C.POINTER(at_dims), C.c_long, C.c_long, _P]),
    "at_rays_dims": (None, [_I, _I, _I, _F, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "at_rays_plan": (None, [_I, _I, _I, _I, _F, _P, _P, _P, _P, _P]),
    "at_rays_setup": (None, [C.POINTER(at_rays)]),
    "at_ray_gather": (None, [C.POINTER(at_rays), _P, _P, _I, _I]),
    "at_ray_scatter": (None, [C.POINTER(at_rays), _P, _P, _I, _I]),
    "at_scroll_pos": (None, [_I, _I, _I, _I, _I, _P, _P, _P]),
    "at_fa_fwd": (None, [_P, _P, _P, C.POINTER(at_geom), _I, _I]),
}
ATTN_EXPORTS = tuple(_ATTN_PROTOS)
# include/mi_predict.h
_PRED_PROTOS = {
    "nn_set_pred_iso": (None, [_I]),
    "nn_get_pred_iso": (_I, []),
    "nn_pred_place_d": (None, [_P, _P] + [_I] * 11 + [_P]),
    "nn_pred_place": (None, [_P, _P] + [_I] * 9 + [_P]),
    "mi_ct_window": (None, [_P] + [C.c_int64] * 6 + [_I, _P, _I, _I, _P]),
    "mi_ct_windows": (None, [_P] + [C.c_int64] * 3 + [C.POINTER(C.c_int64), _I, _I, _P, _I, _I, _P]),
    "mi_ct_flags": (None, [_P] + [C.c_int64] * 3 + [_I, C.POINTER(C.c_int64), _I, _P]),
    "mi_pred_place_n": (None, [_P, C.c_size_t, _P, C.c_size_t, _I, C.POINTER(C.c_int64)] + [_I] * 11 + [_P]),
    "mi_feather_blend": (_I, [_P, _P, _I, _I, C.POINTER(C.c_int64), C.POINTER(C.c_int64), _P]),
}
PRED_EXPORTS = tuple(_PRED_PROTOS)
_lib = None


def load():
    """Load libufsm_lp.so and set the prototypes. Raises if the library is not built: there is no fallback path."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("%s is not built: run `python -c 'import __graft_entry__ as g; g.build()'` (hipcc, gfx950)" % LIB_PATH)
    L = C.CDLL(LIB_PATH)
    for name, (res, args) in list(_PROTOS.items()) + list(_ATTN_PROTOS.items()) + list(_PRED_PROTOS.items()):
        f = getattr(L, name)  # AttributeError names the missing symbol
        f.restype = res
        f.argtypes = args
    _lib = L
    return L


class _Lazy:
    def __getattr__(self, k):
        return getattr(load(), k)


lib = _Lazy()


class DevBuf:
    """A device allocation owned by the caller (mi_malloc / mi_free), with numpy copies in and out."""

    def __init__(self, nbytes, zero=True):
        self.nbytes = int(nbytes)
        self.ptr = lib.mi_malloc(max(self.nbytes, 1))
        if zero and self.nbytes:
            lib.mi_zero(self.ptr, self.nbytes)

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes, zero=False)
        if a.nbytes:
            lib.mi_h2d(b.ptr, a.ctypes.data, a.nbytes)
        return b

    def to_numpy(self, dtype, shape=None):
        lib.mi_sync()
        out = np.empty(self.nbytes // np.dtype(dtype).itemsize, dtype=dtype)
        if self.nbytes:
            lib.mi_d2h(out.ctypes.data, self.ptr, out.nbytes)
        return out.reshape(shape) if shape is not None else out

    def free(self):
        if self.ptr:
            lib.mi_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class LP:
    """Thin Python mirror of the lp_* entry points (argument meaning as in src/nn_lp.h)."""

    @staticmethod
    def gn(gamma=None, beta=None, mean=None, rstd=None, G=0):
        g = gnp_t()
        if G:
            g.gamma, g.beta, g.mean, g.rstd, g.G = gamma.ptr, beta.ptr, mean.ptr, rstd.ptr, G
        return g

    @staticmethod
    def check():
        lib.mi_sync()
        e = lib.lp_check()
        if e:
            raise RuntimeError("HIP error: " + e.decode())
