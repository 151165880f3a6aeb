"""ctypes mirror of include/mi_unet.h: the C23 host layer (op dispatch and U-Net graph) in libufsm_host.so."""
import ctypes as C
import os

import numpy as np

from .lp import shape5, load as _load_lp

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "libufsm_host.so")
UNET_MAXLEV = 8


class unet_cfg(C.Structure):
    _fields_ = [("cin", C.c_int), ("nlev", C.c_int), ("widths", C.c_int * UNET_MAXLEV), ("G", C.c_int), ("head_out", C.c_int),
                ("act_dt", C.c_int), ("prec", C.c_int), ("attn_blocks", C.c_int), ("attn_pe", C.c_int), ("attn_reg", C.c_int), ("attn_mlp", C.c_int), ("down_norm", C.c_int)]


_host = None


def load_host():
    global _host
    if _host is not None:
        return _host
    _load_lp()                                      # the kernels' library first (the host layer links against it)
    if not os.path.exists(HOST_LIB_PATH):
        raise RuntimeError("%s is not built: run __graft_entry__.build()" % HOST_LIB_PATH)
    L = C.CDLL(HOST_LIB_PATH)
    L.unet_create.restype = C.c_void_p; L.unet_create.argtypes = [C.POINTER(unet_cfg), shape5]
    L.unet_free.restype = None; L.unet_free.argtypes = [C.c_void_p]
    L.unet_nparams.restype = C.c_size_t; L.unet_nparams.argtypes = [C.c_void_p]
    L.unet_init.restype = None; L.unet_init.argtypes = [C.c_void_p, C.c_uint64]
    L.unet_get_params.restype = None; L.unet_get_params.argtypes = [C.c_void_p, C.c_void_p]
    L.unet_set_params.restype = None; L.unet_set_params.argtypes = [C.c_void_p, C.c_void_p]
    L.unet_forward_x.restype = C.c_int; L.unet_forward_x.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
    L.unet_forward_ct.restype = C.c_int
    L.unet_forward_ct.argtypes = [C.c_void_p, C.c_void_p, C.c_float, C.c_float, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p]
    L.unet_layer_out.restype = C.c_void_p; L.unet_layer_out.argtypes = [C.c_void_p, C.c_int, C.POINTER(shape5), C.POINTER(C.c_char_p)]
    L.unet_layer_stats.restype = C.c_int; L.unet_layer_stats.argtypes = [C.c_void_p, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_void_p)]
    L.nn_set_storage.restype = None; L.nn_set_storage.argtypes = [C.c_void_p, C.c_size_t, C.c_int]
    L.nn_storage.restype = C.c_int; L.nn_storage.argtypes = [C.c_void_p]
    L.nn_set_prec.restype = None; L.nn_set_prec.argtypes = [C.c_int]
    L.nn_set_gn_stored.restype = None; L.nn_set_gn_stored.argtypes = [C.c_int]
    L.nn_check.restype = C.c_char_p
    L.unet_in_shape.restype = shape5; L.unet_in_shape.argtypes = [C.c_void_p]
    L.unet_set_infer_slab.restype = None; L.unet_set_infer_slab.argtypes = [C.c_int]
    L.unet_get_infer_slab.restype = C.c_int; L.unet_get_infer_slab.argtypes = []
    L.nn_set_zrange.restype = None; L.nn_set_zrange.argtypes = [C.c_int] * 6
    L.nn_set_zrange_out.restype = None; L.nn_set_zrange_out.argtypes = [C.c_int]
    L.unet_config.restype = C.POINTER(unet_cfg); L.unet_config.argtypes = [C.c_void_p]
    L.unet_read_header.restype = C.c_int; L.unet_read_header.argtypes = [C.c_char_p, C.POINTER(unet_cfg), C.POINTER(C.c_size_t), C.POINTER(C.c_int)]
    L.unet_load.restype = C.c_int; L.unet_load.argtypes = [C.c_void_p, C.c_char_p]
    L.unet_load_ema.restype = C.c_int; L.unet_load_ema.argtypes = [C.c_void_p, C.c_char_p]
    L.unet_save.restype = C.c_int; L.unet_save.argtypes = [C.c_void_p, C.c_char_p, C.c_int, C.c_char_p]
    L.unet_predict_volume.restype = C.c_int
    L.unet_predict_volume.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_int64), C.c_int, C.c_int, C.c_float, C.c_float, C.c_int, C.c_float, C.c_float,
                                      C.c_void_p, C.POINTER(C.c_int64)]
    _host = L
    return L


def make_cfg(cin, widths, G=8, head_out=8, act_dt=8, prec=0, attn_blocks=0, attn_pe=2, attn_reg=0, attn_mlp=0, down_norm=0):
    c = unet_cfg()
    c.cin, c.nlev, c.G, c.head_out, c.act_dt, c.prec = cin, len(widths), G, head_out, act_dt, prec
    c.attn_blocks, c.attn_pe, c.attn_reg, c.attn_mlp, c.down_norm = attn_blocks, attn_pe, attn_reg, attn_mlp, down_norm
    for i, w in enumerate(widths):
        c.widths[i] = w
    return c


class UNet:
    """A U-Net instance owned by the host library."""

    def __init__(self, cfg, N, D, H, W, seed=1):
        self.L = load_host()
        self.cfg = cfg
        self.shape = shape5(N, cfg.cin, D, H, W)
        self.h = self.L.unet_create(C.byref(cfg), self.shape)
        if not self.h:
            raise RuntimeError("unet_create failed")
        self.L.unet_init(self.h, seed)

    def params(self):
        p = np.zeros(self.L.unet_nparams(self.h), dtype=np.float32)
        self.L.unet_get_params(self.h, p.ctypes.data)
        return p

    def set_params(self, p):
        p = np.ascontiguousarray(p, dtype=np.float32)
        assert p.size == self.L.unet_nparams(self.h)
        self.L.unet_set_params(self.h, p.ctypes.data)

    def forward_x(self, x_ptr, logits_ptr):
        return self.L.unet_forward_x(self.h, x_ptr, logits_ptr)

    def forward_ct(self, ct_ptr, mean, isd, dyo_ptr, dxo_ptr, axis, logits_ptr):
        return self.L.unet_forward_ct(self.h, ct_ptr, mean, isd, dyo_ptr, dxo_ptr, axis, logits_ptr)

    def predict_volume(self, vol_ptr, dims, halo, feather, mean, isd, axis, cy, cx, out_ptr):
        """Sliding-window prediction of a device uint8 volume; returns (rc, windows, windows computed)."""
        d = (C.c_int64 * 3)(*dims); nw = (C.c_int64 * 2)(0, 0)
        rc = self.L.unet_predict_volume(self.h, vol_ptr, d, halo, feather, mean, isd, axis, cy, cx, out_ptr, nw)
        return rc, nw[0], nw[1]

    def save(self, path, step=0, extra=None):
        return self.L.unet_save(self.h, path.encode(), step, extra.encode() if extra else None)

    def load(self, path, ema=False):
        return (self.L.unet_load_ema if ema else self.L.unet_load)(self.h, path.encode())

    def layer_outs(self):
        out, k = [], 0
        while True:
            s = shape5(); name = C.c_char_p()
            p = self.L.unet_layer_out(self.h, k, C.byref(s), C.byref(name))
            if not p:
                return out
            out.append((name.value.decode(), p, (s.n, s.c, s.d, s.h, s.w)))
            k += 1

    def layer_stats(self, k):
        """(G, mean ptr, rstd ptr) of the k-th conv output (G 0: no statistics)."""
        m, r = C.c_void_p(), C.c_void_p()
        G = self.L.unet_layer_stats(self.h, k, C.byref(m), C.byref(r))
        return G, m.value, r.value

    def close(self):
        if self.h:
            self.L.unet_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
