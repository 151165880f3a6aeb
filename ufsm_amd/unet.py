"""ctypes mirror of include/mi_unet.h: the C23 host layer (op dispatch and U-Net graph) in libufsm_host.so."""
import ctypes as C
import os

import numpy as np

from .lp import shape5, load as _load_lp

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "libufsm_host.so")
UNET_MAXLEV = 8
_I = C.c_int


class unet_cfg(C.Structure):  # src/unet.h:18-128, field for field
    _fields_ = [("nlev", _I), ("widths", _I * UNET_MAXLEV), ("cin", _I), ("cout", _I), ("G", _I), ("down_norm", _I), ("scale_cond", _I),
                ("dec_widths", _I * UNET_MAXLEV), ("enc_blocks", _I * UNET_MAXLEV), ("dec_convs", _I * UNET_MAXLEV), ("ds_levels", _I), ("lat_guide", _I),
                ("lat_nsub", _I), ("lat_sub", C.c_int8 * 16), ("half_res", _I), ("w4_2d", _I), ("l0_norm", _I), ("l0_slab", _I), ("gfilm", _I), ("scan_norm", _I),
                ("gn_ema", _I), ("attn_blocks", _I), ("attn_pe", _I), ("attn_reg", _I), ("attn_mlp", _I), ("attn_vres", _I), ("attn_axis", _I), ("attn_repeat", _I),
                ("attn_mem", _I), ("view_P", _I), ("view_patch", _I), ("attn_deform", _I), ("attn_dlev", _I), ("attn_dco", _I), ("attn_dinit", _I), ("emb_lev", _I),
                ("emb_ch", _I), ("film", _I), ("skip_thr", _I), ("skip_margin", _I), ("skip_nl", _I), ("fstem", _I), ("fstem_out", _I),
                ("lat_dec", _I), ("lat_dec_raw", _I), ("lat_dec_ng", _I), ("lat_dec_wq", _I)]


_host = None


def load_host():
    global _host
    if _host is not None:
        return _host
    _load_lp()                                      # the kernels' library first (the host layer links against it)
    if not os.path.exists(HOST_LIB_PATH):
        raise RuntimeError("%s is not built: run __graft_entry__.build()" % HOST_LIB_PATH)
    L = C.CDLL(HOST_LIB_PATH)
    P = C.c_void_p
    L.unet_create.restype = P; L.unet_create.argtypes = [C.POINTER(unet_cfg)]
    L.unet_free.restype = None; L.unet_free.argtypes = [P]
    L.unet_cfg_of.restype = C.POINTER(unet_cfg); L.unet_cfg_of.argtypes = [P]
    L.unet_nparams.restype = C.c_size_t; L.unet_nparams.argtypes = [P]
    L.unet_init.restype = None; L.unet_init.argtypes = [P, C.c_uint64]
    L.unet_param_ptr.restype = P; L.unet_param_ptr.argtypes = [P]
    L.unet_ema_ptr.restype = P; L.unet_ema_ptr.argtypes = [P]
    L.unet_use_ema.restype = None; L.unet_use_ema.argtypes = [P, _I]
    L.mi_unet_weights_changed.restype = None; L.mi_unet_weights_changed.argtypes = [P]
    L.unet_set_act_mx8.restype = None; L.unet_set_act_mx8.argtypes = [_I]
    L.unet_set_act_mx4.restype = None; L.unet_set_act_mx4.argtypes = [_I]
    L.unet_act_mx.restype = _I; L.unet_act_mx.argtypes = []
    L.unet_forward.restype = P; L.unet_forward.argtypes = [P, P, shape5, _I]
    L.unet_forward_x.restype = P; L.unet_forward_x.argtypes = [P, P, shape5, _I, _I]
    L.unet_out_shape.restype = shape5; L.unet_out_shape.argtypes = [P, shape5]
    L.unet_forward_ct.restype = P; L.unet_forward_ct.argtypes = [P, P, C.c_float, C.c_float, P, P, _I, shape5, _I]
    L.mi_unet_forward_ct_n.restype = P; L.mi_unet_forward_ct_n.argtypes = [P, P, C.c_float, C.c_float, P, P, _I, shape5, _I]
    L.mi_unet_forward_mx.restype = P; L.mi_unet_forward_mx.argtypes = [P, P, shape5]
    L.mi_unet_get_params.restype = None; L.mi_unet_get_params.argtypes = [P, P]
    L.mi_unet_set_params.restype = None; L.mi_unet_set_params.argtypes = [P, P]
    L.mi_unet_layer_out.restype = P; L.mi_unet_layer_out.argtypes = [P, _I, C.POINTER(shape5), C.POINTER(C.c_char_p)]
    L.mi_unet_layer_stats.restype = _I; L.mi_unet_layer_stats.argtypes = [P, _I, C.POINTER(P), C.POINTER(P)]
    F = C.c_float
    L.nn_conv3d_out_shape.restype = shape5; L.nn_conv3d_out_shape.argtypes = [shape5, _I, _I, _I]
    L.nn_conv3d_fwd.restype = None; L.nn_conv3d_fwd.argtypes = [P, shape5, P, P, _I, _I, _I, P]
    L.nn_conv3d_fwd_gn.restype = _I; L.nn_conv3d_fwd_gn.argtypes = [P, shape5, _I, P, P, P, P, P, P, _I, P]
    L.nn_conv3d_fwd_gn_stats.restype = _I; L.nn_conv3d_fwd_gn_stats.argtypes = [P, shape5, _I, P, P, P, P, P, P, _I, P, _I, F, P, P]
    L.nn_conv3d_fwd_split.restype = _I; L.nn_conv3d_fwd_split.argtypes = [P, P, _I, shape5, _I, P, P, P, P, P, P, _I, P, _I, F, P, P]
    L.nn_set_storage.restype = None; L.nn_set_storage.argtypes = [P, C.c_size_t, _I]
    L.nn_storage.restype = _I; L.nn_storage.argtypes = [P]
    L.nn_storage_forget.restype = None; L.nn_storage_forget.argtypes = [P]
    L.nn_set_prec.restype = None; L.nn_set_prec.argtypes = [_I]
    L.nn_get_prec.restype = _I; L.nn_get_prec.argtypes = []
    L.nn_set_gn_stored.restype = None; L.nn_set_gn_stored.argtypes = [_I]
    L.nn_check.restype = C.c_char_p
    L.unet_set_infer_slab.restype = None; L.unet_set_infer_slab.argtypes = [_I]
    L.unet_set_slab_direct.restype = None; L.unet_set_slab_direct.argtypes = [_I]
    L.unet_l0_updates.restype = C.c_long; L.unet_l0_updates.argtypes = [C.c_void_p]
    L.unet_gn_ema_updates.restype = C.c_long; L.unet_gn_ema_updates.argtypes = [C.c_void_p]
    L.unet_gn_ema_live.restype = None; L.unet_gn_ema_live.argtypes = [C.c_void_p, _I]
    L.unet_set_scale.restype = None; L.unet_set_scale.argtypes = [C.c_void_p, C.c_double]
    L.unet_set_cond.restype = None; L.unet_set_cond.argtypes = [C.c_void_p, C.c_float]
    L.unet_set_attn_axis.restype = None; L.unet_set_attn_axis.argtypes = [C.c_void_p, C.c_void_p, _I, _I]
    L.unet_attn_rays.restype = _I; L.unet_attn_rays.argtypes = [C.c_void_p, C.POINTER(_I), C.POINTER(_I), C.POINTER(C.c_double)]
    L.unet_set_film.restype = None; L.unet_set_film.argtypes = [C.c_void_p, C.POINTER(C.c_float), _I]
    L.unet_gfilm_off.restype = C.c_size_t; L.unet_gfilm_off.argtypes = [C.c_void_p]
    L.mi_unet_film_off.restype = C.c_size_t; L.mi_unet_film_off.argtypes = [C.c_void_p]
    L.mi_unet_gfilm_codes.restype = C.c_void_p; L.mi_unet_gfilm_codes.argtypes = [C.c_void_p]
    L.mi_unet_infer_slab.restype = _I; L.mi_unet_infer_slab.argtypes = []
    L.nn_set_zrange.restype = None; L.nn_set_zrange.argtypes = [_I] * 6
    L.nn_set_zrange_out.restype = None; L.nn_set_zrange_out.argtypes = [_I]
    L.unet_peek.restype = _I; L.unet_peek.argtypes = [C.c_char_p, C.POINTER(unet_cfg), C.POINTER(_I)]
    L.mi_unet_peek_nparams.restype = C.c_size_t; L.mi_unet_peek_nparams.argtypes = [C.c_char_p]
    L.unet_load.restype = _I; L.unet_load.argtypes = [P, C.c_char_p]
    L.unet_save.restype = _I; L.unet_save.argtypes = [P, C.c_char_p, _I, C.c_char_p]
    L.mi_unet_predict_volume.restype = _I
    L.mi_unet_predict_volume.argtypes = [P, _I, _I, P, C.POINTER(C.c_int64), _I, _I, C.c_float, C.c_float, _I, C.c_float, C.c_float, P, C.POINTER(C.c_int64)]
    _host = L
    return L


def make_cfg(cin, widths, G=8, head_out=8, act_dt=8, prec=0, attn_blocks=0, attn_pe=2, attn_reg=0, attn_mlp=0, attn_repeat=0, down_norm=0, w4_2d=0, l0_norm=0, l0_slab=0, gn_ema=0, dec_widths=None, dec_convs=None, enc_blocks=None, ds_levels=0, emb_lev=0, emb_ch=0, scale_cond=0, film=0, gfilm=0, attn_vres=0, attn_axis=0):
    """The reference's configuration record plus, as Python attributes, what the reference keeps in process-wide switches: the activation
    storage (unet_set_act_mx4) and the compute precision policy (nn_set_prec), which UNet applies around its calls."""
    c = unet_cfg()
    c.cin, c.nlev, c.G, c.cout = cin, len(widths), G, head_out
    c.attn_blocks, c.attn_pe, c.attn_reg, c.attn_mlp, c.down_norm, c.w4_2d = attn_blocks, attn_pe if attn_blocks else 0, attn_reg, attn_mlp, down_norm, w4_2d
    for i, w in enumerate(widths):
        c.widths[i] = w
    c.l0_norm, c.l0_slab, c.gn_ema = l0_norm, l0_slab, gn_ema
    c.attn_repeat = attn_repeat if attn_blocks else 0
    c.ds_levels, c.emb_lev, c.emb_ch, c.scale_cond = ds_levels, emb_lev, emb_ch, scale_cond
    c.film, c.gfilm, c.attn_vres = film, gfilm, attn_vres
    c.attn_axis = attn_axis if attn_blocks else 0
    for i, d in enumerate(dec_widths or []):
        c.dec_widths[i] = d
    for i, d in enumerate(dec_convs or []):
        c.dec_convs[i] = d
    for i, d in enumerate(enc_blocks or []):
        c.enc_blocks[i] = d
    c.act_dt, c.prec = act_dt, prec
    return c


class UNet:
    """A U-Net instance owned by the host library, used at one input shape (N, cin, D, H, W)."""

    def __init__(self, cfg, N, D, H, W, seed=1):
        self.L = load_host()
        self.cfg = cfg
        self.act_dt, self.prec = getattr(cfg, "act_dt", 8), getattr(cfg, "prec", 0)
        self.shape = shape5(N, cfg.cin, D, H, W)
        self.h = self.L.unet_create(C.byref(cfg))
        if not self.h:
            raise RuntimeError("unet_create failed")
        self.L.unet_init(self.h, seed)

    def _mode(self):
        self.L.unet_set_act_mx4(1 if self.act_dt == 4 else 0)
        self.L.nn_set_prec(self.prec)

    def _unmode(self):
        self.L.unet_set_act_mx4(0)
        self.L.nn_set_prec(0)

    def params(self):
        p = np.zeros(self.L.unet_nparams(self.h), dtype=np.float32)
        self.L.mi_unet_get_params(self.h, p.ctypes.data)
        return p

    def set_params(self, p):
        p = np.ascontiguousarray(p, dtype=np.float32)
        assert p.size == self.L.unet_nparams(self.h)
        self.L.mi_unet_set_params(self.h, p.ctypes.data)

    def logits_bytes(self):
        s = self.shape
        return s.n * self.cfg.cout * s.d * s.h * s.w * 4

    def forward_mx(self, x_ptr):
        """The forward on an MX input tensor; returns the device pointer of the net's own logits (0 on failure)."""
        self._mode()
        try:
            return self.L.mi_unet_forward_mx(self.h, x_ptr, self.shape) or 0
        finally:
            self._unmode()

    def forward_x(self, x_ptr, logits_ptr):
        """forward_mx, the logits copied into the caller's device buffer; 0 on success."""
        from .lp import lib
        p = self.forward_mx(x_ptr)
        if not p:
            return -1
        lib.mi_d2d(logits_ptr, p, self.logits_bytes())
        return 0

    def forward_planes(self, x_ptr, h16=False):
        """unet_forward_x: fp32 (or fp16) planes in, the net's logits pointer out."""
        self._mode()
        try:
            return self.L.unet_forward_x(self.h, x_ptr, self.shape, 0, 1 if h16 else 0) or 0
        finally:
            self._unmode()

    def forward_ct(self, ct_ptr, mean, isd, dyo_ptr, dxo_ptr, axis, logits_ptr, h16=2):
        from .lp import lib
        self._mode()
        try:
            p = self.L.unet_forward_ct(self.h, ct_ptr, mean, isd, dyo_ptr, dxo_ptr, axis, self.shape, h16)
        finally:
            self._unmode()
        if not p:
            return -1
        lib.mi_d2d(logits_ptr, p, self.logits_bytes())
        return 0

    def predict_volume(self, vol_ptr, dims, halo, feather, mean, isd, axis, cy, cx, out_ptr):
        """Sliding-window prediction of a device uint8 volume; returns (rc, windows, windows computed)."""
        d = (C.c_int64 * 3)(*dims); nw = (C.c_int64 * 2)(0, 0)
        self._mode()
        try:
            rc = self.L.mi_unet_predict_volume(self.h, self.shape.w, self.shape.n, vol_ptr, d, halo, feather, mean, isd, axis, cy, cx, out_ptr, nw)
        finally:
            self._unmode()
        return rc, nw[0], nw[1]

    def save(self, path, step=0, extra=None):
        return self.L.unet_save(self.h, path.encode(), step, extra.encode() if extra else None)

    def load(self, path):
        """The saved step, or -1."""
        return self.L.unet_load(self.h, path.encode())

    def use_ema(self, on):
        self.L.unet_use_ema(self.h, 1 if on else 0)

    def layer_outs(self):
        out, k = [], 0
        while True:
            s = shape5(); name = C.c_char_p()
            p = self.L.mi_unet_layer_out(self.h, k, C.byref(s), C.byref(name))
            if not p:
                return out
            out.append((name.value.decode(), p, (s.n, s.c, s.d, s.h, s.w)))
            k += 1

    def layer_stats(self, k):
        """(G, mean ptr, rstd ptr) of the k-th conv output (G 0: no statistics)."""
        m, r = C.c_void_p(), C.c_void_p()
        G = self.L.mi_unet_layer_stats(self.h, k, C.byref(m), C.byref(r))
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
