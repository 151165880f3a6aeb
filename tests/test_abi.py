"""The C-ABI library loads and exports every symbol include/mi_lp.h declares; descriptor layouts match the reference's (no compute, no GPU)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions(header="mi_lp.h", prefixes=("lp_", "mi_", "gnp_", "nn_", "zw_")):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b([a-z][a-z0-9_]*)\s*\([^;{]*\)\s*;", text)
    return sorted(set(n for n in names if n.startswith(prefixes)))


def test_header_declares_the_forward_subset():
    names = header_functions()
    for must in ["lp_conv_fwd_f8", "lp_conv_fwd_f4", "lp_conv_fwd_s2_f8", "lp_f32_to_mx8", "lp_f32_to_mx4", "lp_h16_to_mx8", "lp_mx8_to_f32", "lp_mx4_to_f32",
                 "lp_mx8_bytes", "lp_mx4_bytes", "lp_pred_input_mx", "lp_pred_input_mx8", "lp_gn_silu_apply_mx", "lp_add_mx", "lp_up2_fwd_mx", "lp_up2_fwd_mx_blocks",
                 "lp_conv1_fwd_mx", "lp_conv1_fwd_mx_h16", "lp_conv1_fwd_mx_h16_r", "lp_conv1_fwd_mx_r", "lp_gn_sums_mx", "lp_gn_sums_mx_n", "lp_check", "gnp_mk",
                 "lp_gn_slab_any", "lp_gn_slab_reg", "lp_wmemo_step", "lp_wmemo_clear", "lp_skip_get", "nn_skip_masks", "zw_win"]:
        assert must in names, must


def test_library_exports_every_declared_symbol():
    from ufsm_amd import lp
    L = lp.load()
    for n in header_functions():
        assert hasattr(L, n), "libufsm_lp.so does not export %s" % n
    assert set(header_functions()) == set(lp.EXPORTS)


def test_library_exports_the_attention_header():
    from ufsm_amd import lp
    L = lp.load()
    names = header_functions("mi_attn.h", ("lp_", "at_"))
    assert set(names) == set(lp.ATTN_EXPORTS) and {"lp_mx_gemm", "lp_mx_gemm_ex", "at_fa8_fwd", "at_block_fwd", "at_fa_pack", "at_ln_fwd"} <= set(names)
    for n in names:
        assert hasattr(L, n), "libufsm_lp.so does not export %s" % n
    # at_geom as the reference lays it out on LP64 (src/attn.h:81): five ints, padding, seven pointers
    assert C.sizeof(lp.at_geom) == 24 + 7 * 8 and lp.at_geom.lens.offset == 24 and lp.at_geom.dfr.offset == 72


def test_library_exports_the_prediction_header():
    from ufsm_amd import lp
    L = lp.load()
    names = header_functions("mi_predict.h", ("nn_", "mi_"))
    assert set(names) == set(lp.PRED_EXPORTS) and "nn_pred_place" in names and "mi_feather_blend" in names
    for n in names:
        assert hasattr(L, n), "libufsm_lp.so does not export %s" % n


def test_host_library_exports_every_declared_symbol():
    from ufsm_amd import unet
    H = unet.load_host()
    names = header_functions("mi_unet.h", ("nn_", "unet_", "mi_unet_"))
    assert "unet_forward_x" in names and "nn_conv3d_fwd_x" in names and "nn_set_storage" in names and "mi_unet_predict_volume" in names
    assert {"nn_conv3d_fwd", "nn_conv3d_fwd_gn", "nn_conv3d_fwd_gn_stats", "nn_conv3d_fwd_split", "nn_conv3d_out_shape"} <= set(names)      # src/nn.h:399-400, :416, :423, :442
    for n in names:
        assert hasattr(H, n), "libufsm_host.so does not export %s" % n
    # unet_cfg as the reference lays it out (src/unet.h:18-128): 4-byte fields in its order, three arrays of UNET_MAXLEV ints, one of 16 bytes
    c = unet.unet_cfg
    offs = {"nlev": 0, "widths": 4, "cin": 36, "cout": 40, "G": 44, "down_norm": 48, "scale_cond": 52, "dec_widths": 56, "enc_blocks": 88, "dec_convs": 120,
            "ds_levels": 152, "lat_guide": 156, "lat_nsub": 160, "lat_sub": 164, "half_res": 180, "w4_2d": 184, "l0_norm": 188, "gfilm": 196, "gn_ema": 204,
            "attn_blocks": 208, "attn_pe": 212, "attn_reg": 216, "attn_mlp": 220, "attn_vres": 224, "attn_mem": 236, "view_P": 240, "attn_deform": 248,
            "emb_lev": 264, "film": 272, "skip_thr": 276, "fstem": 288, "lat_dec": 296, "lat_dec_wq": 308}
    for k, o in offs.items():
        assert getattr(c, k).offset == o, k
    assert C.sizeof(c) == 312


def test_unet_header_matches_the_cited_reference_signatures():
    """The graph entry points carry the reference's parameter lists (src/unet.h:141, :176, :185-187, :258, :344-347, :357, :369-370, :428)."""
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "mi_unet.h")).read(), flags=re.S)
    flat = re.sub(r"\s+", " ", text)
    for decl in ["unet *unet_create(const unet_cfg *cfg);", "const float *unet_forward(unet *u, const float *x, shape5 xs, int train);",
                 "const float *unet_forward_x(unet *u, const void *x, shape5 xs, int train, int x_h16);", "shape5 unet_out_shape(const unet *u, shape5 xs);",
                 "const float *unet_forward_ct(unet *u, const uint8_t *ct, float mean, float isd, const float *dyo, const float *dxo, int axis, shape5 xs, int h16);",
                 "void unet_use_ema(unet *u, int on);", "int unet_save(const unet *u, const char *path, int step, const char *extra_json);", "int unet_load(unet *u, const char *path);",
                 "int unet_peek(const char *path, unet_cfg *cfg, int *step);", "void unet_set_act_mx8(int on);", "void unet_set_act_mx4(int on);", "void unet_set_infer_slab(int planes);", "void unet_set_slab_direct(int on);", "void unet_set_scale(unet *u, double um);", "void unet_set_cond(unet *u, float c);", "void unet_set_film(unet *u, const float *codes, int k);", "size_t unet_gfilm_off(const unet *u);",
                 "const unet_cfg *unet_cfg_of(const unet *u);", "float *unet_param_ptr(unet *u);", "void unet_init(unet *u, uint64_t seed);"]:
        assert decl in flat, decl


def test_op_layer_header_matches_the_cited_reference_signatures():
    """The op layer's conv entries carry the reference's parameter lists (src/nn.h:399-400, :416, :423-424, :432-433, :442-443)."""
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "mi_unet.h")).read(), flags=re.S)
    flat = re.sub(r"\s+", " ", text)
    for decl in ["shape5 nn_conv3d_out_shape(shape5 xs, int cout, int k, int stride);",
                 "void nn_conv3d_fwd(const float *x, shape5 xs, const float *w, const float *b, int cout, int k, int stride, float *y);",
                 "int nn_conv3d_fwd_gn(const float *x, shape5 xs, int G, const float *gamma, const float *beta, const float *mean, const float *rstd, const float *w, const float *b, int cout, float *y);",
                 "int nn_conv3d_fwd_gn_stats(const float *x, shape5 xs, int G_in, const float *gamma, const float *beta, const float *mean, const float *rstd, const float *w, const float *b, int cout, float *y, int G_out, float eps, float *omean, float *orstd);",
                 "int nn_conv3d_fwd_split(const float *x, const float *x2, int c_split, shape5 xs, int G_in, const float *gamma, const float *beta, const float *mean, const float *rstd, const float *w, const float *b, int cout, float *y, int G_out, float eps, float *omean, float *orstd);",
                 "int nn_conv3d_fwd_x(const float *x, const nn_gn_t *gx, const float *x2, const nn_gn_t *gx2, int c_split, int up, shape5 xs, const float *w, const float *b, int cout, int k, int stride, float *y, int G_out, float eps, float *omean, float *orstd);"]:
        assert decl in flat, decl


def test_descriptor_layouts():
    from ufsm_amd import shape5, gnp_t, split_t
    assert C.sizeof(shape5) == 20
    assert C.sizeof(gnp_t) == 56 and gnp_t.G.offset == 32 and gnp_t.zhw.offset == 48
    assert C.sizeof(split_t) <= 128                                  # src/nn_lp.h:41
    from ufsm_amd.lp import skipm_t
    assert C.sizeof(skipm_t) == 32 and skipm_t.my.offset == 16       # src/nn_lp.h:44
    assert split_t.gp2.offset == 32 and split_t.up.offset == 88 and split_t.wkey.offset == 96 and split_t.stored_stats.offset == 108


def test_size_helpers_and_no_device_behaviour():
    from ufsm_amd import lib
    assert lib.lp_mx8_bytes(2, 128, 1000) == 2 * 4 * 1000 * 33       # src/lp_mx_cvt.cu:6
    assert lib.lp_mx4_bytes(2, 128, 1000) == 2 * 4 * 1000 * 17
    assert lib.lp_mx8_bytes(1, 4, 10) == 10 * 9 and lib.lp_mx8_bytes(1, 12, 10) == 10 * 17 and lib.lp_mx4_bytes(1, 12, 10) == 10 * 9
    assert lib.lp_gn_slab_any() == 0
    # the slab statistics registry is host state: gnp_mk copies a registered mean array's geometry, and only that array's (src/nn_fwd.cu:12-35)
    lib.lp_gn_slab_reg(0x1000, 64, 3, 2, 4096)
    try:
        g = lib.gnp_mk(0x10, 0x20, 0x1000, 0x2000, 8)
        assert lib.lp_gn_slab_any() == 1 and (g.G, g.zs, g.zo, g.ns, g.zhw) == (8, 64, 3, 2, 4096)
        g = lib.gnp_mk(0x10, 0x20, 0x3000, 0x2000, 8)
        assert (g.G, g.zs, g.zo, g.ns, g.zhw) == (8, 0, 0, 0, 0)
        lib.lp_gn_slab_reg(0x1000, 32, 0, 4, 100)          # a second registration of the same array replaces the first
        g = lib.gnp_mk(0x10, 0x20, 0x1000, 0x2000, 8)
        assert (g.zs, g.zo, g.ns, g.zhw) == (32, 0, 4, 100)
        lib.lp_gn_slab_reg(0x1000, 0, 0, 0, 0)              # ns <= 0 removes it
        assert lib.lp_gn_slab_any() == 0 and lib.gnp_mk(0x10, 0x20, 0x1000, 0x2000, 8).ns == 0
    finally:
        lib.lp_gn_slab_reg(None, 0, 0, 0, 0)
    # standing alone the library answers the op-layer questions itself: every conv dense, no z-window (src/nn_lp.h:44-49, src/lp_common.cuh:42)
    from ufsm_amd import shape5, split_t
    sk = lib.lp_skip_get(shape5(1, 32, 8, 8, 16), split_t(), 1)
    assert not sk.m and not sk.mi and lib.nn_skip_masks(shape5(1, 32, 8, 8, 16), split_t()) == 0 and lib.nn_skip_fwd_level(shape5(1, 32, 8, 8, 16), split_t()) == 0
    z = (C.c_int * 2)(7, 9)
    assert lib.zw_win(16, C.byref(z, 0), C.byref(z, 4)) == 0
    if lib.mi_device_count() == 0:
        assert lib.mi_init(0) != 0                                   # fails loudly instead of falling back


def test_oracle_is_not_reachable_from_the_product():
    """Nothing under ufsm_amd/ (the shipped path) may import, link or call the oracle."""
    for dirpath, _, files in os.walk(os.path.join(ROOT, "ufsm_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".c", ".cpp")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "liboracle" not in text or f == "build.py", f
                assert "mx_oracle" not in text and "orc_" not in text, f
