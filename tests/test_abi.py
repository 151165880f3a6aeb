"""The C-ABI library loads and exports every symbol include/mi_lp.h declares; descriptor layouts match the reference's (no compute, no GPU)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_functions(header="mi_lp.h", prefixes=("lp_", "mi_", "gnp_")):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b([a-z][a-z0-9_]*)\s*\([^;{]*\)\s*;", text)
    return sorted(set(n for n in names if n.startswith(prefixes)))


def test_header_declares_the_forward_subset():
    names = header_functions()
    for must in ["lp_conv_fwd_f8", "lp_conv_fwd_f4", "lp_conv_fwd_s2_f8", "lp_f32_to_mx8", "lp_f32_to_mx4", "lp_h16_to_mx8", "lp_mx8_to_f32", "lp_mx4_to_f32",
                 "lp_mx8_bytes", "lp_mx4_bytes", "lp_pred_input_mx", "lp_pred_input_mx8", "lp_gn_silu_apply_mx", "lp_add_mx", "lp_up2_fwd_mx", "lp_up2_fwd_mx_blocks",
                 "lp_conv1_fwd_mx", "lp_conv1_fwd_mx_h16", "lp_conv1_fwd_mx_h16_r", "lp_conv1_fwd_mx_r", "lp_gn_sums_mx", "lp_gn_sums_mx_n", "lp_check", "gnp_mk",
                 "lp_gn_slab_any", "lp_wmemo_step", "lp_wmemo_clear"]:
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
    names = header_functions("mi_unet.h", ("nn_", "unet_"))
    assert "unet_forward_x" in names and "nn_conv3d_fwd_x" in names and "nn_set_storage" in names and "unet_predict_volume" in names
    for n in names:
        assert hasattr(H, n), "libufsm_host.so does not export %s" % n
    assert C.sizeof(unet.unet_cfg) == 4 * (2 + unet.UNET_MAXLEV + 4 + 4 + 1)


def test_descriptor_layouts():
    from ufsm_amd import shape5, gnp_t, split_t
    assert C.sizeof(shape5) == 20
    assert C.sizeof(gnp_t) == 56 and gnp_t.G.offset == 32 and gnp_t.zhw.offset == 48
    assert C.sizeof(split_t) <= 128                                  # src/nn_lp.h:41
    assert split_t.gp2.offset == 32 and split_t.up.offset == 88 and split_t.wkey.offset == 96 and split_t.stored_stats.offset == 108


def test_size_helpers_and_no_device_behaviour():
    from ufsm_amd import lib
    assert lib.lp_mx8_bytes(2, 128, 1000) == 2 * 4 * 1000 * 33       # src/lp_mx_cvt.cu:6
    assert lib.lp_mx4_bytes(2, 128, 1000) == 2 * 4 * 1000 * 17
    assert lib.lp_mx8_bytes(1, 4, 10) == 10 * 9 and lib.lp_mx8_bytes(1, 12, 10) == 10 * 17 and lib.lp_mx4_bytes(1, 12, 10) == 10 * 9
    assert lib.lp_gn_slab_any() == 0
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
