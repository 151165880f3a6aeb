"""The checkpoint header reader on headers as the reference writes them (src/unet.c:5546-5640): host-only, no GPU."""
import ctypes as C

import pytest


def read(tmp_path, header, payload=b""):
    from ufsm_amd.unet import load_host, unet_cfg
    H = load_host()
    p = tmp_path / "h.ckpt"
    p.write_bytes(header.encode() + payload)
    cfg = unet_cfg(); step = C.c_int(0)
    rc = H.unet_peek(str(p).encode(), C.byref(cfg), C.byref(step))
    return rc, cfg, H.mi_unet_peek_nparams(str(p).encode()), step.value


def test_reads_the_reference_header(tmp_path):
    # the test net of tests/test_predict_feather.c:73-76 as unet_save writes it (keys in its order, the caller's runtime object as extra)
    h = ('UFSM{"nlev":2,"widths":[32,64],"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,"nparams":336129,"step":1,"sparse24":0,"wq":0,"muon_mom":0,'
         '"extra":{"runtime":{"version":1,"train_window":96,"prec":1,"f16":1,"act_mx4":0,"act_mx8":1,"grad_mx8":1,"input_mx":1,"input_prec":8,"gn_stored":0,"policy":"","optimizer":"muon"}}}\n')
    rc, cfg, n, step = read(tmp_path, h)
    assert rc == 0 and (cfg.nlev, cfg.widths[0], cfg.widths[1], cfg.cin, cfg.cout, cfg.G, cfg.down_norm, cfg.attn_blocks, cfg.half_res) == (2, 32, 64, 4, 1, 8, 1, 0, 0)
    assert n == 336129 and step == 1


def test_parameter_layout_follows_unet_create():
    """The flat layout the tests' graph (tests/unet_ref.py) and the host library share, against the reference's unet_create (src/unet.c:451-459):
    encoder blocks, down convs, the decoder blocks from the coarsest level to level 0, the head, the down norms; a block is c1.w, c1.b, n1.gamma,
    n1.beta, c2.w, c2.b, n2.gamma, n2.beta. The count of the two-level test net above, term by term."""
    import unet_ref
    lay, n = unet_ref.param_layout(4, [32, 64], 1, 1)
    enc0 = 32 * 4 * 27 + 32 + 64 + 32 * 32 * 27 + 32 + 64
    enc1 = 64 * 32 * 27 + 64 + 128 + 64 * 64 * 27 + 64 + 128
    down0 = 32 * 32 * 27 + 32
    dec0 = 32 * 96 * 27 + 32 + 64 + 32 * 32 * 27 + 32 + 64
    assert n == enc0 + enc1 + down0 + dec0 + (32 + 1) + 64 == 336129
    lay, n = unet_ref.param_layout(4, [8, 16, 32, 64], 2, 1)
    order = [k[:-2] for k in lay if k.endswith(".w")] + [k[:-6] for k in lay if k.startswith("dn") and k.endswith(".gamma")]
    assert order == ["enc0.c1", "enc0.c2", "enc1.c1", "enc1.c2", "enc2.c1", "enc2.c2", "enc3.c1", "enc3.c2", "down0", "down1", "down2",
                     "dec2.c1", "dec2.c2", "dec1.c1", "dec1.c2", "dec0.c1", "dec0.c2", "head", "dn0", "dn1", "dn2"]
    offs = [lay[k][0] for k in lay]
    assert offs == sorted(offs) and lay["dec2.c1.w"][1] == (32, 64 + 32, 27) and lay["dec0.c1.w"][1] == (8, 16 + 8, 27)      # [up(coarse) | skip] input channels
    keys = list(lay)
    i = keys.index("dec1.c1.w")
    assert keys[i:i + 8] == ["dec1.c1.w", "dec1.c1.b", "dec1.n1.gamma", "dec1.n1.beta", "dec1.c2.w", "dec1.c2.b", "dec1.n2.gamma", "dec1.n2.beta"]


def test_attention_keys_and_extra_shadowing(tmp_path):
    h = ('UFSM{"nlev":4,"widths":[32,64,128,192],"attn_blocks":2,"attn_pe":1,"attn_reg":4,"attn_mlp":512,"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,'
         '"nparams":5,"step":77,"sparse24":0,"wq":0,"muon_mom":0,"extra":{"nlev":9,"film":3}}\n')
    rc, cfg, n, step = read(tmp_path, h)                                 # keys inside the caller's extra object do not count
    assert rc == 0 and (cfg.nlev, cfg.widths[3], cfg.attn_blocks, cfg.attn_pe, cfg.attn_reg, cfg.attn_mlp) == (4, 192, 2, 1, 4, 512) and step == 77


def test_caller_side_keys_pass_through(tmp_path):
    # half-resolution windows and per-scan normalisation are transforms the caller applies around the forward (src/unet.h:52-56, :88-89): no refusal
    h = 'UFSM{"nlev":2,"widths":[32,64],"half_res":1,"scan_norm":1,"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,"nparams":10,"step":1,"extra":{}}\n'
    rc, cfg, n, step = read(tmp_path, h)
    assert rc == 0 and cfg.half_res == 1 and cfg.scan_norm == 1


@pytest.mark.parametrize("feature", ['"lat_guide":1', '"attn_mem":4', '"lat_dec":[16,0,1]', '"film":7', '"fstem":[2,16]', '"view_P":4', '"attn_deform":4', '"l0_norm":7'])
def test_refuses_architectures_it_does_not_run(tmp_path, feature):
    h = 'UFSM{"nlev":2,"widths":[32,64],%s,"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,"nparams":10,"step":1,"extra":{}}\n' % feature
    assert read(tmp_path, h)[0] == -2


@pytest.mark.parametrize("keys", ['"sparse24":1,"wq":0', '"sparse24":3,"wq":0,"muon_mom":0,"sparse24_lv":6,"sparse24_hard":1', '"sparse24":0,"wq":4', '"sparse24":0,"wq":8'])
def test_refuses_transformed_weight_storage(tmp_path, keys):
    """2:4-masked or packed fp8 / fp4 weights: the reference applies the masks / packs the weights after reading the same fp32 payload
    (src/unet.c:5703-5707, :5839-5840); loading the file as dense master weights would run another function, so it is refused by name."""
    h = 'UFSM{"nlev":2,"widths":[32,64],"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,"nparams":336129,"step":1,%s,"extra":{}}\n' % keys
    assert read(tmp_path, h)[0] == -2
    h0 = 'UFSM{"nlev":2,"widths":[32,64],"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,"nparams":336129,"step":1,"sparse24":0,"wq":0,"extra":{}}\n'
    assert read(tmp_path, h0)[0] == 0


def test_reads_the_2d_weight_scale_key(tmp_path):
    h = 'UFSM{"nlev":2,"widths":[32,64],"w4_2d":1,"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,"nparams":10,"step":3,"extra":{}}\n'
    rc, cfg, n, step = read(tmp_path, h)
    assert rc == 0 and cfg.w4_2d == 1 and step == 3


def test_reads_the_slab_statistics_keys(tmp_path):
    # cfg.l0_norm as unet_save writes it (src/unet.c:5577-5584, read at :5726-5739): 4 with its slab depth, 1 (none) / 3 (ws) bare, 2 (ema) with the running statistics
    h = 'UFSM{"nlev":2,"widths":[32,64],"l0_norm":4,"l0_slab":16,"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,"nparams":10,"step":3,"extra":{"l0_norm":2}}\n'
    rc, cfg, n, step = read(tmp_path, h)
    assert rc == 0 and (cfg.l0_norm, cfg.l0_slab) == (4, 16)
    for mode in (1, 3):
        rc, cfg, n, step = read(tmp_path, h.replace('"l0_norm":4,"l0_slab":16', '"l0_norm":%d' % mode))
        assert rc == 0 and (cfg.l0_norm, cfg.l0_slab) == (mode, 0)
    rc, cfg, n, step = read(tmp_path, h.replace('"l0_norm":4,"l0_slab":16', '"l0_norm":2,"l0_n":40,"l0_warm":100,"l0_mom":0.01,"l0_run":[0.5,1,2]'))
    assert rc == 0 and cfg.l0_norm == 2


def test_reads_the_decoder_variants(tmp_path):
    # cfg.dec_widths / cfg.dec_convs as unet_save writes them (src/unet.c:5549-5550, :5595-5596; read at :5674, :5700)
    h = 'UFSM{"nlev":3,"widths":[32,64,128],"dec_widths":[0,32,0],"enc_blocks":[0,2,1],"dec_convs":[2,1,0],"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,"nparams":10,"step":3,"extra":{}}\n'
    rc, cfg, n, step = read(tmp_path, h)
    assert rc == 0 and list(cfg.dec_widths[:3]) == [0, 32, 0] and list(cfg.dec_convs[:3]) == [2, 1, 0] and list(cfg.widths[:3]) == [32, 64, 128] and list(cfg.enc_blocks[:3]) == [0, 2, 1]


def test_reads_the_running_statistics_key(tmp_path):
    # cfg.gn_ema with its statistics (src/unet.c:5587-5592, read at :5744-5751)
    h = 'UFSM{"nlev":2,"widths":[32,64],"gn_ema":1,"ge_n":5,"ge_warm":500,"ge_mom":0.01,"ge_run":[0,1,0,1],"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,"nparams":10,"step":3,"extra":{}}\n'
    rc, cfg, n, step = read(tmp_path, h)
    assert rc == 0 and cfg.gn_ema == 1 and cfg.l0_norm == 0 and cfg.scale_cond == 0
    rc, cfg, n, step = read(tmp_path, 'UFSM{"nlev":2,"widths":[32,64],"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":1,"nparams":10,"step":3,"extra":{}}\n')
    assert rc == 0 and cfg.scale_cond == 1                          # voxel-size conditioning (src/unet.c:5672)
    rc, cfg, n, step = read(tmp_path, 'UFSM{"nlev":2,"widths":[32,96],"film":3,"attn_blocks":1,"attn_pe":1,"attn_reg":0,"attn_mlp":256,"gfilm":1,"cin":4,"cout":1,"G":8,"down_norm":1,"scale_cond":0,"nparams":10,"step":3,"extra":{"film":1}}\n')
    assert rc == 0 and cfg.film == 3 and cfg.gfilm == 1             # FiLM by host codes and by the pooled attention output (src/unet.c:5683, :5742)


def test_rejects_foreign_files(tmp_path):
    assert read(tmp_path, "not a checkpoint\n")[0] == -1
    assert read(tmp_path, 'UFSM{"nlev":2,"widths":[32,64],"cin":4,"cout":1,"skip_empty":[80,2,1],"nparams":1}\n')[0] == -2   # trained with masked convs
    rc, cfg, n, step = read(tmp_path, 'UFSM{"nlev":2,"widths":[32,96],"attn_blocks":1,"attn_pe":3,"attn_reg":0,"attn_mlp":256,"attn_axis":1,"cin":4,"cout":1,"nparams":1}\n')
    assert rc == 0 and cfg.attn_pe == 3 and cfg.attn_axis == 1     # scroll RoPE, radial attention (src/unet.c:5691)
    assert read(tmp_path, 'UFSM{"nlev":2,"widths":[32,96],"attn_blocks":1,"attn_pe":4,"attn_reg":0,"attn_mlp":256,"cin":4,"cout":1,"nparams":1}\n')[0] == -2
    assert read(tmp_path, 'UFSM{"nlev":2,"widths":[32,96],"attn_blocks":1,"attn_pe":1,"attn_reg":0,"attn_mlp":256,"attn_axis":2,"cin":4,"cout":1,"nparams":1}\n')[0] == -2
    rc, cfg, n, step = read(tmp_path, 'UFSM{"nlev":2,"widths":[32,96],"attn_blocks":1,"attn_pe":0,"attn_reg":0,"attn_mlp":256,"attn_vres":1,"cin":4,"cout":1,"nparams":1}\n')
    assert rc == 0 and cfg.attn_pe == 0 and cfg.attn_vres == 1     # PEG, value residual
