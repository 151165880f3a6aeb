/* Host side (C23) of the MX U-Net forward: the op layer and the graph the reference keeps above its lp_* kernels, restated over
 * the C ABI of include/mi_lp.h. Names, argument meaning and error behaviour follow the reference's own declarations:
 *   nn_set_storage / nn_storage / nn_set_prec / nn_conv3d_fwd / _gn / _gn_stats / _split / _x / nn_gn_stats   src/nn.h:100, :194-195, :399-400, :416, :423-433, :442, :484
 *   unet_cfg / unet_create / unet_init / unet_forward_x / unet_forward_ct                               src/unet.h:18-128, :141, :176, :186, :428
 * Tensors are device pointers; an activation is an MX tensor registered with nn_set_storage (dt 8 / 4), as in the reference.
 */
#ifndef MI_UNET_H
#define MI_UNET_H
#include "mi_lp.h"
#include "mi_attn.h"
#ifdef __cplusplus
extern "C" {
#endif

/* ---- op layer (src/nn.h) ---- */
void nn_set_storage(const void *p, size_t bytes, int dt);      /* dt 8 MX-fp8, 4 MX-fp4, 2 fp16 planes, 0 forgets (fp32 planes) */
int nn_storage(const void *p);                                 /* the dt of the registered range holding p, else 0 */
void nn_storage_forget(const void *p);
void nn_set_prec(int p);                                       /* 3: MX-fp4 compute for every conv, else the storage decides; on tensors without MX storage 2 / 3 run the
                                                                  fp8 / fp4 entry on the planes as they are (src/nn.h:100, src/nn_bwd.cu:97-119) */
int nn_get_prec(void);                                         /* src/nn.h:115 */
void nn_set_gn_stored(int on);                                 /* GroupNorm statistics of the decoded stored output (src/nn_core.cu:7; default 0) */
size_t nn_mx8_bytes(shape5 s);
size_t nn_mx4_bytes(shape5 s);
typedef struct { const float *gamma, *beta, *mean, *rstd; int G; } nn_gn_t;          /* src/nn.h:431 */
/* y = conv3(silu(gn(x))) (G_in 0: x as is) with the GroupNorm statistics of y for G_out groups written to omean / orstd (src/nn.h:423) */
int nn_conv3d_fwd_gn_stats(const float *x, shape5 xs, int G_in, const float *gamma, const float *beta, const float *mean, const float *rstd,
                           const float *w, const float *b, int cout, float *y, int G_out, float eps, float *omean, float *orstd);
/* The reference's other conv entries of this path, same names and signatures (src/nn.h:399-400, :416, :442). The kernel family follows its rule
   (conv_fwd_tc, src/nn_bwd.cu:97-119): MX storage in means MX storage of the same format out; MX-fp4 storage or precision 3 runs the fp4 kernels,
   everything else fp8; an input of <= 8 channels runs the tap-packed fp8 stem whatever the format; a combination with no kernel prints and
   aborts. nn_conv3d_fwd: k 1 (the head of an MX tensor), k 3 stride 1 or 2, no GroupNorm. nn_conv3d_fwd_gn: the conv of silu(gn(x)).
   nn_conv3d_fwd_split: the conv of the channel concat [x (c_split channels), x2] under one GroupNorm of G_in groups over all xs.c channels
   (G_in 0: none), with the output's statistics for G_out groups. */
shape5 nn_conv3d_out_shape(shape5 xs, int cout, int k, int stride);
void nn_conv3d_fwd(const float *x, shape5 xs, const float *w, const float *b, int cout, int k, int stride, float *y);
int nn_conv3d_fwd_gn(const float *x, shape5 xs, int G, const float *gamma, const float *beta, const float *mean, const float *rstd,
                     const float *w, const float *b, int cout, float *y);
int nn_conv3d_fwd_split(const float *x, const float *x2, int c_split, shape5 xs, int G_in, const float *gamma, const float *beta, const float *mean, const float *rstd,
                        const float *w, const float *b, int cout, float *y, int G_out, float eps, float *omean, float *orstd);
/* input-side recompute conv: k 3 stride 1 (split / fused upsample / output statistics), k 3 stride 2, k 1 head (src/nn.h:432) */
int nn_conv3d_fwd_x(const float *x, const nn_gn_t *gx, const float *x2, const nn_gn_t *gx2, int c_split, int up, shape5 xs,
                    const float *w, const float *b, int cout, int k, int stride, float *y, int G_out, float eps, float *omean, float *orstd);
void nn_set_zrange(int zi0, int Di, int first, int last, int Do, int zo);   /* the next stride-1 MX convs compute output planes [zo, zo + xs.d) of a depth-Do tensor, plane z reading
                                                                               input plane z + zi0 of a depth-Di input; sums zeroed by the first, finalised by the last call; Di 0 = off
                                                                               (src/nn_bwd.cu:33-36) */
void nn_set_zrange_out(int on);                                /* ... straight into their planes of the depth-Do MX output (src/nn_bwd.cu:41-42) */
int nn_gn_stats(const float *x, shape5 s, int G, float eps, float *mean, float *rstd);   /* of a stored MX tensor; -1 when unsupported (src/nn.h:484) */
const char *nn_check(void);                                    /* src/nn.h:28 */

/* ---- U-Net graph (src/unet.h, src/unet.c:2567-2636, :2867-3121; inference, recompute mode) ----
   The entry points below carry the reference's names AND signatures (src/unet.h:18-128 unet_cfg, :141 unet_create, :157 unet_free, :159-160,
   :176, :185-187 forward, :258 unet_use_ema, :344-347 checkpoints, :357 unet_peek, :369-370 storage, :422 slabs, :428 unet_forward_ct), so a
   caller written against src/unet.h (predict.c) links against this library unchanged. Everything this build adds is named mi_unet_*. */
#define UNET_MAXLEV 8
/* The reference's configuration record, field for field (src/unet.h:18-128): the layout is part of the boundary. This build runs the plain
   U-Net (+ down_norm, + self-attention blocks with RoPE / no positional encoding and register tokens). Fields it honours: nlev, widths, cin,
   cout, G, down_norm, attn_blocks, attn_pe (0 PEG, 1 RoPE, 2 none, 3 scroll RoPE), attn_axis (1: radial attention), attn_reg, attn_mlp, dec_widths (0: the encoder's width), dec_convs (1: one-conv decoder block),
   enc_blocks (residual blocks after encoder levels >= 1), w4_2d, l0_norm (0 .. 4) with l0_slab, gn_ema; half_res and scan_norm concern the caller only. Any other field must be 0: unet_create prints which one is not and returns NULL. */
typedef struct {
    int nlev;
    int widths[UNET_MAXLEV];
    int cin, cout;
    int G;
    int down_norm;
    int scale_cond;
    int dec_widths[UNET_MAXLEV];
    int enc_blocks[UNET_MAXLEV];
    int dec_convs[UNET_MAXLEV];
    int ds_levels;
    int lat_guide;
    int lat_nsub;
    int8_t lat_sub[16];
    int half_res;
    int w4_2d;
    int l0_norm;
    int l0_slab;
    int gfilm;
    int scan_norm;
    int gn_ema;
    int attn_blocks;
    int attn_pe;
    int attn_reg;
    int attn_mlp;
    int attn_vres;
    int attn_axis;
    int attn_repeat;
    int attn_mem;
    int view_P, view_patch;
    int attn_deform, attn_dlev;
    int attn_dco;
    int attn_dinit;
    int emb_lev, emb_ch;
    int film;
    int skip_thr, skip_margin, skip_nl;
    int fstem, fstem_out;
    int lat_dec, lat_dec_raw, lat_dec_ng, lat_dec_wq;
} unet_cfg;
typedef struct unet unet;
unet *unet_create(const unet_cfg *cfg);                        /* src/unet.h:141; parameters allocated, activations when the first forward names a shape */
void unet_free(unet *u);
const unet_cfg *unet_cfg_of(const unet *u);                    /* src/unet.h:159 */
size_t unet_nparams(const unet *u);
void unet_init(unet *u, uint64_t seed);                        /* Kaiming normal sqrt(2 / (cin 27)), biases 0, head bias -2, gamma 1, beta 0 (src/unet.c:588-607); the EMA copy = the weights */
float *unet_param_ptr(unet *u);                                /* device pointers of the flat fp32 weights and of their EMA copy (src/unet.h:203-204), in unet_create's layout (src/unet.c:451-459: encoder blocks, downs, decoder blocks from the coarsest, head, down norms, attention stage) */
float *unet_ema_ptr(unet *u);
void unet_use_ema(unet *u, int on);                            /* forward with the EMA weights (1) or the live ones (0) (src/unet.h:258) */
/* no counterpart in the reference, which re-forms the forward copy of a cfg.w4_2d net's weights before every forward (src/unet.c:5310-5326): here
   the copy (fp4 convs' weights rounded per 32 x 32 block and tap) is re-formed after unet_load / mi_unet_set_params / unet_use_ema; a caller that
   writes the weights through unet_param_ptr / unet_ema_ptr says so with this call (it also drops the prepared-weight memo) */
void mi_unet_weights_changed(unet *u);
/* activation storage of the networks built from now on (src/unet.h:369-370): MX-fp8 (the default here; this build has no 16-bit storage, so
   unet_set_act_mx8(0) without mx4 is refused at the next forward) or packed MX-fp4, which takes precedence. The compute precision follows the
   op layer's policy (nn_set_prec(3): MX-fp4 weights over either storage). A change rebuilds the activations at the next forward. */
void unet_set_act_mx8(int on);
void unet_set_act_mx4(int on);
int unet_act_mx(void);                                         /* src/unet.h:430 */
/* Forward for one input shape xs = (n, cin, d, h, w), dims divisible by 2^(nlev-1); activation buffers are (re)allocated when the shape or
   the storage mode changes. train must be 0 (inference build: 1 aborts with a message). Returns the logits, fp32 [n][cout][d][h][w] on the
   device, owned by the net and valid until its next forward (src/unet.h:183-187). x: fp32 planes [n][cin][d][h][w]; unet_forward_x with
   x_h16: fp16 planes, read in place. Either is converted to the MX input tensor first (lp_f32_to_mx* / lp_h16_to_mx*, src/unet.c:2909-2919). */
const float *unet_forward(unet *u, const float *x, shape5 xs, int train);
const float *unet_forward_x(unet *u, const void *x, shape5 xs, int train, int x_h16);
shape5 unet_out_shape(const unet *u, shape5 xs);
/* the input built on the device from the uint8 CT window(s) (src/unet.h:428, src/unet.c:2858-2865, src/lp_mx_cvt.cu:29-55), then the forward.
   ct: xs.n windows of d x h x w voxels back to back (the reference's predict passes one); dyo / dxo: per window plane the row / column offset
   from the scroll axis, xs.d floats per window back to back; h16: the 16-bit type the input values are rounded to (2 fp16, 1 bf16, 0 none).
   xs.c must be 4 and xs.h == xs.w. */
const float *unet_forward_ct(unet *u, const uint8_t *ct, float mean, float isd, const float *dyo, const float *dxo, int axis, shape5 xs, int h16);
void unet_set_infer_slab(int planes);                         /* inference: the convs of level 0 (and of level 1 when the net has three or more levels; UFSM_INFER_SLAB_L1=0:
                                                                 level 0 only) in z-slabs of this many planes (rounded up to a multiple of 4); byte-identical logits; 0 = off
                                                                 (src/unet.h:422) */
void unet_set_slab_direct(int on);                            /* on (the default): each slab is written straight into the full-depth tensors. Off: the in-place form, one buffer per
                                                                 slab level for all its tensors, a slab temp and a carry plane, plane copies after each slab (src/unet.h:424,
                                                                 src/unet.c:2435-2440, :2540-2542); the same bytes, about four tensors of each such level less memory. The reference
                                                                 picks the form from the card's free memory (src/unet.c:1168-1173); here the caller does. */
/* ---- checkpoints in the reference's format (src/unet.h:342-357; src/unet.c:5534-5650 unet_save, :5650-5755 header, :5774-5800 unet_load): one
   line "UFSM{json}\n", then nparams fp32 weights, the EMA weights and optionally optimizer state (skipped here). unet_peek fills cfg and step
   from the header: 0, -1 when the file is unreadable, -2 naming (stderr) a feature of the checkpoint this build does not run. unet_load copies
   weights and EMA weights into a net of the same architecture (checked: nlev, widths, cin, cout, attention blocks, down_norm, nparams,
   payload size) and returns the saved step, or -1. unet_save writes weights and EMA. ---- */
int unet_peek(const char *path, unet_cfg *cfg, int *step);
void unet_set_scale(unet *u, double um);                       /* cfg.scale_cond nets: the input voxel size of the following forwards; the stem bias is b + c v with c = log2(um / 4.8) (src/unet.h:24, :141-144) */
void unet_set_film(unet *u, const float *codes, int k);        /* cfg.film nets: the k <= 4 codes of the following forwards (src/unet.h:148-149); the block norms' effective affines are remade when they change */
size_t unet_gfilm_off(const unet *u);                          /* cfg.gfilm: the offset of its first scale / shift pair in the parameter vector (src/unet.h:160) */
const float *mi_unet_gfilm_codes(const unet *u);               /* cfg.gfilm: the pooled codes of the last forward, widths[nlev-1] device floats (no counterpart in the reference's interface: its tests freeze them through the environment) */
size_t mi_unet_film_off(const unet *u);                        /* cfg.film: the same for its pairs (no counterpart in the reference's interface: its tests print the offset) */
/* cfg.attn_axis 1 / attn_pe 3 (src/unet.h:13-16, :470-474): the scroll axis of every sample of the following forwards. n records of stride floats
   (host memory, copied): ad (the window dim of the scroll axis: 0 z, 1 y, 2 x), valid (0: no axis), np (window planes along ad), div (window
   voxels per network input voxel), then per window plane along ad the axis centre (u, v) on the other two window dims in order, in window
   voxels (voxel centres at integers; may lie outside the window). n 0 / null, a record count other than the forward's sample count, or a plane
   count that does not fit the net's bottleneck grid: no axis (rays along the grid rows, grid-index coordinates) */
#define UNET_AXR(np) (4 + 2 * (np))
void unet_set_attn_axis(unet *u, const float *rec, int n, int stride);
/* radial attention's ray set after a forward (src/unet.h:475-477): rays per sample, slots per ray, the share of grid tokens a sample touches; -1 without */
int unet_attn_rays(const unet *u, int *Q, int *Nr, double *coverage);
void unet_set_cond(unet *u, float c);                          /* ... or the code c itself (src/unet.h:146-147) */
void unet_gn_ema_live(unet *u, int on);                        /* cfg.gn_ema: 1 = forwards normalise with the window's own statistics instead of the running ones (src/unet.h:172) */
long unet_gn_ema_updates(const unet *u);                       /* cfg.gn_ema: updates the loaded running statistics have seen (src/unet.h:288); 0: live statistics */
long unet_l0_updates(const unet *u);                           /* cfg.l0_norm 2: updates the loaded running statistics have seen (src/unet.h:275-299); the forward uses them
                                                                  once that count has reached the checkpoint's warm-up, live GroupNorm statistics before */
int unet_load(unet *u, const char *path);
int unet_save(const unet *u, const char *path, int step, const char *extra_json);
/* ---- additions of this build (no counterpart in src/unet.h) ---- */
void mi_unet_get_params(const unet *u, float *host);           /* the live weights, flat, in that layout */
void mi_unet_set_params(unet *u, const float *host);           /* ... and the EMA copy with them; drops the prepared-weight memos */
/* the forward on an input that already is the net's MX tensor (lp_f32_to_mx* output or lp_pred_input_mx rows), device pointer */
const float *mi_unet_forward_mx(unet *u, const void *xmx, shape5 xs);
/* unet_forward_ct with the windows and their offset rows given one pointer each (window n -> sample n; windows of a batch need not be contiguous) */
const float *mi_unet_forward_ct_n(unet *u, const uint8_t *const *ct, float mean, float isd, const float *const *dyo, const float *const *dxo, int axis, shape5 xs, int h16);
/* per-layer introspection for parity tests: the k-th conv output tensor of the last forward (device MX) and its shape, in execution order; NULL past the end */
const void *mi_unet_layer_out(const unet *u, int k, shape5 *s, const char **name);
/* the GroupNorm statistics the k-th conv produced (device [n * G] each); returns G, 0 when the layer has none */
int mi_unet_layer_stats(const unet *u, int k, const float **mean, const float **rstd);
int mi_unet_infer_slab(void);                                  /* unet_set_infer_slab's current value */
size_t mi_unet_peek_nparams(const char *path);                 /* the header's "nparams" (0: unreadable) */
/* ---- sliding-window prediction of a volume resident in device memory (src/predict.c: the --feather single pass, :282-333, :2538-2545,
   :3420-3436). vol: uint8 CT [dims0][dims1][dims2]; cubic windows of `window` voxels, up to `nbatch` (1 .. 64) per forward (the windows that hold material are
   spread evenly over the forwards that many need: 726 windows at up to 64 are 12 forwards of 61; the graph is rebuilt for that sample count if it was built for another), with
   `halo` voxels of context per side tile the volume at stride window - 2 halo in z-y-x order; each runs as a sample of unet_forward_ct (z-score mean / isd; axis, cy, cx: the scroll axis
   sign and its centre in volume y / x, axis 0: no direction channels) and places uint8(255 sigmoid(logit 0) + .5) where CT >= the
   prediction iso over its interior plus `feather` voxels of its upper halo; the window borders are then blended over `feather` voxels
   (0: none; <= halo) into out: uint8 [dims0][dims1][dims2]. Windows whose CT holds no voxel >= iso are skipped (their interior stays 0
   and their neighbours' blends renormalise). nwin[0..1] (may be null): windows in all, windows computed. Returns 0, or -1 for a
   geometry the graph cannot run. Every window's prediction stays in device memory until the blend: nwin (stride + feather)^3 bytes. */
int mi_unet_predict_volume(unet *u, int window, int nbatch, const uint8_t *vol, const int64_t dims[3], int halo, int feather, float mean, float isd,
                           int axis, float cy, float cx, uint8_t *out, int64_t nwin[2]);
#ifdef __cplusplus
}
#endif
#endif
