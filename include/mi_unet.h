/* Host side (C23) of the MX U-Net forward: the op layer and the graph the reference keeps above its lp_* kernels, restated over
 * the C ABI of include/mi_lp.h. Names, argument meaning and error behaviour follow the reference's own declarations:
 *   nn_set_storage / nn_storage / nn_set_prec / nn_conv3d_fwd_gn_stats / nn_conv3d_fwd_x / nn_gn_stats   src/nn.h:100, :194-195, :423-433, :484
 *   unet_cfg / unet_create / unet_init / unet_forward_x / unet_forward_ct                               src/unet.h:1-30, :141, :186, :428
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
void nn_set_prec(int p);                                       /* 3: MX-fp4 compute for every conv, else the storage decides (src/nn_bwd.cu:110-112) */
void nn_set_gn_stored(int on);                                 /* GroupNorm statistics of the decoded stored output (src/nn_core.cu:7; default 0) */
size_t nn_mx8_bytes(shape5 s);
size_t nn_mx4_bytes(shape5 s);
typedef struct { const float *gamma, *beta, *mean, *rstd; int G; } nn_gn_t;          /* src/nn.h:431 */
/* y = conv3(silu(gn(x))) (G_in 0: x as is) with the GroupNorm statistics of y for G_out groups written to omean / orstd (src/nn.h:423) */
int nn_conv3d_fwd_gn_stats(const float *x, shape5 xs, int G_in, const float *gamma, const float *beta, const float *mean, const float *rstd,
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

/* ---- U-Net graph (src/unet.h, src/unet.c:2567-2636, :2867-3121; inference, recompute mode, no residual blocks) ---- */
#define UNET_MAXLEV 8
typedef struct {
    int cin;                   /* input channels (4 for CT windows: z-scored CT, 0, radial dy, dx) */
    int nlev;                  /* levels */
    int widths[UNET_MAXLEV];   /* channels per level */
    int G;                     /* GroupNorm groups (min(G, C) is used, src/unet.c:297) */
    int head_out;              /* logits */
    int act_dt;                /* activation storage: 8 MX-fp8, 4 MX-fp4 */
    int prec;                  /* 3: fp4 compute everywhere (MX-fp4 weights over MX-fp8 storage), else by storage */
    /* transformer blocks on the bottleneck level's raw output (src/unet.h:72-80; 0 = none): tokens = attn_reg learned register rows + the
       bottleneck grid, pre-LN blocks (MHSA with QK-norm, heads of 48, SwiGLU) on the MX-fp8 attention core with MX-fp8 linears; the level's
       output GroupNorm moves after the stage. The bottleneck width must be a multiple of 48 */
    int attn_blocks;
    int attn_pe;               /* 1 axial 3-D RoPE, 2 none (0 PEG and 3 scroll RoPE are not provided) */
    int attn_reg;              /* register tokens per sample */
    int attn_mlp;              /* SwiGLU hidden width (0: 8/3 of the width rounded up to 32) */
    int down_norm;             /* 1: GroupNorm + SiLU after each stride-2 down conv, applied by the next block's conv1 while it stages its input
                                  (parameters after the head, src/unet.h:23, src/unet.c:459); 0: the older layout without it */
} unet_cfg;
typedef struct unet unet;
unet *unet_create(const unet_cfg *cfg, shape5 in);             /* in: the window (n, cin, d, h, w); dims divisible by 2^(nlev-1) */
void unet_free(unet *u);
size_t unet_nparams(const unet *u);
void unet_init(unet *u, uint64_t seed);                        /* Kaiming normal sqrt(2 / (cin 27)), biases 0, head bias -2, gamma 1, beta 0 (src/unet.c:588-607) */
void unet_get_params(const unet *u, float *host);              /* the flat parameter vector in unet_init's order */
void unet_set_params(unet *u, const float *host);
int unet_forward_x(unet *u, const void *x, float *logits);     /* x: device MX tensor (act_dt) of the input; logits: device fp32 [n][head_out][S] */
/* the input built on the device from a uint8 CT window of one sample (src/unet.c:2858-2865, src/lp_mx_cvt.cu:29-55), then the forward */
int unet_forward_ct(unet *u, const uint8_t *ct, float mean, float isd, const float *dyo, const float *dxo, int axis, float *logits);
/* the same over the network's in.n windows in one forward (window n -> sample n; per-sample results equal the one-window forward's) */
int unet_forward_ct_n(unet *u, const uint8_t *const *ct, float mean, float isd, const float *const *dyo, const float *const *dxo, int axis, float *logits);
/* per-layer introspection for parity tests: the k-th conv output tensor (device MX) and its shape, in execution order; NULL past the end */
const void *unet_layer_out(const unet *u, int k, shape5 *s, const char **name);
/* the GroupNorm statistics the k-th conv produced (device [n * G] each); returns G, 0 when the layer has none */
int unet_layer_stats(const unet *u, int k, const float **mean, const float **rstd);
/* ---- checkpoints in the reference's format (src/unet.c:5534-5650 unet_save, :5650-5700 read_header, :5774-5800 unet_load): one line
   "UFSM{json}\n", then nparams fp32 weights, the EMA weights and optionally optimizer state. unet_read_header fills cfg (act_dt 8, prec 0)
   from the header's architecture keys; it returns 0, -1 when the file is unreadable, or -2 naming (stderr) a feature of the checkpoint this
   build does not run (decoder widths, residual blocks, latent grids, deep supervision, FiLM, fine stems, running-statistics norms, the
   attention stage's other forms). unet_load / unet_load_ema copy the weights / the EMA weights into a net of the same architecture
   (checked: nlev, widths, cin, cout, attention blocks, nparams, payload size); unet_save writes weights and EMA (= the weights). ---- */
int unet_read_header(const char *path, unet_cfg *cfg, size_t *nparams, int *step);
int unet_load(unet *u, const char *path);
int unet_load_ema(unet *u, const char *path);
int unet_save(const unet *u, const char *path, int step, const char *extra);   /* extra: a JSON object for the header's "extra" key, or null */
void unet_set_infer_slab(int planes);                         /* inference: the level-0 convs in z-slabs of this many planes (rounded up to a multiple of 4), each slab written
                                                                 straight into the full-depth tensors; byte-identical logits; 0 = off (src/unet.h:422-424, direct slab outputs) */
int unet_get_infer_slab(void);
shape5 unet_in_shape(const unet *u);                          /* the window the graph was created for */
const unet_cfg *unet_config(const unet *u);
/* ---- sliding-window prediction of a volume resident in device memory (src/predict.c: the --feather single pass, :282-333, :2538-2545,
   :3420-3436). vol: uint8 CT [dims0][dims1][dims2]; windows of the graph's size (cubic; the graph's in.n samples are that many windows per forward) with
   `halo` voxels of context per side tile the volume at stride window - 2 halo in z-y-x order; each runs as a sample of unet_forward_ct_n (z-score mean / isd; axis, cy, cx: the scroll axis
   sign and its centre in volume y / x, axis 0: no direction channels) and places uint8(255 sigmoid(logit 0) + .5) where CT >= the
   prediction iso over its interior plus `feather` voxels of its upper halo; the window borders are then blended over `feather` voxels
   (0: none; <= halo) into out: uint8 [dims0][dims1][dims2]. Windows whose CT holds no voxel >= iso are skipped (their interior stays 0
   and their neighbours' blends renormalise). nwin[0..1] (may be null): windows in all, windows computed. Returns 0, or -1 for a
   geometry the graph cannot run. Every window's prediction stays in device memory until the blend: nwin (stride + feather)^3 bytes. */
int unet_predict_volume(unet *u, const uint8_t *vol, const int64_t dims[3], int halo, int feather, float mean, float isd,
                        int axis, float cy, float cx, uint8_t *out, int64_t nwin[2]);
#ifdef __cplusplus
}
#endif
#endif
