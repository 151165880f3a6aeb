/* C ABI of the MI355X (gfx950) MX low-precision 3-D U-Net forward kernels.
 *
 * Drop-in for the forward subset of the reference's internal kernel interface src/nn_lp.h: same entry-point names,
 * argument order, dtype codes, by-value descriptors and tensor / scale layouts. Every declaration cites the reference
 * declaration it replaces. All pointers named x / y / w / b / gamma ... are DEVICE pointers unless stated otherwise;
 * all work is issued on the HIP null stream, asynchronously, in stream order (as the reference on the default stream).
 *
 * dtype codes (src/lp_f4fwd.cuh:1224): 0 fp32 planes [n][C][S], 1 bf16 planes, 2 fp16 planes, 3 MX-fp8, 4 MX-fp4.
 * MX tensor of N x C x S (src/lp_common.cuh:100-106, :132-134): bw = 8 / 16 / 32 for C <= 8 / <= 16 / else,
 * nb = ceil(C / bw); data[n][blk][voxel][bw] e4m3 bytes (fp4: bw/2 bytes, channel k = nibble k&1 of byte k/2) followed by
 * the scale plane sc[n][blk][voxel] of E8M0 bytes.
 */
#ifndef MI_LP_H
#define MI_LP_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* ---- descriptors, passed by value (layouts identical to the reference's) ---- */
typedef struct { int n, c, d, h, w; } shape5;                                   /* src/nn.h:21 */
typedef struct { const float *gamma, *beta, *mean, *rstd; int G; int zs, zo, ns, zhw; } gnp_t;   /* src/nn_lp.h:15; G == 0: no transform */
typedef struct {                                                                 /* src/nn_lp.h:32 */
    const void *x2; int c_split; void *y2; int o_split; int accum; gnp_t gp2; int16_t up, yD; unsigned sr; unsigned wkey;
    int zlo, zhi; int stored_stats; unsigned osr; int16_t zi0, Di, o_pad, zw0, zw1, yzo;
} split_t;
/* Fields honoured by this build: x2, c_split, gp2, up, wkey, stored_stats, zlo, zhi, and the z-range of the reference's slab inference:
   zi0 / Di (output plane z of the xs.d planes computed reads input plane z + zi0 of depth-Di inputs; Di 0 = off) and yzo / yD (the MX
   output is planes [yzo, yzo + xs.d) of a depth-yD tensor; yD 0 = a depth-xs.d tensor), stride 1 (src/nn_lp.h:36-40). Training and
   z-window fields (y2, o_split, accum, sr, osr, o_pad, zw0, zw1) must be zero: a call that sets one prints a message and aborts, as the
   reference does for unsupported combinations (src/lp_f8fwd.cu:28).
   Slab-local GroupNorm statistics (gnp_t.ns > 0, src/nn_lp.h:15-18: mean / rstd hold one row per (sample, z-slab), [n][ns][G]; plane z reads
   row n * ns + clamp((z + zo) / zs, 0, ns - 1); zhw = voxels per plane) are honoured by every reader of an MX tensor: the conv entries (both
   segments' of a split input; not the upsampled segment's), the stride-2 entry, the 1x1x1 head, lp_gn_silu_apply_mx and mi_conv_prestage. */

/* tile masks of a masked ("skip-empty") conv (src/nn_lp.h:44): m the output tiles to compute, nullptr: dense */
typedef struct { const uint8_t *m, *mi; int my, mx, zoff; } skipm_t;
/* What the reference's kernel units ask its op layer before a conv (src/nn_lp.h:45-48, src/lp_common.cuh:42; defined there in
   src/nn_skip.cu:130-157 and src/nn_bwd.cu:57). This library asks the same questions before every conv launch and refuses (message +
   abort) a masked conv or an active z-window, which it does not build. Its own definitions are weak and answer "dense" / "no window":
   linked into the reference, the reference's definitions take over. */
skipm_t lp_skip_get(shape5 xs, split_t sp, int fwd);
int nn_skip_fwd_level(shape5 xs, split_t sp);
int nn_skip_masks(shape5 xs, split_t sp);
int zw_win(int D, int *z0, int *z1);

/* GroupNorm sum slots (src/gnacc.cuh:8-9): `osum` / `sums` buffers are arrays of 3 x uint64 fixed-point slots (24 bytes each:
   fraction in units of 2^-64, signed integer part, count of non-finite contributions), two per (sample, group): sum, sum of squares */
#define MI_GN_SLOT_BYTES 24

/* ---- convolutions ---- */
/* 3x3x3, stride 1, pad 1; MX-fp8 (e4m3) compute. Replaces src/nn_lp.h:53 (lp_conv_fwd_f8, src/lp_f8fwd.cu:26-52). Returns 0. */
int lp_conv_fwd_f8(const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp, double *osum, int Go, split_t sp);
/* the same with MX-fp4 (e2m1) compute. Replaces src/nn_lp.h:54 (src/lp_f4fwd.cu:30-51). */
int lp_conv_fwd_f4(const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp, double *osum, int Go, split_t sp);
/* 3x3x3, stride 2, pad 1 (ys = output shape). Replaces src/nn_lp.h:104 (src/lp_s2.cu:647-754). Returns 0, or 3 when fp4 compute ran. */
int lp_conv_fwd_s2_f8(const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, shape5 ys, gnp_t gp);
/* prepared-weight memo (src/nn_lp.h:56-57): a conv called with sp.wkey != 0 reuses its quantised weights until the next step / clear */
void lp_wmemo_step(unsigned step);
void lp_wmemo_clear(void);
/* 2-D fp4 weight scales (src/nn_lp.h:58, src/lp_f4fwd.cu:67-83): the stride-1 e2m1 weight preps of more than 16 input channels take one E8M0
   scale per tap and 32 x 32 (output x input channel) tile; a change drops the prepared weights. Default from UFSM_W4_2D (0). */
void lp_set_w4_2d(int on);
/* w [Co][Ci][T] rounded in place to MX-fp4 values, one scale per Bo x Bi block and tap (src/nn_lp.h:124, src/lp_mx_cvt.cu:369-395);
   nn_fakeq_w4_2d (src/nn.h:774): B x B blocks */
void lp_fakeq_w4(float *w, int Co, int Ci, int T, int Bo, int Bi);
void nn_fakeq_w4_2d(float *w, int Co, int Ci, int T, int B);
/* the level-0 normalisation alternatives' device helpers (src/nn.h:465-477, src/nn_l0norm.cu): constant GroupNorm statistics for N samples (run
   null: mean 0, rstd 1; else run = [mean G | var G] and rstd = 1 / sqrt(var + eps)); scaled weight standardisation per output channel over its
   fan-in of n contiguous weights, wh = gain (w - mean) / (std sqrt(n) + eps) (wh may be w) */
void nn_gn_const_fill(float *mean, float *rstd, const float *run, int N, int G, float eps);
void nn_axpy(float *y, float a, const float *x, size_t n);      /* y += a x (src/nn.h) */
/* FiLM on a GroupNorm's affine (src/nn.h:494-504): the norm's C channels at offsets gam / bet of the parameter vector p, its K x C pairs at fo
   (scales first); the effective pair goes into the forward weights fw. nn_film_fwd: K <= 4 host codes, from p's affine. nn_gfilm_fwd: K device
   codes gv, from the affine fw holds (kept in g1). nn_gfilm_pool: g[c] = mean over S of x[c S + s] */
void nn_film_fwd(const float *p, float *fw, size_t gam, size_t bet, size_t fo, int C, int K, const float *codes);
void nn_gfilm_pool(const float *x, int C, long S, float *g);
void nn_gfilm_fwd(const float *p, float *fw, size_t gam, size_t bet, size_t fo, int C, int K, const float *gv, float *g1);
void nn_ws_fwd(float *wh, const float *w, int cout, int n, float gain, float eps);
/* no counterpart in the reference (its stride-2 entry carries no split_t and prepares the weights per call): memo id of the calling thread's
   next lp_conv_fwd_s2_f8, mi_conv_down2_fwd or mi_convt_up2_fwd, as split_t.wkey for the stride-1 entries; consumed by that call. For inference
   loops with constant weights (lp_wmemo_step / lp_wmemo_clear drop the prepared images as for the other convs). */
void mi_conv_s2_wkey(unsigned wkey);
/* Tuning knob of the tap-packed kernel for <= 4 input channels: consecutive z tiles a workgroup walks (weights and constants set up once,
 * the next tile's input in flight during this tile's MFMAs). 0 (default) = chosen from the launch size. Results do not depend on it.
 * Calling thread only. The reference's kernel walks up to 32 (8 for wider rows),
 * overridden by UFSM_F8S_ZC (src/lp_f8fwd.cuh:412-416). */
void mi_conv_stem_zc(int zc);
/* tuning knob of the calling thread (no counterpart in the reference): stride-1 launches with fewer tiles of 128 output channels than this run as
   slices of 64 channels, twice the workgroups; 0: never, -1: the default (192, or MI_CONV_SPLIT). The results do not depend on it. */
void mi_conv_split(int tiles);
/* Extension: which kernel takes the calling thread's 3x3x3 stride-2 convs on 32-channel rows. -1 (default): the kernel that reads the taps' rows
   straight from the stored tensor when the launch has enough output voxels to fill the device, else the general kernel (staged halo);
   0: always the general kernel; 1: the direct kernel whenever its operands allow it. The results are the same conv either way. */
void mi_conv_s2_direct(int mode);
/* 1x1x1 head with eight outputs on whole 32-channel blocks: where its 8 x 32 products per voxel run. mode 1: the matrix pipe (batched 4 x 4 x 1
   fp32 outer products, one product per accumulator and step, in channel order), 0: fused multiply-adds on the vector ALUs, -1: the default
   (1, or the environment's MI_HEAD_MFMA). The two give the same bits; the setting is the calling thread's. No counterpart in the reference. */
void mi_conv1_matrix(int mode);
/* no counterpart in the reference (its convs transform their input while staging, every time): GroupNorm + SiLU of x and re-quantisation to
   MX-fp8 / MX-fp4 (ybits 8 / 4) once, for a tensor several convs read; they then take y with no GroupNorm. s.c a multiple of 32. In a split
   input, gp2.G = -1 says "x2 carries no GroupNorm, gp is x's own" (gp2.G = 0 keeps the reference's meaning: gp spans both segments). */
int mi_conv_prestage(const void *x, int xdt, shape5 s, gnp_t gp, void *y, int ybits);
/* the same from an MX-fp8 tensor into both formats at once (y8 MX-fp8, y4 MX-fp4: the bytes of the two single calls from one read and one
   evaluation): a tensor whose readers compute in different formats. mi_conv_x2_dt(4) before a conv entry says that the calling thread's next
   split conv's second segment is stored as MX-fp4 although x is MX-fp8 (3: MX-fp8 beside an MX-fp4 x; the descriptor carries one format) */
int mi_conv_prestage2(const void *x, shape5 s, gnp_t gp, void *y8, void *y4);
void mi_conv_x2_dt(int dt);
gnp_t gnp_mk(const float *gamma, const float *beta, const float *mean, const float *rstd, int G);   /* src/nn_lp.h:19 */
int lp_gn_slab_any(void);                                                                         /* src/nn_lp.h:20: any statistics array registered */
/* the statistics array `mean` holds one row per (sample, z-slab) with this geometry: every gnp_t gnp_mk builds from it (and lp_gn_silu_apply_mx,
   which takes the pointers) carries it. ns <= 0 removes the entry, a null mean clears the registry (src/nn.h:471, src/nn_fwd.cu:12-22) */
void lp_gn_slab_reg(const float *mean, int zs, int zo, int ns, int zhw);

/* ---- MX tensor conversions (src/nn_lp.h:111-118, :126; src/lp_mx_cvt.cu:6-79, :429-447) ---- */
size_t lp_mx8_bytes(int N, int C, size_t S);
size_t lp_mx4_bytes(int N, int C, size_t S);
void lp_f32_to_mx8(const float *x, int N, int C, size_t S, void *y);
void lp_f32_to_mx4(const float *x, int N, int C, size_t S, void *y);
void lp_h16_to_mx8(const void *x, int dt, int N, int C, size_t S, void *y);   /* dt 1 bf16, 2 fp16 */
void lp_h16_to_mx4(const void *x, int dt, int N, int C, size_t S, void *y);
void lp_mx8_to_f32(const void *x, int N, int C, size_t S, float *y);
void lp_mx4_to_f32(const void *x, int N, int C, size_t S, float *y);
/* network input rows from a uint8 CT window (src/nn_lp.h:164-165; src/lp_mx_cvt.cu:29-55) */
void lp_pred_input_mx(const uint8_t *ct, int W, float mean, float isd, const float *dyo, const float *dxo, int axis, int z0, int nz, void *y, int hd, int bits);
void lp_pred_input_mx8(const uint8_t *ct, int W, float mean, float isd, const float *dyo, const float *dxo, int axis, int z0, int nz, void *y, int hd);
/* the same into sample n of an N-sample input tensor (windows batched for one forward; the reference's entry is N 1, n 0: src/lp_mx_cvt.cu:42-55) */
void mi_pred_input_mx_n(const uint8_t *ct, int W, float mean, float isd, const float *dyo, const float *dxo, int axis, int z0, int nz, void *y, int hd, int bits, int N, int n);
/* the same for samples n0 .. n0 + nw - 1 from nw windows in one launch (ct, dyo, dxo: host arrays of nw device pointers) */
void mi_pred_input_mx_batch(const uint8_t *const *ct, int W, float mean, float isd, const float *const *dyo, const float *const *dxo, int axis, int z0, int nz, void *y, int hd, int bits,
                            int N, int n0, int nw);

/* ---- MX elementwise ops (src/nn_lp.h:134-137, :175-176) ---- */
void lp_gn_silu_apply_mx(const void *x, int xdt, shape5 s, int G, const float *gamma, const float *beta, const float *mean, const float *rstd, void *y, int ydt);
void lp_add_mx(void *y, const void *x, shape5 s, int dt, unsigned sr);   /* sr must be 0 (round to nearest) */
void lp_up2_fwd_mx(const void *x, int xdt, shape5 xs, void *y, int ydt, gnp_t gp);
void lp_up2_fwd_mx_blocks(const void *x, int xdt, shape5 xs, int b0, int nbk, void *y, int ydt);
int lp_gn_sums_mx(const void *x, int xdt, int N, int C, int G, size_t S, double *sums, size_t v0, size_t v1);
int lp_gn_sums_mx_n(const void *x, int xdt, int N, int C, int G, size_t S, double *sums, size_t v0, size_t v1, int n0, int cnt);

/* ---- 1x1x1 head (src/nn_lp.h:138-141; src/lp_mx_conv1.cu:370-445) ---- */
void lp_conv1_fwd_mx(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, float *y, gnp_t gp);
void lp_conv1_fwd_mx_h16(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, void *y, gnp_t gp);
void lp_conv1_fwd_mx_h16_r(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, void *y, gnp_t gp, size_t vb, size_t nv);
int lp_conv1_fwd_mx_r(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, float *y, gnp_t gp, size_t vb, size_t nv, size_t ly);

/* ---- error latch (src/nn_lp.h:172; src/lp_common.cuh:35-38): message of the first HIP error since the last call, else NULL ---- */
const char *lp_check(void);

/* ---- what the reference's lp_* units pull from its op layer, provided here so the library stands alone ----
   (the reference side: nn_malloc / nn_free / nn_zero / nn_h2d / nn_d2h / nn_sync, src/nn.h:34-48; gn_finalize_k, src/nn_elem.cu:5-11;
   nn_ws, src/nn_core.cu:751). In an integration these stay the reference's own. */
int mi_init(int device);                       /* selects the device, 0 on success; fails (non-zero) when no gfx950 device is present */
int mi_device_count(void);
void *mi_malloc(size_t bytes);                 /* device memory; aborts with a message when it cannot be had */
void mi_free(void *p);
void mi_zero(void *p, size_t bytes);
void mi_h2d(void *dst, const void *src, size_t bytes);
/* pinned host memory, a copy from it in stream order that the host does not wait for, and a fence: set in stream order, waited for by the host
   (before it rewrites the source of such a copy) */
void *mi_host_alloc(size_t bytes);
void mi_host_free(void *p);
void mi_h2d_async(void *dst, const void *src, size_t bytes);
void *mi_fence_new(void);
void mi_fence_set(void *f);
void mi_fence_wait(void *f);
void mi_fence_free(void *f);
void mi_d2h(void *dst, const void *src, size_t bytes);
void mi_d2d(void *dst, const void *src, size_t bytes);
void mi_d2d_rows(void *dst, size_t dpitch, const void *src, size_t spitch, size_t width, size_t rows);   /* rows runs of width bytes at the two pitches, in stream order */
void mi_sync(void);
void mi_ws_release(void);                      /* frees the per-device scratch (prepared weights, staged operands) */
/* GroupNorm finalize from sum slots: mean, rstd of NG = N * G groups of `len` elements each (src/nn_elem.cu:5-11) */
void mi_gn_finalize(const double *sums, int NG, size_t len, float eps, float *mean, float *rstd);
void mi_gn_sums_zero(double *sums, int nslots);          /* clear slots with a kernel (safe inside graph capture) */
void mi_gn_sums_get(const double *sums, int nslots, double *out);   /* slots -> doubles (device to device), src/gnacc.cuh:21-25 */
/* timing on the stream the kernels run on */
void *mi_event_create(void);
void mi_event_record(void *ev);
float mi_event_elapsed_ms(void *ev0, void *ev1);   /* synchronises on ev1 */
void mi_event_destroy(void *ev);
/* extension with no counterpart in the reference: the same conv with a fused epilogue affine + activation before the MX
   re-quantisation (frozen GroupNorm statistics folded into per-channel a, b): v = act(a[co] * (conv + bias) + b[co]);
   act 0 none, 1 SiLU, 2 GELU (erf), 3 ReLU. bits 8 / 4 selects the compute format. */
int mi_conv_fwd_fused(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf,
                      const float *ep_a, const float *ep_b, int act, gnp_t gp, double *osum, int Go, split_t sp);
/* extensions with no counterpart in the reference (whose down conv is 3x3x3 stride 2, src/lp_s2.cu:4-9, and whose upsample is trilinear,
   src/lp_mx_gn.cu:32-33): the 2x2x2 stride-2 conv (w [cout][cin][2][2][2], output dims halved: the input's must be even) and the 2x2x2 stride-2
   transposed conv (w [cin][cout][2][2][2], output dims doubled) with the operand rules of the 3x3x3 entries: x an MX tensor (xbf 3 / 4) with an
   optional GroupNorm + SiLU (gp), rows re-quantised to the compute format (bits 8 / 4) per voxel and 32 channels unless they are stored in it,
   weights scaled per (tap, output channel, 32 input channels), fp32 accumulation, bias, y an MX tensor (ybf 3 / 4) or fp32 / fp16 planes (0 / 2).
   No output statistics. 0 on success, -1 for arguments they do not take. */
int mi_conv_down2_fwd(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp);
int mi_convt_up2_fwd(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp);
/* extension with no counterpart in the reference (which zeroes the sum slots, runs the conv and finalizes in three launches,
   src/nn_bwd.cu:37-56, src/nn_elem.cu:5-17): the stride-1 conv with its output GroupNorm statistics finalized by the conv's own
   reduction. osum (2 N Go slots) need not be cleared: it is set to this conv's sums; omean / orstd (N Go floats) get
   mean and 1 / sqrt(var + eps), bit-identical to mi_gn_sums_zero + lp_conv_fwd_f8 / _f4 + mi_gn_finalize. */
int mi_conv_fwd_gn(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp,
                   double *osum, int Go, split_t sp, float eps, float *omean, float *orstd);
/* timing of the 3x3x3 conv kernel launches alone (benchmarks): on != 0 starts recording an event pair around every launch on the
   stream it runs on and clears the totals; read returns the total milliseconds so far and the number of launches (synchronises) */
void mi_kernel_timing(int on);
double mi_kernel_timing_read(long *launches);
/* launch i of the log kept since mi_kernel_timing(1), in launch order: its milliseconds, its algorithmic FLOPs (2 x 27 x Cin x Cout x output
   voxels, logical channels) and its kernel variant's name; returns the number of launches logged (synchronises) */
long mi_kernel_timing_launch(long i, float *ms, double *flops, char *name, size_t name_bytes);
/* No counterpart in the reference. lp_conv_fwd_f8 / lp_conv_fwd_f4 (bits 8 / 4) for callers that cannot allocate device memory: tight serving
   loops, harnesses that forbid hipMalloc. Same arguments, same kernels and bit-identical results, but every byte of scratch (prepared weights,
   re-staged operands, statistics partials, the constant page) comes from one fixed device array of mi_conv_static_scratch_bytes() = 64 MiB that
   each GPU the library runs on holds until the process ends; the call makes no hipMalloc / hipFree (split_t.wkey is ignored: weights are
   prepared per call). mi_init addresses the array on the device it selects and writes its 128-byte constant page (one synchronous copy); on a
   device nobody passed to mi_init the first call does that itself. Like every entry of this library it launches on the null stream, so it
   cannot be recorded into a HIP graph by stream capture. A call whose scratch could exceed the array prints what it needs and returns -1 with
   nothing launched (an input already in the compute format without GroupNorm, or a network input of few channels on the tap-packed kernels,
   needs only its weights: any size fits; with GroupNorm or another storage format the re-staged operand must fit: e.g. 128 channels at
   2 x 32^3). Calls on one GPU share the array: calls that overlap on a GPU (two host threads, two streams) race; nothing in it needs clearing
   between calls. */
int mi_conv_fwd_static(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp, double *osum, int Go, split_t sp);
size_t mi_conv_static_scratch_bytes(void);
long mi_alloc_count(void);                     /* device allocations made by this library so far (scratch growth, memo entries, mi_malloc): diagnostics */
/* Every fp32 bit pattern through the hardware encoder (bits 8: v_cvt_scalef32_pk_fp8_f32, 4: v_cvt_scalef32_pk_fp4_f32) at block exponent e
   against the software encoder of x 2^-e (the reference checks its conversion instruction the same way, src/lp_mxsw.cu:45-61). out[0]: inputs
   inside the domain the kernels use the instruction on (e4m3: |x 2^-e| <= 464 and not NaN; e2m1: not NaN), out[1]: mismatches among them (0
   expected), out[2] / out[3]: inputs outside it and their mismatches (those blocks take the software encoder). Synchronises. 0, or -1 for bad arguments */
int mi_cvt_sweep(int bits, int e, unsigned long long out[4]);
/* name of the conv kernel variant the last conv call on this thread launched (diagnostics / tests), "" if none */
const char *mi_last_kernel(void);
#ifdef __cplusplus
}
#endif
#endif
