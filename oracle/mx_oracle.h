/* CPU oracle of the MX (fp8 e4m3 / fp4 e2m1, E8M0 block scale) 3-D U-Net forward arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain-C restatement of the reference's algorithm, used as the checker by the
 * tests, by the smoke test and as the timed "cpu_baseline" leg of the benchmark. Nothing in the shipped GPU path may
 * call it. Every function names the reference lines it follows (paths relative to the reference checkout).
 *
 * Pinning status (what holds each function to the reference without running the reference):
 *   orc_enc_e4m3 / orc_enc_e2m1   pinned: == independent nearest-grid-point search (orc_ref_*) over all 2^32 floats
 *   orc_mx_exp                    pinned: closed form "smallest e with amax * fl(1/qmax) <= 2^e", cross-checked
 *                                 against the ceil(log2(amax/qmax)) form of tests/test_mx4.c:51
 *   orc_store_row / orc_f32_to_mx pinned: decoded output == host_mx4 / q_rn style quantiser written from the format
 *   orc_conv3 (copy staging)      pinned: exact-operand construction (tests/test_mx4_wide.c:81-98) == fp64 direct conv
 *   orc_conv3 epilogue requant    pinned: == block quantiser of the exact conv (cmp_mx, tests/test_mx4_wide.c:252-265)
 *   GroupNorm sums / finalize     pinned: independent fp64 statistics; constant group => rstd = 1/sqrt(eps)
 *   trilinear staging, up2        pinned: closed form 0.75/0.25 separable weights with edge clamp, grid data exact
 *   1x1x1 head                    pinned: plain dot product (GEMM special case)
 *   orc_mx_gemm                   pinned: == fp64 product of operands quantised by an independent numpy block quantiser
 *                                 (tests/test_attn.c:375-396), all transpose flags, ragged M / N / K; exact-operand case == integer product
 *   orc_fa8_fwd                   pinned: closed forms (uniform logits -> mean of the quantised V and lse = log2 S; one dominant key ->
 *                                 that key's quantised V row, also when the maximum moves between key tiles; keys past S never
 *                                 contribute) and the reference's own gate, rel. L2 < 0.1 against exact fp64 attention
 *                                 (tests/test_attn.c:445-446)
 *   orc_ln_fwd, orc_glu_fwd,      pinned: textbook formulas in numpy fp64 (LayerNorm eps 1e-5, SiLU(a) b, RMS-norm eps 1e-6 times gains, rotary
 *   orc_fa_pack, orc_cs_to_tok    pairs = complex multiplication by exp(i pos base^(-f/8)), norm-preserving), fp16 rounding by numpy
 *   orc_block_fwd                 pinned: the reference's gate (tests/test_attn.c:398-424): rel. L2 against the exact fp64 block
 *   orc_peg_fwd                   pinned: scipy's correlate (zero padding) per channel in fp64, plus bias and the token itself; register rows
 *                                 are copies; one tap set gives the shifted tensor (tests/test_oracle_block.py)
 *   orc_block_fwd_vr              the value residual (src/nn_attn.cu:535-542, :609-610): pinned by the exact fp64 block with V mixed from the
 *                                 definition, within the same gate, and by the special cases lam 0 (the plain block, bit for bit) and
 *                                 lam 1 on one head (that head's V rows replaced by another projection's, the other heads untouched)
 *   orc_pred_place                pinned: box intersection by brute force over all voxels; 255 sigmoid rounded to nearest in fp64
 *   orc_feather_blend             pinned: the reference's own checks (tests/test_predict_feather.c:95-121): core and first-window voxels
 *                                 equal the window's own prediction, a z-shell voxel is u(j) own + (1 - u(j)) lower within 1; constant
 *                                 fields are fixed points; an absent neighbour renormalises
 *   SiLU in GN staging            PARITY UNPINNED to the bit: the reference evaluates tanh with NVIDIA's
 *                                 tanh.approx.f32 (src/lp_common.cuh:469-473), not reproducible off that hardware;
 *                                 checked to floor/ceil code neighbours as tests/test_mx4_wide.c:165-175 does
 *   orc_conv3 with stem_tile      the tap-packed small-channel conv (src/lp_f8fwd.cuh:153-400): exact operands equal the fp64
 *                                 convolution for the three channel paddings and all input types; one large value coarsens exactly the
 *                                 output voxels of the 2 x 8 x 16 tiles whose 4 x 10 x 18 halo holds it; a one-tile volume returns the
 *                                 tensor under one scale (tests/test_oracle_stem.py)
 *   ... with stem_tile 2          the 9 .. 16 channel form with one scale per staged row (src/lp_f8fwd.cuh:447-563): exact operands equal the
 *                                 fp64 convolution; one large value coarsens exactly the outputs of its x tile that read its (z, y) line
 *   slab-local statistics         pinned (orc_gn_row and its use in orc_conv3, orc_gn_silu_apply_mx, orc_conv1_mx; src/lp_slab.cuh:7-12): rows
 *                                 against slab ranges written from the definition; a slab's planes cut out of the tensor and run through
 *                                 the per-sample function with that slab's rows give the same bytes; conv output planes away from a slab
 *                                 boundary equal the per-sample conv's, those at it equal neither (tests/test_oracle_slab_gn.py)
 *   orc_h16_to_mx                 pinned: numpy float16 values through the independent block quantiser (tests/test_oracle_elem.py)
 *   orc_pred_input_mx             pinned: a numpy statement of src/lp_mx_cvt.cu:24-41 through the independent block quantiser, all axes, the
 *                                 16-bit roundings, signed zeros (tests/test_oracle_elem.py). PARITY UNPINNED against the reference binary for
 *                                 channels 2 and 3: it is built with -use_fast_math, whose approximate division and square root are not
 *                                 defined to the bit; this restatement and the device use IEEE operations
 *   orc_gn_silu_apply_mx          pinned: fp64 SiLU of the fp32 affine through the independent quantiser with the reference's neighbour-code
 *                                 acceptance, and closed forms (tests/test_oracle_elem.py); its SiLU bits as above
 *   binary16 upsample blend       pinned: orc_h16_fma == one rounding of the exact rational result; the staged operand == src/lp_common.cuh:674-712
 *                                 restated in exact rationals rounded per step; grid data == the fp64 interpolation (tests/test_oracle_elem.py)
 *   orc_conv2                     pinned: fp64 closed forms on exact operands, orc_conv3 at stride 2 with the taps embedded in a 3x3x3 kernel,
 *                                 adjointness of the two ops (tests/test_oracle_conv2.py). No counterpart in the reference.
 *   2-D fp4 weight scales,        pinned: the numpy block quantiser on whole tiles; the reference's invariant that per-channel blocks re-quantise
 *   orc_fakeq_w4                  the fake-quantised values exactly (tests/test_oracle_w4_2d.py)
 */
#ifndef MX_ORACLE_H
#define MX_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar format arithmetic ---- */
int orc_mx_bw(int C);                                 /* src/lp_common.cuh:132 */
int orc_mx_nb(int C);                                 /* src/lp_common.cuh:133 */
size_t orc_mx_bytes(int bits, int N, int C, size_t S);/* src/lp_mx_cvt.cu:6-7 */
int orc_mx_exp(float amax, float inv_qmax);           /* src/lp_common.cuh:492-500 */
float orc_exp2i(int e);                               /* src/lp_common.cuh:501 */
float orc_mx_scale(unsigned sbyte);                   /* src/lp_common.cuh:186 */
unsigned orc_enc_e4m3(float x);                       /* src/mx_sw.cuh:14-36 (semantics), own formulation */
unsigned orc_enc_e2m1(float x);                       /* src/mx_sw.cuh:37-56 */
float orc_dec_e4m3(unsigned b);                       /* src/mx_sw.cuh:78-83 */
float orc_dec_e2m1(unsigned n);                       /* src/mx_sw.cuh:84-87 */
unsigned orc_ref_e4m3(float x);                       /* nearest-grid search, the pin of orc_enc_e4m3 */
unsigned orc_ref_e2m1(float x);
/* sweep [first, first + count) of fp32 bit patterns: number of inputs where enc != ref (either format); first bad in *bad */
uint64_t orc_enc_sweep(uint32_t first, uint64_t count, uint32_t stride, uint32_t *bad);

/* one block row: v[bw] -> codes (bw bytes fp8 / bw/2 bytes fp4) + scale byte. nanprop: NaN-propagating amax
   (src/lp_mxops.cuh:45-65) else fmaxf amax (src/lp_f8fwd.cuh:91) */
uint8_t orc_store_row(int bits, const float *v, int bw, uint8_t *codes, int nanprop);
void orc_load_row(int bits, const uint8_t *codes, uint8_t sbyte, int bw, float *v);   /* src/lp_common.cuh:189-232 */

/* ---- tensor converters (src/lp_mx_cvt.cu:9-19, 429-447) ---- */
void orc_f32_to_mx(int bits, const float *x, int N, int C, size_t S, uint8_t *y);
void orc_h16_to_mx(int bits, const uint16_t *x, int N, int C, size_t S, uint8_t *y);   /* fp16 source */
void orc_mx_to_f32(int bits, const uint8_t *x, int N, int C, size_t S, float *y);
/* network input (src/lp_mx_cvt.cu:29-41): hd 2 = fp16 rounding, 0 none */
void orc_pred_input_mx(int bits, const uint8_t *ct, int W, float mean, float isd, const float *dyo, const float *dxo, int axis,
                       int z0, int nz, uint8_t *y, int hd);

/* ---- weights (src/lp_f8fwd.cu:54-71, src/lp_f4fwd.cu:53-66): w[co][ci][27] -> decoded block values wv[t][co][Cip] (code
   values, not yet scaled) and scale bytes ws[t][co][Cip/32]; Cip = padded input channels of the (split) input ---- */
void orc_prep_w(int bits, const float *w, int Co, int Ci, int Cx, int CxP, int Cip, float *wv, uint8_t *ws, uint8_t *wcodes);

/* ---- GroupNorm descriptor of an input segment (src/nn_lp.h:15-18). ns > 0, slab-local statistics: mean / rstd hold one row per (sample,
   z-slab), [n][ns][G]; plane z reads row n * ns + clamp((z + zo) / zs, 0, ns - 1) (src/lp_slab.cuh:7-12); zhw = voxels per plane ---- */
typedef struct { const float *gamma, *beta, *mean, *rstd; int G; int zs, zo, ns, zhw; } orc_gn_t;
int orc_gn_row(const orc_gn_t *g, int n, int z);      /* the statistics row of sample n at plane z */

typedef struct {
    /* input */
    const void *x; int xdt;            /* 0 fp32 planes, 2 fp16 planes, 3 MX-fp8, 4 MX-fp4 */
    int N, Ci, D, H, W;                /* output-resolution input dims for stride 1; the input's dims for stride 2 */
    const void *x2; int c_split;       /* channels >= c_split come from x2 (same dtype) */
    int up;                            /* the x segment is stored at D/2 x H/2 x W/2 and read trilinearly upsampled: 1 the entry's own blend (fp32 chain
                                          for e4m3 compute, binary16 for e2m1 compute), 2 binary16, 3 fp32 */
    orc_gn_t gp, gp2;                  /* GN + SiLU of x (or of all channels when gp2.G == 0) and of x2 */
    /* weights */
    const float *w, *b; int Co; int stride;   /* 3x3x3, pad 1, stride 1 or 2 */
    int cbits;                         /* compute format: 8 (e4m3) or 4 (e2m1) */
    /* output */
    void *y; int ydt;                  /* 0 fp32 planes, 2 fp16 planes, 3 MX-fp8, 4 MX-fp4 */
    double *osum; int Go; int stored_stats;   /* plain doubles [N][Go][2] (sum, sum of squares), accumulated */
    int acc64;                         /* 1: accumulate in fp64 (exact-operand checks); 2: fp32 with every add rounded toward zero, 3: an aligning, truncating block adder (drift studies) */
    int fused_act; const float *ep_a, *ep_b;   /* extension: epilogue affine + activation (1 SiLU, 2 GELU, 3 ReLU) before requant */
    int z0, z1;                        /* output z planes [z0, z1) only (z1 0: all): the bounded CPU-baseline slab */
    int stem_tile;                     /* 1: one activation scale per staged 4x10x18 tile (Ci <= 8 tap-packed stem); 2: 9 .. 16 channels, two taps per K
                                          block, one activation scale per staged row of 18 positions */
} orc_conv_t;
/* 3x3x3 forward conv with MX operands (src/lp_f8fwd.cuh:19-151, src/lp_common.cuh:1465-1597, src/lp_s2.cu:4-9) */
int orc_conv3(const orc_conv_t *c);
/* 2x2x2 stride-2 conv (up 0: w [Co][Ci][2][2][2], output dims halved) or transposed conv (up 1: w [Ci][Co][2][2][2], output dims doubled) with
   MX operands: c->x an MX tensor of c->D x c->H x c->W, optional c->gp; stride, x2, up, osum, z0 / z1 and stem_tile of c are not used */
int orc_conv2(const orc_conv_t *c, int up);
/* 2-D fp4 weight scales of the stride-1 e2m1 preps (lp_set_w4_2d, src/lp_f4fwd.cu:67-83) and the in-place fake quantisation (src/lp_mx_cvt.cu:369-395) */
void orc_set_w4_2d(int on);
void orc_fakeq_w4(float *w, int Co, int Ci, int T, int Bo, int Bi);
/* staged (quantised) operand of a conv's input only: values = decoded code * scale per (n, padded channel, voxel) */
int orc_conv3_staged(const orc_conv_t *c, float *staged);

/* GroupNorm finalize (src/nn_elem.cu:5-11) */
void orc_gn_finalize(const double *sums, int NG, size_t len, float eps, float *mean, float *rstd);
/* (sum, sumsq) per (n, group) of a stored MX tensor over voxels [v0, v1) (src/lp_mx_gnsums.cu:8-80) */
void orc_gn_sums_mx(int bits, const uint8_t *x, int N, int C, int G, size_t S, double *sums, size_t v0, size_t v1);
/* y = MX(silu(gn(x))) (src/lp_mx_gn.cu:5-21; exp form v / (1 + exp(-v))) */
void orc_gn_silu_apply_mx(const void *x, int xdt, int N, int C, size_t S, orc_gn_t gp, uint8_t *y, int ybits);
/* trilinear 2x upsample of an MX tensor, optional GN + SiLU of the coarse values (src/lp_mx_gn.cu:34-73) */
void orc_up2_mx(int xbits, const uint8_t *x, int N, int C, int D, int H, int W, orc_gn_t gp, uint8_t *y, int ybits);
/* 1x1x1 head (src/lp_mx_conv1.cu:5-21): y[n][co][v] fp32 */
void orc_conv1_mx(int xbits, const uint8_t *x, int N, int Ci, size_t S, const float *w, const float *b, int Co, orc_gn_t gp, float *y);
/* GN affine + SiLU of the conv staging (src/lp_common.cuh:474-482): u = fma(v, a, b), u sigmoid(u) correctly rounded */
/* MX GEMM of row-major fp32 operands quantised along K (src/lp_mxgemm.cu:266-297); 0, or -1 for unsupported bits */
int orc_mx_gemm(int bits, int ta, int tb, int M, int N, int K, const float *A, const float *B, float *C, float beta, const float *bias, const float *res);
/* MX-fp8 attention forward on the fp16 head-major pack (src/lp_attn8.cu:124-180, :319-328); head dim 48 */
void orc_fa8_fwd(const uint16_t *qkvh, float *o, float *lse, int nseq, int S, int H, int C);
/* the attention block's elementwise pieces and its forward composed from them, orc_mx_gemm and orc_fa8_fwd (src/nn_attn.cu:150-167, :438-446,
   :460-480, :587-633, :748-759; src/nn_attn_tc.cu:99-136) */
void orc_ln_fwd(const float *x, const float *g, const float *b, float *y, float *mean, float *rstd, long T, int C);
void orc_glu_fwd(const float *h, float *gg, long T, int F);
void orc_cs_to_tok(const float *x, float *t, const float *reg, int n, int C, long Sg, int nreg);
void orc_tok_to_cs(const float *t, float *x, int n, int C, long Sg, int nreg);
void orc_fa_pack(const float *qkv, const float *qg, const float *kg, uint16_t *qkvh, float *rq, float *rk, float *amx, int nseq, int S, int Hh, int W, int nreg, int C, int rope, float base);
size_t orc_block_layout(int C, int F, size_t off, size_t *o);
int orc_block_fwd(int bits, int C, int H, int F, int rope, int nreg, float rope_base, const float *P, const float *x, float *y, int nseq, int S, int Hh, int W);
void orc_peg_fwd(const float *x, float *y, const float *w, const float *b, int nseq, int S, int D, int Hh, int W, int nreg, int C);
int orc_block_fwd_vr(int bits, int C, int H, int F, int rope, int nreg, float rope_base, const float *P, const float *x, float *y, int nseq, int S, int Hh, int W, int vr, float *v1, const float *lam);
/* sliding-window prediction: sigmoid -> uint8 placement (src/nn_elem.cu:1105-1125) and the one-sided sin^2 feather blend of window borders
   (src/predict.c:282-333) */
void orc_pred_place(const float *lg, const uint8_t *ct, int D, int W, int hz, int halo, int oz, int oy, int ox, int ez, int ey, int ex, int shard, int iso, uint8_t *dsh);
void orc_feather_blend(const uint8_t *E, const uint8_t *present, int S, int B, const int64_t nss[3], const int64_t bn[3], uint8_t *out);
float orc_act_ab(float v, float a, float b);
void orc_set_align_bits(int b);         /* drift studies: width of the acc64 == 3 adder (default 24) */
void orc_set_act_mode(int m);          /* drift studies: 1 evaluates the activation by a fast fp32 path (a few ulp off), 0 (default) exactly */
uint16_t orc_f32_to_h16(float f);
float orc_h16_to_f32(uint16_t h);
uint16_t orc_h16_fma(uint16_t a, uint16_t b, uint16_t c);   /* binary16 fused multiply-add, one rounding */
int orc_threads(void);
#ifdef __cplusplus
}
#endif
#endif
