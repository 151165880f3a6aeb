/* MX GEMM for the attention stage's linear layers and the MX-fp8 attention forward core, for AMD MI355X (gfx950).
 *
 * Drop-in for the corresponding declarations of the reference's src/attn.h: same names, argument order and meaning,
 * operand layouts and return codes. Device pointers everywhere; asynchronous on the null stream; device errors are
 * latched for lp_check() (include/mi_lp.h). Scratch (packed operands, quantised q / k / v) is per device and grows on
 * demand; mi_ws_release() frees it. */
#ifndef MI_ATTN_H
#define MI_ATTN_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define AT_HD 48            /* head dimension (src/attn.h:17) */
#define AT_DFM_MAXL 3       /* (src/attn.h:24; only sizes at_geom) */

/* geometry of an attention stage: nseq sequences of S tokens (src/attn.h:73-81). This build reads nseq and S; lens, pos, rays, dfx, dfr
   belong to paths that are not provided and must be null */
typedef struct at_rays at_rays;
typedef struct { int nseq, S, D, Hh, W; const int *lens; const float *pos; const at_rays *rays; const float *dfx[AT_DFM_MAXL]; const float *dfr; } at_geom;

/* replaces lp_mx_gemm (src/attn.h:186; src/lp_mxgemm.cu:295-297): C[M][N] = op(A) op(B) + beta C for row-major fp32 operands, A [M][K]
   (ta 0) or [K][M] (ta 1), B [K][N] (tb 0) or [N][K] (tb 1). Both operands are quantised along K to MX-fp4 (bits 4) or MX-fp8 (bits 8),
   one E8M0 scale per 32 K from the fmaxf maximum, round to nearest; block-scaled MFMA products, fp32 accumulation. Returns 0, or -1 for
   another bit width. */
int lp_mx_gemm(int bits, int ta, int tb, int M, int N, int K, const float *A, const float *B, float *Cm, float beta);
/* replaces lp_mx_gemm_ex (src/attn.h:189; src/lp_mxgemm.cu:281-294): the same with an epilogue, C = op(A) op(B) + bias[col] (null: none)
   + res[row][col] (null: none; row stride N; may alias C only with beta 0) + beta C. With few output tiles and a long K (no bias,
   no residual, beta 0 or 1) the K range is split over workgroups that add into C with floating-point atomics, as the reference does:
   the sum order of those calls is not fixed. */
int lp_mx_gemm_ex(int bits, int ta, int tb, int M, int N, int K, const float *A, const float *B, float *Cm, float beta, const float *bias, const float *res);

/* replaces at_fa8_fwd (src/attn.h:232; src/lp_attn8.cu:319-328): softmax(Q K^T / sqrt(48)) V per sequence and head on block-scaled
   e4m3 MFMA. qkvh: fp16 head-major q, k, v as at_fa_pack leaves them, [3][H][nseq S + 64][48], token i of sequence s in row s S + i.
   Q and K rows are quantised in two blocks (dims 0..31 and 32..47), V along the tokens in blocks of 32 per dim, P per query per
   32 keys inside each tile of 64 keys. o: fp32 [nseq S][C], head h in columns h 48 ... ; lse: fp32 [nseq][H][S], base-2 logarithm of the
   softmax denominator plus the maximum logit in base-2 units. C must equal 48 H. Returns 0, or -1 when scratch cannot be allocated. */
int at_fa8_fwd(const void *qkvh, float *o, float *lse, const at_geom *g, int H, int C);

#ifdef __cplusplus
}
#endif
#endif
