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
/* no counterpart in the reference: keep operand B's packed MX form across this thread's calls, keyed by pointer and shape (inference: B is a
   constant weight matrix); dropped by lp_wmemo_clear(). Off by default. */
void lp_mx_gemm_bmemo(int on);
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
/* (no counterpart: a tuning knob for tests) wavefronts per workgroup of at_fa8_fwd's kernel: 1 or 4, anything else = chosen from the launch
   size. With 4, a sequence's last 32-query tile, when it is the only one of its workgroup, is worked on by all four wavefronts (a range of the
   keys each, merged in wavefront order): the same probabilities and codes as with 1, their sums added in another order (~1e-7 relative) */
void at_fa8_waves(int nw);
/* (no counterpart: a knob for tests) 0: at_block_fwd writes the fp32 rows of its LayerNorms and its SwiGLU (at_ws.xn, .xn2, .gg) and the GEMMs
   pack them; 1: with e4m3 linears and C, F multiples of 64 those kernels write the GEMMs' packed operands themselves and the three fp32 buffers
   are left untouched (a forward never reads them again); 2 (default): also, for C <= 256, the up projection forms the SwiGLU in its epilogue and
   writes the down projection's packed operand, and at_ws.h is left untouched too. The block's output has the same bits in all three */
void at_fuse_pack(int on);

/* ---- the attention block around those two (forward, self-attention path; src/attn.h:26-81, src/nn_attn.cu) ---- */
#define AT_DFM_NLV (AT_DFM_MAXL + 1)
/* channels (H x 48), heads, SwiGLU hidden width, RoPE (0 none, 1 axial on the grid index), register tokens; the deformable fields must be 0
   (src/attn.h:33) */
typedef struct { int C, H, F, rope, nreg; float rope_base; int dK, dL, dC[AT_DFM_MAXL]; int dCo, dInit; } at_dims;
/* one block's parameters: offsets into the flat parameter array, weights [out][in] row major (src/attn.h:39, src/nn_attn.cu:460-480) */
typedef struct { size_t ln1g, ln1b, wqkv, bqkv, qg, kg, wo, bo, ln2g, ln2b, w1, b1, w2, b2, woa, boa, wvl[AT_DFM_MAXL], bvl[AT_DFM_MAXL]; } at_bp;
size_t at_block_nparams(const at_dims *d);
size_t at_block_layout(const at_dims *d, at_bp *bp, size_t off);   /* assigns offsets from off, returns the end */
/* scratch of one block over T tokens, field for field the reference's (src/attn.h:47-60); this build carves and uses the forward tensors
   xn, qkv, o, x1, xn2, h, gg, m1, r1, m2, r2, rq, rk, lse, qkvh, amx and leaves the others null */
typedef struct {
    float *xn, *qkv, *qkn, *o, *x1, *xn2, *h, *gg, *m1, *r1, *m2, *r2, *rq, *rk, *lse, *dv;
    float *bA, *bB, *bC, *dx1;
    float *qkvh, *doh, *amx;
    float *qkvr, *orr, *dor, *dqr, *dqr2;
    float *vl[AT_DFM_NLV], *oa, *aw, *dvl[AT_DFM_NLV], *doa;
    int kept;
    int vr; float *v1, *own, *dv1; const float *lam; float *glam;
} at_ws;
size_t at_ws_bytes(const at_dims *d, long T);                       /* replaces src/nn_attn.cu:529 (forward tensors only here) */
void at_ws_carve(at_ws *w, const at_dims *d, long T, void *base);   /* replaces src/nn_attn.cu:530 */
/* the linear layers' precision (src/attn.h:194-195, src/nn_attn.cu:97-135): 4 / 8 = lp_mx_gemm_ex; this build has no fp32 GEMM, 0 is refused */
void at_set_mx(int bits);
int at_get_mx(void);
int at_gemm_ex(int ta, int tb, int M, int N, int K, const float *A, const float *B, float *Cm, float beta, const float *bias, const float *res);
/* replaces at_ln_fwd (src/attn.h:241, src/nn_attn.cu:150-168): LayerNorm over C per row, eps 1e-5, affine g / b; mean / rstd [T] */
void at_ln_fwd(const float *x, const float *g, const float *b, float *y, float *mean, float *rstd, long T, int C);
/* replaces at_glu_fwd (src/attn.h:248, src/nn_attn.cu:438-455): h [T][2F] = [a | b] -> gg [T][F] = silu(a) b */
void at_glu_fwd(const float *h, float *gg, long T, int F);
/* replaces at_fa_pack (src/attn.h:203, src/nn_attn_tc.cu:99-136, :371-378): qkv fp32 [T][3C] -> fp16 head-major q, k, v [3][H][T + 64][48];
   q and k RMS-normalised over the head dims (eps 1e-6) times the gains qg / kg [H][48], then axial rotary pairs on grid tokens (rope 1;
   g->pos must be null); rq / rk [T][H] the normalisers, amx[1] = max |v| (amx: 4 floats, zeroed here); rows past T zero */
void at_fa_pack(const float *qkv, const float *qg, const float *kg, void *qkvh, float *rq, float *rk, float *amx, const at_geom *g, int nreg, int C, int rope, float base);
/* replace at_cs_to_tok / at_tok_to_cs (src/nn_attn.cu:748-759, :802-803): channel-major planes [n][C][Sg] <-> token rows [n][nreg + Sg][C]
   with the learned register rows reg [nreg][C] prepended (dropped on the way back) */
void at_cs_to_tok(const float *x, float *t, const float *reg, int n, int C, long Sg, int nreg);
/* replaces at_peg_fwd (src/attn.h:141-144, src/nn_attn.cu:688-705, :738-740): conv positional encoding, y = x + b + depthwise 3^3 conv of x on the
   grid tokens of each sequence (zero padding), register rows copied; w [C][27], b [C]; x and y separate buffers, g->S = nreg + g->D g->Hh g->W */
void at_peg_fwd(const float *x, float *y, const float *w, const float *b, const at_geom *g, int nreg, int C);
void at_tok_to_cs(const float *t, float *x, int n, int C, long Sg, int nreg);
/* replaces at_block_fwd (src/attn.h:..., src/nn_attn.cu:587-633) for self-attention blocks on the MX-fp8 core with MX linears:
   y = x1 + W2 swiglu(W1 LN2(x1)), x1 = x + Wo attention(pack(Wqkv LN1(x))). P: the parameter array, bp: the block's offsets; x, y fp32
   [T][C] (T = g->nseq g->S); 0, or -1 for a configuration this build does not run (deformable, rays, fp32 linears). w->vr 1 keeps the block's V rows in w->v1; 2 replaces V by
   v + w->lam[head] (w->v1 - v) and keeps the own rows in w->own when given (the value residual, src/nn_attn.cu:535-542, :609-610) */
int at_block_fwd(const at_dims *d, const float *P, const at_bp *bp, const float *x, float *y, const at_geom *g, at_ws *w);

#ifdef __cplusplus
}
#endif
#endif
