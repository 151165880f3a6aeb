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

/* geometry of an attention stage: nseq sequences of S tokens on a D x Hh x W grid after the registers (src/attn.h:73-81). lens: per sequence
   the number of keys that count (at_fa_fwd; null: S); pos: per token its rotary coordinates [nseq S][3] (at_dims.rope 2; null: the grid
   indices); rays: radial attention (below; with it nreg must be 0). dfx, dfr belong to deformable attention, which is not provided: null */
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

/* ---- radial attention and scroll coordinates (src/attn.h:83-128, src/nn_attn_ray.cu) ----
   Each sample's grid (D x Hh x W tokens, no registers) has a scroll axis along grid dim ad (0 D, 1 Hh, 2 W) with a centre (cu, cv) per plane k
   along ad (u, v: the other two dims in z, y, x order). Per plane Nt rays leave the centre at angles that cover the plane's rectangle (all
   angles when the centre lies inside it), each sampled at unit spacing from where it enters the rectangle to where it leaves (centred on the
   chord, at most Nr samples). A sample's value is the bilinear interpolation (edge-clamped) of the four grid tokens around it. A block with
   rays gathers q / k / v onto the samples, runs QK-norm, RoPE and the attention per ray (keys past the ray's length masked) and scatters the
   result back normalised: o[v] = sum_s w(s, v) o_s / sum_s w(s, v) (0 where no sample touches v). Without an axis the rays are the grid rows
   along v. Every sample has Q = Pmax Nt rays (Pmax = max(D, Hh, W); unused ones are zero-weight dummies of length 1) of Nr slots. */
#define AT_RAY_F 8   /* ray record (src/attn.h:92): u0, v0 (plane coordinates of sample 0), du, dv (unit step), r0 (radius of sample 0), arc (theta x rc), len, k */
struct at_rays {     /* (src/attn.h:93-100) */
    int n, Q, Nt, Nr, D, Hh, W;
    const int *ad;       /* device [n]: the axis dim per sample */
    const float *ray;    /* device [n][Q][AT_RAY_F] */
    const int *lens;     /* device [n Q]: max(1, len) */
    const float *pos;    /* device [n Q Nr][3]: (r, arc, k) of every ray slot (written by at_rays_setup) */
    const float *wsum;   /* device [n D Hh W]: 1 / the summed stencil weights per grid token, 0 where uncovered (written by at_rays_setup) */
};
/* per sample axis record at the grid's resolution (src/attn.h:101-102): ad, valid, then per plane along ad: cu, cv (grid voxels) */
#define AT_AXR(pmax) (2 + 2 * (pmax))
/* replaces at_rays_dims (src/attn.h:104; src/nn_attn_ray.cu:12-20): the fixed sizes for a grid; mult = rays per plane / Pmax (the reference's
   driver uses 2) */
void at_rays_dims(int D, int Hh, int W, float mult, int *Q, int *Nt, int *Nr);
/* replaces at_rays_plan (src/attn.h:107; src/nn_attn_ray.cu:43-104). Host: from n axis records the ray table ray_h [n][Q][AT_RAY_F], lens_h
   [n Q], ad_h [n] and the scroll frame cen_h [n][Pmax][4] = (cu, cv, rc, phi_m) per plane (rc -1 in every plane of a sample without an axis).
   Reads the reference's environment knob UFSM_SCROLL_PE_V2 once (one reference angle and radius per sample) */
void at_rays_plan(int n, int D, int Hh, int W, float mult, const float *axr, float *ray_h, int *lens_h, int *ad_h, float *cen_h);
/* replaces at_rays_setup (src/attn.h:109; src/nn_attn_ray.cu:137-144). Device: R's pos and wsum (into its buffers) from its ray table */
void at_rays_setup(const at_rays *R);
/* replace at_ray_gather / at_ray_scatter (src/attn.h:111-113; src/nn_attn_ray.cu:145-173): grid rows x [n D Hh W][Cc] -> ray rows y [Tr][Cc]
   (norm: each corner's weight x wsum of its token, the adjoint of the normalised scatter), and ray rows -> grid rows (zeroed first; x wsum with
   norm). Cc a multiple of 4, rows 16-byte aligned. The scatter (and at_rays_setup's weight sums) walk, per grid token, the list of ray samples
   that touch it in (ray, sample) order: the same bits on every run, where the reference's floating-point atomics leave the last bits to
   the order of arrival; the lists (5 Nt pairs per token) are library scratch that grows on demand */
void at_ray_gather(const at_rays *R, const float *x, float *y, int Cc, int norm);
void at_ray_scatter(const at_rays *R, const float *y, float *x, int Cc, int norm);
/* replaces at_scroll_pos (src/attn.h:116; src/nn_attn_ray.cu:174-192): the scroll coordinates of the grid tokens for full attention with
   at_dims.rope 2: pos [n][nreg + D Hh W][3] = (r, arc, k) around the axis (registers 0); without an axis (v, u, k): the grid indices.
   ad: device [n]; cen: device [n][Pmax][4] as at_rays_plan writes it */
void at_scroll_pos(int n, int nreg, int D, int Hh, int W, const int *ad, const float *cen, float *pos);
/* replaces at_fa_fwd (src/attn.h:207; src/nn_attn_tc.cu:139-197, :391-397): softmax(Q K^T / sqrt(48)) V per sequence and head from the fp16
   head-major q / k / v of at_fa_pack, fp32 sums, probabilities rounded to fp16 before they meet V; g->lens (device, per sequence; null: S):
   keys past the sequence's length are masked, a length of 0 gives zero output. o [nseq S][C] fp32, lse [nseq][H][S] (base 2). The core of
   radial attention, whose sequences are rays of 20 - 50 slots */
void at_fa_fwd(const void *qkvh, float *o, float *lse, const at_geom *g, int H, int C);

/* ---- the attention block around those two (forward, self-attention path; src/attn.h:26-81, src/nn_attn.cu) ---- */
#define AT_DFM_NLV (AT_DFM_MAXL + 1)
/* channels (H x 48), heads, SwiGLU hidden width, RoPE (0 none, 1 axial on the grid index, 2 on the scroll coordinates at_geom.pos / at_rays.pos),
   register tokens; the deformable fields must be 0 (src/attn.h:26-33) */
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
/* replace at_ws_bytes_r / at_ws_carve_r (src/attn.h:67-69): the same for radial attention with Tr ray tokens (at_rays: n Q Nr): the attention's
   tensors (qkvh, rq, rk, lse) are sized by Tr and the ray rows qkvr [Tr][3 C], orr [Tr][C] are added; Tr 0 = the two above */
size_t at_ws_bytes_r(const at_dims *d, long T, long Tr);
void at_ws_carve_r(at_ws *w, const at_dims *d, long T, long Tr, void *base);
/* the linear layers' precision (src/attn.h:194-195, src/nn_attn.cu:97-135): 4 / 8 = lp_mx_gemm_ex; this build has no fp32 GEMM, 0 is refused */
void at_set_mx(int bits);
int at_get_mx(void);
int at_gemm_ex(int ta, int tb, int M, int N, int K, const float *A, const float *B, float *Cm, float beta, const float *bias, const float *res);
/* replaces at_ln_fwd (src/attn.h:241, src/nn_attn.cu:150-168): LayerNorm over C per row, eps 1e-5, affine g / b; mean / rstd [T] */
void at_ln_fwd(const float *x, const float *g, const float *b, float *y, float *mean, float *rstd, long T, int C);
/* replaces at_glu_fwd (src/attn.h:248, src/nn_attn.cu:438-455): h [T][2F] = [a | b] -> gg [T][F] = silu(a) b */
void at_glu_fwd(const float *h, float *gg, long T, int F);
/* replaces at_fa_pack (src/attn.h:203, src/nn_attn_tc.cu:99-136, :371-378): qkv fp32 [T][3C] -> fp16 head-major q, k, v [3][H][T + 64][48];
   q and k RMS-normalised over the head dims (eps 1e-6) times the gains qg / kg [H][48], then rotary pairs on grid tokens (rope != 0: 16 head
   dims per coordinate; the coordinates are g->pos [T][3] when given, else the grid indices z, y, x of the token); rq / rk [T][H] the normalisers, amx[1] = max |v| (amx: 4 floats, zeroed here); rows past T zero */
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
   [T][C] (T = g->nseq g->S); 0, or -1 for a configuration this build does not run (deformable attention, fp32 linears). With g->rays
   (radial attention; d->nreg must be 0, w carved by at_ws_carve_r) q / k / v are gathered onto the ray samples, packed with the rays'
   positions (d->rope 2) or slot indices (1), attended per ray by at_fa_fwd (fp16 q / k / v: ray lengths, src/nn_attn.cu:583-586) and
   scattered back normalised (src/nn_attn.cu:611-624). w->vr 1 keeps the block's V rows in w->v1; 2 replaces V by
   v + w->lam[head] (w->v1 - v) and keeps the own rows in w->own when given (the value residual, src/nn_attn.cu:535-542, :609-610) */
int at_block_fwd(const at_dims *d, const float *P, const at_bp *bp, const float *x, float *y, const at_geom *g, at_ws *w);

#ifdef __cplusplus
}
#endif
#endif
