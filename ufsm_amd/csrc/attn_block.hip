// The attention block around the MX GEMM and the MX-fp8 attention core: LayerNorm, QK-norm + gains + RoPE pack to fp16, SwiGLU, token
// layout, parameter layout, scratch carving and the block forward (src/nn_attn.cu:150-168, :438-455, :460-530, :587-633, :748-759 and
// src/nn_attn_tc.cu:99-136 of the reference). The elementwise kernels are HBM-bound row kernels.
#include <hip/hip_fp16.h>
#include "mx_dev.hpp"
#include "../../include/mi_attn.h"
#include "attn_ray.hpp"

#define HD AT_HD
#define FT 64

// ---- LayerNorm (src/nn_attn.cu:150-168): y = (x - mean) rstd g + b, mean and biased variance of the row, eps 1e-5 ----
// One wavefront per token row, the row resident in registers: lane l holds the float4 chunks l, l + 64, ... (NV of them), so the row is read
// from HBM once (16-byte accesses, a wavefront 1 KiB contiguous), the mean and the centred sum of squares are two butterfly reductions over
// register values, and the result leaves as 16-byte stores.
// PK: the normalised row does not leave as fp32 values but as the MX-fp8 operand rows of the GEMM that reads it (mx_pack_k<8, 0>'s layout and
// arithmetic: per 32 channels the fmaxf maximum, one E8M0 byte, e4m3 codes): a block of 32 channels is the float4 chunks of eight neighbouring
// lanes, whose maxima meet through three lane exchanges. C a multiple of 64
template <int NV, bool PK = false>
__global__ void __launch_bounds__(256) ln_row_k(const float4 *__restrict__ x, const float *__restrict__ g, const float *__restrict__ b, float4 *__restrict__ y,
                                                float *__restrict__ mean, float *__restrict__ rstd, long long T, int C4, uint8_t *__restrict__ pq = nullptr, uint8_t *__restrict__ ps = nullptr) {
    const long long row = blockIdx.x * 4ll + (threadIdx.x >> 6); const int lane = threadIdx.x & 63;
    if (row >= T) return;
    const float4 *xr = x + row * C4;
    float4 v[NV];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int c = lane + 64 * i;
        v[i] = c < C4 ? xr[c] : make_float4(0.f, 0.f, 0.f, 0.f);
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
#pragma unroll
    for (int o = 32; o; o >>= 1) s += __shfl_xor(s, o);
    const float C = (float)(4 * C4), m = s / C;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        if (lane + 64 * i < C4) {
            v[i].x -= m; v[i].y -= m; v[i].z -= m; v[i].w -= m;
            q += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
        }
    }
#pragma unroll
    for (int o = 32; o; o >>= 1) q += __shfl_xor(q, o);
    const float r = 1.f / sqrtf(q / C + 1e-5f);
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int c = lane + 64 * i;
        if (c < C4) {
            // (gains and shifts sit at arbitrary offsets of the flat parameter vector: dword loads)
            const float4 gg = make_float4(g[4 * c], g[4 * c + 1], g[4 * c + 2], g[4 * c + 3]), bb = make_float4(b[4 * c], b[4 * c + 1], b[4 * c + 2], b[4 * c + 3]);
            const float4 o = make_float4(fmaf(v[i].x * r, gg.x, bb.x), fmaf(v[i].y * r, gg.y, bb.y), fmaf(v[i].z * r, gg.z, bb.z), fmaf(v[i].w * r, gg.w, bb.w));
            if constexpr (!PK) y[row * C4 + c] = o; else v[i] = o;
        }
    }
    if constexpr (PK) {
        // (C4 is a multiple of 16, so the lanes of a group of eight hold chunks together or not at all, and the exchanges below run on every lane)
#pragma unroll
        for (int i = 0; i < NV; i++) {
            const int c = lane + 64 * i;
            const bool on = c < C4;
            float am = on ? fmaxf(fmaxf(fabsf(v[i].x), fabsf(v[i].y)), fmaxf(fabsf(v[i].z), fabsf(v[i].w))) : 0.f;       // (fmaxf drops NaN, as the pack kernel's)
            unsigned au = __float_as_uint(am);                                 // (non-negative, never NaN: orders as its bits)
            au = max(au, d_quad_xor_u<1>(au)); au = max(au, d_quad_xor_u<2>(au));
            au = max(au, d_oct_mirror_u(au));
            const int e = d_mx_exp(__uint_as_float(au), MI_INVQ8);
            const unsigned code = d_enc4_e4m3(v[i].x, v[i].y, v[i].z, v[i].w, e);
            if (on) {
                *(unsigned *)(pq + ((size_t)row * (C4 >> 3) + (c >> 3)) * 32 + (c & 7) * 4) = code;
                if (!(c & 7)) ps[(size_t)row * (C4 >> 3) + (c >> 3)] = (uint8_t)(e + 127);
            }
        }
    }
    if (!lane) { if (mean) mean[row] = m; if (rstd) rstd[row] = r; }
}
extern "C" void at_ln_fwd(const float *x, const float *g, const float *b, float *y, float *mean, float *rstd, long T, int C) {
    if (T <= 0) return;
    if (C <= 0 || (C & 3) || C > 2048 || (((uintptr_t)x | (uintptr_t)y) & 15)) mi_die("at_ln_fwd: rows of %d channels (a multiple of 4, at most 2048, rows 16-byte aligned)", C);
    const int C4 = C / 4, nv = (C4 + 63) / 64;
    const unsigned grid = nblk_((size_t)T, 4);
#define LN(NV) ln_row_k<NV><<<grid, 256>>>((const float4 *)x, g, b, (float4 *)y, mean, rstd, T, C4)
    if (nv <= 1) LN(1); else if (nv <= 2) LN(2); else if (nv <= 4) LN(4); else LN(8);
#undef LN
    MICK();
}
// at_ln_fwd with the normalised rows written as the packed MX-fp8 A operand of the GEMM that follows (no fp32 rows); C a multiple of 64
static void ln_pack_fwd(const float *x, const float *g, const float *b, float *mean, float *rstd, long T, int C, uint8_t *pq, uint8_t *ps) {
    const int C4 = C / 4, nv = (C4 + 63) / 64;
    const unsigned grid = nblk_((size_t)T, 4);
#define LN(NV) ln_row_k<NV, true><<<grid, 256>>>((const float4 *)x, g, b, nullptr, mean, rstd, T, C4, pq, ps)
    if (nv <= 1) LN(1); else if (nv <= 2) LN(2); else if (nv <= 4) LN(4); else LN(8);
#undef LN
    MICK();
}
// ---- SwiGLU (src/nn_attn.cu:438-455): gg[t][f] = silu(h[t][f]) h[t][F + f]; four features per thread, 16-byte accesses. silu(a) = a rcp(1 +
// exp2(-a log2 e)) on the hardware's exp2 and reciprocal, the form the reference's device fast-math build gives a / (1.f + expf(-a)) (approximate
// exponential and division) and the one the conv path's SiLU has ----
__global__ void __launch_bounds__(256) glu_rows_k(const float4 *__restrict__ h, float4 *__restrict__ gg, size_t n4, unsigned F4) {
    const size_t i = blockIdx.x * (size_t)256 + threadIdx.x;      // one float4 chunk of one token's output row: any token count, full workgroups
    if (i >= n4) return;
    const size_t t = i / F4; const unsigned f = (unsigned)(i - t * F4);
    const float4 a = h[t * 2 * F4 + f], b = h[t * 2 * F4 + F4 + f];
    gg[i] = make_float4(d_silu(a.x) * b.x, d_silu(a.y) * b.y, d_silu(a.z) * b.z, d_silu(a.w) * b.w);
}
__global__ void __launch_bounds__(256) glu_any_k(const float *__restrict__ h, float *__restrict__ gg, size_t n, int F) {       // widths that are not a multiple of 4
    const size_t i = blockIdx.x * (size_t)256 + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / (unsigned)F; const int f = (int)(i - t * F);
    const float a = h[t * 2 * F + f];
    gg[i] = d_silu(a) * h[t * 2 * F + F + f];
}
// at_glu_fwd with the result written as the packed MX-fp8 A operand of the GEMM that follows: glu_rows_k's thread (one float4 chunk of a token's
// row, the same expression per value: contiguous 16-byte reads across a wavefront), then mx_pack_k<8, 0>'s quantisation of the block of 32
// features that eight neighbouring lanes hold (their maxima meet through three lane exchanges). F a multiple of 64
__global__ void __launch_bounds__(256) glu_pack_k(const float4 *__restrict__ h, size_t n4, unsigned F4, uint8_t *__restrict__ pq, uint8_t *__restrict__ ps) {
    const size_t i = blockIdx.x * (size_t)256 + threadIdx.x;
    if (i >= n4) return;                                   // (n4 is a multiple of 8: the lanes of a group of eight leave together)
    const size_t t = i / F4; const unsigned f = (unsigned)(i - t * F4);
    const float4 a = h[t * 2 * F4 + f], b = h[t * 2 * F4 + F4 + f];
    const float4 o = make_float4(d_silu(a.x) * b.x, d_silu(a.y) * b.y, d_silu(a.z) * b.z, d_silu(a.w) * b.w);
    unsigned au = __float_as_uint(fmaxf(fmaxf(fabsf(o.x), fabsf(o.y)), fmaxf(fabsf(o.z), fabsf(o.w))));       // (fmaxf drops NaN; a non-negative number orders as its bits)
    au = max(au, d_quad_xor_u<1>(au)); au = max(au, d_quad_xor_u<2>(au));
    au = max(au, d_oct_mirror_u(au));
    const int e = d_mx_exp(__uint_as_float(au), MI_INVQ8);
    *(unsigned *)(pq + i * 4) = d_enc4_e4m3(o.x, o.y, o.z, o.w, e);            // (block (t, f / 8) lies at ((t F4 + f) / 8) 32 bytes: the chunks' codes are consecutive)
    if (!(f & 7)) ps[i >> 3] = (uint8_t)(e + 127);
}
extern "C" void at_glu_fwd(const float *h, float *gg, long T, int F) {
    if (T <= 0 || F <= 0) return;
    if ((F & 3) == 0 && !(((uintptr_t)h | (uintptr_t)gg) & 15)) {
        const size_t n4 = (size_t)T * (F / 4);
        glu_rows_k<<<nblk_(n4, 256), 256>>>((const float4 *)h, (float4 *)gg, n4, (unsigned)(F / 4));
    } else glu_any_k<<<nblk_((size_t)T * F, 256), 256>>>(h, gg, (size_t)T * F, F);
    MICK();
}
// ---- channel planes [n][C][Sg] <-> token rows [n][nreg + Sg][C] (src/nn_attn.cu:748-759): a transpose, done through 32 x 32 LDS tiles so that
// both the plane side (contiguous in the token index) and the row side (contiguous in the channel) move whole 128-byte lines; the learned
// register rows are copied in front of each sample's tokens ----
template <bool TO_TOK>
__global__ void __launch_bounds__(256) tok_transpose_k(const float *__restrict__ src, float *__restrict__ dst, int C, long long Sg, int nreg) {
    __shared__ float tile[32][33];
    const int n = blockIdx.z, c0 = blockIdx.y * 32, tx = threadIdx.x & 31, ty = threadIdx.x >> 5;      // ty 0 .. 7
    const long long s0 = blockIdx.x * 32ll, S = Sg + nreg;
    const float *planes = TO_TOK ? src : nullptr; float *planes_o = TO_TOK ? nullptr : dst;
    if (TO_TOK) {
#pragma unroll
        for (int k = 0; k < 4; k++) { const int c = c0 + ty + 8 * k; const long long sp = s0 + tx; tile[ty + 8 * k][tx] = c < C && sp < Sg ? planes[((long long)n * C + c) * Sg + sp] : 0.f; }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 4; k++) { const long long sp = s0 + ty + 8 * k; const int c = c0 + tx; if (sp < Sg && c < C) dst[((long long)n * S + nreg + sp) * C + c] = tile[tx][ty + 8 * k]; }
    } else {
#pragma unroll
        for (int k = 0; k < 4; k++) { const long long sp = s0 + ty + 8 * k; const int c = c0 + tx; tile[ty + 8 * k][tx] = sp < Sg && c < C ? src[((long long)n * S + nreg + sp) * C + c] : 0.f; }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 4; k++) { const int c = c0 + ty + 8 * k; const long long sp = s0 + tx; if (c < C && sp < Sg) planes_o[((long long)n * C + c) * Sg + sp] = tile[tx][ty + 8 * k]; }
    }
}
__global__ void __launch_bounds__(256) reg_rows_k(const float *__restrict__ reg, float *__restrict__ t, int n, int C, long long S, int nreg) {
    const size_t i = blockIdx.x * (size_t)256 + threadIdx.x, per = (size_t)nreg * C;
    if (i >= per * n) return;
    const size_t s = i / per, k = i - s * per;
    t[s * (size_t)S * C + k] = reg[k];
}
extern "C" void at_cs_to_tok(const float *x, float *t, const float *reg, int n, int C, long Sg, int nreg) {
    if (n <= 0 || C <= 0) return;
    if (n > 65535 || (C + 31) / 32 > 65535) mi_die("at_cs_to_tok: %d samples x %d channels exceed the launch grid", n, C);
    if (Sg > 0) tok_transpose_k<true><<<dim3(nblk_((size_t)Sg, 32), (unsigned)((C + 31) / 32), (unsigned)n), 256>>>(x, t, C, Sg, nreg);
    if (nreg > 0) reg_rows_k<<<nblk_((size_t)n * nreg * C, 256), 256>>>(reg, t, n, C, Sg + nreg, nreg);
    MICK();
}
extern "C" void at_tok_to_cs(const float *t, float *x, int n, int C, long Sg, int nreg) {
    if (n <= 0 || C <= 0 || Sg <= 0) return;
    if (n > 65535 || (C + 31) / 32 > 65535) mi_die("at_tok_to_cs: %d samples x %d channels exceed the launch grid", n, C);
    tok_transpose_k<false><<<dim3(nblk_((size_t)Sg, 32), (unsigned)((C + 31) / 32), (unsigned)n), 256>>>(t, x, C, Sg, nreg);
    MICK();
}

// ---- QKV pack (src/nn_attn_tc.cu:99-136): per (token, head) the 48 q and k dims are RMS-normalised (eps 1e-6) and scaled by their learned
// gains, grid tokens rotated by the 3-D rotary embedding (16 dims per coordinate: pair f of coordinate a turns by pos_a base^(-f / 8); pos = the
// token's grid indices, or its row of a coordinate array: src/nn_attn.cu:272-289), v passes
// through; all three go to the fp16 head-major layout [3][H][T + 64][48] the attention core reads (64 zero rows of padding).
// A unit = one (token, part, head) = 48 values = six 8-dim slices; eight neighbouring lanes own a unit (two idle), each slice is two 16-byte
// loads and one 16-byte store of eight halves. The sum of squares meets over the unit's lanes; a rotary pair never leaves its lane
// (slice j covers pairs 4 (j & 1) .. + 3 of axis j / 2). ----
struct ray_src { ray_geo G; const float *ray; const int *ad; };      // ray: null = the rows are the tokens' own
__global__ void __launch_bounds__(256) qkv_pack_k(const float *__restrict__ qkv, const float *__restrict__ qg, const float *__restrict__ kg, __half *__restrict__ out,
                                                  float *__restrict__ rq, float *__restrict__ rk, float *__restrict__ amx, long long T, int H, int S, int Hh, int W, int nreg, int rope, float lbase,
                                                  const float *__restrict__ gpos, ray_src rs) {
    // the rotary angles take few values - position along an axis x frequency - and a sine / cosine pair costs far more than the rest of a unit:
    // a block forms the table once (the same expression the per-value form evaluates, so the same bits), positions up to RP per axis
    constexpr int RP = 64;
    __shared__ float2 rtab[RP * 8];
    const int pmax = max(max(S / (Hh * W), Hh), W);         // positions along an axis: < pmax (registers included in S: an upper bound)
    const bool tab = rope && !gpos && pmax <= RP;            // (gpos: per-token coordinates, real numbers: every angle is evaluated)
    if (tab) {
        for (int i = threadIdx.x; i < pmax * 8; i += 256) { float sn, cs; sincosf((float)(i >> 3) * exp2f(-lbase * (float)(i & 7) / 8.f), &sn, &cs); rtab[i] = make_float2(sn, cs); }
        __syncthreads();
    }
    const long long unit = (blockIdx.x * 256ll + threadIdx.x) >> 3; const int j = threadIdx.x & 7;
    const long long Tp = T + FT, nunits = Tp * H * 3;
    // the largest |v| of the call: per unit over its lanes, per block through one LDS word, one global atomic per block (one per unit made
    // 10^5 atomics on one address the kernel's whole run time)
    __shared__ unsigned bmax;
    if (threadIdx.x == 0) bmax = 0u;
    __syncthreads();
    if (unit < nunits) {
        const int h = (int)(unit % H); const long long tp = unit / H; const int p = (int)(tp % 3); const long long t = tp / 3;      // units of a token are neighbours: its 3 H x 192 bytes are read together
        const int C = H * HD;
        __half *dst = out + (((size_t)p * H + h) * Tp + t) * HD + 8 * j;
        if (t >= T) { if (j < 6) *(uint4 *)dst = make_uint4(0u, 0u, 0u, 0u); }
        else {
            float v[8];
            if (j < 6 && rs.ray) {
                // radial attention: token t is a ray slot, its row the bilinear mix of the grid rows under it (at_ray_gather's arithmetic, corner by
                // corner in its order), formed here instead of in a [slots][3 C] array that this kernel would read back
                long long row[4]; float w[4];
                const int nc = slot_stencil(rs.G, rs.ray, rs.ad, t, row, w);
#pragma unroll
                for (int i = 0; i < 8; i++) v[i] = 0.f;
                for (int c = 0; c < nc; c++) {
                    if (w[c] == 0.f) continue;
                    const float4 *xs = (const float4 *)(qkv + row[c] * 3 * C + p * C + h * HD + 8 * j);
                    const float4 a = xs[0], b = xs[1];
                    v[0] = fmaf(w[c], a.x, v[0]); v[1] = fmaf(w[c], a.y, v[1]); v[2] = fmaf(w[c], a.z, v[2]); v[3] = fmaf(w[c], a.w, v[3]);
                    v[4] = fmaf(w[c], b.x, v[4]); v[5] = fmaf(w[c], b.y, v[5]); v[6] = fmaf(w[c], b.z, v[6]); v[7] = fmaf(w[c], b.w, v[7]);
                }
            } else if (j < 6) {
                const float4 *xs = (const float4 *)(qkv + t * 3 * C + p * C + h * HD + 8 * j);
                const float4 a = xs[0], b = xs[1];
                v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) v[i] = 0.f;
            }
            if (p < 2) {
                float ss = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) ss = fmaf(v[i], v[i], ss);
                ss += d_quad_xor_f<1>(ss); ss += d_quad_xor_f<2>(ss); ss += d_oct_mirror_f(ss);      // (the unit's eight lanes: the same sums as the xor butterfly's, no LDS round trips)
                const float r = 1.f / sqrtf(ss / HD + 1e-6f);
                if (j == 0) (p ? rk : rq)[t * H + h] = r;
                if (j < 6) {
                    const float *gs = (p ? kg : qg) + h * HD + 8 * j;      // (the gains sit at an arbitrary offset of the flat parameter vector: dword loads)
#pragma unroll
                    for (int i = 0; i < 8; i++) v[i] *= r * gs[i];
                    const int ts = (int)(t % S) - nreg;
                    if (rope && ts >= 0) {
                        const int ax = j >> 1;
                        const float pos = gpos ? gpos[3 * t + ax] : ax == 0 ? (float)(ts / (Hh * W)) : ax == 1 ? (float)((ts / W) % Hh) : (float)(ts % W);
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const int fi = 4 * (j & 1) + i;
                            float sn, cs;
                            if (tab) { const float2 sc2 = rtab[(int)pos * 8 + fi]; sn = sc2.x; cs = sc2.y; }
                            else if (gpos) { const float ang = pos * exp2f(-lbase * (float)fi / 8.f); sn = __sinf(ang); cs = __cosf(ang); }      // (real coordinates: the hardware sine / cosine, as the reference's fast-math build)
                            else sincosf(pos * exp2f(-lbase * (float)fi / 8.f), &sn, &cs);
                            const float a = v[2 * i], b = v[2 * i + 1];
                            v[2 * i] = a * cs - b * sn; v[2 * i + 1] = a * sn + b * cs;
                        }
                    }
                }
            } else {
                float m = 0.f;
#pragma unroll
                for (int i = 0; i < 8; i++) m = fmaxf(m, fabsf(v[i]));
                m = fmaxf(m, d_quad_xor_f<1>(m)); m = fmaxf(m, d_quad_xor_f<2>(m)); m = fmaxf(m, d_oct_mirror_f(m));
                if (j == 0) atomicMax(&bmax, __float_as_uint(m));               // (non-negative floats order as their bit patterns)
            }
            if (j < 6) {
                const __half2 h0 = __floats2half2_rn(v[0], v[1]), h1 = __floats2half2_rn(v[2], v[3]), h2 = __floats2half2_rn(v[4], v[5]), h3 = __floats2half2_rn(v[6], v[7]);
                *(uint4 *)dst = make_uint4(*(const unsigned *)&h0, *(const unsigned *)&h1, *(const unsigned *)&h2, *(const unsigned *)&h3);
            }
        }
    }
    __syncthreads();
    // (the running maximum only grows: a block whose own maximum does not exceed the value it reads has nothing to add, which spares the
    // single address all but a few of the 10^4 blocks' atomics)
    if (threadIdx.x == 0 && bmax > *(volatile unsigned *)((unsigned *)amx + 1)) atomicMax((unsigned *)amx + 1, bmax);
}
__global__ void at_zero4_k(float *p) { if (threadIdx.x < 4) p[threadIdx.x] = 0.f; }
static void fa_pack(const float *qkv, const float *qg, const float *kg, void *qkvh, float *rq, float *rk, float *amx, const at_geom *g, int nreg, int C, int rope, float base, const at_rays *R) {
    if (C % HD || (C & 3)) mi_die("at_fa_pack: C %d is not a whole number of heads of %d", C, HD);
    const long long T = (long long)g->nseq * g->S, Tp = T + FT; const int H = C / HD;
    ray_src rs = {};
    if (R) { rs.G = geo_of(R); rs.ray = R->ray; rs.ad = R->ad; }
    at_zero4_k<<<1, 64>>>(amx);
    qkv_pack_k<<<nblk_((size_t)Tp * H * 3 * 8, 256), 256>>>(qkv, qg, kg, (__half *)qkvh, rq, rk, amx, T, H, g->S, g->Hh, g->W, nreg, rope, log2f(base), rope ? g->pos : nullptr, rs);
    MICK();
}
extern "C" void at_fa_pack(const float *qkv, const float *qg, const float *kg, void *qkvh, float *rq, float *rk, float *amx, const at_geom *g, int nreg, int C, int rope, float base) {
    fa_pack(qkv, qg, kg, qkvh, rq, rk, amx, g, nreg, C, rope, base, nullptr);
}

// ---- parameters and scratch ----
extern "C" size_t at_block_layout(const at_dims *d, at_bp *bp, size_t off) {
    if (d->dK > 0) mi_die("at_block_layout: deformable attention blocks are not supported");
    const size_t C = d->C, F = d->F;
    for (int l = 0; l < AT_DFM_MAXL; l++) bp->wvl[l] = bp->bvl[l] = 0;
    bp->woa = bp->boa = 0;
    size_t *order[] = {&bp->ln1g, &bp->ln1b, &bp->wqkv, &bp->bqkv, &bp->qg, &bp->kg, &bp->wo, &bp->bo, &bp->ln2g, &bp->ln2b, &bp->w1, &bp->b1, &bp->w2, &bp->b2};
    const size_t len[] = {C, C, 3 * C * C, 3 * C, C, C, C * C, C, C, C, 2 * F * C, 2 * F, C * F, C};
    for (int k = 0; k < 14; k++) { *order[k] = off; off += len[k]; }
    return off;
}
extern "C" size_t at_block_nparams(const at_dims *d) { at_bp bp; return at_block_layout(d, &bp, 0); }
static size_t ws_walk(at_ws *w, const at_dims *d, long T, long Tr, float *base) {      // pieces of whole 256 bytes; base null: sizes only. Tr: ray tokens (0: none)
    const size_t C = d->C, F = d->F, H = d->H, t = (size_t)T, ta = Tr > 0 ? (size_t)Tr : t;   // ta: the tokens the attention itself runs on
    size_t n = 0;
    auto take = [&](float *&f, size_t m) { f = base ? base + n : nullptr; n += (m + 63) & ~(size_t)63; };
    at_ws tmp; if (!w) w = &tmp;
    *w = at_ws{};
    take(w->xn, t * C); take(w->o, t * C); take(w->x1, t * C); take(w->xn2, t * C); take(w->qkv, t * 3 * C); take(w->h, t * 2 * F); take(w->gg, t * F);
    take(w->m1, t); take(w->r1, t); take(w->m2, t); take(w->r2, t); take(w->rq, ta * H); take(w->rk, ta * H); take(w->lse, ta * H);
    take(w->qkvh, 3 * C * (ta + FT) / 2); take(w->amx, 4);
    if (Tr > 0) { take(w->qkvr, ta * 3 * C); take(w->orr, ta * C); }
    return n;
}
extern "C" size_t at_ws_bytes(const at_dims *d, long T) { return ws_walk(nullptr, d, T, 0, nullptr) * sizeof(float); }
extern "C" void at_ws_carve(at_ws *w, const at_dims *d, long T, void *base) { ws_walk(w, d, T, 0, (float *)base); }
extern "C" size_t at_ws_bytes_r(const at_dims *d, long T, long Tr) { return ws_walk(nullptr, d, T, Tr, nullptr) * sizeof(float); }
extern "C" void at_ws_carve_r(at_ws *w, const at_dims *d, long T, long Tr, void *base) { ws_walk(w, d, T, Tr, (float *)base); }

static thread_local int g_at_mx = 8;
extern "C" void at_set_mx(int bits) { g_at_mx = bits; }
extern "C" int at_get_mx(void) { return g_at_mx; }
extern "C" int at_gemm_ex(int ta, int tb, int M, int N, int K, const float *A, const float *B, float *Cm, float beta, const float *bias, const float *res) {
    if (g_at_mx != 4 && g_at_mx != 8) { fprintf(stderr, "at_gemm_ex: the linear layers run as MX GEMMs here (at_set_mx(4) or (8)); precision %d is not provided\n", g_at_mx); return -1; }
    return lp_mx_gemm_ex(g_at_mx, ta, tb, M, N, K, A, B, Cm, beta, bias, res);
}

// The pre-LN block (src/nn_attn.cu:587-633): x1 = x + Wo attn(pack(Wqkv LN1(x))), y = x1 + W2 swiglu(W1 LN2(x1)). Each of the four linears
// is one MX GEMM with its bias and, for the two that close a residual branch, the residual folded into the GEMM's epilogue.
namespace {
struct linear_t { const float *w, *b; int out, in; };
inline int linear(const linear_t &l, long T, const float *in, float *out, const float *residual) {
    return at_gemm_ex(0, 1, (int)T, l.out, l.in, in, l.w, out, 0.f, l.b, residual);
}
}
// Conv positional encoding (at_peg_fwd, src/attn.h:141-144, src/nn_attn.cu:688-705): y = x + b + depthwise 3^3 conv of x over the grid tokens of a
// sequence (zero padding: taps outside the grid add nothing), register rows copied. w [C][27] with the taps in (dz, dy, dx) order, b [C].
// A thread takes one token's four neighbouring channels; each channel's sum starts from x + b and takes its taps in that order, one fused
// multiply-add each, as the reference's contracted loop.
__global__ void __launch_bounds__(256) peg_rows_k(const float *__restrict__ x, float *__restrict__ y, const float *__restrict__ w, const float *__restrict__ b,
                                                  size_t n4, int S, int D, int Hh, int W, int nreg, int C4) {
    const size_t i = blockIdx.x * (size_t)256 + threadIdx.x;
    if (i >= n4) return;
    const size_t t = i / C4; const int c4 = (int)(i - t * C4), ts = (int)(t % S) - nreg;
    const float4 xv = ((const float4 *)x)[i];
    if (ts < 0) { ((float4 *)y)[i] = xv; return; }
    const size_t row0 = t - (size_t)ts;                            // the sequence's first grid token
    const int z = ts / (Hh * W), yy = (ts / W) % Hh, xx = ts % W;
    const float *bc = b + (size_t)c4 * 4;                          // (scalar loads: the bias sits at any float offset of the parameter vector, not at a multiple of 16 bytes)
    float a[4] = {xv.x + bc[0], xv.y + bc[1], xv.z + bc[2], xv.w + bc[3]};
    const float *wc = w + (size_t)c4 * 4 * 27;
    for (int dz = -1; dz <= 1; dz++) for (int dy = -1; dy <= 1; dy++) for (int dx = -1; dx <= 1; dx++) {
        const int zz = z + dz, y2 = yy + dy, x2 = xx + dx;
        if (zz < 0 || zz >= D || y2 < 0 || y2 >= Hh || x2 < 0 || x2 >= W) continue;
        const float4 nv = ((const float4 *)x)[(row0 + ((size_t)zz * Hh + y2) * W + x2) * C4 + c4];
        const int tap = (dz + 1) * 9 + (dy + 1) * 3 + dx + 1;
        a[0] = fmaf(wc[tap], nv.x, a[0]); a[1] = fmaf(wc[27 + tap], nv.y, a[1]); a[2] = fmaf(wc[54 + tap], nv.z, a[2]); a[3] = fmaf(wc[81 + tap], nv.w, a[3]);
    }
    ((float4 *)y)[i] = make_float4(a[0], a[1], a[2], a[3]);
}
extern "C" void at_peg_fwd(const float *x, float *y, const float *w, const float *b, const at_geom *g, int nreg, int C) {
    if (C % 4 || x == y || (long)g->D * g->Hh * g->W + nreg != g->S) mi_die("at_peg_fwd: C %d (a multiple of 4), separate buffers, S %d = nreg %d + %d x %d x %d", C, g->S, nreg, g->D, g->Hh, g->W);
    const size_t n4 = (size_t)g->nseq * g->S * C / 4;
    if (!n4) return;
    peg_rows_k<<<nblk_(n4, 256), 256>>>(x, y, w, b, n4, g->S, g->D, g->Hh, g->W, nreg, C / 4); MICK();
}
// Value residual (at_ws.vr, src/nn_attn.cu:535-542, :609-610) on the V third of the qkv rows [T][3 C]: the first block of a stage (vr 1) keeps its
// V in v1; a later one (vr 2) replaces its own V by v + lam[head] (v1 - v), one fused multiply-add, and keeps the own V when a buffer is given.
__global__ void __launch_bounds__(256) v_keep_k(const float *__restrict__ qkv, float *__restrict__ v1, size_t n4, int C4) {
    const size_t i = blockIdx.x * (size_t)256 + threadIdx.x;
    if (i >= n4) return;
    const size_t t = i / C4; const int c = (int)(i - t * C4);
    ((float4 *)v1)[i] = ((const float4 *)qkv)[t * 3 * C4 + 2 * C4 + c];
}
__global__ void __launch_bounds__(256) v_mix_k(float *__restrict__ qkv, const float *__restrict__ v1, float *__restrict__ own, const float *__restrict__ lam, size_t n4, int C4) {
    const size_t i = blockIdx.x * (size_t)256 + threadIdx.x;
    if (i >= n4) return;
    const size_t t = i / C4; const int c = (int)(i - t * C4);
    float4 *v = (float4 *)qkv + t * 3 * C4 + 2 * C4 + c;
    const float4 o = *v, f = ((const float4 *)v1)[i];
    const float l = lam[c * 4 / HD];                               // (a head is 48 channels: a group of four lies in one)
    if (own) ((float4 *)own)[i] = o;
    *v = make_float4(fmaf(l, f.x - o.x, o.x), fmaf(l, f.y - o.y, o.y), fmaf(l, f.z - o.z, o.z), fmaf(l, f.w - o.w, o.w));
}
static int g_fuse_pack = 2;
extern "C" void at_fuse_pack(int on) { g_fuse_pack = on < 0 ? 0 : on > 2 ? 2 : on; }
extern "C" int at_block_fwd(const at_dims *d, const float *P, const at_bp *bp, const float *x, float *y, const at_geom *g, at_ws *w) {
    const at_rays *R = g->rays;
    if (d->dK > 0 || w->vr < 0 || w->vr > 2 || (w->vr && (!w->v1 || (w->vr == 2 && !w->lam))) || d->rope < 0 || d->rope > 2 || d->C != d->H * HD) return -1;
    if (R ? d->nreg != 0 || !w->qkvr || !w->orr || !R->lens || !R->wsum || (d->rope == 2 && !R->pos) || (long)R->n * R->D * R->Hh * R->W != (long)g->nseq * g->S
          : g->lens != nullptr || (d->rope == 2 && !g->pos)) return -1;      // (sequence lengths belong to the ray path; scroll RoPE needs its coordinates)
    const long T = (long)g->nseq * g->S; const int C = d->C, F = d->F;
    // the attention's own geometry: the grid's, or (radial attention) the rays' - R->n Q sequences of Nr slots, their lengths and positions (src/nn_attn.cu:576-581)
    at_geom ga = *g;
    if (R) { ga = at_geom{}; ga.nseq = R->n * R->Q; ga.S = R->Nr; ga.D = 1; ga.Hh = 1; ga.W = R->Nr; ga.lens = R->lens; ga.pos = d->rope == 2 ? R->pos : nullptr; }
    else if (d->rope != 2) ga.pos = nullptr;
    const linear_t qkv = {P + bp->wqkv, P + bp->bqkv, 3 * C, C}, proj = {P + bp->wo, P + bp->bo, C, C}, up = {P + bp->w1, P + bp->b1, 2 * F, C}, down = {P + bp->w2, P + bp->b2, C, F};
    // The rows a LayerNorm or the SwiGLU produces are read by one GEMM only: with e4m3 linears and widths that are multiples of 64 they are
    // written as that GEMM's packed operand directly and the fp32 rows (xn, xn2, gg of the scratch record, which only a backward pass would
    // read again) are not: per block 1.8 GB less HBM traffic at 250 000 tokens and three launches fewer. The same values quantised the same way
    const bool fuse = g_fuse_pack && g_at_mx == 8 && C % 64 == 0 && F % 64 == 0 && !((uintptr_t)x & 15) && !((uintptr_t)w->x1 & 15) && !((uintptr_t)w->h & 15);
    uint8_t *aq = nullptr, *as = nullptr;
    // attention branch
    if (fuse && mi_mx_gemm_abuf(8, (int)T, 3 * C, C, &aq, &as)) {
        ln_pack_fwd(x, P + bp->ln1g, P + bp->ln1b, w->m1, w->r1, T, C, aq, as);
        if (int e = mi_mx_gemm_apacked(8, 1, (int)T, 3 * C, C, qkv.w, w->qkv, 0.f, qkv.b, nullptr)) return e;
    } else {
        at_ln_fwd(x, P + bp->ln1g, P + bp->ln1b, w->xn, w->m1, w->r1, T, C);
        if (int e = linear(qkv, T, w->xn, w->qkv, nullptr)) return e;
    }
    if (w->vr) {
        const size_t n4 = (size_t)T * C / 4;
        if (w->vr == 1) v_keep_k<<<nblk_(n4, 256), 256>>>(w->qkv, w->v1, n4, C / 4); else v_mix_k<<<nblk_(n4, 256), 256>>>(w->qkv, w->v1, w->own, w->lam, n4, C / 4);
        MICK();
    }
    if (R) {
        // (the pack reads the grid's rows through the rays' stencils: at_ray_gather's rows without their round trip through w->qkvr, which stays unwritten)
        fa_pack(w->qkv, P + bp->qg, P + bp->kg, w->qkvh, w->rq, w->rk, w->amx, &ga, 0, C, d->rope, d->rope_base, R);
        at_fa_fwd(w->qkvh, w->orr, w->lse, &ga, d->H, C);
        at_ray_scatter(R, w->orr, w->o, C, 1);
    } else {
        at_fa_pack(w->qkv, P + bp->qg, P + bp->kg, w->qkvh, w->rq, w->rk, w->amx, &ga, d->nreg, C, d->rope, d->rope_base);
        if (int e = at_fa8_fwd(w->qkvh, w->o, w->lse, &ga, d->H, C)) return e;
    }
    if (int e = linear(proj, T, w->o, w->x1, x)) return e;
    // MLP branch
    if (fuse && mi_mx_gemm_abuf(8, (int)T, 2 * F, C, &aq, &as)) {
        ln_pack_fwd(w->x1, P + bp->ln2g, P + bp->ln2b, w->m2, w->r2, T, C, aq, as);
        if (g_fuse_pack > 1 && C <= 256) {
            // ... and the up projection forms the SwiGLU in its epilogue and writes the down projection's packed operand: h is not stored either
            const size_t nb = (size_t)T * (F / 32);
            uint8_t *gq = (uint8_t *)mi_ws(MI_WS_GEMM2, nb * 32 + ((nb + 255) & ~(size_t)255) + 256), *gs = gq + nb * 32;
            if (int e = mi_mx_gemm_glu((int)T, F, C, up.w, up.b, gq, gs)) return e;
            return mi_mx_gemm_apacked_at(8, 1, (int)T, C, F, gq, gs, down.w, y, 0.f, down.b, w->x1);
        }
        if (int e = mi_mx_gemm_apacked(8, 1, (int)T, 2 * F, C, up.w, w->h, 0.f, up.b, nullptr)) return e;
    } else {
        at_ln_fwd(w->x1, P + bp->ln2g, P + bp->ln2b, w->xn2, w->m2, w->r2, T, C);
        if (int e = linear(up, T, w->xn2, w->h, nullptr)) return e;
    }
    if (fuse && mi_mx_gemm_abuf(8, (int)T, C, F, &aq, &as)) {
        const size_t n4 = (size_t)T * (F / 4);
        glu_pack_k<<<nblk_(n4, 256), 256>>>((const float4 *)w->h, n4, (unsigned)(F / 4), aq, as); MICK();
        return mi_mx_gemm_apacked(8, 1, (int)T, C, F, down.w, y, 0.f, down.b, w->x1);
    }
    at_glu_fwd(w->h, w->gg, T, F);
    return linear(down, T, w->gg, y, w->x1);
}
