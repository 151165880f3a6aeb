// The attention block around the MX GEMM and the MX-fp8 attention core: LayerNorm, QK-norm + gains + RoPE pack to fp16, SwiGLU, token
// layout, parameter layout, scratch carving and the block forward (src/nn_attn.cu:150-168, :438-455, :460-530, :587-633, :748-759 and
// src/nn_attn_tc.cu:99-136 of the reference). The elementwise kernels are HBM-bound row kernels.
#include <hip/hip_fp16.h>
#include "mx_dev.hpp"
#include "../../include/mi_attn.h"

#define HD AT_HD
#define FT 64

// LayerNorm: one wavefront per row; two passes over the row (mean, then centred squares), as the reference
__global__ void __launch_bounds__(256) at_ln_k(const float *__restrict__ x, const float *__restrict__ g, const float *__restrict__ b, float *__restrict__ y,
                                               float *__restrict__ mean, float *__restrict__ rstd, long long T, int C) {
    const long long row = (blockIdx.x * (long long)blockDim.x + threadIdx.x) >> 6; const int lane = threadIdx.x & 63;
    if (row >= T) return;
    const float *xr = x + row * C;
    float s = 0.f;
    for (int c = lane; c < C; c += 64) s += xr[c];
    for (int o = 32; o; o >>= 1) s += __shfl_xor(s, o);
    const float m = s / C; float q = 0.f;
    for (int c = lane; c < C; c += 64) { const float d = xr[c] - m; q += d * d; }
    for (int o = 32; o; o >>= 1) q += __shfl_xor(q, o);
    const float r = 1.f / sqrtf(q / C + 1e-5f);
    for (int c = lane; c < C; c += 64) y[row * C + c] = (xr[c] - m) * r * g[c] + b[c];
    if (!lane) { if (mean) mean[row] = m; if (rstd) rstd[row] = r; }
}
extern "C" void at_ln_fwd(const float *x, const float *g, const float *b, float *y, float *mean, float *rstd, long T, int C) {
    if (T <= 0) return;
    at_ln_k<<<nblk_((size_t)T * 64, 256), 256>>>(x, g, b, y, mean, rstd, T, C);
    MICK();
}
__global__ void __launch_bounds__(256) at_glu_k(const float *__restrict__ h, float *__restrict__ gg, long long T, int F) {
    const long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x;
    if (i >= T * F) return;
    const long long t = i / F; const int f = (int)(i % F);
    const float a = h[t * 2 * F + f], b = h[t * 2 * F + F + f];
    gg[i] = a / (1.f + expf(-a)) * b;
}
extern "C" void at_glu_fwd(const float *h, float *gg, long T, int F) {
    if (T <= 0 || F <= 0) return;
    at_glu_k<<<nblk_((size_t)T * F, 256), 256>>>(h, gg, T, F);
    MICK();
}
__global__ void __launch_bounds__(256) at_cs_to_tok_k(const float *__restrict__ x, float *__restrict__ t, const float *__restrict__ reg, int n, int C, long long Sg, int nreg) {
    const long long S = Sg + nreg, i = blockIdx.x * (long long)blockDim.x + threadIdx.x;
    if (i >= (long long)n * S * C) return;
    const int c = (int)(i % C); const long long r = i / C; const int s = (int)(r / S); const long long ts = r % S - nreg;
    t[i] = ts < 0 ? reg[(r % S) * C + c] : x[((long long)s * C + c) * Sg + ts];
}
__global__ void __launch_bounds__(256) at_tok_to_cs_k(const float *__restrict__ t, float *__restrict__ x, int n, int C, long long Sg, int nreg) {
    const long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x;
    if (i >= (long long)n * C * Sg) return;
    const long long ts = i % Sg; const int c = (int)((i / Sg) % C), s = (int)(i / (Sg * C));
    x[i] = t[((long long)s * (Sg + nreg) + nreg + ts) * C + c];
}
extern "C" void at_cs_to_tok(const float *x, float *t, const float *reg, int n, int C, long Sg, int nreg) {
    const size_t m = (size_t)n * (Sg + nreg) * C; if (!m) return;
    at_cs_to_tok_k<<<nblk_(m, 256), 256>>>(x, t, reg, n, C, Sg, nreg); MICK();
}
extern "C" void at_tok_to_cs(const float *t, float *x, int n, int C, long Sg, int nreg) {
    const size_t m = (size_t)n * C * Sg; if (!m) return;
    at_tok_to_cs_k<<<nblk_(m, 256), 256>>>(t, x, n, C, Sg, nreg); MICK();
}

// one thread per (token row incl. the 64 padding rows, head, q / k / v): 48 values in registers
__global__ void __launch_bounds__(128) at_pack_k(const float *__restrict__ qkv, const float *__restrict__ qg, const float *__restrict__ kg, __half *Qh, __half *Kh, __half *Vh,
                                                 float *rq, float *rk, float *amx, long long T, int C, int S, int Hh, int W, int nreg, int rope, float lbase) {
    const int H = C / HD; const long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x;
    if (i >= (T + FT) * H * 3) return;
    const int p = (int)(i % 3); const long long th = i / 3; const int h = (int)(th % H); const long long t = th / H;
    __half *dst = (p == 0 ? Qh : p == 1 ? Kh : Vh) + ((size_t)h * (T + FT) + t) * HD;
    if (t >= T) { for (int d = 0; d < HD; d += 8) *(uint4 *)(dst + d) = make_uint4(0, 0, 0, 0); return; }
    const float *xs = qkv + t * 3 * C + p * C + h * HD;
    float v[HD];
#pragma unroll
    for (int d = 0; d < HD; d += 4) { const float4 f = *(const float4 *)(xs + d); v[d] = f.x; v[d + 1] = f.y; v[d + 2] = f.z; v[d + 3] = f.w; }
    if (p < 2) {
        float s = 0.f;
#pragma unroll
        for (int d = 0; d < HD; d++) s += v[d] * v[d];
        const float r = 1.f / sqrtf(s / HD + 1e-6f); const float *gs = (p ? kg : qg) + h * HD;
#pragma unroll
        for (int d = 0; d < HD; d++) v[d] *= r * gs[d];
        (p ? rk : rq)[t * H + h] = r;
        const int ts = (int)(t % S) - nreg;
        if (rope && ts >= 0) {
            const float pos[3] = {(float)(ts / (Hh * W)), (float)((ts / W) % Hh), (float)(ts % W)};
#pragma unroll
            for (int pr = 0; pr < 24; pr++) {
                const int ax = pr / 8, fi = pr % 8; float sn, cs; sincosf(pos[ax] * exp2f(-lbase * (float)fi / 8.f), &sn, &cs);
                const float a = v[ax * 16 + 2 * fi], b = v[ax * 16 + 2 * fi + 1];
                v[ax * 16 + 2 * fi] = a * cs - b * sn; v[ax * 16 + 2 * fi + 1] = a * sn + b * cs;
            }
        }
    } else {
        float m = 0.f;
#pragma unroll
        for (int d = 0; d < HD; d++) m = fmaxf(m, fabsf(v[d]));
        atomicMax((unsigned *)amx + 1, __float_as_uint(m));     // (non-negative floats order as their bit patterns)
    }
#pragma unroll
    for (int d = 0; d < HD; d += 2) *(__half2 *)(dst + d) = __floats2half2_rn(v[d], v[d + 1]);
}
__global__ void at_zero4_k(float *p) { if (threadIdx.x < 4) p[threadIdx.x] = 0.f; }
extern "C" void at_fa_pack(const float *qkv, const float *qg, const float *kg, void *qkvh, float *rq, float *rk, float *amx, const at_geom *g, int nreg, int C, int rope, float base) {
    if (g->pos) mi_die("at_fa_pack: per-token rotary positions are not supported");
    if (C % HD || (C & 3)) mi_die("at_fa_pack: C %d is not a whole number of heads of %d", C, HD);
    const long long T = (long long)g->nseq * g->S, Tp = T + FT; const int H = C / HD;
    __half *Qh = (__half *)qkvh, *Kh = Qh + (size_t)H * Tp * HD, *Vh = Kh + (size_t)H * Tp * HD;
    at_zero4_k<<<1, 64>>>(amx);
    at_pack_k<<<nblk_((size_t)Tp * H * 3, 128), 128>>>(qkv, qg, kg, Qh, Kh, Vh, rq, rk, amx, T, C, g->S, g->Hh, g->W, nreg, rope, log2f(base));
    MICK();
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
static size_t ws_walk(at_ws *w, const at_dims *d, long T, float *base) {      // pieces of whole 256 bytes; base null: sizes only
    const size_t C = d->C, F = d->F, H = d->H, t = (size_t)T;
    size_t n = 0;
    auto take = [&](float *&f, size_t m) { f = base ? base + n : nullptr; n += (m + 63) & ~(size_t)63; };
    at_ws tmp; if (!w) w = &tmp;
    *w = at_ws{};
    take(w->xn, t * C); take(w->o, t * C); take(w->x1, t * C); take(w->xn2, t * C); take(w->qkv, t * 3 * C); take(w->h, t * 2 * F); take(w->gg, t * F);
    take(w->m1, t); take(w->r1, t); take(w->m2, t); take(w->r2, t); take(w->rq, t * H); take(w->rk, t * H); take(w->lse, t * H);
    take(w->qkvh, 3 * C * (t + FT) / 2); take(w->amx, 4);
    return n;
}
extern "C" size_t at_ws_bytes(const at_dims *d, long T) { return ws_walk(nullptr, d, T, nullptr) * sizeof(float); }
extern "C" void at_ws_carve(at_ws *w, const at_dims *d, long T, void *base) { ws_walk(w, d, T, (float *)base); }

static thread_local int g_at_mx = 8;
extern "C" void at_set_mx(int bits) { g_at_mx = bits; }
extern "C" int at_get_mx(void) { return g_at_mx; }
extern "C" int at_gemm_ex(int ta, int tb, int M, int N, int K, const float *A, const float *B, float *Cm, float beta, const float *bias, const float *res) {
    if (g_at_mx != 4 && g_at_mx != 8) { fprintf(stderr, "at_gemm_ex: the linear layers run as MX GEMMs here (at_set_mx(4) or (8)); precision %d is not provided\n", g_at_mx); return -1; }
    return lp_mx_gemm_ex(g_at_mx, ta, tb, M, N, K, A, B, Cm, beta, bias, res);
}

extern "C" int at_block_fwd(const at_dims *d, const float *P, const at_bp *bp, const float *x, float *y, const at_geom *g, at_ws *w) {
    if (d->dK > 0 || g->rays || g->lens || g->pos || w->vr || d->rope > 1 || d->C != d->H * HD) return -1;
    const long T = (long)g->nseq * g->S; const int C = d->C, F = d->F;
    int e = 0;
    at_ln_fwd(x, P + bp->ln1g, P + bp->ln1b, w->xn, w->m1, w->r1, T, C);
    e |= at_gemm_ex(0, 1, (int)T, 3 * C, C, w->xn, P + bp->wqkv, w->qkv, 0.f, P + bp->bqkv, nullptr); if (e) return e;
    at_fa_pack(w->qkv, P + bp->qg, P + bp->kg, w->qkvh, w->rq, w->rk, w->amx, g, d->nreg, C, d->rope, d->rope_base);
    e |= at_fa8_fwd(w->qkvh, w->o, w->lse, g, d->H, C); if (e) return e;
    e |= at_gemm_ex(0, 1, (int)T, C, C, w->o, P + bp->wo, w->x1, 0.f, P + bp->bo, x); if (e) return e;
    at_ln_fwd(w->x1, P + bp->ln2g, P + bp->ln2b, w->xn2, w->m2, w->r2, T, C);
    e |= at_gemm_ex(0, 1, (int)T, 2 * F, C, w->xn2, P + bp->w1, w->h, 0.f, P + bp->b1, nullptr); if (e) return e;
    at_glu_fwd(w->h, w->gg, T, F);
    e |= at_gemm_ex(0, 1, (int)T, C, F, w->gg, P + bp->w2, y, 0.f, P + bp->b2, w->x1);
    return e;
}
