// MX-fp8 attention forward core: softmax(Q K^T / sqrt(48)) V per sequence and head on block-scaled e4m3 MFMA (32x32x64).
// Interface and arithmetic: src/lp_attn8.cu:1-13 (definition), :29-76 (conversions), :124-180 (forward), :319-328 (entry) of the reference.
//
// The products are formed transposed, S^T = K Q^T and O^T = V^T P^T, so a query is a column of every accumulator: a lane (r, h) holds,
// for query r of its wavefront, 16 of the 32 keys of each key block and its partner lane (r, h ^ 1) the other 16. All row statistics
// of the softmax (maximum, sum, the rescale factor, the MX scale of P) are then per lane plus one exchange with the partner.
// An 8-bit operand fragment of the 32x32x64 MFMA holds, in lane (r, h), bytes 16 h ... 16 h + 15 of both 32-K blocks of row r (and
// that lane's scale operand is block h's): exactly the 16 + 16 keys whose P the lane has in its accumulators, so P goes from
// accumulators to the B fragment of the second product in registers with no data exchange at all. The transposed V stores the tokens
// of a block in the matching order.
#include <hip/hip_fp16.h>
#include "mx_dev.hpp"
#include "../../include/mi_attn.h"

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
#define HD AT_HD
#define FT 64            // keys per tile; sequences are padded to a multiple of it in the quantised tensors (rows past S are zero)

// Slot k of a 32-token block of the transposed V holds token a8_slot_token(k) of the block: slots 16 h + 4 q + c are lane half h's
// accumulator elements 4 q + c, which are the block's keys 8 q + 4 h + c.
__host__ __device__ __forceinline__ int a8_slot_token(int k) { return 8 * ((k >> 2) & 3) + 4 * (k >> 4) + (k & 3); }

// ---- operand quantisation (src/lp_attn8.cu:29-76): the fp16 head-major pack [3][H][Tp][48] -> e4m3 blocks of 32 with one E8M0 scale each ----
// q and k rows: dst [H][R][64] e4m3 + scales [H][R][2], R = nseq Sp rows (token i of sequence s in row s Sp + i, rows past S zero). A row's 64
// output bytes are four 16-byte quarters: dims 0-15 and 16-31 (block 0), 32-47 and sixteen zeros (block 1). Four neighbouring lanes own a row,
// each one quarter: 32 bytes of halves in (two 16-byte loads), 16 bytes of codes out, the block's amax through one exchange with the
// partner quarter. blockIdx.y: 0 the queries, 1 the keys.
__global__ void __launch_bounds__(256) a8_rows_k(const __half *__restrict__ src_q, uint8_t *__restrict__ dst_q, uint8_t *__restrict__ sc_q, int H, int nseq, int S, int Sp, long long Tp, size_t part_src, size_t part_dst, size_t part_sc) {
    const long long R = (long long)nseq * Sp, i = blockIdx.x * 256ll + threadIdx.x, hr = i >> 2;
    if (hr >= (long long)H * R) return;
    const int qt = (int)(i & 3), h = (int)(hr / R); const long long row = hr - (long long)h * R;
    const int seq = (int)(row / Sp), ii = (int)(row - (long long)seq * Sp);
    const __half *src = src_q + blockIdx.y * part_src; uint8_t *dst = dst_q + blockIdx.y * part_dst, *sc = sc_q + blockIdx.y * part_sc;
    float v[16];
#pragma unroll
    for (int k = 0; k < 16; k++) v[k] = 0.f;
    if (ii < S && qt < 3) {
        const uint4 *p = (const uint4 *)(src + ((size_t)h * Tp + (size_t)seq * S + ii) * HD + 16 * qt);
        const uint4 a = p[0], b = p[1];
        const unsigned w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int k = 0; k < 8; k++) { const __half2 hh = *(const __half2 *)&w[k]; v[2 * k] = __low2float(hh); v[2 * k + 1] = __high2float(hh); }
    }
    float am = 0.f;
#pragma unroll
    for (int k = 0; k < 16; k++) am = fmaxf(am, fabsf(v[k]));
    am = __uint_as_float(max(__float_as_uint(am), d_quad_xor_u<1>(__float_as_uint(am))));       // quarters (0, 1) and (2, 3) are the two blocks (am >= 0, never NaN: it orders as its bits; the four lanes of a row leave together)
    const int e = d_mx_exp(am, MI_INVQ8);
    *(uint4 *)(dst + (size_t)hr * 64 + 16 * qt) = make_uint4(d_enc4_e4m3(v[0], v[1], v[2], v[3], e), d_enc4_e4m3(v[4], v[5], v[6], v[7], e), d_enc4_e4m3(v[8], v[9], v[10], v[11], e), d_enc4_e4m3(v[12], v[13], v[14], v[15], e));
    if (!(qt & 1)) sc[(size_t)hr * 2 + (qt >> 1)] = (uint8_t)(e + 127);
}
// transposed v: dst [H][48][R] with the 32 tokens of a block in slot order + scales [H][48][R / 32]. One wavefront per (head, 32-token block),
// lane d < 48 owns dim d: it gathers the block's 32 values of its dim (each gather reads one token's 96 contiguous bytes across the lanes),
// quantises them as one block and writes 32 contiguous bytes.
__global__ void __launch_bounds__(256) a8_vt_k(const __half *__restrict__ src, uint8_t *__restrict__ dst, uint8_t *__restrict__ sc, int H, int nseq, int S, int Sp, long long Tp) {
    const long long R = (long long)nseq * Sp, nb = R / 32, wb = blockIdx.x * 4ll + (threadIdx.x >> 6);
    const int d = threadIdx.x & 63;
    if (wb >= (long long)H * nb || d >= HD) return;
    const int h = (int)(wb / nb); const long long b = wb - (long long)h * nb, r0 = b * 32;
    const int seq = (int)(r0 / Sp), i0 = (int)(r0 - (long long)seq * Sp);       // (Sp is a multiple of 64: a block never straddles two sequences)
    const __half *base = src + ((size_t)h * Tp + (size_t)seq * S) * HD + d;
    float v[32];
#pragma unroll
    for (int k = 0; k < 32; k++) { const int ii = i0 + a8_slot_token(k); v[k] = ii < S ? __half2float(base[(size_t)ii * HD]) : 0.f; }
    unsigned codes[8];
    const unsigned sb = d_quant_row<8, false>(v, 32, codes);
    uint4 *o = (uint4 *)(dst + ((size_t)h * HD + d) * R + r0);
    o[0] = make_uint4(codes[0], codes[1], codes[2], codes[3]); o[1] = make_uint4(codes[4], codes[5], codes[6], codes[7]);
    sc[((size_t)h * HD + d) * nb + b] = (uint8_t)sb;
}

__device__ __forceinline__ float a8_xor32f(float x, int h) {
    const unsigned u = __float_as_uint(x);
    const auto r2 = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(h ? r2[0] : r2[1]);
}
// the lane's fragment of a 64-byte row of two 32-K blocks: bytes 16 h ... of each (p already points at byte 16 h)
__device__ __forceinline__ v8i a8_frag(const uint8_t *p) {
    const v4i lo = *(const v4i *)p, hi = *(const v4i *)(p + 32);
    return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

// grid (ceil(S / (32 nw)), H, nseq), nw = 4 or 1 wavefronts of 32 queries each. Fragments are the quantised tensors' rows as they lie in memory
// (32 contiguous bytes per lane), loaded from global memory directly: a sequence's K and V of one head are 7 KB per 64 keys and stay in
// L2 / the vector cache across the workgroup's wavefronts.
__global__ void __launch_bounds__(256) a8_fwd_k(const uint8_t *__restrict__ Q8, const uint8_t *__restrict__ Q8s, const uint8_t *__restrict__ K8, const uint8_t *__restrict__ K8s,
                                                const uint8_t *__restrict__ Vt, const uint8_t *__restrict__ Vts, float *__restrict__ o, float *__restrict__ lse,
                                                int S, int Sp, int H, int C, long long R, float sl2) {
    const int seq = blockIdx.z, hd = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;
    const int nwv = blockDim.x >> 6, tq = blockIdx.x * nwv;
    // A four-wavefront workgroup whose first wavefront alone has queries (the sequence's last 32-query tile: the few tokens past a multiple
    // of 128) shares that tile's keys among its wavefronts, a range of the key tiles each, and wavefront 0 merges the four partial
    // softmaxes: the tile costs a third of a wavefront's full pass instead of one that the rest of the GPU waits for. Each wavefront starts
    // from the running maximum of the tiles before its range, so the probabilities and their e4m3 codes are those of the one-wavefront
    // pass; only the order in which the partial sums are added differs
    const bool split = nwv == 4 && (tq + 1) * 32 >= S;
    const int q0 = (split ? tq : tq + wave) * 32;
    if (q0 >= S) return;                                   // (no barriers outside a split workgroup: a wavefront without queries leaves)
    const long long rb = (long long)hd * R + (long long)seq * Sp;          // the sequence's first row in the row-quantised tensors
    const long long c0 = (long long)seq * Sp;                              // its first column in the transposed one
    const v8i qf = a8_frag(Q8 + (rb + q0 + r) * 64 + 16 * h);
    const int qs = Q8s[(rb + q0 + r) * 2 + h];
    const uint8_t *kp = K8 + (rb + r) * 64 + 16 * h, *ksp = K8s + (rb + r) * 2 + h;
    // V^T rows: dims r and 32 + r (the second tile has 16 real rows; the others multiply zeros)
    const int d1 = min(32 + r, HD - 1); const bool d1ok = 32 + r < HD;
    const uint8_t *vp0 = Vt + ((size_t)hd * HD + r) * R + c0 + 16 * h, *vp1 = Vt + ((size_t)hd * HD + d1) * R + c0 + 16 * h;
    const uint8_t *vs0 = Vts + ((size_t)hd * HD + r) * (R / 32) + c0 / 32 + h, *vs1 = Vts + ((size_t)hd * HD + d1) * (R / 32) + c0 / 32 + h;
    float m = -INFINITY, l = 0.f;
    v16f oa[2];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) oa[t][i] = 0.f;
    const int nt = (S + FT - 1) / FT;
    // (split: later ranges are shorter, since their wavefronts first look through the earlier tiles for the running maximum)
    const int cut[5] = {0, nt * 34 / 100, nt * 61 / 100, nt * 83 / 100, nt};
    const int it0 = split ? cut[wave] : 0, it1 = split ? cut[wave + 1] : nt;
    // The K and V fragments of tile it + 1 are requested before tile it is worked on: with one or a few wavefronts per SIMD nothing else hides
    // the L2 latency of a tile's loads. (The last iteration re-requests its own tile.)
    v8i kfn[2], vfn[2]; int ksn[2], evn[2];
    auto request = [&](int it) {
        const int kb = it * FT;
#pragma unroll
        for (int b = 0; b < 2; b++) { kfn[b] = a8_frag(kp + (size_t)(kb + 32 * b) * 64); ksn[b] = ksp[(size_t)(kb + 32 * b) * 2]; }
        vfn[0] = a8_frag(vp0 + kb); vfn[1] = a8_frag(vp1 + kb);
        evn[0] = vs0[kb / 32]; evn[1] = vs1[kb / 32];
    };
    if (split && it0 > 0) {
        // the running maximum the single-wavefront pass holds when it reaches tile it0: the logits of the tiles before it (the two products
        // and the scaling of the main loop, nothing else), so that every probability of this range is the value that pass computes
        v8i kq[2]; int kqs[2];
        auto reqk = [&](int it) {
#pragma unroll
            for (int b = 0; b < 2; b++) { kq[b] = a8_frag(kp + (size_t)(it * FT + 32 * b) * 64); kqs[b] = ksp[(size_t)(it * FT + 32 * b) * 2]; }
        };
        reqk(0);
        float mx = -INFINITY;
        for (int it = 0; it < it0; it++) {
            const v8i kf[2] = {kq[0], kq[1]}; const int ks[2] = {kqs[0], kqs[1]};
            reqk(min(it + 1, it0 - 1));
#pragma unroll
            for (int b = 0; b < 2; b++) {
                v16f z;
#pragma unroll
                for (int i = 0; i < 16; i++) z[i] = 0.f;
                const v16f sb = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf[b], qf, z, 0, 0, 0, ks[b], 0, qs);
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int key = it * FT + 32 * b + (i & 3) + 4 * h + 8 * (i >> 2);
                    mx = fmaxf(mx, key < S ? sb[i] * sl2 : -INFINITY);
                }
            }
        }
        m = fmaxf(mx, a8_xor32f(mx, h));
    }
    request(min(it0, nt - 1));
    for (int it = it0; it < it1; it++) {
        const int kb = it * FT;
        const v8i kf[2] = {kfn[0], kfn[1]}; const int ks[2] = {ksn[0], ksn[1]};
        v8i vf0 = vfn[0], vf1 = vfn[1];
        const int e0v = evn[0], e1v = evn[1];
        request(min(it + 1, nt - 1));
        // ---- S^T = K Q^T for the tile's two blocks of 32 keys ----
        v16f s[2];
#pragma unroll
        for (int b = 0; b < 2; b++) {
            v16f z;
#pragma unroll
            for (int i = 0; i < 16; i++) z[i] = 0.f;
            s[b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kf[b], qf, z, 0, 0, 0, ks[b], 0, qs);
        }
        if (!d1ok) vf1 = (v8i){0, 0, 0, 0, 0, 0, 0, 0};
        // ---- logits in base-2 units, keys past S masked (only the last tile can hold them) ----
        const bool full = kb + FT <= S;
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) s[b][i] *= sl2;
        if (!full) {                                       // (uniform: no per-element key test on the tiles before the last)
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int i = 0; i < 16; i++) { const int key = kb + 32 * b + (i & 3) + 4 * h + 8 * (i >> 2); if (key >= S) s[b][i] = -INFINITY; }
        }
        float mx = -INFINITY;
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) mx = fmaxf(mx, s[b][i]);
        mx = fmaxf(mx, a8_xor32f(mx, h));
        const float mn = fmaxf(m, mx), corr = __builtin_amdgcn_exp2f(m - mn);
        m = mn; l *= corr;
        float am[2] = {0.f, 0.f};
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) { const float p = __builtin_amdgcn_exp2f(s[b][i] - m); s[b][i] = p; l += p; am[b] = fmaxf(am[b], p); }
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) oa[t][i] *= corr;
        // ---- P -> e4m3 with one scale per query per 32 keys; the lane's codes are its B fragment, its scale operand is block h's ----
        unsigned cw[2][4]; int ep[2];
#pragma unroll
        for (int b = 0; b < 2; b++) {
            am[b] = fmaxf(am[b], a8_xor32f(am[b], h));
            ep[b] = d_mx_exp(am[b], MI_INVQ8);
            const float p2e = d_exp2i(ep[b]);
#pragma unroll
            for (int q = 0; q < 4; q++) cw[b][q] = d_enc_e4m3x4_hw(s[b][4 * q], s[b][4 * q + 1], s[b][4 * q + 2], s[b][4 * q + 3], p2e);
        }
        const v8i pf = {(int)cw[0][0], (int)cw[0][1], (int)cw[0][2], (int)cw[0][3], (int)cw[1][0], (int)cw[1][1], (int)cw[1][2], (int)cw[1][3]};
        const int ps = (h ? ep[1] : ep[0]) + 127;
        // ---- O^T += V^T P^T ----
        oa[0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf0, pf, oa[0], 0, 0, 0, e0v, 0, ps);
        oa[1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(vf1, pf, oa[1], 0, 0, 0, e1v, 0, ps);
    }
    l += a8_xor32f(l, h);
    if (split) {
        // partial (m, l, O^T) of the four key ranges -> LDS [wavefront][value][lane]; wavefront 0 adds them in wavefront order at the common
        // maximum (a wavefront without keys holds m = -inf, l = 0, O = 0: its factor is 0)
        extern __shared__ float cmb[];
        float *mine = cmb + (size_t)wave * 34 * 64 + lane;
        mine[0] = m; mine[64] = l;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int k = 0; k < 16; k++) mine[(2 + 16 * t + k) * 64] = oa[t][k];
        __syncthreads();
        if (wave) return;
        float mm = m;
#pragma unroll
        for (int w = 1; w < 4; w++) mm = fmaxf(mm, cmb[(size_t)w * 34 * 64 + lane]);
        float ls = 0.f;
        v16f os[2];
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int k = 0; k < 16; k++) os[t][k] = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float *pw = cmb + (size_t)w * 34 * 64 + lane;
            const float f = __builtin_amdgcn_exp2f(pw[0] - mm);
            ls = fmaf(pw[64], f, ls);
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int k = 0; k < 16; k++) os[t][k] = fmaf(pw[(2 + 16 * t + k) * 64], f, os[t][k]);
        }
        m = mm; l = ls; oa[0] = os[0]; oa[1] = os[1];
    }
    const int i = q0 + r;
    if (i >= S) return;
    const float il = 1.f / l;
    float *orow = o + ((size_t)seq * S + i) * C + hd * HD;
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int d0 = 32 * t + 4 * h + 8 * g;         // accumulator elements 4 g ... 4 g + 3: dims d0 ... d0 + 3
            if (d0 < HD) *(float4 *)(orow + d0) = make_float4(oa[t][4 * g] * il, oa[t][4 * g + 1] * il, oa[t][4 * g + 2] * il, oa[t][4 * g + 3] * il);
        }
    if (!h) lse[((size_t)seq * H + hd) * S + i] = m + __log2f(l);
}

static int g_a8_waves = 0;
extern "C" void at_fa8_waves(int nw) { g_a8_waves = nw == 1 || nw == 4 ? nw : 0; }
extern "C" int at_fa8_fwd(const void *qkvh, float *o, float *lse, const at_geom *g, int H, int C) {
    if (!g || g->nseq <= 0 || g->S <= 0 || H <= 0) return 0;
    if (C != H * HD) mi_die("at_fa8_fwd: C %d is not %d heads of %d", C, H, HD);
    if (g->lens || g->rays) mi_die("at_fa8_fwd: per-sequence lengths and ray geometry are not supported");
    const long long T = (long long)g->nseq * g->S, Tp = T + FT; const int Sp = (g->S + FT - 1) / FT * FT; const long long R = (long long)g->nseq * Sp;
    const size_t rq = (size_t)H * R * 64, rqs = (size_t)H * R * 2, tq = (size_t)H * HD * R, tqs = (size_t)H * HD * (R / 32);
    auto al = [](size_t n) { return (n + 255) & ~(size_t)255; };
    uint8_t *base = (uint8_t *)mi_ws(MI_WS_ATTN, 2 * (al(rq) + al(rqs)) + al(tq) + al(tqs));
    if (!base) return -1;
    uint8_t *q8 = base, *k8 = q8 + al(rq), *qs = k8 + al(rq), *ks = qs + al(rqs), *vt = ks + al(rqs), *vts = vt + al(tq);
    const __half *Qh = (const __half *)qkvh, *Kh = Qh + (size_t)H * Tp * HD, *Vh = Kh + (size_t)H * Tp * HD;
    // (queries and keys in one launch: their sources, code planes and scale planes each lie one fixed stride apart)
    a8_rows_k<<<dim3(nblk_((size_t)H * R * 4, 256), 2), 256>>>(Qh, q8, qs, H, g->nseq, g->S, Sp, Tp, (size_t)(Kh - Qh), (size_t)(k8 - q8), (size_t)(ks - qs));
    a8_vt_k<<<nblk_((size_t)H * (R / 32), 4), 256>>>(Vh, vt, vts, H, g->nseq, g->S, Sp, Tp);
    // few query tiles (a 16^3 bottleneck: 129 per head): one wavefront per workgroup, so that every CU gets some
    const int nw = g_a8_waves ? g_a8_waves : (size_t)((g->S + 127) / 128) * H * g->nseq >= 512 ? 4 : 1;
    const dim3 grid((unsigned)((g->S + 32 * nw - 1) / (32 * nw)), (unsigned)H, (unsigned)g->nseq);
    a8_fwd_k<<<grid, 64 * nw, nw == 4 ? 4 * 34 * 64 * sizeof(float) : 0>>>(q8, qs, k8, ks, vt, vts, o, lse, g->S, Sp, H, C, R, 1.4426950408889634f / sqrtf((float)HD));
    MICK();
    return 0;
}
