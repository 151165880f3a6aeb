// MX GEMM of row-major fp32 operands (the attention stage's linear layers): both operands are quantised along K once, into block rows
// that are MFMA fragments as they lie in memory, then a block-scaled MFMA GEMM runs over the packed bytes.
// Interface and arithmetic: src/lp_mxgemm.cu:1-5 (definition), :88-113 (packing), :266-297 (entry points) of the reference.
#include <vector>
#include <mutex>
#include "mx_dev.hpp"
#include "../../include/mi_attn.h"

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

// one thread per (row, 32-K block): X is [rows][K] (TR 0; ld = row stride) or [K][rows] (TR 1). Packed row r = nkb blocks of BPB bytes
// (K past the operand's K is zero), scales [rows][nkb]. TR: neighbouring threads take neighbouring rows (contiguous reads of each K row).
template <int BITS, int TR>
__global__ void __launch_bounds__(256) mx_pack_k(const float *__restrict__ X, int ld, int rows, int K, int nkb, uint8_t *__restrict__ q, uint8_t *__restrict__ sc) {
    constexpr int BPB = BITS == 8 ? 32 : 16;
    const long long nblk = (long long)rows * nkb;
    const bool v4 = (ld & 3) == 0 && ((size_t)X & 15) == 0;     // rows start on 16 bytes
    for (long long b = blockIdx.x * (long long)blockDim.x + threadIdx.x; b < nblk; b += (long long)gridDim.x * blockDim.x) {
        const int r = TR ? (int)(b % rows) : (int)(b / nkb), kb = TR ? (int)(b / rows) : (int)(b % nkb);
        float v[32];
        if (!TR && v4 && kb * 32 + 32 <= K) {                // a whole block of a row-major operand: eight 16-byte loads (a lane's 128 bytes are contiguous)
            const float4 *p4 = (const float4 *)(X + (size_t)r * ld + kb * 32);
#pragma unroll
            for (int j = 0; j < 8; j++) { const float4 t = p4[j]; v[4 * j] = t.x; v[4 * j + 1] = t.y; v[4 * j + 2] = t.z; v[4 * j + 3] = t.w; }
        } else {
#pragma unroll
            for (int j = 0; j < 32; j++) { const int k = kb * 32 + j; v[j] = k < K ? (TR ? X[(size_t)k * ld + r] : X[(size_t)r * ld + k]) : 0.f; }
        }
        unsigned codes[8];
        const unsigned sb = d_quant_row<BITS, false>(v, 32, codes);
        uint8_t *o = q + ((size_t)r * nkb + kb) * BPB;
        *(uint4 *)o = make_uint4(codes[0], codes[1], codes[2], codes[3]);
        if (BITS == 8) *(uint4 *)(o + 16) = make_uint4(codes[4], codes[5], codes[6], codes[7]);
        sc[(size_t)r * nkb + kb] = (uint8_t)sb;
    }
}

// mx_pack_k<8, 0> for a row-major operand whose K is a multiple of 64 and whose rows start on 16 bytes: a thread takes one float4 of a row (a
// wavefront reads 1 KiB contiguous instead of 64 runs of 128 bytes), the block of 32 values is eight neighbouring lanes' and their maxima meet
// through three lane exchanges; the same maximum, exponent and codes
__global__ void __launch_bounds__(256) mx_pack8_rows_k(const float4 *__restrict__ X, int ld4, size_t n4, unsigned K4, uint8_t *__restrict__ q, uint8_t *__restrict__ sc) {
    const size_t i = blockIdx.x * (size_t)256 + threadIdx.x;
    if (i >= n4) return;                                   // (n4 is a multiple of 8: the lanes of a group of eight leave together)
    const size_t r = i / K4; const unsigned k = (unsigned)(i - r * K4);
    const float4 o = X[r * ld4 + k];
    unsigned au = __float_as_uint(fmaxf(fmaxf(fabsf(o.x), fabsf(o.y)), fmaxf(fabsf(o.z), fabsf(o.w))));       // (fmaxf drops NaN; a non-negative number orders as its bits)
    au = max(au, d_quad_xor_u<1>(au)); au = max(au, d_quad_xor_u<2>(au));
    au = max(au, d_oct_mirror_u(au));
    const int e = d_mx_exp(__uint_as_float(au), MI_INVQ8);
    *(unsigned *)(q + i * 4) = d_enc4_e4m3(o.x, o.y, o.z, o.w, e);
    if (!(k & 7)) sc[i >> 3] = (uint8_t)(e + 127);
}

__global__ void gemm_zero_k(float *c, size_t n) {
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) c[i] = 0.f;
}

// C tile of 64 x 256 per workgroup (four wavefronts side by side along N), 64 x 64 per wavefront = 2 x 2 MFMA tiles of 32 x 32; K in steps of 64 = the two 32-K blocks the
// scale operands of the lane halves of a 32x32x64 MFMA cover. A lane's fragment is 16 bytes of each of the two blocks (e4m3: bytes
// 16 h ... of both; e2m1: all 16 bytes of block h), so fragments are loaded from the packed rows in global memory directly: the four
// wavefronts of a workgroup read the same A rows through the vector cache.
// gridDim.z > 1: split K, each split adds its part into C atomically (C zeroed or kept by the host; no bias / residual then).
template <int BITS>
__global__ void __launch_bounds__(256) mx_gemm_k(const uint8_t *__restrict__ Aq, const uint8_t *__restrict__ As, const uint8_t *__restrict__ Bq, const uint8_t *__restrict__ Bs,
                                                 float *C, int M, int N, int nkb, float beta, const float *__restrict__ bias, const float *res, int sper) {
    constexpr int BPB = BITS == 8 ? 32 : 16, FM = BITS == 8 ? 0 : 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;
    // a wavefront owns a 64 x 64 tile; a workgroup is four of them in a row, or a single one (few tiles: more workgroups than CUs that way)
    // (four wavefronts: side by side along N, so the workgroup writes runs of 1 KiB of a C row and shares its A rows)
    const int wn = blockDim.x >> 6;
    const int m0 = blockIdx.y * 64, n0 = (blockIdx.x * wn + wave) * 64;
    if (m0 >= M || n0 >= N) return;                        // (no barriers in this kernel: a wavefront without work leaves)
    const int nst = nkb >> 1, s0 = (int)blockIdx.z * sper, s1 = min(nst, s0 + sper);
    const uint8_t *pa[2], *pb[2], *sa[2], *sb[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const size_t ra = (size_t)min(m0 + 32 * i + r, M - 1), rb = (size_t)min(n0 + 32 * i + r, N - 1);       // rows past the edge repeat the last one (never stored)
        pa[i] = Aq + ra * nkb * BPB + 16 * h; sa[i] = As + ra * nkb + h;         // (e2m1: + 16 h is block h of a step; e4m3: the lane's half of both blocks)
        pb[i] = Bq + rb * nkb * BPB + 16 * h; sb[i] = Bs + rb * nkb + h;
    }
    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int q = 0; q < 16; q++) acc[i][j][q] = 0.f;
    auto frag = [&](const uint8_t *p) {
        const v4i lo = *(const v4i *)p;
        if (BITS == 8) { const v4i hi = *(const v4i *)(p + 32); return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]}; }
        return (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
    };
    // the fragments of step s + 1 are requested before the MFMAs of step s (rows are read straight from global memory / L2)
    v8i fa[2], fb[2]; int ea[2], eb[2];
    auto load = [&](int s) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            fa[i] = frag(pa[i] + (size_t)s * 2 * BPB); ea[i] = sa[i][2 * s];
            fb[i] = frag(pb[i] + (size_t)s * 2 * BPB); eb[i] = sb[i][2 * s];
        }
    };
    if (s0 < s1) load(s0);
    for (int s = s0; s < s1; s++) {
        v8i ca[2] = {fa[0], fa[1]}, cb[2] = {fb[0], fb[1]}; const int xa[2] = {ea[0], ea[1]}, xb[2] = {eb[0], eb[1]};
        if (s + 1 < s1) load(s + 1);
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ca[i], cb[j], acc[i][j], FM, FM, 0, xa[i], 0, xb[j]);
    }
    // accumulator element q of lane (r, h): row (q & 3) + 4 h + 8 (q >> 2), column r of its 32 x 32 tile
    const bool split = gridDim.z > 1;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int col = n0 + 32 * j + r;
            if (col >= N) continue;
            const float bv = bias ? bias[col] : 0.f;
            // the tile's 16 residual and 16 old values are read first, then everything is stored: C and res may be the same array, so a load
            // written after a store could not be moved above it, and 64 dependent round trips to memory were most of this kernel's time
            float add[16];
#pragma unroll
            for (int q = 0; q < 16; q++) add[q] = bv;
            if (res && !split) {                                // (uniform)
#pragma unroll
                for (int q = 0; q < 16; q++) add[q] += res[(size_t)min(m0 + 32 * i + (q & 3) + 4 * h + 8 * (q >> 2), M - 1) * N + col];
            }
            if (beta != 0.f && !split) {                        // (uniform)
#pragma unroll
                for (int q = 0; q < 16; q++) add[q] += beta * C[(size_t)min(m0 + 32 * i + (q & 3) + 4 * h + 8 * (q >> 2), M - 1) * N + col];
            }
#pragma unroll
            for (int q = 0; q < 16; q++) {
                const int row = m0 + 32 * i + (q & 3) + 4 * h + 8 * (q >> 2);
                if (row >= M) continue;
                float *p = C + (size_t)row * N + col;
                if (split) atomicAdd(p, acc[i][j][q]); else *p = acc[i][j][q] + add[q];
            }
        }
}

// Packed form of operand B kept across calls (inference: B is a weight matrix that does not change): keyed by pointer and shape, on by
// lp_mx_gemm_bmemo(1) for the calling thread, dropped by lp_wmemo_clear() like the convs' prepared weights.
struct bmemo_t { const float *B; int bits, tb, N, K, dev; uint8_t *q, *s; };
static std::vector<bmemo_t> g_bmemo;
static std::mutex g_bmemo_mu;
static thread_local int g_bmemo_on = 0;
extern "C" void lp_mx_gemm_bmemo(int on) { g_bmemo_on = on != 0; }
void mx_gemm_memo_clear(void) {
    std::lock_guard<std::mutex> lk(g_bmemo_mu);
    for (auto &m : g_bmemo) { MIRT(hipFree(m.q)); MIRT(hipFree(m.s)); }
    g_bmemo.clear();
}

// the workspace of one product: packed rows and scales of both operands (the same carving for every call of one shape)
struct gemm_ws_t { uint8_t *Aq, *Bq, *As, *Bs; int nkb; };
static bool gemm_ws(int bits, int M, int N, int K, gemm_ws_t *w) {
    const int nkb = (K + 63) / 64 * 2, BPB = bits == 8 ? 32 : 16;         // 32-K blocks of the packed rows (K rounded up to 64)
    const size_t qa = (size_t)M * nkb * BPB, qb = (size_t)N * nkb * BPB, sa = (size_t)M * nkb, sb = (size_t)N * nkb;
    auto al = [](size_t n) { return (n + 255) & ~(size_t)255; };
    uint8_t *base = (uint8_t *)mi_ws(MI_WS_GEMM, al(qa) + al(qb) + al(sa) + al(sb) + 256);
    if (!base) return false;
    w->Aq = base; w->Bq = w->Aq + al(qa); w->As = w->Bq + al(qb); w->Bs = w->As + al(sa); w->nkb = nkb;
    return true;
}
// (internal) where a kernel that produces A's rows quantises them itself, instead of writing fp32 rows for mx_pack_k to read back: the packed
// rows of A of the product (M, N, K) that mi_mx_gemm_apacked then runs, in mx_pack_k<bits, 0>'s layout: codes [M][K / 32][32 (e4m3) or 16 (e2m1)
// bytes], scales [M][K / 32]. K must be a multiple of 64 (no padding blocks)
bool mi_mx_gemm_abuf(int bits, int M, int N, int K, uint8_t **Aq, uint8_t **As) {
    gemm_ws_t w;
    if ((bits != 4 && bits != 8) || M <= 0 || N <= 0 || K <= 0 || K % 64 || !gemm_ws(bits, M, N, K, &w)) return false;
    *Aq = w.Aq; *As = w.As;
    return true;
}
// B's packed rows and scales for a product (M, N, K): the memoised copy when the memo is on (packed on its first use), else packed into the
// call's workspace
static void gemm_b_operand(int bits, int tb, int N, int K, const float *B, const gemm_ws_t &ws, uint8_t **Bq_, uint8_t **Bs_) {
    const int nkb = ws.nkb, BPB = bits == 8 ? 32 : 16, ldb = tb ? K : N;
    const size_t qb = (size_t)N * nkb * BPB, sb = (size_t)N * nkb;
    auto al = [](size_t n) { return (n + 255) & ~(size_t)255; };
    uint8_t *Bq = ws.Bq, *Bs = ws.Bs;
    bool bhave = false;
    if (g_bmemo_on && nkb) {
        int dev = 0; MIRT(hipGetDevice(&dev));
        std::lock_guard<std::mutex> lk(g_bmemo_mu);
        for (auto &m : g_bmemo) if (m.B == B && m.bits == bits && m.tb == tb && m.N == N && m.K == K && m.dev == dev) { Bq = m.q; Bs = m.s; bhave = true; break; }
        if (!bhave) {
            uint8_t *q = nullptr, *sc = nullptr;
            MIRT(hipMalloc((void **)&q, al(qb))); MIRT(hipMalloc((void **)&sc, al(sb)));
            if (q && sc) { g_bmemo.push_back(bmemo_t{B, bits, tb, N, K, dev, q, sc}); Bq = q; Bs = sc; }     // (packed below, found by the next call)
        }
    }
    if (nkb && !bhave) {
        const unsigned gb = nblk_((size_t)N * nkb, 256);
        if (bits == 8) { if (tb) mx_pack_k<8, 0><<<gb, 256>>>(B, ldb, N, K, nkb, Bq, Bs); else mx_pack_k<8, 1><<<gb, 256>>>(B, ldb, N, K, nkb, Bq, Bs); }
        else { if (tb) mx_pack_k<4, 0><<<gb, 256>>>(B, ldb, N, K, nkb, Bq, Bs); else mx_pack_k<4, 1><<<gb, 256>>>(B, ldb, N, K, nkb, Bq, Bs); }
    }
    *Bq_ = Bq; *Bs_ = Bs;
}
static int gemm_impl(int bits, int ta, int tb, int M, int N, int K, const float *A, const float *B, float *C, float beta, const float *bias, const float *res, bool apacked,
                     const uint8_t *Aq_at = nullptr, const uint8_t *As_at = nullptr) {
    if (bits != 4 && bits != 8) return -1;
    if (M <= 0 || N <= 0) return 0;
    if (K < 0) K = 0;
    gemm_ws_t ws;
    if (!gemm_ws(bits, M, N, K, &ws)) return -1;
    const int nkb = ws.nkb;
    const uint8_t *Aq = Aq_at ? Aq_at : ws.Aq, *As = As_at ? As_at : ws.As;
    uint8_t *Bq, *Bs;
    const int lda = ta ? M : K;
    gemm_b_operand(bits, tb, N, K, B, ws, &Bq, &Bs);
    if (nkb && !apacked) {
        const unsigned ga = nblk_((size_t)M * nkb, 256);
        if (bits == 8) {
            if (ta) mx_pack_k<8, 1><<<ga, 256>>>(A, lda, M, K, nkb, ws.Aq, ws.As);
            else if (K % 64 == 0 && (lda & 3) == 0 && ((size_t)A & 15) == 0) { const size_t n4 = (size_t)M * (K / 4); mx_pack8_rows_k<<<nblk_(n4, 256), 256>>>((const float4 *)A, lda / 4, n4, (unsigned)(K / 4), ws.Aq, ws.As); }
            else mx_pack_k<8, 0><<<ga, 256>>>(A, lda, M, K, nkb, ws.Aq, ws.As);
        } else { if (ta) mx_pack_k<4, 1><<<ga, 256>>>(A, lda, M, K, nkb, ws.Aq, ws.As); else mx_pack_k<4, 0><<<ga, 256>>>(A, lda, M, K, nkb, ws.Aq, ws.As); }
    }
    // few output tiles and a long K (the weight-gradient shape, src/lp_mxgemm.cu:259-265): split K so the GPU's 256 CUs have work
    const int tiles = ((N + 127) / 128) * ((M + 127) / 128), nst = nkb / 2;
    int ns = !bias && !res && (beta == 0.f || beta == 1.f) && tiles < 128 ? (256 + tiles - 1) / tiles : 1;
    if (ns > nst / 4) ns = nst / 4 > 1 ? nst / 4 : 1;
    const int sper = ns > 1 ? (nst + ns - 1) / ns : (nst > 0 ? nst : 1);
    ns = nst > 0 ? (nst + sper - 1) / sper : 1;
    if (ns > 1 && beta == 0.f) gemm_zero_k<<<nblk_((size_t)M * N, 256 * 4), 256>>>(C, (size_t)M * N);   // (a kernel, not a memset node: safe under graph capture)
    const int wt = (size_t)tiles * ns >= 512 ? 2 : 1;              // (few tiles: one wavefront per workgroup)
    const int wn = wt == 2 ? 4 : 1;                                // wavefronts per workgroup, side by side along N
    const dim3 grid((unsigned)((N + 64 * wn - 1) / (64 * wn)), (unsigned)((M + 63) / 64), (unsigned)ns);
    if (bits == 8) mx_gemm_k<8><<<grid, 64 * wn>>>(Aq, As, Bq, Bs, C, M, N, nkb, beta, bias, res, sper);
    else mx_gemm_k<4><<<grid, 64 * wn>>>(Aq, As, Bq, Bs, C, M, N, nkb, beta, bias, res, sper);
    MICK();
    return 0;
}
extern "C" int lp_mx_gemm_ex(int bits, int ta, int tb, int M, int N, int K, const float *A, const float *B, float *C, float beta, const float *bias, const float *res) {
    return gemm_impl(bits, ta, tb, M, N, K, A, B, C, beta, bias, res, false);
}
// (internal) lp_mx_gemm_ex with A's rows already packed where mi_mx_gemm_abuf said
int mi_mx_gemm_apacked(int bits, int tb, int M, int N, int K, const float *B, float *C, float beta, const float *bias, const float *res) {
    if (K <= 0 || K % 64) return -1;
    return gemm_impl(bits, 0, tb, M, N, K, nullptr, B, C, beta, bias, res, true);
}
int mi_mx_gemm_apacked_at(int bits, int tb, int M, int N, int K, const uint8_t *Aq, const uint8_t *As, const float *B, float *C, float beta, const float *bias, const float *res) {
    if (K <= 0 || K % 64 || !Aq || !As) return -1;
    return gemm_impl(bits, 0, tb, M, N, K, nullptr, B, C, beta, bias, res, true, Aq, As);
}
// ---- the MLP's up projection with the SwiGLU in its epilogue (e4m3 operands): g[t][f] = silu(h[t][f]) h[t][F + f], h = x W^T + b ----
// The product is formed transposed, h^T = W x^T, so a token is a COLUMN of the accumulators: lane (r, h) holds, for token r of its wavefront's 32,
// features (q & 3) + 4 h + 8 (q >> 2) of a 32-feature tile in element q - of the gate rows W[f] and of the value rows W[F + f] in two accumulators.
// gate and value of one (token, feature) then sit in the same element of the same lane, the block of 32 features that the down projection's
// operand quantises together is the lane's 16 values and its partner lane's (r, h ^ 1) 16: one lane exchange for the maximum, two for handing
// each lane a contiguous half of the block's 32 codes. The 1 GB of h that a 61-window forward wrote and read back is never stored.
// A wavefront keeps the operand fragments of its 64 tokens in registers (NST steps of 64 channels) and walks feature tiles; the weights' fragments
// come from L2 (196 KB for 1024 x 192), each serving both token tiles (with one token tile per wavefront the launch was bound by that traffic). The same MFMA steps in the same order on the same operand bytes as mx_gemm_k's, bias added and SwiGLU formed by the
// expressions of the separate kernels.
template <int NST>
__global__ void __launch_bounds__(256) glu_gemm_k(const uint8_t *__restrict__ Xq, const uint8_t *__restrict__ Xs, const uint8_t *__restrict__ Wq, const uint8_t *__restrict__ Ws,
                                                  const float *__restrict__ bias, uint8_t *__restrict__ gq, uint8_t *__restrict__ gs, int T, int F, int tiles_per_y) {
    extern __shared__ __align__(16) float sbias[];           // [2 F]: the bias vector sits at an arbitrary offset of the parameter array; LDS reads are 16-byte ones
    constexpr int nkb = 2 * NST, TT = 2;                     // TT: token tiles of 32 per wavefront (a weight fragment fetched from L2 serves both)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;
    for (int i = tid; i < 2 * F; i += 256) sbias[i] = bias ? bias[i] : 0.f;
    __syncthreads();
    const int t0 = (blockIdx.x * 4 + wave) * 32 * TT;
    if (t0 >= T) return;                                   // (no barrier below)
    auto frag = [&](const uint8_t *p) {
        const v4i lo = *(const v4i *)p, hi = *(const v4i *)(p + 32);
        return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    size_t tr[TT];                                         // (tokens past the end repeat the last one and store nothing)
    v8i fx[TT][NST]; int ex[TT][NST];
#pragma unroll
    for (int u = 0; u < TT; u++) {
        tr[u] = (size_t)min(t0 + 32 * u + r, T - 1);
#pragma unroll
        for (int s = 0; s < NST; s++) { fx[u][s] = frag(Xq + tr[u] * nkb * 32 + s * 64 + 16 * h); ex[u][s] = Xs[tr[u] * nkb + 2 * s + h]; }
    }
    const int nft = F / 32, ft0 = blockIdx.y * tiles_per_y, ft1 = min(nft, ft0 + tiles_per_y);
    for (int ft = ft0; ft < ft1; ft++) {
        const int f0 = ft * 32;
        const uint8_t *pa = Wq + (size_t)(f0 + r) * nkb * 32 + 16 * h, *pb = Wq + (size_t)(F + f0 + r) * nkb * 32 + 16 * h;
        const uint8_t *sa = Ws + (size_t)(f0 + r) * nkb + h, *sb = Ws + (size_t)(F + f0 + r) * nkb + h;
        v8i fa[NST], fb[NST]; int ea[NST], eb[NST];
#pragma unroll
        for (int s = 0; s < NST; s++) { fa[s] = frag(pa + s * 64); ea[s] = sa[2 * s]; fb[s] = frag(pb + s * 64); eb[s] = sb[2 * s]; }
        v16f ca[TT], cb[TT];
#pragma unroll
        for (int u = 0; u < TT; u++)
#pragma unroll
            for (int q = 0; q < 16; q++) { ca[u][q] = 0.f; cb[u][q] = 0.f; }
#pragma unroll
        for (int s = 0; s < NST; s++)
#pragma unroll
            for (int u = 0; u < TT; u++) {
                ca[u] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[s], fx[u][s], ca[u], 0, 0, 0, ea[s], 0, ex[u][s]);
                cb[u] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[s], fx[u][s], cb[u], 0, 0, 0, eb[s], 0, ex[u][s]);
            }
#pragma unroll
        for (int u = 0; u < TT; u++) {
            float v[16], am = 0.f;
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float4 ba = *(const float4 *)(sbias + f0 + 8 * g + 4 * h), bb = *(const float4 *)(sbias + F + f0 + 8 * g + 4 * h);
                const float a4[4] = {ca[u][4 * g] + ba.x, ca[u][4 * g + 1] + ba.y, ca[u][4 * g + 2] + ba.z, ca[u][4 * g + 3] + ba.w};
                const float b4[4] = {cb[u][4 * g] + bb.x, cb[u][4 * g + 1] + bb.y, cb[u][4 * g + 2] + bb.z, cb[u][4 * g + 3] + bb.w};
#pragma unroll
                for (int c = 0; c < 4; c++) { v[4 * g + c] = d_silu(a4[c]) * b4[c]; am = fmaxf(am, fabsf(v[4 * g + c])); }
            }
            {   // the other half of the block is the partner lane's (am is a non-negative number: it orders as its bits)
                const unsigned w = __float_as_uint(am);
                const auto r2 = __builtin_amdgcn_permlane32_swap(w, w, false, false);
                am = __uint_as_float(max(r2[0], r2[1]));
            }
            const int e = d_mx_exp(am, MI_INVQ8);
            unsigned d[4];
#pragma unroll
            for (int g = 0; g < 4; g++) d[g] = d_enc4_e4m3(v[4 * g], v[4 * g + 1], v[4 * g + 2], v[4 * g + 3], e);
            // word g of half h is word 2 g + h of the block's eight: half 0 keeps its words 0, 1 and takes the partner's, half 1 keeps its words 2, 3
            const auto s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false), s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
            if (t0 + 32 * u + r < T) {
                *(uint4 *)(gq + (tr[u] * nft + ft) * 32 + 16 * h) = make_uint4(s02[0], s02[1], s13[0], s13[1]);
                if (!h) gs[tr[u] * nft + ft] = (uint8_t)(e + 127);
            }
        }
    }
}
int mi_mx_gemm_glu(int T, int F, int C, const float *W, const float *bias, uint8_t *gq, uint8_t *gs) {
    if (T <= 0 || F <= 0 || C <= 0 || C % 64 || C > 256 || F % 32 || !gq || !gs) return -1;
    gemm_ws_t ws;
    if (!gemm_ws(8, T, 2 * F, C, &ws)) return -1;          // (x's packed rows lie where mi_mx_gemm_abuf(8, T, 2 F, C) said)
    uint8_t *Wq, *Wsc;
    gemm_b_operand(8, 1, 2 * F, C, W, ws, &Wq, &Wsc);
    // feature tiles per workgroup row: all of them when the token tiles alone fill the GPU, else split so that about 2 048 wavefronts run
    const int nft = F / 32, ntt = (T + 255) / 256;         // (a workgroup: four wavefronts of 64 tokens)
    int ny = 1; while (ny < nft && (size_t)ntt * 4 * ny < 2048) ny *= 2;
    const int tpy = (nft + ny - 1) / ny;
    const dim3 grid((unsigned)ntt, (unsigned)((nft + tpy - 1) / tpy));
    const size_t sm = (size_t)2 * F * sizeof(float);
    switch (C / 64) {
        case 1: glu_gemm_k<1><<<grid, 256, sm>>>(ws.Aq, ws.As, Wq, Wsc, bias, gq, gs, T, F, tpy); break;
        case 2: glu_gemm_k<2><<<grid, 256, sm>>>(ws.Aq, ws.As, Wq, Wsc, bias, gq, gs, T, F, tpy); break;
        case 3: glu_gemm_k<3><<<grid, 256, sm>>>(ws.Aq, ws.As, Wq, Wsc, bias, gq, gs, T, F, tpy); break;
        default: glu_gemm_k<4><<<grid, 256, sm>>>(ws.Aq, ws.As, Wq, Wsc, bias, gq, gs, T, F, tpy); break;
    }
    MICK();
    return 0;
}
extern "C" int lp_mx_gemm(int bits, int ta, int tb, int M, int N, int K, const float *A, const float *B, float *C, float beta) {
    return lp_mx_gemm_ex(bits, ta, tb, M, N, K, A, B, C, beta, nullptr, nullptr);
}
