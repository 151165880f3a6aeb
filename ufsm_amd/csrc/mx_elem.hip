// MX tensor conversions and elementwise / pointwise ops (HBM-bound): fp32 / fp16 <-> MX, network input rows, GN + SiLU apply,
// trilinear 2x upsample, add, GroupNorm sums, 1x1x1 head, and the operand re-staging used by the conv dispatch.
// One thread owns one (n, block, voxel) row, so the per-row amax that defines the output scale is thread-local
// (the reference's arrangement, src/lp_mxops.cuh:5-7); consecutive threads walk consecutive voxels, so both the plane-major
// reads (one coalesced run per channel) and the 8..32-byte row writes are contiguous across a wavefront.
#include "mx_dev.hpp"
#include <hip/hip_fp16.h>
#include <stdio.h>
#include <stdlib.h>

extern "C" size_t lp_mx8_bytes(int N, int C, size_t S) { return (size_t)N * mx_nb(C) * S * (mx_bw(C) + 1); }       // src/lp_mx_cvt.cu:6
extern "C" size_t lp_mx4_bytes(int N, int C, size_t S) { return (size_t)N * mx_nb(C) * S * (mx_bw(C) / 2 + 1); }   // src/lp_mx_cvt.cu:7

template <typename T> __device__ __forceinline__ float ldx(const T *p, size_t i);
template <> __device__ __forceinline__ float ldx<float>(const float *p, size_t i) { return p[i]; }
template <> __device__ __forceinline__ float ldx<__half>(const __half *p, size_t i) { return __half2float(p[i]); }
struct bf16_t { unsigned short v; };
template <> __device__ __forceinline__ float ldx<bf16_t>(const bf16_t *p, size_t i) { return __uint_as_float((unsigned)p[i].v << 16); }

template <int B> __device__ __forceinline__ uint8_t *mx_scp(uint8_t *q, int N, int C, size_t S) { return q + (size_t)N * mx_nb(C) * S * mx_rb(mx_bw(C), B); }
template <int B> __device__ __forceinline__ const uint8_t *mx_scp(const uint8_t *q, int N, int C, size_t S) { return q + (size_t)N * mx_nb(C) * S * mx_rb(mx_bw(C), B); }

// row i of an MX tensor -> 32 floats (zero past bw)
template <int B> __device__ __forceinline__ void load_row(const uint8_t *x, const uint8_t *sc, size_t i, int bw, float *r) {
    unsigned w[8];
    d_load_row_words<B>(x + i * mx_rb(bw, B), bw, w);
    if (B == 4) { w[4] = w[5] = w[6] = w[7] = 0u; }
    d_dequant_row<B>(w, sc[i], r);
}
template <int B, bool NANPROP> __device__ __forceinline__ void store_row(uint8_t *y, uint8_t *sc, size_t i, int bw, const float *r) {
    unsigned w[8];
    const unsigned sb = d_quant_row<B, NANPROP>(r, bw, w);
    d_store_row_words<B>(y + i * mx_rb(bw, B), bw, w);
    sc[i] = (uint8_t)sb;
}

// launch shape of the row kernels: 256 voxels per workgroup along x, (sample, block) along y
static dim3 rows_grid(int N, int nb, size_t S) {
    if ((size_t)N * nb > 65535) mi_die("MX row kernel: %d samples x %d blocks exceed the launch grid", N, nb);
    return dim3(nblk_(S, 256), (unsigned)(N * nb));
}
// ---- fp32 / 16-bit planes [n][C][S] -> MX (src/lp_mx_cvt.cu:9-19) ----
template <int B, typename TI>
__global__ void __launch_bounds__(256) f32_to_mx_k(const TI *x, uint8_t *y, int N, int C, size_t S) {
    const int bw = mx_bw(C), nb = mx_nb(C);
    const size_t v = blockIdx.x * (size_t)blockDim.x + threadIdx.x;       // grid: x over the voxels, y = n nb + blk (uniform: no per-thread divisions)
    if (v >= S) return;
    const int blk = (int)(blockIdx.y % (unsigned)nb), n = (int)(blockIdx.y / (unsigned)nb);
    const size_t i = (size_t)blockIdx.y * S + v;
    float r[32];
#pragma unroll
    for (int k = 0; k < 32; k++) { const int c = blk * bw + k; r[k] = k < bw && c < C ? ldx(x, ((size_t)n * C + c) * S + v) : 0.f; }
    store_row<B, true>(y, mx_scp<B>(y, N, C, S), i, bw, r);
}
template <int B> static void f32_to_mx(const float *x, int N, int C, size_t S, void *y) {
    const size_t n = (size_t)N * mx_nb(C) * S;
    if (!n) return;
    f32_to_mx_k<B, float><<<rows_grid(N, mx_nb(C), S), 256>>>(x, (uint8_t *)y, N, C, S); MICK();
}
extern "C" void lp_f32_to_mx8(const float *x, int N, int C, size_t S, void *y) { f32_to_mx<8>(x, N, C, S, y); }
extern "C" void lp_f32_to_mx4(const float *x, int N, int C, size_t S, void *y) { f32_to_mx<4>(x, N, C, S, y); }
template <int B> static void h16_to_mx(const void *x, int dt, int N, int C, size_t S, void *y) {
    const size_t n = (size_t)N * mx_nb(C) * S;
    if (!n) return;
    if (dt == 2) f32_to_mx_k<B, __half><<<rows_grid(N, mx_nb(C), S), 256>>>((const __half *)x, (uint8_t *)y, N, C, S);
    else if (dt == 1) f32_to_mx_k<B, bf16_t><<<rows_grid(N, mx_nb(C), S), 256>>>((const bf16_t *)x, (uint8_t *)y, N, C, S);
    else mi_die("lp_h16_to_mx%d: dtype %d is not 16-bit (1 bf16, 2 fp16)", B, dt);
    MICK();
}
extern "C" void lp_h16_to_mx8(const void *x, int dt, int N, int C, size_t S, void *y) { h16_to_mx<8>(x, dt, N, C, S, y); }
extern "C" void lp_h16_to_mx4(const void *x, int dt, int N, int C, size_t S, void *y) { h16_to_mx<4>(x, dt, N, C, S, y); }

// ---- MX -> fp32 planes (src/lp_mx_cvt.cu:429-447) ----
template <int B>
__global__ void __launch_bounds__(256) mx_to_f32_k(const uint8_t *x, float *y, int N, int C, size_t S) {
    const int bw = mx_bw(C), nb = mx_nb(C);
    const size_t v = blockIdx.x * (size_t)blockDim.x + threadIdx.x;       // grid: x over the voxels, y = n nb + blk (uniform: no per-thread divisions)
    if (v >= S) return;
    const int blk = (int)(blockIdx.y % (unsigned)nb), n = (int)(blockIdx.y / (unsigned)nb);
    const size_t i = (size_t)blockIdx.y * S + v;
    float r[32];
    load_row<B>(x, mx_scp<B>(x, N, C, S), i, bw, r);
#pragma unroll
    for (int k = 0; k < 32; k++) { const int c = blk * bw + k; if (k < bw && c < C) y[((size_t)n * C + c) * S + v] = r[k]; }
}
extern "C" void lp_mx8_to_f32(const void *x, int N, int C, size_t S, float *y) {
    const size_t n = (size_t)N * mx_nb(C) * S; if (!n) return;
    mx_to_f32_k<8><<<rows_grid(N, mx_nb(C), S), 256>>>((const uint8_t *)x, y, N, C, S); MICK();
}
extern "C" void lp_mx4_to_f32(const void *x, int N, int C, size_t S, float *y) {
    const size_t n = (size_t)N * mx_nb(C) * S; if (!n) return;
    mx_to_f32_k<4><<<rows_grid(N, mx_nb(C), S), 256>>>((const uint8_t *)x, y, N, C, S); MICK();
}

// ---- every fp32 bit pattern through the hardware encoders (v_cvt_scalef32_pk_fp8_f32, v_cvt_scalef32_pk_fp4_f32) at a block exponent e,
// against the software encoders of the scaled value x 2^-e, which equal the checker's over all 2^32 inputs (the reference checks its own
// conversion instruction the same way, src/lp_mxsw.cu:45-61). Counts: [0] inputs inside the domain the kernels use the instruction on
// (e4m3: |x 2^-e| <= 464, not NaN; e2m1: not NaN), [1] mismatches among them, [2] inputs outside it, [3] mismatches among those ----
__global__ void __launch_bounds__(256) cvt_sweep_k(int bits, int e, unsigned long long *cnt) {
    const unsigned first = (blockIdx.x * 256u + threadIdx.x) * 4096u;         // 2^20 threads x 4096 patterns
    const float p2e = d_exp2i(e), inv = d_exp2i(-e);
    unsigned n_in = 0, bad_in = 0, n_out = 0, bad_out = 0;
    for (unsigned k = 0; k < 4096u; k += 2) {
        const float a = __uint_as_float(first + k), b = __uint_as_float(first + k + 1);
        unsigned ha, hb, sa, sb;
        if (bits == 8) {
            const unsigned wv = d_enc_e4m3x4_hw(a, b, a, b, p2e);
            ha = wv & 255u; hb = (wv >> 8) & 255u;
            sa = d_enc_e4m3(a * inv); sb = d_enc_e4m3(b * inv);
        } else {
            const float v8[8] = {a, b, a, b, a, b, a, b};
            const unsigned wv = d_enc_e2m1x8_hw(v8, p2e);
            ha = wv & 15u; hb = (wv >> 4) & 15u;
            sa = d_enc_e2m1(a * inv); sb = d_enc_e2m1(b * inv);
        }
        const bool ia = bits == 8 ? fabsf(a * inv) <= 464.f : a == a, ib = bits == 8 ? fabsf(b * inv) <= 464.f : b == b;     // (NaN compares false)
        n_in += ia + ib; n_out += !ia + !ib;
        bad_in += (ia && ha != sa) + (ib && hb != sb); bad_out += (!ia && ha != sa) + (!ib && hb != sb);
    }
    atomicAdd(&cnt[0], (unsigned long long)n_in); atomicAdd(&cnt[1], (unsigned long long)bad_in);
    atomicAdd(&cnt[2], (unsigned long long)n_out); atomicAdd(&cnt[3], (unsigned long long)bad_out);
}
extern "C" int mi_cvt_sweep(int bits, int e, unsigned long long out[4]) {
    if ((bits != 8 && bits != 4) || e < -126 || e > 126) return -1;
    unsigned long long *cnt = (unsigned long long *)mi_ws(MI_WS_MISC, 4 * sizeof(unsigned long long));
    MIRT(hipMemsetAsync(cnt, 0, 4 * sizeof(unsigned long long), 0));
    cvt_sweep_k<<<4096, 256>>>(bits, e, cnt);
    MICK();
    MIRT(hipMemcpy(out, cnt, 4 * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    return 0;
}

// ---- network input rows (src/lp_mx_cvt.cu:29-55): z-scored CT, 0, unit direction away from the axis -> one 8-wide row per voxel ----
// Only channels 0, 2 and 3 of a row are ever non-zero, so a row is formed in registers from three values: amax over the three (integer,
// NaN-propagating), one exponent, one packed encode. A thread owns VPT = 4 neighbouring voxels of a row of the window when W % 4 == 0
// (one 4-byte CT load, 32 or 16 contiguous bytes of rows and one word of scale bytes out), else one voxel.
template <int HD> __device__ __forceinline__ float in_round(float v) {                         // the 16-bit type the reference's input passes through
    if (HD == 2) return __half2float(__float2half(v));
    if (HD == 1) { unsigned u = __float_as_uint(v); if ((u & 0x7fffffffu) > 0x7f800000u) return v; u += 0x7fffu + ((u >> 16) & 1u); return __uint_as_float(u & 0xffff0000u); }
    return v;
}
constexpr int PRED_BATCH = 16;                     // windows of one launch (their pointers travel in the kernel arguments)
struct pred_src_t { const uint8_t *ct[PRED_BATCH]; const float *dyo[PRED_BATCH], *dxo[PRED_BATCH]; };
template <int B, int HD, int VPT>
__global__ void __launch_bounds__(256) pred_rows_k(pred_src_t src_of, int W, float mean, float isd, int axis, int z0, size_t S,
                                                   uint8_t *__restrict__ yrows0, uint8_t *__restrict__ ysc0) {
    const size_t v0 = (blockIdx.x * (size_t)256 + threadIdx.x) * VPT;         // first voxel of the thread, relative to plane z0
    if (v0 >= S) return;
    // blockIdx.y: the window of the launch, i.e. the sample of the tensor counted from the launch's first
    const uint8_t *__restrict__ ct = src_of.ct[blockIdx.y]; const float *__restrict__ dyo = src_of.dyo[blockIdx.y], *__restrict__ dxo = src_of.dxo[blockIdx.y];
    uint8_t *__restrict__ yrows = yrows0 + blockIdx.y * S * (B == 8 ? 8 : 4), *__restrict__ ysc = ysc0 + blockIdx.y * S;
    const unsigned row = (unsigned)(v0 / (unsigned)W), xx0 = (unsigned)(v0 - (size_t)row * W), yy = row % (unsigned)W, z = (unsigned)z0 + row / (unsigned)W;
    const uint8_t *src = ct + ((size_t)z * W + yy) * W + xx0;
    unsigned cw;
    if (VPT == 4) cw = *(const unsigned *)src; else cw = *src;
    const float dy = dyo[z] + (float)yy, dx0 = dxo[z] + (float)xx0;
    unsigned codes[VPT * (B == 8 ? 2 : 1)], sb = 0u;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const float dx = i ? dxo[z] + (float)(xx0 + i) : dx0;
        float r0 = ((float)((cw >> (8 * i)) & 255u) - mean) * isd, r2, r3;
        if (axis) {
            const float inv = (float)axis / (sqrtf(fmaf(dy, dy, dx * dx)) + 1e-6f);
            r2 = __fmul_rn(dy, inv); r3 = __fmul_rn(dx, inv);
        } else { r2 = copysignf(0.f, dy); r3 = copysignf(0.f, dx); }       // d * 0: a zero with d's sign, which the 16-bit rounding and the encoders keep
        r0 = in_round<HD>(r0); r2 = in_round<HD>(r2); r3 = in_round<HD>(r3);
        unsigned am = d_amax_u(d_amax_u(d_amax_u(0u, r0), r2), r3);
        const int e = d_mx_exp(__uint_as_float(am), B == 8 ? MI_INVQ8 : MI_INVQ4);
        if (B == 8) {
            codes[2 * i] = d_enc4_e4m3(r0, 0.f, r2, r3, e);
            codes[2 * i + 1] = e == 128 ? 0x7f7f7f7fu : 0u;                   // (a non-finite row: its zeros encode as NaN too, src/lp_common.cuh:501)
        } else {
            const float r[8] = {r0, 0.f, r2, r3, 0.f, 0.f, 0.f, 0.f};
            codes[i] = d_enc8_e2m1(r, e);
        }
        sb |= (unsigned)(e + 127) << (8 * i);
    }
    if (VPT == 4) {
        if (B == 8) { *(uint4 *)(yrows + v0 * 8) = make_uint4(codes[0], codes[1], codes[2], codes[3]); *(uint4 *)(yrows + v0 * 8 + 16) = make_uint4(codes[4], codes[5], codes[6], codes[7]); }
        else *(uint4 *)(yrows + v0 * 4) = make_uint4(codes[0], codes[1], codes[2], codes[3]);
        *(unsigned *)(ysc + v0) = sb;
    } else {
        if (B == 8) *(uint2 *)(yrows + v0 * 8) = make_uint2(codes[0], codes[1]); else *(unsigned *)(yrows + v0 * 4) = codes[0];
        ysc[v0] = (uint8_t)sb;
    }
}
// samples n0 .. n0 + nw - 1 of an N-sample input tensor from nw windows (ct, dyo, dxo: host arrays of nw device pointers)
extern "C" void mi_pred_input_mx_batch(const uint8_t *const *ct, int W, float mean, float isd, const float *const *dyo, const float *const *dxo, int axis, int z0, int nz, void *y, int hd, int bits,
                                       int N, int n0, int nw) {
    const size_t S = (size_t)nz * W * W; if (!S || nw <= 0) return;
    if (N < 1 || n0 < 0 || n0 + nw > N) mi_die("mi_pred_input_mx_batch: samples %d .. %d of %d", n0, n0 + nw - 1, N);
    const int rb = bits == 4 ? 4 : 8;                                           // bytes of an 8-channel row
    for (int j0 = 0; j0 < nw; j0 += PRED_BATCH) {
        const int nb = nw - j0 < PRED_BATCH ? nw - j0 : PRED_BATCH, n = n0 + j0;
        uint8_t *yrows = (uint8_t *)y + (size_t)n * S * rb, *ysc = (uint8_t *)y + (size_t)N * S * rb + (size_t)n * S;      // sample n's rows; the tensor's scale plane follows all rows
        pred_src_t src;
        bool v4 = W % 4 == 0 && ((uintptr_t)ysc & 3) == 0 && ((uintptr_t)yrows & 15) == 0;
        for (int j = 0; j < PRED_BATCH; j++) {
            const int k = j0 + (j < nb ? j : 0);
            src.ct[j] = ct[k]; src.dyo[j] = dyo[k]; src.dxo[j] = dxo[k];
            v4 = v4 && ((uintptr_t)ct[k] & 3) == 0;
        }
#define PIN(B, HD) do { if (v4) pred_rows_k<B, HD, 4><<<dim3(nblk_(S / 4, 256), nb), 256>>>(src, W, mean, isd, axis, z0, S, yrows, ysc); \
                        else pred_rows_k<B, HD, 1><<<dim3(nblk_(S, 256), nb), 256>>>(src, W, mean, isd, axis, z0, S, yrows, ysc); } while (0)
        if (bits == 4) { if (hd == 2) PIN(4, 2); else if (hd == 1) PIN(4, 1); else PIN(4, 0); }
        else { if (hd == 2) PIN(8, 2); else if (hd == 1) PIN(8, 1); else PIN(8, 0); }
#undef PIN
    }
    MICK();
}
// sample n of an N-sample input tensor (the reference's entry is one window: N 1, n 0)
extern "C" void mi_pred_input_mx_n(const uint8_t *ct, int W, float mean, float isd, const float *dyo, const float *dxo, int axis, int z0, int nz, void *y, int hd, int bits, int N, int n) {
    if (N < 1 || n < 0 || n >= N) mi_die("mi_pred_input_mx_n: sample %d of %d", n, N);
    mi_pred_input_mx_batch(&ct, W, mean, isd, &dyo, &dxo, axis, z0, nz, y, hd, bits, N, n, 1);
}
extern "C" void lp_pred_input_mx(const uint8_t *ct, int W, float mean, float isd, const float *dyo, const float *dxo, int axis, int z0, int nz, void *y, int hd, int bits) {
    mi_pred_input_mx_n(ct, W, mean, isd, dyo, dxo, axis, z0, nz, y, hd, bits, 1, 0);
}
extern "C" void lp_pred_input_mx8(const uint8_t *ct, int W, float mean, float isd, const float *dyo, const float *dxo, int axis, int z0, int nz, void *y, int hd) {
    lp_pred_input_mx(ct, W, mean, isd, dyo, dxo, axis, z0, nz, y, hd, 8);
}

// ---- y = MX(silu(gn(x))) (src/lp_mx_gn.cu:5-31): v = (x - mean) rstd gamma + beta, v / (1 + exp(-v)) ----
// Any source (MX rows of 8 / 16 / 32 channels, fp32 / fp16 / bf16 planes) and channel count: a thread owns one (sample, block, voxel) row; the
// block's per-channel (mean, rstd, gamma, beta) are formed once per workgroup in LDS; the row is transformed in place eight channels at a time
template <int BX, int BY, typename TI>
__global__ void __launch_bounds__(256) gn_silu_rows_k(const void *__restrict__ xv, uint8_t *__restrict__ y, int N, int C, int G, size_t S,
                                                      const float *__restrict__ gamma, const float *__restrict__ beta, const float *__restrict__ mean, const float *__restrict__ rstd,
                                                      size_t v0, size_t nv, int rs, int r0) {       // voxels [v0, v0 + nv) of each sample; statistics row n * rs + r0
    const int bw = mx_bw(C), nb = mx_nb(C);
    const int blk = (int)(blockIdx.y % (unsigned)nb), n = (int)(blockIdx.y / (unsigned)nb), c0 = blk * bw, live = min(bw, C - c0);
    __shared__ float4 co[32];
    if (threadIdx.x < 32) {
        const int c = c0 + (int)threadIdx.x;
        float4 q = make_float4(0.f, 0.f, 0.f, 0.f);
        if ((int)threadIdx.x < live) { const int ng = (n * rs + r0) * G + c / (C / G); q = make_float4(mean[ng], rstd[ng], gamma[c], beta[c]); }
        co[threadIdx.x] = q;
    }
    __syncthreads();
    const size_t vi = blockIdx.x * (size_t)256 + threadIdx.x;
    if (vi >= nv) return;
    const size_t v = v0 + vi;
    const size_t row = (size_t)blockIdx.y * S + v;
    float r[32];
    if (BX != 0) { const uint8_t *x = (const uint8_t *)xv; load_row<BX ? BX : 8>(x, mx_scp<BX ? BX : 8>(x, N, C, S), row, bw, r); }
    else {
        const TI *xp = (const TI *)xv + ((size_t)n * C + c0) * S + v;
#pragma unroll
        for (int k = 0; k < 32; k++) r[k] = k < live ? ldx(xp, (size_t)k * S) : 0.f;
    }
#pragma unroll
    for (int g8 = 0; g8 < 4; g8++) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int k = 8 * g8 + i;
            const float4 q = co[k];
            const float u = fmaf((r[k] - q.x) * q.y, q.z, q.w);
            r[k] = k < live ? d_silu(u) : 0.f;
        }
    }
    store_row<BY, true>(y, mx_scp<BY>(y, N, C, S), row, bw, r);
}
// the same for an MX source of 32-channel blocks, two lanes per row (each lane one contiguous 16-channel half in and out, the per-channel
// mean / rstd / gamma / beta of the block in LDS): a wavefront reads and writes contiguous memory
template <int BX, int BY>
__global__ void __launch_bounds__(256) gn_silu_apply32_k(const uint8_t *x, uint8_t *y, int N, int C, int G, size_t S, const float *gamma, const float *beta, const float *mean, const float *rstd,
                                                         size_t v0, size_t nv, int rs, int r0) {    // voxels [v0, v0 + nv) of each sample; statistics row n * rs + r0
    const int nb = C / 32, blk = blockIdx.y, n = blockIdx.z;
    __shared__ float4 co[32];                                      // (mean, rstd, gamma, beta) of the block's channels
    if (threadIdx.x < 32) { const int c = blk * 32 + threadIdx.x, ng = (n * rs + r0) * G + c / (C / G); co[threadIdx.x] = make_float4(mean[ng], rstd[ng], gamma[c], beta[c]); }
    __syncthreads();
    const size_t t = blockIdx.x * (size_t)256 + threadIdx.x;
    const int hf = (int)(t & 1);
    if ((t >> 1) >= nv) return;
    const size_t v = v0 + (t >> 1);
    constexpr int IB = BX * 2, OB = BY * 2;                        // bytes of a 16-channel half row
    const size_t row = ((size_t)n * nb + blk) * S + v;
    const uint8_t *xs = x + (size_t)N * nb * S * (IB * 2);
    uint8_t *ys = y + (size_t)N * nb * S * (OB * 2);
    unsigned w[4] = {0u, 0u, 0u, 0u};
    if (BX == 8) { const uint4 q = *(const uint4 *)(x + row * 32 + hf * 16); w[0] = q.x; w[1] = q.y; w[2] = q.z; w[3] = q.w; }
    else { const uint2 q = *(const uint2 *)(x + row * 16 + hf * 8); w[0] = q.x; w[1] = q.y; }
    const unsigned sby = xs[row];
    const float sc = d_mx_scale(sby);
    float r[16];
    if (d_scale_plain(sby)) {                                 // (uniform) the conversions apply the scale
        if (BX == 8) { d_dec4_e4m3_scaled(w[0], sc, r); d_dec4_e4m3_scaled(w[1], sc, r + 4); d_dec4_e4m3_scaled(w[2], sc, r + 8); d_dec4_e4m3_scaled(w[3], sc, r + 12); }
        else { d_dec8_e2m1_scaled(w[0], sc, r); d_dec8_e2m1_scaled(w[1], sc, r + 8); }
    } else {
        if (BX == 8) { d_dec4_e4m3(w[0], r); d_dec4_e4m3(w[1], r + 4); d_dec4_e4m3(w[2], r + 8); d_dec4_e4m3(w[3], r + 12); }
        else { d_dec8_e2m1(w[0], r); d_dec8_e2m1(w[1], r + 8); }
#pragma unroll
        for (int k = 0; k < 16; k++) r[k] *= sc;
    }
    unsigned am = 0u;
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const float4 q = co[hf * 16 + k];
        const float u = fmaf((r[k] - q.x) * q.y, q.z, q.w);
        r[k] = d_silu(u);
        am = d_amax_u(am, r[k]);
    }
    const unsigned ao = (unsigned)__shfl_xor((int)am, 1);
    am = ao > am ? ao : am;
    const int e = d_mx_exp(__uint_as_float(am), BY == 8 ? MI_INVQ8 : MI_INVQ4);
    if (BY == 8) {
        uint4 o;
        o.x = d_enc4_e4m3(r[0], r[1], r[2], r[3], e); o.y = d_enc4_e4m3(r[4], r[5], r[6], r[7], e);
        o.z = d_enc4_e4m3(r[8], r[9], r[10], r[11], e); o.w = d_enc4_e4m3(r[12], r[13], r[14], r[15], e);
        *(uint4 *)(y + row * 32 + hf * 16) = o;
    } else {
        uint2 o; o.x = d_enc8_e2m1(r, e); o.y = d_enc8_e2m1(r + 8, e);
        *(uint2 *)(y + row * 16 + hf * 8) = o;
    }
    if (!hf) ys[row] = (uint8_t)(e + 127);
}
// voxels [v0, v0 + nv) of each sample, statistics row n * rs + r0
static void gn_silu_apply_range(const void *x, int xdt, shape5 s, int G, const float *gamma, const float *beta, const float *mean, const float *rstd, void *y, int ydt,
                                size_t v0, size_t nv, int rs, int r0) {
    const size_t S = (size_t)s.d * s.h * s.w;
    if (!nv) return;
    if (xdt >= 3 && s.c % 32 == 0) {
        const dim3 grid(nblk_(2 * nv, 256), (unsigned)(s.c / 32), (unsigned)s.n);
        const uint8_t *xq = (const uint8_t *)x; uint8_t *yq = (uint8_t *)y;
#define GS32(BX, BY) gn_silu_apply32_k<BX, BY><<<grid, 256>>>(xq, yq, s.n, s.c, G, S, gamma, beta, mean, rstd, v0, nv, rs, r0)
        if (xdt == 3) { if (ydt == 3) GS32(8, 8); else GS32(8, 4); } else { if (ydt == 3) GS32(4, 8); else GS32(4, 4); }
#undef GS32
        MICK();
        return;
    }
#define GSA(BX, BY, TI) gn_silu_rows_k<BX, BY, TI><<<rows_grid(s.n, mx_nb(s.c), nv), 256>>>(x, (uint8_t *)y, s.n, s.c, G, S, gamma, beta, mean, rstd, v0, nv, rs, r0)
#define GSA_Y(BX, TI) do { if (ydt == 4) GSA(BX, 4, TI); else GSA(BX, 8, TI); } while (0)
    if (xdt == 4) GSA_Y(4, float); else if (xdt == 3) GSA_Y(8, float); else if (xdt == 2) GSA_Y(0, __half); else if (xdt == 1) GSA_Y(0, bf16_t); else GSA_Y(0, float);
#undef GSA_Y
#undef GSA
    MICK();
}
// a mean array registered with lp_gn_slab_reg holds one row per (sample, z-slab): each slab's planes with their row (the registry lookup of
// the reference's to_gnp, src/nn_lp.h:18)
extern "C" void lp_gn_silu_apply_mx(const void *x, int xdt, shape5 s, int G, const float *gamma, const float *beta, const float *mean, const float *rstd, void *y, int ydt) {
    const size_t hw = (size_t)s.h * s.w, S = (size_t)s.d * hw, n = (size_t)s.n * mx_nb(s.c) * S;
    if (ydt != 3 && ydt != 4) mi_die("lp_gn_silu_apply_mx: output dtype %d is not MX", ydt);
    if (G <= 0 || s.c % G) mi_die("lp_gn_silu_apply_mx: %d channels in %d groups", s.c, G);
    if (!n) return;
    gn_for_slabs("lp_gn_silu_apply_mx", gnp_mk(gamma, beta, mean, rstd, G), s.h * s.w, 0, s.d, [&](int z0, int z1, gnp_t gs) {
        gn_silu_apply_range(x, xdt, s, G, gamma, beta, mean, rstd, y, ydt, (size_t)z0 * hw, (size_t)(z1 - z0) * hw, gs.ns ? gs.ns : 1, gs.ns ? gs.zo : 0);
    });
}

// ---- trilinear 2x upsample (src/lp_mx_gn.cu:34-73, :151-186): out[o] = .75 in[o/2] + .25 in[o/2 -+ 1] per axis, edge clamp ----
// Cell form: the 8 fine voxels 2m + 1 + {0, 1}^3 read exactly the 8 coarse rows m + {0, 1}^3 (clamped), so a thread owns one cell (mz, my, mx),
// each in [-1, dim - 1], for one 8-channel granule of the block: every coarse row is decoded (and, with GroupNorm, activated) once per cell
// instead of once per fine voxel, and the eight blends are register arithmetic. BW / 8 neighbouring threads share a cell and meet for the row's
// amax through lane exchanges. The 8-term sum keeps the reference's order: own row first, then the x, y, z neighbours (a, b, c loops, c fastest).
template <int BX, int BY, int BW>
__global__ void __launch_bounds__(256) up2_cell_k(const uint8_t *__restrict__ x, uint8_t *__restrict__ y, int N, int Cx, int b0, int Cy, int D, int H, int W, gnp_t gp) {
    constexpr int QP = BW / 8, IB = BX, OB = BY;                   // threads per cell; bytes of an 8-channel granule in and out
    const int nbx = mx_nb(Cx), nby = mx_nb(Cy), Do = 2 * D, Ho = 2 * H, Wo = 2 * W;
    const size_t S = (size_t)D * H * W, So = (size_t)Do * Ho * Wo;
    const int nbk = blockIdx.y, n = nbk / nby, blk = nbk % nby, live = min(BW, Cy - blk * BW);
    __shared__ float ca[32], cb[32];
    if (threadIdx.x < 32) {
        const int k = threadIdx.x, ci = blk * BW + k;
        float a = 1.f, b = 0.f;
        if (gp.G && k < live) { const int ng = n * gp.G + ci / (Cy / gp.G); a = gp.rstd[ng] * gp.gamma[ci]; b = fmaf(-gp.mean[ng], a, gp.beta[ci]); }
        ca[k] = a; cb[k] = b;
    }
    __syncthreads();
    const unsigned t = blockIdx.x * 256u + threadIdx.x, q = t % QP, cell = t / QP, ncx = (unsigned)W + 1u, ncy = (unsigned)H + 1u;
    const bool have = cell < ncx * ncy;
    const unsigned cc = have ? cell : 0u, cyi = cc / ncx;
    const int mx = (int)(cc - cyi * ncx) - 1, my = (int)cyi - 1, mz = (int)blockIdx.z - 1;
    const int cz[2] = {max(mz, 0), min(mz + 1, D - 1)}, cy[2] = {max(my, 0), min(my + 1, H - 1)}, cx[2] = {max(mx, 0), min(mx + 1, W - 1)};
    const uint8_t *xs = mx_scp<BX>(x, N, Cx, S);
    const size_t xrow0 = ((size_t)n * nbx + b0 + blk) * S;
    float f[8][8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const size_t row = xrow0 + ((size_t)cz[k >> 2] * H + cy[(k >> 1) & 1]) * W + cx[k & 1];
        const uint8_t *p = x + row * (BW * BX / 8) + q * IB;
        if (BX == 8) { const uint2 w = *(const uint2 *)p; d_dec4_e4m3(w.x, f[k]); d_dec4_e4m3(w.y, f[k] + 4); }
        else d_dec8_e2m1(*(const unsigned *)p, f[k]);
        const float sc = d_mx_scale(xs[row]);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int ch = (int)q * 8 + i;
            const float v = f[k][i] * sc;
            f[k][i] = gp.G && ch < live ? d_act_ab(v, ca[ch], cb[ch]) : v;
        }
    }
    uint8_t *ysc = mx_scp<BY>(y, N, Cy, So);
#pragma unroll
    for (int p = 0; p < 8; p++) {
        const int pz = p >> 2, py = (p >> 1) & 1, px = p & 1;                 // fine voxel 2m + 1 + p: for p = 0 its own coarse row is m, for p = 1 it is m + 1
        const int gz = 2 * mz + 1 + pz, gy = 2 * my + 1 + py, gx = 2 * mx + 1 + px;
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = 0.f;
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    const int k = ((a ^ pz) << 2) | ((b ^ py) << 1) | (c ^ px);
                    const float w3 = (a ? 0.25f : 0.75f) * (b ? 0.25f : 0.75f) * (c ? 0.25f : 0.75f);
#pragma unroll
                    for (int i = 0; i < 8; i++) acc[i] = fmaf(w3, f[k][i], acc[i]);
                }
        unsigned am = 0u;                                                      // NaN-propagating amax (src/lp_mxops.cpp row store), over the cell's QP lanes
#pragma unroll
        for (int i = 0; i < 8; i++) am = d_amax_u(am, acc[i]);
        if (QP >= 2) { const unsigned o = (unsigned)__shfl_xor((int)am, 1); am = o > am ? o : am; }
        if (QP >= 4) { const unsigned o = (unsigned)__shfl_xor((int)am, 2); am = o > am ? o : am; }
        const int e = d_mx_exp(__uint_as_float(am), BY == 8 ? MI_INVQ8 : MI_INVQ4);
        if (!have || gz < 0 || gz >= Do || gy < 0 || gy >= Ho || gx < 0 || gx >= Wo) continue;
        const size_t row = (size_t)nbk * So + ((size_t)gz * Ho + gy) * Wo + gx;
        uint8_t *dst = y + row * (BW * BY / 8) + q * OB;
        if (BY == 8) *(uint2 *)dst = make_uint2(d_enc4_e4m3(acc[0], acc[1], acc[2], acc[3], e), d_enc4_e4m3(acc[4], acc[5], acc[6], acc[7], e));
        else *(unsigned *)dst = d_enc8_e2m1(acc, e);
        if (!q) ysc[row] = (uint8_t)(e + 127);
    }
}
static void up2_launch(const void *x, int xdt, shape5 xs, int b0, int Cy, void *y, int ydt, gnp_t gp, const char *who) {
    if ((xdt != 3 && xdt != 4) || (ydt != 3 && ydt != 4)) mi_die("%s: dtypes %d -> %d are not MX", who, xdt, ydt);
    if (gp.G && (gp.ns || xs.c % gp.G)) mi_die("%s: GroupNorm of %d channels in %d groups (slab-local statistics are not supported)", who, xs.c, gp.G);
    if (!xs.d || !xs.h || !xs.w || !xs.n) return;
    const int bw = mx_bw(Cy), qp = bw / 8;
    if ((size_t)xs.n * mx_nb(Cy) > 65535 || xs.d + 1 > 65535) mi_die("%s: launch grid (%d samples x %d blocks, %d cell layers)", who, xs.n, mx_nb(Cy), xs.d + 1);
    const dim3 grid(nblk_((size_t)(xs.h + 1) * (xs.w + 1) * qp, 256), (unsigned)(xs.n * mx_nb(Cy)), (unsigned)(xs.d + 1));
    const uint8_t *xq = (const uint8_t *)x; uint8_t *yq = (uint8_t *)y;
#define U2W(BX, BY, BW) up2_cell_k<BX, BY, BW><<<grid, 256>>>(xq, yq, xs.n, xs.c, b0, Cy, xs.d, xs.h, xs.w, gp)
#define U2(BX, BY) do { if (bw == 32) U2W(BX, BY, 32); else if (bw == 16) U2W(BX, BY, 16); else U2W(BX, BY, 8); } while (0)
    if (xdt == 4) { if (ydt == 4) U2(4, 4); else U2(4, 8); } else { if (ydt == 4) U2(8, 4); else U2(8, 8); }
#undef U2
#undef U2W
    MICK();
}
extern "C" void lp_up2_fwd_mx(const void *x, int xdt, shape5 xs, void *y, int ydt, gnp_t gp) { up2_launch(x, xdt, xs, 0, xs.c, y, ydt, gp, "lp_up2_fwd_mx"); }
extern "C" void lp_up2_fwd_mx_blocks(const void *x, int xdt, shape5 xs, int b0, int nbk, void *y, int ydt) {
    if (mx_bw(xs.c) != 32 || b0 < 0 || b0 + nbk > mx_nb(xs.c)) mi_die("lp_up2_fwd_mx_blocks: blocks %d + %d of %d channels", b0, nbk, xs.c);
    gnp_t g0 = gnp_mk(nullptr, nullptr, nullptr, nullptr, 0);
    up2_launch(x, xdt, xs, b0, 32 * nbk, y, ydt, g0, "lp_up2_fwd_mx_blocks");
}

// ---- y += x (src/lp_mx_gn.cu:134-150): both rows decoded, summed in fp32, the sum re-quantised with its own scale ----
// 32-channel blocks: two lanes per row, a lane one contiguous 16-channel half of both operands and of the result (a wavefront reads and
// writes contiguous memory), ROWS rows per thread requested together; the halves' amaxes meet through one lane exchange
constexpr int ADD_ROWS = 4;
template <int B>
__global__ void __launch_bounds__(256) add32_k(uint8_t *__restrict__ y, const uint8_t *__restrict__ x, size_t rows) {
    constexpr int HB = B * 2;                                      // bytes of a 16-channel half row
    const int hf = threadIdx.x & 1;
    const size_t r0 = blockIdx.x * (size_t)(128 * ADD_ROWS) + (threadIdx.x >> 1);
    uint8_t *ys = y + rows * (2 * HB); const uint8_t *xs = x + rows * (2 * HB);
    unsigned wa[ADD_ROWS][4], wb[ADD_ROWS][4], sa[ADD_ROWS], sb[ADD_ROWS];
#pragma unroll
    for (int i = 0; i < ADD_ROWS; i++) {
        const size_t r = r0 + (size_t)i * 128, rr = r < rows ? r : rows - 1;
        if (B == 8) { const uint4 p = *(const uint4 *)(y + rr * 32 + hf * 16), q = *(const uint4 *)(x + rr * 32 + hf * 16); wa[i][0] = p.x; wa[i][1] = p.y; wa[i][2] = p.z; wa[i][3] = p.w; wb[i][0] = q.x; wb[i][1] = q.y; wb[i][2] = q.z; wb[i][3] = q.w; }
        else { const uint2 p = *(const uint2 *)(y + rr * 16 + hf * 8), q = *(const uint2 *)(x + rr * 16 + hf * 8); wa[i][0] = p.x; wa[i][1] = p.y; wb[i][0] = q.x; wb[i][1] = q.y; wa[i][2] = wa[i][3] = wb[i][2] = wb[i][3] = 0u; }
        sa[i] = ys[rr]; sb[i] = xs[rr];
    }
#pragma unroll
    for (int i = 0; i < ADD_ROWS; i++) {
        const size_t r = r0 + (size_t)i * 128;
        float a[16], b[16];
        if (B == 8) { for (int j = 0; j < 4; j++) { d_dec4_e4m3(wa[i][j], a + 4 * j); d_dec4_e4m3(wb[i][j], b + 4 * j); } }
        else { for (int j = 0; j < 2; j++) { d_dec8_e2m1(wa[i][j], a + 8 * j); d_dec8_e2m1(wb[i][j], b + 8 * j); } }
        const float fa = d_mx_scale(sa[i]), fb = d_mx_scale(sb[i]);
        unsigned am = 0u;
#pragma unroll
        for (int k = 0; k < 16; k++) { a[k] = __fadd_rn(a[k] * fa, b[k] * fb); am = d_amax_u(am, a[k]); }     // (two rounded products, one rounded sum: no contraction)
        const unsigned ao = (unsigned)__shfl_xor((int)am, 1);
        am = ao > am ? ao : am;
        const int e = d_mx_exp(__uint_as_float(am), B == 8 ? MI_INVQ8 : MI_INVQ4);
        if (r >= rows) continue;
        if (B == 8) *(uint4 *)(y + r * 32 + hf * 16) = make_uint4(d_enc4_e4m3(a[0], a[1], a[2], a[3], e), d_enc4_e4m3(a[4], a[5], a[6], a[7], e), d_enc4_e4m3(a[8], a[9], a[10], a[11], e), d_enc4_e4m3(a[12], a[13], a[14], a[15], e));
        else *(uint2 *)(y + r * 16 + hf * 8) = make_uint2(d_enc8_e2m1(a, e), d_enc8_e2m1(a + 8, e));
        if (!hf) ys[r] = (uint8_t)(e + 127);
    }
}
// narrow rows (<= 16 channels): one thread per row
template <int B> __global__ void __launch_bounds__(256) add_rows_k(uint8_t *__restrict__ y, const uint8_t *__restrict__ x, size_t rows, int bw) {
    const size_t r = blockIdx.x * (size_t)256 + threadIdx.x;
    if (r >= rows) return;
    uint8_t *ys = y + rows * mx_rb(bw, B); const uint8_t *xs = x + rows * mx_rb(bw, B);
    float a[32], b[32];
    load_row<B>(y, ys, r, bw, a); load_row<B>(x, xs, r, bw, b);
#pragma unroll
    for (int k = 0; k < 32; k++) a[k] = __fadd_rn(a[k], b[k]);
    store_row<B, true>(y, ys, r, bw, a);
}
extern "C" void lp_add_mx(void *y, const void *x, shape5 s, int dt, unsigned sr) {
    if (sr) mi_die("lp_add_mx: stochastic rounding (sr %u) belongs to training and is not built here", sr);
    const size_t rows = (size_t)s.n * mx_nb(s.c) * s.d * s.h * s.w; if (!rows) return;
    const int bw = mx_bw(s.c);
    if (bw == 32) {
        if (dt == 4) add32_k<4><<<nblk_(rows, 128 * ADD_ROWS), 256>>>((uint8_t *)y, (const uint8_t *)x, rows);
        else add32_k<8><<<nblk_(rows, 128 * ADD_ROWS), 256>>>((uint8_t *)y, (const uint8_t *)x, rows);
    } else if (dt == 4) add_rows_k<4><<<nblk_(rows, 256), 256>>>((uint8_t *)y, (const uint8_t *)x, rows, bw);
    else add_rows_k<8><<<nblk_(rows, 256), 256>>>((uint8_t *)y, (const uint8_t *)x, rows, bw);
    MICK();
}

// ---- GroupNorm (sum, sum of squares) of a stored MX tensor into fixed-point slots (src/lp_mx_gnsums.cu:8-101) ----
// Sums 32 per-lane fp64 values over the 32 lanes of each wavefront half in a fixed order: step k pairs lane r with r ^ 2^k and the pair
// splits the values left (the lane whose bit k is clear keeps the lower half of the indices and receives the partner's). Returns the index
// of the value whose total the lane holds in v[0] afterwards: sum over k of bit k of r times 16 >> k.
template <int K>
__device__ __forceinline__ void wave_half_reduce_f64_step(double (&v)[32], int r, int &idx) {      // (a template per step: every index is a constant, the values stay in registers)
    constexpr int half = 16 >> K;
    const bool bit = (r >> K) & 1;
#pragma unroll
    for (int i = 0; i < half; i++) {
        const double send = bit ? v[i] : v[i + half], keep = bit ? v[i + half] : v[i];
        v[i] = keep + __shfl_xor(send, 1 << K);
    }
    idx += bit ? half : 0;
}
__device__ __forceinline__ int wave_half_reduce_f64(double (&v)[32], int r) {
    int idx = 0;
    wave_half_reduce_f64_step<0>(v, r, idx); wave_half_reduce_f64_step<1>(v, r, idx); wave_half_reduce_f64_step<2>(v, r, idx);
    wave_half_reduce_f64_step<3>(v, r, idx); wave_half_reduce_f64_step<4>(v, r, idx);
    return idx;
}
// A block reduces a slab of voxels of one (n, channel block): per-thread fp64 partials per channel, then a fixed-order (deterministic)
// reduction over the block.
template <int B>
__global__ void __launch_bounds__(256) gn_sums_mx_k(const uint8_t *x, int N, int C, int G, size_t S, double *sums, size_t v0, size_t v1, int n0) {
    const int bw = mx_bw(C), nb = mx_nb(C), cpg = C / G, blk = blockIdx.y, n = n0 + (int)blockIdx.z, nsl = gridDim.x;
    size_t q0 = v0 + (v1 - v0) * blockIdx.x / nsl, q1 = v0 + (v1 - v0) * (blockIdx.x + 1) / nsl;
    const uint8_t *sc = mx_scp<B>(x, N, C, S);
    double s1[32], s2[32];
#pragma unroll
    for (int k = 0; k < 32; k++) { s1[k] = 0.0; s2[k] = 0.0; }
    for (size_t q = q0 + threadIdx.x; q < q1; q += 256) {
        float r[32];
        load_row<B>(x, sc, ((size_t)n * nb + blk) * S + q, bw, r);
#pragma unroll
        for (int k = 0; k < 32; k++) { const double d = (double)r[k]; s1[k] += d; s2[k] += d * d; }
    }
    // each channel's partials: a fixed-order exchange tree over the 32 lanes of a wavefront half (every step halves the values a lane
    // carries), the other half by one more exchange, the four wavefronts through LDS; then one slot add per channel and moment
    const int lane = threadIdx.x & 63, r = lane & 31;
    const int i1 = wave_half_reduce_f64(s1, r), i2 = wave_half_reduce_f64(s2, r);
    const double t1 = s1[0] + __shfl_xor(s1[0], 32), t2 = s2[0] + __shfl_xor(s2[0], 32);
    __shared__ double red[4][64], tot[64];
    if (lane < 32) { red[threadIdx.x >> 6][i1] = t1; red[threadIdx.x >> 6][32 + i2] = t2; }
    __syncthreads();
    if (threadIdx.x < 64) tot[threadIdx.x] = ((red[0][threadIdx.x] + red[1][threadIdx.x]) + red[2][threadIdx.x]) + red[3][threadIdx.x];
    __syncthreads();
    if (threadIdx.x < 64) {                                  // the first channel of every group inside the block adds the group's channels in order
        const int k = threadIdx.x & 31, pass = threadIdx.x >> 5, c = blk * bw + k, g = c / cpg;
        if (k < bw && c < C && (k == 0 || (c - 1) / cpg != g)) {
            double acc = 0.0;
            for (int kk = k; kk < bw && blk * bw + kk < C && (blk * bw + kk) / cpg == g; kk++) acc += tot[pass * 32 + kk];
            gn_acc_add(sums, 2 * ((size_t)n * G + g) + pass, acc);
        }
    }
}
extern "C" int lp_gn_sums_mx_n(const void *x, int xdt, int N, int C, int G, size_t S, double *sums, size_t v0, size_t v1, int n0, int cnt) {
    if ((xdt != 3 && xdt != 4) || G <= 0 || C % G) return -1;
    if (v1 <= v0 || cnt <= 0) return 0;
    size_t nsl = (v1 - v0 + 8191) / 8192; if (nsl > 512) nsl = 512;      // (few, large slabs: every block ends in atomic adds to the same few slots)
    const dim3 grid((unsigned)nsl, (unsigned)mx_nb(C), (unsigned)cnt);
    if (xdt == 4) gn_sums_mx_k<4><<<grid, 256>>>((const uint8_t *)x, N, C, G, S, sums, v0, v1, n0);
    else gn_sums_mx_k<8><<<grid, 256>>>((const uint8_t *)x, N, C, G, S, sums, v0, v1, n0);
    MICK();
    return 0;
}
extern "C" int lp_gn_sums_mx(const void *x, int xdt, int N, int C, int G, size_t S, double *sums, size_t v0, size_t v1) {
    return lp_gn_sums_mx_n(x, xdt, N, C, G, S, sums, v0, v1, 0, N);
}

// ---- 1x1x1 head (src/lp_mx_conv1.cu:5-21): y[n][co][v] = b[co] + sum_ci w[co][ci] act(x[ci][v]), fp32 FMA in ci order ----
// Thread per voxel; weights, bias and the GN coefficients of the sample staged in LDS once per block; CO outputs per pass in registers.
// MF (CO 8, whole 32-channel blocks): the 8 x 32 products of a voxel go through the matrix pipe as batched 4 x 4 outer products
// (v_mfma_f32_4x4x1: 16 blocks of four lanes; a lane supplies its voxel's activation as column j = lane % 4 of its block and output channel
// lane % 4 (+ 4) of the weights as row, and receives the four channels of its own voxel). One product is added per step, in ci order, so the
// sums are those of the fused multiply-add chain; what moves is 256 of a voxel's vector instructions, into a pipe the sigmoids do not use.
// Every lane of a wavefront must take part: a voxel past the range computes on voxel 0's row and stores nothing.
typedef float v4f __attribute__((ext_vector_type(4)));
template <int B, int CO, typename YT, bool MF = false>
__global__ void __launch_bounds__(256, 4) conv1_mx_k(const uint8_t *x, const float *w, const float *b, YT *y, int N, int Ci, size_t S, gnp_t gp, int Co, int co0,
                                                  size_t vb, size_t nv, size_t ly) {
    extern __shared__ __align__(16) float c1s[];          // [Ci][CO] weights (input-channel major: a channel's CO weights are one or two 16-byte reads at an
                                                          // immediate offset from the block's base), [CO] bias, [Ci] a, [Ci] b
    float *sw = c1s, *sb = sw + ((CO * Ci + 3) & ~3), *sa = sb + 8, *sbb = sa + ((Ci + 3) & ~3);      // (every array starts on 16 bytes: the fast path reads 16-byte vectors of sw, sa and sbb)
    const int n = blockIdx.y, bw = mx_bw(Ci), nb = mx_nb(Ci);
    for (int i = threadIdx.x; i < CO * Ci; i += 256) { const int co = co0 + i % CO, ci = i / CO; sw[i] = co < Co ? w[(size_t)co * Ci + ci] : 0.f; }
    for (int i = threadIdx.x; i < CO; i += 256) sb[i] = b && co0 + i < Co ? b[co0 + i] : 0.f;
    for (int i = threadIdx.x; i < Ci; i += 256) {
        float a = 1.f, bb = 0.f;
        if (gp.G) { const int ng = d_gn_row(gp, n) * gp.G + i / (Ci / gp.G); a = gp.rstd[ng] * gp.gamma[i]; bb = fmaf(-gp.mean[ng], a, gp.beta[i]); }
        sa[i] = a; sbb[i] = bb;
    }
    __syncthreads();
    const size_t vi = blockIdx.x * (size_t)256 + threadIdx.x;
    const bool live = vi < nv;
    if (!MF && !live) return;
    const size_t v = vb + (live ? vi : 0);
    float acc[CO];
#pragma unroll
    for (int co = 0; co < CO; co++) acc[co] = sb[co];
    const uint8_t *sc = mx_scp<B>(x, N, Ci, S);
    for (int blk = 0; blk < nb; blk++) {
        float r[32];
        load_row<B>(x, sc, ((size_t)n * nb + blk) * S + v, bw, r);
        if (bw == 32 && (blk + 1) * 32 <= Ci) {                  // (uniform) a whole 32-channel block: straight-line code, every LDS operand at an immediate offset
            const float *swb = sw + (size_t)blk * 32 * CO, *sab = sa + blk * 32, *sbb2 = sbb + blk * 32;
            if (gp.G) {
#pragma unroll
                for (int k4 = 0; k4 < 8; k4++) {
                    const float4 ta = *(const float4 *)(sab + 4 * k4), tb = *(const float4 *)(sbb2 + 4 * k4);
                    r[4 * k4] = d_act_ab(r[4 * k4], ta.x, tb.x); r[4 * k4 + 1] = d_act_ab(r[4 * k4 + 1], ta.y, tb.y);
                    r[4 * k4 + 2] = d_act_ab(r[4 * k4 + 2], ta.z, tb.z); r[4 * k4 + 3] = d_act_ab(r[4 * k4 + 3], ta.w, tb.w);
                }
            }
            if constexpr (MF) {
                static_assert(!MF || CO == 8, "matrix-pipe head: eight output channels");
                const float *wl = swb + (threadIdx.x & 3);       // the lane's row of its block's two weight tiles: channels lane % 4 and 4 + lane % 4
                v4f lo = {acc[0], acc[1], acc[2], acc[3]}, hi = {acc[4], acc[5], acc[6], acc[7]};
#pragma unroll
                for (int k = 0; k < 32; k++) {
                    lo = __builtin_amdgcn_mfma_f32_4x4x1f32(wl[k * 8], r[k], lo, 0, 0, 0);
                    hi = __builtin_amdgcn_mfma_f32_4x4x1f32(wl[k * 8 + 4], r[k], hi, 0, 0, 0);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) { acc[i] = lo[i]; acc[4 + i] = hi[i]; }
                continue;
            }
#pragma unroll
            for (int k = 0; k < 32; k++) {
                float wv[CO];
                if constexpr (CO >= 4) {
#pragma unroll
                    for (int q = 0; q < CO / 4; q++) { const float4 w4 = *(const float4 *)(swb + k * CO + 4 * q); wv[4 * q] = w4.x; wv[4 * q + 1] = w4.y; wv[4 * q + 2] = w4.z; wv[4 * q + 3] = w4.w; }
                } else {
#pragma unroll
                    for (int co = 0; co < CO; co++) wv[co] = swb[k * CO + co];
                }
#pragma unroll
                for (int co = 0; co < CO; co++) acc[co] = fmaf(wv[co], r[k], acc[co]);
                if (k % 4 == 3) __builtin_amdgcn_sched_barrier(0);     // (a thread uses each weight once: reading them all ahead only costs registers)
            }
            continue;
        }
#pragma unroll
        for (int k = 0; k < 32; k++) {
            const int ci = blk * bw + k;
            if (k < bw && ci < Ci) {
                const float xv = gp.G ? d_act_ab(r[k], sa[ci], sbb[ci]) : r[k];
                float wv[CO];
                if constexpr (CO >= 4) {
#pragma unroll
                    for (int q = 0; q < CO / 4; q++) { const float4 w4 = *(const float4 *)(sw + (size_t)ci * CO + 4 * q); wv[4 * q] = w4.x; wv[4 * q + 1] = w4.y; wv[4 * q + 2] = w4.z; wv[4 * q + 3] = w4.w; }
                } else {
#pragma unroll
                    for (int co = 0; co < CO; co++) wv[co] = sw[ci * CO + co];
                }
#pragma unroll
                for (int co = 0; co < CO; co++) acc[co] = fmaf(wv[co], xv, acc[co]);
            }
        }
    }
    if (!live) return;
#pragma unroll
    for (int co = 0; co < CO; co++) if (co0 + co < Co) {
        const size_t o = ((size_t)n * Co + co0 + co) * ly + vi;
        if (sizeof(YT) == 2) ((__half *)y)[o] = __float2half(acc[co]); else ((float *)y)[o] = acc[co];
    }
}
static thread_local int g_conv1_matrix = -1;      // mi_conv1_matrix: the calling thread's choice of where the head's products run (-1: the default)
extern "C" void mi_conv1_matrix(int mode) { g_conv1_matrix = mode; }
template <typename YT>
static void conv1_launch_row(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, YT *y, gnp_t gp, size_t vb, size_t nv, size_t ly, const char *who);
// voxels [vb, vb + nv) of every sample; with slab-local GroupNorm statistics one launch per slab the range meets (its voxels, its statistics row)
template <typename YT>
static void conv1_launch(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, YT *y, gnp_t gp, size_t vb, size_t nv, size_t ly, const char *who) {
    if (!gp.G || !gp.ns || !nv) { conv1_launch_row<YT>(x, xdt, xs, w, b, cout, y, gp, vb, nv, ly, who); return; }
    const size_t hw = (size_t)xs.h * xs.w;
    gn_for_slabs(who, gp, xs.h * xs.w, (int)(vb / hw), (int)((vb + nv + hw - 1) / hw), [&](int z0, int z1, gnp_t gs) {
        const size_t a = (size_t)z0 * hw > vb ? (size_t)z0 * hw : vb, e = (size_t)z1 * hw < vb + nv ? (size_t)z1 * hw : vb + nv;
        if (a < e) conv1_launch_row<YT>(x, xdt, xs, w, b, cout, y + (a - vb), gs, a, e - a, ly, who);
    });
}
template <typename YT>
static void conv1_launch_row(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, YT *y, gnp_t gp, size_t vb, size_t nv, size_t ly, const char *who) {
    if (xdt != 3 && xdt != 4) mi_die("%s: input dtype %d is not MX", who, xdt);
    if (gp.G && xs.c % gp.G) mi_die("%s: GroupNorm of %d channels in %d groups", who, xs.c, gp.G);
    if (xs.c > 1024) mi_die("%s: %d input channels (at most 1024)", who, xs.c);
    const size_t S = (size_t)xs.d * xs.h * xs.w;
    if (!nv || !xs.n) return;
    const dim3 grid(nblk_(nv, 256), (unsigned)xs.n);
    const uint8_t *xq = (const uint8_t *)x;
    for (int co0 = 0; co0 < cout; co0 += 8) {
        const int rem = cout - co0;
        const size_t sm = ((size_t)8 * xs.c + 8 + 2 * (size_t)((xs.c + 3) & ~3)) * sizeof(float);
#define C1(B, CO) conv1_mx_k<B, CO, YT><<<grid, 256, sm>>>(xq, w, b, y, xs.n, xs.c, S, gp, cout, co0, vb, nv, ly)
        static int mf_env = -1;
        if (mf_env < 0) mf_env = getenv("MI_HEAD_MFMA") ? atoi(getenv("MI_HEAD_MFMA")) : 1;     // tuning knob: 0 keeps the products on the vector ALUs
        if ((g_conv1_matrix < 0 ? mf_env : g_conv1_matrix) && rem >= 8 && xs.c % 32 == 0) {
            if (xdt == 4) conv1_mx_k<4, 8, YT, true><<<grid, 256, sm>>>(xq, w, b, y, xs.n, xs.c, S, gp, cout, co0, vb, nv, ly);
            else conv1_mx_k<8, 8, YT, true><<<grid, 256, sm>>>(xq, w, b, y, xs.n, xs.c, S, gp, cout, co0, vb, nv, ly);
            continue;
        }
        if (xdt == 4) { if (rem >= 8) C1(4, 8); else if (rem >= 4) { C1(4, 4); co0 -= 4; } else if (rem >= 2) { C1(4, 2); co0 -= 6; } else { C1(4, 1); co0 -= 7; } }
        else { if (rem >= 8) C1(8, 8); else if (rem >= 4) { C1(8, 4); co0 -= 4; } else if (rem >= 2) { C1(8, 2); co0 -= 6; } else { C1(8, 1); co0 -= 7; } }
#undef C1
    }
    MICK();
}
extern "C" void lp_conv1_fwd_mx(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, float *y, gnp_t gp) {
    const size_t S = (size_t)xs.d * xs.h * xs.w; conv1_launch<float>(x, xdt, xs, w, b, cout, y, gp, 0, S, S, "lp_conv1_fwd_mx");
}
extern "C" void lp_conv1_fwd_mx_h16(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, void *y, gnp_t gp) {
    const size_t S = (size_t)xs.d * xs.h * xs.w; conv1_launch<__half>(x, xdt, xs, w, b, cout, (__half *)y, gp, 0, S, S, "lp_conv1_fwd_mx_h16");
}
extern "C" void lp_conv1_fwd_mx_h16_r(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, void *y, gnp_t gp, size_t vb, size_t nv) {
    conv1_launch<__half>(x, xdt, xs, w, b, cout, (__half *)y, gp, vb, nv, nv, "lp_conv1_fwd_mx_h16_r");
}
extern "C" int lp_conv1_fwd_mx_r(const void *x, int xdt, shape5 xs, const float *w, const float *b, int cout, float *y, gnp_t gp, size_t vb, size_t nv, size_t ly) {
    conv1_launch<float>(x, xdt, xs, w, b, cout, y, gp, vb, nv, ly ? ly : nv, "lp_conv1_fwd_mx_r");
    return 1;
}

// ---- operand re-staging for the conv dispatch (the arithmetic of src/lp_f8fwd.cuh:88-113 applied once per tensor instead of once per
// staged halo position): any source (planes or MX) -> optional GN + SiLU (staging form) -> rows in the compute format, blocks of 32 ----
template <int BX, int BY, typename TI>
__global__ void __launch_bounds__(256) restage_k(const void *xv, uint8_t *y, int N, int C, size_t S, gnp_t gp, int Cg, int cg0, size_t Ss, size_t v0) {
    // voxels [v0, v0 + S) of tensors holding Ss voxels per (sample, channel / block), source and result alike; y: an MX tensor of nbo * 32 channels (bw 32). gp over Cg channels of which this tensor holds [cg0, cg0 + C) (whole-input GroupNorm of a split input)
    const int nbo = (C + 31) / 32, bwx = mx_bw(C), Cy = nbo * 32;
    const size_t v = blockIdx.x * (size_t)blockDim.x + threadIdx.x;       // grid: x over the voxels, y = n nbo + blk (uniform: no per-thread divisions)
    if (v >= S) return;
    const int blk = (int)(blockIdx.y % (unsigned)nbo), n = (int)(blockIdx.y / (unsigned)nbo);
    float r[32];
    if (BX != 0) {
        const uint8_t *x = (const uint8_t *)xv; const uint8_t *sc = mx_scp<BX ? BX : 8>(x, N, C, Ss);
        if (bwx == 32) load_row<BX ? BX : 8>(x, sc, ((size_t)n * mx_nb(C) + blk) * Ss + v0 + v, 32, r);
        else load_row<BX ? BX : 8>(x, sc, (size_t)n * Ss + v0 + v, bwx, r);     // C <= 16: one narrow block, zero-extended
    } else {
#pragma unroll
        for (int k = 0; k < 32; k++) { const int c = blk * 32 + k; r[k] = c < C ? ldx((const TI *)xv, ((size_t)n * C + c) * Ss + v0 + v) : 0.f; }
    }
    if (gp.G) {
        const int cpg = Cg / gp.G;
#pragma unroll
        for (int k = 0; k < 32; k++) {
            const int c = blk * 32 + k;
            if (c < C) { const int ng = d_gn_row(gp, n) * gp.G + (cg0 + c) / cpg; const float a = gp.rstd[ng] * gp.gamma[cg0 + c], b = fmaf(-gp.mean[ng], a, gp.beta[cg0 + c]); r[k] = d_act_ab(r[k], a, b); }
            else r[k] = 0.f;
        }
    }
    store_row<BY, false>(y, mx_scp<BY>(y, N, Cy, Ss), ((size_t)n * nbo + blk) * Ss + v0 + v, 32, r);
}
// the same for an MX source with 32-wide blocks, two lanes per row: each lane moves one 16-channel half (16 or 8 contiguous bytes in,
// 16 or 8 out), so a wavefront reads and writes contiguous memory; the halves' amaxes meet through one lane exchange. The (a, b)
// coefficients of the block's 32 channels are formed once per workgroup in LDS. HBM-bound: (bits_in + bits_out) / 8 + 2/32 bytes per element.
constexpr int RS32_R = 4;                                          // rows per thread of restage32_k
// BY2 (4, with BY 8): the same values also leave as a second tensor y2 in MX-fp4 - a skip tensor whose two readers compute in different
// formats (the stride-2 down conv in e4m3, the decoder's conv in e2m1) is read and transformed once
template <int BX, int BY, int BY2 = 0>
__global__ void __launch_bounds__(256) restage32_k(const uint8_t *x, uint8_t *y, int N, int C, size_t S, gnp_t gp, int Cg, int cg0, size_t Ss, size_t v0, uint8_t *y2 = nullptr) {
    const int nb = C / 32, blk = blockIdx.y, n = blockIdx.z;
    __shared__ float sa[32], sb[32];
    // A workgroup moves RS32_R x 128 consecutive voxels of the block, a thread one 16-channel half of RS32_R rows 128 voxels apart: the rows are
    // requested together (one memory round trip per thread instead of one per row) and the coefficients' set-up is paid once per RS32_R rows
    constexpr int IB = BX * 2, OB = BY * 2;                        // bytes of a 16-channel half row
    const int hf = threadIdx.x & 1;
    const size_t vb = blockIdx.x * (size_t)(128 * RS32_R) + (threadIdx.x >> 1);
    const size_t row0 = ((size_t)n * nb + blk) * Ss + v0;
    const uint8_t *xs = x + (size_t)N * nb * Ss * (IB * 2);
    uint8_t *ys = y + (size_t)N * nb * Ss * (OB * 2);
    unsigned w[RS32_R][4]; unsigned sby[RS32_R];
#pragma unroll
    for (int i = 0; i < RS32_R; i++) {
        const size_t v = vb + (size_t)i * 128, row = row0 + (v < S ? v : S - 1);      // (rows past the end re-read the last one and are not stored)
        w[i][2] = 0u; w[i][3] = 0u;
        if (BX == 8) { const uint4 q = *(const uint4 *)(x + row * 32 + hf * 16); w[i][0] = q.x; w[i][1] = q.y; w[i][2] = q.z; w[i][3] = q.w; }
        else { const uint2 q = *(const uint2 *)(x + row * 16 + hf * 8); w[i][0] = q.x; w[i][1] = q.y; }
        sby[i] = xs[row];
    }
    // (the rows are requested before the block's coefficients are formed: the two chains of dependent loads overlap)
    if (threadIdx.x < 32) {
        float a = 1.f, b = 0.f;
        if (gp.G) { const int c = cg0 + blk * 32 + threadIdx.x, ng = d_gn_row(gp, n) * gp.G + c / (Cg / gp.G); a = gp.rstd[ng] * gp.gamma[c]; b = fmaf(-gp.mean[ng], a, gp.beta[c]); }
        sa[threadIdx.x] = a; sb[threadIdx.x] = b;
    }
    __syncthreads();
    float ca[16], cb[16];
#pragma unroll
    for (int k = 0; k < 16; k++) { ca[k] = sa[hf * 16 + k]; cb[k] = sb[hf * 16 + k]; }
#pragma unroll
    for (int i = 0; i < RS32_R; i++) {
        const size_t v = vb + (size_t)i * 128, row = row0 + v;
        const float sc = d_mx_scale(sby[i]);
        float r[16];
        if (d_scale_plain(sby[i])) {                          // (uniform) the conversions apply the scale
            if (BX == 8) { d_dec4_e4m3_scaled(w[i][0], sc, r); d_dec4_e4m3_scaled(w[i][1], sc, r + 4); d_dec4_e4m3_scaled(w[i][2], sc, r + 8); d_dec4_e4m3_scaled(w[i][3], sc, r + 12); }
            else { d_dec8_e2m1_scaled(w[i][0], sc, r); d_dec8_e2m1_scaled(w[i][1], sc, r + 8); }
        } else {
            if (BX == 8) { d_dec4_e4m3(w[i][0], r); d_dec4_e4m3(w[i][1], r + 4); d_dec4_e4m3(w[i][2], r + 8); d_dec4_e4m3(w[i][3], r + 12); }
            else { d_dec8_e2m1(w[i][0], r); d_dec8_e2m1(w[i][1], r + 8); }
#pragma unroll
            for (int k = 0; k < 16; k++) r[k] *= sc;
        }
        if (gp.G) {                                               // (one uniform branch around sixteen independent chains: a select per value made sixteen blocks of one dependent chain each)
#pragma unroll
            for (int k = 0; k < 16; k++) r[k] = d_act_ab(r[k], ca[k], cb[k]);
        }
        float am = 0.f;
#pragma unroll
        for (int k = 0; k < 16; k++) am = fmaxf(am, fabsf(r[k]));
        am = __uint_as_float(max(__float_as_uint(am), d_quad_xor_u<1>(__float_as_uint(am))));       // (a non-negative number, never NaN: it orders as its bits)
        const int e = d_mx_exp(am, BY == 8 ? MI_INVQ8 : MI_INVQ4);
        if (BY == 8) {
            uint4 o;
            o.x = d_enc4_e4m3(r[0], r[1], r[2], r[3], e); o.y = d_enc4_e4m3(r[4], r[5], r[6], r[7], e);
            o.z = d_enc4_e4m3(r[8], r[9], r[10], r[11], e); o.w = d_enc4_e4m3(r[12], r[13], r[14], r[15], e);
            if (v < S) *(uint4 *)(y + row * 32 + hf * 16) = o;
        } else {
            uint2 o; o.x = d_enc8_e2m1(r, e); o.y = d_enc8_e2m1(r + 8, e);
            if (v < S) *(uint2 *)(y + row * 16 + hf * 8) = o;
        }
        if (!hf && v < S) ys[row] = (uint8_t)(e + 127);
        if (BY2 == 4) {
            const int e2 = d_mx_exp(am, MI_INVQ4);
            uint2 o; o.x = d_enc8_e2m1(r, e2); o.y = d_enc8_e2m1(r + 8, e2);
            if (v < S) { *(uint2 *)(y2 + row * 16 + hf * 8) = o; if (!hf) (y2 + (size_t)N * nb * Ss * 16)[row] = (uint8_t)(e2 + 127); }
        }
    }
}
// MX-fp8 source with 32-wide blocks -> the transformed rows in both formats from one read (y8 MX-fp8, y4 MX-fp4), the bytes of the two single calls
void mi_restage_sub2(const void *x, int N, int C, size_t S, gnp_t gp, void *y8, void *y4, size_t Ss, size_t v0) {
    if (!N || !S) return;
    const dim3 grid(nblk_(S, 128 * RS32_R), (unsigned)(C / 32), (unsigned)N);
    restage32_k<8, 8, 4><<<grid, 256>>>((const uint8_t *)x, (uint8_t *)y8, N, C, S, gp, C, 0, Ss, v0, (uint8_t *)y4);
    MICK();
}
// voxels [v0, v0 + S) of tensors holding Ss voxels per (sample, channel / block): the result has the source's geometry, only that range is written
void mi_restage_sub(const void *x, int xdt, int N, int C, size_t S, gnp_t gp, int Cg, int cg0, void *y, int ybits, size_t Ss, size_t v0) {
    const size_t n = (size_t)N * ((C + 31) / 32) * S; if (!n) return;
    if (xdt >= 3 && C % 32 == 0) {
        const dim3 grid(nblk_(S, 128 * RS32_R), (unsigned)(C / 32), (unsigned)N);
        const uint8_t *xq = (const uint8_t *)x; uint8_t *yq = (uint8_t *)y;
        if (xdt == 3) { if (ybits == 8) restage32_k<8, 8><<<grid, 256>>>(xq, yq, N, C, S, gp, Cg, cg0, Ss, v0); else restage32_k<8, 4><<<grid, 256>>>(xq, yq, N, C, S, gp, Cg, cg0, Ss, v0); }
        else { if (ybits == 8) restage32_k<4, 8><<<grid, 256>>>(xq, yq, N, C, S, gp, Cg, cg0, Ss, v0); else restage32_k<4, 4><<<grid, 256>>>(xq, yq, N, C, S, gp, Cg, cg0, Ss, v0); }
        MICK();
        return;
    }
#define RS(BX, BY, TI) restage_k<BX, BY, TI><<<rows_grid(N, (C + 31) / 32, S), 256>>>(x, (uint8_t *)y, N, C, S, gp, Cg, cg0, Ss, v0)
#define RS_Y(BX, TI) do { if (ybits == 4) RS(BX, 4, TI); else RS(BX, 8, TI); } while (0)
    if (xdt == 4) RS_Y(4, float); else if (xdt == 3) RS_Y(8, float); else if (xdt == 2) RS_Y(0, __half); else if (xdt == 1) RS_Y(0, bf16_t); else RS_Y(0, float);
#undef RS_Y
#undef RS
    MICK();
}
void mi_restage(const void *x, int xdt, int N, int C, size_t S, gnp_t gp, int Cg, int cg0, void *y, int ybits) { mi_restage_sub(x, xdt, N, C, S, gp, Cg, cg0, y, ybits, S, 0); }
// decoder up segment (src/lp_common.cuh:618-670): coarse rows -> GN + SiLU -> e4m3 rows with a row scale (amax ignoring NaN) -> 8-term fp32
// blend (weights .75 / .25, fma order z, y, x, the row scale folded into the weight) -> rows in the compute format at the fine resolution.
// Two passes: the coarse rows are activated and re-quantised once (mi_restage into an MX-fp8 scratch tensor, an eighth of the output),
// then up_blend_k forms the fine rows. A thread owns the 8 fine voxels whose blend reads one 2x2x2 cell of coarse rows, for 8 of the
// block's 32 channels: cell (mz, my, mx), each in [-1, dim/2 - 1], covers coarse {m, m + 1} (clamped) and fine {2m + 1, 2m + 2}; the four
// threads of a cell meet for the row amax through lane exchanges. Each coarse row is decoded once per cell instead of once per fine voxel.
// H2: the fp4 entry's blend (stage_up_smem_h2, src/lp_common.cuh:674-712): binary16 weights relative to the largest of the cell's 8 scale bytes,
// binary16 fused multiply-adds in the same z, y, x order (an e4m3 code is a binary16 value), the sum widened and scaled by 2^e_max.
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
// CH: channels of the block per thread, 8 (four threads per cell) for the fp32 blend and 16 (two threads per cell) for the binary16 blend: what
// a fine voxel costs beside its multiply-adds (block maximum, exponent, scale, stores) is then paid by two lanes instead of four (0.52 -> 0.40 ms
// at 8 x 64 channels 64^3 -> 128^3). The fp32 blend with 16 holds 128 row values and 190 registers, two wavefronts per SIMD: measured no faster
template <int BY, bool H2, int CH = H2 ? 16 : 8>
__global__ void __launch_bounds__(256) up_blend_k(const uint8_t *xc, uint8_t *y, int N, int nbo, int D, int H, int W, int zlo, int zhi, int clo, int Dcs, int mz0, int ncz_) {
    // fine planes [zlo, zhi) of the depth-D result, written at their place in the depth-D tensor y; xc holds the coarse planes [clo, clo + Dcs)
    // compactly; cells mz0 .. mz0 + ncz_ - 1 along z (the whole tensor: zlo 0, zhi D, clo 0, Dcs D / 2, mz0 -1, ncz_ D / 2 + 1)
    static_assert(CH == 8 || CH == 16, "8 or 16 channels per thread");
    constexpr int QP = 32 / CH, NP = CH / 2;                                      // threads per cell; binary16 pairs per thread
    const int Dc = D >> 1, Hc = H >> 1, Wc = W >> 1;
    const size_t S = (size_t)D * H * W, Sc = (size_t)Dcs * Hc * Wc;
    const int nbk = blockIdx.y;                                                   // (n, blk)
    // grid: x over the (my, mx) cells of one z layer of cells (QP threads each), y = (n, blk), z = the layer: one 32-bit division per thread
    const unsigned t = blockIdx.x * 256u + threadIdx.x;
    const int q = (int)(t & (unsigned)(QP - 1));
    const unsigned cell = t / (unsigned)QP, ncx = (unsigned)Wc + 1u, ncy = (unsigned)Hc + 1u;
    const bool live = cell < ncx * ncy;
    const unsigned cc = live ? cell : 0u, cyi = cc / ncx;
    const int mx = (int)(cc - cyi * ncx) - 1, my = (int)cyi - 1, mz = (int)blockIdx.z + mz0;
    const int cz[2] = {max(mz, 0), min(mz + 1, Dc - 1)}, cy[2] = {max(my, 0), min(my + 1, Hc - 1)}, cx[2] = {max(mx, 0), min(mx + 1, Wc - 1)};
    const uint8_t *xs = xc + (size_t)N * nbo * Sc * 32;
    float f[H2 ? 1 : 8][H2 ? 1 : CH], sc[8];
    h2_t hf[H2 ? 8 : 1][H2 ? NP : 1];                         // H2: the rows' values as binary16 pairs (an e4m3 value is one exactly), formed once per cell
    unsigned sb[8], em = 0u;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const size_t row = (size_t)nbk * Sc + ((size_t)(cz[k >> 2] - clo) * Hc + cy[(k >> 1) & 1]) * Wc + cx[k & 1];
        unsigned w[CH / 4];
        if constexpr (CH == 8) { const uint2 v = *(const uint2 *)(xc + row * 32 + q * 8); w[0] = v.x; w[1] = v.y; }
        else { const uint4 v = *(const uint4 *)(xc + row * 32 + q * 16); w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w; }
#pragma unroll
        for (int j = 0; j < CH / 4; j++) {
            if constexpr (H2) {
                hf[k][2 * j] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[j], 1.f, false);
                hf[k][2 * j + 1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[j], 1.f, true);
            } else d_dec4_e4m3(w[j], f[k] + 4 * j);
        }
        sb[k] = xs[row]; em = max(em, sb[k]);
        sc[k] = d_mx_scale(sb[k]);
    }
    if constexpr (H2) {
#pragma unroll
        for (int k = 0; k < 8; k++) { const int de = (int)sb[k] - (int)em; sc[k] = de >= -126 ? __uint_as_float((unsigned)(127 + de) << 23) : 0.f; }     // 2^(e_row - e_max)
    }
    const float smax = d_mx_scale(em);
    // the blend weight of coarse row k for a fine voxel that is `far` axes away from it: (3/4)^(3 - far) (1/4)^far times the row's scale
    // (the products of .75 and .25 are exact, so this is the value of the reference's ((wz wy) wx) s). 32 per cell, shared by its 8 fine voxels
    const float cw[4] = {0.421875f, 0.140625f, 0.046875f, 0.015625f};
    float w32[H2 ? 1 : 8][4];
    _Float16 w16[H2 ? 8 : 1][4];                              // (the packed multiply-add takes one half as the multiplier of both products)
#pragma unroll
    for (int k = 0; k < 8; k++)
#pragma unroll
        for (int far = 0; far < 4; far++) {
            if constexpr (H2) w16[k][far] = (_Float16)(cw[far] * sc[k]); else w32[k][far] = cw[far] * sc[k];      // (round to nearest even)
        }
    // output rows: fine voxel p = (pz, py, px) of the cell is voxel (2 mz + 1 + pz, 2 my + 1 + py, 2 mx + 1 + px); row0 is p = 0's row in the
    // tensor (outside it for cells on the low borders, whose p = 0 is not stored)
    constexpr int RB = BY * 4;                                                    // bytes of a 32-channel row
    const long long row0 = (long long)nbk * (long long)S + ((long long)(2 * mz + 1) * H + (2 * my + 1)) * W + (2 * mx + 1);
    uint8_t *ys = y + (size_t)N * nbo * S * RB;
    const bool okz[2] = {2 * mz + 1 >= zlo && 2 * mz + 1 < zhi, 2 * mz + 2 >= zlo && 2 * mz + 2 < zhi};
    const bool oky[2] = {my >= 0, 2 * my + 2 < H}, okx[2] = {live && mx >= 0, live && 2 * mx + 2 < W};
    // the binary16 form can encode straight from the binary16 sums when widening them (x 2^e_max) is exact, i.e. no product leaves the
    // normal binary32 range: 2^-24 2^(e_max - 127) >= 2^-126 and 65504 2^(e_max - 127) < 2^128. Decided per wavefront
    const bool direct = H2 && BY == 4 && __builtin_amdgcn_ballot_w64(em < 25u || em > 238u) == 0ull;
    const float am_direct = __uint_as_float((em - 9u) << 23);                    // 2^-9 of the cell's scale: block maxima below it take the widened form (binary16 subnormals)
    int eq[4];                                                                     // the scale bytes of the four voxels of a z layer of the cell
#pragma unroll
    for (int p = 0; p < 8; p++) {
        const int pz = p >> 2, py = (p >> 1) & 1, px = p & 1;                     // p = 0 has its own coarse row at m, p = 1 at m + 1
        float acc[CH], am;
        h2_t hacc[H2 ? NP : 1];
        if constexpr (H2) {
            // two channels per packed fused multiply-add: each half rounds once, as the scalar form
#pragma unroll
            for (int i = 0; i < NP; i++) hacc[i] = (h2_t){(_Float16)0.f, (_Float16)0.f};
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int b = 0; b < 2; b++)
#pragma unroll
                    for (int c = 0; c < 2; c++) {
                        const int k = ((a ^ pz) << 2) | ((b ^ py) << 1) | (c ^ px);
#pragma unroll
                        for (int i = 0; i < NP; i++) hacc[i] = __builtin_elementwise_fma((h2_t){w16[k][a + b + c], w16[k][a + b + c]}, hf[k][i], hacc[i]);
                    }
            // max |sum| 2^e_max: the widening is monotone, so the largest sum gives the largest product (NaN sums are skipped, as fmaxf skips
            // them below; a product that is NaN - 0 x inf - counts as 0 there too)
            h2_t m = __builtin_elementwise_abs(hacc[0]);
#pragma unroll
            for (int i = 1; i < NP; i++) m = __builtin_elementwise_max(m, __builtin_elementwise_abs(hacc[i]));
            am = fmaxf(0.f, fmaxf((float)m.x, (float)m.y) * smax);
        } else {
#pragma unroll
            for (int i = 0; i < CH; i++) acc[i] = 0.f;
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int b = 0; b < 2; b++)
#pragma unroll
                    for (int c = 0; c < 2; c++) {
                        const int k = ((a ^ pz) << 2) | ((b ^ py) << 1) | (c ^ px);   // a = 0: the voxel's own coarse row, a = 1: its neighbour
#pragma unroll
                        for (int i = 0; i < CH; i++) acc[i] = fmaf(w32[k][a + b + c], f[k][i], acc[i]);
                    }
            am = 0.f;
#pragma unroll
            for (int i = 0; i < CH; i++) am = fmaxf(am, fabsf(acc[i]));
        }
        {   // the QP threads of the cell hold the row's 32 channels; am is a non-negative number (no NaN, no -0): it orders as its bit pattern
            unsigned au = __float_as_uint(am);
            au = max(au, d_quad_xor_u<1>(au));
            if constexpr (QP == 4) au = max(au, d_quad_xor_u<2>(au));
            am = __uint_as_float(au);
        }
        // the block's E8M0 byte; 255 for a block with an infinity (am is never NaN here)
        const bool inf = __float_as_uint(am) >= 0x7f800000u;
        const int eb = inf ? 255 : d_mx_expb_fin(am, BY == 8 ? MI_INVQ8 : MI_INVQ4);
        eq[p & 3] = eb;
        const bool ok = okz[pz] && oky[py] && okx[px];
        uint8_t *dst = y + (row0 + ((long long)pz * H + py) * W + px) * RB + q * (RB / QP);
        bool widen = true;                                                          // (uniform)
        if constexpr (H2 && BY == 4) widen = !direct || __builtin_amdgcn_ballot_w64(!(am >= am_direct) || inf) != 0ull;
        if (!widen) {
            if constexpr (H2 && BY == 4) {
                // (sum 2^(e_max - 127)) / 2^e = sum / 2^(e - e_max + 127): the same quotient, rounded once by the conversion either way
                const float ds = __uint_as_float((unsigned)(eb - (int)em + 127) << 23);
                unsigned w[NP / 4];
#pragma unroll
                for (int j = 0; j < NP / 4; j++) {
                    w[j] = 0u;
                    w[j] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(w[j], hacc[4 * j], ds, 0);
                    w[j] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(w[j], hacc[4 * j + 1], ds, 1);
                    w[j] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(w[j], hacc[4 * j + 2], ds, 2);
                    w[j] = __builtin_amdgcn_cvt_scalef32_pk_fp4_f16(w[j], hacc[4 * j + 3], ds, 3);
                }
                if (ok) { if constexpr (CH == 8) *(unsigned *)dst = w[0]; else *(uint2 *)dst = make_uint2(w[0], w[NP / 4 - 1]); }
            }
        } else {
            const int e = eb - 127;
            if constexpr (H2) {
#pragma unroll
                for (int i = 0; i < NP; i++) { acc[2 * i] = (float)hacc[i].x * smax; acc[2 * i + 1] = (float)hacc[i].y * smax; }
            }
            if (BY == 8) {
                unsigned o[CH / 4];
#pragma unroll
                for (int j = 0; j < CH / 4; j++) o[j] = d_enc4_e4m3(acc[4 * j], acc[4 * j + 1], acc[4 * j + 2], acc[4 * j + 3], e);
                if (ok) { if constexpr (CH == 8) *(uint2 *)dst = make_uint2(o[0], o[1]); else *(uint4 *)dst = make_uint4(o[0], o[1], o[CH / 4 - 2], o[CH / 4 - 1]); }
            } else {
                unsigned o[CH / 8];
#pragma unroll
                for (int j = 0; j < CH / 8; j++) o[j] = d_enc8_e2m1(acc + 8 * j, e);
                if (ok) { if constexpr (CH == 8) *(unsigned *)dst = o[0]; else *(uint2 *)dst = make_uint2(o[0], o[CH / 8 - 1]); }
            }
        }
        if ((p & 3) == 3) {
            // the scale bytes of the layer's four voxels: four threads per cell: thread q writes voxel (pz, q >> 1, q & 1); two: thread q the two of row q
            if constexpr (QP == 4) {
                const int ev = q == 0 ? eq[0] : q == 1 ? eq[1] : q == 2 ? eq[2] : eq[3];
                const bool oks = okz[pz] && (q & 2 ? oky[1] : oky[0]) && (q & 1 ? okx[1] : okx[0]);
                if (oks) ys[row0 + ((long long)pz * H + (q >> 1)) * W + (q & 1)] = (uint8_t)ev;
            } else {
                const int e0 = q ? eq[2] : eq[0], e1 = q ? eq[3] : eq[1];
                const bool oky_q = okz[pz] && (q ? oky[1] : oky[0]);
                uint8_t *yq = ys + row0 + ((long long)pz * H + q) * W;
                if (oky_q && okx[0]) yq[0] = (uint8_t)e0;
                if (oky_q && okx[1]) yq[1] = (uint8_t)e1;
            }
        }
    }
}
// fine planes [zlo, zhi) of the upsampled depth-D tensor, written at their place in the depth-D MX tensor y
void mi_restage_up_sub(const void *x, int xdt, int N, int C, int D, int H, int W, gnp_t gp, int Cg, void *y, int ybits, int zlo, int zhi, int h2) {
    if (!N || zhi <= zlo || !H || !W) return;
    if (xdt != 3 && xdt != 4) mi_die("fused-upsample input must be an MX tensor (dtype %d)", xdt);
    if ((D | H | W) & 1) mi_die("fused-upsample output dims must be even (%d %d %d)", D, H, W);
    const int nbo = (C + 31) / 32, Dc = D / 2;
    // cells mz cover fine planes 2 mz + 1, 2 mz + 2 and read coarse planes mz, mz + 1 (clamped)
    const int mz0 = (zlo - 2) >> 1 < -1 ? -1 : (zlo - 2) >> 1, mz1 = (zhi - 2) >> 1, ncz = mz1 - mz0 + 1;
    const int clo = mz0 < 0 ? 0 : mz0, chi = (mz1 + 1 > Dc - 1 ? Dc - 1 : mz1 + 1) + 1, Dcs = chi - clo;
    const size_t Scp = (size_t)(H / 2) * (W / 2);
    uint8_t *xc = (uint8_t *)mi_ws(MI_WS_UPCOARSE, (size_t)N * nbo * Dc * Scp * 33);          // the coarse tensor's geometry; planes [clo, clo + Dcs) are filled
    mi_restage_sub(x, xdt, N, C, (size_t)Dcs * Scp, gp, Cg, 0, xc, 8, (size_t)Dc * Scp, (size_t)clo * Scp);
    const size_t cells = (size_t)(H / 2 + 1) * (W / 2 + 1);                                   // per z layer of cells
    if ((size_t)N * nbo > 65535 || ncz > 65535) mi_die("fused upsample: launch grid (%d x %d blocks, %d cell layers)", N, nbo, ncz);
    const dim3 grid(nblk_(cells * (h2 ? 2 : 4), 256), (unsigned)(N * nbo), (unsigned)ncz);      // (threads per cell: two in the binary16 blend, four in the fp32 one)
#define UB(BY, H2) up_blend_k<BY, H2><<<grid, 256>>>(xc, (uint8_t *)y, N, nbo, D, H, W, zlo, zhi, 0, Dc, mz0, ncz)
    if (ybits == 4) { if (h2) UB(4, true); else UB(4, false); } else { if (h2) UB(8, true); else UB(8, false); }
#undef UB
    MICK();
}
void mi_restage_up(const void *x, int xdt, int N, int C, int D, int H, int W, gnp_t gp, int Cg, void *y, int ybits, int h2) { mi_restage_up_sub(x, xdt, N, C, D, H, W, gp, Cg, y, ybits, 0, D, h2); }

// weights w [Co][Ci][T] rounded in place to MX-fp4 values with one E8M0 scale per Bo x Bi (output x input channel) block and tap (src/lp_mx_cvt.cu:369-395):
// the forward's per-output-channel blocks of 32 inputs inside a 32 x 32 block then re-quantise these values exactly.
// The taps are the innermost index of the weight array, so a block's rows are runs of Bi x T contiguous floats: one workgroup takes a whole
// block with all its taps and walks those runs with consecutive lanes on consecutive floats. First walk: every tap's maximum magnitude into
// its LDS word (non-negative floats order as their bit patterns; NaN skipped, as fmaxf drops it); second walk: each float rounded at its
// tap's scale and written back.
__global__ void __launch_bounds__(256) fakeq_w4_k(float *w, int Co, int Ci, int T, int Bo, int Bi, int col_blocks) {
    extern __shared__ unsigned tap_max[];                     // [T] bit patterns of the taps' maxima, then [T] their exponents
    int *tap_exp = (int *)(tap_max + T);
    const int row0 = (int)(blockIdx.x / col_blocks) * Bo, col0 = (int)(blockIdx.x % col_blocks) * Bi;
    const int rows = min(Bo, Co - row0), run = min(Bi, Ci - col0) * T;                   // floats of the block per output row
    float *base = w + ((size_t)row0 * Ci + col0) * T;
    const size_t pitch = (size_t)Ci * T;
    for (int t = threadIdx.x; t < T; t += blockDim.x) tap_max[t] = 0u;
    __syncthreads();
    const int total = rows * run;
    for (int k = threadIdx.x; k < total; k += blockDim.x) {
        const int rr = k / run, j = k - rr * run;
        const float v = fabsf(base[rr * pitch + j]);
        if (v == v) atomicMax(&tap_max[j % T], __float_as_uint(v));
    }
    __syncthreads();
    for (int t = threadIdx.x; t < T; t += blockDim.x) tap_exp[t] = d_mx_exp(__uint_as_float(tap_max[t]), MI_INVQ4);
    __syncthreads();
    for (int k = threadIdx.x; k < total; k += blockDim.x) {
        const int rr = k / run, j = k - rr * run, ex = tap_exp[j % T];
        float *q = base + rr * pitch + j;
        *q = d_dec_e2m1(d_enc_e2m1(*q * d_exp2i(-ex))) * d_exp2i(ex);
    }
}
extern "C" void lp_fakeq_w4(float *w, int Co, int Ci, int T, int Bo, int Bi) {
    if (Co <= 0 || Ci <= 0 || T <= 0 || Bo <= 0 || Bi <= 0) return;
    const int row_blocks = (Co + Bo - 1) / Bo, col_blocks = (Ci + Bi - 1) / Bi;
    if ((size_t)row_blocks * col_blocks > 0x7fffffffu || (size_t)T * 8 > 48 * 1024 || (size_t)Bo * Bi * T > 0x7fffffffu) mi_die("lp_fakeq_w4: %d x %d weights, %d taps in blocks of %d x %d", Co, Ci, T, Bo, Bi);
    fakeq_w4_k<<<(unsigned)(row_blocks * col_blocks), 256, (size_t)T * 8>>>(w, Co, Ci, T, Bo, Bi, col_blocks);
    MICK();
}
extern "C" void nn_fakeq_w4_2d(float *w, int Co, int Ci, int T, int B) { lp_fakeq_w4(w, Co, Ci, T, B, B); }      // src/nn_elem.cu:192
