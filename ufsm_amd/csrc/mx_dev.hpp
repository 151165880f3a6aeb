// Device-side MX arithmetic for gfx950: E8M0 scale selection, e4m3 / e2m1 element encode / decode, block-row helpers.
// Semantics follow the reference's conversion routines (src/lp_common.cuh:484-555, src/mx_sw.cuh:1-56); the formulations are this
// build's own (magic-number rounding for e4m3, midpoint thresholds for e2m1) and are checked bit for bit on the device.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/mi_lp.h"

#define MI_INVQ8 (1.f / 448.f)
#define MI_INVQ4 (1.f / 6.f)

__host__ __device__ __forceinline__ int mx_bw(int C) { return C <= 8 ? 8 : C <= 16 ? 16 : 32; }       // src/lp_common.cuh:132
__host__ __device__ __forceinline__ int mx_nb(int C) { const int bw = mx_bw(C); return (C + bw - 1) / bw; }
__host__ __device__ __forceinline__ int mx_rb(int bw, int bits) { return bw * bits / 8; }

// scale exponent: smallest e with amax * fl(1 / qmax) <= 2^e, clamped; NaN / inf (or an overflowing product) -> 128 (src/lp_common.cuh:492-500)
__device__ __forceinline__ int d_mx_exp(float amax, float inv_qmax) {
    const unsigned u = __float_as_uint(amax * inv_qmax) & 0x7fffffffu;
    const int e = (int)(u >> 23) - 127 + ((u & 0x7fffffu) ? 1 : 0);
    const int ec = e < -126 ? -126 : e > 126 ? 126 : e;
    return u >= 0x7f800000u ? 128 : ec;
}
// d_mx_exp(amax, inv_qmax) + 127, i.e. the E8M0 byte itself, of a finite amax >= 0 (not NaN, not -0): adding 0x7fffff to the bits carries into
// the exponent field exactly when the mantissa is not zero
__device__ __forceinline__ int d_mx_expb_fin(float amax, float inv_qmax) {
    const unsigned u = __float_as_uint(amax * inv_qmax);
    const int eb = (int)((u + 0x7fffffu) >> 23);
    return eb < 1 ? 1 : eb > 253 ? 253 : eb;
}
__device__ __forceinline__ float d_exp2i(int e) { return __uint_as_float((unsigned)(127 + e) << 23); }   // e = -128: the bits of -inf, as the reference (src/lp_common.cuh:501)
__device__ __forceinline__ float d_mx_scale(unsigned sbyte) { return __uint_as_float((sbyte & 255u) << 23); }   // 0xFF -> +inf

// NaN-propagating |v| max on the bit patterns (src/lp_common.cuh:487)
// the value of lane ^ M (M 1 or 2: inside the lane's group of four) through the vector pipe's lane permute: no LDS round trip. Every lane
// of the group must be active
template <int M> __device__ __forceinline__ unsigned d_quad_xor_u(unsigned x) {
    static_assert(M == 1 || M == 2, "d_quad_xor_u: lanes of one group of four");
    return (unsigned)__builtin_amdgcn_mov_dpp((int)x, M == 1 ? 0xB1 : 0x4E, 0xF, 0xF, true);        // quad_perm [1, 0, 3, 2] / [2, 3, 0, 1]
}
template <int M> __device__ __forceinline__ float d_quad_xor_f(float x) { return __uint_as_float(d_quad_xor_u<M>(__float_as_uint(x))); }
// the value of lane 7 - i of the lane's group of eight (row_half_mirror): after the two exchanges inside the groups of four, every lane of a
// group of four holds the same partial result, and this brings the other group's - the third step of a reduction over eight lanes
__device__ __forceinline__ unsigned d_oct_mirror_u(unsigned x) { return (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0x141, 0xF, 0xF, true); }
__device__ __forceinline__ float d_oct_mirror_f(float x) { return __uint_as_float(d_oct_mirror_u(__float_as_uint(x))); }
__device__ __forceinline__ unsigned d_amax_u(unsigned a, float v) { const unsigned b = __float_as_uint(v) & 0x7fffffffu; return b > a ? b : a; }

// e4m3 (OCP FN: max 448, 0x7f NaN), round to nearest even, saturating. For |x| < 448 the value is rounded to a multiple of the
// binade's quantum 2^(E-3) (E >= -6) by adding and subtracting 1.5 * 2^(E+20), whose ulp is that quantum; the rounded value is
// exactly representable, so its code is a re-biased bit field (normal) or value * 2^9 (subnormal).
__device__ __forceinline__ unsigned d_enc_e4m3(float x) {
    const unsigned u = __float_as_uint(x), a = u & 0x7fffffffu;
    unsigned ef = a >> 23; ef = ef < 121u ? 121u : ef; ef = ef > 136u ? 136u : ef;
    const float M = __uint_as_float(((ef + 20u) << 23) | 0x400000u);
    const float ax = __uint_as_float(a);
    float r = ax + M;
    asm volatile("" : "+v"(r));            // keep (ax + M) - M as two rounded operations
    r -= M;
    const unsigned rb = __float_as_uint(r);
    unsigned code = rb >= 0x3c800000u ? (rb >> 20) - 0x3c0u : (unsigned)(r * 512.f);
    code = a >= 0x43e00000u ? 0x7eu : code;             // >= 448 (incl. inf) saturates
    code |= (u >> 24) & 0x80u;
    return a > 0x7f800000u ? 0x7fu : code;              // NaN of either sign
}
__device__ __forceinline__ unsigned d_enc_e4m3x4(float a, float b, float c, float d) {
    return d_enc_e4m3(a) | (d_enc_e4m3(b) << 8) | (d_enc_e4m3(c) << 16) | (d_enc_e4m3(d) << 24);
}
// e2m1: grid {0, .5, 1, 1.5, 2, 3, 4, 6}; the code is the number of midpoints passed, ties to the even code; > 6 -> 6; NaN -> +6
__device__ __forceinline__ unsigned d_enc_e2m1(float x) {
    const unsigned u = __float_as_uint(x), a = u & 0x7fffffffu;
    const float ax = __uint_as_float(a);
    unsigned c = (unsigned)(ax > 0.25f) + (unsigned)(ax >= 0.75f) + (unsigned)(ax > 1.25f) + (unsigned)(ax >= 1.75f) +
                 (unsigned)(ax > 2.5f) + (unsigned)(ax >= 3.5f) + (unsigned)(ax > 5.f);
    c |= (u >> 28) & 8u;
    return a > 0x7f800000u ? 7u : c;
}
__device__ __forceinline__ unsigned d_enc_e2m1x8(const float *v, float m) {   // 8 values -> 8 nibbles, v[0] lowest
    unsigned w = 0u;
#pragma unroll
    for (int k = 0; k < 8; k++) w |= d_enc_e2m1(v[k] * m) << (4 * k);
    return w;
}
// decoders (exact): e4m3 byte, e2m1 nibble -> fp32
__device__ __forceinline__ float d_dec_e4m3(unsigned b) {
    const unsigned em = b & 0x7fu, e = em >> 3, m = em & 7u;
    // normal: 1.m * 2^(e-7) -> fp32 field; subnormal: m * 2^-9 as an exact int -> float product
    const float nv = __uint_as_float(((e + 120u) << 23) | (m << 20));
    float v = e ? nv : (float)m * 0.001953125f;
    v = em == 0x7fu ? __uint_as_float(0x7fc00000u) : v;
    return __uint_as_float(__float_as_uint(v) | ((b & 0x80u) << 24));
}
__device__ __forceinline__ float d_dec_e2m1(unsigned n) {
    const unsigned c = n & 7u;
    // {0, .5, 1, 1.5, 2, 3, 4, 6} = mantissa bit c & 1, exponent (c >> 1): c < 2 is the subnormal pair {0, .5}
    const float v = c < 2u ? 0.5f * (float)c : __uint_as_float(((126u + (c >> 1)) << 23) | ((c & 1u) << 22));
    return (n & 8u) ? -v : v;
}

// ---- hardware conversions of gfx950 (v_cvt_scalef32_pk_fp8_f32 / _fp4_f32, v_cvt_pk_f32_fp8, v_cvt_scalef32_pk_f32_fp4) ----
// Checked on the device against the software encoders above over all 2^32 fp32 inputs: the fp8 instruction agrees for every |x| <= 464
// (round to nearest even, subnormals included) but returns NaN instead of saturating beyond, and encodes NaN differently; the fp4
// instruction agrees for every finite input and infinities (saturating), not for negative NaN; both decoders agree on every code.
// A finite block never scales past 448 (1 + 2^-23), so the hardware encoders serve every block whose exponent is not 128 (the
// non-finite marker); those rare blocks take the software encoders. The scale operand divides: x / 2^e, exact for a power of two.
typedef short mi_v2s __attribute__((ext_vector_type(2)));
typedef float mi_v2f __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned d_enc_e4m3x4_hw(float a, float b, float c, float d, float pow2e) {
    mi_v2s o = __builtin_bit_cast(mi_v2s, a);                  // (any bits: each conversion writes one half of the word, the two write both)
    o = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(o, a, b, pow2e, false);
    o = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(o, c, d, pow2e, true);
    return __builtin_bit_cast(unsigned, o);
}
__device__ __forceinline__ unsigned d_enc_e2m1x8_hw(const float *v, float pow2e) {
    unsigned w = 0u;
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[0], v[1], pow2e, 0);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[2], v[3], pow2e, 1);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[4], v[5], pow2e, 2);
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, v[6], v[7], pow2e, 3);
    return w;
}
// encode with the block exponent e. 128 marks a block holding an infinity or NaN: the reference then multiplies by exp2i(-128), the
// bits of -inf (src/lp_common.cuh:501), so a finite non-zero value or an infinity saturates with the opposite sign and a zero or a
// NaN becomes NaN. Those codes have a closed form; they are formed under a wave-uniform branch that finite data never takes.
__device__ __forceinline__ unsigned d_enc_e4m3_nf(float x) {
    const unsigned u = __float_as_uint(x), a = u & 0x7fffffffu;
    return (a == 0u || a > 0x7f800000u) ? 0x7fu : (0x7eu | ((~u >> 24) & 0x80u));
}
__device__ __forceinline__ unsigned d_enc_e2m1_nf(float x) {
    const unsigned u = __float_as_uint(x), a = u & 0x7fffffffu;
    return (a == 0u || a > 0x7f800000u) ? 7u : (7u | ((~u >> 28) & 8u));
}
__device__ __forceinline__ unsigned d_enc4_e4m3_nf(float a, float b, float c, float d) {
    return d_enc_e4m3_nf(a) | (d_enc_e4m3_nf(b) << 8) | (d_enc_e4m3_nf(c) << 16) | (d_enc_e4m3_nf(d) << 24);
}
__device__ __forceinline__ unsigned d_enc8_e2m1_nf(const float *v) {
    unsigned w = 0u;
#pragma unroll
    for (int k = 0; k < 8; k++) w |= d_enc_e2m1_nf(v[k]) << (4 * k);
    return w;
}
__device__ __forceinline__ unsigned d_enc4_e4m3(float a, float b, float c, float d, int e) {
    unsigned w = d_enc_e4m3x4_hw(a, b, c, d, d_exp2i(e));
    if (__builtin_amdgcn_ballot_w64(e == 128) != 0ull) {
        if (e == 128) w = d_enc4_e4m3_nf(a, b, c, d);
    }
    return w;
}
__device__ __forceinline__ unsigned d_enc8_e2m1(const float *v, int e) {
    unsigned w = d_enc_e2m1x8_hw(v, d_exp2i(e));
    if (__builtin_amdgcn_ballot_w64(e == 128) != 0ull) {
        if (e == 128) w = d_enc8_e2m1_nf(v);
    }
    return w;
}
// decode one word: 4 e4m3 bytes / 8 e2m1 nibbles -> floats (unscaled)
__device__ __forceinline__ void d_dec4_e4m3(unsigned w, float *v) {
    const mi_v2f lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false), hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
    v[0] = lo[0]; v[1] = lo[1]; v[2] = hi[0]; v[3] = hi[1];
}
__device__ __forceinline__ void d_dec8_e2m1(unsigned w, float *v) {
    const mi_v2f a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1);
    const mi_v2f c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3);
    v[0] = a[0]; v[1] = a[1]; v[2] = b[0]; v[3] = b[1]; v[4] = c[0]; v[5] = c[1]; v[6] = d[0]; v[7] = d[1];
}

// one block row of bw values -> codes + scale byte. NANPROP: the NaN-propagating amax of the converters and elementwise ops
// (src/lp_mxops.cuh:45-65), else fmaxf (conv staging, src/lp_f8fwd.cuh:91). codes: 8 words (fp8) / 4 words (fp4), zero past bw.
template <int BITS, bool NANPROP>
__device__ __forceinline__ unsigned d_quant_row(const float *v, int bw, unsigned *codes) {
    float amax;
    if (NANPROP) {
        unsigned am = 0u;
#pragma unroll
        for (int k = 0; k < 32; k++) if (k < bw) am = d_amax_u(am, v[k]);
        amax = __uint_as_float(am);
    } else {
        amax = 0.f;
#pragma unroll
        for (int k = 0; k < 32; k++) if (k < bw) amax = fmaxf(amax, fabsf(v[k]));
    }
    const int e = d_mx_exp(amax, BITS == 8 ? MI_INVQ8 : MI_INVQ4);
    if (BITS == 8) {
#pragma unroll
        for (int j = 0; j < 8; j++) codes[j] = 4 * j < bw ? d_enc4_e4m3(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3], e) : 0u;
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) codes[j] = 8 * j < bw ? d_enc8_e2m1(v + 8 * j, e) : 0u;
    }
    return (unsigned)(e + 127);
}
// decode a row held in words (8 words fp8 / 4 words fp4) times the scale
// The converting instructions take the scale as an operand: checked on the device over every code and scale byte, their result equals
// decode x d_mx_scale(sbyte) bit for bit for the scale bytes 1 .. 254 (subnormal and overflowing products included) and differs for 0 (the
// reference's scale is 0.0 there, the instruction's 2^-127) and 255 (inf against NaN). Wavefronts that hold neither byte take the one-instruction
// form; the others decode and multiply.
__device__ __forceinline__ bool d_scale_plain(unsigned sbyte) { return __builtin_amdgcn_ballot_w64(((sbyte + 1u) & 255u) < 2u) == 0ull; }
__device__ __forceinline__ void d_dec4_e4m3_scaled(unsigned w, float s, float *v) {
    const mi_v2f lo = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(w, s, false), hi = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(w, s, true);
    v[0] = lo[0]; v[1] = lo[1]; v[2] = hi[0]; v[3] = hi[1];
}
__device__ __forceinline__ void d_dec8_e2m1_scaled(unsigned w, float s, float *v) {
    const mi_v2f a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, s, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, s, 1);
    const mi_v2f c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, s, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, s, 3);
    v[0] = a[0]; v[1] = a[1]; v[2] = b[0]; v[3] = b[1]; v[4] = c[0]; v[5] = c[1]; v[6] = d[0]; v[7] = d[1];
}
template <int BITS>
__device__ __forceinline__ void d_dequant_row(const unsigned *codes, unsigned sbyte, float *v) {
    const float s = d_mx_scale(sbyte);
    if (d_scale_plain(sbyte)) {
        if (BITS == 8) {
#pragma unroll
            for (int j = 0; j < 8; j++) d_dec4_e4m3_scaled(codes[j], s, v + 4 * j);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) d_dec8_e2m1_scaled(codes[j], s, v + 8 * j);
        }
        return;
    }
    if (BITS == 8) {
#pragma unroll
        for (int j = 0; j < 8; j++) d_dec4_e4m3(codes[j], v + 4 * j);
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) d_dec8_e2m1(codes[j], v + 8 * j);
    }
#pragma unroll
    for (int k = 0; k < 32; k++) v[k] *= s;
}
// load the words of a stored row of bw channels (zero past the row)
template <int BITS>
__device__ __forceinline__ void d_load_row_words(const uint8_t *p, int bw, unsigned *w) {
    constexpr int NW = BITS == 8 ? 8 : 4;
#pragma unroll
    for (int j = 0; j < NW; j++) w[j] = 0u;
    const int nbytes = mx_rb(bw, BITS);
    if (nbytes == 32) { const uint4 a = *(const uint4 *)p, b = *(const uint4 *)(p + 16); w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w; if (NW == 8) { w[4] = b.x; w[5] = b.y; w[6] = b.z; w[7] = b.w; } }
    else if (nbytes == 16) { const uint4 a = *(const uint4 *)p; w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w; }
    else if (nbytes == 8) { const uint2 a = *(const uint2 *)p; w[0] = a.x; w[1] = a.y; }
    else w[0] = *(const unsigned *)p;
}
template <int BITS>
__device__ __forceinline__ void d_store_row_words(uint8_t *p, int bw, const unsigned *w) {
    const int nbytes = mx_rb(bw, BITS);
    if (nbytes == 32) { *(uint4 *)p = make_uint4(w[0], w[1], w[2], w[3]); *(uint4 *)(p + 16) = make_uint4(w[BITS == 8 ? 4 : 0], w[BITS == 8 ? 5 : 0], w[BITS == 8 ? 6 : 0], w[BITS == 8 ? 7 : 0]); }
    else if (nbytes == 16) *(uint4 *)p = make_uint4(w[0], w[1], w[2], w[3]);
    else if (nbytes == 8) *(uint2 *)p = make_uint2(w[0], w[1]);
    else *(unsigned *)p = w[0];
}
// GN + SiLU of the conv staging (src/lp_common.cuh:474-482): u = fma(x, a, b), then u * sigmoid(u) (= h + h tanh(h), h = u / 2)
// silu(u) = u / (1 + exp(-u)) by the hardware exponential and reciprocal (v_exp_f32, v_rcp_f32: about 2 ulp in all; a true division
// would be eleven more instructions per element, and every kernel that applies it is bound by its instruction count). u -> -inf: the
// exponential overflows to inf, its reciprocal is 0 and the product -0
__device__ __forceinline__ float d_silu(float u) { return u * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(u * -1.44269504f)); }
__device__ __forceinline__ float d_act_ab(float v, float a, float b) {
    const float u = fmaf(v, a, b);
    return d_silu(u);
}

// exact fixed-point GroupNorm sum slot add (src/gnacc.cuh:12-20): slot = [fraction, 2^-64 units][integer part][non-finite count];
// integer atomics, so the sums do not depend on the order of the adds
__device__ __forceinline__ void gn_acc_add(double *b, size_t i, double v) {
    unsigned long long *w = (unsigned long long *)b + 3 * i;
    if (!(fabs(v) < 4.611686018427387904e18)) { atomicAdd(&w[2], 1ull); return; }
    const double f = floor(v);
    const long long hi = (long long)f;
    const unsigned long long lo = (unsigned long long)((v - f) * 18446744073709551616.0);
    if (lo) { const unsigned long long o = atomicAdd(&w[0], lo); if (o + lo < o) atomicAdd(&w[1], 1ull); }
    if (hi) atomicAdd(&w[1], (unsigned long long)hi);
}

// ---- host-side shared declarations of the library's units ----
void mi_restage(const void *x, int xdt, int N, int C, size_t S, gnp_t gp, int Cg, int cg0, void *y, int ybits);
void mi_restage_up(const void *x, int xdt, int N, int C, int D, int H, int W, gnp_t gp, int Cg, void *y, int ybits, int h2);    // h2: the binary16 blend
// the MX GEMM with A's rows quantised by the kernel that produces them (csrc/mx_gemm.hip): where to write them, then the product
bool mi_mx_gemm_abuf(int bits, int M, int N, int K, uint8_t **Aq, uint8_t **As);
int mi_mx_gemm_apacked(int bits, int tb, int M, int N, int K, const float *B, float *C, float beta, const float *bias, const float *res);
// the same with A's packed rows and scales anywhere in device memory
int mi_mx_gemm_apacked_at(int bits, int tb, int M, int N, int K, const uint8_t *Aq, const uint8_t *As, const float *B, float *C, float beta, const float *bias, const float *res);
// the up projection and the SwiGLU in one kernel (e4m3): g[t][f] = silu(h[t][f]) h[t][F + f], h = x W^T + b with x's packed rows where
// mi_mx_gemm_abuf(8, T, 2 F, C) said and W [2 F][C] row-major, written as the packed A operand (gq, gs) of the down projection; h is not stored
int mi_mx_gemm_glu(int T, int F, int C, const float *W, const float *bias, uint8_t *gq, uint8_t *gs);
void mi_restage_sub(const void *x, int xdt, int N, int C, size_t S, gnp_t gp, int Cg, int cg0, void *y, int ybits, size_t Ss, size_t v0);     // only voxels [v0, v0 + S) of tensors of Ss voxels
void mi_restage_sub2(const void *x, int N, int C, size_t S, gnp_t gp, void *y8, void *y4, size_t Ss, size_t v0);      // MX-fp8 source, 32-wide blocks: both formats from one read
void mi_restage_up_sub(const void *x, int xdt, int N, int C, int D, int H, int W, gnp_t gp, int Cg, void *y, int ybits, int zlo, int zhi, int h2);   // only fine planes [zlo, zhi)
void mi_post_error(hipError_t e, const char *file, int line);
#define MICK() do { hipError_t e_ = hipGetLastError(); if (e_ != hipSuccess) mi_post_error(e_, __FILE__, __LINE__); } while (0)
#define MIRT(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) mi_post_error(e_, __FILE__, __LINE__); } while (0)
void *mi_ws(int slot, size_t bytes);        // per-device grow-on-demand scratch (the reference's nn_ws, src/nn_core.cu:751)
void mi_ws_arena(void *base, size_t cap);   // the calling thread's scratch requests come from this fixed region until mi_ws_arena(nullptr, 0)
bool mi_ws_arena_on(void);
void mi_count_alloc(void);                  // bookkeeping: one more device allocation made by the library
enum { MI_WS_WQ = 0, MI_WS_WSC = 1, MI_WS_XSTAGE = 2, MI_WS_X2STAGE = 3, MI_WS_MISC = 4, MI_WS_UPCOARSE = 5, MI_WS_GEMM = 6, MI_WS_ATTN = 7, MI_WS_GEMM2 = 8, MI_WS_RAY = 9, MI_WS_NSLOTS = 10 };
static inline unsigned nblk_(size_t n, unsigned b) { return (unsigned)((n + b - 1) / b); }
[[noreturn]] void mi_die(const char *fmt, ...);
// ---- slab-local GroupNorm statistics (gnp_t.ns > 0: src/nn_lp.h:15-18, src/lp_slab.cuh:7-12): the statistics hold one row per (sample,
// z-slab), [n][ns][G]; plane z of the tensor reads row n * ns + clamp((z + zo) / zs, 0, ns - 1). The kernels here read ONE row per sample and
// launch: the host walks the slabs that meet the planes a launch covers and hands each launch a gnp_t resolved to its slab (zs = 0, zo = the
// slab's index), which d_gn_row turns into the row. ns == 0: the per-sample statistics, row n. ----
__device__ __forceinline__ int d_gn_row(const gnp_t &g, int n) { return g.ns ? n * g.ns + g.zo : n; }
// f(z0, z1, g) for the planes [z0, z1) of each slab that meets [zlo, zhi) (once, with g itself, for per-sample statistics); hw: the tensor's
// voxels per plane, which the geometry must agree with
template <class F> static void gn_for_slabs(const char *who, gnp_t g, int hw, int zlo, int zhi, F f) {
    if (!g.G || !g.ns) { f(zlo, zhi, g); return; }
    if (g.zs <= 0 || g.zo < 0 || g.zo >= g.zs || g.zhw != hw) mi_die("%s: slab-local GroupNorm geometry (zs %d, zo %d, ns %d, zhw %d) does not fit planes of %d voxels", who, g.zs, g.zo, g.ns, g.zhw, hw);
    for (int s = 0; s < g.ns; s++) {
        const long long a = s == 0 ? zlo : (long long)s * g.zs - g.zo, b = s == g.ns - 1 ? zhi : (long long)(s + 1) * g.zs - g.zo;
        const int z0 = (int)(a > zlo ? a : zlo), z1 = (int)(b < zhi ? b : zhi);
        if (z0 < z1) { gnp_t r = g; r.zs = 0; r.zo = s; f(z0, z1, r); }
    }
}

