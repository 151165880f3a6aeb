/* CPU oracle: see mx_oracle.h. Test infrastructure, never linked into the shipped GPU library.
   Build: gcc -O3 -march=native -ffp-contract=off -fopenmp -shared -fPIC (no fast-math: the quantiser is bit-exact). */
#include "mx_oracle.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
int orc_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---------- block geometry (src/lp_common.cuh:132-134) ---------- */
int orc_mx_bw(int C) { return C <= 8 ? 8 : C <= 16 ? 16 : 32; }
int orc_mx_nb(int C) { int bw = orc_mx_bw(C); return (C + bw - 1) / bw; }
static int rowbytes(int bw, int bits) { return bw * bits / 8; }
size_t orc_mx_bytes(int bits, int N, int C, size_t S) { return (size_t)N * orc_mx_nb(C) * S * (rowbytes(orc_mx_bw(C), bits) + 1); }

/* ---------- scale selection (src/lp_common.cuh:492-501): the product with the rounded reciprocal, exponent rounded up ---------- */
int orc_mx_exp(float amax, float inv_qmax) {
    const uint32_t u = f2u(amax * inv_qmax) & 0x7fffffffu;
    if (u >= 0x7f800000u) return 128;                       /* NaN, inf, or the product overflowed */
    int e = (int)(u >> 23) - 127 + ((u & 0x7fffffu) ? 1 : 0);
    return e < -126 ? -126 : e > 126 ? 126 : e;
}
float orc_exp2i(int e) { return u2f((uint32_t)(127 + e) << 23); }   /* e = -128 gives the bits of -inf, as the reference's shift does */
float orc_mx_scale(unsigned sbyte) { return u2f((uint32_t)(sbyte & 255u) << 23); }   /* 0xFF -> +inf (src/lp_common.cuh:186) */
static const float INVQ8 = 1.f / 448.f, INVQ4 = 1.f / 6.f;

/* ---------- element decode (src/mx_sw.cuh:78-87) ---------- */
float orc_dec_e4m3(unsigned b) {
    const unsigned e = (b >> 3) & 15u, m = b & 7u;
    if ((b & 0x7fu) == 0x7fu) return u2f(0x7fc00000u | ((b & 0x80u) << 24));
    const float v = e ? ldexpf((float)(8u + m), (int)e - 10) : ldexpf((float)m, -9);
    return (b & 0x80u) ? -v : v;
}
static const float E2M1_GRID[8] = {0.f, 0.5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f};
float orc_dec_e2m1(unsigned n) { const float v = E2M1_GRID[n & 7u]; return (n & 8u) ? -v : v; }

/* ---------- element encode: round to nearest, ties to even code, saturating (semantics of src/mx_sw.cuh:1-12) ----------
   e4m3: arithmetic formulation. The quantum of the binade holding |x| is 2^(max(E, -6) - 3); |x| / quantum is an exact
   power-of-two scaling, rintf rounds it to nearest-even (default rounding mode), and the rounded multiple maps to a code. */
unsigned orc_enc_e4m3(float x) {
    const uint32_t u = f2u(x), s = (u >> 24) & 0x80u, a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return 0x7fu;                      /* NaN of either sign */
    const float ax = u2f(a);
    if (ax >= 448.f) return s | 0x7eu;                      /* 448..464 would round to 448 anyway, the rest saturates */
    if (ax < 0x1p-11f) return s;                            /* below half the subnormal step 2^-9 (2^-10 itself ties to even 0) */
    int ex; (void)frexpf(ax, &ex);                          /* ax = f 2^ex, f in [0.5, 1): binade exponent ex - 1 */
    int E = ex - 1; if (E < -6) E = -6;
    const float k = rintf(ldexpf(ax, 3 - E));               /* multiple of the quantum, 0..16 */
    if (E == -6 && k < 8.f) return s | (unsigned)k;         /* subnormal codes 0..7 */
    unsigned ki = (unsigned)k;
    if (ki == 16u) { ki = 8u; E++; }                        /* rounded up into the next binade */
    return s | (((unsigned)(E + 7) << 3) | (ki - 8u));
}
/* e2m1: threshold formulation on the midpoints of {0, .5, 1, 1.5, 2, 3, 4, 6}; a tie goes to the even code */
unsigned orc_enc_e2m1(float x) {
    const uint32_t u = f2u(x), s = (u >> 28) & 8u, a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return 7u;                         /* NaN -> +6 */
    const float ax = u2f(a);
    unsigned c;
    if (ax <= 0.25f) c = 0; else if (ax < 0.75f) c = 1; else if (ax <= 1.25f) c = 2; else if (ax < 1.75f) c = 3;
    else if (ax <= 2.5f) c = 4; else if (ax < 3.5f) c = 5; else if (ax <= 5.f) c = 6; else c = 7;
    return s | c;
}
/* the pins: nearest grid point by exhaustive scan of the code values; exact-midpoint ties to the even code; no arithmetic on x
   beyond exact differences in double */
unsigned orc_ref_e4m3(float x) {
    const uint32_t u = f2u(x), s = (u >> 24) & 0x80u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fu;
    const double a = fabs((double)x);
    if (a >= 448.0) return s | 0x7eu;                       /* saturation: beyond the largest grid value (also keeps the differences below exact) */
    unsigned best = 0; double bd = INFINITY;
    for (unsigned c = 0; c <= 0x7eu; c++) {
        const double d = fabs((double)orc_dec_e4m3(c) - a);
        if (d < bd || (d == bd && !(c & 1u))) { bd = d; best = c; }
    }
    return s | best;
}
unsigned orc_ref_e2m1(float x) {
    const uint32_t u = f2u(x), s = (u >> 28) & 8u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return 7u;
    const double a = fabs((double)x);
    if (a >= 6.0) return s | 7u;
    unsigned best = 0; double bd = INFINITY;
    for (unsigned c = 0; c < 8u; c++) {
        const double d = fabs((double)E2M1_GRID[c] - a);
        if (d < bd || (d == bd && !(c & 1u))) { bd = d; best = c; }
    }
    return s | best;
}
uint64_t orc_enc_sweep(uint32_t first, uint64_t count, uint32_t stride, uint32_t *bad) {
    uint64_t nbad = 0; uint32_t firstbad = 0; int have = 0;
    if (!stride) stride = 1;
    const uint64_t n = (count + stride - 1) / stride;
#pragma omp parallel for schedule(static) reduction(+ : nbad)
    for (uint64_t i = 0; i < n; i++) {
        const uint32_t u = first + (uint32_t)(i * stride);
        const float x = u2f(u);
        if (orc_enc_e4m3(x) != orc_ref_e4m3(x) || orc_enc_e2m1(x) != orc_ref_e2m1(x)) {
            nbad++;
#pragma omp critical
            { if (!have || u < firstbad) { firstbad = u; have = 1; } }
        }
    }
    if (bad) *bad = firstbad;
    return nbad;
}

/* ---------- fp16 (IEEE binary16) conversions, round to nearest even ---------- */
uint16_t orc_f32_to_h16(float f) {
    const uint32_t u = f2u(f), s = (u >> 16) & 0x8000u, a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(s | 0x7e00u);
    if (a >= 0x477ff000u) return (uint16_t)(s | 0x7c00u);   /* >= 65520 rounds to inf */
    if (a < 0x33000001u) return (uint16_t)s;                /* <= 2^-25: rounds to zero (2^-25 ties to even 0) */
    const int e = (int)(a >> 23) - 127;
    if (e < -14) {                                          /* subnormal half: units of 2^-24 */
        const float r = rintf(ldexpf(u2f(a), 24));
        return (uint16_t)(s | (unsigned)r);
    }
    const uint32_t m = a & 0x7fffffu, keep = m >> 13, rem = m & 0x1fffu;
    uint32_t h = ((uint32_t)(e + 15) << 10) | keep;
    if (rem > 0x1000u || (rem == 0x1000u && (keep & 1u))) h++;
    return (uint16_t)(s | h);
}
float orc_h16_to_f32(uint16_t h) {
    const uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 0x3ffu;
    if (e == 31u) return u2f(s | 0x7f800000u | (m << 13));
    if (!e) { const float v = ldexpf((float)m, -24); return s ? -v : v; }
    return u2f(s | ((e + 112u) << 23) | (m << 13));
}

/* a double -> binary16, round to nearest even (the double is the exact value to round) */
static uint16_t f64_to_h16(double x) {
    const uint16_t s = signbit(x) ? 0x8000u : 0u;
    double a = fabs(x);
    if (a != a) return (uint16_t)(s | 0x7e00u);
    if (a >= 65520.0) return (uint16_t)(s | 0x7c00u);
    if (a == 0.0) return s;
    int ex; frexp(a, &ex);                                  /* a = f 2^ex, f in [.5, 1): leading bit at 2^(ex - 1) */
    const int q = ex - 1 < -14 ? -24 : ex - 1 - 10;          /* the quantum's exponent: 11 significant bits, or the subnormal step */
    const double k = rint(ldexp(a, -q));                    /* exact scaling, rint ties to even in the default rounding mode */
    const double r = ldexp(k, q);
    if (r >= 65536.0) return (uint16_t)(s | 0x7c00u);
    return (uint16_t)(s | orc_f32_to_h16((float)r));        /* r is a binary16 value: the conversion is exact */
}
/* binary16 fused multiply-add of binary16 operands, one rounding (HFMA2, src/lp_common.cuh:703). The product of two 11-bit significands
   is exact in a double; the sum with c is formed with its rounding error (two-sum), and where the double sum sits exactly on a binary16
   tie while the error is not zero it is moved off the tie in the error's direction before the one rounding to binary16 */
static uint16_t h16_fma(uint16_t a, uint16_t b, uint16_t c) {
    const double p = (double)orc_h16_to_f32(a) * (double)orc_h16_to_f32(b), cd = (double)orc_h16_to_f32(c);
    if (p != p || cd != cd || isinf(p) || isinf(cd)) return f64_to_h16(p + cd);
    double sum = p + cd;
    const double bb = sum - p, err = (p - (sum - bb)) + (cd - bb);
    if (err != 0.0) sum = nextafter(sum, err > 0.0 ? INFINITY : -INFINITY);   /* (only matters on a tie; elsewhere one double ulp changes nothing) */
    return f64_to_h16(sum);
}
uint16_t orc_h16_fma(uint16_t a, uint16_t b, uint16_t c) { return h16_fma(a, b, c); }

/* ---------- one block row (src/lp_mxops.cuh:45-65 for the NaN-propagating amax; src/lp_f8fwd.cuh:90-103 for fmaxf) ---------- */
static void enc_codes(int bits, const float *v, int bw, float m, uint8_t *codes) {
    if (bits == 8) for (int k = 0; k < bw; k++) codes[k] = (uint8_t)orc_enc_e4m3(v[k] * m);
    else for (int k = 0; k < bw; k += 2) codes[k >> 1] = (uint8_t)(orc_enc_e2m1(v[k] * m) | (orc_enc_e2m1(v[k + 1] * m) << 4));   /* low nibble first */
}
uint8_t orc_store_row(int bits, const float *v, int bw, uint8_t *codes, int nanprop) {
    float amax;
    if (nanprop) { uint32_t am = 0; for (int k = 0; k < bw; k++) { const uint32_t a = f2u(v[k]) & 0x7fffffffu; if (a > am) am = a; } amax = u2f(am); }
    else { amax = 0.f; for (int k = 0; k < bw; k++) amax = fmaxf(amax, fabsf(v[k])); }
    const int e = orc_mx_exp(amax, bits == 8 ? INVQ8 : INVQ4);
    enc_codes(bits, v, bw, orc_exp2i(-e), codes);
    return (uint8_t)(e + 127);
}
void orc_load_row(int bits, const uint8_t *codes, uint8_t sbyte, int bw, float *v) {
    const float s = orc_mx_scale(sbyte);
    if (bits == 8) for (int k = 0; k < bw; k++) v[k] = orc_dec_e4m3(codes[k]) * s;
    else for (int k = 0; k < bw; k++) v[k] = orc_dec_e2m1((codes[k >> 1] >> (4 * (k & 1))) & 15u) * s;
}

/* ---------- tensor layout (src/lp_common.cuh:100-106, src/lp_mxops.cuh:69-70) ---------- */
typedef struct { const uint8_t *q, *sc; int bits, bw, nb, rb, N, C; size_t S; } mxt_t;
static mxt_t mxt(const void *p, int bits, int N, int C, size_t S) {
    mxt_t t; t.q = (const uint8_t *)p; t.bits = bits; t.bw = orc_mx_bw(C); t.nb = orc_mx_nb(C); t.rb = rowbytes(t.bw, bits);
    t.N = N; t.C = C; t.S = S; t.sc = t.q + (size_t)N * t.nb * S * t.rb; return t;
}
static inline size_t mxrow(const mxt_t *t, int n, int blk, size_t v) { return ((size_t)n * t->nb + blk) * t->S + v; }
/* decoded 32 channels of block blk at voxel v (channels past bw are zero) */
static void mx_row32(const mxt_t *t, int n, int blk, size_t v, float *r) {
    for (int k = 0; k < 32; k++) r[k] = 0.f;
    if (blk >= t->nb) return;
    const size_t ri = mxrow(t, n, blk, v);
    orc_load_row(t->bits, t->q + ri * t->rb, t->sc[ri], t->bw, r);
}

void orc_f32_to_mx(int bits, const float *x, int N, int C, size_t S, uint8_t *y) {
    const mxt_t t = mxt(y, bits, N, C, S);
    uint8_t *q = y, *sc = y + (size_t)N * t.nb * S * t.rb;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)((size_t)N * t.nb * S); i++) {
        const size_t v = (size_t)i % S; const int blk = (int)(((size_t)i / S) % t.nb), n = (int)((size_t)i / (S * t.nb));
        float r[32];
        for (int k = 0; k < t.bw; k++) { const int c = blk * t.bw + k; r[k] = c < C ? x[((size_t)n * C + c) * S + v] : 0.f; }
        sc[i] = orc_store_row(bits, r, t.bw, q + (size_t)i * t.rb, 1);
    }
}
void orc_h16_to_mx(int bits, const uint16_t *x, int N, int C, size_t S, uint8_t *y) {
    const mxt_t t = mxt(y, bits, N, C, S);
    uint8_t *q = y, *sc = y + (size_t)N * t.nb * S * t.rb;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)((size_t)N * t.nb * S); i++) {
        const size_t v = (size_t)i % S; const int blk = (int)(((size_t)i / S) % t.nb), n = (int)((size_t)i / (S * t.nb));
        float r[32];
        for (int k = 0; k < t.bw; k++) { const int c = blk * t.bw + k; r[k] = c < C ? orc_h16_to_f32(x[((size_t)n * C + c) * S + v]) : 0.f; }
        sc[i] = orc_store_row(bits, r, t.bw, q + (size_t)i * t.rb, 1);
    }
}
void orc_mx_to_f32(int bits, const uint8_t *x, int N, int C, size_t S, float *y) {
    const mxt_t t = mxt(x, bits, N, C, S);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)((size_t)N * t.nb * S); i++) {
        const size_t v = (size_t)i % S; const int blk = (int)(((size_t)i / S) % t.nb), n = (int)((size_t)i / (S * t.nb));
        float r[32];
        orc_load_row(bits, t.q + (size_t)i * t.rb, t.sc[i], t.bw, r);
        for (int k = 0; k < t.bw; k++) { const int c = blk * t.bw + k; if (c < C) y[((size_t)n * C + c) * S + v] = r[k]; }
    }
}
/* src/lp_mx_cvt.cu:29-41 */
void orc_pred_input_mx(int bits, const uint8_t *ct, int W, float mean, float isd, const float *dyo, const float *dxo, int axis,
                       int z0, int nz, uint8_t *y, int hd) {
    const size_t S = (size_t)nz * W * W; const int rb = rowbytes(8, bits);
    uint8_t *sc = y + S * rb;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)S; i++) {
        const int xx = (int)(i % W), yy = (int)((i / W) % W), z = z0 + (int)(i / ((int64_t)W * W));
        const float dy = dyo[z] + (float)yy, dx = dxo[z] + (float)xx, inv = axis ? (float)axis / (sqrtf(fmaf(dy, dy, dx * dx)) + 1e-6f) : 0.f;   /* (the reference builds with fused multiply-add contraction) */
        float r[8] = {0};
        r[0] = ((float)ct[(size_t)z * W * W + (size_t)yy * W + xx] - mean) * isd; r[2] = dy * inv; r[3] = dx * inv;
        if (hd == 2) for (int k = 0; k < 4; k++) r[k] = orc_h16_to_f32(orc_f32_to_h16(r[k]));
        else if (hd == 1) for (int k = 0; k < 4; k++) { uint32_t u = f2u(r[k]); if ((u & 0x7fffffffu) <= 0x7f800000u) { u += 0x7fffu + ((u >> 16) & 1u); r[k] = u2f(u & 0xffff0000u); } }   /* bf16, round to nearest even */
        sc[i] = orc_store_row(bits, r, 8, y + (size_t)i * rb, 1);
    }
}

/* ---------- weights (src/lp_f8fwd.cu:54-71; src/lp_f4fwd.cu:53-66): one block = the 32 ci of one (tap, co) ----------
   padded input channel cp -> real channel (src/lp_common.cuh:235): MX inputs pad each of the two segments to 32 */
static int seg_ci(int cp, int Ci, int Cx, int CxP) { if (cp < CxP) return cp < Cx ? cp : -1; const int c = Cx + cp - CxP; return c < Ci ? c : -1; }
/* 2-D fp4 weight scales (src/lp_f4fwd.cu:67-83, lp_set_w4_2d): the e2m1 prep takes the amax, and so the scale, over the 32 x 32 tile of 32
   output channels (co / 32; rows past Co are zeros) and the 32 input channels of the block, instead of per output channel */
static int g_w4_2d = 0;
void orc_set_w4_2d(int on) { g_w4_2d = on; }
static uint8_t store_row_amax(int bits, const float *v, float amax, uint8_t *codes) {
    const int e = orc_mx_exp(amax, bits == 8 ? INVQ8 : INVQ4);
    enc_codes(bits, v, 32, orc_exp2i(-e), codes);
    return (uint8_t)(e + 127);
}
static void prep_w(int bits, const float *w, int Co, int Ci, int Cx, int CxP, int Cip, float *wv, uint8_t *ws, uint8_t *wcodes, int w2d_on) {
    const int nch = Cip / 32;
    const int w2d = w2d_on && bits == 4 && Ci > 16;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < 27 * Co * nch; i++) {
        const int ch = i % nch, co = (i / nch) % Co, t = i / (nch * Co);
        float v[32]; uint8_t codes[32];
        for (int k = 0; k < 32; k++) { const int ci = seg_ci(ch * 32 + k, Ci, Cx, CxP); v[k] = ci >= 0 ? w[((size_t)co * Ci + ci) * 27 + t] : 0.f; }
        float am2 = 0.f;
        if (w2d) for (int c2 = co / 32 * 32; c2 < co / 32 * 32 + 32 && c2 < Co; c2++) for (int k = 0; k < 32; k++) { const int ci = seg_ci(ch * 32 + k, Ci, Cx, CxP); if (ci >= 0) am2 = fmaxf(am2, fabsf(w[((size_t)c2 * Ci + ci) * 27 + t])); }
        const uint8_t sb = w2d ? store_row_amax(bits, v, am2, codes) : orc_store_row(bits, v, 32, codes, 0);
        ws[i] = sb;
        if (wcodes) memcpy(wcodes + (size_t)i * rowbytes(32, bits), codes, rowbytes(32, bits));
        float *dst = wv + ((size_t)t * Co + co) * Cip + ch * 32;
        for (int k = 0; k < 32; k++) dst[k] = bits == 8 ? orc_dec_e4m3(codes[k]) : orc_dec_e2m1((codes[k >> 1] >> (4 * (k & 1))) & 15u);
    }
}
void orc_prep_w(int bits, const float *w, int Co, int Ci, int Cx, int CxP, int Cip, float *wv, uint8_t *ws, uint8_t *wcodes) { prep_w(bits, w, Co, Ci, Cx, CxP, Cip, wv, ws, wcodes, g_w4_2d); }

/* w [Co][Ci][T] rounded in place to MX-fp4 values with one scale per Bo x Bi block and tap (src/lp_mx_cvt.cu:369-395) */
void orc_fakeq_w4(float *w, int Co, int Ci, int T, int Bo, int Bi) {
    for (int o0 = 0; o0 < Co; o0 += Bo) for (int i0 = 0; i0 < Ci; i0 += Bi) for (int t = 0; t < T; t++) {
        const int no = Co - o0 < Bo ? Co - o0 : Bo, ni = Ci - i0 < Bi ? Ci - i0 : Bi;
        float amax = 0.f;
        for (int o = 0; o < no; o++) for (int i = 0; i < ni; i++) amax = fmaxf(amax, fabsf(w[((size_t)(o0 + o) * Ci + i0 + i) * T + t]));
        const int e = orc_mx_exp(amax, INVQ4); const float m = orc_exp2i(-e), sc = orc_exp2i(e);
        for (int o = 0; o < no; o++) for (int i = 0; i < ni; i++) { float *p = w + ((size_t)(o0 + o) * Ci + i0 + i) * T + t; *p = orc_dec_e2m1(orc_enc_e2m1(*p * m)) * sc; }
    }
}
/* a third summation order for drift studies (acc64 == 2): fp32 accumulation whose every add is rounded toward zero, as a datapath that
   aligns and truncates its addends does. A legitimate fp32-accumulated result, within one ulp per add of the other two. */
static float add_chop(float acc, double blk) {
    const double t = (double)acc + blk; float f = (float)t;
    if (isfinite(f) && fabs((double)f) > fabs(t)) f = nextafterf(f, 0.f);
    return f;
}
/* 0 (default): the exact u sigmoid(u), correctly rounded; 1: the same function evaluated in fp32 by a fast path (product with the fp32
   reciprocal of 1 + expf(-u): a few ulp off), the kind of evaluation a GPU makes. For drift studies only. */
static int g_act_mode = 0, g_align_bits = 24;
void orc_set_act_mode(int m) { g_act_mode = m; }
void orc_set_align_bits(int b) { g_align_bits = b; }   /* width of the acc64 == 3 adder below its largest addend's leading bit */
/* ---------- GN + SiLU of the conv staging (src/lp_common.cuh:258, :474-482): u = fma(x, a, b), h = u / 2, h + h tanh(h) ---------- */
float orc_act_ab(float v, float a, float b) {
    /* the reference's h + h tanh(h), h = u / 2, is u sigmoid(u); its tanh is NVIDIA's tanh.approx (about 2^-11), so the oracle takes
       the exact value of the same function, correctly rounded: any faithful evaluation is inside the reference's own error */
    const float u = fmaf(v, a, b);
    if (g_act_mode == 1) { const float d = 1.f + expf(-u), r = 1.f / d; return u * r; }
    return (float)((double)u / (1.0 + exp(-(double)u)));
}
/* src/lp_slab.cuh:7-12: per-sample statistics read row n; slab-local ones the row of the plane's slab, the first and last slab taking
   whatever lies before and after them */
int orc_gn_row(const orc_gn_t *g, int n, int z) {
    if (!g->ns) return n;
    int s = (z + g->zo) / g->zs;
    s = s < 0 ? 0 : s >= g->ns ? g->ns - 1 : s;
    return n * g->ns + s;
}
/* (nr: the statistics row) */
static void gn_ab(const orc_gn_t *g, int nr, int cc, int Cg, float *a, float *b) {
    const int ng = nr * g->G + cc / (Cg / g->G);
    *a = g->rstd[ng] * g->gamma[cc];
    *b = fmaf(-g->mean[ng], *a, g->beta[cc]);               /* tests/test_mx4_wide.c:119 */
}
/* per padded-channel (a, b, has_gn) table of sample n at input plane z (the plane only matters to slab-local statistics) */
typedef struct { float a, b; int g, ci; } chab_t;
static void chan_table(const orc_conv_t *c, int n, int z, int Cx, int CxP, int Cip, chab_t *tab) {
    const int s2g = c->x2 && c->gp2.G;
    for (int cp = 0; cp < Cip; cp++) {
        const int mxin = c->xdt >= 3;
        const int ci = mxin ? seg_ci(cp, c->Ci, Cx, CxP) : (cp < c->Ci ? cp : -1);
        chab_t t = {1.f, 0.f, 0, ci};
        if (ci >= 0) {
            const orc_gn_t *q = s2g && ci >= Cx ? &c->gp2 : &c->gp;
            const int cc = s2g && ci >= Cx ? ci - Cx : ci, Cg = s2g ? (ci >= Cx ? c->Ci - Cx : Cx) : c->Ci;
            if (q->G) { gn_ab(q, orc_gn_row(q, n, z), cc, Cg, &t.a, &t.b); t.g = 1; }
        }
        tab[cp] = t;
    }
}

/* ---------- staging (src/lp_f8fwd.cuh:66-113): per (n, 32-channel chunk, input voxel) the compute-format codes and scale ----------
   Returned as decoded code values sv[n][chunk][voxel][32] and scale sf[n][chunk][voxel] (fp32 power of two).
   Staged geometry = the input's own grid (stride 1: D x H x W; stride 2: the input dims). */
typedef struct { float *sv; float *sf; int nch, Cip, Cx, CxP; size_t S; } staged_t;
static void quant_row(int cbits, const float *v, float *sv, float *sf) {
    uint8_t codes[32];
    const uint8_t sb = orc_store_row(cbits, v, 32, codes, 0);
    *sf = orc_mx_scale(sb);
    for (int k = 0; k < 32; k++) sv[k] = cbits == 8 ? orc_dec_e4m3(codes[k]) : orc_dec_e2m1((codes[k >> 1] >> (4 * (k & 1))) & 15u);
}
/* decoder up segment (src/lp_common.cuh:618-670): coarse rows -> GN + SiLU -> e4m3 rows with a row scale (amax ignoring NaN) */
static void coarse_rows(const orc_conv_t *c, int n, int blk, int Cx, const chab_t *tab, int Dc, int Hc, int Wc, float *cv /* [Sc][32 codes + scale] */, uint8_t *cvsb /* [Sc] scale bytes */) {
    const size_t Sc = (size_t)Dc * Hc * Wc;
    const mxt_t t = mxt(c->x, c->xdt == 3 ? 8 : 4, c->N, Cx, Sc);
    for (size_t v = 0; v < Sc; v++) {
        float r[32];
        mx_row32(&t, n, blk, v, r);
        for (int k = 0; k < 32; k++) if (tab[blk * 32 + k].g) r[k] = orc_act_ab(r[k], tab[blk * 32 + k].a, tab[blk * 32 + k].b);
        uint32_t am = 0; for (int k = 0; k < 32; k++) { const uint32_t u = f2u(fabsf(r[k])); if (u <= 0x7f800000u && u > am) am = u; }
        const int e = orc_mx_exp(u2f(am), INVQ8); const float m = orc_exp2i(-e), s = orc_mx_scale((unsigned)(e + 127));
        /* stored as code and scale; the blend multiplies the weight by the scale first (stage_up_smem) */
        for (int k = 0; k < 32; k++) cv[v * 33 + k] = orc_dec_e4m3(orc_enc_e4m3(r[k] * m));
        cv[v * 33 + 32] = s;
        cvsb[v] = (uint8_t)(e + 127);
    }
}
static int build_staged(const orc_conv_t *c, staged_t *st) {
    const int mxin = c->xdt >= 3, xbits = c->xdt == 3 ? 8 : 4;
    const int Cx = c->x2 ? c->c_split : c->Ci, CxP = (Cx + 31) / 32 * 32;
    const int Cip = mxin ? CxP + (c->Ci - Cx + 31) / 32 * 32 : (c->Ci + 31) / 32 * 32;
    const size_t S = (size_t)c->D * c->H * c->W;
    st->nch = Cip / 32; st->Cip = Cip; st->Cx = Cx; st->CxP = CxP; st->S = S;
    st->sv = (float *)malloc((size_t)c->N * st->nch * S * 32 * sizeof(float));
    st->sf = (float *)malloc((size_t)c->N * st->nch * S * sizeof(float));
    if (!st->sv || !st->sf) return -1;
    const int G = c->gp.G || c->gp2.G;
    /* the fp4 entry blends the fused upsample in binary16 (src/lp_f4fwd.cuh:1135-1136, UFSM_UP_H2 default), the fp8 entry in fp32; up 2 / 3 force one */
    const int uph2 = c->up == 2 || (c->up == 1 && c->cbits == 4);
    const int Dc = c->D >> 1, Hc = c->H >> 1, Wc = c->W >> 1;
    if (c->up && c->gp.G && c->gp.ns) return -1;           /* (slab-local statistics of the upsampled segment: no reader of the reference takes them) */
    const int slabs = (c->gp.G && c->gp.ns) || (c->gp2.G && c->gp2.ns);
    const size_t HW = (size_t)c->H * c->W;
    for (int n = 0; n < c->N; n++) {
        /* the table of plane 0, and with slab-local statistics one per input plane behind it */
        chab_t *tab = (chab_t *)malloc((size_t)Cip * (slabs ? c->D : 1) * sizeof(chab_t));
        for (int z = 0; z < (slabs ? c->D : 1); z++) chan_table(c, n, z, Cx, CxP, Cip, tab + (size_t)z * Cip);
        for (int ch = 0; ch < st->nch; ch++) {
            const int upc = mxin && c->up && ch * 32 < CxP;
            const int sec = mxin && ch * 32 >= CxP;       /* chunk of the x2 segment */
            float *cv = NULL; uint8_t *cvsb = NULL;
            if (upc) { cv = (float *)malloc((size_t)Dc * Hc * Wc * 33 * sizeof(float)); cvsb = (uint8_t *)malloc((size_t)Dc * Hc * Wc); coarse_rows(c, n, ch, Cx, tab, Dc, Hc, Wc, cv, cvsb); }
            mxt_t t;
            if (mxin) t = sec ? mxt(c->x2, xbits, c->N, c->Ci - Cx, S) : mxt(c->x, xbits, c->N, Cx, S);
            const int blk = sec ? ch - CxP / 32 : ch;
#pragma omp parallel for schedule(static)
            for (int64_t vi = 0; vi < (int64_t)S; vi++) {
                const size_t v = (size_t)vi;
                float *sv = st->sv + (((size_t)n * st->nch + ch) * S + v) * 32, *sf = st->sf + ((size_t)n * st->nch + ch) * S + v;
                float r[32];
                if (upc) {   /* 8-term blend, fma order a (z), b (y), c (x) (stage_up_smem) */
                    const int gz = (int)(v / ((size_t)c->H * c->W)), gy = (int)(v / c->W % c->H), gx = (int)(v % c->W);
                    int mz[2], my[2], mx[2];
                    mz[0] = gz >> 1; mz[1] = mz[0] + ((gz & 1) ? 1 : -1); if (mz[1] < 0) mz[1] = 0; if (mz[1] > Dc - 1) mz[1] = Dc - 1;
                    my[0] = gy >> 1; my[1] = my[0] + ((gy & 1) ? 1 : -1); if (my[1] < 0) my[1] = 0; if (my[1] > Hc - 1) my[1] = Hc - 1;
                    mx[0] = gx >> 1; mx[1] = mx[0] + ((gx & 1) ? 1 : -1); if (mx[1] < 0) mx[1] = 0; if (mx[1] > Wc - 1) mx[1] = Wc - 1;
                    for (int k = 0; k < 32; k++) r[k] = 0.f;
                    if (uph2) {   /* binary16 blend (stage_up_smem_h2, src/lp_common.cuh:674-712): weights relative to the largest of the 8 rows' scales */
                        unsigned em = 0;
                        for (int t8 = 0; t8 < 8; t8++) { const unsigned sb = cvsb[((size_t)mz[t8 >> 2] * Hc + my[(t8 >> 1) & 1]) * Wc + mx[t8 & 1]]; if (sb > em) em = sb; }
                        uint16_t acc[32];
                        for (int k = 0; k < 32; k++) acc[k] = 0;
                        for (int a = 0; a < 2; a++) for (int b = 0; b < 2; b++) for (int cc = 0; cc < 2; cc++) {
                            const size_t ri = ((size_t)mz[a] * Hc + my[b]) * Wc + mx[cc];
                            const float *row = cv + ri * 33;
                            const int de = (int)cvsb[ri] - (int)em;
                            const uint16_t w3 = orc_f32_to_h16((a ? 0.25f : 0.75f) * (b ? 0.25f : 0.75f) * (cc ? 0.25f : 0.75f) * (de >= -126 ? u2f((uint32_t)(127 + de) << 23) : 0.f));
                            for (int k = 0; k < 32; k++) acc[k] = h16_fma(w3, orc_f32_to_h16(row[k]), acc[k]);      /* (an e4m3 value is a binary16 value) */
                        }
                        const float sm = orc_mx_scale(em);
                        for (int k = 0; k < 32; k++) r[k] = orc_h16_to_f32(acc[k]) * sm;
                    } else
                    for (int a = 0; a < 2; a++) for (int b = 0; b < 2; b++) for (int cc = 0; cc < 2; cc++) {
                        const float *row = cv + (((size_t)mz[a] * Hc + my[b]) * Wc + mx[cc]) * 33;
                        const float w3 = (a ? 0.25f : 0.75f) * (b ? 0.25f : 0.75f) * (cc ? 0.25f : 0.75f) * row[32];
                        for (int k = 0; k < 32; k++) r[k] = fmaf(w3, row[k], r[k]);
                    }
                    quant_row(c->cbits, r, sv, sf);
                } else if (mxin) {
                    const int copy = !G && ((c->xdt == 3 && c->cbits == 8) || (c->xdt == 4 && c->cbits == 4));
                    if (copy) {   /* stored block used as is (src/lp_f8fwd.cuh:68-87) */
                        for (int k = 0; k < 32; k++) sv[k] = 0.f;
                        *sf = orc_mx_scale(1);
                        if (blk < t.nb) {
                            const size_t ri = mxrow(&t, n, blk, v);
                            for (int k = 0; k < t.bw; k++) sv[k] = xbits == 8 ? orc_dec_e4m3(t.q[ri * t.rb + k]) : orc_dec_e2m1((t.q[ri * t.rb + (k >> 1)] >> (4 * (k & 1))) & 15u);
                            *sf = orc_mx_scale(t.sc[ri]);
                        }
                    } else {
                        mx_row32(&t, n, blk, v, r);
                        const chab_t *tz = tab + (slabs ? (v / HW) * (size_t)Cip : 0);
                        for (int k = 0; k < 32; k++) { const chab_t *q = &tz[ch * 32 + k]; r[k] = q->ci < 0 ? 0.f : q->g ? orc_act_ab(r[k], q->a, q->b) : r[k]; }
                        quant_row(c->cbits, r, sv, sf);
                    }
                } else {     /* plane-major fp32 / fp16 input, quantised per (voxel, 32 channels) */
                    const chab_t *tz = tab + (slabs ? (v / HW) * (size_t)Cip : 0);
                    for (int k = 0; k < 32; k++) {
                        const chab_t *q = &tz[ch * 32 + k];
                        float xv = 0.f;
                        if (q->ci >= 0) {
                            const int sec2 = c->x2 && q->ci >= Cx;
                            const size_t idx = sec2 ? ((size_t)n * (c->Ci - Cx) + q->ci - Cx) * S + v : ((size_t)n * Cx + q->ci) * S + v;
                            const void *src = sec2 ? c->x2 : c->x;
                            xv = c->xdt == 2 ? orc_h16_to_f32(((const uint16_t *)src)[idx]) : ((const float *)src)[idx];
                            if (q->g) xv = orc_act_ab(xv, q->a, q->b);
                        }
                        r[k] = xv;
                    }
                    quant_row(c->cbits, r, sv, sf);
                }
            }
            free(cv); free(cvsb);
        }
        free(tab);
    }
    /* tap-packed stem (src/lp_f8fwd.cuh:374-380): one scale per staged tile of 4 x 10 x 18 positions around a 2 x 8 x 16 output tile.
       The per-position rows above are replaced by rows quantised with the tile's scale at conv time (see orc_conv3). */
    return 0;
}
int orc_conv3_staged(const orc_conv_t *c, float *out) {
    staged_t st;
    if (build_staged(c, &st)) return -1;
    const size_t n = (size_t)c->N * st.nch * st.S;
    for (size_t i = 0; i < n; i++) for (int k = 0; k < 32; k++) out[i * 32 + k] = st.sv[i * 32 + k] * st.sf[i];
    free(st.sv); free(st.sf);
    return st.Cip;
}

static float gelu_f(float x) { return 0.5f * x * (1.f + (float)erf((double)x * 0.70710678118654752440)); }
static float silu_f(float x) { return (float)((double)x / (1.0 + exp(-(double)x))); }

/* epilogue of one output voxel (src/lp_common.cuh:1492-1535): bias, optional fused activation, store in the output type, statistics */
static void conv_epilogue(const orc_conv_t *c, int n, size_t ov, size_t So, float *acc, const double *acc64, double *ls) {
    const int Co = c->Co, cpg = c->Go ? Co / c->Go : 1;
    const int ybits = c->ydt == 3 ? 8 : 4, ybw = orc_mx_bw(Co), ynb = orc_mx_nb(Co), yrb = rowbytes(ybw, ybits);
    uint8_t *yq = (uint8_t *)c->y, *ysc = yq + (size_t)c->N * ynb * So * yrb;
    /* epilogue (src/lp_common.cuh:1492-1535) */
    for (int co = 0; co < Co; co++) {
        float v = c->acc64 == 1 ? (float)(acc64[co] + (c->b ? (double)c->b[co] : 0.0)) : acc[co] + (c->b ? c->b[co] : 0.f);
        if (c->fused_act) {
            if (c->ep_a) v = fmaf(v, c->ep_a[co], c->ep_b[co]);
            v = c->fused_act == 1 ? silu_f(v) : c->fused_act == 2 ? gelu_f(v) : c->fused_act == 3 ? fmaxf(v, 0.f) : v;
        }
        acc[co] = v;
    }
    if (c->ydt >= 3) {
        for (int blk = 0; blk < ynb; blk++) {
            float r[32]; uint8_t codes[32];
            for (int k = 0; k < ybw; k++) { const int co = blk * ybw + k; r[k] = co < Co ? acc[co] : 0.f; }
            const size_t ri = ((size_t)n * ynb + blk) * So + ov;
            const uint8_t sb = orc_store_row(ybits, r, ybw, codes, 0);
            memcpy(yq + ri * yrb, codes, (size_t)yrb); ysc[ri] = sb;
            if (ls && c->stored_stats) { float d[32]; orc_load_row(ybits, codes, sb, ybw, d); for (int k = 0; k < ybw; k++) { const int co = blk * ybw + k; if (co < Co) acc[co] = d[k]; } }
        }
    } else if (c->ydt == 2) {
        for (int co = 0; co < Co; co++) {
            float v = acc[co];
            if (c->Go > 0 && fabsf(v) > 65504.f) v = copysignf(65504.f, v);   /* sat_h16 (src/lp_common.cuh:465, :1567-1569) */
            ((uint16_t *)c->y)[((size_t)n * Co + co) * So + ov] = orc_f32_to_h16(v);
            acc[co] = v;
        }
    } else for (int co = 0; co < Co; co++) ((float *)c->y)[((size_t)n * Co + co) * So + ov] = acc[co];
    if (ls) for (int co = 0; co < Co; co++) { const double v = acc[co]; ls[2 * (co / cpg)] += v; ls[2 * (co / cpg) + 1] += v * v; }
}

/* ---------- tap-packed small-channel convs ----------
   stem_tile 1 (src/lp_f8fwd.cuh:153-177 weights, :178-400 kernel, :601-609 dispatch): channels padded to CP in {4, 8, 16}; a K block of 32 =
   32 / CP taps x CP channels, so a block mixes positions and the activation operand has ONE scale per staged tile: the 4 x 10 x 18 input
   positions around a 2 x 8 x 16 output tile (tiles on the output grid from the origin).
   stem_tile 2 (src/lp_f8fwd.cu:72-92 weights, src/lp_f8fwd.cuh:447-563 kernel, :626 dispatch): 9 .. 16 channels in slots of 16, two K blocks
   per tap row (kz, ky): [kx0 | kx1] and [kx2 | 0], so a block spans two positions of one staged row and the activation operand has one
   scale per staged ROW: the 18 positions x - 1 .. x + 16 of a (z, y) line inside a 16-wide x tile.
   Values outside the volume and channels >= Ci are zeros; amax ignores NaN (fmaxf). */
static int conv3_stem(const orc_conv_t *c) {
    const int Ci = c->Ci, Co = c->Co, D = c->D, H = c->H, W = c->W, rowmode = c->stem_tile == 2;
    if (c->x2 || c->up || c->stride == 2 || c->cbits != 8 || Ci > 16 || (!rowmode && c->xdt != 0 && Ci > 8)) return -2;
    const int CP = rowmode ? 16 : Ci <= 4 ? 4 : Ci <= 8 ? 8 : 16, TPK = 32 / CP, NKB = rowmode ? 18 : (27 + TPK - 1) / TPK;
    const size_t S = (size_t)D * H * W;
    /* K block kb, element k -> (tap, channel), tap 27 = none */
#define STEM_TAP(kb, k) (rowmode ? (2 * ((kb) & 1) + ((k) >> 4) < 3 ? ((kb) >> 1) * 3 + 2 * ((kb) & 1) + ((k) >> 4) : 27) : ((kb) * TPK + (k) / CP < 27 ? (kb) * TPK + (k) / CP : 27))
    float *wv = (float *)malloc((size_t)NKB * Co * 32 * sizeof(float)), *wsf = (float *)malloc((size_t)NKB * Co * sizeof(float));
    for (int kb = 0; kb < NKB; kb++) for (int co = 0; co < Co; co++) {            /* prep_w8s_k / prep_w8p_k */
        float v[32], amax = 0.f;
        for (int k = 0; k < 32; k++) { const int tap = STEM_TAP(kb, k), ci = k % CP; v[k] = ci < Ci && tap < 27 ? c->w[((size_t)co * Ci + ci) * 27 + tap] : 0.f; amax = fmaxf(amax, fabsf(v[k])); }
        const int e = orc_mx_exp(amax, INVQ8); const float m = orc_exp2i(-e);
        for (int k = 0; k < 32; k++) wv[((size_t)kb * Co + co) * 32 + k] = orc_dec_e4m3(orc_enc_e4m3(v[k] * m));
        wsf[(size_t)kb * Co + co] = orc_mx_scale((unsigned)(e + 127));
    }
    const int z0 = c->z1 ? c->z0 : 0, z1 = c->z1 ? c->z1 : D;
    const int ntz = (D + 1) / 2, nty = (H + 7) / 8, ntx = (W + 15) / 16;
    float *val = (float *)malloc(S * CP * sizeof(float));
    const int slabs = c->gp.G && c->gp.ns;
    chab_t *tab = (chab_t *)malloc((size_t)32 * (slabs ? D : 1) * sizeof(chab_t));
    for (int n = 0; n < c->N; n++) {
        /* the conv's input values of this sample: val[voxel][CP] (decoded, after GN + SiLU when the input has one; slab-local statistics: each
           plane's own coefficients, src/lp_f8fwd.cuh:497) */
        for (int z = 0; z < (slabs ? D : 1); z++) chan_table(c, n, z, Ci, (Ci + 31) / 32 * 32, 32, tab + (size_t)z * 32);
        mxt_t t; if (c->xdt >= 3) t = mxt(c->x, c->xdt == 3 ? 8 : 4, c->N, Ci, S);
#pragma omp parallel for schedule(static)
        for (int64_t vi = 0; vi < (int64_t)S; vi++) {
            float r[32] = {0};
            if (c->xdt >= 3) mx_row32(&t, n, 0, (size_t)vi, r);
            else for (int k = 0; k < Ci; k++) { const size_t idx = ((size_t)n * Ci + k) * S + (size_t)vi; r[k] = c->xdt == 2 ? orc_h16_to_f32(((const uint16_t *)c->x)[idx]) : ((const float *)c->x)[idx]; }
            const chab_t *tz = tab + (slabs ? (size_t)(vi / ((int64_t)H * W)) * 32 : 0);
            for (int k = 0; k < CP; k++) val[(size_t)vi * CP + k] = k >= Ci ? 0.f : tz[k].g ? orc_act_ab(r[k], tz[k].a, tz[k].b) : r[k];
        }
        double *gs = c->osum ? (double *)calloc((size_t)2 * c->Go, sizeof(double)) : NULL;
#pragma omp parallel
        {
            float *acc = (float *)malloc((size_t)Co * sizeof(float)), *bq = (float *)malloc((size_t)720 * CP * sizeof(float));
            double *acc64 = (double *)malloc((size_t)Co * sizeof(double));
            double *ls = gs ? (double *)calloc((size_t)2 * c->Go, sizeof(double)) : NULL;
            double rsf[40];                                   /* scale of each staged row (rowmode) or of the tile (all equal) */
#pragma omp for schedule(dynamic, 4)
            for (int ti = 0; ti < ntz * nty * ntx; ti++) {
                const int tz = ti / (nty * ntx), ty = ti / ntx % nty, tx = ti % ntx;
                if (2 * tz + 2 <= z0 || 2 * tz >= z1) continue;
                /* the tile's 720 staged positions = 40 rows of 18, their amax and scales (src/lp_f8fwd.cuh:340-388, :480-520) */
                float amax[40]; for (int r = 0; r < 40; r++) amax[r] = 0.f;
                for (int p = 0; p < 720; p++) {
                    const int gz = 2 * tz - 1 + p / 180, gy = 8 * ty - 1 + p / 18 % 10, gx = 16 * tx - 1 + p % 18;
                    const int inb = gz >= 0 && gz < D && gy >= 0 && gy < H && gx >= 0 && gx < W;
                    for (int k = 0; k < CP; k++) { const float v = inb ? val[(((size_t)gz * H + gy) * W + gx) * CP + k] : 0.f; bq[p * CP + k] = v; amax[p / 18] = fmaxf(amax[p / 18], fabsf(v)); }
                }
                if (!rowmode) { float am = 0.f; for (int r = 0; r < 40; r++) am = fmaxf(am, amax[r]); for (int r = 0; r < 40; r++) amax[r] = am; }
                for (int r = 0; r < 40; r++) {
                    const int e = orc_mx_exp(amax[r], INVQ8); const float m = orc_exp2i(-e);
                    rsf[r] = orc_mx_scale((unsigned)(e + 127));
                    for (int i = r * 18 * CP; i < (r + 1) * 18 * CP; i++) bq[i] = orc_dec_e4m3(orc_enc_e4m3(bq[i] * m));
                }
                for (int l = 0; l < 256; l++) {
                    const int oz = 2 * tz + l / 128, oy = 8 * ty + l / 16 % 8, ox = 16 * tx + l % 16;
                    if (oz >= D || oy >= H || ox >= W || oz < z0 || oz >= z1) continue;
                    const int p0 = ((l / 128) * 10 + l / 16 % 8) * 18 + l % 16;            /* staged position of tap (0, 0, 0) */
                    for (int co = 0; co < Co; co++) { acc[co] = 0.f; acc64[co] = 0.0; }
                    for (int kb = 0; kb < NKB; kb++)
                        for (int co = 0; co < Co; co++) {
                            const float *wr = wv + ((size_t)kb * Co + co) * 32;
                            double d = 0.0; int row = 0;
                            for (int k = 0; k < 32; k++) {
                                const int tap = STEM_TAP(kb, k); if (tap >= 27) continue;
                                const int p = p0 + (tap / 9) * 180 + (tap / 3 % 3) * 18 + tap % 3;
                                d += (double)wr[k] * (double)bq[p * CP + k % CP]; row = p / 18;
                            }
                            const double blk = d * (double)wsf[(size_t)kb * Co + co] * rsf[row];     /* (a block's positions share the row, or the tile, scale) */
                            if (c->acc64 == 1) acc64[co] += blk; else if (c->acc64 == 2) acc[co] = add_chop(acc[co], blk); else acc[co] += (float)blk;
                        }
                    conv_epilogue(c, n, ((size_t)oz * H + oy) * W + ox, S, acc, acc64, ls);
                }
            }
            if (ls) {
#pragma omp critical
                for (int i = 0; i < 2 * c->Go; i++) gs[i] += ls[i];
                free(ls);
            }
            free(acc); free(acc64); free(bq);
        }
        if (gs) { for (int i = 0; i < 2 * c->Go; i++) c->osum[(size_t)n * 2 * c->Go + i] += gs[i]; free(gs); }
    }
#undef STEM_TAP
    free(val); free(wv); free(wsf); free(tab);
    return 0;
}

/* ---------- the convolution (src/lp_f8fwd.cuh:52, :114-148; src/lp_common.cuh:1465-1597) ---------- */
int orc_conv3(const orc_conv_t *c) {
    staged_t st;
    if (c->cbits != 8 && c->cbits != 4) return -2;
    if (c->stem_tile) return conv3_stem(c);
    if (build_staged(c, &st)) return -1;
    const int Co = c->Co, nch = st.nch, Cip = st.Cip, s = c->stride == 2 ? 2 : 1;
    const int Do = s == 2 ? (c->D - 1) / 2 + 1 : c->D, Ho = s == 2 ? (c->H - 1) / 2 + 1 : c->H, Wo = s == 2 ? (c->W - 1) / 2 + 1 : c->W;   /* src/nn_bwd.cu:132-135 */
    const size_t So = (size_t)Do * Ho * Wo;
    float *wv = (float *)malloc((size_t)27 * Co * Cip * sizeof(float));
    uint8_t *ws = (uint8_t *)malloc((size_t)27 * Co * nch);
    prep_w(c->cbits, c->w, Co, c->Ci, c->xdt >= 3 ? st.Cx : c->Ci, c->xdt >= 3 ? st.CxP : (c->Ci + 31) / 32 * 32, Cip, wv, ws, NULL, g_w4_2d && s == 1);   /* (2-D scales: the stride-1 preps only, src/lp_f4fwd.cuh:1163) */
    float *wsf = (float *)malloc((size_t)27 * Co * nch * sizeof(float));
    for (size_t i = 0; i < (size_t)27 * Co * nch; i++) wsf[i] = orc_mx_scale(ws[i]);
    const int z0 = c->z1 ? c->z0 : 0, z1 = c->z1 ? c->z1 : Do;
    for (int n = 0; n < c->N; n++) {
        double *gs = c->osum ? (double *)calloc((size_t)2 * c->Go, sizeof(double)) : NULL;
#pragma omp parallel
        {
            float *acc = (float *)malloc((size_t)Co * sizeof(float));
            double *acc64 = (double *)malloc((size_t)Co * sizeof(double));
            double *ls = gs ? (double *)calloc((size_t)2 * c->Go, sizeof(double)) : NULL;
#pragma omp for schedule(dynamic, 64)
            for (int64_t vi = (int64_t)z0 * Ho * Wo; vi < (int64_t)z1 * Ho * Wo; vi++) {
                const int oz = (int)(vi / ((int64_t)Ho * Wo)), oy = (int)(vi / Wo % Ho), ox = (int)(vi % Wo);
                for (int co = 0; co < Co; co++) { acc[co] = 0.f; acc64[co] = 0.0; }
                for (int ch = 0; ch < nch; ch++)                       /* chunk-major, tap-minor (src/lp_f8fwd.cuh:52) */
                    for (int t = 0; t < 27; t++) {
                        const int iz = s * oz - 1 + t / 9, iy = s * oy - 1 + (t / 3) % 3, ix = s * ox - 1 + t % 3;
                        if (iz < 0 || iz >= c->D || iy < 0 || iy >= c->H || ix < 0 || ix >= c->W) continue;   /* stored zeros contribute +0 */
                        const size_t iv = ((size_t)iz * c->H + iy) * c->W + ix;
                        const float *xv = st.sv + (((size_t)n * nch + ch) * st.S + iv) * 32;
                        const float xs = st.sf[((size_t)n * nch + ch) * st.S + iv];
                        for (int co = 0; co < Co; co++) {
                            const float *wr = wv + ((size_t)t * Co + co) * Cip + ch * 32;
                            double d = 0.0;                              /* exact: products of code values, 32 terms */
                            for (int k = 0; k < 32; k++) d += (double)wr[k] * (double)xv[k];
                            const double blk = d * (double)wsf[((size_t)t * Co + co) * nch + ch] * (double)xs;
                            if (c->acc64 == 3) {                        /* drift studies: an adder that aligns the block's products and the running sum to the
                                                                           largest exponent among them and drops what falls below g_align_bits bits of it */
                                const double sc = (double)wsf[((size_t)t * Co + co) * nch + ch] * (double)xs;
                                double mx = fabs((double)acc[co]);
                                for (int k = 0; k < 32; k++) { const double pk = fabs((double)wr[k] * (double)xv[k] * sc); if (pk > mx) mx = pk; }
                                if (mx > 0 && isfinite(mx)) {
                                    int ex; (void)frexp(mx, &ex);
                                    const double q = ldexp(1.0, ex - g_align_bits);
                                    double tsum = trunc((double)acc[co] / q);
                                    for (int k = 0; k < 32; k++) tsum += trunc((double)wr[k] * (double)xv[k] * sc / q);
                                    acc[co] = add_chop(0.f, tsum * q);
                                } else acc[co] += (float)blk;
                            } else
                            if (c->acc64 == 1) acc64[co] += blk; else if (c->acc64 == 2) acc[co] = add_chop(acc[co], blk); else acc[co] += (float)blk;
                        }
                    }
                conv_epilogue(c, n, (size_t)vi, So, acc, acc64, ls);
            }
            if (ls) {
#pragma omp critical
                for (int i = 0; i < 2 * c->Go; i++) gs[i] += ls[i];
                free(ls);
            }
            free(acc); free(acc64);
        }
        if (gs) { for (int i = 0; i < 2 * c->Go; i++) c->osum[(size_t)n * 2 * c->Go + i] += gs[i]; free(gs); }
    }
    free(wv); free(ws); free(wsf); free(st.sv); free(st.sf);
    return 0;
}

/* ---------- 2x2x2 stride-2 convolutions (no counterpart in the reference, whose down conv is 3x3x3 stride 2 and whose upsample is trilinear:
   src/lp_s2.cu:4-9, src/lp_mx_gn.cu:32-33): the same operand rules as orc_conv3 applied to the two other stride-2 layers a U-Net can have.
   Activations: the staged rows of build_staged (stored MX block as is, or GN + SiLU and re-quantisation per voxel and 32 channels); weights:
   one E8M0 scale per (tap, output channel, 32 input channels) as orc_prep_w; block products summed in fp32 (acc64: fp64) tap-major then
   block; the epilogue of orc_conv3.
   down: y[co][oz][oy][ox] = b[co] + sum_{ci, dz, dy, dx} w[co][ci][dz][dy][dx] x[ci][2 oz + dz][2 oy + dy][2 ox + dx]          (w as torch Conv3d)
   up:   y[co][2 iz + dz][2 iy + dy][2 ix + dx] = b[co] + sum_ci w[ci][co][dz][dy][dx] x[ci][iz][iy][ix]                        (w as torch ConvTranspose3d)
   Pins: tests/test_oracle_conv2.py (fp64 closed forms on exact operands; down = orc_conv3 at stride 2 with the taps embedded in a 3x3x3 kernel) */
int orc_conv2(const orc_conv_t *c, int up) {
    staged_t st;
    if ((c->cbits != 8 && c->cbits != 4) || c->x2 || c->up || c->xdt < 3) return -2;
    if (!up && ((c->D | c->H | c->W) & 1)) return -2;
    orc_conv_t cs = *c; cs.stride = 1;
    if (build_staged(&cs, &st)) return -1;
    const int Co = c->Co, Ci = c->Ci, nch = st.nch, Cip = st.Cip;
    const int Do = up ? 2 * c->D : c->D / 2, Ho = up ? 2 * c->H : c->H / 2, Wo = up ? 2 * c->W : c->W / 2;
    const size_t So = (size_t)Do * Ho * Wo;
    float *wv = (float *)malloc((size_t)8 * Co * Cip * sizeof(float)), *wsf = (float *)malloc((size_t)8 * Co * nch * sizeof(float));
    for (int i = 0; i < 8 * Co * nch; i++) {
        const int ch = i % nch, co = (i / nch) % Co, t = i / (nch * Co);
        float v[32]; uint8_t codes[32];
        for (int k = 0; k < 32; k++) { const int ci = ch * 32 + k; v[k] = ci < Ci ? (up ? c->w[((size_t)ci * Co + co) * 8 + t] : c->w[((size_t)co * Ci + ci) * 8 + t]) : 0.f; }
        wsf[i] = orc_mx_scale(orc_store_row(c->cbits, v, 32, codes, 0));
        for (int k = 0; k < 32; k++) wv[(size_t)i * 32 + k] = c->cbits == 8 ? orc_dec_e4m3(codes[k]) : orc_dec_e2m1((codes[k >> 1] >> (4 * (k & 1))) & 15u);
    }
    orc_conv_t ce = *c; ce.osum = NULL; ce.Go = 0;
    for (int n = 0; n < c->N; n++) {
#pragma omp parallel
        {
            float *acc = (float *)malloc((size_t)Co * sizeof(float));
            double *acc64 = (double *)malloc((size_t)Co * sizeof(double));
#pragma omp for schedule(dynamic, 64)
            for (int64_t vi = 0; vi < (int64_t)So; vi++) {
                const int oz = (int)(vi / ((int64_t)Ho * Wo)), oy = (int)(vi / Wo % Ho), ox = (int)(vi % Wo);
                for (int co = 0; co < Co; co++) { acc[co] = 0.f; acc64[co] = 0.0; }
                for (int t = 0; t < 8; t++) {
                    if (up && t != ((oz & 1) << 2 | (oy & 1) << 1 | (ox & 1))) continue;          /* an output voxel of the transposed conv has one tap */
                    const int iz = up ? oz >> 1 : 2 * oz + (t >> 2), iy = up ? oy >> 1 : 2 * oy + ((t >> 1) & 1), ix = up ? ox >> 1 : 2 * ox + (t & 1);
                    const size_t iv = ((size_t)iz * c->H + iy) * c->W + ix;
                    for (int ch = 0; ch < nch; ch++) {
                        const float *xv = st.sv + (((size_t)n * nch + ch) * st.S + iv) * 32;
                        const float xs = st.sf[((size_t)n * nch + ch) * st.S + iv];
                        for (int co = 0; co < Co; co++) {
                            const float *wr = wv + (((size_t)t * Co + co) * nch + ch) * 32;
                            double d = 0.0;
                            for (int k = 0; k < 32; k++) d += (double)wr[k] * (double)xv[k];
                            const double blk = d * (double)wsf[((size_t)t * Co + co) * nch + ch] * (double)xs;
                            if (c->acc64 == 1) acc64[co] += blk; else acc[co] += (float)blk;
                        }
                    }
                }
                conv_epilogue(&ce, n, (size_t)vi, So, acc, acc64, NULL);
            }
            free(acc); free(acc64);
        }
    }
    free(wv); free(wsf); free(st.sv); free(st.sf);
    return 0;
}

/* ---------- GroupNorm ---------- */
void orc_gn_finalize(const double *sums, int NG, size_t len, float eps, float *mean, float *rstd) {   /* src/nn_elem.cu:5-11 */
    for (int i = 0; i < NG; i++) {
        const double m = sums[2 * i] / (double)len, v = sums[2 * i + 1] / (double)len - m * m;
        mean[i] = (float)m; rstd[i] = (float)(1.0 / sqrt((v > 0 ? v : 0) + (double)eps));
    }
}
void orc_gn_sums_mx(int bits, const uint8_t *x, int N, int C, int G, size_t S, double *sums, size_t v0, size_t v1) {
    const mxt_t t = mxt(x, bits, N, C, S); const int cpg = C / G;
    for (int n = 0; n < N; n++) for (int blk = 0; blk < t.nb; blk++)
        for (size_t v = v0; v < v1; v++) {
            float r[32]; mx_row32(&t, n, blk, v, r);
            for (int k = 0; k < t.bw; k++) { const int c = blk * t.bw + k; if (c < C) { const double d = r[k]; sums[2 * ((size_t)n * G + c / cpg)] += d; sums[2 * ((size_t)n * G + c / cpg) + 1] += d * d; } }
        }
}
/* src/lp_mx_gn.cu:17: v = (x - mean) rstd gamma + beta (left to right, the last multiply-add contracted), v / (1 + exp(-v)) */
static float apply_silu(float x, float mean, float rstd, float gamma, float beta) {
    const float v = fmaf((x - mean) * rstd, gamma, beta);
    return (float)((double)v / (1.0 + exp(-(double)v)));
}
void orc_gn_silu_apply_mx(const void *x, int xdt, int N, int C, size_t S, orc_gn_t gp, uint8_t *y, int ybits) {
    const int bw = orc_mx_bw(C), nb = orc_mx_nb(C), yrb = rowbytes(bw, ybits), cpg = C / gp.G;
    uint8_t *ysc = y + (size_t)N * nb * S * yrb;
    mxt_t t; if (xdt >= 3) t = mxt(x, xdt == 3 ? 8 : 4, N, C, S);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)((size_t)N * nb * S); i++) {
        const size_t v = (size_t)i % S; const int blk = (int)(((size_t)i / S) % nb), n = (int)((size_t)i / (S * nb));
        float r[32] = {0};
        if (xdt >= 3) mx_row32(&t, n, blk, v, r);
        else for (int k = 0; k < bw; k++) { const int c = blk * bw + k; if (c < C) r[k] = ((const float *)x)[((size_t)n * C + c) * S + v]; }
        for (int k = 0; k < bw; k++) {
            const int c = blk * bw + k; if (c >= C) { r[k] = 0.f; continue; }
            const int ng = orc_gn_row(&gp, n, gp.ns ? (int)(v / (size_t)gp.zhw) : 0) * gp.G + c / cpg;
            r[k] = apply_silu(r[k], gp.mean[ng], gp.rstd[ng], gp.gamma[c], gp.beta[c]);
        }
        ysc[i] = orc_store_row(ybits, r, bw, y + (size_t)i * yrb, 1);
    }
}
/* src/lp_mx_gn.cu:34-73: fine (z, y, x) <- 8 coarse rows, weights .75 / .25 per axis, edge clamp, fma order z, y, x */
void orc_up2_mx(int xbits, const uint8_t *x, int N, int C, int D, int H, int W, orc_gn_t gp, uint8_t *y, int ybits) {
    const size_t Sc = (size_t)D * H * W, Sf = Sc * 8; const int Hf = 2 * H, Wf = 2 * W;
    const mxt_t t = mxt(x, xbits, N, C, Sc);
    const int bw = t.bw, nb = t.nb, yrb = rowbytes(bw, ybits), cpg = gp.G ? C / gp.G : 1;
    uint8_t *ysc = y + (size_t)N * nb * Sf * yrb;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)((size_t)N * nb * Sf); i++) {
        const size_t v = (size_t)i % Sf; const int blk = (int)(((size_t)i / Sf) % nb), n = (int)((size_t)i / (Sf * nb));
        const int gz = (int)(v / ((size_t)Hf * Wf)), gy = (int)(v / Wf % Hf), gx = (int)(v % Wf);
        int mz[2], my[2], mx[2];
        mz[0] = gz >> 1; mz[1] = mz[0] + ((gz & 1) ? 1 : -1); if (mz[1] < 0) mz[1] = 0; if (mz[1] > D - 1) mz[1] = D - 1;
        my[0] = gy >> 1; my[1] = my[0] + ((gy & 1) ? 1 : -1); if (my[1] < 0) my[1] = 0; if (my[1] > H - 1) my[1] = H - 1;
        mx[0] = gx >> 1; mx[1] = mx[0] + ((gx & 1) ? 1 : -1); if (mx[1] < 0) mx[1] = 0; if (mx[1] > W - 1) mx[1] = W - 1;
        float o[32] = {0};
        for (int a = 0; a < 2; a++) for (int b = 0; b < 2; b++) for (int c = 0; c < 2; c++) {
            float r[32]; mx_row32(&t, n, blk, ((size_t)mz[a] * H + my[b]) * W + mx[c], r);
            if (gp.G) for (int k = 0; k < bw; k++) {
                const int ch = blk * bw + k; if (ch >= C) continue;
                const int ng = n * gp.G + ch / cpg; const float aa = gp.rstd[ng] * gp.gamma[ch], bb = fmaf(-gp.mean[ng], aa, gp.beta[ch]);
                r[k] = orc_act_ab(r[k], aa, bb);   /* src/lp_mx_gn.cu:66-67: the staging form of GN + SiLU */
            }
            const float w3 = (a ? 0.25f : 0.75f) * (b ? 0.25f : 0.75f) * (c ? 0.25f : 0.75f);
            for (int k = 0; k < bw; k++) o[k] = fmaf(w3, r[k], o[k]);
        }
        ysc[i] = orc_store_row(ybits, o, bw, y + (size_t)i * yrb, 1);
    }
}
/* src/lp_mx_conv1.cu:5-21: fp32 FMA in ci order, bias first */
void orc_conv1_mx(int xbits, const uint8_t *x, int N, int Ci, size_t S, const float *w, const float *b, int Co, orc_gn_t gp, float *y) {
    const mxt_t t = mxt(x, xbits, N, Ci, S); const int cpg = gp.G ? Ci / gp.G : 1;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)((size_t)N * S); i++) {
        const size_t v = (size_t)i % S; const int n = (int)((size_t)i / S);
        float xin[1024];
        for (int blk = 0; blk < t.nb; blk++) mx_row32(&t, n, blk, v, xin + blk * t.bw);
        if (gp.G) for (int ci = 0; ci < Ci; ci++) { const int ng = orc_gn_row(&gp, n, gp.ns ? (int)(v / (size_t)gp.zhw) : 0) * gp.G + ci / cpg; const float a = gp.rstd[ng] * gp.gamma[ci], bb = fmaf(-gp.mean[ng], a, gp.beta[ci]); xin[ci] = orc_act_ab(xin[ci], a, bb); }
        for (int co = 0; co < Co; co++) {
            float acc = b ? b[co] : 0.f;
            for (int ci = 0; ci < Ci; ci++) acc = fmaf(w[(size_t)co * Ci + ci], xin[ci], acc);
            y[((size_t)n * Co + co) * S + v] = acc;
        }
    }
}

/* ---------- MX GEMM (src/lp_mxgemm.cu:1-5, :17-41 staging, :88-113 packing, :266-297 entry) ----------
   C[M][N] = op(A) op(B) + bias[col] + res[row][col] + beta C; A is [M][K] (ta 0) or [K][M] (ta 1), B is [K][N] (tb 0) or [N][K] (tb 1).
   Every 32 K-values of an A row / B column get one scale from the fmaxf amax (zero past K), the elements round to e2m1 / e4m3; the
   products of one 32-K block are summed exactly, the block sums accumulate in fp32 in K order. */
static void gemm_quant_rows(int bits, const float *X, int tr, int ld, int rows, int K, int nkb, float *Q) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < (int64_t)rows * nkb; i++) {
        const int r = (int)(i / nkb), kb = (int)(i % nkb);
        float v[32]; uint8_t codes[32];
        for (int j = 0; j < 32; j++) { const int k = kb * 32 + j; v[j] = k < K ? (tr ? X[(size_t)k * ld + r] : X[(size_t)r * ld + k]) : 0.f; }
        const uint8_t sb = orc_store_row(bits, v, 32, codes, 0);
        orc_load_row(bits, codes, sb, 32, Q + (size_t)i * 32);
    }
}
int orc_mx_gemm(int bits, int ta, int tb, int M, int N, int K, const float *A, const float *B, float *C, float beta, const float *bias, const float *res) {
    if (bits != 4 && bits != 8) return -1;
    if (M <= 0 || N <= 0) return 0;
    const int nkb = (K + 31) / 32;
    float *Aq = (float *)malloc((size_t)M * nkb * 32 * sizeof(float) + 4), *Bq = (float *)malloc((size_t)N * nkb * 32 * sizeof(float) + 4);
    gemm_quant_rows(bits, A, ta, ta ? M : K, M, K, nkb, Aq);
    gemm_quant_rows(bits, B, !tb, tb ? K : N, N, K, nkb, Bq);    /* B's "rows" are the output columns */
#pragma omp parallel for schedule(static)
    for (int64_t ij = 0; ij < (int64_t)M * N; ij++) {
        const int i = (int)(ij / N), j = (int)(ij % N);
        const float *a = Aq + (size_t)i * nkb * 32, *b = Bq + (size_t)j * nkb * 32;
        float acc = 0.f;
        for (int kb = 0; kb < nkb; kb++) { double s = 0.0; for (int k = 0; k < 32; k++) s += (double)a[kb * 32 + k] * (double)b[kb * 32 + k]; acc += (float)s; }
        float *p = C + (size_t)i * N + j;
        *p = acc + (bias ? bias[j] : 0.f) + (res ? res[(size_t)i * N + j] : 0.f) + (beta != 0.f ? beta * *p : 0.f);
    }
    free(Aq); free(Bq);
    return 0;
}

/* ---------- MX-fp8 attention forward (src/lp_attn8.cu:29-76 conversions, :124-180 forward, :319-328 entry) ----------
   qkvh: fp16 [3][H][T + 64][48] (T = nseq S; row of token i of sequence s = s S + i). Q and K rows are quantised in two blocks (dims
   0..31, dims 32..47 zero-padded to 32); V is quantised along the tokens: per (head, dim) one scale per 32 tokens of the sequence
   (tokens past S are zero). Keys are visited in tiles of 64: logits s = (q . k) log2(e) / sqrt(48), keys past S masked; running maximum
   m and sum l in base 2; P = 2^(s - m) is quantised per query per 32 keys and multiplied with the quantised V, the accumulator rescaled
   by 2^(m_old - m_new). o [T][C] = acc / l at column h 48 + d; lse [nseq][H][S] = m + log2(l). */
void orc_fa8_fwd(const uint16_t *qkvh, float *o, float *lse, int nseq, int S, int H, int C) {
    enum { HD = 48, FT = 64 };
    const int64_t T = (int64_t)nseq * S, Tp = T + FT; const int Sp = (S + FT - 1) / FT * FT;
    const float sl2 = 1.4426950408889634f / sqrtf((float)HD);
    const uint16_t *Qh = qkvh, *Kh = Qh + (size_t)H * Tp * HD, *Vh = Kh + (size_t)H * Tp * HD;
    for (int seq = 0; seq < nseq; seq++) for (int h = 0; h < H; h++) {
        float *qd = (float *)calloc((size_t)Sp * 64, sizeof(float)), *kd = (float *)calloc((size_t)Sp * 64, sizeof(float)), *vd = (float *)calloc((size_t)HD * Sp, sizeof(float));
        for (int p = 0; p < 2; p++) {
            const uint16_t *src = (p ? Kh : Qh) + ((size_t)h * Tp + (size_t)seq * S) * HD; float *dst = p ? kd : qd;
#pragma omp parallel for schedule(static)
            for (int i = 0; i < S; i++) for (int kb = 0; kb < 2; kb++) {
                float v[32]; uint8_t codes[32]; const int n = kb ? HD - 32 : 32;
                for (int j = 0; j < 32; j++) v[j] = j < n ? orc_h16_to_f32(src[(size_t)i * HD + 32 * kb + j]) : 0.f;
                const uint8_t sb = orc_store_row(8, v, 32, codes, 0);
                orc_load_row(8, codes, sb, 32, dst + (size_t)i * 64 + 32 * kb);
            }
        }
        const uint16_t *vs = Vh + ((size_t)h * Tp + (size_t)seq * S) * HD;
#pragma omp parallel for schedule(static)
        for (int d = 0; d < HD; d++) for (int b = 0; b < Sp / 32; b++) {
            float v[32]; uint8_t codes[32];
            for (int r = 0; r < 32; r++) { const int i = b * 32 + r; v[r] = i < S ? orc_h16_to_f32(vs[(size_t)i * HD + d]) : 0.f; }
            const uint8_t sb = orc_store_row(8, v, 32, codes, 0);
            orc_load_row(8, codes, sb, 32, vd + (size_t)d * Sp + b * 32);
        }
#pragma omp parallel for schedule(dynamic, 16)
        for (int i = 0; i < S; i++) {
            float m = -INFINITY, l = 0.f, acc[HD]; for (int d = 0; d < HD; d++) acc[d] = 0.f;
            const float *q = qd + (size_t)i * 64;
            for (int kb = 0; kb < S; kb += FT) {
                float s[FT], mx = -INFINITY;
                for (int j = 0; j < FT; j++) {
                    const float *k = kd + (size_t)(kb + j) * 64; float a = 0.f;
                    for (int b = 0; b < 2; b++) { double t = 0.0; for (int c = 0; c < 32; c++) t += (double)q[32 * b + c] * (double)k[32 * b + c]; a += (float)t; }
                    s[j] = kb + j < S ? a * sl2 : -INFINITY; mx = fmaxf(mx, s[j]);
                }
                const float mn = fmaxf(m, mx), corr = exp2f(m - mn); m = mn; l *= corr;
                for (int j = 0; j < FT; j++) { s[j] = exp2f(s[j] - m); l += s[j]; }
                for (int d = 0; d < HD; d++) acc[d] *= corr;
                for (int b = 0; b < 2; b++) {
                    uint8_t codes[32]; float pq[32];
                    const uint8_t sb = orc_store_row(8, s + 32 * b, 32, codes, 0);
                    orc_load_row(8, codes, sb, 32, pq);
                    for (int d = 0; d < HD; d++) {
                        const float *v = vd + (size_t)d * Sp + kb + 32 * b; double t = 0.0;
                        for (int j = 0; j < 32; j++) t += (double)pq[j] * (double)v[j];
                        acc[d] += (float)t;
                    }
                }
            }
            const float il = 1.f / l; float *orow = o + ((size_t)seq * S + i) * C + h * HD;
            for (int d = 0; d < HD; d++) orow[d] = acc[d] * il;
            lse[((size_t)seq * H + h) * S + i] = m + log2f(l);
        }
        free(qd); free(kd); free(vd);
    }
}

/* ---------- sliding-window prediction: placement and feather blend ---------- */
/* src/nn_elem.cu:1105-1125 (place_isect, pred_place_k): the window voxels inside both the window's interior ([hz, D - hz) x [halo, W - halo)^2)
   and the target box ([-o, e - o)) become uint8 probabilities at target index ((o_z + z) shard + o_y + y) shard + o_x + x; CT below iso -> 0 */
void orc_pred_place(const float *lg, const uint8_t *ct, int D, int W, int hz, int halo, int oz, int oy, int ox, int ez, int ey, int ex, int shard, int iso, uint8_t *dsh) {
    const int z0 = hz > -oz ? hz : -oz, y0 = halo > -oy ? halo : -oy, x0 = halo > -ox ? halo : -ox;
    const int z1 = D - hz < ez - oz ? D - hz : ez - oz, y1 = W - halo < ey - oy ? W - halo : ey - oy, x1 = W - halo < ex - ox ? W - halo : ex - ox;
    for (int z = z0; z < z1; z++) for (int y = y0; y < y1; y++) for (int x = x0; x < x1; x++) {
        const size_t k = ((size_t)z * W + y) * W + x;
        dsh[((size_t)(oz + z) * shard + (oy + y)) * shard + (ox + x)] = ct[k] >= iso ? (uint8_t)(255.f / (1.f + expf(-lg[k])) + 0.5f) : 0;
    }
}
/* src/predict.c:282-333 (feather_t, fe_val, fe_blend, fe_rows), :334-375 (which earlier windows are held): windows of interior S on a grid
   nss[3] in z-y-x order, each with its prediction E over [0, S + B)^3 from its interior origin (E: [window][S + B]^3 bytes; present: which
   windows were computed). The output over a window's interior is its own E except in the lower shell (a coordinate < B), where the
   windows shifted back by delta in {0,1}^3 that are present are blended with weights prod_d (delta_d ? 1 - u(v_d) : u(v_d)),
   u(j) = sin^2(pi/2 (j + .5) / B), normalised; bn: the output box, clipped inside the window grid. */
void orc_feather_blend(const uint8_t *E, const uint8_t *present, int S, int B, const int64_t nss[3], const int64_t bn[3], uint8_t *out) {
    const int En = S + B; const size_t e3 = (size_t)En * En * En;
    float u[2][1024];
    for (int j = 0; j < B; j++) { const double s = sin(M_PI / 2 * (j + 0.5) / B); u[0][j] = (float)(s * s); u[1][j] = (float)(1 - s * s); }
#pragma omp parallel for schedule(static)
    for (int64_t gz = 0; gz < bn[0]; gz++) for (int64_t gy = 0; gy < bn[1]; gy++) for (int64_t gx = 0; gx < bn[2]; gx++) {
        const int64_t a = gz / S, b = gy / S, c = gx / S; const int z = (int)(gz - a * S), y = (int)(gy - b * S), x = (int)(gx - c * S);
        const int64_t id = (a * nss[1] + b) * nss[2] + c;
        uint8_t *o = out + ((size_t)gz * bn[1] + gy) * bn[2] + gx;
        if (!present[id]) { *o = 0; continue; }
        const uint8_t *e = E + (size_t)id * e3;
        if (z >= B && y >= B && x >= B) { *o = e[((size_t)z * En + y) * En + x]; continue; }
        float s = 0, w = 0;
        for (int d = 0; d < 8; d++) {
            const int dz = d >> 2 & 1, dy = d >> 1 & 1, dx = d & 1;
            const int64_t qa = a - dz, qb = b - dy, qc = c - dx;
            if (qa < 0 || qb < 0 || qc < 0) continue;
            const int64_t qid = (qa * nss[1] + qb) * nss[2] + qc;
            if (d && !present[qid]) continue;
            if ((dz && z >= B) || (dy && y >= B) || (dx && x >= B)) continue;
            const float wi = (z < B ? u[dz][z] : 1.f) * (y < B ? u[dy][y] : 1.f) * (x < B ? u[dx][x] : 1.f);
            const uint8_t v = E[(size_t)qid * e3 + ((size_t)(z + dz * S) * En + (y + dy * S)) * En + (x + dx * S)];
            s += wi * v; w += wi;
        }
        *o = w > 0 ? (uint8_t)fminf(255.f, s / w + 0.5f) : 0;
    }
}

/* ---------- attention block around the MX GEMM and the fp8 attention core (src/nn_attn.cu:150-167 LayerNorm, :438-446 SwiGLU, :748-759 token
   layout, :587-633 block forward; src/nn_attn_tc.cu:99-136 QK-norm + gains + RoPE pack) ---------- */
void orc_ln_fwd(const float *x, const float *g, const float *b, float *y, float *mean, float *rstd, long T, int C) {
#pragma omp parallel for schedule(static)
    for (long r = 0; r < T; r++) {
        const float *xr = x + (size_t)r * C; double s = 0, q = 0;
        for (int c = 0; c < C; c++) s += xr[c];
        const float m = (float)(s / C);
        for (int c = 0; c < C; c++) { const double d = (double)xr[c] - m; q += d * d; }
        const float rs = 1.f / sqrtf((float)(q / C) + 1e-5f);
        for (int c = 0; c < C; c++) y[(size_t)r * C + c] = (xr[c] - m) * rs * g[c] + b[c];
        if (mean) mean[r] = m;
        if (rstd) rstd[r] = rs;
    }
}
void orc_glu_fwd(const float *h, float *gg, long T, int F) {
    for (long t = 0; t < T; t++) for (int f = 0; f < F; f++) { const float a = h[(size_t)t * 2 * F + f], b = h[(size_t)t * 2 * F + F + f]; gg[(size_t)t * F + f] = a / (1.f + expf(-a)) * b; }
}
void orc_cs_to_tok(const float *x, float *t, const float *reg, int n, int C, long Sg, int nreg) {
    const long S = Sg + nreg;
    for (long r = 0; r < (long)n * S; r++) for (int c = 0; c < C; c++) {
        const long s = r / S, ts = r % S - nreg;
        t[(size_t)r * C + c] = ts < 0 ? reg[(size_t)(r % S) * C + c] : x[((size_t)s * C + c) * Sg + ts];
    }
}
/* conv positional encoding (src/attn.h:141-144, src/nn_attn.cu:688-705): y = x + b + depthwise 3^3 conv of x on the grid tokens (zero padding),
   register rows copied; each sum starts from x + b and takes the taps inside the grid in (dz, dy, dx) order, one fused multiply-add each */
void orc_peg_fwd(const float *x, float *y, const float *w, const float *b, int nseq, int S, int D, int Hh, int W, int nreg, int C) {
    for (long t = 0; t < (long)nseq * S; t++) for (int c = 0; c < C; c++) {
        const int ts = (int)(t % S) - nreg;
        const size_t i = (size_t)t * C + c;
        if (ts < 0) { y[i] = x[i]; continue; }
        const long g0 = t - ts;
        const int z = ts / (Hh * W), yy = (ts / W) % Hh, xx = ts % W;
        float a = x[i] + b[c];
        for (int dz = -1; dz <= 1; dz++) for (int dy = -1; dy <= 1; dy++) for (int dx = -1; dx <= 1; dx++) {
            const int zz = z + dz, y2 = yy + dy, x2 = xx + dx;
            if (zz < 0 || zz >= D || y2 < 0 || y2 >= Hh || x2 < 0 || x2 >= W) continue;
            a = fmaf(w[c * 27 + (dz + 1) * 9 + (dy + 1) * 3 + dx + 1], x[(size_t)(g0 + ((long)zz * Hh + y2) * W + x2) * C + c], a);
        }
        y[i] = a;
    }
}
void orc_tok_to_cs(const float *t, float *x, int n, int C, long Sg, int nreg) {
    for (long s = 0; s < n; s++) for (int c = 0; c < C; c++) for (long ts = 0; ts < Sg; ts++) x[((size_t)s * C + c) * Sg + ts] = t[((size_t)s * (Sg + nreg) + nreg + ts) * C + c];
}
/* qkv fp32 [T][3C] -> fp16 head-major q, k, v [3][H][T + 64][48]: q and k rows RMS-normalised over the 48 head dims (eps 1e-6) times the gains,
   then (rope 1, grid tokens only) axial rotary pairs: 16 dims per axis z, y, x, 8 frequencies base^(-f / 8); rq / rk the normalisers,
   amx[1] = max |v| (amx[0], [2], [3] zero); the 64 rows past T are zero */
void orc_fa_pack(const float *qkv, const float *qg, const float *kg, uint16_t *qkvh, float *rq, float *rk, float *amx, int nseq, int S, int Hh, int W, int nreg, int C, int rope, float base) {
    enum { HD = 48, FT = 64 };
    const int H = C / HD; const long T = (long)nseq * S, Tp = T + FT; const float lbase = log2f(base);
    float vmax = 0.f;
    for (int p = 0; p < 3; p++) for (int h = 0; h < H; h++) for (long t = 0; t < Tp; t++) {
        uint16_t *dst = qkvh + ((size_t)p * H * Tp + (size_t)h * Tp + t) * HD;
        if (t >= T) { for (int d = 0; d < HD; d++) dst[d] = 0; continue; }
        float v[HD];
        for (int d = 0; d < HD; d++) v[d] = qkv[(size_t)t * 3 * C + (size_t)p * C + h * HD + d];
        if (p < 2) {
            float s = 0.f; for (int d = 0; d < HD; d++) s += v[d] * v[d];
            const float r = 1.f / sqrtf(s / HD + 1e-6f); const float *gs = (p ? kg : qg) + h * HD;
            for (int d = 0; d < HD; d++) v[d] *= r * gs[d];
            (p ? rk : rq)[t * H + h] = r;
            const int ts = (int)(t % S) - nreg;
            if (rope && ts >= 0) {
                const float pos[3] = {(float)(ts / (Hh * W)), (float)((ts / W) % Hh), (float)(ts % W)};
                for (int pr = 0; pr < 24; pr++) {
                    const int ax = pr / 8, fi = pr % 8; const float ang = pos[ax] * exp2f(-lbase * (float)fi / 8.f), sn = sinf(ang), cs = cosf(ang);
                    const float a = v[ax * 16 + 2 * fi], b = v[ax * 16 + 2 * fi + 1];
                    v[ax * 16 + 2 * fi] = a * cs - b * sn; v[ax * 16 + 2 * fi + 1] = a * sn + b * cs;
                }
            }
        } else for (int d = 0; d < HD; d++) vmax = fmaxf(vmax, fabsf(v[d]));
        for (int d = 0; d < HD; d++) dst[d] = orc_f32_to_h16(v[d]);
    }
    if (amx) { amx[0] = 0.f; amx[1] = vmax; amx[2] = 0.f; amx[3] = 0.f; }
}
/* the self-attention block (pre-LN, MHSA with QK-norm, SwiGLU) with MX linears of `bits` and the fp8 attention core; P: the block's
   parameters at the offsets of orc_block_layout; x, y fp32 [T][C] */
size_t orc_block_layout(int C, int F, size_t off, size_t *o) {   /* o[14]: ln1g ln1b wqkv bqkv qg kg wo bo ln2g ln2b w1 b1 w2 b2 (src/nn_attn.cu:460-480) */
    const size_t c = C, f = F;
    o[0] = off; off += c; o[1] = off; off += c; o[2] = off; off += 3 * c * c; o[3] = off; off += 3 * c; o[4] = off; off += c; o[5] = off; off += c;
    o[6] = off; off += c * c; o[7] = off; off += c; o[8] = off; off += c; o[9] = off; off += c; o[10] = off; off += 2 * f * c; o[11] = off; off += 2 * f;
    o[12] = off; off += c * f; o[13] = off; off += c;
    return off;
}
int orc_block_fwd(int bits, int C, int H, int F, int rope, int nreg, float rope_base, const float *P, const float *x, float *y, int nseq, int S, int Hh, int W) {
    return orc_block_fwd_vr(bits, C, H, F, rope, nreg, rope_base, P, x, y, nseq, S, Hh, W, 0, NULL, NULL);
}
/* the same with the value residual (src/nn_attn.cu:535-542, :609-610): vr 1 copies the block's V rows [T][C] into v1; vr 2 replaces V by
   v + lam[head] (v1 - v), one fused multiply-add, before the pack. Pinned by its special cases (lam 0: the plain block; lam 1: the
   first block's V) and by the exact block in fp64 (tests/test_oracle_block.py) */
int orc_block_fwd_vr(int bits, int C, int H, int F, int rope, int nreg, float rope_base, const float *P, const float *x, float *y, int nseq, int S, int Hh, int W, int vr, float *v1, const float *lam) {
    size_t o[14]; orc_block_layout(C, F, 0, o);
    const long T = (long)nseq * S;
    float *xn = malloc((size_t)T * C * 4), *qkv = malloc((size_t)T * 3 * C * 4), *att = malloc((size_t)T * C * 4), *x1 = malloc((size_t)T * C * 4), *hh = malloc((size_t)T * 2 * F * 4), *gg = malloc((size_t)T * F * 4);
    float *rq = malloc((size_t)T * H * 4), *rk = malloc((size_t)T * H * 4), *lse = malloc((size_t)T * H * 4), amx[4];
    uint16_t *qh = malloc((size_t)3 * C * (T + 64) * 2);
    orc_ln_fwd(x, P + o[0], P + o[1], xn, NULL, NULL, T, C);
    int e = orc_mx_gemm(bits, 0, 1, (int)T, 3 * C, C, xn, P + o[2], qkv, 0.f, P + o[3], NULL);
    for (long t = 0; vr && t < T; t++) for (int c = 0; c < C; c++) {
        float *v = qkv + (size_t)t * 3 * C + 2 * C + c;
        if (vr == 1) v1[(size_t)t * C + c] = *v; else *v = fmaf(lam[c / (C / H)], v1[(size_t)t * C + c] - *v, *v);
    }
    orc_fa_pack(qkv, P + o[4], P + o[5], qh, rq, rk, amx, nseq, S, Hh, W, nreg, C, rope, rope_base);
    orc_fa8_fwd(qh, att, lse, nseq, S, H, C);
    e |= orc_mx_gemm(bits, 0, 1, (int)T, C, C, att, P + o[6], x1, 0.f, P + o[7], x);
    orc_ln_fwd(x1, P + o[8], P + o[9], xn, NULL, NULL, T, C);
    e |= orc_mx_gemm(bits, 0, 1, (int)T, 2 * F, C, xn, P + o[10], hh, 0.f, P + o[11], NULL);
    orc_glu_fwd(hh, gg, T, F);
    e |= orc_mx_gemm(bits, 0, 1, (int)T, C, F, gg, P + o[12], y, 0.f, P + o[13], x1);
    free(xn); free(qkv); free(att); free(x1); free(hh); free(gg); free(rq); free(rk); free(lse); free(qh);
    return e;
}
