// Radial attention and scroll coordinates (src/nn_attn_ray.cu and src/attn.h:83-128 of the reference): the attention of a block runs along
// rays that leave the scroll axis in every axis-normal plane of the bottleneck grid instead of over the whole grid. This file holds the ray plan
// (host), the maps between grid token rows and ray samples (bilinear in the plane, edge-clamped), the scroll coordinates (r, arc, k) the rotary
// embedding turns by, and the attention core for such sequences: fp16 q / k / v, fp32 sums, keys past a sequence's length masked
// (at_fa_fwd, src/nn_attn_tc.cu:139-197). All device kernels here are short HBM- or latency-bound row kernels.
#include <hip/hip_fp16.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include "mx_dev.hpp"
#include "../../include/mi_attn.h"
#include "attn_ray.hpp"

#define HD AT_HD
#define FT 64

namespace {
inline int max3(int a, int b, int c) { return a > b ? (a > c ? a : c) : (b > c ? b : c); }

// One ray record: the half line from (cu, cv) at angle th, clipped to the plane's rectangle [-0.5, Nu - 0.5] x [-0.5, Nv - 0.5]; L = floor(chord)
// samples (at least one, at most Nr) at unit spacing, centred on the chord (src/nn_attn_ray.cu:22-41). Record: u0, v0, du, dv, r0, arc, len, k
void ray_record(float *rr, double cu, double cv, double th, double rc, int Nu, int Nv, int Nr, int k) {
    for (int i = 0; i < AT_RAY_F; i++) rr[i] = 0.f;
    rr[7] = (float)k;
    const double org[2] = {cu, cv}, dir[2] = {cos(th), sin(th)}, top[2] = {Nu - 0.5, Nv - 0.5};
    double t_in = 0, t_out = 1e300; bool miss = false;
    for (int e = 0; e < 2; e++) {
        if (fabs(dir[e]) < 1e-12) { miss |= org[e] < -0.5 || org[e] > top[e]; continue; }      // parallel to this pair of edges
        const double ta = (-0.5 - org[e]) / dir[e], tb = (top[e] - org[e]) / dir[e], tn = ta < tb ? ta : tb, tf = ta < tb ? tb : ta;
        if (tn > t_in) t_in = tn;
        if (tf < t_out) t_out = tf;
    }
    const double chord = t_out - t_in;
    if (miss || !(chord > 1e-6)) return;                            // a dummy of length 0
    int L = chord < 1 ? 1 : (int)floor(chord);
    if (L > Nr) L = Nr;
    const double t0 = t_in + 0.5 * (chord - (L - 1));
    rr[0] = (float)(cu + t0 * dir[0]); rr[1] = (float)(cv + t0 * dir[1]); rr[2] = (float)dir[0]; rr[3] = (float)dir[1];
    rr[4] = (float)t0; rr[5] = (float)(th * rc); rr[6] = (float)L;
}
}

extern "C" void at_rays_dims(int D, int Hh, int W, float mult, int *Q, int *Nt, int *Nr) {
    const int P = max3(D, Hh, W);
    int nt = (int)ceilf(mult * (float)P);
    if (nt < 1) nt = 1;
    const int lo = D < Hh ? (D < W ? D : W) : (Hh < W ? Hh : W);   // the longest plane diagonal over the axis choices spans the two largest dims
    const long long s2 = (long long)D * D + (long long)Hh * Hh + (long long)W * W - (long long)lo * lo;
    *Nr = (int)ceil(sqrt((double)s2)) + 1; *Nt = nt; *Q = P * nt;
}

extern "C" void at_rays_plan(int n, int D, int Hh, int W, float mult, const float *axr, float *ray_h, int *lens_h, int *ad_h, float *cen_h) {
    int Q, Nt, Nr; at_rays_dims(D, Hh, W, mult, &Q, &Nt, &Nr);
    const int P = max3(D, Hh, W);
    // UFSM_SCROLL_PE_V2 (the reference's knob, src/nn_attn_ray.cu:54-58; a net must have been trained with it): one reference angle and one
    // radius per sample for all its planes instead of one per plane
    static int v2 = -1;
    if (v2 < 0) { const char *e = getenv("UFSM_SCROLL_PE_V2"); v2 = e && atoi(e) > 0; }
    for (int b = 0; b < n; b++) {
        const float *a = axr + (size_t)b * AT_AXR(P);
        int ad = (int)a[0];
        if (ad < 0 || ad > 2) ad = 0;
        const bool valid = a[1] != 0.f;
        const plane_t pl = ray_plane(ad, D, Hh, W);
        const double mu = 0.5 * (pl.Nu - 1), mv = 0.5 * (pl.Nv - 1), rmin = 0.5 * (pl.Nu > pl.Nv ? pl.Nu : pl.Nv);      // the plane's middle; the smallest arc radius
        ad_h[b] = ad;
        float *rb = ray_h + (size_t)b * Q * AT_RAY_F, *cb = cen_h + (size_t)b * P * 4;
        int *lb = lens_h + (size_t)b * Q;
        memset(cb, 0, (size_t)P * 4 * sizeof *cb);
        double rc_all = 0, phi_all = 0;
        if (v2 && valid) {
            double sx = 0, sy = 0, sr = 0;
            for (int k = 0; k < pl.Np; k++) { const double du = mu - a[2 + 2 * k], dv = mv - a[3 + 2 * k]; sx += du; sy += dv; sr += hypot(du, dv); }
            rc_all = sr / pl.Np; if (rc_all < rmin) rc_all = rmin;
            phi_all = hypot(sx, sy) > 0.25 * pl.Np ? atan2(sy, sx) : 0.0;
        }
        for (int k = 0; k < P; k++) {
            // plane k's fan: all directions when the centre lies in the rectangle, else the angles the rectangle's corners span as seen from the centre
            double cu = 0, cv = 0, rc = 0, phim = 0, th0 = -M_PI, th1 = M_PI;
            if (valid && k < pl.Np) {
                cu = a[2 + 2 * k]; cv = a[3 + 2 * k];
                rc = hypot(mu - cu, mv - cv); if (rc < rmin) rc = rmin;
                if (v2) { rc = rc_all; phim = phi_all; th0 = phi_all - M_PI; th1 = phi_all + M_PI; }
                const bool inside = cu >= -0.5 && cu <= pl.Nu - 0.5 && cv >= -0.5 && cv <= pl.Nv - 0.5;
                if (!inside) {
                    if (!v2) phim = atan2(mv - cv, mu - cu);
                    th0 = 1e300; th1 = -1e300;
                    for (int q = 0; q < 4; q++) {
                        const double qu = q & 1 ? pl.Nu - 0.5 : -0.5, qv = q & 2 ? pl.Nv - 0.5 : -0.5;
                        const double th = phim + remainder(atan2(qv - cv, qu - cu) - phim, 2 * M_PI);
                        if (th < th0) th0 = th;
                        if (th > th1) th1 = th;
                    }
                }
                cb[4 * k] = (float)cu; cb[4 * k + 1] = (float)cv; cb[4 * k + 2] = (float)rc; cb[4 * k + 3] = (float)phim;
            }
            for (int j = 0; j < Nt; j++) {
                float *rr = rb + ((size_t)k * Nt + j) * AT_RAY_F;
                for (int i = 0; i < AT_RAY_F; i++) rr[i] = 0.f;
                rr[7] = (float)k;
                if (k >= pl.Np) continue;
                if (!valid) {                                      // no axis: the grid rows along v
                    if (j < pl.Nu) { rr[0] = (float)j; rr[3] = 1.f; rr[5] = (float)j; rr[6] = (float)(pl.Nv < Nr ? pl.Nv : Nr); }
                    continue;
                }
                ray_record(rr, cu, cv, th0 + (j + 0.5) * (th1 - th0) / Nt, rc, pl.Nu, pl.Nv, Nr, k);
            }
        }
        if (!valid) for (int k = 0; k < P; k++) cb[4 * k + 2] = -1.f;      // (no axis: at_scroll_pos gives the grid indices)
        for (int q = 0; q < Q; q++) { const int L = (int)rb[(size_t)q * AT_RAY_F + 6]; lb[q] = L > 0 ? L : 1; }
    }
}

// ---- device ----
namespace {
__global__ void __launch_bounds__(256) ray_pos_k(const float *__restrict__ ray, int Nr, long long n, float *__restrict__ pos) {
    const long long s = blockIdx.x * 256ll + threadIdx.x;
    if (s >= n) return;
    const float *rr = ray + (s / Nr) * AT_RAY_F;
    pos[3 * s] = rr[4] + (float)(s % Nr); pos[3 * s + 1] = rr[5]; pos[3 * s + 2] = rr[7];
}
// The inverse of the slots' stencils, per grid token: which ray samples touch it and with what weight. A token of plane k can only be touched by
// the rays of that plane (Nt of them), and on a ray only by the samples within 1.5 voxels of it in both plane coordinates (a sample's corners are
// at most one voxel from its clamped position, clamping moves a sample by at most half a voxel): at most five consecutive samples around the
// token's projection on the ray. Those candidates are run through the very stencil function the gather uses, so the two maps are exact
// adjoints. A thread lists its token's (slot, weight) pairs in (ray, sample) order: sums over the list have a fixed order, so the scatter and
// the weight sums give the same bits on every run (the reference adds with floating-point atomics in the order of arrival), and no atomics run.
struct ray_ent { int slot; float w; };
__global__ void __launch_bounds__(256) ray_inverse_k(ray_geo G, const float *__restrict__ ray, const int *__restrict__ ad, long long Tg, int Nt, int cap,
                                                     ray_ent *__restrict__ tab, int *__restrict__ cnt, float *__restrict__ winv) {
    const long long t = blockIdx.x * 256ll + threadIdx.x;
    if (t >= Tg) return;
    const int b = (int)(t / G.Sg); const long long ts = t - (long long)b * G.Sg;
    const int z = (int)(ts / ((long long)G.Hh * G.W)), y = (int)(ts / G.W % G.Hh), x = (int)(ts % G.W), axd = ad[b];
    const int k = axd == 0 ? z : axd == 1 ? y : x, ua = axd == 0 ? y : z, vb = axd == 2 ? y : x;
    int n = 0; float sum = 0.f;
    for (int j = 0; j < Nt; j++) {
        const long long rq = (long long)b * G.Q + (long long)k * Nt + j;
        const float *rr = ray + rq * AT_RAY_F;
        const int L = min((int)rr[6], G.Nr);
        if (L <= 0) continue;
        const float ist = ((float)ua - rr[0]) * rr[2] + ((float)vb - rr[1]) * rr[3];      // the token's projection on the ray, in samples
        const int i0 = max(0, (int)ceilf(ist - 2.2f)), i1 = min(L - 1, (int)floorf(ist + 2.2f));
        for (int i = i0; i <= i1; i++) {
            long long row[4]; float w[4];
            const long long sl = rq * G.Nr + i;
            const int nc = slot_stencil(G, ray, ad, sl, row, w);
            float ws = 0.f;
            for (int c = 0; c < nc; c++) if (row[c] == t) ws += w[c];
            if (ws != 0.f && n < cap) { if (tab) tab[t * cap + n] = ray_ent{(int)sl, ws}; n++; sum += ws; }
        }
    }
    if (cnt) cnt[t] = n;
    if (winv) winv[t] = sum > 1e-6f ? 1.f / sum : 0.f;
}
// grid rows -> ray rows: a thread forms four neighbouring channels of one slot. NORM: each corner's weight times the token's 1 / weight sum
template <bool NORM>
__global__ void __launch_bounds__(256) ray_gather_k(ray_geo G, const float *__restrict__ ray, const int *__restrict__ ad, const float *__restrict__ wsum,
                                                    long long n, int C4, const float4 *__restrict__ x, float4 *__restrict__ y) {
    const long long i = blockIdx.x * 256ll + threadIdx.x;
    if (i >= n * C4) return;
    const long long s = i / C4; const int c4 = (int)(i - s * C4);
    long long row[4]; float w[4];
    const int nc = slot_stencil(G, ray, ad, s, row, w);
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int c = 0; c < nc; c++) {
        const float wc = NORM ? w[c] * wsum[row[c]] : w[c];
        if (wc == 0.f) continue;
        const float4 v = x[row[c] * C4 + c4];
        a.x = fmaf(wc, v.x, a.x); a.y = fmaf(wc, v.y, a.y); a.z = fmaf(wc, v.z, a.z); a.w = fmaf(wc, v.w, a.w);
    }
    y[i] = a;
}
// ray rows -> grid rows: the adjoint, in gather form over the token's list. NORM: each weight times the token's 1 / weight sum
template <bool NORM>
__global__ void __launch_bounds__(256) ray_scatter_k(const ray_ent *__restrict__ tab, const int *__restrict__ cnt, int cap, const float *__restrict__ wsum, size_t n4, int C4,
                                                     const float4 *__restrict__ y, float4 *__restrict__ x) {
    const size_t i = blockIdx.x * (size_t)256 + threadIdx.x;
    if (i >= n4) return;
    const size_t t = i / C4; const int c4 = (int)(i - t * C4), n = cnt[t];
    const float sc = NORM ? wsum[t] : 1.f;
    const ray_ent *e = tab + t * cap;
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int q = 0; q < n; q++) {
        const float wc = e[q].w * sc;
        const float4 v = y[(size_t)e[q].slot * C4 + c4];
        a.x = fmaf(wc, v.x, a.x); a.y = fmaf(wc, v.y, a.y); a.z = fmaf(wc, v.z, a.z); a.w = fmaf(wc, v.w, a.w);
    }
    x[i] = a;
}
// the grid tokens' scroll coordinates (src/nn_attn_ray.cu:174-188): (r, arc, k) around the plane's centre, the angle unwrapped around the
// plane's reference angle; registers (0, 0, 0); without an axis (cen's radius < 0) the grid indices (v, u, k)
__global__ void __launch_bounds__(256) scroll_pos_k(long long n, long long S, int nreg, int Hh, int W, int P, const int *__restrict__ ad, const float *__restrict__ cen, float *__restrict__ pos) {
    const long long t = blockIdx.x * 256ll + threadIdx.x;
    if (t >= n) return;
    const int b = (int)(t / S); const long long ts = t % S - nreg;
    float *p = pos + 3 * t;
    if (ts < 0) { p[0] = p[1] = p[2] = 0.f; return; }
    const int z = (int)(ts / ((long long)Hh * W)), y = (int)(ts / W % Hh), x = (int)(ts % W), axd = ad[b];
    const int k = axd == 0 ? z : axd == 1 ? y : x, ua = axd == 0 ? y : z, vb = axd == 2 ? y : x;
    const float *c = cen + ((size_t)b * P + k) * 4;
    if (c[2] < 0.f) { p[0] = (float)vb; p[1] = (float)ua; p[2] = (float)k; return; }
    const float du = (float)ua - c[0], dv = (float)vb - c[1];
    const float th = c[3] + remainderf(atan2f(dv, du) - c[3], 6.283185307179586f);
    p[0] = sqrtf(du * du + dv * dv); p[1] = th * c[2]; p[2] = (float)k;
}

// ---- the attention core for sequences with lengths (at_fa_fwd): softmax(q k^T / sqrt(48)) v over the first lens[seq] keys of each sequence.
// A wavefront takes 64 queries of one (sequence, head), a lane one query: its q row and its output sums live in registers; the keys are walked
// in groups of eight, a key's k and v rows are the same for every lane, so they arrive through the scalar unit's loads and enter the
// multiply-adds as scalar operands (no LDS, no lane exchange). Probabilities are rounded to fp16 before they meet v, the denominator adds the
// unrounded ones: the rounding points of the fp16 tensor-core kernel this replaces. Ray sequences are 20 - 50 slots long: the arithmetic is
// a few percent of a block's and the kernel is latency-bound.
// QL: queries per (sequence, head) unit, 64 or - for sequences of at most 32 tokens - 32, two units per wavefront: a ray of 24 slots fills 75 % of
// the lanes instead of 37 % (the keys' rows are per-lane addresses either way; the walk runs to the longer of the two units' lengths)
template <int QL>
__global__ void __launch_bounds__(256) fa16_rows_k(const __half *__restrict__ Qh, const __half *__restrict__ Kh, const __half *__restrict__ Vh, float *__restrict__ o, float *__restrict__ lse,
                                                   int S, int H, int C, long long Tp, int nseq, float sl2, const int *__restrict__ lens) {
    const int nqt = (S + QL - 1) / QL, lane = threadIdx.x & 63;
    const long long nun = (long long)nseq * H * nqt;
    long long un = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * (64 / QL) + lane / QL;
    const bool live = un < nun;
    if (!live) un = nun - 1;                                       // (an idle half: the last unit's rows, nothing stored)
    const int qt = (int)(un % nqt), h = (int)(un / nqt % H), seq = (int)(un / nqt / H);
    const size_t base = ((size_t)h * Tp + (size_t)seq * S) * HD;
    const int SK = !live ? 0 : lens ? min(lens[seq], S) : S;
    const int SKw = QL == 64 ? SK : max(SK, __shfl_xor(SK, 32));   // how far this wavefront walks
    const int i = qt * QL + lane % QL;
    float q[HD], acc[HD];
    {
        const uint4 *qr = (const uint4 *)(Qh + base + (size_t)i * HD);      // (rows past the sequence's end are other rows of the padded array: read, never stored)
#pragma unroll
        for (int c = 0; c < HD / 8; c++) {
            const uint4 u = qr[c]; const __half2 *hp = (const __half2 *)&u;
#pragma unroll
            for (int e = 0; e < 4; e++) { const float2 f = __half22float2(hp[e]); q[8 * c + 2 * e] = f.x; q[8 * c + 2 * e + 1] = f.y; }
        }
    }
#pragma unroll
    for (int d = 0; d < HD; d++) acc[d] = 0.f;
    float m = -INFINITY, l = 0.f;
    const __half *K = Kh + base, *V = Vh + base;
    for (int j0 = 0; j0 < SKw; j0 += 8) {
        if (j0 >= SK) continue;                                    // (the other unit of the wavefront is longer)
        float s[8];
#pragma unroll
        for (int jj = 0; jj < 8; jj++) {
            const __half *kr = K + (size_t)(j0 + jj) * HD;                 // (a group may run past the length: rows of the padded array, masked)
            float a = 0.f;
#pragma unroll
            for (int d = 0; d < HD; d++) a = fmaf(q[d], __half2float(kr[d]), a);
            s[jj] = j0 + jj < SK ? a * sl2 : -INFINITY;
        }
        float mt = s[0];
#pragma unroll
        for (int jj = 1; jj < 8; jj++) mt = fmaxf(mt, s[jj]);
        const float mn = fmaxf(m, mt), corr = exp2f(m - mn);
        m = mn; l *= corr;
#pragma unroll
        for (int d = 0; d < HD; d++) acc[d] *= corr;
#pragma unroll
        for (int jj = 0; jj < 8; jj++) {
            const float p = exp2f(s[jj] - m), ph = __half2float(__float2half_rn(p));
            l += p;
            const __half *vr = V + (size_t)(j0 + jj) * HD;
#pragma unroll
            for (int d = 0; d < HD; d++) acc[d] = fmaf(ph, __half2float(vr[d]), acc[d]);
        }
    }
    if (i >= S || !live) return;
    const float il = l > 0.f ? 1.f / l : 0.f;
    float4 *orow = (float4 *)(o + ((size_t)seq * S + i) * C + h * HD);
#pragma unroll
    for (int c = 0; c < HD / 4; c++) orow[c] = make_float4(acc[4 * c] * il, acc[4 * c + 1] * il, acc[4 * c + 2] * il, acc[4 * c + 3] * il);
    lse[((size_t)seq * H + h) * S + i] = l > 0.f ? m + log2f(l) : 0.f;    // (a length-0 sequence: zero output)
}
}

// The tokens' sample lists live in library scratch: 5 Nt (slot, weight) pairs and a count per grid token. at_rays_setup builds them with the weight
// sums; a scatter whose ray set is the one last set up on this thread (same table pointer, same sizes, the scratch still where it was) reuses them,
// any other builds its own first (0.2 ms per 250 000 tokens) - a ray table changed in place needs a new at_rays_setup for its weight sums anyway.
namespace {
struct inv_key {
    const float *ray; const int *ad; const void *ws; int n, Q, Nt, Nr, D, Hh, W;
    bool operator==(const inv_key &o) const { return ray == o.ray && ad == o.ad && ws == o.ws && n == o.n && Q == o.Q && Nt == o.Nt && Nr == o.Nr && D == o.D && Hh == o.Hh && W == o.W; }
};
thread_local inv_key g_inv = {};
struct inv_tab { int *cnt; ray_ent *tab; int cap; };
inv_tab inverse_table(const at_rays *R, float *winv) {
    const ray_geo G = geo_of(R); const size_t Tg = (size_t)R->n * G.Sg; const int cap = 5 * R->Nt;
    int *cnt = (int *)mi_ws(MI_WS_RAY, Tg * ((size_t)cap * sizeof(ray_ent) + sizeof(int)) + 256);
    const inv_tab t = {cnt, (ray_ent *)(cnt + ((Tg + 63) & ~(size_t)63)), cap};
    const inv_key k = {R->ray, R->ad, cnt, R->n, R->Q, R->Nt, R->Nr, R->D, R->Hh, R->W};
    if (!winv && k == g_inv) return t;
    ray_inverse_k<<<nblk_(Tg, 256), 256>>>(G, R->ray, R->ad, (long long)Tg, R->Nt, cap, t.tab, t.cnt, winv);
    g_inv = k;
    return t;
}
}
static void rays_check(const at_rays *R, const char *who) {
    if (!R || R->n < 0 || R->Q <= 0 || R->Nr <= 0 || R->D <= 0 || R->Hh <= 0 || R->W <= 0 || !R->ad || !R->ray) mi_die("%s: an incomplete ray set", who);
}
extern "C" void at_rays_setup(const at_rays *R) {
    rays_check(R, "at_rays_setup");
    if (!R->pos || !R->wsum) mi_die("at_rays_setup: the ray set has no position / weight-sum buffers");
    const ray_geo G = geo_of(R); const long long Tr = (long long)R->n * R->Q * R->Nr, Tg = (long long)R->n * G.Sg;
    if (!Tr) return;
    ray_pos_k<<<nblk_((size_t)Tr, 256), 256>>>(R->ray, R->Nr, Tr, (float *)R->pos);
    if (Tr > 0x7fffffffll) mi_die("at_rays_setup: %lld ray slots", Tr);
    inverse_table(R, (float *)R->wsum);
    MICK();
}
extern "C" void at_ray_gather(const at_rays *R, const float *x, float *y, int Cc, int norm) {
    rays_check(R, "at_ray_gather");
    if (Cc <= 0 || Cc % 4 || ((uintptr_t)x & 15) || ((uintptr_t)y & 15) || (norm && !R->wsum)) mi_die("at_ray_gather: %d channels (a multiple of 4), 16-byte aligned rows", Cc);
    const ray_geo G = geo_of(R); const long long Tr = (long long)R->n * R->Q * R->Nr; const int C4 = Cc / 4;
    if (!Tr) return;
    if (norm) ray_gather_k<true><<<nblk_((size_t)Tr * C4, 256), 256>>>(G, R->ray, R->ad, R->wsum, Tr, C4, (const float4 *)x, (float4 *)y);
    else ray_gather_k<false><<<nblk_((size_t)Tr * C4, 256), 256>>>(G, R->ray, R->ad, R->wsum, Tr, C4, (const float4 *)x, (float4 *)y);
    MICK();
}
extern "C" void at_ray_scatter(const at_rays *R, const float *y, float *x, int Cc, int norm) {
    rays_check(R, "at_ray_scatter");
    if (Cc <= 0 || Cc % 4 || ((uintptr_t)x & 15) || ((uintptr_t)y & 15) || (norm && !R->wsum)) mi_die("at_ray_scatter: %d channels (a multiple of 4), 16-byte aligned rows", Cc);
    const ray_geo G = geo_of(R); const long long Tr = (long long)R->n * R->Q * R->Nr; const int C4 = Cc / 4;
    const size_t ng = (size_t)R->n * G.Sg * Cc;
    if (!ng) return;
    if ((long long)R->n * R->Q * R->Nr > 0x7fffffffll) mi_die("at_ray_scatter: %lld ray slots", (long long)R->n * R->Q * R->Nr);
    const inv_tab it = inverse_table(R, nullptr);
    const ray_ent *tab = it.tab; const int *cnt = it.cnt; const int cap = it.cap;
    if (norm) ray_scatter_k<true><<<nblk_(ng / 4, 256), 256>>>(tab, cnt, cap, R->wsum, ng / 4, C4, (const float4 *)y, (float4 *)x);
    else ray_scatter_k<false><<<nblk_(ng / 4, 256), 256>>>(tab, cnt, cap, R->wsum, ng / 4, C4, (const float4 *)y, (float4 *)x);
    MICK();
}
extern "C" void at_scroll_pos(int n, int nreg, int D, int Hh, int W, const int *ad, const float *cen, float *pos) {
    const long long S = nreg + (long long)D * Hh * W, N = (long long)n * S;
    if (N <= 0) return;
    scroll_pos_k<<<nblk_((size_t)N, 256), 256>>>(N, S, nreg, Hh, W, max3(D, Hh, W), ad, cen, pos);
    MICK();
}
extern "C" void at_fa_fwd(const void *qkvh, float *o, float *lse, const at_geom *g, int H, int C) {
    if (C != H * HD || g->nseq < 0 || g->S <= 0) mi_die("at_fa_fwd: C %d is not %d heads of %d, or an empty geometry", C, H, HD);
    const long long T = (long long)g->nseq * g->S, Tp = T + FT;
    if (!T) return;
    const __half *Qh = (const __half *)qkvh, *Kh = Qh + (size_t)H * Tp * HD, *Vh = Kh + (size_t)H * Tp * HD;
    const int QL = g->S <= 32 ? 32 : 64;
    const long long nw = ((long long)g->nseq * H * ((g->S + QL - 1) / QL) + 64 / QL - 1) / (64 / QL);      // wavefronts
    if (nw > 0x7fffffffll) mi_die("at_fa_fwd: %lld wavefronts", nw);
    const float sl2 = 1.4426950408889634f / sqrtf((float)HD);
    if (QL == 32) fa16_rows_k<32><<<nblk_((size_t)nw, 4), 256>>>(Qh, Kh, Vh, o, lse, g->S, H, C, Tp, g->nseq, sl2, g->lens);
    else fa16_rows_k<64><<<nblk_((size_t)nw, 4), 256>>>(Qh, Kh, Vh, o, lse, g->S, H, C, Tp, g->nseq, sl2, g->lens);
    MICK();
}
