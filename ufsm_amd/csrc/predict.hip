// Sliding-window prediction: logits -> uint8 placement (src/nn_elem.cu:1103-1130 of the reference), window gather from a resident volume,
// and the feather blend of window borders (src/predict.c:282-333) as a device kernel over the whole output box. All HBM-bound byte work.
#include <math.h>
#include "mx_dev.hpp"
#include "../../include/mi_predict.h"

static int g_pred_iso = 1;
extern "C" void nn_set_pred_iso(int t) { g_pred_iso = t < 1 ? 1 : t; }
extern "C" int nn_get_pred_iso(void) { return g_pred_iso; }

// ---- placement (src/nn_elem.cu:1103-1130): out = CT >= iso ? uint8(255 sigmoid(logit) + .5) : 0 over the window's interior clipped to the
// target box. The clipped region is rows of nx voxels; a thread owns a run of PLACE_RUN voxels of one row (its logits and CT bytes are two
// contiguous reads, its bytes one contiguous write), the runs of a row are neighbouring threads ----
constexpr int PLACE_RUN = 8;
struct place_rows_t { int z0, y0, x0, ny, nx, nrun; };
constexpr int PRED_BATCH = 16;                     // windows of one launch (their offsets travel in the kernel arguments)
struct place_dst_t { long long off[PRED_BATCH]; };      // window j (blockIdx.y) writes from dsh + off[j]
__global__ void __launch_bounds__(256) place_rows_k(const float *__restrict__ lg0, size_t lstride, const uint8_t *__restrict__ ct0, size_t cstride, place_rows_t P, size_t nthreads, int W,
                                                    int oz, int oy, int ox, int shard, uint8_t *__restrict__ dsh0, place_dst_t dst, int iso) {
    const size_t t = blockIdx.x * (size_t)256 + threadIdx.x;
    if (t >= nthreads) return;
    const float *lg = lg0 + blockIdx.y * lstride; const uint8_t *ct = ct0 + blockIdx.y * cstride; uint8_t *dsh = dsh0 + dst.off[blockIdx.y];
    const size_t row = t / (unsigned)P.nrun;
    const int run = (int)(t - row * P.nrun), y = P.y0 + (int)(row % (unsigned)P.ny), z = P.z0 + (int)(row / (unsigned)P.ny), x = P.x0 + run * PLACE_RUN;
    const int n = min(PLACE_RUN, P.x0 + P.nx - x);
    const float *l = lg + ((size_t)z * W + y) * W + x; const uint8_t *c = ct + ((size_t)z * W + y) * W + x;
    uint8_t *o = dsh + ((size_t)(oz + z) * shard + (oy + y)) * shard + (ox + x);
    float v[PLACE_RUN]; uint8_t m[PLACE_RUN];
#pragma unroll
    for (int i = 0; i < PLACE_RUN; i++) { const int k = i < n ? i : 0; v[i] = l[k]; m[i] = c[k]; }
#pragma unroll
    for (int i = 0; i < PLACE_RUN; i++) if (i < n) o[i] = m[i] >= iso ? (uint8_t)(255.f / (1.f + expf(-v[i])) + 0.5f) : (uint8_t)0;
}
// n windows of one geometry: window j's logits at lg + j lstride (floats), its CT at ct + j cstride, its target dsh + doff[j] (doff on the host)
extern "C" void mi_pred_place_n(const float *lg, size_t lstride, const uint8_t *ct, size_t cstride, int n, const int64_t *doff, int D, int W, int hz, int halo, int oz, int oy, int ox,
                                int ez, int ey, int ex, int shard, uint8_t *dsh) {
    // window voxel v lands at o + v of the target; kept: v inside the interior [h, dim - h) of its axis and o + v inside [0, e)
    const int lo[3] = {max(hz, -oz), max(halo, -oy), max(halo, -ox)}, hi[3] = {min(D - hz, ez - oz), min(W - halo, ey - oy), min(W - halo, ex - ox)};
    if (hi[0] <= lo[0] || hi[1] <= lo[1] || hi[2] <= lo[2]) return;
    place_rows_t P = {lo[0], lo[1], lo[2], hi[1] - lo[1], hi[2] - lo[2], (hi[2] - lo[2] + PLACE_RUN - 1) / PLACE_RUN};
    const size_t nthreads = (size_t)(hi[0] - lo[0]) * P.ny * P.nrun;
    for (int j0 = 0; j0 < n; j0 += PRED_BATCH) {
        const int nb = min(PRED_BATCH, n - j0);
        place_dst_t dst;
        for (int j = 0; j < PRED_BATCH; j++) dst.off[j] = j < nb ? (doff ? doff[j0 + j] : 0) : 0;
        place_rows_k<<<dim3(nblk_(nthreads, 256), nb), 256>>>(lg + (size_t)j0 * lstride, lstride, ct + (size_t)j0 * cstride, cstride, P, nthreads, W, oz, oy, ox, shard, dsh, dst, g_pred_iso);
    }
    MICK();
}
extern "C" void nn_pred_place_d(const float *lg, const uint8_t *ct, int D, int W, int hz, int halo, int oz, int oy, int ox, int ez, int ey, int ex, int shard, uint8_t *dsh) {
    mi_pred_place_n(lg, 0, ct, 0, 1, nullptr, D, W, hz, halo, oz, oy, ox, ez, ey, ex, shard, dsh);
}
extern "C" void nn_pred_place(const float *lg, const uint8_t *ct, int W, int halo, int oz, int oy, int ox, int ez, int ey, int ex, int shard, uint8_t *dsh) {
    nn_pred_place_d(lg, ct, W, W, halo, halo, oz, oy, ox, ez, ey, ex, shard, dsh);
}

// a thread moves 16 consecutive x of one window row: one 16-byte store, byte loads on the volume side (window origins are not aligned).
// blockIdx.y is the window of the launch: its origin from the kernel arguments, its bytes at win + y W^3, its flag at any + y
struct ctw_org_t { long long o[PRED_BATCH][3]; };
__global__ void __launch_bounds__(256) ct_window_k(const uint8_t *__restrict__ vol, long long Z, long long Y, long long X, ctw_org_t org,
                                                   int W, uint8_t *__restrict__ win0, int iso, int halo, unsigned *any0) {
    const int W16 = (W + 15) >> 4;
    const size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    if (i >= (size_t)W * W * W16) return;
    const long long oz = org.o[blockIdx.y][0], oy = org.o[blockIdx.y][1], ox = org.o[blockIdx.y][2];
    uint8_t *win = win0 + blockIdx.y * ((size_t)W * W * W);
    unsigned *any = any0 ? any0 + blockIdx.y : nullptr;
    const int xc = (int)(i % W16), y = (int)((i / W16) % W), z = (int)(i / ((size_t)W16 * W));
    const long long gz = oz + z, gy = oy + y;
    const bool rowin = gz >= 0 && gz < Z && gy >= 0 && gy < Y;
    const uint8_t *src = vol + ((size_t)(rowin ? gz : 0) * Y + (rowin ? gy : 0)) * X;
    unsigned found = 0u;
    uint8_t *dst = win + ((size_t)z * W + y) * W + xc * 16;
    const bool core_zy = z >= halo && z < W - halo && y >= halo && y < W - halo;
    unsigned wd[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const int xw = xc * 16 + k;
        const long long gx = ox + xw;
        const unsigned v = rowin && xw < W && gx >= 0 && gx < X ? (unsigned)src[gx] : 0u;
        wd[k >> 2] |= v << (8 * (k & 3));
        found |= (int)v >= iso && core_zy && xw >= halo && xw < W - halo;
    }
    if (xc * 16 + 16 <= W && (W & 15) == 0) *(uint4 *)dst = make_uint4(wd[0], wd[1], wd[2], wd[3]);      // (rows of a multiple of 16 voxels: 16-byte aligned)
    else for (int k = 0; k < 16 && xc * 16 + k < W; k++) dst[k] = (uint8_t)(wd[k >> 2] >> (8 * (k & 3)));
    // the flag only ever becomes 1: one atomic per wavefront that found material, and none once the flag reads set (a window of material made
    // every thread's atomic queue on the one address)
    if (any && __builtin_amdgcn_ballot_w64(found != 0u) != 0ull) {
        if ((threadIdx.x & 63) == __builtin_ctzll(__builtin_amdgcn_ballot_w64(true)) && *(volatile unsigned *)any == 0u) atomicOr(any, 1u);
    }
}
// n windows: window j's origin org[3 j .. 3 j + 2] (host), its bytes at win + j W^3, its flag any + j (any may be null)
extern "C" void mi_ct_windows(const uint8_t *vol, int64_t Z, int64_t Y, int64_t X, const int64_t *org, int n, int W, uint8_t *win, int iso, int halo, unsigned *any) {
    if (W <= 0 || n <= 0) return;
    const size_t nt = (size_t)W * W * ((W + 15) >> 4), w3 = (size_t)W * W * W;
    for (int j0 = 0; j0 < n; j0 += PRED_BATCH) {
        const int nb = min(PRED_BATCH, n - j0);
        ctw_org_t o;
        for (int j = 0; j < PRED_BATCH; j++) for (int d = 0; d < 3; d++) o.o[j][d] = j < nb ? org[3 * (j0 + j) + d] : 0;
        ct_window_k<<<dim3(nblk_(nt, 256), nb), 256>>>(vol, Z, Y, X, o, W, win + (size_t)j0 * w3, iso, halo, any ? any + j0 : nullptr);
    }
    MICK();
}
extern "C" void mi_ct_window(const uint8_t *vol, int64_t Z, int64_t Y, int64_t X, int64_t oz, int64_t oy, int64_t ox, int W, uint8_t *win, int iso, int halo, unsigned *any) {
    const int64_t org[3] = {oz, oy, ox};
    mi_ct_windows(vol, Z, Y, X, org, 1, W, win, iso, halo, any);
}

// "holds a voxel >= iso" of every cell of a grid over the volume: cell (a, b, c) of nss[3] is [a S, a S + S) x [b S, ..) x [c S, ..) clipped to the
// volume, i.e. the interior of the sliding window with that index. The cells tile the volume, so this is one read of it. A thread tests 16
// consecutive x of a cell row (one 16-byte load where the row start allows, else bytes); a workgroup's rows belong to one cell
__global__ void __launch_bounds__(256) ct_flags_k(const uint8_t *__restrict__ vol, long long Z, long long Y, long long X, int S, int n1, int n2, int iso, unsigned *__restrict__ any, int vec) {
    const int S16 = (S + 15) >> 4;
    const unsigned cell = blockIdx.x, c = cell % (unsigned)n2, b = (cell / (unsigned)n2) % (unsigned)n1, a = cell / ((unsigned)n2 * (unsigned)n1);
    const size_t i = blockIdx.y * (size_t)256 + threadIdx.x;
    unsigned found = 0u;
    if (i < (size_t)S * S * S16) {
        const int xc = (int)(i % S16), y = (int)((i / S16) % S), z = (int)(i / ((size_t)S16 * S));
        const long long gz = (long long)a * S + z, gy = (long long)b * S + y, gx0 = (long long)c * S + xc * 16;
        if (gz < Z && gy < Y && gx0 < X) {
            const uint8_t *src = vol + ((size_t)gz * Y + gy) * X + gx0;
            const int nx = (int)min((long long)min(16, S - xc * 16), X - gx0);
            if (vec && nx == 16) {
                const uint4 q = *(const uint4 *)src;
                const unsigned w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                for (int k = 0; k < 16; k++) found |= (int)((w[k >> 2] >> (8 * (k & 3))) & 255u) >= iso;
            } else for (int k = 0; k < nx; k++) found |= (int)src[k] >= iso;
        }
    }
    if (__builtin_amdgcn_ballot_w64(found != 0u) != 0ull) {
        if ((threadIdx.x & 63) == __builtin_ctzll(__builtin_amdgcn_ballot_w64(true)) && *(volatile unsigned *)(any + cell) == 0u) atomicOr(any + cell, 1u);
    }
}
extern "C" void mi_ct_flags(const uint8_t *vol, int64_t Z, int64_t Y, int64_t X, int S, const int64_t nss[3], int iso, unsigned *any) {
    const int64_t total = nss[0] * nss[1] * nss[2];
    if (S <= 0 || total <= 0) return;
    const size_t nt = (size_t)S * S * ((S + 15) >> 4);
    if (total > 0x7fffffff || nblk_(nt, 256) > 65535u) mi_die("mi_ct_flags: %lld cells of %d^3 do not fit one launch", (long long)total, S);
    const int vec = S % 16 == 0 && X % 16 == 0 && ((uintptr_t)vol & 15) == 0;
    ct_flags_k<<<dim3((unsigned)total, nblk_(nt, 256)), 256>>>(vol, Z, Y, X, S, (int)nss[1], (int)nss[2], iso, any, vec);
    MICK();
}

struct blend_geo { int S, B, En; long long n0, n1, n2, b0, b1, b2; };
// one thread per output voxel. Core voxels (the bulk) copy a byte; shell voxels gather up to eight windows in the reference's order
// (delta = 0 first, then bit 0 x, bit 1 y, bit 2 z) with separately rounded fp32 products and sums, as the host routine computes them.
__global__ void __launch_bounds__(256) feather_blend_k(const uint8_t *__restrict__ E, const uint8_t *__restrict__ present, blend_geo G, const float *__restrict__ u,
                                                       uint8_t *__restrict__ out) {
#pragma clang fp contract(off)       // products and sums round separately, as the host routine's do (no fused multiply-add)
    const size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    if (i >= (size_t)G.b0 * G.b1 * G.b2) return;
    const long long gx = (long long)(i % G.b2), gy = (long long)((i / G.b2) % G.b1), gz = (long long)(i / ((size_t)G.b2 * G.b1));
    const long long a = gz / G.S, b = gy / G.S, c = gx / G.S;
    const int z = (int)(gz - a * G.S), y = (int)(gy - b * G.S), x = (int)(gx - c * G.S), B = G.B, En = G.En;
    const size_t e3 = (size_t)En * En * En;
    const long long id = (a * G.n1 + b) * G.n2 + c;
    if (!present[id]) { out[i] = 0; return; }
    if (z >= B && y >= B && x >= B) { out[i] = E[(size_t)id * e3 + ((size_t)z * En + y) * En + x]; return; }
    float s = 0.f, w = 0.f;
#pragma unroll
    for (int d = 0; d < 8; d++) {
        const int dz = d >> 2 & 1, dy = d >> 1 & 1, dx = d & 1;
        const long long qa = a - dz, qb = b - dy, qc = c - dx;
        if (qa < 0 || qb < 0 || qc < 0) continue;
        const long long qid = (qa * G.n1 + qb) * G.n2 + qc;
        if (d && !present[qid]) continue;
        if ((dz && z >= B) || (dy && y >= B) || (dx && x >= B)) continue;
        const float wz = z < B ? u[dz * 1024 + z] : 1.f, wy = y < B ? u[dy * 1024 + y] : 1.f, wx = x < B ? u[dx * 1024 + x] : 1.f;
        const float wi = (wz * wy) * wx;
        const float v = (float)E[(size_t)qid * e3 + ((size_t)(z + dz * G.S) * En + (y + dy * G.S)) * En + (x + dx * G.S)];
        s += wi * v; w += wi;
    }
    out[i] = w > 0.f ? (uint8_t)fminf(255.f, s / w + 0.5f) : (uint8_t)0;
}
extern "C" int mi_feather_blend(const uint8_t *E, const uint8_t *present, int S, int B, const int64_t nss[3], const int64_t bn[3], uint8_t *out) {
    if (S <= 0 || B < 0 || B > S || B > 1024) return -1;            // (B 0: no blend, every voxel is its window's own)
    for (int d = 0; d < 3; d++) if (nss[d] <= 0 || bn[d] <= 0 || bn[d] > nss[d] * S) return -1;
    // u(j) = sin^2(pi/2 (j + .5) / B) and 1 - u(j) in double, rounded to fp32 (src/predict.c:337); the table lives in per-device scratch
    static thread_local float hu[2048];
    for (int j = 0; j < B; j++) { const double s = sin(M_PI / 2 * (j + 0.5) / B); hu[j] = (float)(s * s); hu[1024 + j] = (float)(1 - s * s); }
    float *du = (float *)mi_ws(MI_WS_MISC, sizeof hu);
    MIRT(hipMemcpyAsync(du, hu, sizeof hu, hipMemcpyHostToDevice, 0));
    MIRT(hipStreamSynchronize(0));                           // (hu is reused by the next call)
    blend_geo g = {S, B, S + B, nss[0], nss[1], nss[2], bn[0], bn[1], bn[2]};
    const size_t n = (size_t)bn[0] * bn[1] * bn[2];
    feather_blend_k<<<nblk_(n, 256), 256>>>(E, present, g, du, out);
    MICK();
    return 0;
}
