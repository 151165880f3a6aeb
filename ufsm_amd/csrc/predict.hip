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
__global__ void __launch_bounds__(256) place_rows_k(const float *__restrict__ lg, const uint8_t *__restrict__ ct, place_rows_t P, size_t nthreads, int W, int oz, int oy, int ox, int shard,
                                                    uint8_t *__restrict__ dsh, int iso) {
    const size_t t = blockIdx.x * (size_t)256 + threadIdx.x;
    if (t >= nthreads) return;
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
extern "C" void nn_pred_place_d(const float *lg, const uint8_t *ct, int D, int W, int hz, int halo, int oz, int oy, int ox, int ez, int ey, int ex, int shard, uint8_t *dsh) {
    // window voxel v lands at o + v of the target; kept: v inside the interior [h, dim - h) of its axis and o + v inside [0, e)
    const int lo[3] = {max(hz, -oz), max(halo, -oy), max(halo, -ox)}, hi[3] = {min(D - hz, ez - oz), min(W - halo, ey - oy), min(W - halo, ex - ox)};
    if (hi[0] <= lo[0] || hi[1] <= lo[1] || hi[2] <= lo[2]) return;
    place_rows_t P = {lo[0], lo[1], lo[2], hi[1] - lo[1], hi[2] - lo[2], (hi[2] - lo[2] + PLACE_RUN - 1) / PLACE_RUN};
    const size_t nthreads = (size_t)(hi[0] - lo[0]) * P.ny * P.nrun;
    place_rows_k<<<nblk_(nthreads, 256), 256>>>(lg, ct, P, nthreads, W, oz, oy, ox, shard, dsh, g_pred_iso);
    MICK();
}
extern "C" void nn_pred_place(const float *lg, const uint8_t *ct, int W, int halo, int oz, int oy, int ox, int ez, int ey, int ex, int shard, uint8_t *dsh) {
    nn_pred_place_d(lg, ct, W, W, halo, halo, oz, oy, ox, ez, ey, ex, shard, dsh);
}

// a thread moves 16 consecutive x of one window row: one 16-byte store, byte loads on the volume side (window origins are not aligned)
__global__ void __launch_bounds__(256) ct_window_k(const uint8_t *__restrict__ vol, long long Z, long long Y, long long X, long long oz, long long oy, long long ox,
                                                   int W, uint8_t *__restrict__ win, int iso, int halo, unsigned *any) {
    const int W16 = (W + 15) >> 4;
    const size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    if (i >= (size_t)W * W * W16) return;
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
extern "C" void mi_ct_window(const uint8_t *vol, int64_t Z, int64_t Y, int64_t X, int64_t oz, int64_t oy, int64_t ox, int W, uint8_t *win, int iso, int halo, unsigned *any) {
    if (W <= 0) return;
    const size_t n = (size_t)W * W * ((W + 15) >> 4);
    ct_window_k<<<nblk_(n, 256), 256>>>(vol, Z, Y, X, oz, oy, ox, W, win, iso, halo, any);
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
