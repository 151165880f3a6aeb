// Device-side geometry of radial attention shared by the ray maps (attn_ray.hip) and the QKV pack that reads through them (attn_block.hip):
// plane / token mapping and the bilinear stencil of a ray slot (src/attn.h:118-136 of the reference).
#pragma once
#include "mx_dev.hpp"
#include "../../include/mi_attn.h"

namespace {
struct plane_t { int Np, Nu, Nv; };                                 // planes along the axis dim, and the plane's two dims (u before v in z, y, x order)
__host__ __device__ inline plane_t ray_plane(int ad, int D, int Hh, int W) { return plane_t{ad == 0 ? D : ad == 1 ? Hh : W, ad == 0 ? Hh : D, ad == 2 ? Hh : W}; }
__host__ __device__ inline long long ray_token(int ad, int k, int a, int b, int Hh, int W) {      // grid token of in-plane (a, b) of plane k (src/attn.h:130-133)
    const int z = ad == 0 ? k : a, y = ad == 0 ? a : ad == 1 ? k : b, x = ad == 2 ? k : b;
    return ((long long)z * Hh + y) * W + x;
}
struct ray_geo { int Q, Nr, D, Hh, W; long long Sg; };
inline ray_geo geo_of(const at_rays *R) { return ray_geo{R->Q, R->Nr, R->D, R->Hh, R->W, (long long)R->D * R->Hh * R->W}; }
// the up to four grid rows under ray slot s and their bilinear weights (src/attn.h:118-128); 0 past the ray's length
__device__ __forceinline__ int slot_stencil(const ray_geo &G, const float *__restrict__ ray, const int *__restrict__ ad, long long s, long long *row, float *w) {
    const long long rq = s / G.Nr; const int i = (int)(s - rq * G.Nr), b = (int)(rq / G.Q);
    const float *rr = ray + rq * AT_RAY_F;
    if (i >= (int)rr[6]) return 0;
    const int axd = ad[b], k = (int)rr[7];
    const plane_t pl = ray_plane(axd, G.D, G.Hh, G.W);
    const float pu = fminf(fmaxf(fmaf((float)i, rr[2], rr[0]), 0.f), (float)(pl.Nu - 1)), pv = fminf(fmaxf(fmaf((float)i, rr[3], rr[1]), 0.f), (float)(pl.Nv - 1));
    const int a0 = max(min((int)pu, pl.Nu - 2), 0), b0 = max(min((int)pv, pl.Nv - 2), 0), a1 = min(a0 + 1, pl.Nu - 1), b1 = min(b0 + 1, pl.Nv - 1);
    const float fu = pu - (float)a0, fv = pv - (float)b0;
    const long long base = (long long)b * G.Sg;
    row[0] = base + ray_token(axd, k, a0, b0, G.Hh, G.W); w[0] = (1.f - fu) * (1.f - fv);
    row[1] = base + ray_token(axd, k, a1, b0, G.Hh, G.W); w[1] = fu * (1.f - fv);
    row[2] = base + ray_token(axd, k, a0, b1, G.Hh, G.W); w[2] = (1.f - fu) * fv;
    row[3] = base + ray_token(axd, k, a1, b1, G.Hh, G.W); w[3] = fu * fv;
    return 4;
}
}
