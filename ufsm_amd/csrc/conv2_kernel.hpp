// 2x2x2 stride-2 convolution and transposed convolution with MX operands: the two other stride-2 layers a U-Net can have (the reference has a 3x3x3
// stride-2 down conv and a trilinear upsample, src/lp_s2.cu:4-9, src/lp_mx_gn.cu:32-33; these follow the same operand rules: rows of 32 channels per
// voxel with their E8M0 scale, weights scaled per (tap, output channel, 32 input channels), fp32 accumulation, the convs' own epilogue).
//
// Neither op has a halo: an input row feeds exactly one output voxel (down) or the eight voxels above it, one per tap (up). So both are GEMMs
// whose activation operand is read straight from the stored tensor into MFMA fragments, with no LDS and no re-layout: a voxel's row of block b is
// 32 (e4m3) or 16 (e2m1) contiguous bytes, lanes of a voxel tile read neighbouring rows, and lane (r, h) of a 32x32x64 MFMA takes bytes 16 h .. of
// both rows of a K pair (e4m3) or the whole row of unit h (e2m1), with unit h's scale byte.
//   down: column = output voxel, K = (tap, block) tap-major: pair units 2 p, 2 p + 1; the row of unit (t, b) is voxel (2 oz + dz, 2 oy + dy, 2 ox + dx)
//   up:   column = input voxel; the eight taps are eight GEMMs over K = blocks on the same rows (one tap per workgroup), each followed by an
//         epilogue whose output voxel is (2 iz + dz, 2 iy + dy, 2 ix + dx)
// A wavefront owns NT = 2 tiles of 32 consecutive columns (linear voxel index) and MT channel tiles of 32; the weights' fragments come from
// global memory in the prepared lane order (a few KiB per K pair, shared by every wavefront: cache hits).
#pragma once
#include "conv3_kernel.hpp"

template <int FMT, int OUT, bool UP, int MT>
__global__ void __launch_bounds__(256, 2) conv2_mx_k(const conv_args a) {
    constexpr int NT = 2, RB = fmt_t<FMT>::RB, WTILE = fmt_t<FMT>::WTILE;
    extern __shared__ __align__(16) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;
    const int n = blockIdx.z, cs = UP ? (int)(blockIdx.y % (unsigned)a.ncs) : (int)blockIdx.y, nb = a.nbs[0];      // (up: blockIdx.y = tap x channel slices)
    const size_t Sin = (size_t)a.D * a.H * a.W;
    const long long Scol = UP ? (long long)Sin : (long long)a.Do * a.Ho * a.Wo;
    conv_epi_consts<MT, false>(a, lds, cs, tid);
    __syncthreads();
    const long long ct0 = ((long long)blockIdx.x * 4 + wave) * NT;
    if (ct0 * 32 >= Scol) return;                            // (no barrier follows)
    // the lane's column of each tile: its input voxel (down: the voxel of tap (0, 0, 0)) and, for the epilogue, the coordinates
    size_t iv0[NT]; int c0[NT], c1[NT], c2[NT]; bool cok[NT];
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const long long col = (ct0 + j) * 32 + r;
        cok[j] = col < Scol;
        const long long cc = cok[j] ? col : 0;
        const int Wc = UP ? a.W : a.Wo, Hc = UP ? a.H : a.Ho;
        c2[j] = (int)(cc % Wc); c1[j] = (int)(cc / Wc % Hc); c0[j] = (int)(cc / ((long long)Wc * Hc));
        iv0[j] = UP ? (size_t)cc : ((size_t)(2 * c0[j]) * a.H + 2 * c1[j]) * a.W + 2 * c2[j];
    }
    const uint8_t *xq = a.xq[0] + (size_t)n * nb * Sin * RB, *xsc = a.xsc[0] + (size_t)n * nb * Sin;
    // the activation fragment of tile j for the K pair (block b0 at voxel offset o0 | block b1 at o1; ok1: the second unit exists)
    struct bfrag { v4i lo, hi; int sb; };
    auto fetch = [&](int j, int b0, size_t o0, int b1, size_t o1, bool ok1) {
        bfrag q;
        const size_t v0 = (size_t)b0 * Sin + iv0[j] + o0, v1 = (size_t)b1 * Sin + iv0[j] + o1;
        const v4i z4 = {0, 0, 0, 0};
        if constexpr (FMT == 8) {
            q.lo = *(const v4i *)(xq + v0 * RB + 16 * h);
            q.hi = *(const v4i *)(xq + v1 * RB + 16 * h);    // (ok1 false: v1 is v0's row again, its codes dropped)
            q.hi = ok1 ? q.hi : z4;
        } else {
            q.lo = *(const v4i *)(xq + (h ? v1 : v0) * RB);
            q.lo = (!h || ok1) ? q.lo : z4; q.hi = z4;
        }
        q.sb = h ? (ok1 ? (int)xsc[v1] : 127) : (int)xsc[v0];
        return q;
    };
    struct afrag { v4i lo, hi; int s; };
    auto wfetch = [&](int gp, int m) {
        afrag q;
        const size_t t = (size_t)gp * a.nmt_all + cs * MT + m;
        q.lo = *(const v4i *)(a.wq + t * WTILE + lane * 16);
        if constexpr (FMT == 8) q.hi = *(const v4i *)(a.wq + t * WTILE + 1024 + lane * 16); else q.hi = (v4i){0, 0, 0, 0};
        q.s = *(const int *)(a.wsc + (t * 64 + lane) * 4);
        return q;
    };
    v16f acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[m][j][i] = 0.f;
    // register rings: the weights of pair p + 1 (cache hits) and the rows of pairs p + 1 .. p + AR - 1 (HBM) are in flight while pair p is multiplied.
    // A wavefront has two MFMAs per channel tile and pair to hide a load's latency behind, so the launch runs at bytes in flight / latency: an
    // e2m1 row set is 10 registers, and four of them fit beside the accumulators
    constexpr int AR = FMT == 4 ? 4 : 2;
    bfrag fb[AR][NT]; afrag fa[2][MT];
    const int t_up = UP ? (int)(blockIdx.y / (unsigned)a.ncs) : 0, npt = (nb + 1) >> 1;      // up: one tap per workgroup (eight times the workgroups, the rows re-read through the L2)
    const int np = UP ? npt : 4 * nb;                        // down: 8 taps x nb blocks, in pairs, tap-major
    auto request_rows = [&](int p, auto SET) {
        constexpr int set = decltype(SET)::value;
        if constexpr (UP) {
            const bool ok1 = 2 * p + 1 < nb;
#pragma unroll
            for (int j = 0; j < NT; j++) fb[set][j] = fetch(j, 2 * p, 0, ok1 ? 2 * p + 1 : 2 * p, 0, ok1);
        } else {
            const int u0 = 2 * p, u1 = u0 + 1, t0 = u0 / nb, b0 = u0 - t0 * nb, t1 = u1 / nb, b1 = u1 - t1 * nb;
            const size_t o0 = ((size_t)(t0 >> 2) * a.H + ((t0 >> 1) & 1)) * a.W + (t0 & 1), o1 = ((size_t)(t1 >> 2) * a.H + ((t1 >> 1) & 1)) * a.W + (t1 & 1);
#pragma unroll
            for (int j = 0; j < NT; j++) fb[set][j] = fetch(j, b0, o0, b1, o1, true);
        }
    };
    auto request_weights = [&](int p, auto SET) {
        constexpr int set = decltype(SET)::value;
#pragma unroll
        for (int m = 0; m < MT; m++) fa[set][m] = wfetch(UP ? t_up * npt + p : p, m);
    };
    auto multiply = [&](auto BS, auto AS) {
        constexpr int bs = decltype(BS)::value, as = decltype(AS)::value;
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int j = 0; j < NT; j++) {
                const v8i A = {fa[as][m].lo[0], fa[as][m].lo[1], fa[as][m].lo[2], fa[as][m].lo[3], fa[as][m].hi[0], fa[as][m].hi[1], fa[as][m].hi[2], fa[as][m].hi[3]};
                const v8i B = {fb[bs][j].lo[0], fb[bs][j].lo[1], fb[bs][j].lo[2], fb[bs][j].lo[3], fb[bs][j].hi[0], fb[bs][j].hi[1], fb[bs][j].hi[2], fb[bs][j].hi[3]};
                acc[m][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A, B, acc[m][j], FMT == 8 ? 0 : 4, FMT == 8 ? 0 : 4, 0, fa[as][m].s, 0, fb[bs][j].sb);
            }
    };
    request_weights(0, std::integral_constant<int, 0>{});
    static_for<AR - 1>([&](auto I) { if (decltype(I)::value < np) request_rows(decltype(I)::value, I); });
    for (int p = 0; p < np; p += AR) {                       // (uniform branches)
        static_for<AR>([&](auto I) {
            constexpr int i = decltype(I)::value;
            if (p + i < np) {
                // (the weights first: loads return in order, so waiting for the next pair's weights also waits for everything requested before them)
                if (p + i + 1 < np) request_weights(p + i + 1, std::integral_constant<int, (i + 1) % 2>{});
                if (p + i + AR - 1 < np) request_rows(p + i + AR - 1, std::integral_constant<int, (i + AR - 1) % AR>{});
                multiply(I, std::integral_constant<int, i % 2>{});
            }
        });
    }
    long long ovx[NT];
#pragma unroll
    for (int j = 0; j < NT; j++) {
        if constexpr (UP) ovx[j] = cok[j] ? ((long long)(2 * c0[j] + (t_up >> 2)) * a.Ho + 2 * c1[j] + ((t_up >> 1) & 1)) * a.Wo + 2 * c2[j] + (t_up & 1) : -1;
        else ovx[j] = cok[j] ? (ct0 + j) * 32 + r : -1;
    }
    conv_epilogue<MT, NT, OUT, false, false, false, false, true, 4, true>(a, acc, lds, 0u, n, cs, 0, 0, 0, 0, 0, tid, ovx);
}

// ---- the 3x3x3 stride-2 conv (src/lp_s2.cu:4-9) read the same way: no LDS staging, every tap's rows straight from the stored tensor ----
// A staged halo serves a stride-2 tile badly (5 x 17 x 33 positions through registers and LDS for 2 x 8 x 16 outputs), and the rows a tap needs lie
// 64 bytes apart: the three kx taps of a wavefront's 64 consecutive output voxels together read one contiguous run of input rows, which the vector
// cache serves line by line. Column = output voxel, K in the pair order of mi_s2_unit (the weights are prepared in the same order); unit (t, b) of a column is the row of block b at voxel (2 oz + kz - 1, 2 oy + ky - 1, 2 ox + kx - 1), zeros outside the volume.
// The next pair's rows and weights are requested before the current pair is multiplied. Workgroups take the runs in launch order (dealing each XCD
// a contiguous range of runs measured slower: 32 -> 32 from 2 x 128^3 0.077 against 0.068 ms; the HBM side reads the input 1.9 times either way).
template <int FMT, int OUT, int MT>
__global__ void __launch_bounds__(256, MT <= 2 ? 4 : 2) conv3s2_mx_k(const conv_args a) {
    constexpr int NT = 2, RB = fmt_t<FMT>::RB, WTILE = fmt_t<FMT>::WTILE;
    extern __shared__ __align__(16) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;
    const int n = blockIdx.z, cs = (int)blockIdx.y, nb = a.nbt;
    const size_t Sin = (size_t)a.D * a.H * a.W;
    const long long Scol = (long long)a.Do * a.Ho * a.Wo;
    conv_epi_consts<MT, false>(a, lds, cs, tid);
    // the K order as a table (after the statistics scratch): per pair and side, tap | block << 5, bit 31 set for a padding unit
    const int np = (27 * nb + 1) >> 1;
    int *utab = (int *)(lds + a.red_o + 1024);
    for (int i = tid; i < 2 * np + 8; i += 256) {
        int t = 13, b = 0;
        const bool ok = (i >> 1) < np && mi_s2_unit(i >> 1, i & 1, nb, &t, &b);
        utab[i] = ok ? t | (b << 5) : (int)0x80000000u | 13;
    }
    __syncthreads();
    const long long ct0 = ((long long)blockIdx.x * 4 + wave) * NT;
    if (ct0 * 32 >= Scol) return;                            // (no barrier follows)
    // the lane's column of each tile: the input voxel of the centre tap and, per dimension, which of the offsets -1, 0, +1 stay inside the volume
    long long ivc[NT]; unsigned vm[NT]; bool cok[NT];
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const long long col = (ct0 + j) * 32 + r;
        cok[j] = col < Scol;
        const long long cc = cok[j] ? col : 0;
        const int ox = (int)(cc % a.Wo), oy = (int)(cc / a.Wo % a.Ho), oz = (int)(cc / ((long long)a.Wo * a.Ho));
        ivc[j] = ((long long)(2 * oz) * a.H + 2 * oy) * a.W + 2 * ox;
        unsigned m = 0;
#pragma unroll
        for (int d = 0; d < 3; d++) {
            m |= ((unsigned)(2 * oz + d - 1) < (unsigned)a.D ? 1u : 0u) << d;
            m |= ((unsigned)(2 * oy + d - 1) < (unsigned)a.H ? 1u : 0u) << (3 + d);
            m |= ((unsigned)(2 * ox + d - 1) < (unsigned)a.W ? 1u : 0u) << (6 + d);
        }
        vm[j] = cok[j] ? m : 0u;
    }
    const uint8_t *xq[2] = {a.xq[0], a.xq[1]}, *xsc[2] = {a.xsc[0], a.xsc[1]};
    struct bfrag { v4i lo, hi; int sb; };
    struct unit_t { const uint8_t *q, *sc; long long off; unsigned bit; };      // (uniform) rows and scale bytes of the unit's block, voxel offset from the centre tap, validity bits
    auto unit = [&](int p, int side) {
        unit_t q;
        const int e = __builtin_amdgcn_readfirstlane(utab[2 * p + side]);      // (p <= np + 3: the entries past the last pair are padding units)
        const bool ok = e >= 0;
        const int t = e & 31, b = (e & 0x7fffffff) >> 5;
        const int kz = t / 9, ky = (t / 3) % 3, kx = t % 3;
        const int seg = b >= a.nb0p, bl = seg ? b - a.nb0p : b;
        const size_t plane = ((size_t)n * (seg ? a.nbs[1] : a.nbs[0]) + bl) * Sin;
        q.q = (seg ? xq[1] : xq[0]) + plane * RB; q.sc = (seg ? xsc[1] : xsc[0]) + plane;
        q.off = ((long long)(kz - 1) * a.H + (ky - 1)) * a.W + (kx - 1);
        q.bit = ok ? (1u << kz) | (8u << ky) | (64u << kx) : 0x80000000u;      // (a padding unit, the pair past the end: never valid)
        return q;
    };
    auto fetch = [&](int j, const unit_t &u0, const unit_t &u1) {
        bfrag q;
        const bool v0 = (vm[j] & u0.bit) == u0.bit, v1 = (vm[j] & u1.bit) == u1.bit;
        const long long p0 = v0 ? ivc[j] + u0.off : 0, p1 = v1 ? ivc[j] + u1.off : 0;
        const v4i z4 = {0, 0, 0, 0};
        if constexpr (FMT == 8) {
            q.lo = *(const v4i *)(u0.q + p0 * RB + 16 * h); q.hi = *(const v4i *)(u1.q + p1 * RB + 16 * h);
            q.lo = v0 ? q.lo : z4; q.hi = v1 ? q.hi : z4;
        } else {
            q.lo = *(const v4i *)((h ? u1.q : u0.q) + (h ? p1 : p0) * RB);
            q.lo = (h ? v1 : v0) ? q.lo : z4; q.hi = z4;
        }
        q.sb = h ? (v1 ? (int)u1.sc[p1] : 127) : (v0 ? (int)u0.sc[p0] : 127);      // (a row outside the volume: zero codes, scale 1)
        return q;
    };
    struct afrag { v4i lo, hi; int s; };
    auto wfetch = [&](int gp, int m) {
        afrag q;
        const size_t t = (size_t)gp * a.nmt_all + cs * MT + m;
        q.lo = *(const v4i *)(a.wq + t * WTILE + lane * 16);
        if constexpr (FMT == 8) q.hi = *(const v4i *)(a.wq + t * WTILE + 1024 + lane * 16); else q.hi = (v4i){0, 0, 0, 0};
        q.s = *(const int *)(a.wsc + (t * 64 + lane) * 4);
        return q;
    };
    v16f acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[m][j][i] = 0.f;
    // a ring of RING register sets: the rows and weights of pairs p + 1 .. p + RING - 1 are in flight while pair p is multiplied (a wavefront has
    // little else to hide the loads' latency behind: two MFMAs per channel tile and pair)
    constexpr int RING = 2;                                  // (measured, 32 -> 32 from 2 x 128^3: two sets at four wavefronts per SIMD 0.071 ms, four sets at three 0.075 ms)
    bfrag fb[RING][NT]; afrag fa[RING][MT];
    auto request = [&](int p, auto SET) {
        constexpr int set = decltype(SET)::value;
        const unit_t u0 = unit(p, 0), u1 = unit(p, 1);
#pragma unroll
        for (int j = 0; j < NT; j++) fb[set][j] = fetch(j, u0, u1);
#pragma unroll
        for (int m = 0; m < MT; m++) fa[set][m] = wfetch(p, m);
    };
    auto multiply = [&](auto SET) {
        constexpr int set = decltype(SET)::value;
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int j = 0; j < NT; j++) {
                const v8i A = {fa[set][m].lo[0], fa[set][m].lo[1], fa[set][m].lo[2], fa[set][m].lo[3], fa[set][m].hi[0], fa[set][m].hi[1], fa[set][m].hi[2], fa[set][m].hi[3]};
                const v8i B = {fb[set][j].lo[0], fb[set][j].lo[1], fb[set][j].lo[2], fb[set][j].lo[3], fb[set][j].hi[0], fb[set][j].hi[1], fb[set][j].hi[2], fb[set][j].hi[3]};
                acc[m][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(A, B, acc[m][j], FMT == 8 ? 0 : 4, FMT == 8 ? 0 : 4, 0, fa[set][m].s, 0, fb[set][j].sb);
            }
    };
    static_for<RING - 1>([&](auto I) { request(decltype(I)::value, I); });
    for (int p = 0; p < np; p += RING) {                     // (pairs past the last one are padding units with zero weights; their products are never formed)
        static_for<RING>([&](auto I) {
            constexpr int i = decltype(I)::value;
            if (p + i < np) {                                // (uniform)
                request(p + i + RING - 1, std::integral_constant<int, (i + RING - 1) % RING>{});
                multiply(I);
            }
        });
    }
    long long ovx[NT];
#pragma unroll
    for (int j = 0; j < NT; j++) ovx[j] = cok[j] ? (ct0 + j) * 32 + r : -1;
    conv_epilogue<MT, NT, OUT, false, false, false, false, true, 4, true>(a, acc, lds, 0u, n, cs, 0, 0, 0, 0, 0, tid, ovx);
}

template <int FMT, int OUT, int MT>
static void launch_conv3s2_mt(const conv_args &a, dim3 grid, size_t smem) {
    conv3s2_mx_k<FMT, OUT, MT><<<grid, 256, smem>>>(a);
    MICK();
    snprintf(g_last_kernel, sizeof g_last_kernel, "conv3s2_mx_k<fmt %d, out %d, MT %d> blocks %d grid %u x %u x %u", FMT, OUT, MT, a.nbt, grid.x, grid.y, grid.z);
}
template <int FMT>
static void launch_conv3s2(int out, int MT, const conv_args &a, dim3 grid, size_t smem) {
#define C3S2_MT(OUT) do { if (MT == 4) launch_conv3s2_mt<FMT, OUT, 4>(a, grid, smem); else if (MT == 2) launch_conv3s2_mt<FMT, OUT, 2>(a, grid, smem); else launch_conv3s2_mt<FMT, OUT, 1>(a, grid, smem); } while (0)
    if (out == 8) C3S2_MT(8); else if (out == 4) C3S2_MT(4); else C3S2_MT(0);
#undef C3S2_MT
}
template <int FMT, int OUT, bool UP, int MT>
static void launch_conv2_mt(const conv_args &a, dim3 grid, size_t smem) {
    conv2_mx_k<FMT, OUT, UP, MT><<<grid, 256, smem>>>(a);
    MICK();
    snprintf(g_last_kernel, sizeof g_last_kernel, "conv2_mx_k<fmt %d, out %d, up %d, MT %d> blocks %d grid %u x %u x %u", FMT, OUT, (int)UP, MT, a.nbs[0], grid.x, grid.y, grid.z);
}
template <int FMT>
static void launch_conv2(int out, int up, int MT, const conv_args &a, dim3 grid, size_t smem) {
#define C2_MT(OUT, UP) do { if (MT == 4) launch_conv2_mt<FMT, OUT, UP, 4>(a, grid, smem); else if (MT == 2) launch_conv2_mt<FMT, OUT, UP, 2>(a, grid, smem); else launch_conv2_mt<FMT, OUT, UP, 1>(a, grid, smem); } while (0)
#define C2_UP(OUT) do { if (up) C2_MT(OUT, true); else C2_MT(OUT, false); } while (0)
    if (out == 8) C2_UP(8); else if (out == 4) C2_UP(4); else C2_UP(0);
#undef C2_UP
#undef C2_MT
}
void conv2_launch_f8(int out, int up, int MT, const conv_args &a, dim3 grid, size_t smem);
void conv2_launch_f4(int out, int up, int MT, const conv_args &a, dim3 grid, size_t smem);
