// 3x3x3 (stride 1 / 2, pad 1) implicit-GEMM convolution on MX operands for gfx950 (CDNA4), fp32 accumulate.
//
// Mapping (one workgroup = 4 wavefronts = one output tile of TZ x 8 x 16 voxels x up to 128 output channels):
//   * GEMM view: M = output channels (A operand = prepared weights), N = output voxels (B operand = staged input halo),
//     K = (tap, 32-channel input block) "units". One v_mfma_scale_f32_32x32x64_f8f6f4 consumes two units (K = 64): each
//     32-element K block carries its own E8M0 scale, supplied per lane: lanes 0-31 give the scale of K block 0 of their row,
//     lanes 32-63 that of K block 1. That is exactly the reference's "one scale per (voxel, 32 channels)" for the input and
//     "per (tap, co, 32 ci)" for the weights (src/lp_common.cuh:16-19).
//   * fp8 operand registers: lane (r, h) holds bytes [16h, 16h+16) of K block 0 in v0-3 and of K block 1 in v4-7;
//     fp4: lane (r, h) holds the 32 nibbles of K block h in v0-3.
//   * The input halo of the tile ((S(TZ-1)+3) x (7S+3) x (15S+3) positions, S = stride) for up to CB 32-channel blocks is
//     staged once into LDS as [block][16-byte half][position]; a wavefront's operand read for any tap is then one
//     ds_read_b128 per K block at a per-lane address (position of the lane's voxel + the tap's offset): no im2col.
//   * Each wavefront owns NT voxel tiles of 32 (2 rows x 16 x) and all MT channel tiles of 32 of the workgroup: MT x NT
//     accumulators of 32x32 (16 VGPRs each), every weight fragment reused NT times and every input fragment MT times.
//   * Weights are prepared once per call (or memoised) in fragment order, streamed L2 -> LDS through a 2-slot ring, one
//     barrier per K pair; two workgroups share a CU, so one's MFMAs cover the other's LDS latency, staging and epilogue.
//   * Epilogue (src/lp_common.cuh:1465-1597): bias -> optional affine + activation -> per (voxel, 32-channel block) amax across
//     the lane pair (l, l^32) -> E8M0 exponent -> e4m3 / e2m1 codes -> 16-byte row halves stored coalesced along x,
//     GroupNorm (sum, sum of squares) reduced in a fixed order and added to exact fixed-point slots.
#pragma once
#include "mx_dev.hpp"
#include <hip/hip_fp16.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <utility>
#include <vector>

// compile-time loops: accumulator tiles must be indexed with constants to stay in registers
template <int... Is, typename F> __device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, Is...>) { (f(std::integral_constant<int, Is>{}), ...); }
template <int N, typename F> __device__ __forceinline__ void static_for(F &&f) { static_for_impl(f, std::make_integer_sequence<int, N>{}); }

// ---- lane exchanges without LDS addressing: l ^ 32 by v_permlane32_swap (after swapping x with itself the first result holds the low half
// twice, the second the high half twice), l ^ 1 and l ^ 2 by DPP quad permutes, l ^ 4 / 8 / 16 by ds_swizzle's bit mode ----
__device__ __forceinline__ unsigned lane_xor32(unsigned x, int h) {
    const auto r2 = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return h ? r2[0] : r2[1];
}
__device__ __forceinline__ float lane_xor32f(float x, int h) { return __uint_as_float(lane_xor32(__float_as_uint(x), h)); }
// the maximum of a lane's value and its partner's (l ^ 32) for values that are not negative and not NaN (an amax): such floats order as their
// bit patterns; the swap leaves the low halves' values in one result and the high halves' in the other
__device__ __forceinline__ float lane_pair_max(float x) {
    const auto r2 = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r2[0] > r2[1] ? r2[0] : r2[1]);
}
// Output channel (within its tile of 32) of row r of a prepared weight tile. The 32x32 MFMA leaves row (i & 3) + 4 h + 8 (i >> 2) in register i
// of lane half h; the weights' rows are laid out so that this is channel 16 h + i: a lane holds 16 consecutive channels, i.e. its half of a
// stored 32-channel row, and nothing is exchanged between the halves
__host__ __device__ constexpr int mi_row_chan(int r) { return 16 * ((r >> 2) & 1) + (r & 3) + 4 * (r >> 3); }
template <int MASK> __device__ __forceinline__ float lane_xorf(float x) {
    static_assert(MASK == 1 || MASK == 2 || MASK == 4 || MASK == 8 || MASK == 16, "lane_xorf mask");
    const int xi = (int)__float_as_uint(x);
    int y;
    if constexpr (MASK == 1) y = __builtin_amdgcn_mov_dpp(xi, 0xB1, 0xF, 0xF, true);          // quad_perm [1, 0, 3, 2]
    else if constexpr (MASK == 2) y = __builtin_amdgcn_mov_dpp(xi, 0x4E, 0xF, 0xF, true);     // quad_perm [2, 3, 0, 1]
    else y = __builtin_amdgcn_ds_swizzle(xi, (MASK << 10) | 0x1f);                            // and 0x1f, or 0, xor MASK within 32 lanes
    return __uint_as_float((unsigned)y);
}
// Sums NV (a power of two <= 32) per-lane values over the 32 lanes of each wavefront half in a fixed order. Step k pairs lane r with
// r ^ 2^k; while more than one value is left the pair splits them (the lane whose bit k is clear keeps the lower half of the indices and
// receives the partner's lower half), so every step moves half as much as the one before. Returns the index of the value whose total
// the lane ends with in v[0]: sum over k of bit k of r times NV >> (k + 1); lanes with a set bit at or above log2(NV) hold duplicates.
template <int NV>
__device__ __forceinline__ int wave_half_reduce(float (&v)[NV], int r) {
    int idx = 0;
    static_for<5>([&](auto K) {
        constexpr int k = decltype(K)::value, nk = NV >> k;           // values left before this step (0: already one)
        const bool bit = (r >> k) & 1;
        if constexpr (nk >= 2) {
            constexpr int half = nk / 2;
#pragma unroll
            for (int i = 0; i < half; i++) {
                const float send = bit ? v[i] : v[i + half], keep = bit ? v[i + half] : v[i];
                v[i] = keep + lane_xorf<(1 << k)>(send);
            }
            idx += bit ? half : 0;
        } else v[0] += lane_xorf<(1 << k)>(v[0]);
    });
    return idx;
}

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

#ifdef DBG_TIMING
__device__ long long g_dbg[64];
#define DBG_MARK(i) do { if (blockIdx.x == 8 && threadIdx.x == 0) g_dbg[i] = (long long)__builtin_amdgcn_s_memtime(); } while (0)
#else
#define DBG_MARK(i) do { } while (0)
#endif

struct conv_args {
    const uint8_t *xq[2], *xsc[2];     // input segments (compute-format MX tensors): data, scale plane
    int nbs[2], bws[2];                // blocks per sample and block width of each segment's tensor
    int nb0p;                          // padded blocks of segment 0 (staged blocks [0, nb0p) come from segment 0)
    int nbt, CB;                       // staged 32-channel blocks in total, blocks per LDS chunk
    int wide;                          // every staged tensor has 32-channel blocks
    int N, D, H, W, Do, Ho, Wo;       // D x H x W: the staged input tensors; Do x Ho x Wo: the output planes this launch computes
    int zi0;                           // z-range: output plane z reads input plane z + zi0 (stride 1)
    int yD, yzo;                       // direct slab output: the MX output is planes [yzo, yzo + Do) of a depth-yD tensor (yD 0: a depth-Do tensor)
    const uint8_t *wq, *wsc; int nmt_all;
    unsigned wstride;                  // wide kernel: bytes between the weight images of two 128-channel slices
    const float *bias; int Co;
    void *y; int ydt;
    double *osum; float *part; int Go, stored_stats, zs0, zs1;   // part: per tile and channel quad (sum, sum of squares)
    int stat_ch;                       // 1: per-channel records, 32 per tile (channels per group not a multiple of 4; one channel tile per workgroup)
    const float *ep_a, *ep_b; int act;
    unsigned epi_o;                    // LDS byte offset of the epilogue's per-channel constants: bias, then ep_a, ep_b (MT x 32 floats each)
    unsigned red_o;                    // LDS byte offset of the statistics scratch (1 KiB)
    unsigned wl_o;                     // row kernel, weights resident in LDS: byte offset of their image (per pair 1 KiB of codes + 64 scale words; 0: loaded from global memory)
    const uint8_t *zpage;              // device memory: 64 zero bytes, then 64 bytes of value 1 (rows and scale bytes of positions outside the volume)
    int ntx, nty, ntz, ncs; unsigned ntiles;
    // tap-packed stem only: the input as stored (0 fp32 planes, 2 fp16 planes, 3 MX-fp8, 4 MX-fp4: one row of 8 channels per voxel) and its GroupNorm
    const void *sx; int sxdt, sCi;
    const float *sgam, *sbet, *smean, *srstd; int sG;
    int szs, szo, sns;            // slab-local statistics of the few-channel kernels' input (gnp_t zs / zo / ns; sns 0: per sample): plane z reads row n sns + clamp((z + szo) / szs)
    int zc; unsigned ngrp;             // consecutive z tiles a workgroup walks, workgroups with work
    bool big;                          // the wide kernel takes the launch (MT 4, or MT 2 with NT 4)
    bool areg;                         // the persistent small-channel kernel (one channel tile, one input block, weights in registers) takes the launch
    bool row;                          // the row kernel (one channel tile, any number of input blocks, 4 x 8 x 32 voxel tiles) takes the launch
    bool row1;                         // ... its one-input-block form (weights in registers, the two halves of the workgroup half a tile apart)
};

template <int FMT> struct fmt_t;
template <> struct fmt_t<8> { static constexpr int RB = 32, NH = 2, WTILE = 2048; };
template <> struct fmt_t<4> { static constexpr int RB = 16, NH = 1, WTILE = 1024; };

// GELU, x Phi(x) = 0.5 x (1 + erf(x / sqrt 2)), with erf by the rational-times-Gaussian form erf z = 1 - (a1 t + ... + a5 t^5) exp(-z^2),
// t = 1 / (1 + p z), z >= 0 (Abramowitz & Stegun 7.1.26, |error| < 1.5e-7): about 16 instructions with one reciprocal and one exponential where
// the library's erff takes about 60 (14 here); the epilogue that applies it runs alone on its SIMD, so every instruction is time. With
// q = 0.5 |x| (a1 t + ...) exp(-z^2) the result is max(x, 0) - q for either sign. NaN stays NaN; +-inf: z^2 overflows, the exponential is 0, q = inf 0
// would be NaN, so q takes the exponential's zero through a select
__device__ __forceinline__ float gelu_erf(float x) {
    // (z never formed: p z = |x| p / sqrt 2, -z^2 log2 e = -x^2 log2 e / 2, and the factor 0.5 sits in the coefficients)
    const float ax = fabsf(x);
    const float t = __builtin_amdgcn_rcpf(fmaf(ax, 0.23164189f, 1.f));
    const float poly = t * fmaf(t, fmaf(t, fmaf(t, fmaf(t, 0.5307027145f, -0.7265760135f), 0.7107068705f), -0.142248368f), 0.127414796f);
    const float ex = __builtin_amdgcn_exp2f(ax * ax * -0.72134752f);
    const float q = ex == 0.f ? 0.f : ax * poly * ex;
    return fmaxf(x, 0.f) - q;
}

// geometry of a workgroup's halo: output tile TZ x 8 x 16, input halo HZ x HY x HX positions
template <int FMT, int STRIDE, int TZ> struct halo_t {
    static constexpr int HZ = STRIDE * (TZ - 1) + 3, HY = STRIDE * 7 + 3, HX = STRIDE * 15 + 3, TT = HZ * HY * HX, NH = fmt_t<FMT>::NH;
};

// ---- pair table: per pair and lane half, the byte offsets of the pair's two units (fp8: both; fp4: the half's own) and of
// the half's scale word. unit u = (tap u / nbc, local block u % nbc); the odd padding unit (zero weights) re-reads unit A ----
template <int FMT, int STRIDE, int TZ>
__device__ __forceinline__ void conv_pair_table(unsigned char *lds, unsigned tab_o, int nbc, int tid) {
    using HL = halo_t<FMT, STRIDE, TZ>;
    constexpr int HY = HL::HY, HX = HL::HX, TT = HL::TT, NH = HL::NH;
    const int nunits = 27 * nbc, npairs = (nunits + 1) >> 1;
    for (int i = tid; i < (npairs + 2) * 2; i += 256) {
        const int q = min(i >> 1, npairs - 1), hh = i & 1;
        const int uA = 2 * q, uB = 2 * q + 1 < nunits ? 2 * q + 1 : 2 * q;
        const int tA = uA / nbc, bA = uA - tA * nbc, tB = uB / nbc, bB = uB - tB * nbc;
        const int pA = ((tA / 9) * HY + (tA / 3) % 3) * HX + tA % 3, pB = ((tB / 9) * HY + (tB / 3) % 3) * HX + tB % 3;
        const int dA = (bA * NH * TT + pA) * 16, dB = (bB * NH * TT + pB) * 16, sA = (bA * TT + pA) * 4, sB = (bB * TT + pB) * 4;
        *(v4i *)(lds + tab_o + i * 16) = (v4i){NH == 2 ? dA : (hh ? dB : dA), dB, hh ? sB : sA, 0};
    }
}

// ---- stage the halo of blocks [b0, b0 + nbc): rows copied as stored, zero rows (scale byte 1) outside the tensor.
// A thread owns up to NE (position, 16-byte half) elements and NS scale positions of the tile, the same for every block, so
// the index arithmetic is done once and each block costs one address add per element. Loads read a clamped in-tensor
// address and are zeroed afterwards when the position is outside: no divergent branches. The rows and scale bytes of GB blocks
// are requested before any of them is written to LDS: one memory round trip per GB blocks. WIDE: all staged tensors have 32-channel
// blocks (anything but a stored tensor of <= 16 channels read as it is); the narrow-row cases branch per element ----
template <int FMT, int STRIDE, int TZ, int GB, bool WIDE>
__device__ __forceinline__ void conv_stage_halo(const conv_args &a, unsigned char *lds, unsigned act_o, unsigned asc_o, int b0, int nbc, int n,
                                                int iz0, int iy0, int ix0, int tid) {
    using HL = halo_t<FMT, STRIDE, TZ>;
    constexpr int HY = HL::HY, HX = HL::HX, TT = HL::TT, NH = HL::NH;
    // Thread t owns the (position, 16-byte half) elements (t / NH + k PS, t % NH), k < NE, PS = 256 / NH positions apart, and (its half-0
    // lanes) the scale bytes of the same positions: one set of coordinates serves both. The coordinates of element k + 1 follow from
    // element k by adding PS = DZ HY HX + DY HX + DX with carries, so only the first needs divisions.
    constexpr int PS = 256 / NH, NE = (TT + PS - 1) / PS;
    constexpr int DZ = PS / (HY * HX), DY = (PS - DZ * HY * HX) / HX, DX = PS - DZ * HY * HX - DY * HX;
    const size_t Sin = (size_t)a.D * a.H * a.W;
    const int hf = NH == 2 ? tid & 1 : 0, p0 = tid / NH;
    unsigned evox[NE]; unsigned edst[NE]; bool eok[NE];
    {
        int px = p0 % HX, py = (p0 / HX) % HY, pz = p0 / (HX * HY);
#pragma unroll
        for (int k = 0; k < NE; k++) {
            const int gz = iz0 + pz, gy = iy0 + py, gx = ix0 + px;
            eok[k] = p0 + k * PS < TT && (unsigned)gz < (unsigned)a.D && (unsigned)gy < (unsigned)a.H && (unsigned)gx < (unsigned)a.W;
            const int cz = min(max(gz, 0), a.D - 1), cy = min(max(gy, 0), a.H - 1), cx = min(max(gx, 0), a.W - 1);      // (a clamped in-tensor address; zeroed after the load)
            evox[k] = (unsigned)((cz * a.H + cy) * a.W + cx);
            edst[k] = (unsigned)(hf * TT + min(p0 + k * PS, TT - 1)) * 16u;
            px += DX; py += DY; pz += DZ;
            if (px >= HX) { px -= HX; py++; }
            if (py >= HY) { py -= HY; pz++; }
        }
    }
    for (int bl0 = 0; bl0 < nbc; bl0 += GB) {
        v4i val[GB][NE]; bool ok[GB][NE]; unsigned sv[GB][NE]; bool bokg[GB];
#pragma unroll
        for (int g = 0; g < GB; g++) {
            const int bl = min(bl0 + g, nbc - 1);        // (a group's tail re-reads the last block and is not stored)
            const int sb = b0 + bl, seg = sb >= a.nb0p, blk = seg ? sb - a.nb0p : sb;
            const int rb = a.bws[seg] * FMT / 8;         // stored row bytes (16 NH for 32-wide blocks)
            const bool bok = blk < a.nbs[seg];
            bokg[g] = bok;
            const uint8_t *base = a.xq[seg] + ((size_t)n * a.nbs[seg] + min(blk, a.nbs[seg] - 1)) * Sin * rb;
#pragma unroll
            for (int k = 0; k < NE; k++) {
                const unsigned vox = evox[k];
                if (WIDE) {                              // every staged tensor has 32-channel blocks: straight-line loads, all in flight together
                    val[g][k] = *(const v4i *)(base + (size_t)vox * (16 * NH) + hf * 16);
                    ok[g][k] = eok[k] && bok;
                } else if (rb >= 16) {
                    const bool have = rb >= (int)(hf + 1) * 16;
                    val[g][k] = *(const v4i *)(base + (size_t)vox * rb + (have ? hf * 16 : 0));
                    ok[g][k] = eok[k] && bok && have;
                } else {                                 // 8- or 4-byte rows of a <= 8 / <= 16 channel tensor: only half 0 holds data
                    val[g][k] = (v4i){0, 0, 0, 0};
                    if (rb == 8) { const int2 t = *(const int2 *)(base + (size_t)vox * 8); val[g][k][0] = t.x; val[g][k][1] = t.y; }
                    else val[g][k][0] = *(const int *)(base + (size_t)vox * 4);
                    ok[g][k] = eok[k] && bok && hf == 0;
                }
            }
            const uint8_t *sbase = a.xsc[seg] + ((size_t)n * a.nbs[seg] + min(blk, a.nbs[seg] - 1)) * Sin;
            if (hf == 0) {
#pragma unroll
                for (int k = 0; k < NE; k++) sv[g][k] = sbase[evox[k]];
            }
        }
#pragma unroll
        for (int g = 0; g < GB; g++) {
            const int bl = bl0 + g;
            if (bl < nbc) {
#pragma unroll
                for (int k = 0; k < NE; k++)
                    if (p0 + k * PS < TT) *(v4i *)(lds + act_o + edst[k] + bl * NH * TT * 16) = ok[g][k] ? val[g][k] : (v4i){0, 0, 0, 0};
                if (hf == 0) {
#pragma unroll
                    for (int k = 0; k < NE; k++)
                        if (p0 + k * PS < TT) *(unsigned *)(lds + asc_o + (bl * TT + p0 + k * PS) * 4) = eok[k] && bokg[g] ? sv[g][k] : 1u;
                }
            }
        }
    }
}

// the epilogue's per-channel constants of the workgroup's MT x 32 channels -> LDS (padding channels: bias 0, affine 1, 0); read after a barrier
template <int MT, bool EPI>
__device__ __forceinline__ void conv_epi_consts(const conv_args &a, unsigned char *lds, int cs, int tid) {
    if (tid < MT * 32) {
        const int co = cs * MT * 32 + tid;
        float *p = (float *)(lds + a.epi_o);
        p[tid] = a.bias && co < a.Co ? a.bias[co] : 0.f;
        if (EPI) { p[MT * 32 + tid] = a.ep_a && co < a.Co ? a.ep_a[co] : 1.f; p[MT * 64 + tid] = a.ep_a && co < a.Co ? a.ep_b[co] : 0.f; }
    }
}

// ---- epilogue (src/lp_common.cuh:1465-1597): bias -> optional affine + activation -> per (voxel, 32-channel block) amax across the
// lane pair (l, l ^ 32) -> E8M0 exponent -> codes -> row stores; GroupNorm partial sums per tile. acc: the wavefront's MT x NT accumulators;
// register i of lane (r, h) is channel 16 h + i of the tile (mi_row_chan: the prepared weights' row order); lane (r, h) of tile j holds voxel (oz0 + lz, oy0 + ly0 + 2 j + (r >> 4), ox0 + (r & 15)) ----
// FULL: the tile lies inside the output and the statistics cover all of its planes (uniform, checked by the caller): no per-lane predicates,
// so the whole epilogue is straight-line code the scheduler can interleave across the accumulator tiles
// NOCH: this call takes no per-channel statistics records (the caller has checked stat_ch, or never sets it): their 32 sums are not kept
// NW: wavefronts of the workgroup (their partial statistics are summed in wave order); ROW: the row kernel's voxel mapping, lane r of tile j
// holds voxel (oz0 + lz, oy0 + ly0 + j, ox0 + r) of a 32-voxel run along x
// WPART: every wavefront writes its own statistics record (record tile NW + wave: the reduce kernel then sees NW records per tile) and the
// epilogue has no workgroup barrier and touches no LDS scratch, so the wavefronts of a workgroup need not run it at the same time (one channel tile)
template <int MT, int NT, int OUT, bool EPI, bool PIN = false, bool W32 = false, bool FULL = false, bool NOCH = false, int NW = 4, bool ROW = false, bool WPART = false>
__device__ __forceinline__ void conv_epilogue(const conv_args &a, v16f (&acc)[MT][NT], unsigned char *lds, unsigned tile, int n, int cs,
                                              int oz0, int oy0, int ox0, int lz, int ly0, int tid, const long long *ovx = nullptr) {
    const int lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;
    // accumulator layout of the 32x32 MFMA: lane (r = voxel within the tile, h), register i -> row (i & 3) + 4 h + 8 (i >> 2) = channel 16 h + i
    const size_t So = (size_t)(a.yD ? a.yD : a.Do) * a.Ho * a.Wo;      // voxels per channel plane of the output tensor
    const int co_base = cs * MT * 32;
    float *red = (float *)(lds + a.red_o);          // stats scratch [4 waves][MT][8 quads][2] floats
    const bool stats = a.osum != nullptr;
    float qs[MT][4], qss[MT][4];                    // per lane: sums over its voxels of the 4-channel quads (m, i >> 2)
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) { qs[m][q4] = 0.f; qss[m][q4] = 0.f; }
    constexpr bool CH = MT == 1 && !NOCH;
    static_assert(!CH || NW == 4, "per-channel statistics records: four wavefronts");
    float chs[CH ? 16 : 1], chss[CH ? 16 : 1];               // per-channel sums (MT 1, stat_ch)
#pragma unroll
    for (int i = 0; i < (CH ? 16 : 1); i++) { chs[i] = 0.f; chss[i] = 0.f; }
    constexpr int YB = OUT == 4 ? 4 : 8;
    const int bwo = W32 ? 32 : mx_bw(a.Co), nbo = W32 ? (a.Co + 31) >> 5 : mx_nb(a.Co), rbo = mx_rb(bwo, YB);     // W32: more than 16 output channels, known at compile time
    uint8_t *yq = (uint8_t *)a.y, *ysc = yq + (size_t)a.N * nbo * So * rbo;
    // the lane's output voxel: tile j lies JS rows of the volume below tile 0, so one offset per lane and epilogue and a uniform step per tile;
    // the row index of (tile m, tile j) = rowb + m * mstep + j * jstep (bwo < 32 only when Co <= 16: one channel tile, block 0)
    constexpr int JS = ROW ? 1 : 2;
    const int oz = oz0 + lz, oyb = ROW ? oy0 + ly0 : oy0 + ly0 + (r >> 4), ox = ROW ? ox0 + r : ox0 + (r & 15);
    const size_t ovb = ovx ? 0 : ((size_t)(oz + a.yzo) * a.Ho + oyb) * a.Wo + ox;
    const size_t rowb = ((size_t)n * nbo + co_base / bwo) * So + ovb, mstep = bwo == 32 ? So : 0, jstep = ovx ? 0 : (size_t)JS * a.Wo;
    static_for<MT>([&](auto M) {
        constexpr int m = M;
        DBG_MARK(16 + m);
        // the lane's 16 channels of tile m: 16 h + i
        float bias[16], ea[16], eb[16];
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const unsigned o = a.epi_o + (m * 32 + 16 * h + 4 * q4) * 4;
            const float4 b4 = *(const float4 *)(lds + o);
            bias[4 * q4] = b4.x; bias[4 * q4 + 1] = b4.y; bias[4 * q4 + 2] = b4.z; bias[4 * q4 + 3] = b4.w;
            if (EPI) {
                const float4 a4 = *(const float4 *)(lds + o + MT * 128), e4 = *(const float4 *)(lds + o + MT * 256);
                ea[4 * q4] = a4.x; ea[4 * q4 + 1] = a4.y; ea[4 * q4 + 2] = a4.z; ea[4 * q4 + 3] = a4.w;
                eb[4 * q4] = e4.x; eb[4 * q4 + 1] = e4.y; eb[4 * q4 + 2] = e4.z; eb[4 * q4 + 3] = e4.w;
            }
        }
        static_for<NT>([&](auto J) {
            constexpr int j = J;
            const int oy = oyb + JS * j;
            // ovx: the caller's own voxel mapping (the 2x2x2 stride-2 kernels): the lane's output voxel of tile j, negative = none
            const bool ok = ovx ? ovx[j] >= 0 : (FULL || (oz < a.Do && oy < a.Ho && ox < a.Wo));
            const size_t ov = ovx ? (size_t)ovx[j] : ovb + j * jstep;
            const bool zst = ovx ? ok : (FULL || (ok && oz >= a.zs0 && oz < a.zs1));
            float v[16];
            float am = 0.f;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float av = acc[m][j][i];
                if (PIN) asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(av) : "a"(acc[m][j][i]));   // the accumulators stay in AGPRs until their tile's turn
                float t = av + bias[i];                       // (padding channels: zero weights and no bias, so they stay 0)
                if (EPI) {
                    t = fmaf(t, ea[i], eb[i]);
                    t = a.act == 1 ? d_silu(t) : a.act == 2 ? gelu_erf(t) : a.act == 3 ? fmaxf(t, 0.f) : t;
                    if (co_base + m * 32 + 16 * h + i >= a.Co) t = 0.f;
                }
                v[i] = t; am = fmaxf(am, fabsf(t));
            }
            if (OUT != 0) {
                am = lane_pair_max(am);
                const int e = d_mx_exp(am, YB == 8 ? MI_INVQ8 : MI_INVQ4);
                const size_t row = rowb + m * mstep + (ovx ? (size_t)ovx[j] : j * jstep);
                if (OUT == 8) {
                    unsigned d[4];
                    const float p2e = d_exp2i(e);
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++) d[q4] = d_enc_e4m3x4_hw(v[4 * q4], v[4 * q4 + 1], v[4 * q4 + 2], v[4 * q4 + 3], p2e);
                    if (__builtin_amdgcn_ballot_w64(e == 128) != 0ull) {      // a block with an infinity or NaN: closed-form codes (never taken by finite data)
                        if (e == 128) {
#pragma unroll
                            for (int q4 = 0; q4 < 4; q4++) d[q4] = d_enc4_e4m3_nf(v[4 * q4], v[4 * q4 + 1], v[4 * q4 + 2], v[4 * q4 + 3]);
                        }
                    }
                    if (a.stored_stats) {                // the statistics are those of the stored values: decode the codes at the block's scale
                        const float sc = d_exp2i(e);
#pragma unroll
                        for (int q4 = 0; q4 < 4; q4++) {
                            const mi_v2f lo = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(d[q4], sc, false), hi = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(d[q4], sc, true);
                            v[4 * q4] = lo[0]; v[4 * q4 + 1] = lo[1]; v[4 * q4 + 2] = hi[0]; v[4 * q4 + 3] = hi[1];
                        }
                    }
                    const uint4 out = make_uint4(d[0], d[1], d[2], d[3]);      // bytes 16 h .. 16 h + 15 of the row
                    if (ok) {
                        if (bwo == 32) *(uint4 *)(yq + row * 32 + 16 * h) = out;
                        else if (bwo == 16) { if (!h) *(uint4 *)(yq + row * 16) = out; }
                        else if (!h) *(uint2 *)(yq + row * 8) = make_uint2(out.x, out.y);
                    }
                } else {
                    const float p2e = d_exp2i(e);
                    unsigned w01 = d_enc_e2m1x8_hw(v, p2e), w23 = d_enc_e2m1x8_hw(v + 8, p2e);
                    if (__builtin_amdgcn_ballot_w64(e == 128) != 0ull) {
                        if (e == 128) { w01 = d_enc8_e2m1_nf(v); w23 = d_enc8_e2m1_nf(v + 8); }
                    }
                    if (a.stored_stats) {
                        const float sc = d_exp2i(e);
                        d_dec8_e2m1(w01, v); d_dec8_e2m1(w23, v + 8);
#pragma unroll
                        for (int i = 0; i < 16; i++) v[i] *= sc;
                    }
                    const uint2 out = make_uint2(w01, w23);           // bytes 8 h .. 8 h + 7 of the row
                    if (ok) {
                        if (bwo == 32) *(uint2 *)(yq + row * 16 + 8 * h) = out;
                        else if (bwo == 16) { if (!h) *(uint2 *)(yq + row * 8) = out; }
                        else if (!h) *(unsigned *)(yq + row * 4) = out.x;
                    }
                }
                if (ok && !h) ysc[row] = (uint8_t)(e + 127);
            } else {
                const size_t o0 = ((size_t)n * a.Co + co_base + m * 32 + 16 * h) * So + ov;
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int cl = i;                                 // channel offset from co_base + 32 m + 16 h
                    const bool cok = ok && co_base + m * 32 + 16 * h + cl < a.Co;
                    if (a.ydt == 2) {
                        if (a.Go > 0) v[i] = fabsf(v[i]) > 65504.f ? copysignf(65504.f, v[i]) : v[i];     // src/lp_common.cuh:465, :1567-1569
                        if (cok) ((__half *)a.y)[o0 + (size_t)cl * So] = __float2half(v[i]);
                    } else if (cok) ((float *)a.y)[o0 + (size_t)cl * So] = v[i];
                }
            }
            if (stats && zst) {
                if (CH && a.stat_ch) {
#pragma unroll
                    for (int i = 0; i < (CH ? 16 : 1); i++) { chs[i] += v[i]; chss[i] += v[i] * v[i]; }
                } else {
#pragma unroll
                    for (int i = 0; i < 16; i++) { qs[m][i >> 2] += v[i]; qss[m][i >> 2] += v[i] * v[i]; }
                }
            }
            if (!PIN) __builtin_amdgcn_sched_barrier(0);     // one accumulator tile at a time: hoisting the next tiles' reads only costs registers
        });
    });
    DBG_MARK(20);
    if constexpr (WPART) {
        static_assert(!WPART || (MT == 1 && NOCH), "per-wavefront statistics records: one channel tile, no per-channel records");
        if (stats) {
            float v[8];
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) { v[q4 * 2] = qs[0][q4]; v[q4 * 2 + 1] = qss[0][q4]; }
            const int idx = wave_half_reduce<8>(v, r);
            // (record (tile NW + wave) of slice cs: with channel slices the records of a (tile, wavefront) lie slice by slice, as a tile's do)
            if ((r >> 3) == 0) a.part[((((size_t)tile * NW + wave) * a.ncs + cs) * 8 + 4 * h + (idx >> 1)) * 2 + (idx & 1)] = v[0];
        }
        return;
    }
    if (stats) __syncthreads();
    DBG_MARK(21);
    if (CH && stats && a.stat_ch) {
        // any group size (one channel tile): per-channel sums over the 32 voxel lanes, then over the waves; channel of register i of
        // half h = 16 h + i; value index 2 i + t (t 0 sum, 1 sum of squares)
        float v[32];
#pragma unroll
        for (int i = 0; i < (CH ? 16 : 1); i++) { v[2 * i] = chs[i]; v[2 * i + 1] = chss[i]; }
        const int idx = wave_half_reduce<32>(v, r), i = idx >> 1;
        red[(wave * 32 + 16 * h + i) * 2 + (idx & 1)] = v[0];
        __syncthreads();
        if (tid < 32) {
            float s1 = 0.f, s2 = 0.f;
            for (int w = 0; w < NW; w++) { s1 += red[(w * 32 + tid) * 2]; s2 += red[(w * 32 + tid) * 2 + 1]; }
            a.part[((size_t)tile * 32 + tid) * 2] = s1; a.part[((size_t)tile * 32 + tid) * 2 + 1] = s2;
        }
    } else if (stats) {
        // channels per group a multiple of 4: a quad (m, q4, h) = channels co_base + 32 m + 16 h + 4 q4 .. +3 lies in one group.
        // Sum over the 32 voxel lanes of each half (fixed order), then over the 4 waves in wave order; value index (4 m + q4) 2 + t
        constexpr int NV = MT <= 1 ? 8 : MT <= 2 ? 16 : 32;
        float v[NV];
#pragma unroll
        for (int i = 0; i < NV; i++) v[i] = 0.f;
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) { v[(4 * m + q4) * 2] = qs[m][q4]; v[(4 * m + q4) * 2 + 1] = qss[m][q4]; }
        const int idx = wave_half_reduce<NV>(v, r);
        if ((r >> (NV == 8 ? 3 : NV == 16 ? 4 : 5)) == 0 && idx < MT * 8) {
            const int mq = idx >> 1;                                    // 4 m + q4
            red[((wave * MT + (mq >> 2)) * 8 + 4 * h + (mq & 3)) * 2 + (idx & 1)] = v[0];
        }
        __syncthreads();
        if (tid < MT * 8) {
            // per tile and channel quad, the sums over the tile's voxels in wave order; a second kernel adds the tiles of a sample
            // in a fixed order into the exact sum slots, so the statistics do not depend on the order workgroups finish in
            const int m = tid >> 3, q8 = tid & 7;                       // q8 = 4 h + q4: channels co_base + 32 m + 4 q8 .. + 3
            float s = 0.f, ss = 0.f;
            for (int w = 0; w < NW; w++) { s += red[((w * MT + m) * 8 + q8) * 2]; ss += red[((w * MT + m) * 8 + q8) * 2 + 1]; }
            a.part[((size_t)tile * MT * 8 + tid) * 2] = s;
            a.part[((size_t)tile * MT * 8 + tid) * 2 + 1] = ss;
        }
    }
    DBG_MARK(22);
}

// one unit (32 input channels of one tap and output channel) of a prepared weight tile: E8M0 scale from the amax, codes, the lane order the MFMA
// reads (e4m3: lane (r, h) holds bytes 16 h .. of both units of the pair; e2m1: lane (r, side) holds unit side), scale word per lane
// tile2d: one scale for the 32 x 32 (output x input channel) tile, the maximum over the 32 lanes that hold the tile's rows (2-D weight scales)
template <int FMT>
__device__ __forceinline__ void prep_store_unit(uint8_t *tile, unsigned *tsc, int tss, int side, int r, const float *v, bool tile2d = false) {
    float amax = 0.f;
#pragma unroll
    for (int k = 0; k < 32; k++) amax = fmaxf(amax, fabsf(v[k]));
    if (tile2d) {
#pragma unroll
        for (int o = 16; o; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    }
    const int e = d_mx_exp(amax, FMT == 8 ? MI_INVQ8 : MI_INVQ4);
    const float mult = d_exp2i(-e);
    if (FMT == 8) {
        unsigned c[8];
#pragma unroll
        for (int j = 0; j < 8; j++) c[j] = d_enc_e4m3x4(v[4 * j] * mult, v[4 * j + 1] * mult, v[4 * j + 2] * mult, v[4 * j + 3] * mult);
        *(uint4 *)(tile + ((size_t)(side * 64 + r) * 16)) = make_uint4(c[0], c[1], c[2], c[3]);            // lane (r, 0): bytes 0-15
        *(uint4 *)(tile + ((size_t)(side * 64 + r + 32) * 16)) = make_uint4(c[4], c[5], c[6], c[7]);       // lane (r, 1): bytes 16-31
    } else {
        unsigned c[4];
#pragma unroll
        for (int j = 0; j < 4; j++) c[j] = d_enc_e2m1x8(v + 8 * j, mult);
        *(uint4 *)(tile + ((size_t)(r + 32 * side) * 16)) = make_uint4(c[0], c[1], c[2], c[3]);            // lane (r, side): the unit's 32 nibbles
    }
    tsc[(r + 32 * side) * tss] = (unsigned)(e + 127);
}

// FMT: compute format (8 e4m3, 4 e2m1); OUT: 8 / 4 = MX-fp8 / MX-fp4 rows, 0 = fp32 or fp16 planes; EPI: fused affine + activation
template <int FMT, int STRIDE, int MT, int NT, int OUT, bool EPI>
__global__ void __launch_bounds__(256, 2) conv3_mx_k(const conv_args a) {
    constexpr int TZ = NT == 1 ? 1 : NT == 2 ? 2 : 4;       // output planes of a workgroup's tile (x 8 x 16)
    constexpr int HZ = STRIDE * (TZ - 1) + 3, HY = STRIDE * 7 + 3, HX = STRIDE * 15 + 3, TT = HZ * HY * HX;
    constexpr int NH = fmt_t<FMT>::NH, WTILE = fmt_t<FMT>::WTILE;
    constexpr int STG = MT * (WTILE + 256);              // the weights of one pair: MT tiles of codes, then MT x 64 scale words
    constexpr int PPS = MT == 1 ? 7 : MT == 2 ? 2 : 1;   // pairs per ring stage
    extern __shared__ __align__(16) unsigned char lds[];
    // LDS: [2 weight stages][pair table (npairs + 2) x 2 x 16 B][halo rows CB * NH * TT * 16 B][halo scales CB * TT words]
    const int tab_bytes = (((27 * a.CB + 1) >> 1) + 2) * 32;
    const unsigned wring_o = 0, tab_o = 2 * PPS * STG, act_o = tab_o + tab_bytes, asc_o = act_o + a.CB * NH * TT * 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;

    // XCD-aware tile order: consecutive workgroup ids land on different XCDs (8, round robin), so give each XCD a contiguous
    // range of tiles: neighbouring tiles (shared halo, same weights) then share one L2
    unsigned tile;
    {
        const unsigned per = (a.ntiles + 7u) / 8u;
        tile = (blockIdx.x & 7u) * per + (blockIdx.x >> 3);
        if (tile >= a.ntiles) return;
    }
    int tt = (int)tile;
    const int cs = tt % a.ncs; tt /= a.ncs;
    const int tx = tt % a.ntx; tt /= a.ntx;
    const int ty = tt % a.nty; tt /= a.nty;
    const int tz = tt % a.ntz; const int n = tt / a.ntz;
    const int ox0 = tx * 16, oy0 = ty * 8, oz0 = tz * TZ;
    const int ix0 = STRIDE * ox0 - 1, iy0 = STRIDE * oy0 - 1, iz0 = STRIDE * oz0 - 1 + a.zi0;

    // the lane's voxel in each of its NT tiles: wave -> y row pair for TZ 1, (z, y half) for TZ 2, z for TZ 4; tile j -> rows 2j, 2j+1; r -> (row, x)
    int lz, ly0;
    if (NT == 1) { lz = 0; ly0 = wave * 2; } else if (NT == 2) { lz = wave >> 1; ly0 = (wave & 1) * 4; } else { lz = wave; ly0 = 0; }
    // LDS byte addresses of the lane's halo row (its 16-byte half) and scale word for tap (0, 0, 0) of block 0, first voxel tile; tile j
    // lies 2 STRIDE halo rows further: a constant the loads carry in their offset field
    const int p00 = ((STRIDE * lz) * HY + STRIDE * (ly0 + (r >> 4))) * HX + STRIDE * (r & 15);
    const unsigned ab0 = act_o + ((NH == 2 ? h * TT : 0) + p00) * 16, sb0 = asc_o + p00 * 4;
    constexpr unsigned ABJ = 2 * STRIDE * HX * 16, SBJ = 2 * STRIDE * HX * 4;
    const unsigned wfa = wring_o + lane * 16, wfs = wring_o + MT * WTILE + lane * 4;    // the lane's weight fragment / scale word of the ring's first pair, tile 0

    v16f acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[m][j][i] = 0.f;

    const size_t wq_ps = (size_t)a.nmt_all * WTILE, wsc_ps = (size_t)a.nmt_all * 256;
    int pair0 = 0;                                       // global pair index of the chunk's first pair
    conv_epi_consts<MT, EPI>(a, lds, cs, tid);

    for (int b0 = 0; b0 < a.nbt; b0 += a.CB) {
        const int nbc = min(a.CB, a.nbt - b0), nunits = 27 * nbc, npairs = (nunits + 1) >> 1;
        __syncthreads();                                 // the previous chunk's readers are done with the halo
        DBG_MARK(0);
        conv_pair_table<FMT, STRIDE, TZ>(lds, tab_o, nbc, tid);
        DBG_MARK(1);
        if (a.wide) conv_stage_halo<FMT, STRIDE, TZ, 1, true>(a, lds, act_o, asc_o, b0, nbc, n, iz0, iy0, ix0, tid);
        else conv_stage_halo<FMT, STRIDE, TZ, 1, false>(a, lds, act_o, asc_o, b0, nbc, n, iz0, iy0, ix0, tid);
        // ---- weight stages: global -> registers -> ring slot, PPS pairs per stage (more pairs per stage for few channel tiles: with one
        // tile a pair is only NT MFMAs per wavefront, too little work between two barriers). A thread moves up to UPS 16-byte units per
        // stage; the prepared-weight buffers carry padding pairs, so the loads that run ahead of the last stage stay inside them ----
        constexpr int U16 = STG / 16, C16 = MT * WTILE / 16;     // 16-byte units of a pair: codes, then scale words
        constexpr int UPS = (PPS * U16 + 255) / 256;
        v4i g[UPS];
        int wstage = 0;                                      // the next stage to load
        auto wload = [&]() {
#pragma unroll
            for (int k = 0; k < UPS; k++) {
                const int u = min(tid + k * 256, PPS * U16 - 1), p = u / U16, w16 = u - p * U16;
                const size_t gp = (size_t)(pair0 + wstage * PPS + p);
                const uint8_t *src = w16 < C16 ? a.wq + gp * wq_ps + (size_t)cs * MT * WTILE + w16 * 16 : a.wsc + gp * wsc_ps + (size_t)cs * MT * 256 + (w16 - C16) * 16;
                g[k] = *(const v4i *)src;
            }
            wstage++;
        };
        auto wstore = [&](int slot) {
#pragma unroll
            for (int k = 0; k < UPS; k++) {
                const int u = tid + k * 256;
                if (u < PPS * U16) *(v4i *)(lds + wring_o + slot * PPS * STG + u * 16) = g[k];
            }
        };
        DBG_MARK(2);
        wload(); wstore(0);
        __syncthreads();
        DBG_MARK(3);

        // ---- K loop over stages of PPS unit pairs. Stage st: start loading stage st + 1 from L2; for each of its pairs fetch the fragments
        // from LDS (halo rows at the table's offsets, weights from ring slot st & 1) and run the MFMAs; move stage st + 1 into the other
        // slot; one barrier. A second workgroup on the CU covers this one's LDS latency and barriers ----
        v8i fb[NT], fa[MT]; int sb[NT], sa[MT];
        v4i T;
        unsigned tabp = tab_o + (lane >> 5) * 16;          // this half's entry of pair 0
        auto fetch = [&](unsigned wo) {
            const v4i t = T;
#pragma unroll
            for (int j = 0; j < NT; j++) {
                const v4i lo = *(const v4i *)(lds + (ab0 + t[0]) + j * ABJ);
                if (FMT == 8) {
                    const v4i hi = *(const v4i *)(lds + (ab0 + t[1]) + j * ABJ);
                    fb[j] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                } else fb[j] = (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
                sb[j] = *(const int *)(lds + (sb0 + t[2]) + j * SBJ);
            }
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const v4i lo = *(const v4i *)(lds + wfa + wo + m * WTILE);
                if (FMT == 8) {
                    const v4i hi = *(const v4i *)(lds + wfa + wo + m * WTILE + 1024);
                    fa[m] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                } else fa[m] = (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
                sa[m] = *(const int *)(lds + wfs + wo + m * 256);
            }
            T = *(const v4i *)(lds + tabp + 32); tabp += 32;      // the next pair's table entry
        };
        auto mma = [&]() {
#pragma unroll
            for (int m = 0; m < MT; m++)
#pragma unroll
                for (int j = 0; j < NT; j++)
                    acc[m][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[m], fb[j], acc[m][j], FMT == 8 ? 0 : 4, FMT == 8 ? 0 : 4, 0, sa[m], 0, sb[j]);
        };
        T = *(const v4i *)(lds + tabp);
        const int nstg = (npairs + PPS - 1) / PPS;
        for (int st = 0; st < nstg; st++) {
            const unsigned so = (unsigned)(st & 1) * (PPS * STG);
            wload();
#pragma unroll
            for (int p = 0; p < PPS; p++)
                if (st * PPS + p < npairs) { fetch(so + p * STG); mma(); }
            wstore((st & 1) ^ 1);
            __syncthreads();
        }
        DBG_MARK(4);
        pair0 += npairs;
    }

    __syncthreads();                                     // the ring and halo are dead: the epilogue reuses LDS for its statistics scratch
    // (uniform) more than 16 output channels, always so with two or more channel tiles: 32-wide output rows known at compile time
    if (MT > 1 || a.Co > 16) conv_epilogue<MT, NT, OUT, EPI, false, true>(a, acc, lds, tile, n, cs, oz0, oy0, ox0, lz, ly0, tid);
    else conv_epilogue<MT, NT, OUT, EPI>(a, acc, lds, tile, n, cs, oz0, oy0, ox0, lz, ly0, tid);
}

extern thread_local char g_last_kernel[128];
template <int FMT, int STRIDE, int MT, int NT, int OUT, bool EPI>
static void launch_conv(const conv_args &a, size_t smem) {
    static bool attr[8];
    int d = 0; MIRT(hipGetDevice(&d)); d &= 7;
    if (!attr[d]) { MIRT(hipFuncSetAttribute((const void *)conv3_mx_k<FMT, STRIDE, MT, NT, OUT, EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)); attr[d] = true; }
    const unsigned per = (a.ntiles + 7u) / 8u;
    conv3_mx_k<FMT, STRIDE, MT, NT, OUT, EPI><<<per * 8u, 256, smem>>>(a);
    MICK();
    snprintf(g_last_kernel, sizeof g_last_kernel, "conv3_mx_k<fmt %d, stride %d, MT %d, NT %d, out %d, epi %d> CB %d tiles %u", FMT, STRIDE, MT, NT, OUT, (int)EPI, a.CB, a.ntiles);
}
#include "conv3_wide.hpp"
#include "conv3_small.hpp"
#include "conv3_row.hpp"
#include "conv3_row1.hpp"
template <int FMT, int STRIDE, int OUT, bool EPI>
static void launch_mt(int MT, int NT, const conv_args &a, size_t smem) {
    switch (MT * 10 + NT) {
    case 44: if constexpr (STRIDE == 1) launch_wide<FMT, OUT, EPI>(a, smem); else mi_die("conv3: the wide kernel is stride 1 only"); break;
    // (one-plane tiles, stride 2 only: its halo is 8 input positions per output, and a 3 x 17 x 33 halo lets two workgroups share a CU)
    case 11: if constexpr (STRIDE == 2) { launch_conv<FMT, 2, 1, 1, OUT, EPI>(a, smem); break; }
    case 21: if constexpr (STRIDE == 2) { launch_conv<FMT, 2, 2, 1, OUT, EPI>(a, smem); break; }
    case 41: if constexpr (STRIDE == 2) { launch_conv<FMT, 2, 4, 1, OUT, EPI>(a, smem); break; }
    case 12: if constexpr (STRIDE == 1) { if (a.areg) { launch_small<FMT, 2, OUT, EPI>(a, smem); break; } }
             launch_conv<FMT, STRIDE, 1, 2, OUT, EPI>(a, smem); break;
    case 22: launch_conv<FMT, STRIDE, 2, 2, OUT, EPI>(a, smem); break;
    case 32: launch_conv<FMT, STRIDE, 3, 2, OUT, EPI>(a, smem); break;
    case 42: launch_conv<FMT, STRIDE, 4, 2, OUT, EPI>(a, smem); break;
    case 14: if constexpr (STRIDE == 1) { if (a.row1) launch_row1<FMT, OUT, EPI>(a, smem); else if (a.row) { if constexpr (FMT == 4) { if (a.wl_o) { launch_row<FMT, OUT, EPI, true>(a, smem); break; } } launch_row<FMT, OUT, EPI, false>(a, smem); } else if (a.areg) launch_small<FMT, 4, OUT, EPI>(a, smem); else launch_conv<FMT, 1, 1, 4, OUT, EPI>(a, smem); break; }
    case 24: if constexpr (STRIDE == 1) { if (a.big) launch_wide<FMT, OUT, EPI, 2>(a, smem); else launch_conv<FMT, 1, 2, 4, OUT, EPI>(a, smem); break; }
    default: mi_die("conv3: no kernel for MT %d NT %d stride %d", MT, NT, STRIDE);
    }
}
// the fused-activation epilogue is built for stride 1 only
template <int FMT, int OUT>
static void launch_out(int stride, bool epi, int MT, int NT, const conv_args &a, size_t smem) {
    if (epi) { if (stride != 1) mi_die("conv3: the fused activation epilogue needs stride 1"); launch_mt<FMT, 1, OUT, true>(MT, NT, a, smem); }
    else if (stride == 1) launch_mt<FMT, 1, OUT, false>(MT, NT, a, smem);
    else launch_mt<FMT, 2, OUT, false>(MT, NT, a, smem);
}


// one translation unit per (compute format, output kind) instantiates its kernels behind this entry
// K order of the direct stride-2 kernel. The rows of taps kx = 0 and kx = 1 of a column are neighbours in memory (voxels 2 ox - 1, 2 ox), so they
// form a pair: its two loads read whole cache lines. Rows (kz, ky) are taken two at a time: per row and block the pair (kx 0 | kx 1), then the
// kx = 2 units of both rows, block after block, in pairs of their own (their lines were fetched by the pairs just before). nb blocks:
// 3 nb pairs per two rows, the ninth row nb + ceil(nb / 2); ceil(27 nb / 2) pairs in all. Returns whether the unit exists (else: padding).
__host__ __device__ __forceinline__ bool mi_s2_unit(int gp, int side, int nb, int *tap, int *blk) {
    const int G = gp < 12 * nb ? gp / (3 * nb) : 4, q = gp - G * 3 * nb, nrow = G < 4 ? 2 : 1;
    int row, b, kx; bool ok = true;
    if (q < nrow * nb) { row = 2 * G + q / nb; b = q % nb; kx = side; }
    else { const int idx = 2 * (q - nrow * nb) + side; ok = idx < nrow * nb; const int id = ok ? idx : 0; row = 2 * G + id / nb; b = id % nb; kx = 2; }
    *tap = row * 3 + kx; *blk = b;
    return ok;
}
void conv3s2_launch_f8(int out, int MT, const conv_args &a, dim3 grid, size_t smem);      // (the direct stride-2 kernel: conv2_kernel.hpp)
void conv3s2_launch_f4(int out, int MT, const conv_args &a, dim3 grid, size_t smem);
#define CONV3_LAUNCH_DECL(FMT, OUT) void conv3_launch_f##FMT##_o##OUT(int stride, bool epi, int MT, int NT, const conv_args &a, size_t smem)
CONV3_LAUNCH_DECL(8, 8); CONV3_LAUNCH_DECL(8, 4); CONV3_LAUNCH_DECL(8, 0);
CONV3_LAUNCH_DECL(4, 8); CONV3_LAUNCH_DECL(4, 4); CONV3_LAUNCH_DECL(4, 0);
// the tap-packed stem (conv3_stem.hip): weight preparation for CP padded channels, kernel launch
void conv3_stem_prep(int CP, const float *w, uint8_t *wq, uint8_t *wsc, int Co, int Ci, int nmt_all, int np);
void conv3_stem_launch(int CP, int MT, int out, const conv_args &a, size_t smem);
