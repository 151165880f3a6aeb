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

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

struct conv_args {
    const uint8_t *xq[2], *xsc[2];     // input segments (compute-format MX tensors): data, scale plane
    int nbs[2], bws[2];                // blocks per sample and block width of each segment's tensor
    int nb0p;                          // padded blocks of segment 0 (staged blocks [0, nb0p) come from segment 0)
    int nbt, CB;                       // staged 32-channel blocks in total, blocks per LDS chunk
    int N, D, H, W, Do, Ho, Wo;
    const uint8_t *wq, *wsc; int nmt_all;
    const float *bias; int Co;
    void *y; int ydt;
    double *osum; float *part; int Go, stored_stats, zs0, zs1;   // part: per tile and channel quad (sum, sum of squares)
    const float *ep_a, *ep_b; int act;
    int ntx, nty, ntz, ncs; unsigned ntiles;
};

template <int FMT> struct fmt_t;
template <> struct fmt_t<8> { static constexpr int RB = 32, NH = 2, WTILE = 2048; };
template <> struct fmt_t<4> { static constexpr int RB = 16, NH = 1, WTILE = 1024; };

__device__ __forceinline__ float gelu_erf(float x) { return 0.5f * x * (1.f + erff(x * 0.70710678f)); }

template <int FMT, int STRIDE, int MT, int NT>
__global__ void __launch_bounds__(256, 2) conv3_mx_k(const conv_args a) {
    constexpr int TZ = NT == 2 ? 2 : 4;
    constexpr int HZ = STRIDE * (TZ - 1) + 3, HY = STRIDE * 7 + 3, HX = STRIDE * 15 + 3, TT = HZ * HY * HX;
    constexpr int NH = fmt_t<FMT>::NH, WTILE = fmt_t<FMT>::WTILE;
    constexpr int STG = MT * (WTILE + 256);              // one weight stage: MT tiles of codes, then MT x 64 scale words
    constexpr int UPT = (MT * WTILE / 16 + 255) / 256;   // 16-byte weight units per thread and stage
    extern __shared__ __align__(16) unsigned char lds[];
    // LDS: [2 weight stages][pair table (npairs + 2) x 2 x 16 B][halo rows CB * NH * TT * 16 B][halo scales CB * TT words]
    const int tab_bytes = (((27 * a.CB + 1) >> 1) + 2) * 32;
    const unsigned wring_o = 0, tab_o = 2 * STG, act_o = tab_o + tab_bytes, asc_o = act_o + a.CB * NH * TT * 16;
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
    const int ix0 = STRIDE * ox0 - 1, iy0 = STRIDE * oy0 - 1, iz0 = STRIDE * oz0 - 1;

    // the lane's voxel in each of its NT tiles: wave -> (z, y half) for TZ 2, z for TZ 4; tile j -> rows 2j, 2j+1; r -> (row, x)
    int lz, ly0;
    if (NT == 2) { lz = wave >> 1; ly0 = (wave & 1) * 4; } else { lz = wave; ly0 = 0; }
    unsigned ab[NT], sbse[NT];     // LDS byte addresses of the lane's halo row (its 16-byte half) and scale word for tap (0, 0, 0) of block 0
#pragma unroll
    for (int j = 0; j < NT; j++) {
        const int p0 = ((STRIDE * lz) * HY + STRIDE * (ly0 + 2 * j + (r >> 4))) * HX + STRIDE * (r & 15);
        ab[j] = act_o + ((NH == 2 ? h * TT : 0) + p0) * 16;
        sbse[j] = asc_o + p0 * 4;
    }
    const unsigned wfa = wring_o + lane * 16, wfs = wring_o + MT * WTILE + lane * 4;    // the lane's weight fragment / scale word in stage slot 0, tile 0
    const unsigned wcp = wring_o + (tid * UPT * 16) % (MT * WTILE), wcs = wring_o + MT * WTILE + (tid * 4) % (MT * 256);   // the thread's part of a stage copy

    v16f acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[m][j][i] = 0.f;

    const size_t Sin = (size_t)a.D * a.H * a.W;
    const size_t wq_ps = (size_t)a.nmt_all * WTILE, wsc_ps = (size_t)a.nmt_all * 256;
    int pair0 = 0;                                       // global pair index of the chunk's first pair

    for (int b0 = 0; b0 < a.nbt; b0 += a.CB) {
        const int nbc = min(a.CB, a.nbt - b0), nunits = 27 * nbc, npairs = (nunits + 1) >> 1;
        __syncthreads();                                 // the previous chunk's readers are done with the halo
        // ---- pair table: per pair and lane half, the byte offsets of the pair's two units (fp8: both; fp4: the half's own) and of
        // the half's scale word. unit u = (tap u / nbc, local block u % nbc); the odd padding unit (zero weights) re-reads unit A ----
        for (int i = tid; i < (npairs + 2) * 2; i += 256) {
            const int q = min(i >> 1, npairs - 1), hh = i & 1;
            const int uA = 2 * q, uB = 2 * q + 1 < nunits ? 2 * q + 1 : 2 * q;
            const int tA = uA / nbc, bA = uA - tA * nbc, tB = uB / nbc, bB = uB - tB * nbc;
            const int pA = ((tA / 9) * HY + (tA / 3) % 3) * HX + tA % 3, pB = ((tB / 9) * HY + (tB / 3) % 3) * HX + tB % 3;
            const int dA = (bA * NH * TT + pA) * 16, dB = (bB * NH * TT + pB) * 16, sA = (bA * TT + pA) * 4, sB = (bB * TT + pB) * 4;
            *(v4i *)(lds + tab_o + i * 16) = (v4i){NH == 2 ? dA : (hh ? dB : dA), dB, hh ? sB : sA, 0};
        }
#ifndef DBG_NOSTAGE
        // ---- stage the halo of blocks [b0, b0 + nbc): rows copied as stored, zero rows (scale byte 1) outside the tensor.
        // Branch-free: every load reads a clamped in-tensor address and is zeroed afterwards when the position is outside;
        // four independent loads are in flight per thread ----
        {
            constexpr int NB = 4;
            const int E = nbc * TT * NH;
            for (int i0 = tid; i0 < E; i0 += 256 * NB) {
                v4i val[NB]; unsigned dst[NB]; bool inb[NB];
#pragma unroll
                for (int k = 0; k < NB; k++) {
                    const int i = min(i0 + k * 256, E - 1);
                    const int bl = i / (TT * NH), rem = i - bl * (TT * NH), pos = rem / NH, hf = rem - pos * NH;
                    const int px = pos % HX, py = (pos / HX) % HY, pz = pos / (HX * HY);
                    const int gz = iz0 + pz, gy = iy0 + py, gx = ix0 + px;
                    const int sb = b0 + bl, seg = sb >= a.nb0p, blk = seg ? sb - a.nb0p : sb;
                    const int rb = a.bws[seg] * FMT / 8;     // stored row bytes (16 NH for 32-wide blocks)
                    const bool pos_ok = gz >= 0 && gz < a.D && gy >= 0 && gy < a.H && gx >= 0 && gx < a.W && blk < a.nbs[seg];
                    const int cz = min(max(gz, 0), a.D - 1), cy = min(max(gy, 0), a.H - 1), cx = min(max(gx, 0), a.W - 1), cb = min(blk, a.nbs[seg] - 1);
                    const size_t row = ((size_t)n * a.nbs[seg] + cb) * Sin + ((size_t)cz * a.H + cy) * a.W + cx;
                    dst[k] = act_o + ((bl * NH + hf) * TT + pos) * 16;
                    if (rb >= 16) {
                        const bool have = rb >= (hf + 1) * 16;
                        val[k] = *(const v4i *)(a.xq[seg] + row * rb + (have ? hf * 16 : 0));
                        inb[k] = pos_ok && have;
                    } else {                                 // 8- or 4-byte rows of a <= 8 / <= 16 channel tensor: only half 0 holds data
                        val[k] = (v4i){0, 0, 0, 0};
                        if (rb == 8) { const int2 t = *(const int2 *)(a.xq[seg] + row * 8); val[k][0] = t.x; val[k][1] = t.y; }
                        else val[k][0] = *(const int *)(a.xq[seg] + row * 4);
                        inb[k] = pos_ok && hf == 0;
                    }
                }
#pragma unroll
                for (int k = 0; k < NB; k++) *(v4i *)(lds + dst[k]) = inb[k] ? val[k] : (v4i){0, 0, 0, 0};
            }
            const int E2 = nbc * TT;
            for (int i0 = tid; i0 < E2; i0 += 256 * NB) {
                unsigned sv[NB]; unsigned dst[NB];
#pragma unroll
                for (int k = 0; k < NB; k++) {
                    const int i = min(i0 + k * 256, E2 - 1);
                    const int bl = i / TT, pos = i - bl * TT;
                    const int px = pos % HX, py = (pos / HX) % HY, pz = pos / (HX * HY);
                    const int gz = iz0 + pz, gy = iy0 + py, gx = ix0 + px;
                    const int sb = b0 + bl, seg = sb >= a.nb0p, blk = seg ? sb - a.nb0p : sb;
                    const bool ok = gz >= 0 && gz < a.D && gy >= 0 && gy < a.H && gx >= 0 && gx < a.W && blk < a.nbs[seg];
                    const int cz = min(max(gz, 0), a.D - 1), cy = min(max(gy, 0), a.H - 1), cx = min(max(gx, 0), a.W - 1), cb = min(blk, a.nbs[seg] - 1);
                    const unsigned s = a.xsc[seg][((size_t)n * a.nbs[seg] + cb) * Sin + ((size_t)cz * a.H + cy) * a.W + cx];
                    sv[k] = ok ? s : 1u; dst[k] = asc_o + i * 4;
                }
#pragma unroll
                for (int k = 0; k < NB; k++) *(unsigned *)(lds + dst[k]) = sv[k];
            }
        }
#endif
        // ---- weight stages: global -> registers -> ring slot. Every thread moves UPT contiguous 16-byte units and one scale word per
        // stage; offsets wrap instead of being guarded (duplicates store the same value). The prepared-weight buffers carry four
        // stages of padding, so the loads that run ahead of the last pair stay inside them ----
        const uint8_t *wgp = a.wq + (size_t)pair0 * wq_ps + (size_t)cs * MT * WTILE + (tid * UPT * 16) % (MT * WTILE);
        const uint8_t *wgs = a.wsc + (size_t)pair0 * wsc_ps + (size_t)cs * MT * 256 + (tid * 4) % (MT * 256);
        v4i g[UPT]; unsigned gs = 0;
        auto wload = [&]() {            // the next stage in sequence
#ifndef DBG_NOWLOAD
#pragma unroll
            for (int k = 0; k < UPT; k++) g[k] = *(const v4i *)(wgp + k * 16);
            gs = *(const unsigned *)wgs;
            wgp += wq_ps; wgs += wsc_ps;
#endif
        };
        auto wstore = [&](int slot) {
#pragma unroll
            for (int k = 0; k < UPT; k++) *(v4i *)(lds + wcp + slot * STG + k * 16) = g[k];
            *(unsigned *)(lds + wcs + slot * STG) = gs;
        };
        wload(); wstore(0);
        wload();
        __syncthreads();

        // ---- K loop over unit pairs, unrolled by 2 so that the ring slot (pair & 1) is static. Step of pair q: fetch its fragments
        // from LDS (halo rows at the table's offsets, weights from ring slot q & 1), run its MFMAs, move stage q + 1 into the other
        // slot and start loading stage q + 2 from L2. A second workgroup on the CU covers this one's LDS latency and barriers ----
        v8i fb[NT], fa[MT]; int sb[NT], sa[MT];
        v4i T;
        unsigned tabp = tab_o + (lane >> 5) * 16;          // this half's entry of pair 0
        auto fetch = [&](int slot) {
            const v4i t = T;
#pragma unroll
            for (int j = 0; j < NT; j++) {
                const v4i lo = *(const v4i *)(lds + ab[j] + t[0]);
                if (FMT == 8) {
                    const v4i hi = *(const v4i *)(lds + ab[j] + t[1]);
                    fb[j] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                } else fb[j] = (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
                sb[j] = *(const int *)(lds + sbse[j] + t[2]);
            }
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const v4i lo = *(const v4i *)(lds + wfa + slot * STG + m * WTILE);
                if (FMT == 8) {
                    const v4i hi = *(const v4i *)(lds + wfa + slot * STG + m * WTILE + 1024);
                    fa[m] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                } else fa[m] = (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
                sa[m] = *(const int *)(lds + wfs + slot * STG + m * 256);
            }
            T = *(const v4i *)(lds + tabp + 32); tabp += 32;      // the next pair's table entry
        };
        auto mma = [&]() {
#ifndef DBG_NOMMA
#pragma unroll
            for (int m = 0; m < MT; m++)
#pragma unroll
                for (int j = 0; j < NT; j++)
                    acc[m][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[m], fb[j], acc[m][j], FMT == 8 ? 0 : 4, FMT == 8 ? 0 : 4, 0, sa[m], 0, sb[j]);
#else
            for (int m = 0; m < MT; m++) for (int j = 0; j < NT; j++) acc[m][j][0] += (float)(fa[m][0] + fb[j][0] + sa[m] + sb[j]);
#endif
        };
        T = *(const v4i *)(lds + tabp);
        for (int q = 0; q < npairs; q += 2) {
            fetch(0); mma(); wstore(1); wload();
            __syncthreads();
            if (q + 1 >= npairs) break;
            fetch(1); mma(); wstore(0); wload();
            __syncthreads();
        }
        pair0 += npairs;
    }

    // ================= epilogue =================
    // accumulator layout of the 32x32 MFMA: lane (r = voxel within the tile, h), register i -> channel (i & 3) + 4 h + 8 (i >> 2)
    const size_t So = (size_t)a.Do * a.Ho * a.Wo;
    const int co_base = cs * MT * 32;
    float *red = (float *)lds;                      // stats scratch [4 waves][MT][8 quads][2] floats (the ring and halo are dead now)
    const bool stats = a.osum != nullptr;
    if (stats) __syncthreads();
    float qs[MT][4], qss[MT][4];                    // per lane: sums over its voxels of the 4-channel quads (m, i >> 2)
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) { qs[m][q4] = 0.f; qss[m][q4] = 0.f; }
    const int cpg = a.Go > 0 ? a.Co / a.Go : 1;
    static_for<NT>([&](auto J) {
        constexpr int j = J;
        const int oz = oz0 + lz, oy = oy0 + ly0 + 2 * j + (r >> 4), ox = ox0 + (r & 15);
        const bool ok = oz < a.Do && oy < a.Ho && ox < a.Wo;
        const size_t ov = ((size_t)oz * a.Ho + oy) * a.Wo + ox;
        const bool zst = ok && oz >= a.zs0 && oz < a.zs1;
        static_for<MT>([&](auto M) {
            constexpr int m = M;
            float v[16];
            float am = 0.f;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int co = co_base + m * 32 + (i & 3) + 4 * h + 8 * (i >> 2);
                float t = acc[m][j][i];
                if (co < a.Co) {
                    if (a.bias) t += a.bias[co];
                    if (a.act) {
                        if (a.ep_a) t = fmaf(t, a.ep_a[co], a.ep_b[co]);
                        t = a.act == 1 ? __fdividef(t, 1.f + __expf(-t)) : a.act == 2 ? gelu_erf(t) : fmaxf(t, 0.f);
                    }
                } else t = 0.f;
                v[i] = t; am = fmaxf(am, fabsf(t));
            }
            if (a.ydt >= 3) {
                const int ybits = a.ydt == 3 ? 8 : 4;
                am = fmaxf(am, __shfl_xor(am, 32));
                const int e = d_mx_exp(am, ybits == 8 ? MI_INVQ8 : MI_INVQ4);
                const float mult = d_exp2i(-e);
                const int bwo = mx_bw(a.Co), nbo = mx_nb(a.Co);
                uint8_t *yq = (uint8_t *)a.y, *ysc = yq + (size_t)a.N * nbo * So * mx_rb(bwo, ybits);
                const int blk = (co_base + m * 32) / bwo;                  // bwo < 32 only when Co <= 16: one tile, block 0
                const size_t row = ((size_t)n * nbo + blk) * So + ov;
                if (ybits == 8) {
                    unsigned d[4];
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++) d[q4] = d_enc_e4m3x4(v[4 * q4] * mult, v[4 * q4 + 1] * mult, v[4 * q4 + 2] * mult, v[4 * q4 + 3] * mult);
                    if (a.stored_stats) {
                        const float sc = d_exp2i(e);
#pragma unroll
                        for (int i = 0; i < 16; i++) v[i] = d_dec_e4m3(d[i >> 2] >> (8 * (i & 3))) * sc;
                    }
                    // lane h = 0 holds bytes {0-3, 8-11, 16-19, 24-27}, its partner {4-7, 12-15, 20-23, 28-31}: swap so each stores 16 contiguous bytes
                    const unsigned s0 = h ? d[0] : d[2], s1 = h ? d[1] : d[3];
                    const unsigned r0 = __shfl_xor(s0, 32), r1 = __shfl_xor(s1, 32);
                    const uint4 out = h ? make_uint4(r0, d[2], r1, d[3]) : make_uint4(d[0], r0, d[1], r1);
                    if (ok && co_base + m * 32 < a.Co) {
                        if (bwo == 32) *(uint4 *)(yq + row * 32 + 16 * h) = out;
                        else if (bwo == 16) { if (!h) *(uint4 *)(yq + row * 16) = out; }
                        else if (!h) *(uint2 *)(yq + row * 8) = make_uint2(out.x, out.y);
                    }
                } else {
                    unsigned hw[4];   // 4 channels -> 16 bits each
#pragma unroll
                    for (int q4 = 0; q4 < 4; q4++) {
                        hw[q4] = 0u;
#pragma unroll
                        for (int k = 0; k < 4; k++) hw[q4] |= d_enc_e2m1(v[4 * q4 + k] * mult) << (4 * k);
                    }
                    if (a.stored_stats) {
                        const float sc = d_exp2i(e);
#pragma unroll
                        for (int i = 0; i < 16; i++) v[i] = d_dec_e2m1(hw[i >> 2] >> (4 * (i & 3))) * sc;
                    }
                    // halfword q4 of lane h sits at byte 4 q4 + 2 h of the 16-byte row: lane 0 assembles words 0-1, lane 1 words 2-3
                    const unsigned mine01 = hw[0] | (hw[1] << 16), mine23 = hw[2] | (hw[3] << 16);
                    const unsigned send = h ? mine01 : mine23, recv = __shfl_xor(send, 32);
                    uint2 out;
                    if (!h) out = make_uint2((hw[0] & 0xffffu) | ((recv & 0xffffu) << 16), (hw[1] & 0xffffu) | (recv & 0xffff0000u));
                    else out = make_uint2((recv & 0xffffu) | ((hw[2] & 0xffffu) << 16), (recv >> 16) | ((hw[3] & 0xffffu) << 16));
                    if (ok && co_base + m * 32 < a.Co) {
                        if (bwo == 32) *(uint2 *)(yq + row * 16 + 8 * h) = out;
                        else if (bwo == 16) { if (!h) *(uint2 *)(yq + row * 8) = out; }
                        else if (!h) *(unsigned *)(yq + row * 4) = out.x;
                    }
                }
                if (ok && !h && co_base + m * 32 < a.Co) ysc[row] = (uint8_t)(e + 127);
            } else {
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int co = co_base + m * 32 + (i & 3) + 4 * h + 8 * (i >> 2);
                    if (a.ydt == 2) {
                        if (a.Go > 0) v[i] = fabsf(v[i]) > 65504.f ? copysignf(65504.f, v[i]) : v[i];     // src/lp_common.cuh:465, :1567-1569
                        if (ok && co < a.Co) ((__half *)a.y)[((size_t)n * a.Co + co) * So + ov] = __float2half(v[i]);
                    } else if (ok && co < a.Co) ((float *)a.y)[((size_t)n * a.Co + co) * So + ov] = v[i];
                }
            }
            if (stats && zst) {
#pragma unroll
                for (int i = 0; i < 16; i++) { qs[m][i >> 2] += v[i]; qss[m][i >> 2] += v[i] * v[i]; }
            }
        });
    });
    if (stats) {
        // channels per group a multiple of 4: a quad (m, q4, h) = channels co_base + 32 m + 8 q4 + 4 h .. +3 lies in one group.
        // Sum over the 32 voxel lanes of each half (butterfly, fixed order), then over the 4 waves in wave order, then one
        // exact slot add per quad.
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                float s = qs[m][q4], ss = qss[m][q4];
#pragma unroll
                for (int d = 1; d < 32; d <<= 1) { s += __shfl_xor(s, d); ss += __shfl_xor(ss, d); }
                if (r == 0) { red[((wave * MT + m) * 8 + q4 * 2 + h) * 2] = s; red[((wave * MT + m) * 8 + q4 * 2 + h) * 2 + 1] = ss; }
            }
        __syncthreads();
        if (tid < MT * 8) {
            // per tile and channel quad, the sums over the tile's voxels in wave order; a second kernel adds the tiles of a sample
            // in a fixed order into the exact sum slots, so the statistics do not depend on the order workgroups finish in
            const int m = tid >> 3, q8 = tid & 7;                       // q8 = q4 * 2 + h: channels co_base + 32 m + 8 q4 + 4 h .. + 3
            float s = 0.f, ss = 0.f;
            for (int w = 0; w < 4; w++) { s += red[((w * MT + m) * 8 + q8) * 2]; ss += red[((w * MT + m) * 8 + q8) * 2 + 1]; }
            a.part[((size_t)tile * MT * 8 + tid) * 2] = s;
            a.part[((size_t)tile * MT * 8 + tid) * 2 + 1] = ss;
        }
    }
}

// (sum, sum of squares) partials of the tiles -> exact GroupNorm sum slots: one block per (sample, group), double accumulation over
// the sample's tiles in index order, a fixed tree over the block, one slot add per sum (src/lp_common.cuh:1575-1597 does the same with
// one fixed-point atomic per block and channel)
__global__ void __launch_bounds__(256) gn_part_reduce_k(const float *part, int tiles_per_n, int ncs, int MT, int Co, int Go, double *osum) {
    const int n = blockIdx.x / Go, gidx = blockIdx.x % Go, cpg = Co / Go, nq = MT * 8;
    double s = 0.0, ss = 0.0;
    for (int i = threadIdx.x; i < tiles_per_n * nq; i += 256) {
        const int t = i / nq, qd = i - t * nq, cs = t % ncs, m = qd >> 3, q8 = qd & 7;
        const int co = (cs * MT + m) * 32 + 8 * (q8 >> 1) + 4 * (q8 & 1);
        if (co < Co && co / cpg == gidx) {
            const float *p = part + ((size_t)(n * tiles_per_n + t) * nq + qd) * 2;
            s += (double)p[0]; ss += (double)p[1];
        }
    }
    __shared__ double r1[256], r2[256];
    r1[threadIdx.x] = s; r2[threadIdx.x] = ss;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) { if ((int)threadIdx.x < st) { r1[threadIdx.x] += r1[threadIdx.x + st]; r2[threadIdx.x] += r2[threadIdx.x + st]; } __syncthreads(); }
    if (threadIdx.x == 0) { gn_acc_add(osum, 2 * (size_t)blockIdx.x, r1[0]); gn_acc_add(osum, 2 * (size_t)blockIdx.x + 1, r2[0]); }
}

// ---- weights: fp32 w[co][ci][27] -> per (chunk, unit pair, 32-row channel tile) fragment-ordered codes + scale bytes ----
// block = the 32 ci of one (tap, co) (src/lp_f8fwd.cu:54-71, src/lp_f4fwd.cu:53-66); fmaxf amax; padded rows / channels / the odd
// padding unit are zero codes with scale byte 1
__host__ __device__ __forceinline__ int seg_ci(int cp, int Ci, int Cx, int CxP) { if (cp < CxP) return cp < Cx ? cp : -1; const int c = Cx + cp - CxP; return c < Ci ? c : -1; }
template <int FMT>
__global__ void __launch_bounds__(128) prep_w_k(const float *__restrict__ w, uint8_t *__restrict__ wq, unsigned *__restrict__ wsc, int Co, int Ci, int Cx, int CxP,
                                               int nbt, int CB, int nmt_all, int npairs_all) {
    constexpr int WTILE = fmt_t<FMT>::WTILE;
    const size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const int Cop = nmt_all * 32;
    if (i >= (size_t)npairs_all * Cop) return;
    const int cop = (int)(i % Cop), gp = (int)(i / Cop);
    int b0 = 0, pb = 0, nbc = 0;
    for (;; b0 += CB) { nbc = min(CB, nbt - b0); const int np = (27 * nbc + 1) >> 1; if (gp < pb + np) break; pb += np; }
    const int q = gp - pb, m = cop >> 5, r = cop & 31;
    uint8_t *tile = wq + ((size_t)gp * nmt_all + m) * WTILE;
    unsigned *tsc = wsc + ((size_t)gp * nmt_all + m) * 64;      // one word per lane: the byte the MFMA reads is the low one
#pragma unroll
    for (int side = 0; side < 2; side++) {
        const int u = 2 * q + side;
        float v[32]; float amax = 0.f;
        const int t = u / nbc, blk = b0 + u % nbc;
#pragma unroll
        for (int k = 0; k < 32; k++) {
            const int ci = seg_ci(blk * 32 + k, Ci, Cx, CxP);
            v[k] = (u < 27 * nbc && cop < Co && ci >= 0) ? w[((size_t)cop * Ci + ci) * 27 + t] : 0.f;
            amax = fmaxf(amax, fabsf(v[k]));
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
        tsc[r + 32 * side] = (unsigned)(e + 127);
    }
}

// ---- prepared-weight memo (src/lp_f4fwd.cuh:748-770): keyed by the conv id sp.wkey and the layout ----
struct wmemo_t { unsigned key; const float *w; int fmt, Co, Ci, Cx, nbt, CB, nmt_all, dev; uint8_t *wq, *wsc; };
static std::vector<wmemo_t> g_wmemo;
static unsigned g_wstep = 0;
extern "C" void lp_wmemo_clear(void) {
    if (g_wmemo.empty()) return;
    MIRT(hipDeviceSynchronize());
    for (auto &m : g_wmemo) { MIRT(hipFree(m.wq)); MIRT(hipFree(m.wsc)); }
    g_wmemo.clear();
}
extern "C" void lp_wmemo_step(unsigned step) { if (step != g_wstep) { g_wstep = step; lp_wmemo_clear(); } }

static thread_local char g_last_kernel[96] = "";
extern "C" const char *mi_last_kernel(void) { return g_last_kernel; }

template <int FMT, int STRIDE, int MT, int NT>
static void launch_conv(const conv_args &a, size_t smem) {
    static bool attr[8];
    int d = 0; MIRT(hipGetDevice(&d)); d &= 7;
    if (!attr[d]) { MIRT(hipFuncSetAttribute((const void *)conv3_mx_k<FMT, STRIDE, MT, NT>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024)); attr[d] = true; }
    const unsigned per = (a.ntiles + 7u) / 8u;
    conv3_mx_k<FMT, STRIDE, MT, NT><<<per * 8u, 256, smem>>>(a);
    MICK();
    snprintf(g_last_kernel, sizeof g_last_kernel, "conv3_mx_k<fmt %d, stride %d, MT %d, NT %d> CB %d tiles %u", FMT, STRIDE, MT, NT, a.CB, a.ntiles);
}
template <int FMT, int STRIDE>
static void launch_mt(int MT, int NT, const conv_args &a, size_t smem) {
    switch (MT * 10 + NT) {
    case 12: launch_conv<FMT, STRIDE, 1, 2>(a, smem); break;
    case 14: if (STRIDE == 1) { launch_conv<FMT, 1, 1, 4>(a, smem); break; }
    case 22: launch_conv<FMT, STRIDE, 2, 2>(a, smem); break;
    case 24: if (STRIDE == 1) { launch_conv<FMT, 1, 2, 4>(a, smem); break; }
    case 32: launch_conv<FMT, STRIDE, 3, 2>(a, smem); break;
    case 42: launch_conv<FMT, STRIDE, 4, 2>(a, smem); break;
    default: mi_die("conv3: no kernel for MT %d NT %d", MT, NT);
    }
}

// the conv of every entry point: fmt 8 / 4 = compute format, stride 1 / 2
static int conv_dispatch(const char *who, int fmt, int stride, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf,
                         gnp_t gp, double *osum, int Go, split_t sp, const float *ep_a, const float *ep_b, int act) {
    if (sp.y2 || sp.o_split || sp.accum || sp.sr || sp.osr || sp.yD || sp.zi0 || sp.Di || sp.o_pad || sp.zw0 || sp.zw1 || sp.yzo)
        mi_die("%s: split outputs, accumulate, stochastic rounding and z-slab / z-window fields of split_t are not built here (inference forward only)", who);
    if (gp.ns || sp.gp2.ns) mi_die("%s: slab-local GroupNorm statistics are not supported", who);
    if (xbf < 0 || xbf > 4 || !(ybf == 0 || ybf == 2 || ybf == 3 || ybf == 4)) mi_die("%s: unsupported storage types (in %d, out %d)", who, xbf, ybf);
    if (xs.n <= 0 || xs.c <= 0 || xs.d <= 0 || xs.h <= 0 || xs.w <= 0 || cout <= 0) return 0;
    const int Ci = xs.c, Cx = sp.x2 ? sp.c_split : Ci, C2 = Ci - Cx;
    if (sp.x2 && (Cx <= 0 || C2 <= 0)) mi_die("%s: channel split %d of %d", who, sp.c_split, Ci);
    if (sp.x2 && xbf < 3) mi_die("%s: split inputs need MX storage", who);
    if (sp.up && (!sp.x2 || xbf < 3 || (xs.d & 1) || (xs.h & 1) || (xs.w & 1) || stride != 1)) mi_die("%s: the fused upsample needs an MX split input and even dims", who);
    if (osum && (Go <= 0 || cout % Go)) mi_die("%s: %d output channels in %d groups", who, cout, Go);
    if (osum && (cout / Go) % 4) mi_die("%s: fused output statistics need channels per group (%d) to be a multiple of 4", who, cout / Go);
    if (gp.G && ((sp.x2 && sp.gp2.G ? Cx : Ci) % gp.G)) mi_die("%s: GroupNorm groups %d do not divide the channels", who, gp.G);
    if (sp.gp2.G && (!sp.x2 || C2 % sp.gp2.G)) mi_die("%s: second GroupNorm without a matching x2 segment", who);
    const int N = xs.n, D = xs.d, H = xs.h, W = xs.w;
    const int Do = stride == 2 ? (D - 1) / 2 + 1 : D, Ho = stride == 2 ? (H - 1) / 2 + 1 : H, Wo = stride == 2 ? (W - 1) / 2 + 1 : W;   // src/nn_bwd.cu:132-135
    const size_t S = (size_t)D * H * W;
    const int fdt = fmt == 8 ? 3 : 4;
    conv_args a; memset(&a, 0, sizeof a);
    // ---- operands: a segment is read as stored when it already is the compute format with nothing to apply, else re-staged once ----
    const bool s2g = sp.x2 && sp.gp2.G;
    const void *segx[2] = {x, sp.x2}; const int segC[2] = {Cx, C2};
    for (int s = 0; s < (sp.x2 ? 2 : 1); s++) {
        gnp_t g = s2g ? (s ? sp.gp2 : gp) : gp;
        const int Cg = s2g ? segC[s] : Ci, cg0 = s2g ? 0 : (s ? Cx : 0);
        const bool upseg = s == 0 && sp.up;
        const bool direct = xbf == fdt && !g.G && !upseg;
        const int nbp = (segC[s] + 31) / 32;
        if (direct) {
            const int bw = mx_bw(segC[s]), nb = mx_nb(segC[s]);
            a.xq[s] = (const uint8_t *)segx[s]; a.xsc[s] = a.xq[s] + (size_t)N * nb * S * mx_rb(bw, fmt);
            a.nbs[s] = nb; a.bws[s] = bw;
        } else {
            const size_t bytes = (size_t)N * nbp * S * (mx_rb(32, fmt) + 1);
            uint8_t *st = (uint8_t *)mi_ws(s ? MI_WS_X2STAGE : MI_WS_XSTAGE, bytes);
            if (upseg) mi_restage_up(segx[s], xbf, N, segC[s], D, H, W, g, Cg, st, fmt);
            else mi_restage(segx[s], xbf, N, segC[s], S, g, Cg, cg0, st, fmt);
            a.xq[s] = st; a.xsc[s] = st + (size_t)N * nbp * S * mx_rb(32, fmt);
            a.nbs[s] = nbp; a.bws[s] = 32;
        }
        if (s == 0) a.nb0p = nbp;
    }
    a.nbt = a.nb0p + (sp.x2 ? (C2 + 31) / 32 : 0);
    a.N = N; a.D = D; a.H = H; a.W = W; a.Do = Do; a.Ho = Ho; a.Wo = Wo;
    a.bias = b; a.Co = cout; a.y = y; a.ydt = ybf;
    a.osum = osum; a.Go = Go; a.stored_stats = sp.stored_stats && ybf >= 3; a.zs0 = sp.zlo; a.zs1 = Do - sp.zhi;
    a.ep_a = ep_a; a.ep_b = ep_b; a.act = act;
    // ---- tile shape: MT channel tiles of 32 per workgroup, NT voxel tiles of 32 per wavefront, MT * NT <= 8 accumulators ----
    const int nmt_all = (cout + 31) / 32;
    int MT = nmt_all <= 4 ? nmt_all : nmt_all % 4 == 0 ? 4 : nmt_all % 3 == 0 ? 3 : nmt_all % 2 == 0 ? 2 : 1;
    int NT = (stride == 1 && MT <= 2 && Do >= 4) ? 4 : 2;
    const int TZ = NT == 2 ? 2 : 4;
    const int HZ = stride * (TZ - 1) + 3, HY = stride * 7 + 3, HX = stride * 15 + 3, TT = HZ * HY * HX;
    const int RB = fmt == 8 ? 32 : 16, WTILE = fmt == 8 ? 2048 : 1024;
    // LDS of a workgroup holding CB input blocks: weight ring, pair table, halo rows and scale words. Prefer the largest CB that
    // still lets two workgroups share a CU (160 KB): the second one computes while the first stages its halo or runs its epilogue
    auto lds_bytes = [&](int cb) { return (size_t)2 * MT * (WTILE + 256) + (size_t)(((27 * cb + 1) >> 1) + 2) * 32 + (size_t)cb * TT * (RB + 4); };
    int cb2 = 0, cb1 = 0;
    for (int cb = 1; cb <= a.nbt; cb++) { if (lds_bytes(cb) <= 80 * 1024) cb2 = cb; if (lds_bytes(cb) <= 160 * 1024 - 256) cb1 = cb; }
    int cbmax = cb2 ? cb2 : cb1;
    static int cb_env = -1;
    if (cb_env < 0) cb_env = getenv("MI_CONV_CB") ? atoi(getenv("MI_CONV_CB")) : 0;      // tuning knob: blocks per chunk
    if (cb_env > 0 && cb_env <= cb1) cbmax = cb_env;
    if (cbmax < 1) mi_die("%s: tile does not fit LDS", who);
    const int nchunks = (a.nbt + cbmax - 1) / cbmax;
    a.CB = (a.nbt + nchunks - 1) / nchunks;
    size_t smem = lds_bytes(a.CB);
    const size_t red_bytes = (size_t)4 * MT * 8 * 2 * sizeof(float);
    if (smem < red_bytes) smem = red_bytes;
    smem = (smem + 15) & ~(size_t)15;
    a.nmt_all = nmt_all; a.ncs = nmt_all / MT;
    a.ntx = (Wo + 15) / 16; a.nty = (Ho + 7) / 8; a.ntz = (Do + TZ - 1) / TZ;
    a.ntiles = (unsigned)((size_t)a.ntx * a.nty * a.ntz * a.ncs * N);
    // ---- weights ----
    int npairs_all = 0;
    for (int b0 = 0; b0 < a.nbt; b0 += a.CB) npairs_all += (27 * (a.nbt - b0 < a.CB ? a.nbt - b0 : a.CB) + 1) >> 1;
    // (four stages of padding: the kernel's weight loads run up to three pairs ahead of the last one)
    const size_t wq_bytes = (size_t)(npairs_all + 4) * nmt_all * WTILE, wsc_bytes = (size_t)(npairs_all + 4) * nmt_all * 256;
    const int CxP = (Cx + 31) / 32 * 32;
    int dev = 0; MIRT(hipGetDevice(&dev));
    uint8_t *wq = nullptr, *wsc = nullptr; bool have = false;
    if (sp.wkey) {
        for (auto &m : g_wmemo)
            if (m.key == sp.wkey && m.w == w && m.fmt == fmt && m.Co == cout && m.Ci == Ci && m.Cx == Cx && m.nbt == a.nbt && m.CB == a.CB && m.nmt_all == nmt_all && m.dev == dev) { wq = m.wq; wsc = m.wsc; have = true; break; }
        if (!have) {
            MIRT(hipMalloc((void **)&wq, wq_bytes)); MIRT(hipMalloc((void **)&wsc, wsc_bytes));
            if (!wq || !wsc) mi_die("%s: no device memory for the prepared weights", who);
            MIRT(hipMemsetAsync(wq, 0, wq_bytes, 0)); MIRT(hipMemsetAsync(wsc, 0, wsc_bytes, 0));
            g_wmemo.push_back(wmemo_t{sp.wkey, w, fmt, cout, Ci, Cx, a.nbt, a.CB, nmt_all, dev, wq, wsc});
        }
    } else { wq = (uint8_t *)mi_ws(MI_WS_WQ, wq_bytes); wsc = (uint8_t *)mi_ws(MI_WS_WSC, wsc_bytes); }
    if (!have) {
        const size_t nt = (size_t)npairs_all * nmt_all * 32;
        if (fmt == 8) prep_w_k<8><<<nblk_(nt, 128), 128>>>(w, wq, (unsigned *)wsc, cout, Ci, Cx, CxP, a.nbt, a.CB, nmt_all, npairs_all);
        else prep_w_k<4><<<nblk_(nt, 128), 128>>>(w, wq, (unsigned *)wsc, cout, Ci, Cx, CxP, a.nbt, a.CB, nmt_all, npairs_all);
        MICK();
    }
    a.wq = wq; a.wsc = wsc;
    if (osum) a.part = (float *)mi_ws(MI_WS_MISC, (size_t)a.ntiles * MT * 8 * 2 * sizeof(float));
    if (fmt == 8) { if (stride == 1) launch_mt<8, 1>(MT, NT, a, smem); else launch_mt<8, 2>(MT, NT, a, smem); }
    else { if (stride == 1) launch_mt<4, 1>(MT, NT, a, smem); else launch_mt<4, 2>(MT, NT, a, smem); }
    if (osum) {
        gn_part_reduce_k<<<N * Go, 256>>>(a.part, (int)(a.ntiles / N), a.ncs, MT, cout, Go, osum);
        MICK();
    }
    return 0;
}

extern "C" int lp_conv_fwd_f8(const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp, double *osum, int Go, split_t sp) {
    return conv_dispatch("lp_conv_fwd_f8", 8, 1, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp, nullptr, nullptr, 0);
}
extern "C" int lp_conv_fwd_f4(const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp, double *osum, int Go, split_t sp) {
    return conv_dispatch("lp_conv_fwd_f4", 4, 1, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp, nullptr, nullptr, 0);
}
extern "C" int lp_conv_fwd_s2_f8(const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, shape5 ys, gnp_t gp) {
    const int Do = (xs.d - 1) / 2 + 1, Ho = (xs.h - 1) / 2 + 1, Wo = (xs.w - 1) / 2 + 1;
    if (ys.d != Do || ys.h != Ho || ys.w != Wo || ys.c != cout || ys.n != xs.n) mi_die("lp_conv_fwd_s2_f8: output shape %d x %d x %d x %d x %d does not match a stride-2 conv of the input", ys.n, ys.c, ys.d, ys.h, ys.w);
    split_t sp; memset(&sp, 0, sizeof sp);
    // compute format as the reference's dispatch (src/lp_s2.cu:647-754): fp4 only for an MX-fp4 32 -> <= 32 channel conv on even dims, else fp8
    const bool f4 = xbf == 4 && xs.c == 32 && cout <= 32 && !(xs.d & 1) && !(xs.h & 1) && !(xs.w & 1);
    conv_dispatch("lp_conv_fwd_s2_f8", f4 ? 4 : 8, 2, x, xbf, xs, w, b, cout, y, ybf, gp, nullptr, 0, sp, nullptr, nullptr, 0);
    return f4 ? 3 : 0;
}
extern "C" int mi_conv_fwd_fused(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf,
                                 const float *ep_a, const float *ep_b, int act, gnp_t gp, double *osum, int Go, split_t sp) {
    if (bits != 8 && bits != 4) mi_die("mi_conv_fwd_fused: compute format %d (8 or 4)", bits);
    if (act < 0 || act > 3 || (!act && ep_a) || (!ep_a != !ep_b)) mi_die("mi_conv_fwd_fused: activation %d / affine arguments", act);
    return conv_dispatch("mi_conv_fwd_fused", bits, 1, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp, ep_a, ep_b, act);
}
