// Tap-packed small-channel 3x3x3 conv, the network stem (src/lp_f8fwd.cuh:153-177 weights, :178-400 kernel, :601-609 dispatch).
// Input channels are padded to CP in {4, 8, 16}; a K block of 32 = 32 / CP taps x CP channels, so the 27 taps take ceil(27 CP / 32) blocks
// instead of 27 nearly empty ones. A block mixes positions, so the activation operand has ONE E8M0 scale per staged tile: the
// 4 x 10 x 18 input positions around a 2 x 8 x 16 output tile (tiles on the output grid from the origin). The input is read as stored
// (fp32 / fp16 planes or an MX tensor of one block row per voxel), GroupNorm + SiLU applied when the input carries one, the tile's amax
// taken over those values (fmaxf: NaN ignored; zeros outside the volume), and the values re-encoded to e4m3 with the tile's scale in LDS.
//
// One workgroup per output tile and slice of MT x 32 output channels; four wavefronts, each two 32-voxel MFMA tiles. A 32x32x64 MFMA
// takes two K blocks: lane (r, h) supplies bytes 16 h .. 16 h + 15 of both, i.e. 16 / CP taps of CP channels per block, read straight
// from the staged tile [position][CP bytes] at the taps' offsets. The weights' fragments stay in registers. Epilogue: conv_epilogue.
#include "conv3_kernel.hpp"

// PL: the input is fp32 / fp16 planes (else an MX tensor): a template parameter so that the path not taken holds no registers
template <int CP, int MT, int OUT, bool PL>
__global__ void __launch_bounds__(256, MT == 1 ? (CP == 8 ? 4 : 3) : (CP == 8 ? 3 : 2)) conv3_stem_k(const conv_args a) {
    constexpr int TPK = 32 / CP, NKB = (27 + TPK - 1) / TPK, NP = (NKB + 1) / 2, NT = 2;
    constexpr int HY = 10, HX = 18, TT = 4 * HY * HX, WTILE = 2048;
    extern __shared__ __align__(16) unsigned char lds[];
    // LDS: [staged tile TT x CP bytes][amax word, padded to 16][per channel (a, b) of the GroupNorm affine: CP x float2]
    constexpr unsigned am_o = TT * CP, ab_o = am_o + 16;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;
    // a workgroup walks a.zc consecutive z tiles of one (x, y) column: weights, constants and the channel table are set up once, and the next
    // tile's input rows are in flight while this tile is multiplied and stored
    constexpr bool ZL = CP <= 4;                             // (wider rows: the weights' fragments fill the registers, one tile per workgroup)
    const int zc = ZL ? a.zc : 1, nzg = (a.ntz + zc - 1) / zc;
    unsigned grp;
    {
        const unsigned per = (a.ngrp + 7u) / 8u;            // consecutive workgroup ids go round the 8 XCDs: a contiguous range per XCD
        grp = (blockIdx.x & 7u) * per + (blockIdx.x >> 3);
        if (grp >= a.ngrp) return;
    }
    int tt = (int)grp;
    const int cs = tt % a.ncs; tt /= a.ncs;
    const int tx = tt % a.ntx; tt /= a.ntx;
    const int ty = tt % a.nty; tt /= a.nty;
    const int zg = tt % nzg; const int n = tt / nzg;
    const int ox0 = tx * 16, oy0 = ty * 8;
    const int tz0 = zg * zc, tz1 = ZL ? min(a.ntz, tz0 + zc) : tz0 + 1;
    const int Ci = a.sCi;
    const size_t S = (size_t)a.D * a.H * a.W;

    if (tid == 0) *(unsigned *)(lds + am_o) = 0u;
    for (int i = tid; i < CP * (a.sns ? a.sns : 1); i += 256) {          // (slab-local statistics: one table per slab, back to back)
        const int k = i % CP, row = a.sns ? n * a.sns + i / CP : n;
        float ga = 1.f, gb = 0.f;
        if (a.sG && k < Ci) { const int ng = row * a.sG + k / (Ci / a.sG); ga = a.srstd[ng] * a.sgam[k]; gb = fmaf(-a.smean[ng], ga, a.sbet[k]); }
        *(float2 *)(lds + ab_o + i * 8) = make_float2(ga, gb);
    }
    conv_epi_consts<MT, false>(a, lds, cs, tid);

    // ---- the weights' fragments and scale words: pair p = K blocks 2 p, 2 p + 1 ----
    v8i fa[NP][MT]; int sa[NP][MT];
#pragma unroll
    for (int p = 0; p < NP; p++)
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const size_t t = (size_t)p * a.nmt_all + cs * MT + m;
            const v4i lo = *(const v4i *)(a.wq + t * WTILE + lane * 16), hi = *(const v4i *)(a.wq + t * WTILE + 1024 + lane * 16);
            fa[p][m] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            sa[p][m] = *(const int *)(a.wsc + (t * 64 + lane) * 4);
        }

    // ---- a thread owns positions tid, tid + 256, tid + 512 of a tile; their (y, x) part is the same for every z tile ----
    const int xdt = a.sxdt;
    int piz[3]; size_t pyx[3]; bool pin[3];
#pragma unroll
    for (int j = 0; j < 3; j++) {
        const int pos = tid + 256 * j, ix = pos % HX, iy = (pos / HX) % HY;
        const int gy = oy0 - 1 + iy, gx = ox0 - 1 + ix;
        piz[j] = pos / (HY * HX);
        pin[j] = pos < TT && (unsigned)gy < (unsigned)a.H && (unsigned)gx < (unsigned)a.W;
        pyx[j] = pin[j] ? (size_t)gy * a.W + gx : 0;
    }
    unsigned raw0[3], raw1[3]; unsigned rsc[3]; bool rin[3];
    auto request = [&](int tz) __attribute__((always_inline)) {                             // the raw input of tile tz -> registers
#pragma unroll
        for (int j = 0; j < 3; j++) {
            const int gz = 2 * tz - 1 + piz[j] + a.zi0;
            rin[j] = pin[j] && (unsigned)gz < (unsigned)a.D;
            const size_t off = rin[j] ? (size_t)gz * a.H * a.W + pyx[j] : 0;
            if constexpr (CP <= 8) {                         // one MX row of 8 channels per voxel (fp8: 8 bytes, fp4: 4), then the scale plane
                const uint8_t *q = (const uint8_t *)a.sx;
                const size_t rb = xdt == 3 ? 8 : 4;
                const uint8_t *row = q + ((size_t)n * S + off) * rb;
                rsc[j] = q[(size_t)a.N * S * rb + (size_t)n * S + off];
                raw0[j] = *(const unsigned *)row;
                if constexpr (CP == 8) raw1[j] = *(const unsigned *)(row + 4);     // (fp4: the next voxel's row or the scale plane's start, unused)
            }
        }
    };
    constexpr bool planes = PL;
    constexpr bool PFP = CP <= 4;                            // plane inputs are requested a tile ahead only where the registers allow it
    float pv[3][PFP ? CP : 1];                               // plane inputs (fp32, or fp16 widened): the values themselves
    auto plane_vals = [&](int tz, int j, float *dst) __attribute__((always_inline)) {       // position j's CP plane values of tile tz
        const int gz = 2 * tz - 1 + piz[j] + a.zi0;
        rin[j] = pin[j] && (unsigned)gz < (unsigned)a.D;
        const size_t off = rin[j] ? (size_t)gz * a.H * a.W + pyx[j] : 0;
#pragma unroll
        for (int k = 0; k < CP; k++) {
            float f = 0.f;
            if (k < Ci) { const size_t idx = ((size_t)n * Ci + k) * S + off; f = xdt == 2 ? __half2float(((const __half *)a.sx)[idx]) : ((const float *)a.sx)[idx]; }
            dst[k] = f;
        }
    };
    auto request_any = [&](int tz) __attribute__((always_inline)) {
        if (planes) {
            if constexpr (PFP) {
#pragma unroll
                for (int j = 0; j < 3; j++) plane_vals(tz, j, pv[j]);
            }
        } else request(tz);
    };
    request_any(tz0);
    const int lz = wave >> 1, ly0 = (wave & 1) * 4;
    const int p00 = (lz * HY + ly0 + (r >> 4)) * HX + (r & 15);
    __syncthreads();                                         // the affine table, the cleared amax word

    for (int tz = tz0; tz < tz1; tz++) {
        // ---- values of this tile: decode, GroupNorm + SiLU, amax ----
        float v[3][CP];
        float amax = 0.f;
#pragma unroll
        for (int j = 0; j < 3; j++) {
            float x[CP];
#pragma unroll
            for (int k = 0; k < CP; k++) x[k] = 0.f;
            if (planes) {
#pragma unroll
                for (int k = 0; k < CP; k++) { if constexpr (PFP) x[k] = pv[j][k]; }
                if constexpr (!PFP) plane_vals(tz, j, x);
            } else if (xdt == 3) {
                if constexpr (CP <= 8) {
                    const float sc = d_mx_scale(rsc[j]);
                    d_dec4_e4m3(raw0[j], x);
                    if constexpr (CP == 8) d_dec4_e4m3(raw1[j], x + 4);
#pragma unroll
                    for (int k = 0; k < CP; k++) x[k] *= sc;
                }
            } else {
                if constexpr (CP <= 8) {
                    const float sc = d_mx_scale(rsc[j]);
                    float d8[8];
                    d_dec8_e2m1(raw0[j], d8);
#pragma unroll
                    for (int k = 0; k < CP; k++) x[k] = d8[k] * sc;
                }
            }
            unsigned abj = ab_o;
            if (a.sns) { int s = (2 * tz - 1 + piz[j] + a.zi0 + a.szo) / a.szs; s = s < 0 ? 0 : s >= a.sns ? a.sns - 1 : s; abj += (unsigned)s * CP * 8; }     // the table of the position's plane
#pragma unroll
            for (int k = 0; k < CP; k++) {
                float val = x[k];
                if (a.sG) { const float2 ab = *(const float2 *)(lds + abj + k * 8); val = d_act_ab(val, ab.x, ab.y); }
                val = rin[j] && k < Ci ? val : 0.f;
                v[j][k] = val; amax = fmaxf(amax, fabsf(val));
            }
        }
        amax = fmaxf(amax, lane_xorf<1>(amax)); amax = fmaxf(amax, lane_xorf<2>(amax)); amax = fmaxf(amax, lane_xorf<4>(amax));
        amax = fmaxf(amax, lane_xorf<8>(amax)); amax = fmaxf(amax, lane_xorf<16>(amax)); amax = lane_pair_max(amax);
        if (lane == 0) atomicMax((unsigned *)(lds + am_o), __float_as_uint(amax));        // non-negative floats order as their bit patterns
        __syncthreads();
        const int e = d_mx_exp(__uint_as_float(*(const unsigned *)(lds + am_o)), MI_INVQ8);
        const int sb = e + 127;
#pragma unroll
        for (int j = 0; j < 3; j++) {
            const int pos = tid + 256 * j;
            if (pos < TT) {
#pragma unroll
                for (int k = 0; k < CP / 4; k++)
                    *(unsigned *)(lds + pos * CP + 4 * k) = d_enc4_e4m3(v[j][4 * k], v[j][4 * k + 1], v[j][4 * k + 2], v[j][4 * k + 3], e);
            }
        }
        __syncthreads();
        if (tid == 0) *(unsigned *)(lds + am_o) = 0u;        // (everyone has read it; the next tile's maxima come after this tile's last barrier)
        if (tz + 1 < tz1) request_any(tz + 1);       // the next tile's rows travel during this tile's MFMAs and epilogue

        // ---- MFMAs: wavefront -> (z, y half), voxel tile j -> rows 2 j, 2 j + 1 of that half, r -> (row, x) ----
        v16f acc[MT][NT];
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int j = 0; j < NT; j++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[m][j][i] = 0.f;
        auto tapoff = [](int tap) { tap = tap > 26 ? 26 : tap; return ((tap / 9) * HY + (tap / 3) % 3) * HX + tap % 3; };     // (taps past 26: zero weights)
        int p00v = p00, hv = h;                              // (opaque per tile: the fragment addresses are formed here, not kept in registers across the z tiles)
        asm volatile("" : "+v"(p00v), "+v"(hv));
        static_for<NP>([&](auto P) {
            constexpr int p = P;
            constexpr int LT = 16 / CP;                      // taps a lane supplies per K block
            int off[2][LT];
#pragma unroll
            for (int s = 0; s < 2; s++)
#pragma unroll
                for (int i = 0; i < LT; i++) off[s][i] = hv ? tapoff((2 * p + s) * TPK + LT + i) : tapoff((2 * p + s) * TPK + i);
#pragma unroll
            for (int j = 0; j < NT; j++) {
                const int pj = p00v + 2 * j * HX;
                v8i fb;
#pragma unroll
                for (int s = 0; s < 2; s++) {
                    if constexpr (CP == 4) {
#pragma unroll
                        for (int i = 0; i < 4; i++) fb[4 * s + i] = *(const int *)(lds + (pj + off[s][i]) * 4);
                    } else if constexpr (CP == 8) {
#pragma unroll
                        for (int i = 0; i < 2; i++) { const int2 w2 = *(const int2 *)(lds + (pj + off[s][i]) * 8); fb[4 * s + 2 * i] = w2.x; fb[4 * s + 2 * i + 1] = w2.y; }
                    } else {
                        const v4i w4 = *(const v4i *)(lds + (pj + off[s][0]) * 16);
                        fb[4 * s] = w4[0]; fb[4 * s + 1] = w4[1]; fb[4 * s + 2] = w4[2]; fb[4 * s + 3] = w4[3];
                    }
                }
#pragma unroll
                for (int m = 0; m < MT; m++) acc[m][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[p][m], fb, acc[m][j], 0, 0, 0, sa[p][m], 0, sb);
            }
        });
        __syncthreads();                                     // the staged tile has been read: the next tile may overwrite it, the epilogue use its scratch
        const unsigned tile = (unsigned)(((((size_t)n * a.ntz + tz) * a.nty + ty) * a.ntx + tx) * a.ncs + cs);       // the tile's place among the statistics partials
        // (uniform) more than 16 output channels: 32-wide output rows known at compile time; the tile inside the output and the statistics' planes:
        // no per-lane predicates. (The statistics scratch is next written two barriers on)
        // and no per-channel statistics records (their 32 sums per lane would cost the third workgroup per CU)
        if (a.Co > 16 && !a.stat_ch && 2 * tz + 2 <= a.Do && oy0 + 8 <= a.Ho && ox0 + 16 <= a.Wo && a.zs0 <= 2 * tz && a.zs1 >= 2 * tz + 2)
            conv_epilogue<MT, NT, OUT, false, false, true, true, true>(a, acc, lds, tile, n, cs, 2 * tz, oy0, ox0, lz, ly0, tid);
        else conv_epilogue<MT, NT, OUT, false>(a, acc, lds, tile, n, cs, 2 * tz, oy0, ox0, lz, ly0, tid);
    }
}

// ---- 9 .. 16 input channels (src/lp_f8fwd.cuh:447-563, weights src/lp_f8fwd.cu:72-92): the channels sit in slots of 16 and a tap row
// (kz, ky) is two K blocks, [kx0 | kx1] and [kx2 | 0], so a conv is 9 MFMAs per tile pair instead of 27 half-empty ones. A block spans two
// positions of one staged row, so the activation operand has one E8M0 scale per staged ROW: the 18 positions x - 1 .. x + 16 of a (z, y)
// line of the tile (amax by LDS atomicMax over the row; fmaxf semantics). Same tile, wavefront layout and epilogue as the stem kernel.
// Lane (r, h) of an MFMA supplies bytes 16 h .. 16 h + 15 of both blocks: h = 0 the rows of positions p (kx0) and p + 2 (kx2), h = 1 the row of
// p + 1 (kx1) and a zero row; its scale operand is the staged row's.
template <int MT, int OUT>
__global__ void __launch_bounds__(256, 2) conv3_p16_k(const conv_args a) {
    constexpr int NT = 2, HY = 10, HX = 18, NROW = 4 * HY, TT = NROW * HX, WTILE = 2048;
    extern __shared__ __align__(16) unsigned char lds[];
    // LDS: [staged tile TT x 16 bytes][zero row 16][row amax / scale words NROW][per channel (a, b): 16 x float2]
    constexpr unsigned z_o = TT * 16, ra_o = z_o + 16, ab_o = ra_o + NROW * 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, h = lane >> 5;
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
    const int ox0 = tx * 16, oy0 = ty * 8, oz0 = tz * 2;
    const int Ci = a.sCi;
    const size_t S = (size_t)a.D * a.H * a.W;
    if (tid < 4) *(unsigned *)(lds + z_o + tid * 4) = 0u;
    if (tid < NROW) *(unsigned *)(lds + ra_o + tid * 4) = 0u;
    for (int i = tid; i < 16 * (a.sns ? a.sns : 1); i += 256) {          // (slab-local statistics: one table per slab, back to back)
        const int k = i & 15, row = a.sns ? n * a.sns + (i >> 4) : n;
        float ga = 1.f, gb = 0.f;
        if (a.sG && k < Ci) { const int ng = row * a.sG + k / (Ci / a.sG); ga = a.srstd[ng] * a.sgam[k]; gb = fmaf(-a.smean[ng], ga, a.sbet[k]); }
        *(float2 *)(lds + ab_o + i * 8) = make_float2(ga, gb);
    }
    conv_epi_consts<MT, false>(a, lds, cs, tid);
    v8i fa[9][MT]; int sa[9][MT];
#pragma unroll
    for (int p = 0; p < 9; p++)
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const size_t t = (size_t)p * a.nmt_all + cs * MT + m;
            const v4i lo = *(const v4i *)(a.wq + t * WTILE + lane * 16), hi = *(const v4i *)(a.wq + t * WTILE + 1024 + lane * 16);
            fa[p][m] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            sa[p][m] = *(const int *)(a.wsc + (t * 64 + lane) * 4);
        }
    __syncthreads();
    // ---- stage: a thread owns positions tid, tid + 256, tid + 512; values stay in registers until the row's amax is known ----
    float v[3][16];
    const int xdt = a.sxdt;
#pragma unroll
    for (int j = 0; j < 3; j++) {
        const int pos = tid + 256 * j, row = pos / HX, ix = pos - row * HX;
        const int gz = oz0 - 1 + row / HY + a.zi0, gy = oy0 - 1 + row % HY, gx = ox0 - 1 + ix;
        const bool inb = pos < TT && (unsigned)gz < (unsigned)a.D && (unsigned)gy < (unsigned)a.H && (unsigned)gx < (unsigned)a.W;
        const size_t off = inb ? ((size_t)gz * a.H + gy) * a.W + gx : 0;
        float x[16];
#pragma unroll
        for (int k = 0; k < 16; k++) x[k] = 0.f;
        if (xdt == 3) {                                      // one MX-fp8 row of 16 channels per voxel, then the scale plane
            const uint8_t *q = (const uint8_t *)a.sx;
            const float s = d_mx_scale(q[(size_t)a.N * S * 16 + (size_t)n * S + off]);
            const uint4 w4 = *(const uint4 *)(q + ((size_t)n * S + off) * 16);
            d_dec4_e4m3(w4.x, x); d_dec4_e4m3(w4.y, x + 4); d_dec4_e4m3(w4.z, x + 8); d_dec4_e4m3(w4.w, x + 12);
#pragma unroll
            for (int k = 0; k < 16; k++) x[k] *= s;
        } else if (xdt == 4) {                               // one MX-fp4 row of 16 channels (8 bytes) per voxel
            const uint8_t *q = (const uint8_t *)a.sx;
            const float s = d_mx_scale(q[(size_t)a.N * S * 8 + (size_t)n * S + off]);
            const uint2 w2 = *(const uint2 *)(q + ((size_t)n * S + off) * 8);
            d_dec8_e2m1(w2.x, x); d_dec8_e2m1(w2.y, x + 8);
#pragma unroll
            for (int k = 0; k < 16; k++) x[k] *= s;
        } else {
#pragma unroll
            for (int k = 0; k < 16; k++)
                if (k < Ci) {
                    const size_t idx = ((size_t)n * Ci + k) * S + off;
                    x[k] = xdt == 2 ? __half2float(((const __half *)a.sx)[idx]) : ((const float *)a.sx)[idx];
                }
        }
        float am = 0.f;
        unsigned abj = ab_o;
        if (a.sns) { int s = (gz + a.szo) / a.szs; s = s < 0 ? 0 : s >= a.sns ? a.sns - 1 : s; abj += (unsigned)s * 128; }     // the table of the position's plane
#pragma unroll
        for (int k = 0; k < 16; k++) {
            float val = x[k];
            if (a.sG) { const float2 ab = *(const float2 *)(lds + abj + k * 8); val = d_act_ab(val, ab.x, ab.y); }
            val = inb && k < Ci ? val : 0.f;
            v[j][k] = val; am = fmaxf(am, fabsf(val));
        }
        if (pos < TT && am != 0.f) atomicMax((unsigned *)(lds + ra_o + row * 4), __float_as_uint(am));
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 3; j++) {
        const int pos = tid + 256 * j, row = pos / HX;
        if (pos < TT) {
            const int e = d_mx_exp(__uint_as_float(*(const unsigned *)(lds + ra_o + row * 4)), MI_INVQ8);
            uint4 o;
            o.x = d_enc4_e4m3(v[j][0], v[j][1], v[j][2], v[j][3], e); o.y = d_enc4_e4m3(v[j][4], v[j][5], v[j][6], v[j][7], e);
            o.z = d_enc4_e4m3(v[j][8], v[j][9], v[j][10], v[j][11], e); o.w = d_enc4_e4m3(v[j][12], v[j][13], v[j][14], v[j][15], e);
            *(uint4 *)(lds + pos * 16) = o;
        }
    }
    __syncthreads();                                         // every position is encoded with its row's amax ...
    if (tid < NROW) { unsigned *p = (unsigned *)(lds + ra_o + tid * 4); *p = (unsigned)(d_mx_exp(__uint_as_float(*p), MI_INVQ8) + 127); }
    __syncthreads();                                         // ... which then becomes the row's scale word
    const int lz = wave >> 1, ly0 = (wave & 1) * 4;
    const int row00 = lz * HY + ly0 + (r >> 4), p00 = row00 * HX + (r & 15);
    v16f acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int j = 0; j < NT; j++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[m][j][i] = 0.f;
    static_for<9>([&](auto R) {
        constexpr int tr = R, kz = tr / 3, ky = tr % 3;
#pragma unroll
        for (int j = 0; j < NT; j++) {
            const int row = row00 + 2 * j + kz * HY + ky, p = p00 + (2 * j + kz * HY + ky) * HX;
            const v4i lo = *(const v4i *)(lds + (p + h) * 16);
            const v4i hi = *(const v4i *)(lds + (h ? z_o : (unsigned)(p + 2) * 16u));
            const v8i fb = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
            const int sb = *(const int *)(lds + ra_o + row * 4);
#pragma unroll
            for (int m = 0; m < MT; m++) acc[m][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[tr][m], fb, acc[m][j], 0, 0, 0, sa[tr][m], 0, sb);
        }
    });
    __syncthreads();
    conv_epilogue<MT, NT, OUT, false>(a, acc, lds, tile, n, cs, oz0, oy0, ox0, lz, ly0, tid);
}
// its weights: tap row r = (kz, ky), block 2 r = [kx0 | kx1], block 2 r + 1 = [kx2 | 0], 16 channels per slot (src/lp_f8fwd.cu:72-92)
__global__ void __launch_bounds__(128) prep_wp16_k(const float *__restrict__ w, uint8_t *__restrict__ wq, unsigned *__restrict__ wsc, int Co, int Ci, int nmt_all) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x, Cop = nmt_all * 32;
    if (i >= 9 * Cop) return;
    const int cop = i % Cop, p = i / Cop, m = cop >> 5, r = cop & 31, cw = (cop & ~31) + mi_row_chan(r);      // row r of the tile carries output channel cw
    uint8_t *tile = wq + ((size_t)p * nmt_all + m) * 2048;
    unsigned *tsc = wsc + ((size_t)p * nmt_all + m) * 64;
#pragma unroll
    for (int side = 0; side < 2; side++) {
        float v[32]; float amax = 0.f;
#pragma unroll
        for (int k = 0; k < 32; k++) {
            const int kx = 2 * side + (k >> 4), ci = k & 15;
            v[k] = (kx < 3 && cw < Co && ci < Ci) ? w[((size_t)cw * Ci + ci) * 27 + p * 3 + kx] : 0.f;
            amax = fmaxf(amax, fabsf(v[k]));
        }
        const int e = d_mx_exp(amax, MI_INVQ8);
        const float mult = d_exp2i(-e);
        unsigned c[8];
#pragma unroll
        for (int j = 0; j < 8; j++) c[j] = d_enc_e4m3x4(v[4 * j] * mult, v[4 * j + 1] * mult, v[4 * j + 2] * mult, v[4 * j + 3] * mult);
        *(uint4 *)(tile + ((size_t)(side * 64 + r) * 16)) = make_uint4(c[0], c[1], c[2], c[3]);
        *(uint4 *)(tile + ((size_t)(side * 64 + r + 32) * 16)) = make_uint4(c[4], c[5], c[6], c[7]);
        tsc[r + 32 * side] = (unsigned)(e + 127);
    }
}

// weights: fp32 w[co][ci][27] -> per (block pair, 32-row channel tile) fragment-ordered e4m3 codes + one scale word per lane
// (src/lp_f8fwd.cuh:156-177): block kb, k -> tap kb * TPK + k / CP, channel k % CP; zeros past the taps, the channels and the rows
template <int CP>
__global__ void __launch_bounds__(128) prep_ws_k(const float *__restrict__ w, uint8_t *__restrict__ wq, unsigned *__restrict__ wsc, int Co, int Ci, int nmt_all, int np) {
    constexpr int TPK = 32 / CP, NKB = (27 + TPK - 1) / TPK;
    const int i = blockIdx.x * blockDim.x + threadIdx.x, Cop = nmt_all * 32;
    if (i >= np * Cop) return;
    const int cop = i % Cop, p = i / Cop, m = cop >> 5, r = cop & 31, cw = (cop & ~31) + mi_row_chan(r);      // row r of the tile carries output channel cw
    uint8_t *tile = wq + ((size_t)p * nmt_all + m) * 2048;
    unsigned *tsc = wsc + ((size_t)p * nmt_all + m) * 64;
#pragma unroll
    for (int side = 0; side < 2; side++) {
        const int kb = 2 * p + side;
        float v[32]; float amax = 0.f;
#pragma unroll
        for (int k = 0; k < 32; k++) {
            const int tap = kb * TPK + k / CP, ci = k % CP;
            v[k] = (kb < NKB && cw < Co && ci < Ci && tap < 27) ? w[((size_t)cw * Ci + ci) * 27 + tap] : 0.f;
            amax = fmaxf(amax, fabsf(v[k]));
        }
        const int e = d_mx_exp(amax, MI_INVQ8);
        const float mult = d_exp2i(-e);
        unsigned c[8];
#pragma unroll
        for (int j = 0; j < 8; j++) c[j] = d_enc_e4m3x4(v[4 * j] * mult, v[4 * j + 1] * mult, v[4 * j + 2] * mult, v[4 * j + 3] * mult);
        *(uint4 *)(tile + ((size_t)(side * 64 + r) * 16)) = make_uint4(c[0], c[1], c[2], c[3]);            // lane (r, 0): bytes 0-15 of the block
        *(uint4 *)(tile + ((size_t)(side * 64 + r + 32) * 16)) = make_uint4(c[4], c[5], c[6], c[7]);       // lane (r, 1): bytes 16-31
        tsc[r + 32 * side] = (unsigned)(e + 127);
    }
}

void conv3_stem_prep(int CP, const float *w, uint8_t *wq, uint8_t *wsc, int Co, int Ci, int nmt_all, int np) {
    const unsigned nb = nblk_((size_t)np * nmt_all * 32, 128);
    if (CP == 0) { prep_wp16_k<<<nb, 128>>>(w, wq, (unsigned *)wsc, Co, Ci, nmt_all); MICK(); return; }       // (CP 0: the two-taps-per-block layout)
    if (CP == 4) prep_ws_k<4><<<nb, 128>>>(w, wq, (unsigned *)wsc, Co, Ci, nmt_all, np);
    else if (CP == 8) prep_ws_k<8><<<nb, 128>>>(w, wq, (unsigned *)wsc, Co, Ci, nmt_all, np);
    else prep_ws_k<16><<<nb, 128>>>(w, wq, (unsigned *)wsc, Co, Ci, nmt_all, np);
    MICK();
}

template <int CP, int MT, int OUT>
static void launch_stem(const conv_args &a, size_t smem) {
    const unsigned per = (a.ngrp + 7u) / 8u;
    if (a.sxdt < 3) conv3_stem_k<CP, MT, OUT, true><<<per * 8u, 256, smem>>>(a);
    else if constexpr (CP <= 8) conv3_stem_k<CP, MT, OUT, false><<<per * 8u, 256, smem>>>(a);
    else mi_die("conv3 stem: 16-channel rows are fp32 planes");
    MICK();
    snprintf(g_last_kernel, sizeof g_last_kernel, "conv3_stem_k<CP %d, MT %d, out %d> tiles %u", CP, MT, OUT, a.ntiles);
}
template <int CP, int MT>
static void launch_stem_out(int out, const conv_args &a, size_t smem) {
    if (out == 8) launch_stem<CP, MT, 8>(a, smem); else if (out == 4) launch_stem<CP, MT, 4>(a, smem); else launch_stem<CP, MT, 0>(a, smem);
}
template <int MT, int OUT>
static void launch_p16(const conv_args &a, size_t smem) {
    const unsigned per = (a.ntiles + 7u) / 8u;
    conv3_p16_k<MT, OUT><<<per * 8u, 256, smem>>>(a);
    MICK();
    snprintf(g_last_kernel, sizeof g_last_kernel, "conv3_p16_k<MT %d, out %d> tiles %u", MT, OUT, a.ntiles);
}
void conv3_stem_launch(int CP, int MT, int out, const conv_args &a, size_t smem) {
    if (CP == 0) {
        if (MT == 1) { if (out == 8) launch_p16<1, 8>(a, smem); else if (out == 4) launch_p16<1, 4>(a, smem); else launch_p16<1, 0>(a, smem); }
        else mi_die("conv3 p16: no kernel for MT %d", MT);
        return;
    }
    switch (CP * 10 + MT) {
    case 41: launch_stem_out<4, 1>(out, a, smem); break;
    case 42: launch_stem_out<4, 2>(out, a, smem); break;
    case 81: launch_stem_out<8, 1>(out, a, smem); break;
    case 82: launch_stem_out<8, 2>(out, a, smem); break;
    case 161: launch_stem_out<16, 1>(out, a, smem); break;
    default: mi_die("conv3 stem: no kernel for CP %d MT %d", CP, MT);
    }
}
