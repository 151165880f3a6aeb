// The row kernel for ONE input block (<= 32 channels in, 17 .. 32 out; the 32 -> 32 convs of a U-Net's level 0): runs of 32 voxels along x as in
// conv3_row.hpp (an input fragment read from LDS once serves the three ky taps: 0.5 fragment reads per MFMA, no bank conflicts), plus what one
// block allows:
//   * the weight fragments of the block stay with the wavefront for the whole persistent workgroup: the 9 pairs of tap classes 0 .. 2 in registers
//     (72 of them; the E8M0 bytes of four pairs share a register and the MFMA's op_sel picks its byte), the 6 pairs of classes 3 and 4 in 9 KiB of
//     LDS, read one class before their turn. The K loop issues no global loads but the next halo's copies. (All 15 pairs in registers leave the
//     epilogue a dozen registers short, and a spilled register's reload waits for every copy in flight.)
//   * the epilogue (as long as the tile's MFMAs here) runs in the shadow of MFMAs: the workgroup's eight wavefronts form two groups of four, one
//     wavefront per SIMD each, group 1 owning rows 4 .. 7 of the tile and running HALF A TILE BEHIND group 0. While one of a SIMD's two wavefronts
//     multiplies, the other converts and stores. The groups meet at one workgroup barrier per phase (two per tile); nothing else synchronises
//     them: the epilogue keeps its statistics per wavefront (no LDS scratch, no barrier inside), and every wavefront copies its share of the
//     next tile's halo from inside its own K loop, one copy round per tap class.
//   * the halo is a RING of z planes: a workgroup walks its tiles along z (the tiles in column order, an XCD owning a contiguous range and each of
//     its workgroups a contiguous piece of it), so a tile shares two of its six halo planes with the tile before it and copies four: 22 copy
//     groups of 64 positions instead of 32, a third of the K loop's copy requests and of the halo's cache lines gone. Ten slots of one plane
//     (340 positions padded to 352, so that two planes are 11 groups): the six being read and the four landing. When the next tile starts a new
//     column the ring is of no use: both groups take one more phase, in which group 0 copies the tile's six planes and waits for them.
// Barrier 0 ends the set-up. Group 0 runs its K loop K(t) between barriers 2t and 2t + 1 and its epilogue E(t) between 2t + 1 and 2t + 2; group 1
// runs K(t) between 2t + 1 and 2t + 2 and E(t) between 2t + 2 and 2t + 3 (a column start adds one barrier for both): every wavefront passes the
// same barriers. Tile t's planes sit in slots s .. s + 5, read from barrier 2t to 2t + 2; the four new planes of tile t + 1 go to slots s + 6 ..
// s + 9 = s - 4 .. s - 1, last read (tile t - 1, group 1) before barrier 2t; they are requested after barrier 2t (group 0) / 2t + 1 (group 1), and
// each wavefront waits for its own before the barrier that ends its K loop (2t + 1 / 2t + 2), ahead of the first reader after barrier 2t + 2.
// Measured on the same box (32 -> 32, N 2 x 128^3), before the ring: MX-fp8 0.135 - 0.139 against 0.146 - 0.150 ms on the small-channel kernel,
// MX-fp4 0.091 - 0.094 against 0.104 - 0.105 ms; the ring takes another 3 - 8 % inside a U-Net forward (0.108 - 0.110 against 0.111 - 0.118 ms).
// Clock stamps of one workgroup: a K loop alone on its SIMD runs its 60 MFMAs in 4.0 K cycles (96 % of the matrix pipe), with three copy rounds
// inside 5.5 - 6.1 K (each round is about 45 vector and 35 scalar instructions that the wavefront issues between its MFMAs while the SIMD's other
// wavefront keeps the vector ALU busy with its epilogue), the epilogue 3.6 - 3.9 K: the K phase is what a tile costs, and the epilogue's wavefront
// idles a third of its phase. What was tried and lost: copies issued from the epilogue phase instead - all of them, or the last round of three,
// in a burst at the phase's start or spread between the accumulator tiles (the K loop drops to 4.1 - 4.4 K, but each round adds 1 K cycles to
// the epilogue and the kernel is 3 - 6 % slower; a per-lane select between a tensor pointer and the constant page must not become a vector
// load of the pointer from the argument block there, whose wait also waits for the copies); whole 32-byte rows per lane pair (no gain); class
// 2's weights in LDS as well (no gain).
#pragma once

#ifdef DBG_TIMING
#define DBG_R1(i) do { if (blockIdx.x == 8 && it == 2 && (threadIdx.x & 255) == 0) g_dbg[(threadIdx.x >> 8) * 32 + (i)] = (long long)__builtin_amdgcn_s_memtime(); } while (0)
#else
#define DBG_R1(i) do { } while (0)
#endif
template <int FMT, int OUT, bool EPI>
__global__ void __launch_bounds__(512, 1) conv3_row1_k(const conv_args a) {
    constexpr int NT = 4, TZ = 4, TY = 8, TX = 32, NW = 8;
    constexpr int HZ = TZ + 2, HY = TY + 2, HX = TX + 2, NH = fmt_t<FMT>::NH, WTILE = fmt_t<FMT>::WTILE;
    // the halo lives in a RING of z planes: a workgroup walks its tiles along z, so a tile shares two of its six planes with the tile before it
    // and copies only the four new ones. A slot holds one plane, padded from HY HX = 340 to 352 positions so that two planes are exactly 11 copy
    // groups of 64 positions; ten slots: the six being read and the four landing
    constexpr int PP = 352, NS = 10, TTP = NS * PP, NGR = TTP / 64;
    constexpr int GN = TZ * PP / 64, GF = (HZ * PP + 63) / 64;  // copy groups of a tile that continues its column (22), of a column's first tile (33)
    static_assert(PP >= HY * HX && (2 * PP) % 64 == 0 && TTP % 64 == 0 && GN == 2 * NW + 6, "two full copy rounds and one of six groups");
    constexpr int NC = 5, NPB = 3 * NC;                         // tap classes; weight pairs of the block
    extern __shared__ __align__(16) unsigned char lds[];
    const unsigned lds0 = (unsigned)(size_t)lds;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 31, h = lane >> 5;
    const int grp = wave >> 2, lz = wave & 3, ly0 = grp * NT;   // group 0: wavefronts 0 .. 3 (one per SIMD), rows 0 .. 3 of the tile; group 1: rows 4 .. 7
    // the lane's 16-byte row half and scale word of position (ly0, r) of a plane: rows [half][ring position][16 B], then one scale word per position
    const unsigned ab0 = ((NH == 2 ? h * TTP : 0) + ly0 * HX + r) * 16, sb0 = NH * TTP * 16 + (ly0 * HX + r) * 4;
    const size_t Sin = (size_t)a.D * a.H * a.W;

    // XCD-aware persistent walk: the tiles in column order (z fastest), an XCD owns a contiguous range of them and each of its workgroups a
    // contiguous piece of that range, so a workgroup's consecutive tiles are z neighbours of one (sample, y, x) column until the column ends
    // Two channel tiles (33 .. 64 output channels): a workgroup keeps ONE of them for its whole walk, and neighbouring workgroups of an XCD
    // walk the same tiles in the other slice (the halo's second read finds the L2)
    const unsigned ncs = (unsigned)a.ncs, nsp = a.ntiles / ncs;                      // channel slices; spatial tiles
    const int cs = __builtin_amdgcn_readfirstlane((int)((blockIdx.x >> 3) % ncs));
    const unsigned per = (nsp + 7u) / 8u, wg_per_xcd = (gridDim.x >> 3) / ncs, xcd = blockIdx.x & 7u, wix = (blockIdx.x >> 3) / ncs;
    const unsigned cpw = (per + wg_per_xcd - 1u) / wg_per_xcd, k0 = xcd * per + wix * cpw;
    const unsigned kx_ = xcd * per + per, ky_ = k0 + cpw, k1 = min(min(kx_, ky_), nsp);
    struct tile_t { unsigned tile, col; int n, oz0, oy0, ox0; bool ok; };
    auto decode = [&](unsigned it) {
        tile_t t; const unsigned k = k0 + it;
        t.ok = k < k1;
        const unsigned kk = t.ok ? k : 0u;
        t.col = kk / (unsigned)a.ntz;
        const int tz = (int)(kk - t.col * (unsigned)a.ntz);
        int cc = (int)t.col;
        const int tx = cc % a.ntx; cc /= a.ntx;
        const int ty = cc % a.nty; t.n = cc / a.nty;
        t.tile = (unsigned)(((t.n * a.ntz + tz) * a.nty + ty) * a.ntx + tx);        // (the tile's number in x-fastest order: its statistics record)
        t.ox0 = tx * TX; t.oy0 = ty * TY; t.oz0 = tz * TZ;
        return t;
    };
    tile_t cur = decode(0);
    if (!cur.ok) return;                                        // (uniform over the workgroup)

    // copy group g (64 positions) of a run of planes that starts at plane z0 of tile t's column, into ring group rg: the two row halves back to
    // back and the scale bytes; positions outside the volume or in a plane's padding read the constant page. No branch: `on` false reads the
    // constant page (into slots nobody reads)
    auto request = [&](const tile_t &t, int z0, int g, unsigned rg, bool on) {
        const int y0 = t.oy0 - 1, x0 = t.ox0 - 1;
        int ln = lane;
        asm volatile("" : "+v"(ln));                            // (opaque: the coordinates are formed per request, not kept in registers across the K loop)
        const int pos = g * 64 + ln, pz = pos / PP, rem = pos - pz * PP, py = rem / HX, px = rem - py * HX;
        const int gz = z0 + pz, gy = y0 + py, gx = x0 + px;
        const bool in = on & (rem < HY * HX) & ((unsigned)gz < (unsigned)a.D) & ((unsigned)gy < (unsigned)a.H) & ((unsigned)gx < (unsigned)a.W);
        const int sp = (gz * a.H + gy) * a.W + gx;              // (garbage where !in: unused)
        const size_t vox = (size_t)t.n * a.nbs[0] * Sin + (size_t)(in ? sp : 0);
        const uint8_t *row = in ? a.xq[0] + vox * (16 * NH) : a.zpage, *sc = in ? a.xsc[0] + vox : a.zpage + 64;
        dma16(row, lds0 + rg * 1024u);
        if constexpr (NH == 2) dma16(row + 16, lds0 + (unsigned)TTP * 16u + rg * 1024u);
        dma1(sc, lds0 + (unsigned)(NH * TTP * 16) + rg * 256u);
    };
    // all six planes of tile t into slots s .. s + 5 (s even: a whole number of groups), by nw wavefronts of which this is number wi
    auto load_column_start = [&](const tile_t &t, int s, int nw, int wi) {
        const unsigned g0 = (unsigned)(s * (PP / 32)) / 2u;
        for (int g = wi; g < GF; g += nw) { unsigned rg = g0 + (unsigned)g; rg -= rg >= (unsigned)NGR ? (unsigned)NGR : 0u; request(t, t.oz0 - 1 + a.zi0, g, rg, true); }
    };
    int s0 = 0;                                                 // ring slot of the current tile's first plane (even)
    conv_epi_consts<1, EPI>(a, lds, cs, tid);
    load_column_start(cur, 0, NW, wave);

    // the block's weights: pair c 3 + ky of the prepared order (class c, ky), lane-ordered codes; the scale bytes of four pairs per register.
    // Classes 0 .. 2 stay in registers. Classes 3 and 4 wait in LDS (3 x 2 KiB and, the second unit of class 4's pairs being the zero padding
    // unit, 3 x 1 KiB) and are read one class before their turn: 36 registers that are then free while the epilogue runs, which is where the
    // registers run out (a spilled register's reload waits for every copy in flight)
    constexpr int NPR = 3 * (NC - 2);
    v4i wlo[NPR], whi[FMT == 8 ? NPR : 1]; int wsb[(NPB + 3) / 4];
    const unsigned w3_o = a.red_o, w4_o = a.red_o + 3 * 2048;   // (the statistics scratch: this kernel's epilogue keeps its sums per wavefront)
    {
        const size_t wq_ps = (size_t)a.nmt_all * WTILE, wsc_ps = (size_t)a.nmt_all * 256;
        int sw[NPB];
#pragma unroll
        for (int p = 0; p < NPB; p++) {
            const uint8_t *wp = a.wq + (size_t)p * wq_ps + (size_t)cs * WTILE + lane * 16;
            if (p < NPR) { wlo[p] = *(const v4i *)wp; if (FMT == 8) whi[p] = *(const v4i *)(wp + 1024); }
            else if (p < NPR + 3) {                             // class 3: wavefronts 0 .. 5 copy its six 1 KiB pieces (uniform per wavefront)
                if (wave == 2 * (p - NPR)) dma16(wp, lds0 + w3_o + (unsigned)(p - NPR) * 2048u);
                if (FMT == 8 && wave == 2 * (p - NPR) + 1) dma16(wp + 1024, lds0 + w3_o + (unsigned)(p - NPR) * 2048u + 1024u);
            } else if (wave == p - NPR - 3) dma16(wp, lds0 + w4_o + (unsigned)(p - NPR - 3) * 1024u);
            sw[p] = *(const int *)(a.wsc + (size_t)p * wsc_ps + (size_t)cs * 256 + lane * 4);
        }
#pragma unroll
        for (int q = 0; q < (NPB + 3) / 4; q++) {
            wsb[q] = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) if (4 * q + k < NPB) wsb[q] |= (sw[4 * q + k] & 255) << (8 * k);
        }
    }
    wait_vm<0>();
    __syncthreads();                                            // barrier 0: the first halo and the epilogue's constants are in LDS
    if (grp) __syncthreads();                                   // group 1 starts half a tile later (barrier 1)

    for (unsigned it = 0;; it++) {
        const tile_t nxt = decode(it + 1);
        const bool cont = nxt.ok && nxt.col == cur.col;         // the next tile is this one's z neighbour: its first two planes are this tile's last two
        // the three planes wavefront lz reads sit in slots (s0 + lz + kz) mod NS; class c reads unit A = (plane kzA, kx kxA) and unit B beside it:
        // classes 0 .. 2 (plane c; kx 0 | 1), class 3 (kx 2 of planes 0 | 1), class 4 (kx 2 of plane 2 | the zero unit, which re-reads unit A).
        // e4m3 lanes read their row half of both units; e2m1 lanes and the scale words read the unit of the lane's half: five bases per kind
        unsigned abt[3], sbt[3];
#pragma unroll
        for (int k = 0; k < 3; k++) {
            int sl = s0 + lz + k; sl -= sl >= NS ? NS : 0;
            abt[k] = ab0 + (unsigned)(sl * PP * 16); sbt[k] = sb0 + (unsigned)(sl * PP * 4);
        }
        unsigned abx[NC], sbx[NC];
#pragma unroll
        for (int k = 0; k < 3; k++) { sbx[k] = sbt[k] + (h ? 4u : 0u); abx[k] = abt[k] + (h ? 16u : 0u); }
        sbx[3] = h ? sbt[1] : sbt[0]; sbx[4] = sbt[2];
        abx[3] = h ? abt[1] : abt[0]; abx[4] = abt[2];          // (e4m3 does not read abx: dead there)
        struct frag { v4i lo, hi; int sb; };
        auto fetch = [&](auto C, auto S) {
            constexpr int c = decltype(C)::value, s = decltype(S)::value;
            constexpr int kzA = c < 3 ? c : c == 3 ? 0 : 2, kzB = c == 3 ? 1 : kzA, kxA = c < 3 ? 0 : 2, kxB = c < 3 ? 1 : 2;
            frag f;
            if constexpr (FMT == 8) { f.lo = *(const v4i *)(lds + abt[kzA] + (s * HX + kxA) * 16); f.hi = *(const v4i *)(lds + abt[kzB] + (s * HX + kxB) * 16); }
            else { f.lo = *(const v4i *)(lds + abx[c] + (s * HX + kxA) * 16); f.hi = (v4i){0, 0, 0, 0}; }
            f.sb = *(const int *)(lds + sbx[c] + (s * HX + kxA) * 4);
            return f;
        };
        // the next tile's four new planes go to slots s0 + 6 .. s0 + 9 (free since group 1 left tile it - 1): 22 copy groups, requested from inside
        // the K loop, rounds 0 and 1 one group per wavefront, round 2 the last six (wavefronts 6 and 7 repeat groups 16 and 17: the same bytes to the
        // same place, and the K loop stays free of branches). A next tile that starts a column gets nothing here (`on` false: the constant page, into
        // the same free slots)
        int kslot = s0 + HZ; kslot -= kslot >= NS ? NS : 0;
        const unsigned glk = (unsigned)(kslot * (PP / 32)) / 2u;
        // ---- K loop: NC x (NT + 2) row visits as one basic block; visit (c, s) requests the fragment two visits ahead and multiplies its own by
        // the ky weights of the rows it reaches (j = s - ky); the next tile's copy rounds are issued at fixed visits ----
        DBG_R1(0);
        v16f acc[1][NT];
        constexpr int NR = NT + 2, NV = NC * NR, PF = 2;
        {
            frag fr[PF + 1];
            v4i w3lo[3], w3hi[3], w4[3];                        // the weight fragments of classes 3 and 4, read from LDS one class ahead
            static_for<PF>([&](auto V) { constexpr int v = decltype(V)::value; fr[v] = fetch(std::integral_constant<int, v / NR>{}, std::integral_constant<int, v % NR>{}); });
            static_for<NV>([&](auto V) {
                constexpr int v = decltype(V)::value, c = v / NR, s = v % NR, set = v % (PF + 1);
                if constexpr (v + PF < NV) fr[(v + PF) % (PF + 1)] = fetch(std::integral_constant<int, (v + PF) / NR>{}, std::integral_constant<int, (v + PF) % NR>{});
                if constexpr (s == 1 && c < 3) {
                    const int g = c < 2 ? NW * c + wave : 2 * NW + (wave < 6 ? wave : wave - 6);
                    unsigned rg = glk + (unsigned)g; rg -= rg >= (unsigned)NGR ? (unsigned)NGR : 0u;
                    request(nxt, nxt.oz0 + 1 + a.zi0, g, rg, cont);
                }
                if constexpr (c == NC - 3 && s == 2) {
#pragma unroll
                    for (int k = 0; k < 3; k++) { w3lo[k] = *(const v4i *)(lds + w3_o + k * 2048 + lane * 16); if (FMT == 8) w3hi[k] = *(const v4i *)(lds + w3_o + k * 2048 + 1024 + lane * 16); }
                }
                if constexpr (c == NC - 2 && s == 2) {
#pragma unroll
                    for (int k = 0; k < 3; k++) w4[k] = *(const v4i *)(lds + w4_o + k * 1024 + lane * 16);
                }
                const v8i fb = FMT == 8 ? (v8i){fr[set].lo[0], fr[set].lo[1], fr[set].lo[2], fr[set].lo[3], fr[set].hi[0], fr[set].hi[1], fr[set].hi[2], fr[set].hi[3]}
                                        : (v8i){fr[set].lo[0], fr[set].lo[1], fr[set].lo[2], fr[set].lo[3], 0, 0, 0, 0};
                static_for<3>([&](auto KY) {
                    constexpr int ky = decltype(KY)::value, j = s - ky, p = c * 3 + ky;
                    if constexpr (j >= 0 && j < NT) {
                        const v16f c0 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                        // (row j's first product is class 0's: visit (0, j + ky) with ky = 0 comes first for j = s)
                        v8i wa;
                        if constexpr (p < NPR) wa = FMT == 8 ? (v8i){wlo[p][0], wlo[p][1], wlo[p][2], wlo[p][3], whi[FMT == 8 ? p : 0][0], whi[FMT == 8 ? p : 0][1], whi[FMT == 8 ? p : 0][2], whi[FMT == 8 ? p : 0][3]}
                                                             : (v8i){wlo[p][0], wlo[p][1], wlo[p][2], wlo[p][3], 0, 0, 0, 0};
                        else if constexpr (p < NPR + 3) wa = FMT == 8 ? (v8i){w3lo[p - NPR][0], w3lo[p - NPR][1], w3lo[p - NPR][2], w3lo[p - NPR][3], w3hi[p - NPR][0], w3hi[p - NPR][1], w3hi[p - NPR][2], w3hi[p - NPR][3]}
                                                                          : (v8i){w3lo[p - NPR][0], w3lo[p - NPR][1], w3lo[p - NPR][2], w3lo[p - NPR][3], 0, 0, 0, 0};
                        else wa = (v8i){w4[p - NPR - 3][0], w4[p - NPR - 3][1], w4[p - NPR - 3][2], w4[p - NPR - 3][3], 0, 0, 0, 0};
                        acc[0][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wa, fb, (c == 0 && ky == 0) ? c0 : acc[0][j], FMT == 8 ? 0 : 4, FMT == 8 ? 0 : 4,
                                                                                    p % 4, wsb[p / 4], 0, fr[set].sb);
                    }
                });
                static_for<3>([&](auto KY) { constexpr int j = s - decltype(KY)::value; if constexpr (j >= 0 && j < NT) row_pin(acc[0][j]); });
                __builtin_amdgcn_sched_barrier(0);
            });
        }
        DBG_R1(1);
        wait_vm<0>();                                           // this wavefront's copies of the next tile's planes have landed
        DBG_R1(2);
        __syncthreads();                                        // end of this group's K phase (barrier 2 it + 1 for group 0, 2 it + 2 for group 1)
        DBG_R1(3);
        if (cur.oz0 + TZ <= a.Do && cur.oy0 + TY <= a.Ho && cur.ox0 + TX <= a.Wo && a.zs0 <= cur.oz0 && a.zs1 >= cur.oz0 + TZ)      // (uniform)
            conv_epilogue<1, NT, OUT, EPI, false, true, true, true, NW, true, true>(a, acc, lds, cur.tile, cur.n, cs, cur.oz0, cur.oy0, cur.ox0, lz, ly0, tid);
        else conv_epilogue<1, NT, OUT, EPI, false, true, false, true, NW, true, true>(a, acc, lds, cur.tile, cur.n, cs, cur.oz0, cur.oy0, cur.ox0, lz, ly0, tid);
        DBG_R1(4);
        __syncthreads();                                        // end of this group's epilogue phase (barrier 2 it + 2 / 2 it + 3)
        DBG_R1(5);
        if (!nxt.ok) break;
        if (cont) s0 = s0 + TZ >= NS ? s0 + TZ - NS : s0 + TZ;
        else {
            // a new column: nothing in the ring is of use. One more phase for both groups: group 0, done with its epilogue while group 1 (which
            // reads no halo in its own) finishes, copies all six planes of the next tile and waits for them; group 1 arrives a phase later as ever
            s0 = 0;
            if (!grp) { load_column_start(nxt, 0, NW / 2, lz); wait_vm<0>(); }
            __syncthreads();
        }
        cur = nxt;
    }
    if (!grp) __syncthreads();                                  // group 0 waits out group 1's last epilogue phase: every wavefront has passed the same barriers
}

template <int FMT, int OUT, bool EPI>
static void launch_row1(const conv_args &a, size_t smem) {
    static bool attr[8]; static int ncu[8];
    int d = 0; MIRT(hipGetDevice(&d)); d &= 7;
    if (!attr[d]) {
        MIRT(hipFuncSetAttribute((const void *)conv3_row1_k<FMT, OUT, EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        hipDeviceProp_t pr; MIRT(hipGetDeviceProperties(&pr, d));
        ncu[d] = pr.multiProcessorCount > 8 ? pr.multiProcessorCount & ~7 : 8;
        attr[d] = true;
    }
    const unsigned ncs = (unsigned)a.ncs, per = (a.ntiles / ncs + 7u) / 8u;            // spatial tiles per XCD; one persistent workgroup per CU, a multiple of 8 x slices in all
    const unsigned cap0 = (unsigned)ncu[d] / (8u * ncs) * (8u * ncs), cap = cap0 ? cap0 : 8u * ncs, nwg = per * 8u * ncs < cap ? per * 8u * ncs : cap;      // (fewer CUs than 8 x slices: the walk works for any grid)
    conv3_row1_k<FMT, OUT, EPI><<<nwg, 512, smem>>>(a);
    MICK();
    snprintf(g_last_kernel, sizeof g_last_kernel, "conv3_row1_k<fmt %d, out %d, epi %d> tiles %u%s wgs %u", FMT, OUT, (int)EPI, a.ntiles, ncs == 2 ? " (two channel slices)" : ncs > 2 ? " (channel slices)" : "", nwg);
}
