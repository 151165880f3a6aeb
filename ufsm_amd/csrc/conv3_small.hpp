// The small-channel 3x3x3 stride-1 kernel: one channel tile and one input block (<= 32 channels in and out), TZ x 8 x 16 voxels per tile.
//
// With 32 output channels every input fragment feeds a single MFMA (two 16-byte LDS reads and a scale word per lane and MFMA), and the
// epilogue is as long as half the MFMAs, so everything else has to get out of the way:
//   * workgroups are persistent (two per CU) and walk their tiles XCD by XCD; the 14 pairs of weight fragments are loaded into registers
//     once per workgroup, so the K loop has no weight ring, no pair table and no barriers, and the taps' halo offsets are instruction immediates;
//   * the halo of the next tile is copied global -> LDS directly (global_load_lds, no registers) into a second buffer before the current
//     tile's MFMAs start and has landed when they are done: a tile is MFMAs, epilogue and one barrier. Positions outside the volume read
//     a zero row / scale byte 1 from a constant page;
//   * the epilogue's output rows are 32 wide at compile time (more than 16 output channels; fewer go to the general kernel).
// Measured at 32 -> 32 channels, 2 x 128^3, MX-fp8 (8192 tiles): 0.133 ms; before the epilogue's last diet 0.151 ms, of which the K loop alone 0.087 - 0.093 ms with one or with two wavefronts per
// SIMD (72 % of the matrix pipe's cycles at the 1.82 GHz the part settles at under it; 0.077 ms at 1.71 GHz with half the LDS reads), the
// epilogue alone 0.051 ms, the copies 0.01 - 0.03 ms. The parts add up whatever the arrangement: a start offset between the CU's two
// workgroups changes nothing, and one workgroup of two groups of four wavefronts that alternate MFMA and epilogue phases behind barriers
// (one wavefront of a SIMD in its K loop while the other runs its epilogue) took 0.169 ms. What remains is doing less per tile.
#pragma once

template <int FMT, int NT, int OUT, bool EPI>
__global__ void __launch_bounds__(256, 2) conv3_small_k(const conv_args a) {
    constexpr int TZ = NT == 2 ? 2 : 4;
    using HL = halo_t<FMT, 1, TZ>;
    constexpr int TT = HL::TT, HY = HL::HY, HX = HL::HX, NH = HL::NH, WTILE = fmt_t<FMT>::WTILE;
    constexpr int NG = (TT + 63) / 64, TTP = NG * 64;           // copy groups of 64 halo positions; positions per half padded to whole groups
    constexpr int HB = NH * TTP * 16 + TTP * 4;                 // a halo buffer: rows [half][position][16 B], then one scale word per position
    constexpr int NRND = (NG + 3) / 4;                          // copy rounds of a tile: in a round every wave copies one group (its halves and scales)
    constexpr int NP = 14;                                      // 27 taps, two per MFMA; the 28th unit has zero weights
    extern __shared__ __align__(16) unsigned char lds[];
    const unsigned lds0 = (unsigned)(size_t)lds;                // LDS byte offset of the dynamic segment (the low word of its flat address)
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 31, h = lane >> 5;
    int lz, ly0;
    if (NT == 2) { lz = wave >> 1; ly0 = (wave & 1) * 4; } else { lz = wave; ly0 = 0; }
    // the lane's row (its 16-byte half) and scale word of tap (0, 0, 0) inside a halo buffer for its first voxel tile; tile j lies two halo rows further
    const int p00 = (lz * HY + ly0 + (r >> 4)) * HX + (r & 15);
    const unsigned ab0 = ((NH == 2 ? h * TTP : 0) + p00) * 16, sb0 = NH * TTP * 16 + p00 * 4;
    constexpr unsigned ABJ = 2 * HX * 16, SBJ = 2 * HX * 4;
    const size_t Sin = (size_t)a.D * a.H * a.W;

    // XCD-aware persistent tile walk: workgroup ids go round robin over the 8 XCDs, each XCD owns a contiguous range of tiles and its
    // workgroups take them interleaved, so the tiles in flight on an XCD are neighbours (shared halo rows in one L2)
    const unsigned per = (a.ntiles + 7u) / 8u, wg_per_xcd = gridDim.x >> 3, xcd = blockIdx.x & 7u, wix = blockIdx.x >> 3;
    struct tile_t { unsigned tile; int n, oz0, oy0, ox0; bool ok; };
    auto decode = [&](unsigned it) {
        tile_t t; const unsigned k = wix + it * wg_per_xcd;
        t.ok = k < per && xcd * per + k < a.ntiles;
        t.tile = t.ok ? xcd * per + k : 0u;
        int tt = (int)t.tile;
        const int tx = tt % a.ntx; tt /= a.ntx;
        const int ty = tt % a.nty; tt /= a.nty;
        const int tz = tt % a.ntz; t.n = tt / a.ntz;
        t.ox0 = tx * 16; t.oy0 = ty * 8; t.oz0 = tz * TZ;
        return t;
    };
    tile_t cur = decode(0);
    if (!cur.ok) return;

    // the weights' fragments: requested first, their latency hides behind the first halo
    v8i far[NP]; int sap[(NP + 3) / 4];                      // (the E8M0 bytes of four pairs share a register: the MFMA picks its byte)
    {
        const size_t wq_ps = (size_t)a.nmt_all * WTILE, wsc_ps = (size_t)a.nmt_all * 256;
        int sw[NP];
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const uint8_t *wp = a.wq + (size_t)p * wq_ps + lane * 16;
            const v4i lo = *(const v4i *)wp;
            if (FMT == 8) { const v4i hi = *(const v4i *)(wp + 1024); far[p] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]}; }
            else far[p] = (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
            sw[p] = *(const int *)(a.wsc + (size_t)p * wsc_ps + lane * 4);       // the scale byte in the low byte of the lane's word
        }
#pragma unroll
        for (int q = 0; q < (NP + 3) / 4; q++) {
            sap[q] = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) if (4 * q + k < NP) sap[q] |= (sw[4 * q + k] & 255) << (8 * k);
        }
    }
    // the halo of tile t into the buffer at byte offset bo: per round the two row halves back to back (the second finds its cache line) and the scale bytes
    auto request = [&](const tile_t &t, unsigned bo) {
        const int z0 = t.oz0 - 1 + a.zi0, y0 = t.oy0 - 1, x0 = t.ox0 - 1;
        const int base = (z0 * a.H + y0) * a.W + x0;
        int ln = lane;
        asm volatile("" : "+v"(ln));                            // (opaque: the coordinates below are formed per tile, not kept in registers across the K loop)
        const uint8_t *rowb = a.xq[0] + (size_t)t.n * a.nbs[0] * Sin * (16 * NH), *scb = a.xsc[0] + (size_t)t.n * a.nbs[0] * Sin;
#pragma unroll
        for (int rd = 0; rd < NRND; rd++) {
            const int g = 4 * rd + wave;
            if (g < NG) {                                       // (uniform per wavefront)
                const int pos = g * 64 + ln, pz = pos / (HY * HX), rem = pos - pz * (HY * HX), py = rem / HX, px = rem - py * HX;
                const int gz = z0 + pz, gy = y0 + py, gx = x0 + px;
                const bool in = pos < TT && (unsigned)gz < (unsigned)a.D && (unsigned)gy < (unsigned)a.H && (unsigned)gx < (unsigned)a.W;
                const unsigned vox = (unsigned)(base + (pz * a.H + py) * a.W + px);
                const uint8_t *row = in ? rowb + (size_t)vox * (16 * NH) : a.zpage, *sc = in ? scb + vox : a.zpage + 64;
                dma16(row, lds0 + bo + (unsigned)g * 1024u);
                if constexpr (NH == 2) dma16(row + 16, lds0 + bo + (unsigned)TTP * 16u + (unsigned)g * 1024u);
                dma1(sc, lds0 + bo + (unsigned)(NH * TTP * 16) + (unsigned)g * 256u);
            }
        }
    };
    conv_epi_consts<1, EPI>(a, lds, 0, tid);
    request(cur, 0u);
    wait_vm<0>();
    __syncthreads();

    for (unsigned it = 0;; it++) {
        const tile_t nxt = decode(it + 1);
        const unsigned hb = (it & 1u) * (unsigned)HB;
        // the other buffer was last read by the MFMAs of the tile before this one: every wavefront has passed a barrier since
        if (nxt.ok) request(nxt, (unsigned)HB - hb);
        v16f acc[1][NT];
        // A pair's second tap lies D1 = 1 (same row), D2 = HX - 2 (next row) or D3 = (HY - 2) HX - 2 (next plane) positions after its first, so the
        // per-lane addresses that depend on the lane's half (fp4 rows: the half's own unit; scale words: the half's unit) are three bases
        // and every tap offset is an instruction immediate
        constexpr int D1 = 1, D2 = HX - 2, D3 = (HY - 2) * HX - 2;
        const unsigned abt = hb + ab0, sbt = hb + sb0;
        const unsigned abh[4] = {abt, abt + (h ? D1 * 16 : 0), abt + (h ? D2 * 16 : 0), abt + (h ? D3 * 16 : 0)};
        const unsigned sbh[4] = {sbt, sbt + (h ? D1 * 4 : 0), sbt + (h ? D2 * 4 : 0), sbt + (h ? D3 * 4 : 0)};
        // The K loop as one sequence of NP x NT steps (pair p, voxel tile j): a step requests the fragment of the step PF ahead into one of
        // PF + 1 register sets and multiplies its own, so the LDS latency of a fragment is covered by PF MFMAs of the same wavefront
        constexpr int NS = NP * NT, PF = 2;
        v4i flo[PF + 1], fhi[PF + 1]; int fsb[PF + 1];
        auto fetch = [&](auto S) {
            constexpr int st = decltype(S)::value, p = st / NT, jj = st % NT, set = st % (PF + 1), tA = 2 * p, tB = 2 * p + 1 < 27 ? 2 * p + 1 : 2 * p;
            constexpr int pA = ((tA / 9) * HY + (tA / 3) % 3) * HX + tA % 3, pB = ((tB / 9) * HY + (tB / 3) % 3) * HX + tB % 3;
            constexpr int dk = pB - pA == 0 ? 0 : pB - pA == D1 ? 1 : pB - pA == D2 ? 2 : 3;
            static_assert(pB - pA == 0 || pB - pA == D1 || pB - pA == D2 || pB - pA == D3, "tap pair distance");
            if constexpr (FMT == 8) {                           // both units' rows (the lane's half plane)
                flo[set] = *(const v4i *)(lds + abt + pA * 16 + jj * ABJ); fhi[set] = *(const v4i *)(lds + abt + pB * 16 + jj * ABJ);
            } else flo[set] = *(const v4i *)(lds + abh[dk] + pA * 16 + jj * ABJ);       // the half's own unit
            fsb[set] = *(const int *)(lds + sbh[dk] + pA * 4 + jj * SBJ);
        };
        static_for<PF>([&](auto S) { fetch(S); });
        static_for<NS>([&](auto S) {
            constexpr int st = decltype(S)::value, p = st / NT, jj = st % NT, set = st % (PF + 1);
            if constexpr (st + PF < NS) fetch(std::integral_constant<int, st + PF>{});
            const v8i fb = FMT == 8 ? (v8i){flo[set][0], flo[set][1], flo[set][2], flo[set][3], fhi[set][0], fhi[set][1], fhi[set][2], fhi[set][3]}
                                    : (v8i){flo[set][0], flo[set][1], flo[set][2], flo[set][3], 0, 0, 0, 0};
            const v16f c0 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            acc[0][jj] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(far[p], fb, p == 0 ? c0 : acc[0][jj], FMT == 8 ? 0 : 4, FMT == 8 ? 0 : 4, p % 4, sap[p / 4], 0, fsb[set]);
            __builtin_amdgcn_sched_barrier(0);                  // (keeps the steps apart: PF + 1 fragment sets, the registers hold the weights)
        });
        wait_vm<0>();                                           // this wavefront's copies of the next halo have landed (before the epilogue's stores are counted)
        if (cur.oz0 + TZ <= a.Do && cur.oy0 + 8 <= a.Ho && cur.ox0 + 16 <= a.Wo && a.zs0 <= cur.oz0 && a.zs1 >= cur.oz0 + TZ)      // (uniform)
            conv_epilogue<1, NT, OUT, EPI, false, true, true, true>(a, acc, lds, cur.tile, cur.n, 0, cur.oz0, cur.oy0, cur.ox0, lz, ly0, tid);
        else conv_epilogue<1, NT, OUT, EPI, false, true, false, true>(a, acc, lds, cur.tile, cur.n, 0, cur.oz0, cur.oy0, cur.ox0, lz, ly0, tid);
        if (!nxt.ok) break;
        __syncthreads();                                        // every wavefront's copies have landed and everyone is done reading this tile's buffer
        cur = nxt;
    }
}

template <int FMT, int NT, int OUT, bool EPI>
static void launch_small(const conv_args &a, size_t smem) {
    static bool attr[8]; static int ncu[8];
    int d = 0; MIRT(hipGetDevice(&d)); d &= 7;
    if (!attr[d]) {
        MIRT(hipFuncSetAttribute((const void *)conv3_small_k<FMT, NT, OUT, EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        hipDeviceProp_t pr; MIRT(hipGetDeviceProperties(&pr, d));
        ncu[d] = pr.multiProcessorCount > 8 ? pr.multiProcessorCount & ~7 : 8;
        attr[d] = true;
    }
    const unsigned per = (a.ntiles + 7u) / 8u;            // tiles per XCD; two persistent workgroups per CU, a multiple of 8 in all
    const unsigned nwg = per * 8u < 2u * (unsigned)ncu[d] ? per * 8u : 2u * (unsigned)ncu[d];
    conv3_small_k<FMT, NT, OUT, EPI><<<nwg, 256, smem>>>(a);
    MICK();
    snprintf(g_last_kernel, sizeof g_last_kernel, "conv3_small_k<fmt %d, NT %d, out %d, epi %d> tiles %u wgs %u", FMT, NT, OUT, (int)EPI, a.ntiles, nwg);
}
