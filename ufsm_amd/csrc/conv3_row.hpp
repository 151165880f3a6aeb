// The row kernel: 3x3x3 stride-1 conv into ONE channel tile (17 .. 32 output channels) from any number of 32-channel input blocks; the level-0
// layers of a U-Net (32 -> 32, [up(64) | skip(32)] -> 32), where every input fragment feeds a single channel tile and the K loop of the other
// kernels is bound by LDS reads (one 32-byte fragment read per MFMA).
//
//   * A voxel tile of an MFMA is a run of 32 voxels along x of one (z, y) row; a wavefront owns NT = 4 neighbouring rows of one z plane. The
//     input fragment of tap (kz, ky, kx) for row j is the fragment of tap (kz, 0, kx) for halo row j + ky: one fragment read from LDS serves
//     up to three MFMAs (rows s, s - 1, s - 2 with ky 0, 1, 2). The wavefront walks the NT + 2 halo rows of a tap class in order, each row's
//     fragment is read once, multiplied by the three ky weight fragments into the accumulators of the rows it reaches, and dropped:
//     0.5 LDS fragment reads per MFMA instead of 1, in consecutive 16-byte lanes (no bank conflicts).
//   * Taps pair into the MFMA's two K blocks so that both stay fixed under the row walk: class c = kz (c < 3) pairs kx 0 with kx 1 of plane kz,
//     class 3 pairs kx 2 of planes 0 and 1, class 4 is kx 2 of plane 2 beside a zero-weight unit: 5 classes x 3 ky = 15 MFMAs per row and
//     block (14 would be the minimum for 27 taps).
//   * The three weight fragments of a class come straight from global memory (the prepared weights are fragment-ordered; the eight wavefronts
//     of a workgroup read the same 6.75 KiB at about the same time, so the vector cache serves seven of them), requested two classes ahead
//     into three register sets: weights of any number of input blocks need no LDS.
//   * A workgroup is 8 wavefronts = 4 z planes x 2 row groups (a tile of 4 x 8 x 32 voxels), two wavefronts per SIMD, so the copy requests,
//     address arithmetic and LDS reads of one wavefront issue in the shadow of the other's MFMAs. One persistent workgroup per CU walks
//     (tile, input block) steps XCD by XCD; the halo of the next step is copied global -> LDS directly (global_load_lds) into the second of
//     two buffers, one copy round per tap class, and has landed when the step's 60 MFMAs per wavefront are done: a step is MFMAs and one barrier.
#pragma once

__device__ __forceinline__ void row_pin(v16f &x) { asm volatile("" : "+v"(x)::"memory"); }

// WL (MX-fp4 only): the prepared weights of all input blocks are copied into LDS once per workgroup (19 200 bytes per block: an e2m1 fragment is half
// an e4m3 one, and the halo buffers are half as large) and the K loop reads its fragments from there: no global loads but the halo's copies
template <int FMT, int OUT, bool EPI, bool WL = false>
__global__ void __launch_bounds__(512, 1) conv3_row_k(const conv_args a) {
    static_assert(!WL || FMT == 4, "weights resident in LDS: the e2m1 form");
    constexpr int NT = 4, TZ = 4, TY = 8, TX = 32, NW = 8;
    constexpr int HZ = TZ + 2, HY = TY + 2, HX = TX + 2, TT = HZ * HY * HX, NH = fmt_t<FMT>::NH, WTILE = fmt_t<FMT>::WTILE;
    constexpr int NG = (TT + 63) / 64, TTP = NG * 64;           // copy groups of 64 halo positions; positions per half padded to whole groups
    constexpr int HB = NH * TTP * 16 + TTP * 4;                 // a halo buffer: rows [half][position][16 B], then one scale word per position
    constexpr int NRND = (NG + NW - 1) / NW;                    // copy rounds of a step: in a round every wavefront copies one group
    constexpr int NC = 5, NPB = 3 * NC;                         // tap classes; weight pairs per input block
    static_assert(NRND <= NC - 1, "one copy round per tap class, the last class free");
    extern __shared__ __align__(16) unsigned char lds[];
    const unsigned lds0 = (unsigned)(size_t)lds;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 31, h = lane >> 5;
    const int lz = wave >> 1, ly0 = (wave & 1) * NT;
    // the lane's 16-byte row half and scale word of halo position (lz, ly0, r): tap (0, 0, 0) of its first row. A tap class reads the two units
    // of its pairs at fixed position offsets; what depends on the lane's half (fp4 rows: the half's own unit; scale words: the half's unit) is
    // the second unit's distance D from the first: 1 (classes 0 - 2), HY HX (class 3) or 0 (class 4): three bases, everything else immediates
    const int p00 = (lz * HY + ly0) * HX + r;
    const unsigned ab0 = ((NH == 2 ? h * TTP : 0) + p00) * 16, sb0 = NH * TTP * 16 + p00 * 4;
    constexpr int DCL[3] = {1, HY * HX, 0};
    const size_t Sin = (size_t)a.D * a.H * a.W;
    const size_t wq_ps = (size_t)a.nmt_all * WTILE, wsc_ps = (size_t)a.nmt_all * 256;

    // XCD-aware persistent tile walk: workgroup ids go round robin over the 8 XCDs, each XCD owns a contiguous range of tiles
    // Two channel tiles (33 .. 64 output channels): a workgroup keeps ONE of them for its whole walk (bias, weights and statistics records of
    // slice cs), and neighbouring workgroups of an XCD take the same spatial tiles in the other slice, so the halo's second read finds the L2
    const unsigned ncs = (unsigned)a.ncs, nsp = a.ntiles / ncs;                      // channel slices; spatial tiles
    const int cs = __builtin_amdgcn_readfirstlane((int)((blockIdx.x >> 3) % ncs));
    const unsigned per = (nsp + 7u) / 8u, wg_per_xcd = (gridDim.x >> 3) / ncs, xcd = blockIdx.x & 7u, wix = (blockIdx.x >> 3) / ncs;
    struct tile_t { unsigned tile; int n, oz0, oy0, ox0; bool ok; };
    auto decode = [&](unsigned it) {
        tile_t t; const unsigned k = wix + it * wg_per_xcd;
        t.ok = k < per && xcd * per + k < nsp;
        t.tile = t.ok ? xcd * per + k : 0u;
        int tt = (int)t.tile;
        const int tx = tt % a.ntx; tt /= a.ntx;
        const int ty = tt % a.nty; tt /= a.nty;
        const int tz = tt % a.ntz; t.n = tt / a.ntz;
        t.ox0 = tx * TX; t.oy0 = ty * TY; t.oz0 = tz * TZ;
        return t;
    };
    tile_t cur = decode(0);
    if (!cur.ok) return;

    // copy round rd of input block b of tile t into the buffer at byte offset bo: this wavefront's group of 64 halo positions, the two row
    // halves back to back (the second finds its cache line) and the scale bytes; positions outside the volume or past the halo read the
    // constant page (zero row, scale byte 1)
    // (no branch in here: the K loop below must stay one basic block, or the compiler sinks the MFMAs of a step below its loads and spills them;
    // `on` false turns the whole request into reads of the constant page)
    static_assert(NG % NW == 0, "every wavefront copies a group in every round");
    auto request = [&](const tile_t &t, int b, unsigned bo, int rd, bool on) {
        const int g = NW * rd + wave;
        const int seg = b >= a.nb0p, blk = seg ? b - a.nb0p : b;
        const int z0 = t.oz0 - 1 + a.zi0, y0 = t.oy0 - 1, x0 = t.ox0 - 1;
        int ln = lane;
        asm volatile("" : "+v"(ln));                            // (opaque: the coordinates are formed per request, not kept in registers across the K loop)
        const int pos = g * 64 + ln, pz = pos / (HY * HX), rem = pos - pz * (HY * HX), py = rem / HX, px = rem - py * HX;
        const int gz = z0 + pz, gy = y0 + py, gx = x0 + px;
        const bool in = on & (pos < TT) & (blk < a.nbs[seg]) & ((unsigned)gz < (unsigned)a.D) & ((unsigned)gy < (unsigned)a.H) & ((unsigned)gx < (unsigned)a.W);
        const int sp = (gz * a.H + gy) * a.W + gx;                // (garbage where !in: unused)
        const size_t vox = ((size_t)t.n * a.nbs[seg] + (in ? blk : 0)) * Sin + (size_t)(in ? sp : 0);
        const uint8_t *row = in ? a.xq[seg] + vox * (16 * NH) : a.zpage, *sc = in ? a.xsc[seg] + vox : a.zpage + 64;
        dma16(row, lds0 + bo + (unsigned)g * 1024u);
        if constexpr (NH == 2) dma16(row + 16, lds0 + bo + (unsigned)TTP * 16u + (unsigned)g * 1024u);
        dma1(sc, lds0 + bo + (unsigned)(NH * TTP * 16) + (unsigned)g * 256u);
    };
    conv_epi_consts<1, EPI>(a, lds, cs, tid);
#pragma unroll
    for (int rd = 0; rd < NRND; rd++) request(cur, 0, 0u, rd, true);

    // the weight fragments of one tap class of input block b: three pairs (ky 0, 1, 2), lane-ordered codes and the lane's scale word
    struct wcl { v8i f[3]; int s[3]; };
    constexpr int WPB = 1024 + 256;                             // (WL) bytes of a pair in LDS: the lanes' 16 bytes of codes, then their scale words
    if constexpr (WL) {                                         // every pair of every block: 80 16-byte pieces, copied by the whole workgroup
        const size_t wq_ps0 = (size_t)a.nmt_all * WTILE, wsc_ps0 = (size_t)a.nmt_all * 256;
        for (int i = tid; i < a.nbt * NPB * (WPB / 16); i += NW * 64) {
            const int p = i / (WPB / 16), k = i - p * (WPB / 16);
            const v4i v = k < 64 ? *(const v4i *)(a.wq + (size_t)p * wq_ps0 + (size_t)cs * WTILE + k * 16) : *(const v4i *)(a.wsc + (size_t)p * wsc_ps0 + (size_t)cs * 256 + (k - 64) * 16);
            *(v4i *)(lds + a.wl_o + p * WPB + k * 16) = v;
        }
    }
    auto wload = [&](int b, auto C) {
        constexpr int c = decltype(C)::value;
        wcl w;
        if constexpr (WL) {
            const unsigned o = a.wl_o + (unsigned)((b * NPB + c * 3) * WPB);
#pragma unroll
            for (int ky = 0; ky < 3; ky++) {
                const v4i lo = *(const v4i *)(lds + o + ky * WPB + lane * 16);
                w.f[ky] = (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
                w.s[ky] = *(const int *)(lds + o + ky * WPB + 1024 + lane * 4);
            }
            return w;
        }
        const uint8_t *wp = a.wq + ((size_t)b * NPB + c * 3) * wq_ps + (size_t)cs * WTILE + lane * 16, *sp = a.wsc + ((size_t)b * NPB + c * 3) * wsc_ps + (size_t)cs * 256 + lane * 4;
#pragma unroll
        for (int ky = 0; ky < 3; ky++) {
            const v4i lo = *(const v4i *)(wp + ky * wq_ps);
            // (e4m3: the pair's second unit; class 4's is the zero padding unit and is not loaded)
            if (FMT == 8 && c != NC - 1) { const v4i hi = *(const v4i *)(wp + ky * wq_ps + 1024); w.f[ky] = (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]}; }
            else w.f[ky] = (v8i){lo[0], lo[1], lo[2], lo[3], 0, 0, 0, 0};
            w.s[ky] = *(const int *)(sp + ky * wsc_ps);
        }
        return w;
    };
    // three weight sets, loaded two classes ahead: class c of a step reads set CSET[c] while class c + 2 (past the step's last class: the next
    // step's classes 0 and 1) loads into the set class c - 1 has just left; the next step's first two classes land in sets 2 and 0 and are moved
    // to their places (0 and 1) at the step's end
    wcl ws[3];
    if constexpr (WL) { wait_vm<0>(); __syncthreads(); }        // (the weights' image is complete before anyone reads it)
    ws[0] = wload(0, std::integral_constant<int, 0>{});
    ws[1] = wload(0, std::integral_constant<int, 1>{});
    wait_vm<0>();
    __syncthreads();

    v16f acc[1][NT];
#pragma unroll
    for (int j = 0; j < NT; j++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[0][j][i] = 0.f;
    int b = 0;                                                  // the step's input block
    for (unsigned it = 0, step = 0;; step++) {
        const bool last_b = b + 1 == a.nbt;
        const tile_t nxt = last_b ? decode(it + 1) : cur;
        const int nb = last_b ? 0 : b + 1;
        const bool more = !last_b || nxt.ok;                    // a step follows this one
        const unsigned hb = (step & 1u) * (unsigned)HB;
        const unsigned abt = hb + ab0, sbt = hb + sb0;
        unsigned abh[3], sbh[3];
#pragma unroll
        for (int k = 0; k < 3; k++) { abh[k] = abt + (h ? DCL[k] * 16 : 0); sbh[k] = sbt + (h ? DCL[k] * 4 : 0); }
        // halo row s of class c: the lane's fragment (both units' row halves, or the half's own unit) and its scale word
        struct frag { v4i lo, hi; int sb; };
        auto fetch = [&](auto C, auto S) {
            constexpr int c = decltype(C)::value, s = decltype(S)::value;
            constexpr int kzA = c < 3 ? c : c == 3 ? 0 : 2, kxA = c < 3 ? 0 : 2, dk = c < 3 ? 0 : c == 3 ? 1 : 2;
            constexpr int pA = (kzA * HY + s) * HX + kxA, pB = pA + DCL[dk];
            frag f;
            if constexpr (FMT == 8) { f.lo = *(const v4i *)(lds + abt + pA * 16); f.hi = *(const v4i *)(lds + abt + pB * 16); }
            else { f.lo = *(const v4i *)(lds + abh[dk] + pA * 16); f.hi = (v4i){0, 0, 0, 0}; }
            f.sb = *(const int *)(lds + sbh[dk] + pA * 4);
            return f;
        };
        // A step as one sequence of NC x (NT + 2) row visits: visit (c, s) requests the fragment two visits ahead into one of three sets and
        // multiplies its own by the ky weights of the rows it reaches (j = s - ky); the class's copy round and the next class's weights are
        // requested at fixed visits, so the order of the outstanding memory operations is the same in every step
        constexpr int NR = NT + 2, NV = NC * NR, PF = 2;
        constexpr int CSET[NC] = {0, 1, 2, 0, 1};
        {
            frag fr[PF + 1];
            static_for<PF>([&](auto V) { constexpr int v = decltype(V)::value; fr[v] = fetch(std::integral_constant<int, v / NR>{}, std::integral_constant<int, v % NR>{}); });
            static_for<NV>([&](auto V) {
                constexpr int v = decltype(V)::value, c = v / NR, s = v % NR, set = v % (PF + 1);
                if constexpr (v + PF < NV) fr[(v + PF) % (PF + 1)] = fetch(std::integral_constant<int, (v + PF) / NR>{}, std::integral_constant<int, (v + PF) % NR>{});
                if constexpr (s == 0) {                          // the weights two classes ahead (past the last step: block 0 again, unused)
                    if constexpr (c + 2 < NC) ws[CSET[c + 2]] = wload(b, std::integral_constant<int, (c + 2) % NC>{}); else ws[c + 2 == NC ? 2 : 0] = wload(nb, std::integral_constant<int, (c + 2) % NC>{});
                }
                if constexpr (s == 1 && c < NRND) request(nxt, nb, (unsigned)HB - hb, c, more);
                const v8i fb = FMT == 8 ? (v8i){fr[set].lo[0], fr[set].lo[1], fr[set].lo[2], fr[set].lo[3], fr[set].hi[0], fr[set].hi[1], fr[set].hi[2], fr[set].hi[3]}
                                        : (v8i){fr[set].lo[0], fr[set].lo[1], fr[set].lo[2], fr[set].lo[3], 0, 0, 0, 0};
                static_for<3>([&](auto KY) {
                    constexpr int ky = decltype(KY)::value, j = s - ky;
                    if constexpr (j >= 0 && j < NT) {
                        acc[0][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(ws[CSET[c]].f[ky], fb, acc[0][j], FMT == 8 ? 0 : 4, FMT == 8 ? 0 : 4,
                                                                                    0, ws[CSET[c]].s[ky], 0, fr[set].sb);
                    }
                });
                // (keeps the visits apart: three fragment sets, three weight sets. The products are pure values, which the compiler would
                // otherwise sink below every load and copy request of the step; passing them through an empty statement that also orders
                // memory operations keeps each visit's loads, products and requests where they are written)
                static_for<3>([&](auto KY) { constexpr int j = s - decltype(KY)::value; if constexpr (j >= 0 && j < NT) row_pin(acc[0][j]); });
                __builtin_amdgcn_sched_barrier(0);
            });
        }
        wait_vm<0>();                                           // this wavefront's copies of the next step's halo have landed
        ws[1] = ws[0]; ws[0] = ws[2];                           // the next step's classes 1 and 0
        if (last_b) {
            if (cur.oz0 + TZ <= a.Do && cur.oy0 + TY <= a.Ho && cur.ox0 + TX <= a.Wo && a.zs0 <= cur.oz0 && a.zs1 >= cur.oz0 + TZ)      // (uniform)
                conv_epilogue<1, NT, OUT, EPI, false, true, true, true, NW, true>(a, acc, lds, cur.tile * ncs + cs, cur.n, cs, cur.oz0, cur.oy0, cur.ox0, lz, ly0, tid);
            else conv_epilogue<1, NT, OUT, EPI, false, true, false, true, NW, true>(a, acc, lds, cur.tile * ncs + cs, cur.n, cs, cur.oz0, cur.oy0, cur.ox0, lz, ly0, tid);
            if (!nxt.ok) break;
            cur = nxt; it++;
#pragma unroll
            for (int j = 0; j < NT; j++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc[0][j][i] = 0.f;
        }
        b = nb;
        __syncthreads();                                        // every wavefront's copies have landed and everyone is done reading this step's buffer
    }
}

template <int FMT, int OUT, bool EPI, bool WL>
static void launch_row(const conv_args &a, size_t smem) {
    static bool attr[8]; static int ncu[8];
    int d = 0; MIRT(hipGetDevice(&d)); d &= 7;
    if (!attr[d]) {
        MIRT(hipFuncSetAttribute((const void *)conv3_row_k<FMT, OUT, EPI, WL>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        hipDeviceProp_t pr; MIRT(hipGetDeviceProperties(&pr, d));
        ncu[d] = pr.multiProcessorCount > 8 ? pr.multiProcessorCount & ~7 : 8;
        attr[d] = true;
    }
    const unsigned ncs = (unsigned)a.ncs, per = (a.ntiles / ncs + 7u) / 8u;            // spatial tiles per XCD; one persistent workgroup per CU, a multiple of 8 x slices in all
    const unsigned cap0 = (unsigned)ncu[d] / (8u * ncs) * (8u * ncs), cap = cap0 ? cap0 : 8u * ncs, nwg = per * 8u * ncs < cap ? per * 8u * ncs : cap;      // (fewer CUs than 8 x slices: the walk works for any grid)
    conv3_row_k<FMT, OUT, EPI, WL><<<nwg, 512, smem>>>(a);
    MICK();
    snprintf(g_last_kernel, sizeof g_last_kernel, "conv3_row_k<fmt %d, out %d, epi %d%s> blocks %d tiles %u%s wgs %u", FMT, OUT, (int)EPI, WL ? ", weights in LDS" : "", a.nbt, a.ntiles, ncs == 2 ? " (two channel slices)" : ncs > 2 ? " (channel slices)" : "", nwg);
}
