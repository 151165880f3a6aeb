// The wide 3x3x3 stride-1 kernel: 128 output channels x 4 x 8 x 16 voxels per tile, one wavefront per SIMD with 16 accumulators (AGPRs).
//
// Every weight fragment is reused by 4 voxel tiles and every input fragment by 4 channel tiles, which halves the LDS traffic per MFMA of
// the 8-accumulator kernel: at full MFMA rate the 4 wavefronts read about 72 B / clk of the CU's 128 B / clk. With a single wavefront per
// SIMD nothing else hides latency, so the schedule is explicit:
//   * fragments of pair q + 1 are fetched into a second register set between the MFMAs of pair q (sched_group_barrier pins the
//     interleave); one workgroup barrier per two pairs;
//   * all global -> LDS traffic is direct (global_load_lds, no registers): weight stages of two pairs go into a 2-slot ring two stages
//     ahead; input halo blocks of 32 channels live in 3 LDS slots and the K loop walks the blocks one after the other (taps inside), so
//     while blocks b, b + 1 are multiplied block b + 2 streams into the third slot; the first blocks of the next tile follow the last one of
//     this tile and land during the epilogue. Positions outside the volume read a zero row / scale byte 1 from a constant page;
//   * workgroups are persistent (one per CU) and walk their tiles XCD by XCD.
// The asynchronous copies are tracked with vmcnt: every copying step issues its weight copies first and then a fixed number of halo
// copies, all unconditionally (nothing in a step branches, or the MFMA / LDS interleave would fall apart), so "all but the last few"
// is exactly "the weights have landed".
#pragma once

__device__ __forceinline__ void dma16(const void *g, unsigned lds_off) {      // lane l: 16 bytes from g (per lane) to LDS lds_off + 16 l
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_off), "v"(g) : "memory");
}
__device__ __forceinline__ void dma1(const void *g, unsigned lds_off) {       // lane l: 1 byte from g, zero-extended to the word at LDS lds_off + 4 l
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_ubyte %1, off" ::"s"(lds_off), "v"(g) : "memory");
}
// the same with a uniform 64-bit base and a 32-bit per-lane byte offset
__device__ __forceinline__ void dma16s(unsigned off, const void *base, unsigned lds_off) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_off), "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void dma1s(unsigned off, const void *base, unsigned lds_off) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_ubyte %1, %2" ::"s"(lds_off), "v"(off), "s"(base) : "memory");
}
// the same with the LDS offset formed in the instruction: m0 = ldsb + IMM
template <int IMM> __device__ __forceinline__ void dma16si(unsigned off, const void *base, unsigned ldsb) {
    asm volatile("s_add_u32 m0, %0, %3\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(ldsb), "v"(off), "s"(base), "n"(IMM) : "memory", "scc");
}
template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// MT: channel tiles of 32 per workgroup: 4 (slices of 128 output channels) or 2 (64-channel layers: 8 accumulators per wavefront)
template <int FMT, int OUT, bool EPI, int MT = 4>
__global__ void __launch_bounds__(256, 1) conv3_wide_k(const conv_args a) {
    constexpr int NT = 4, TZ = 4;
    static_assert(MT == 4 || MT == 2, "channel tiles per workgroup");
    using HL = halo_t<FMT, 1, TZ>;
    constexpr int TT = HL::TT, HY = HL::HY, HX = HL::HX, NH = HL::NH, WTILE = fmt_t<FMT>::WTILE;
    constexpr int STG = MT * (WTILE + 256), SLOT = 2 * STG;     // a ring slot holds one stage = two pairs, each MT tiles of codes then MT x 64 scale words
    constexpr int NG = (TT + 63) / 64, TTP = NG * 64;           // copy groups of 64 halo positions; positions per half padded to whole groups
    constexpr int HB = NH * TTP * 16 + TTP * 4;                 // a halo slot: rows [half][position][16 B], then one scale word per position
    constexpr int NRND = (NG + 3) / 4;                          // copy rounds of a block: in a round every wave copies one group (both halves and the scales)
    constexpr int NCH = SLOT / 1024;                            // 1 KiB copies per weight stage: the prepared weights hold the ring slot's image, stage after stage
    static_assert(SLOT % 1024 == 0, "a weight stage is a whole number of 1 KiB copies");
    extern __shared__ __align__(16) unsigned char lds[];
    const unsigned lds0 = (unsigned)(size_t)lds;                // LDS byte offset of the dynamic segment (the low word of its flat address)
    constexpr unsigned halo_o = 2 * SLOT, tab_o = halo_o + 3 * HB;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), r = lane & 31, h = lane >> 5;
    const int lz = wave, ly0 = 0;
    // the lane's row (its 16-byte half) and scale word of tap (0, 0, 0) inside a halo slot for its first voxel tile; tile j lies two halo rows
    // further: a constant the loads carry in their offset field
    const int p00 = (lz * HY + (r >> 4)) * HX + (r & 15);
    const unsigned abr0 = halo_o + ((NH == 2 ? h * TTP : 0) + p00) * 16, sbr0 = halo_o + NH * TTP * 16 + p00 * 4;
    constexpr unsigned ABJ = 2 * HX * 16, SBJ = 2 * HX * 4;
    const unsigned wfa = lane * 16, wfs = MT * WTILE + lane * (MT * 4);     // the lane's weight fragment of tile 0 / its MT scale words of pair 0 of a slot
    const size_t Sin = (size_t)a.D * a.H * a.W;
    const int nunits = 27 * a.nbt, npairs = (nunits + 1) >> 1, nfull = npairs >> 1;

    // XCD-aware persistent tile walk: workgroup ids go round robin over the 8 XCDs, each XCD owns a contiguous range of tiles
    const unsigned per = (a.ntiles + 7u) / 8u, wg_per_xcd = gridDim.x >> 3, xcd = blockIdx.x & 7u, wix = blockIdx.x >> 3;
    struct tile_t { unsigned tile; int n, cs, oz0, oy0, ox0; bool ok; };
    auto decode = [&](unsigned it) {
        tile_t t; const unsigned k = wix + it * wg_per_xcd;
        t.ok = k < per && xcd * per + k < a.ntiles;
        t.tile = t.ok ? xcd * per + k : 0u;
        int tt = (int)t.tile;
        t.cs = tt % a.ncs; tt /= a.ncs;
        const int tx = tt % a.ntx; tt /= a.ntx;
        const int ty = tt % a.nty; tt /= a.nty;
        const int tz = tt % a.ntz; t.n = tt / a.ntz;
        t.ox0 = tx * 16; t.oy0 = ty * 8; t.oz0 = tz * TZ;
        return t;
    };
    // One copy round of this wave = the two row halves and the scale bytes of 64 halo positions (group 4 rd + wave of the NG groups a block's
    // halo has) for one block of a tile. The issue is three copies with every lane active and no branch: positions outside the volume, past
    // the halo or of blocks past the stored channels read a constant page (zero row, scale byte 1); a round with nothing to do (go false, or a
    // group past the last) reads the constant page into a junk area. The two halves of a row are requested back to back, so the second one
    // finds its cache line. The request's addresses are prepared one step ahead of its issue from data that is formed once per kernel or
    // once per tile, so that a round costs a handful of instructions the scheduler places between the MFMAs:
    //   * per lane and round rd, the position's offset inside a tile's halo as a voxel offset of the volume, (pz H + py) W + px, and its
    //     packed coordinates (kernel constants). The offsets sit in a ring of five registers that turns by one whenever a round is consumed:
    //     its head is the round to request next (rounds cycle 0 .. NRND - 1 block after block);
    //   * per lane and tile (this one, the next one), a bit per round: the position is inside the halo and the volume;
    //   * per tile, the voxel offset of the halo's first position (may be negative), and in lane i of a register group the base addresses of
    //     the rows and scale bytes of request block i: blocks 0 .. nbt - 1 of this tile, then the first blocks of the next one.
    const unsigned junk = a.red_o;                              // the statistics scratch (1 KiB) is idle while the K loop runs
    struct hreq { const uint8_t *row, *sc; unsigned rdst, sdst; };
    static_assert(NRND == 5, "the round ring below has five entries");
    unsigned pc[NRND];                                          // px | py << 8 | pz << 16 | (position inside the halo) << 24
    unsigned ring0, ring1, ring2, ring3, ring4;
    {
        unsigned dl[NRND];
#pragma unroll
        for (int rd = 0; rd < NRND; rd++) {
            const int g = 4 * rd + wave, pos = g * 64 + lane;
            const int pz = pos / (HY * HX), rem = pos - pz * (HY * HX), py = rem / HX, px = rem - py * HX;
            pc[rd] = (unsigned)px | ((unsigned)py << 8) | ((unsigned)pz << 16) | ((g < NG && pos < TT ? 1u : 0u) << 24);
            dl[rd] = (unsigned)((pz * a.H + py) * a.W + px);
        }
        ring0 = dl[0]; ring1 = dl[1]; ring2 = dl[2]; ring3 = dl[3]; ring4 = dl[4];
    }
    struct treq { unsigned mask; int base; };                   // a tile's validity bits (per lane) and first-position voxel offset (uniform)
    auto tile_req = [&](const tile_t &t) {
        treq q; q.mask = 0u;
        const int z0 = t.oz0 - 1 + a.zi0, y0 = t.oy0 - 1, x0 = t.ox0 - 1;
#pragma unroll
        for (int rd = 0; rd < NRND; rd++) {
            const int gz = z0 + (int)((pc[rd] >> 16) & 255u), gy = y0 + (int)((pc[rd] >> 8) & 255u), gx = x0 + (int)(pc[rd] & 255u);
            const bool in = (pc[rd] >> 24) && (unsigned)gz < (unsigned)a.D && (unsigned)gy < (unsigned)a.H && (unsigned)gx < (unsigned)a.W;
            q.mask |= in ? 1u << rd : 0u;
        }
        q.base = (z0 * a.H + y0) * a.W + x0;
        return q;
    };
    // lane i: request block i (i < nbt: block i of tile c; else block i - nbt of tile x): row base, scale base, block holds stored channels
    unsigned long long tb_row = 0, tb_sc = 0; int tb_ok = 0;
    int tb_gate = 0, tb_base = 0, tb_slot = 0, tb_msh = 0;      // also per request block: first pair after which it may be requested, its tile's first-position
                                                                // voxel offset, its halo slot's byte offset, the shift of its tile's validity bits
    auto block_table = [&](const tile_t &c, const tile_t &x, int fmax, unsigned rot, int bcur, int bnxt) {
        const int i = lane, own = i < a.nbt, blk = own ? i : i - a.nbt, n = own ? c.n : x.n;
        const int seg = blk >= a.nb0p, bl = seg ? blk - a.nb0p : blk;
        const int nbs = seg ? a.nbs[1] : a.nbs[0];
        const uint8_t *xq = seg ? a.xq[1] : a.xq[0], *xsc = seg ? a.xsc[1] : a.xsc[0];
        const size_t plane = ((size_t)n * nbs + min(max(bl, 0), max(nbs - 1, 0))) * Sin;
        tb_row = (unsigned long long)(size_t)(xq + plane * (16 * NH)); tb_sc = (unsigned long long)(size_t)(xsc + plane);
        tb_ok = blk < a.nbt && bl < nbs;
        tb_gate = i > fmax ? 0x7fffffff : i < 3 ? -1 : (27 * (i - 3) + 26) >> 1;       // block i takes the slot block i - 3 is read from until that pair
        tb_base = own ? bcur : bnxt;
        tb_slot = (int)((rot + (unsigned)i) % 3u) * HB;
        tb_msh = own ? 0 : 8;
    };
    treq rq_cur, rq_nxt;
    auto lane64 = [&](unsigned long long v, int i) {
        const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)v, i), hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(v >> 32), i);
        return (unsigned long long)lo | ((unsigned long long)hi << 32);
    };
    // the round rd (uniform) of request block ti of the tile whose data is (mask, base), into the halo slot at byte offset sbase; go false: a
    // round into the junk area. d: the lane's offset for that round (the ring's head, or a compile-time pick)
    auto prepare = [&](hreq &q, unsigned mask, int base, int ti, int rd, unsigned d, unsigned sbase, bool go) {
        const int g = 4 * rd + wave;
        const bool real = go & (g < NG);
        const bool in = real & (__builtin_amdgcn_readlane(tb_ok, ti) != 0) & (((mask >> rd) & 1u) != 0u);
        const unsigned vox = (unsigned)base + d;
        const uint8_t *rb = (const uint8_t *)(size_t)lane64(tb_row, ti), *sb = (const uint8_t *)(size_t)lane64(tb_sc, ti);
        q.row = in ? rb + (size_t)vox * (16 * NH) : a.zpage;
        q.sc = in ? sb + vox : a.zpage + 64;
        q.rdst = real ? halo_o + sbase + g * 1024 : junk;
        q.sdst = real ? halo_o + sbase + NH * TTP * 16 + g * 256 : junk;
    };
    auto issue = [&](const hreq &q) {
        dma16(q.row, lds0 + q.rdst);
        if constexpr (NH == 2) dma16(q.row + 16, lds0 + q.rdst + (q.rdst == junk ? 0u : (unsigned)TTP * 16u));
        dma1(q.sc, lds0 + q.sdst);
    };
    constexpr int NHC = NH + 1;                                 // asynchronous copies of a round
    // The weight stage of pairs 2 s, 2 s + 1 of channel slice cs is SLOT contiguous bytes at wq + cs wstride + s SLOT, the image of a ring
    // slot: per pair the MT tiles of codes, then per lane its MT scale words. Wave w copies the 1 KiB pieces w, w + 4, ... (NW of them; a wave
    // with fewer repeats its last one: the count per step stays fixed). A copy is one instruction pair: m0 = slot + piece, load.
    constexpr int NW = (NCH + 3) / 4;
    unsigned wvo[NW];                                           // the lane's byte offset inside a stage for copy k
#pragma unroll
    for (int k = 0; k < NW; k++) { int c = wave + 4 * k; c = c < NCH ? c : c - 4; wvo[k] = (unsigned)c * 1024u + (unsigned)lane * 16u; }
    const unsigned wd0 = lds0 + (unsigned)wave * 1024u;         // LDS address of the wave's first piece in slot 0
    const unsigned wdl = (wave + 4 * (NW - 1) < NCH) ? (unsigned)(NW - 1) * 4096u : (unsigned)(NW - 2) * 4096u;   // its last piece
    auto wcopy = [&](auto K, const uint8_t *src, unsigned so) {
        constexpr int k = decltype(K)::value;
        if constexpr (k < NW - 1) dma16si<k * 4096>(wvo[k], src, wd0 + so);
        else dma16s(wvo[k], src, wd0 + so + wdl);
    };
    auto wstage = [&](int st, int cs, unsigned so) {            // stage st of slice cs into the ring slot at byte offset so
        const uint8_t *src = a.wq + (size_t)cs * a.wstride + (size_t)st * SLOT;
        static_for<NW>([&](auto K) { wcopy(K, src, so); });
    };

    // K order: unit U = (block U / 27, tap U % 27), pair G = units 2 G, 2 G + 1 (a pair may straddle two blocks; the unit past the end has
    // zero weights and re-reads the one before). Block b of the workgroup's it-th tile lives in halo slot (it nbt + b) % 3: while blocks
    // b, b + 1 are multiplied, block b + 2 streams into the slot block b - 1 left; the first two blocks of the next tile follow the last
    // block of this one.
    tile_t cur = decode(0);
    if (!cur.ok) return;
    const int nnext = min(2, a.nbt);                            // blocks of the next tile requested ahead
    rq_nxt = tile_req(cur);
    block_table(cur, cur, 1, 0u, rq_nxt.base, rq_nxt.base);
    {
        const unsigned d5[NRND] = {ring0, ring1, ring2, ring3, ring4};
#pragma unroll
        for (int rd = 0; rd < NRND; rd++) {
            hreq q;
            prepare(q, rq_nxt.mask, rq_nxt.base, 0, rd, d5[rd], 0, true); issue(q);
            if (nnext > 1) { prepare(q, rq_nxt.mask, rq_nxt.base, 1, rd, d5[rd], HB, true); issue(q); }
        }
    }
    wstage(0, cur.cs, 0); wstage(1, cur.cs, SLOT);
    unsigned rot = 0;                                           // (it nbt) % 3
    for (unsigned it = 0;; it++) {
        const tile_t nxt = decode(it + 1);
        rq_cur = rq_nxt; rq_nxt = tile_req(nxt);
        const int fmax = a.nbt - 1 + (nxt.ok ? nnext : 0);      // blocks to request during this tile: 2 .. nbt - 1 of this tile, then nbt .. of the next
        block_table(cur, nxt, fmax, rot, rq_cur.base, rq_nxt.base);
        const unsigned mask2 = rq_cur.mask | (rq_nxt.mask << 8);            // validity bits of both tiles
        wait_vm<0>();                                           // the tile's first blocks and weight stages (and the last tile's stores) are done
        __syncthreads();
        DBG_MARK(0);
        conv_epi_consts<MT, EPI>(a, lds, cur.cs, tid);
        // pair table of this tile: per pair and lane half {row offset of unit A (fp4: of the half's own unit), of unit B, scale word offset of the half's unit}
        for (int i = tid; i < (npairs + 2) * 2; i += 256) {
            const int g = min(i >> 1, npairs - 1), hh = i & 1;
            const int uA = 2 * g, uB = 2 * g + 1 < nunits ? 2 * g + 1 : 2 * g;
            const int bA = uA / 27, tA = uA - 27 * bA, bB = uB / 27, tB = uB - 27 * bB;
            const int oA = (int)((rot + bA) % 3u) * HB + (((tA / 9) * HY + (tA / 3) % 3) * HX + tA % 3) * 16;
            const int oB = (int)((rot + bB) % 3u) * HB + (((tB / 9) * HY + (tB / 3) % 3) * HX + tB % 3) * 16;
            const int oH = hh ? oB : oA, sH = (oH / HB) * HB + ((oH % HB) >> 2);
            *(v4i *)(lds + tab_o + i * 16) = (v4i){NH == 2 ? oA : oH, oB, sH, 0};
        }
        v16f acc[MT][NT];                                       // (not cleared: the tile's first pair multiplies onto a zero operand)
        __syncthreads();

        v8i fb[2][NT], fa[2][MT]; int sb[2][NT]; int sav[2][MT];
        v4i T;
        unsigned tabp = tab_o + h * 16;
        T = *(const v4i *)(lds + tabp);
        // one LDS load of the fetch of a pair: index i = 3 f + part over the NT input fragments, then the MT weight fragments; the last
        // index reads the table entry of the pair after
        v4i lo[NT + MT], hi[NT + MT];
        auto ld = [&](auto I, auto NXT, const v4i tt2, unsigned wbase) {
            constexpr int i = decltype(I)::value, nx = decltype(NXT)::value;
            constexpr int f = i / 3, part = i % 3;
            if constexpr (i == 3 * (NT + MT)) { T = *(const v4i *)(lds + tabp + 32); tabp += 32; }
            else if constexpr (f < NT) {
                if constexpr (part == 0) lo[f] = *(const v4i *)(lds + (abr0 + tt2[0]) + f * ABJ);
                else if constexpr (part == 1) { if constexpr (FMT == 8) hi[f] = *(const v4i *)(lds + (abr0 + tt2[1]) + f * ABJ); }
                else if constexpr (f % 2 == 0) {                // two tiles' scale words back to back: one two-address LDS read
                    sb[nx][f] = *(const int *)(lds + (sbr0 + tt2[2]) + f * SBJ);
                    sb[nx][f + 1] = *(const int *)(lds + (sbr0 + tt2[2]) + (f + 1) * SBJ);
                }
            } else {
                constexpr int m = f - NT;
                if constexpr (part == 0) lo[f] = *(const v4i *)(lds + wfa + wbase + m * WTILE);
                else if constexpr (part == 1) { if constexpr (FMT == 8) hi[f] = *(const v4i *)(lds + wfa + wbase + m * WTILE + 1024); }
                else if constexpr (m == 0) {                    // the MT scale words of the pair at once
                    if constexpr (MT == 4) { const v4i t4 = *(const v4i *)(lds + wfs + wbase); sav[nx][0] = t4[0]; sav[nx][1] = t4[1]; sav[nx][2] = t4[2]; sav[nx][3] = t4[3]; }
                    else { const int2 t2 = *(const int2 *)(lds + wfs + wbase); sav[nx][0] = t2.x; sav[nx][1] = t2.y; }
                }
            }
        };
        auto pack = [&](auto NXT) {
            constexpr int nx = decltype(NXT)::value;
#pragma unroll
            for (int f = 0; f < NT; f++) fb[nx][f] = FMT == 8 ? (v8i){lo[f][0], lo[f][1], lo[f][2], lo[f][3], hi[f][0], hi[f][1], hi[f][2], hi[f][3]} : (v8i){lo[f][0], lo[f][1], lo[f][2], lo[f][3], 0, 0, 0, 0};
#pragma unroll
            for (int m = 0; m < MT; m++) fa[nx][m] = FMT == 8 ? (v8i){lo[NT + m][0], lo[NT + m][1], lo[NT + m][2], lo[NT + m][3], hi[NT + m][0], hi[NT + m][1], hi[NT + m][2], hi[NT + m][3]} : (v8i){lo[NT + m][0], lo[NT + m][1], lo[NT + m][2], lo[NT + m][3], 0, 0, 0, 0};
        };
        constexpr int NL = 3 * (NT + MT) + 1, NM = MT * NT, NSP = NM - 3;      // the fetch is spread over the first NSP MFMAs so it has landed before the barrier
        {   // pair 0 -> register set 0
            const v4i tt2 = T;
            static_for<NL>([&](auto I) { ld(I, std::integral_constant<int, 0>{}, tt2, 0u); });
            pack(std::integral_constant<int, 0>{});
        }
        DBG_MARK(1);
        // ---- the streaming schedule. fbi: next block to request (>= nbt: of the next tile), frd: its next copy round. A block may be requested
        // once block fbi - 3, whose slot it takes, has been read for the last time (pair (27 (fbi - 3) + 26) / 2). The host has checked that
        // with two rounds per stage every block of a tile lands two barriers before its first fetch ----
        int fbi = nnext, frd = 0;                             // (blocks 0 .. nnext - 1 of this tile were requested during the tile before, or ahead of the first)
        auto prep_next = [&](hreq &q, int upto_pair) {          // prepare one copy round; pairs <= upto_pair will have been fetched by every wavefront when it is issued
            const bool go = __builtin_amdgcn_readlane(tb_gate, fbi) <= upto_pair;
            prepare(q, mask2 >> __builtin_amdgcn_readlane(tb_msh, fbi), __builtin_amdgcn_readlane(tb_base, fbi), fbi, frd, ring0, (unsigned)__builtin_amdgcn_readlane(tb_slot, fbi), go);
            const unsigned t0 = ring0;                          // a consumed round turns the ring
            ring0 = go ? ring1 : ring0; ring1 = go ? ring2 : ring1; ring2 = go ? ring3 : ring2; ring3 = go ? ring4 : ring3; ring4 = go ? t0 : ring4;
            frd += go ? 1 : 0;
            const bool wrap = frd == NRND;
            frd = wrap ? 0 : frd; fbi += wrap ? 1 : 0;
        };
        hreq rq;
        // the MFMAs of the pair in register set CUR with the fetch of the next pair (weights at ring offset wbase) between them.
        // MODE 1: also prepare the copy round the next step will issue. MODE 2: also this step's asynchronous copies, one after every
        // MFMA from the second on: the weight stage of pairs wgp, wgp + 1 into ring offset wso first, then the prepared round (so that
        // "all but the last NHC copies" means "the weights")
        auto step = [&](auto CUR, auto MODE, auto FIRST, unsigned wbase, const uint8_t *wsrc, unsigned wso, int upto_pair) {
            constexpr int cu = decltype(CUR)::value, nx = cu ^ 1, mode = decltype(MODE)::value;
            constexpr bool first = decltype(FIRST)::value;      // the tile's first pair: the accumulators start from its products
            const v4i tt2 = T;
            if constexpr (mode == 1) prep_next(rq, upto_pair);
            static_for<NM>([&](auto K) {
                constexpr int k = decltype(K)::value, m = k / NT, j = k % NT;
                const v16f c0 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                acc[m][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[cu][m], fb[cu][j], first ? c0 : acc[m][j], FMT == 8 ? 0 : 4, FMT == 8 ? 0 : 4, 0, sav[cu][m], 0, sb[cu][j]);
                constexpr int l0 = k < NSP ? (k * NL) / NSP : NL, l1 = k < NSP ? ((k + 1) * NL) / NSP : NL;
                static_for<l1 - l0>([&](auto I) { ld(std::integral_constant<int, l0 + decltype(I)::value>{}, std::integral_constant<int, nx>{}, tt2, wbase); });
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if constexpr (l1 > l0) __builtin_amdgcn_sched_group_barrier(0x100, l1 - l0, 0);
                if constexpr (mode == 1) __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);     // the preparation's arithmetic, a few instructions per MFMA
                if constexpr (mode == 2) {                      // (fenced: otherwise the scheduler lifts the copies, and the fetches ordered with them, above the MFMAs)
                    if constexpr (k >= 1 && k <= NW) { __builtin_amdgcn_sched_barrier(0); wcopy(std::integral_constant<int, k - 1>{}, wsrc, wso); __builtin_amdgcn_sched_barrier(0); }
                    if constexpr (k == NW + 2) { __builtin_amdgcn_sched_barrier(0); issue(rq); __builtin_amdgcn_sched_barrier(0); }
                }
            });
            pack(std::integral_constant<int, nx>{});
        };
        // stage s = pairs 2 s, 2 s + 1 lives in ring slot s & 1. Step 0 consumes pair 2 s and fetches pair 2 s + 1 from the same slot; after the
        // barrier every wavefront is done reading that slot, so step 1 requests stage s + 2 into it (to be there one stage later, when
        // the barrier of stage s + 1 has been passed) and two copy rounds of streaming blocks, while it consumes pair 2 s + 1 and fetches
        // pair 2 s + 2 from the other slot
        const uint8_t *wsrc = a.wq + (size_t)cur.cs * a.wstride + (size_t)2 * SLOT;      // stage s + 2 is requested during stage s
        constexpr std::integral_constant<bool, false> NOTFIRST{};
        {   // stage 0, peeled: its first step starts the accumulators
            step(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}, std::integral_constant<bool, true>{}, STG, nullptr, 0u, 1);
            wait_vm<NHC>();
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            step(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{}, NOTFIRST, SLOT, wsrc, 0u, 0);
            wsrc += SLOT;
        }
        for (int s = 1; s < nfull; s++, wsrc += SLOT) {
            const unsigned so = (s & 1) * SLOT;
            step(std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{}, NOTFIRST, so + STG, nullptr, 0u, 2 * s + 1);
            wait_vm<NHC>();                                     // the weight stage requested one stage ago is in LDS: it was issued before that step's NHC halo copies
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            step(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{}, NOTFIRST, SLOT - so, wsrc, so, 0);
        }
        if (npairs & 1) step(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, NOTFIRST, (nfull & 1) * SLOT + STG, nullptr, 0u, 0);     // the odd last pair (its fetch reads past the end: unused)
        DBG_MARK(2);
        wait_vm<0>();
        __syncthreads();                                        // every wavefront is done with the halo slots and the ring
        while (fbi <= fmax) { prep_next(rq, npairs); issue(rq); }       // (tiles too short to stream everything)
        if (nxt.ok) { wstage(0, nxt.cs, 0); wstage(1, nxt.cs, SLOT); }
        DBG_MARK(3);
        if (cur.oz0 + TZ <= a.Do && cur.oy0 + 8 <= a.Ho && cur.ox0 + 16 <= a.Wo && a.zs0 <= cur.oz0 && a.zs1 >= cur.oz0 + TZ)      // (uniform)
            conv_epilogue<MT, NT, OUT, EPI, true, true, true>(a, acc, lds, cur.tile, cur.n, cur.cs, cur.oz0, cur.oy0, cur.ox0, lz, ly0, tid);
        else conv_epilogue<MT, NT, OUT, EPI, true, true>(a, acc, lds, cur.tile, cur.n, cur.cs, cur.oz0, cur.oy0, cur.ox0, lz, ly0, tid);
        DBG_MARK(4);
        if (!nxt.ok) break;
        cur = nxt; rot = (rot + (unsigned)a.nbt) % 3u;
    }
}

template <int FMT, int OUT, bool EPI, int MT = 4>
static void launch_wide(const conv_args &a, size_t smem) {
    static bool attr[8]; static int ncu[8];
    int d = 0; MIRT(hipGetDevice(&d)); d &= 7;
    if (!attr[d]) {
        MIRT(hipFuncSetAttribute((const void *)conv3_wide_k<FMT, OUT, EPI, MT>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        hipDeviceProp_t pr; MIRT(hipGetDeviceProperties(&pr, d));
        ncu[d] = pr.multiProcessorCount > 8 ? pr.multiProcessorCount & ~7 : 8;
        attr[d] = true;
    }
    const unsigned per = (a.ntiles + 7u) / 8u;            // tiles per XCD; one persistent workgroup per CU, a multiple of 8 in all
    const unsigned nwg = per * 8u < (unsigned)ncu[d] ? per * 8u : (unsigned)ncu[d];
    conv3_wide_k<FMT, OUT, EPI, MT><<<nwg, 256, smem>>>(a);
    MICK();
    snprintf(g_last_kernel, sizeof g_last_kernel, "conv3_wide_k<fmt %d, out %d, epi %d%s> tiles %u wgs %u", FMT, OUT, (int)EPI, MT == 2 ? ", MT 2" : "", a.ntiles, nwg);
}
