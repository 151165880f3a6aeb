// Host side of the 3x3x3 MX convolutions: entry points, operand re-staging, weight preparation and memo, tile-shape selection,
// GroupNorm partial-sum reduction. The kernel itself is conv3_kernel.hpp, instantiated per (compute format, output kind) in
// conv3_f*_o*.hip.
#include "conv3_kernel.hpp"
#include <mutex>

// what a reduce block does with the (sum, sum of squares) of its (sample, group): add them to the caller's sum slots (the reference's contract,
// src/lp_common.cuh:1575-1597), or, for a fused call, set the slots and finalize mean / rstd from them right away (src/nn_elem.cu:5-11), which saves
// the zeroing and finalize launches around the conv
struct gn_fin_t { float *mean, *rstd; double len; float eps; };
__device__ __forceinline__ void gn_part_finish(double *osum, double s, double ss, gn_fin_t fin, unsigned ng) {
    const size_t i = 2 * (size_t)ng;
    if (!fin.mean) { gn_acc_add(osum, i, s); gn_acc_add(osum, i + 1, ss); return; }
    unsigned long long *w = (unsigned long long *)osum + 3 * i;
    double v[2] = {s, ss}, got[2];
#pragma unroll
    for (int k = 0; k < 2; k++) {                       // the slot a single exact add to a cleared slot would leave, and its value read back
        if (!(fabs(v[k]) < 4.611686018427387904e18)) { w[3 * k] = 0ull; w[3 * k + 1] = 0ull; w[3 * k + 2] = 1ull; got[k] = __longlong_as_double(0x7ff8000000000000ll); continue; }
        const double f = floor(v[k]);
        const unsigned long long lo = (unsigned long long)((v[k] - f) * 18446744073709551616.0);
        w[3 * k] = lo; w[3 * k + 1] = (unsigned long long)(long long)f; w[3 * k + 2] = 0ull;
        got[k] = (double)(long long)f + (double)lo * 5.42101086242752217e-20;
    }
    const double m = got[0] / fin.len, var = got[1] / fin.len - m * m;
    fin.mean[ng] = (float)m;
    fin.rstd[ng] = (float)(1.0 / sqrt((var > 0 ? var : 0) + (double)fin.eps));
}

// (sum, sum of squares) partials of the tiles -> exact GroupNorm sum slots (src/lp_common.cuh:1575-1597 does the same with one fixed-point atomic
// per block and channel). A spatial tile's record is Q = Co / 4 (padded to whole channel slices) consecutive float2, one per channel quad; quad
// Q = co / 4 lives in channel slice Q / (8 MT), slot Q % (8 MT). A block takes one sample's tiles [t0, t1) with ALL their quads: thread (j, q) adds
// quad q of tiles t0 + j, t0 + j + J, ... in double (consecutive threads read consecutive records: every fetched line is used whole), then thread
// g adds its group's quads over the J rows in a fixed order. nsplit > 1 (thousands of tiles: the level-0 layers): every block leaves its Go pairs
// in scr and takes a ticket of its sample; the block that draws the last one adds the nsplit pairs of every group in index order - the result
// does not depend on which block that is - and puts the ticket counter back to zero for the next launch
struct gn_split_t { int nsplit; double *scr; unsigned *cnt; };
__global__ void __launch_bounds__(256) gn_part_reduce_k(const float2 *part, int tiles_per_n, int ncs, int MT, int Co, int Go, double *osum, gn_fin_t fin, gn_split_t sp) {
    const int n = (int)blockIdx.x / sp.nsplit, pi = (int)blockIdx.x % sp.nsplit, tid = (int)threadIdx.x;
    const int Q = ncs * MT * 8, nst = tiles_per_n / ncs, qpg = Co / Go / 4, J = 256 / Q;
    const int per = (nst + sp.nsplit - 1) / sp.nsplit, t0 = pi * per, t1 = min(nst, t0 + per);
    const int q = tid % Q, j = tid / Q;
    const float2 *rec = part + (size_t)n * tiles_per_n * (MT * 8) + q;
    double s = 0.0, ss = 0.0;
    if (j < J) {
#pragma unroll 8
        for (int st = t0 + j; st < t1; st += J) {                            // (unrolled: the records' loads of several rounds are in flight together)
            const float2 p = rec[(size_t)st * Q];
            s += (double)p.x; ss += (double)p.y;
        }
    }
    __shared__ double r1[256], r2[256];
    __shared__ unsigned ticket;
    r1[tid] = s; r2[tid] = ss;
    __syncthreads();
    s = 0.0; ss = 0.0;
    if (tid < Go)
        for (int k = 0; k < qpg; k++)
            for (int jj = 0; jj < J; jj++) { s += r1[jj * Q + tid * qpg + k]; ss += r2[jj * Q + tid * qpg + k]; }
    if (sp.nsplit == 1) { if (tid < Go) gn_part_finish(osum, s, ss, fin, (unsigned)(n * Go + tid)); return; }
    if (tid < Go) {
        double *mine = sp.scr + 2 * ((size_t)blockIdx.x * Go + tid);
        __hip_atomic_store(mine, s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); __hip_atomic_store(mine + 1, ss, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __threadfence();                                                    // the pairs are visible device-wide before the ticket is
    }
    __syncthreads();
    if (tid == 0) ticket = atomicAdd(sp.cnt + n, 1u);
    __syncthreads();
    if (ticket != (unsigned)sp.nsplit - 1u) return;                         // (uniform over the block)
    __threadfence();                                                        // the last block of the sample: every other block's pairs are visible
    if (tid == 0) __hip_atomic_store(sp.cnt + n, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid < sp.nsplit * Go) {                                             // (nsplit Go <= 256) all pairs of the sample at once, then added in index order
        const double *theirs = sp.scr + 2 * ((size_t)n * sp.nsplit * Go + tid);
        r1[tid] = __hip_atomic_load(theirs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); r2[tid] = __hip_atomic_load(theirs + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (tid >= Go) return;
    s = 0.0; ss = 0.0;
    for (int k = 0; k < sp.nsplit; k++) { s += r1[k * Go + tid]; ss += r2[k * Go + tid]; }
    gn_part_finish(osum, s, ss, fin, (unsigned)(n * Go + tid));
}
// the same with one block per (sample, group), for records wider than a block (more than 1024 channels) or more than 256 groups
__global__ void __launch_bounds__(256) gn_part_reduce_g_k(const float2 *part, int tiles_per_n, int ncs, int MT, int Co, int Go, double *osum, gn_fin_t fin) {
    const int n = blockIdx.x / Go, gidx = blockIdx.x % Go, qpg = Co / Go / 4, nq = MT * 8, nst = tiles_per_n / ncs;
    double s = 0.0, ss = 0.0;
#pragma unroll 8
    for (int i = threadIdx.x; i < nst * qpg; i += 256) {
        const int st = i / qpg, Q = gidx * qpg + i % qpg, cs = Q / nq, qd = Q - cs * nq;
        const float2 p = part[(size_t)(n * tiles_per_n + st * ncs + cs) * nq + qd];
        s += (double)p.x; ss += (double)p.y;
    }
    __shared__ double r1[256], r2[256];
    r1[threadIdx.x] = s; r2[threadIdx.x] = ss;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) { if ((int)threadIdx.x < st) { r1[threadIdx.x] += r1[threadIdx.x + st]; r2[threadIdx.x] += r2[threadIdx.x + st]; } __syncthreads(); }
    if (threadIdx.x == 0) gn_part_finish(osum, r1[0], r2[0], fin, blockIdx.x);
}

// the same from per-channel records (32 per tile: launches whose channels per group are not a multiple of 4 run one channel tile per workgroup,
// ncs channel slices of 32 per spatial tile)
__global__ void __launch_bounds__(256) gn_part_reduce_ch_k(const float2 *part, int tiles_per_n, int ncs, int Co, int Go, double *osum, gn_fin_t fin) {
    const int n = blockIdx.x / Go, gidx = blockIdx.x % Go, cpg = Co / Go, nst = tiles_per_n / ncs;
    double s = 0.0, ss = 0.0;
    for (int i = threadIdx.x; i < nst * cpg; i += 256) {
        const int st = i / cpg, ch = gidx * cpg + i % cpg;
        const float2 p = part[((size_t)n * tiles_per_n + (size_t)st * ncs + (ch >> 5)) * 32 + (ch & 31)];
        s += (double)p.x; ss += (double)p.y;
    }
    __shared__ double r1[256], r2[256];
    r1[threadIdx.x] = s; r2[threadIdx.x] = ss;
    __syncthreads();
    for (int st = 128; st > 0; st >>= 1) { if ((int)threadIdx.x < st) { r1[threadIdx.x] += r1[threadIdx.x + st]; r2[threadIdx.x] += r2[threadIdx.x + st]; } __syncthreads(); }
    if (threadIdx.x == 0) gn_part_finish(osum, r1[0], r2[0], fin, blockIdx.x);
}

// ---- weights: fp32 w[co][ci][27] -> per (chunk, unit pair, 32-row channel tile) fragment-ordered codes + scale bytes ----
// block = the 32 ci of one (tap, co) (src/lp_f8fwd.cu:54-71, src/lp_f4fwd.cu:53-66); fmaxf amax; padded rows / channels / the odd
// padding unit are zero codes with scale byte 1
__host__ __device__ __forceinline__ int seg_ci(int cp, int Ci, int Cx, int CxP) { if (cp < CxP) return cp < Cx ? cp : -1; const int c = Cx + cp - CxP; return c < Ci ? c : -1; }
template <int FMT>
__global__ void __launch_bounds__(128) prep_w_k(const float *__restrict__ w, uint8_t *__restrict__ wq, unsigned *__restrict__ wsc, int Co, int Ci, int Cx, int CxP,
                                               int nbt, int CB, int nmt_all, int npairs_all, int block_major, int w2d) {
    constexpr int WTILE = fmt_t<FMT>::WTILE;
    const size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const int Cop = nmt_all * 32;
    if (i >= (size_t)npairs_all * Cop) return;
    const int cop = (int)(i % Cop), gp = (int)(i / Cop);
    int b0 = 0, pb = 0, nbc = 0;
    if (block_major >= 0) for (;; b0 += CB) { nbc = min(CB, nbt - b0); const int np = (27 * nbc + 1) >> 1; if (gp < pb + np) break; pb += np; }
    const int q = gp - pb, m = cop >> 5, r = cop & 31, cw = (cop & ~31) + mi_row_chan(r);       // row r of the tile carries output channel cw
    uint8_t *tile = wq + ((size_t)gp * nmt_all + m) * WTILE;
    unsigned *tsc = wsc + ((size_t)gp * nmt_all + m) * 64;      // one word per lane: the byte the MFMA reads is the low one
    int tss = 1;                                                // words between two lanes' scale words
    if (block_major > 0) {
        // the wide kernel's layout (block_major = its channel tiles per workgroup, 4 or 2): per slice of that many tiles, pair after pair the
        // image of its LDS stage: the tiles' codes, then per lane the tiles' scale words
        const int MW = block_major, sl = m / MW, mi = m - sl * MW;
        uint8_t *img = wq + ((size_t)sl * (npairs_all + 16) + gp) * (size_t)(MW * (WTILE + 256));
        tile = img + mi * WTILE; tsc = (unsigned *)(img + MW * WTILE) + mi; tss = MW;
    }
#pragma unroll
    for (int side = 0; side < 2; side++) {
        const int u = 2 * q + side;
        float v[32];
        // K order inside a chunk: tap by tap over its blocks, or (the wide kernel, one chunk) block by block over the taps; the row kernel
        // (block_major -1): per block 15 pairs (class c, ky), class c < 3 = taps (c, ky, 0 | 1), class 3 = (0 | 1, ky, 2), class 4 = (2, ky, 2 | none);
        // the direct stride-2 kernel (block_major -2): mi_s2_unit
        int t = block_major ? u % 27 : u / nbc, blk = block_major ? u / 27 : b0 + u % nbc;
        bool unit_ok = u < 27 * nbc;
        if (block_major == -2) unit_ok = mi_s2_unit(gp, side, nbt, &t, &blk);
        else if (block_major < 0) {
            const int qq = gp % 15, c = qq / 3, ky = qq % 3;
            blk = gp / 15;
            const int kz = c < 3 ? c : c == 3 ? side : 2, kx = c < 3 ? side : 2;
            t = kz * 9 + ky * 3 + kx;
            unit_ok = !(c == 4 && side == 1);
        }
#pragma unroll
        for (int k = 0; k < 32; k++) {
            const int ci = seg_ci(blk * 32 + k, Ci, Cx, CxP);
            v[k] = (unit_ok && cw < Co && ci >= 0) ? w[((size_t)cw * Ci + ci) * 27 + t] : 0.f;
        }
        prep_store_unit<FMT>(tile, tsc, tss, side, r, v, w2d != 0);      // (32 consecutive threads hold a channel tile's rows of this pair)
    }
}

// ---- prepared-weight memo (src/lp_f4fwd.cuh:748-770): keyed by the conv id sp.wkey and the layout ----
// (lay: what else fixes the image's layout: the wide kernel's channel tiles per workgroup, which follow the launch's tile count and mi_conv_split; 0 otherwise)
struct wmemo_t { unsigned key; const float *w; int fmt, Co, Ci, Cx, nbt, CB, nmt_all, dev, lay; uint8_t *wq, *wsc; };
static std::vector<wmemo_t> g_wmemo;
static std::mutex g_wmemo_mu;      // host threads driving different devices share the list (one thread per device: the per-device scratch is not guarded)
static unsigned g_wstep = 0;
void mx_gemm_memo_clear(void);
extern "C" void lp_wmemo_clear(void) {
    MIRT(hipDeviceSynchronize());
    mx_gemm_memo_clear();
    std::lock_guard<std::mutex> lk(g_wmemo_mu);
    if (g_wmemo.empty()) return;
    for (auto &m : g_wmemo) { MIRT(hipFree(m.wq)); MIRT(hipFree(m.wsc)); }
    g_wmemo.clear();
}
// 2-D fp4 weight scales (src/lp_f4fwd.cu:4, :67-83): one E8M0 scale per tap and 32 x 32 (output x input channel) tile instead of per output
// channel; a setting change drops the prepared weights. Default from UFSM_W4_2D, as the reference
static int g_w2d = -1;
static int g_w2d_on(void) { if (g_w2d < 0) g_w2d = getenv("UFSM_W4_2D") ? atoi(getenv("UFSM_W4_2D")) : 0; return g_w2d; }
extern "C" void lp_set_w4_2d(int on) { g_w2d = on ? 1 : 0; lp_wmemo_clear(); }
extern "C" void lp_wmemo_step(unsigned step) { if (step != g_wstep) { g_wstep = step; lp_wmemo_clear(); } }
// memo entries of the layouts other source files prepare (the 2x2x2 stride-2 convs: nbt = -100, lay = down / up): the image's buffers for
// (key, weights, format, shape, lay) on the current device, allocated on first use; returns whether they already hold the prepared image
bool mi_wmemo_other(unsigned key, const float *w, int fmt, int Co, int Ci, int nmt_all, int lay, size_t wq_bytes, size_t wsc_bytes, uint8_t **wq, uint8_t **wsc) {
    int dev = 0; MIRT(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_wmemo_mu);
    for (auto &m : g_wmemo)
        if (m.key == key && m.w == w && m.fmt == fmt && m.Co == Co && m.Ci == Ci && m.nbt == -100 && m.nmt_all == nmt_all && m.dev == dev && m.lay == lay) { *wq = m.wq; *wsc = m.wsc; return true; }
    MIRT(hipMalloc((void **)wq, wq_bytes)); MIRT(hipMalloc((void **)wsc, wsc_bytes)); mi_count_alloc(); mi_count_alloc();
    if (!*wq || !*wsc) mi_die("no device memory for the prepared weights of a 2x2x2 conv");
    g_wmemo.push_back(wmemo_t{key, w, fmt, Co, Ci, Ci, -100, 0, nmt_all, dev, lay, *wq, *wsc});
    return false;
}

thread_local char g_last_kernel[128] = "";

// optional timing of the conv kernel launches alone (benchmarks): event pairs on the stream the kernel runs on
static bool g_ktime = false;
struct kev_t { hipEvent_t e0, e1; double flops; char name[96]; };
static std::vector<kev_t> g_kev;
static double g_kms = 0.0; static long g_kn = 0;
struct klaunch_t { float ms; double flops; char name[96]; };
static std::vector<klaunch_t> g_klog;             // every timed launch since mi_kernel_timing(1), in launch order
extern "C" void mi_kernel_timing(int on) {
    for (auto &e : g_kev) { MIRT(hipEventDestroy(e.e0)); MIRT(hipEventDestroy(e.e1)); }
    g_kev.clear(); g_klog.clear(); g_kms = 0.0; g_kn = 0; g_ktime = on != 0;
}
static void ktime_collect() {
    for (auto &e : g_kev) {
        float ms = 0.f;
        MIRT(hipEventSynchronize(e.e1)); MIRT(hipEventElapsedTime(&ms, e.e0, e.e1));
        g_kms += ms; g_kn++;
        klaunch_t l; l.ms = ms; l.flops = e.flops; memcpy(l.name, e.name, sizeof l.name); g_klog.push_back(l);
        MIRT(hipEventDestroy(e.e0)); MIRT(hipEventDestroy(e.e1));
    }
    g_kev.clear();
}
extern "C" double mi_kernel_timing_read(long *launches) {       // total milliseconds of the timed launches so far (synchronises)
    ktime_collect();
    if (launches) *launches = g_kn;
    return g_kms;
}
extern "C" long mi_kernel_timing_launch(long i, float *ms, double *flops, char *name, size_t name_bytes) {     // launch i of the log; returns the log's length (synchronises)
    ktime_collect();
    if (i >= 0 && i < (long)g_klog.size()) {
        if (ms) *ms = g_klog[i].ms;
        if (flops) *flops = g_klog[i].flops;
        if (name && name_bytes) { strncpy(name, g_klog[i].name, name_bytes - 1); name[name_bytes - 1] = 0; }
    }
    return (long)g_klog.size();
}
static void ktime_push(hipEvent_t ev0, hipEvent_t ev1, double flops) {
    kev_t k; k.e0 = ev0; k.e1 = ev1; k.flops = flops;
    strncpy(k.name, g_last_kernel, sizeof k.name - 1); k.name[sizeof k.name - 1] = 0;
    g_kev.push_back(k);
}
extern "C" const char *mi_last_kernel(void) { return g_last_kernel; }

// the conv of every entry point: fmt 8 / 4 = compute format, stride 1 / 2
// set by mi_conv_fwd_gn around its conv: finalize the statistics in the reduce kernel
static thread_local gn_fin_t g_fin = {nullptr, nullptr, 0.0, 0.f};
// GroupNorm partial sums of a conv's tiles -> the caller's sum slots (and mean / rstd when mi_conv_fwd_gn asked for them)
static void conv_stats_reduce(const char *who, const conv_args &a, int MT, split_t sp, double *osum) {
    gn_fin_t fin = g_fin;
    fin.len = (double)(a.Co / a.Go) * (double)a.Do * a.Ho * a.Wo;
    if (fin.mean && (sp.zlo || sp.zhi)) mi_die("%s: fused finalize with a z range", who);
    if (a.stat_ch) { gn_part_reduce_ch_k<<<a.N * a.Go, 256>>>((const float2 *)a.part, (int)(a.ntiles / a.N), a.ncs, a.Co, a.Go, osum, fin); MICK(); return; }
    const int tiles_per_n = (int)(a.ntiles / a.N) * (a.row1 ? 8 : 1);      // (row1: eight records per tile)
    const int Q = a.ncs * MT * 8, nst = tiles_per_n / a.ncs;
    if (Q > 256 || a.Go > 256) { gn_part_reduce_g_k<<<a.N * a.Go, 256>>>((const float2 *)a.part, tiles_per_n, a.ncs, MT, a.Co, a.Go, osum, fin); MICK(); return; }
    // thousands of tiles per sample: several blocks each (512 tiles or more per block), folded by the last one done. The pairs and ticket
    // counters live in a small buffer per device, allocated on first use and left zeroed by every launch (the entry point that must not
    // allocate keeps one block per sample)
    gn_split_t gs = {1, nullptr, nullptr};
    constexpr int MAXN = 4096, SCR = 1 << 17;                  // samples with a ticket counter; doubles of scratch
    int want = nst < 4096 ? 1 : nst / 512 < 32 ? nst / 512 : 32;          // (the ticket and the fold cost 2 - 3 us: a single pass is faster below a few thousand tiles)
    if (want * a.Go > 256) want = 256 / a.Go;
    while (want > 1 && (size_t)a.N * want * a.Go * 2 > (size_t)SCR) want >>= 1;
    if (want > 1 && a.N <= MAXN && !mi_ws_arena_on()) {
        static double *scr[8]; static unsigned *cnt[8];
        int dv = 0; MIRT(hipGetDevice(&dv)); dv &= 7;
        if (!scr[dv]) {
            MIRT(hipMalloc((void **)&scr[dv], (size_t)SCR * sizeof(double))); MIRT(hipMalloc((void **)&cnt[dv], MAXN * sizeof(unsigned))); mi_count_alloc(); mi_count_alloc();
            if (!scr[dv] || !cnt[dv]) mi_die("%s: no device memory for the statistics fold", who);
            MIRT(hipMemset(cnt[dv], 0, MAXN * sizeof(unsigned)));
        }
        gs.nsplit = want; gs.scr = scr[dv]; gs.cnt = cnt[dv];
    }
    gn_part_reduce_k<<<a.N * gs.nsplit, 256>>>((const float2 *)a.part, tiles_per_n, a.ncs, MT, a.Co, a.Go, osum, fin, gs);
    MICK();
}

// the tap-packed stem (src/lp_f8fwd.cuh:601-609, :421-434): e4m3 compute, one activation scale per staged tile
// rows: the 9 .. 16 channel form, two taps per K block and one activation scale per staged row (src/lp_f8fwd.cuh:447-563, :626)
static thread_local int g_stem_zc = 0;      // tuning knob (mi_conv_stem_zc): z tiles per workgroup of the tap-packed kernel, 0 = chosen from the launch size
static int conv_stem(const char *who, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf,
                     gnp_t gp, double *osum, int Go, split_t sp, bool rows) {
    const int Ci = xs.c, N = xs.n, D = sp.Di ? sp.Di : xs.d, Do = xs.d, H = xs.h, W = xs.w;      // D: the input's depth (z-range), Do: output planes
    if (gp.G && gp.ns && (gp.zs <= 0 || gp.zo < 0 || gp.zo >= gp.zs || gp.zhw != H * W || gp.ns > 256))
        mi_die("%s: slab-local GroupNorm geometry (zs %d, zo %d, ns %d, zhw %d) does not fit planes of %d voxels (at most 256 slabs)", who, gp.zs, gp.zo, gp.ns, gp.zhw, H * W);
    const int CP = rows ? 0 : Ci <= 4 ? 4 : Ci <= 8 ? 8 : 16, TPK = rows ? 2 : 32 / CP, NKB = rows ? 18 : (27 + TPK - 1) / TPK, NP = (NKB + 1) / 2;
    conv_args a; memset(&a, 0, sizeof a);
    a.sx = x; a.sxdt = xbf; a.sCi = Ci;
    a.sgam = gp.gamma; a.sbet = gp.beta; a.smean = gp.mean; a.srstd = gp.rstd; a.sG = gp.G;
    if (gp.G && gp.ns) { a.szs = gp.zs; a.szo = gp.zo; a.sns = gp.ns; }      // (each slab's coefficient table in LDS: the staged positions take their plane's)
    a.N = N; a.D = D; a.H = H; a.W = W; a.Do = Do; a.Ho = H; a.Wo = W;
    a.zi0 = sp.Di ? sp.zi0 : 0; a.yD = sp.yD; a.yzo = sp.yD ? sp.yzo : 0;
    a.bias = b; a.Co = cout; a.y = y; a.ydt = ybf;
    a.osum = osum; a.Go = Go; a.stored_stats = sp.stored_stats && ybf >= 3; a.zs0 = sp.zlo; a.zs1 = Do - sp.zhi;
    // (16 channels per slot: 7 or 9 weight fragment pairs per channel tile, one tile fits the registers; per-channel statistics records: one tile per workgroup)
    const int nmt_all = (cout + 31) / 32, MT = nmt_all % 2 == 0 && CP && CP < 16 && !(osum && (cout / Go) % 4) ? 2 : 1;
    size_t smem = rows ? (size_t)720 * 16 + 16 + 40 * 4 + 16 * 8 : ((size_t)720 * CP + 16 + CP * 8 + 15) & ~(size_t)15;     // staged tile, (zero row, row words | amax word), channel affine
    if (a.sns > 1) smem += (size_t)(a.sns - 1) * (rows ? 16 : CP) * 8;      // (one affine table per slab)
    a.epi_o = (unsigned)smem; smem += (size_t)3 * MT * 32 * sizeof(float);
    a.red_o = (unsigned)smem; smem += 1024;
    a.nmt_all = nmt_all; a.ncs = nmt_all / MT;
    a.ntx = (W + 15) / 16; a.nty = (H + 7) / 8; a.ntz = (Do + 1) / 2;
    a.ntiles = (unsigned)((size_t)a.ntx * a.nty * a.ntz * a.ncs * N);
    // z tiles per workgroup (tap-packed kernel: the set-up is amortised, the next tile's loads overlap): up to 8 while >= 8 workgroups per CU remain
    a.zc = 1;
    if (!rows && CP <= 4 && g_stem_zc > 0) a.zc = g_stem_zc < a.ntz ? g_stem_zc : a.ntz;
    else if (!rows && CP <= 4) { a.zc = 8; while (a.zc > 1 && (size_t)a.ntx * a.nty * ((a.ntz + a.zc - 1) / a.zc) * a.ncs * N < 2048) a.zc--; }
    a.ngrp = (unsigned)((size_t)a.ntx * a.nty * ((a.ntz + a.zc - 1) / a.zc) * a.ncs * N);
    const size_t wq_bytes = (size_t)NP * nmt_all * 2048, wsc_bytes = (size_t)NP * nmt_all * 256;
    int dev = 0; MIRT(hipGetDevice(&dev));
    uint8_t *wq = nullptr, *wsc = nullptr; bool have = false;
    if (sp.wkey && !mi_ws_arena_on()) {                // memo entries of this layout: nbt = -CP (the entry point that must not allocate prepares per call)
        std::lock_guard<std::mutex> lk(g_wmemo_mu);
        for (auto &m : g_wmemo)
            if (m.key == sp.wkey && m.w == w && m.fmt == 8 && m.Co == cout && m.Ci == Ci && m.nbt == -CP - 1 && m.nmt_all == nmt_all && m.dev == dev) { wq = m.wq; wsc = m.wsc; have = true; break; }
        if (!have) {
            MIRT(hipMalloc((void **)&wq, wq_bytes)); MIRT(hipMalloc((void **)&wsc, wsc_bytes)); mi_count_alloc(); mi_count_alloc();
            if (!wq || !wsc) mi_die("%s: no device memory for the prepared weights", who);
            g_wmemo.push_back(wmemo_t{sp.wkey, w, 8, cout, Ci, Ci, -CP - 1, 0, nmt_all, dev, 0, wq, wsc});
        }
    } else { wq = (uint8_t *)mi_ws(MI_WS_WQ, wq_bytes); wsc = (uint8_t *)mi_ws(MI_WS_WSC, wsc_bytes); }
    if (!have) conv3_stem_prep(CP, w, wq, wsc, cout, Ci, nmt_all, NP);
    a.wq = wq; a.wsc = wsc;
    a.stat_ch = osum && (cout / Go) % 4 ? 1 : 0;
    if (osum) a.part = (float *)mi_ws(MI_WS_MISC, (size_t)a.ntiles * (a.stat_ch ? 32 : a.row1 ? 64 : MT * 8) * 2 * sizeof(float));      // (row1: a record per wavefront, eight per tile)
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    const bool ktime = g_ktime && !mi_ws_arena_on();
    if (ktime) { MIRT(hipEventCreate(&ev0)); MIRT(hipEventCreate(&ev1)); MIRT(hipEventRecord(ev0, 0)); }
    conv3_stem_launch(CP, MT, ybf == 3 ? 8 : ybf == 4 ? 4 : 0, a, smem);
    if (ktime) { MIRT(hipEventRecord(ev1, 0)); ktime_push(ev0, ev1, 2.0 * 27 * Ci * (double)cout * N * Do * H * W); }
    if (osum) conv_stats_reduce(who, a, MT, sp, osum);
    return 0;
}

static thread_local const uint8_t *g_static_zpage = nullptr;     // the constant page of the calling thread's conv when it runs on the fixed scratch
static thread_local int g_split = -1;       // mi_conv_split: the calling thread's tile count below which 128-channel slices are halved (-1: the default)
extern "C" void mi_conv_split(int tiles) { g_split = tiles; }
// storage format of the calling thread's next split conv's second segment when it differs from the first's (3 MX-fp8, 4 MX-fp4; the descriptor
// carries one format for both); 0 = the same
static thread_local int g_x2_dt = 0;
extern "C" void mi_conv_x2_dt(int dt) { g_x2_dt = dt == 3 || dt == 4 ? dt : 0; }
static thread_local int g_s2d = -1;         // mi_conv_s2_direct: the calling thread's choice of stride-2 kernel (-1: by launch size)
extern "C" void mi_conv_s2_direct(int mode) { g_s2d = mode; }
static int split_s2_env() { static int v = -1; if (v < 0) v = getenv("MI_CONV_SPLIT_S2") ? atoi(getenv("MI_CONV_SPLIT_S2")) : 1; return v; }      // tuning knob: 0 keeps four channel tiles
static int conv_dispatch(const char *who, int fmt, int stride, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf,
                         gnp_t gp, double *osum, int Go, split_t sp, const float *ep_a, const float *ep_b, int act) {
    if (sp.y2 || sp.o_split || sp.accum || sp.sr || sp.osr || sp.o_pad || sp.zw0 || sp.zw1)
        mi_die("%s: split outputs, accumulate, stochastic rounding and the z-window fields of split_t are not built here (inference forward only)", who);
    // z-range (src/nn_lp.h:36-40, src/nn_bwd.cu:33-36): the xs.d output planes read input plane z + zi0 of depth-Di inputs; direct slab output:
    // the MX output is planes [yzo, yzo + xs.d) of a depth-yD tensor
    if ((sp.Di || sp.zi0) && (stride != 1 || sp.zi0 < 0 || sp.zi0 + xs.d > sp.Di)) mi_die("%s: z-range %d + %d of depth %d (stride %d)", who, sp.zi0, xs.d, sp.Di, stride);
    if ((sp.yD || sp.yzo) && (stride != 1 || sp.yzo < 0 || sp.yzo + xs.d > sp.yD)) mi_die("%s: slab output %d + %d of depth %d (stride %d)", who, sp.yzo, xs.d, sp.yD, stride);
    // slab-local GroupNorm statistics (gnp_t.ns > 0, src/nn_lp.h:15-18): every GroupNorm + SiLU of a conv input is applied by the re-staging pass
    // below, which runs once per slab the launch's input planes meet; the kernels never see statistics
    if (gp.ns && sp.up) mi_die("%s: slab-local GroupNorm statistics on the upsampled segment are not supported (the skip segment's are)", who);
    // the op layer's masks and z-window (the reference's kernels ask the same before a launch: src/lp_f4fwd.cuh:1134-1223, src/nn_bwd.cu:89)
    { int za = 0, zb = 0; if (zw_win(xs.d, &za, &zb)) mi_die("%s: a z-window [%d, %d) is set; windows are not built here (inference forward only)", who, za, zb); }
    if (lp_skip_get(xs, sp, 1).m || nn_skip_masks(xs, sp)) mi_die("%s: the op layer asks for a masked (skip-empty) conv, which is not built here", who);
    if (xbf < 0 || xbf > 4 || !(ybf == 0 || ybf == 2 || ybf == 3 || ybf == 4)) mi_die("%s: unsupported storage types (in %d, out %d)", who, xbf, ybf);
    if (xs.n <= 0 || xs.c <= 0 || xs.d <= 0 || xs.h <= 0 || xs.w <= 0 || cout <= 0) return 0;
    const int Ci = xs.c, Cx = sp.x2 ? sp.c_split : Ci, C2 = Ci - Cx;
    const int entry_fmt = fmt;
    if (fmt == 4 && Ci <= 8) fmt = 8;                  // the network input computes in e4m3 whatever the activations' format (src/lp_f4fwd.cu:37)
    if (sp.x2 && (Cx <= 0 || C2 <= 0)) mi_die("%s: channel split %d of %d", who, sp.c_split, Ci);
    if (sp.x2 && xbf < 3) mi_die("%s: split inputs need MX storage", who);
    if (sp.up && (!sp.x2 || xbf < 3 || ((sp.Di ? sp.Di : xs.d) & 1) || (xs.h & 1) || (xs.w & 1) || stride != 1)) mi_die("%s: the fused upsample needs an MX split input and even dims", who);
    if (osum && (Go <= 0 || cout % Go)) mi_die("%s: %d output channels in %d groups", who, cout, Go);
    if (gp.G > 0 && ((sp.x2 && sp.gp2.G ? Cx : Ci) % gp.G)) mi_die("%s: GroupNorm groups %d do not divide the channels", who, gp.G);
    if (sp.gp2.G > 0 && (!sp.x2 || C2 % sp.gp2.G)) mi_die("%s: second GroupNorm without a matching x2 segment", who);
    // few input channels: the tap-packed kernel with one activation scale per tile (src/lp_f8fwd.cuh:601-609: up to 8 channels of a 16-bit or
    // MX input, 16 of an fp32 one; same input and output type, or an MX output)
    static int stem_env = -1;
    if (stem_env < 0) stem_env = getenv("MI_CONV_STEM") ? atoi(getenv("MI_CONV_STEM")) : 1;     // tuning knob: 0 sends these convs to the general kernel
    if (stem_env && fmt == 8 && stride == 1 && !sp.x2 && !act && (xbf == 0 || xbf >= 2) && Ci <= (xbf == 0 ? 16 : 8) && (xbf == ybf || ybf >= 3))
        return conv_stem(who, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp, false);
    // 9 .. 16 channels of an MX or fp16 input: two taps per K block, one activation scale per staged row (src/lp_f8fwd.cuh:626)
    if (stem_env && fmt == 8 && stride == 1 && !sp.x2 && !act && xbf >= 2 && Ci <= 16 && (xbf == ybf || ybf >= 3))
        return conv_stem(who, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp, true);
    const int N = xs.n, D = sp.Di ? sp.Di : xs.d, H = xs.h, W = xs.w;           // D: the inputs' depth
    const int Do = stride == 2 ? (D - 1) / 2 + 1 : xs.d, Ho = stride == 2 ? (H - 1) / 2 + 1 : H, Wo = stride == 2 ? (W - 1) / 2 + 1 : W;   // src/nn_bwd.cu:132-135
    const size_t S = (size_t)D * H * W;
    const int zlo = sp.Di ? (sp.zi0 > 0 ? sp.zi0 - 1 : 0) : 0, zhi = sp.Di ? (sp.zi0 + xs.d + 1 < D ? sp.zi0 + xs.d + 1 : D) : D;      // input planes this launch reads
    const int fdt = fmt == 8 ? 3 : 4;
    conv_args a; memset(&a, 0, sizeof a);
    // ---- operands: a segment is read as stored when it already is the compute format with nothing to apply, else re-staged once ----
    // (gp2.G < 0, an extension: x2 carries no GroupNorm and gp is x's own; the reference's gp2.G == 0 means gp spans both segments)
    const bool s2g = sp.x2 && sp.gp2.G;
    if (sp.gp2.G < 0) sp.gp2 = gnp_mk(nullptr, nullptr, nullptr, nullptr, 0);
    const void *segx[2] = {x, sp.x2}; const int segC[2] = {Cx, C2};
    const int segbf[2] = {xbf, sp.x2 && g_x2_dt ? g_x2_dt : xbf};
    g_x2_dt = 0;
    for (int s = 0; s < (sp.x2 ? 2 : 1); s++) {
        const gnp_t g = s2g ? (s ? sp.gp2 : gp) : gp;
        const int Cg = s2g ? segC[s] : Ci, cg0 = s2g ? 0 : (s ? Cx : 0);
        const bool upseg = s == 0 && sp.up;
        const int xbf = segbf[s];                                 // (this segment's storage format)
        const bool direct = xbf == fdt && !g.G && !upseg;
        const int nbp = (segC[s] + 31) / 32;
        if (direct) {
            const int bw = mx_bw(segC[s]), nb = mx_nb(segC[s]);
            a.xq[s] = (const uint8_t *)segx[s]; a.xsc[s] = a.xq[s] + (size_t)N * nb * S * mx_rb(bw, fmt);
            a.nbs[s] = nb; a.bws[s] = bw;
        } else {
            const size_t bytes = (size_t)N * nbp * S * (mx_rb(32, fmt) + 1);
            uint8_t *st = (uint8_t *)mi_ws(s ? MI_WS_X2STAGE : MI_WS_XSTAGE, bytes);
            // the fp4 entry blends the upsample in binary16 unless UFSM_UP_H2=0 (src/lp_f4fwd.cuh:1135-1136); sp.up 2 / 3 force one blend
            static int uph2 = -1;
            if (uph2 < 0) uph2 = getenv("UFSM_UP_H2") ? atoi(getenv("UFSM_UP_H2")) : 1;
            if (upseg) mi_restage_up_sub(segx[s], xbf, N, segC[s], D, H, W, g, Cg, st, fmt, zlo, zhi, sp.up == 2 || (sp.up == 1 && entry_fmt == 4 && uph2));
            else gn_for_slabs(who, g, H * W, zlo, zhi, [&](int z0, int z1, gnp_t gs) { mi_restage_sub(segx[s], xbf, N, segC[s], (size_t)(z1 - z0) * H * W, gs, Cg, cg0, st, fmt, S, (size_t)z0 * H * W); });
            a.xq[s] = st; a.xsc[s] = st + (size_t)N * nbp * S * mx_rb(32, fmt);
            a.nbs[s] = nbp; a.bws[s] = 32;
        }
        if (s == 0) a.nb0p = nbp;
    }
    a.nbt = a.nb0p + (sp.x2 ? (C2 + 31) / 32 : 0);
    a.wide = a.bws[0] == 32 && (!sp.x2 || a.bws[1] == 32);
    a.N = N; a.D = D; a.H = H; a.W = W; a.Do = Do; a.Ho = Ho; a.Wo = Wo;
    a.zi0 = sp.Di ? sp.zi0 : 0; a.yD = sp.yD; a.yzo = sp.yD ? sp.yzo : 0;
    a.bias = b; a.Co = cout; a.y = y; a.ydt = ybf;
    a.osum = osum; a.Go = Go; a.stored_stats = sp.stored_stats && ybf >= 3; a.zs0 = sp.zlo; a.zs1 = Do - sp.zhi;
    a.ep_a = ep_a; a.ep_b = ep_b; a.act = act;
    // ---- tile shape: MT channel tiles of 32 per workgroup, NT voxel tiles of 32 per wavefront, MT * NT <= 8 accumulators ----
    const int nmt_all = (cout + 31) / 32;
    int MT = nmt_all <= 4 ? nmt_all : nmt_all % 4 == 0 ? 4 : nmt_all % 3 == 0 ? 3 : nmt_all % 2 == 0 ? 2 : 1;
    // channels per group not a multiple of 4 (80 channels in 8 groups): the statistics are per-channel records of one channel tile per workgroup
    if (osum && (cout / Go) % 4) MT = 1;
    bool halved = false;
    {   // few tiles of 128 channels (the coarse levels): slices of 64 channels double the workgroups of the wide kernel
        static int split_env = -1;
        if (split_env < 0) split_env = getenv("MI_CONV_SPLIT") ? atoi(getenv("MI_CONV_SPLIT")) : 192;    // tuning knob: tile count below which the slices are halved (0: never)
        const int split = g_split >= 0 ? g_split : split_env;
        if (stride == 1 && MT == 4 && nmt_all % 4 == 0 && Do >= 3 &&
            (size_t)((Wo + 15) / 16) * ((Ho + 7) / 8) * ((Do + 3) / 4) * (nmt_all / 4) * N < (size_t)split) { MT = 2; halved = true; }
    }
    int NT = (stride == 1 && MT <= 2 && Do >= 4) ? 4 : 2;
    // ... and when even the slices of 64 give fewer than 128 workgroups (256 -> 256 at 2 x 16^3: 64): one channel tile and two planes per workgroup
    // on the general kernel, four times the workgroups (measured in the 32/64/128/256 forward: 128 -> 256 0.032 -> 0.026 ms, 256 -> 256
    // 0.050 -> 0.038 ms; from 256 slices of 64 on, the wide kernel is the faster one: 128 -> 128 at 2 x 32^3 0.034 against 0.052 ms)
    bool coarse = false;
    {
        static int ce = -1;
        if (ce < 0) ce = getenv("MI_CONV_COARSE") ? atoi(getenv("MI_CONV_COARSE")) : 1;      // tuning knob: 0 keeps the wide kernel's slices of 64 there (as does a split forced through mi_conv_split)
        if (ce && halved && g_split < 0 && (size_t)((Wo + 15) / 16) * ((Ho + 7) / 8) * ((Do + 3) / 4) * (nmt_all / 2) * N < 128) { coarse = true; NT = 2; MT = 1; halved = false; }
    }
    // stride 2 with few tiles (the coarse levels): one-plane tiles double the workgroups; with enough tiles the two-plane tile is faster
    // (measured: 128 -> 128 at 32^3 -> 16^3, N 2: 32 tiles 0.072 ms, 64 tiles 0.042 ms; 32 -> 32 at 128^3: 0.090 vs 0.120 ms)
    if (stride == 2 && (MT == 1 || MT == 2 || MT == 4) &&
        (size_t)((Wo + 15) / 16) * ((Ho + 7) / 8) * ((Do + 1) / 2) * (nmt_all / MT) * N < 256) NT = 1;
    // ... and still fewer one-plane tiles than half the CUs: two channel tiles per workgroup instead of four
    if (stride == 2 && MT == 4 && NT == 1 && split_s2_env() && (size_t)((Wo + 15) / 16) * ((Ho + 7) / 8) * Do * (nmt_all / 4) * N < 128) MT = 2;
    // ... and one while two would still leave CUs idle (128 -> 128 from 2 x 32^3: 128 workgroups 0.035 ms, 256 workgroups 0.024 ms; the two-plane
    // tiles of 64 -> 64 from 2 x 64^3, 256 workgroups, are the fastest form there: 0.030 ms against 0.039 with 512 one-plane tiles)
    if (stride == 2 && MT == 2 && NT == 1 && split_s2_env() && (size_t)((Wo + 15) / 16) * ((Ho + 7) / 8) * Do * (nmt_all / 2) * N < 256) MT = 1;
    // stride 2 on 32-channel rows with enough output voxels (four workgroups per CU or more): the kernel that reads every tap's rows straight from
    // the stored tensor (no staged halo). Measured in the 32/64/128/256 forward at 2 x 128^3: 32 -> 32 from 128^3 0.093 -> 0.071 ms; 64 -> 64 from
    // 64^3 is slower there, 0.030 -> 0.037 ms, and stays with the general kernel. Runs of 64 output voxels per wavefront; channel tiles per
    // workgroup halved while fewer than two workgroups per CU would run
    static int s2d_env = -1;
    if (s2d_env < 0) s2d_env = getenv("MI_CONV_S2D") ? atoi(getenv("MI_CONV_S2D")) : 8;       // tuning knob: 0 keeps the general kernel for stride 2, else the launch size (in units of 128 workgroups of 256 output voxels) from which the direct kernel runs
    const size_t s2runs = ((size_t)Do * Ho * Wo + 63) / 64;
    // (by default only one input block and one channel tile, the shape it is measured faster on: 64 -> 64 takes 0.034 against 0.030 ms from 2 x 64^3
    // and 0.36 against 0.09 ms from 8 x 64^3)
    const bool s2d = s2d_env && g_s2d != 0 && stride == 2 && a.wide && !act && N <= 65535 &&
                     (g_s2d > 0 || (a.nbt == 1 && nmt_all == 1 && (s2runs + 3) / 4 * N >= (size_t)s2d_env * 128));
    if (s2d) {
        MT = nmt_all % 4 == 0 ? 4 : nmt_all % 2 == 0 ? 2 : 1;
        while (MT > 1 && (s2runs + 3) / 4 * (size_t)(nmt_all / MT) * N < 512) MT >>= 1;
        NT = 2;
    }
    // 128-channel output slices at stride 1 take the wide kernel (16 accumulators per wavefront, one workgroup per CU)
    static int big_env = -1;
    if (big_env < 0) big_env = getenv("MI_CONV_WIDE") ? atoi(getenv("MI_CONV_WIDE")) : 1;      // tuning knob: 0 keeps the 8-accumulator kernel, 2 sends every 64-channel layer to the wide kernel too
    // (64 output channels: two channel tiles per workgroup; it pays from four input blocks on: 192 -> 64 at 2 x 64^3 0.190 -> 0.178 ms, 64 -> 64 the same
    // as the general kernel. MI_CONV_WIDE=2 sends every such layer there)
    static int rowcs4_env = -1;
    if (rowcs4_env < 0) rowcs4_env = getenv("MI_CONV_ROW_CS4") ? atoi(getenv("MI_CONV_ROW_CS4")) : 1;      // tuning knob: input blocks up to which 65 .. 128 output channels run the row kernels as three or four slices (0: never).
    // Measured: 32 -> 128 at 2 x 64^3 0.079 -> 0.064 ms on the one-block kernel; from two blocks on the wide kernel is as fast (64 -> 128 and 128 -> 128 at 2 x 32^3)
    // or faster (e2m1 at 32 x 32^3: 0.151 against 0.164 ms), hence 1
    const bool row_cs4 = rowcs4_env > 0 && g_split < 0 && (nmt_all == 3 || nmt_all == 4) && a.nbt <= rowcs4_env && stride == 1 && !coarse && a.wide && Wo > 16 && Do >= 4 && !(osum && (cout / Go) % 4);
    if (row_cs4) { MT = 1; NT = 4; halved = false; }
    bool big = !row_cs4 && !coarse && big_env && stride == 1 && (MT == 4 || (MT == 2 && (big_env > 1 || a.nbt >= 4 || halved))) && Do >= 3 && a.wide && a.nbt <= 12;            // (its per-tile pair table must fit LDS)
    if (big) {
        // The wide kernel streams input block b >= 2 of a tile into LDS while the tile's earlier blocks are multiplied, one copy round per
        // stage of two pairs, NRND rounds per block, a block starting once block b - 3 has been read for the last time (pair (27 (b - 3) + 26) / 2).
        // A round issued in stage s is visible two barriers later. Check that every block lands before the step that first fetches from it.
        const int NRND = ((6 * 10 * 18 + 63) / 64 + 3) / 4, npairs = (27 * a.nbt + 1) >> 1, nfull = npairs >> 1;
        int fbi = 2, frd = 0;
        for (int s = 0; s < nfull && big; s++) {
            if (fbi < a.nbt && (fbi < 3 || ((27 * (fbi - 3) + 26) >> 1) <= 2 * s + 1) && ++frd == NRND) {
                const int pf = ((27 * fbi) >> 1) - 1;               // the pair during which the block's first fragments are fetched
                const int need = pf & 1 ? (pf >> 1) - 2 : (pf >> 1) - 3;
                if (s > need) big = false;
                frd = 0; fbi++;
            }
        }
        if (fbi < a.nbt) big = false;
    }
    if (big) NT = 4;
    const int TZ = NT == 1 ? 1 : NT == 2 ? 2 : 4;
    const int HZ = stride * (TZ - 1) + 3, HY = stride * 7 + 3, HX = stride * 15 + 3, TT = HZ * HY * HX;
    const int RB = fmt == 8 ? 32 : 16, WTILE = fmt == 8 ? 2048 : 1024;
    // LDS of a workgroup holding CB input blocks: weight ring, pair table, halo rows and scale words. Prefer the largest CB that
    // still lets two workgroups share a CU (160 KB): the second one computes while the first stages its halo or runs its epilogue.
    // The wide kernel has a fixed layout: ring of two slots of two pairs, three halo slots of one block, two pair tables.
    const int PPS = MT == 1 ? 7 : MT == 2 ? 2 : 1;        // pairs per ring stage of the general kernel
    auto lds_bytes = [&](int cb) { return (size_t)2 * PPS * MT * (WTILE + 256) + (size_t)(((27 * cb + 1) >> 1) + 2) * 32 + (size_t)cb * TT * (RB + 4); };
    int cb2 = 0, cb1 = 0;
    for (int cb = 1; cb <= a.nbt; cb++) { if (lds_bytes(cb) <= 80 * 1024 - 2816) cb2 = cb; if (lds_bytes(cb) <= 160 * 1024 - 3072) cb1 = cb; }   // (room for the epilogue's constants and scratch)
    int cbmax = cb2 ? cb2 : cb1;
    static int cb_env = -1;
    if (cb_env < 0) cb_env = getenv("MI_CONV_CB") ? atoi(getenv("MI_CONV_CB")) : 0;      // tuning knob: blocks per chunk
    if (cb_env > 0 && cb_env <= cb1) cbmax = cb_env;
    if (cbmax < 1) mi_die("%s: tile does not fit LDS", who);
    const int nchunks = (a.nbt + cbmax - 1) / cbmax;
    a.CB = big || s2d ? a.nbt : (a.nbt + nchunks - 1) / nchunks; // (the wide kernel has no chunks: its K loop walks block by block; the direct stride-2 kernel: one chunk, tap-major)
    static int areg_env = -1;
    if (areg_env < 0) areg_env = getenv("MI_CONV_AREG") ? atoi(getenv("MI_CONV_AREG")) : 1;      // tuning knob: 0 keeps the general kernel for every shape
    a.areg = areg_env && !big && !s2d && !(osum && (cout / Go) % 4) && cout > 16 && nmt_all == 1 && stride == 1 && a.nbt == 1 && a.wide && (NT == 2 || NT == 4);      // (one channel tile in all: these kernels have no channel slices)
    // one channel tile of 17 .. 32 output channels from two or more input blocks on a volume wider than one 16-voxel tile: the row kernel (runs
    // of 32 voxels along x, input fragments shared by the three ky taps). One input block stays with the kernel that keeps its weights in
    // registers, which measures a few percent faster there (both are bound by the halo's cache misses in flight, and it loads no weights)
    static int row_env = -1;
    if (row_env < 0) row_env = getenv("MI_CONV_ROW") ? atoi(getenv("MI_CONV_ROW")) : 1;      // tuning knob: 0 keeps the other kernels for these shapes, 2 also takes one input block
    // ... and one input block takes the row kernel's one-block form: weights in registers, the workgroup's two halves half a tile apart so that
    // one half's epilogue runs under the other's MFMAs (MI_CONV_ROW1=0: the small-channel kernel)
    static int row1_env = -1;
    if (row1_env < 0) row1_env = getenv("MI_CONV_ROW1") ? atoi(getenv("MI_CONV_ROW1")) : 1;
    // ... and 33 .. 64 output channels from one to three input blocks run the two row kernels as two channel slices, one per workgroup (MI_CONV_ROW_CS=0:
    // the general kernel). Measured at 2 x 64^3 in e4m3: 32 -> 64 0.046 -> 0.039 ms, 64 -> 64 0.073 -> 0.067 ms, 96 -> 64 0.100 -> 0.095 ms; from four
    // blocks on the wide kernel keeps these layers
    static int rowcs_env = -1;
    if (rowcs_env < 0) rowcs_env = getenv("MI_CONV_ROW_CS") ? atoi(getenv("MI_CONV_ROW_CS")) : 1;
    const bool row_cs = (rowcs_env && nmt_all == 2 && MT == 2) || row_cs4;
    a.row = row_env && !big && !s2d && !(osum && (cout / Go) % 4) && cout > 16 && (nmt_all == 1 || row_cs) && stride == 1 && NT == 4 && a.wide && Wo > 16 && a.nbt >= (row_env > 1 || row1_env ? 1 : 2) && a.nbt <= 64;
    a.row1 = a.row && a.nbt == 1 && row1_env && row_env < 2;
    if (a.row && nmt_all >= 2) MT = 1;
    if (a.row) { a.areg = false; a.CB = a.nbt; }
    size_t smem = a.row1 ? (size_t)10 * 352 * (RB + 4) : a.row ? (size_t)2 * 2048 * (RB + 4) : a.areg ? (size_t)2 * ((TT + 63) / 64 * 64) * (RB + 4) : big ? (size_t)4 * MT * (WTILE + 256) + (size_t)3 * ((TT + 63) / 64 * 64) * (RB + 4) + (size_t)(((27 * a.nbt + 1) >> 1) + 2) * 32 : lds_bytes(a.CB);
    if (s2d) smem = 0;
    smem = (smem + 15) & ~(size_t)15;
    a.epi_o = (unsigned)smem; smem += (size_t)3 * MT * 32 * sizeof(float);      // bias, affine a, b of the workgroup's channels
    a.red_o = (unsigned)smem; smem += a.row1 ? 3 * 2048 + 3 * 1024 : 1024;      // statistics scratch (the one-block row kernel: the weight fragments of two tap classes instead)
    if (s2d) smem += (size_t)(27 * a.nbt + 1 + 8) * sizeof(int);                // the direct stride-2 kernel's K-order table
    // the row kernel in e2m1: the prepared weights of up to four input blocks stay in LDS (MI_CONV_ROW_WL=0: loaded from global memory per tap class)
    static int wl_env = -1;
    if (wl_env < 0) wl_env = getenv("MI_CONV_ROW_WL") ? atoi(getenv("MI_CONV_ROW_WL")) : 1;
    a.wl_o = 0;
    if (a.row && !a.row1 && fmt == 4 && wl_env && smem + (size_t)a.nbt * 15 * 1280 <= 160 * 1024) { a.wl_o = (unsigned)smem; smem += (size_t)a.nbt * 15 * 1280; }
    if (big || a.areg || a.row) {
        // rows and scale bytes of positions outside the volume: 64 zero bytes, then 64 bytes of value 1; one page per device, kept for the process
        // (the entry point that must not allocate keeps its own at the head of its fixed scratch)
        static uint8_t *zpage[8];
        int dv = 0; MIRT(hipGetDevice(&dv)); dv &= 7;
        if (mi_ws_arena_on()) a.zpage = g_static_zpage;
        else {
            if (!zpage[dv]) {
                uint8_t init[128]; memset(init, 0, 64); memset(init + 64, 1, 64);
                MIRT(hipMalloc((void **)&zpage[dv], 128)); mi_count_alloc();
                if (!zpage[dv]) mi_die("%s: no device memory for the constant page", who);
                MIRT(hipMemcpy(zpage[dv], init, 128, hipMemcpyHostToDevice));
            }
            a.zpage = zpage[dv];
        }
    }
    a.nmt_all = nmt_all; a.ncs = nmt_all / MT;
    a.ntx = a.row ? (Wo + 31) / 32 : (Wo + 15) / 16; a.nty = (Ho + 7) / 8; a.ntz = (Do + TZ - 1) / TZ;      // (the row kernel: 4 x 8 x 32 voxels per tile)
    a.ntiles = (unsigned)((size_t)a.ntx * a.nty * a.ntz * a.ncs * N);
    // ---- weights ----
    int npairs_all = 0;
    for (int b0 = 0; b0 < a.nbt; b0 += a.CB) npairs_all += (27 * (a.nbt - b0 < a.CB ? a.nbt - b0 : a.CB) + 1) >> 1;
    if (a.row) npairs_all = 15 * a.nbt;              // (15 pairs per input block: its tap classes)
    // (sixteen pairs of padding: the kernels' weight loads run up to two ring stages ahead of the last pair)
    // (the wide kernel's weights are one buffer: codes and scale words interleaved pair by pair; its scale buffer is a stub)
    const size_t wq_bytes = (size_t)(npairs_all + 16) * nmt_all * (big ? WTILE + 256 : WTILE), wsc_bytes = big ? 256 : (size_t)(npairs_all + 16) * nmt_all * 256;
    a.wstride = (unsigned)((size_t)(npairs_all + 16) * MT * (WTILE + 256));
    const int memoCB = big ? -a.CB : a.CB;
    a.big = big;
    const int CxP = (Cx + 31) / 32 * 32;
    int dev = 0; MIRT(hipGetDevice(&dev));
    uint8_t *wq = nullptr, *wsc = nullptr; bool have = false;
    if (sp.wkey && !mi_ws_arena_on()) {
        std::lock_guard<std::mutex> lk(g_wmemo_mu);
        for (auto &m : g_wmemo)
            if (m.key == sp.wkey && m.w == w && m.fmt == fmt && m.Co == cout && m.Ci == Ci && m.Cx == Cx && m.nbt == a.nbt && m.CB == memoCB && m.nmt_all == nmt_all && m.dev == dev && m.lay == (big ? MT : a.row ? 100 : s2d ? 200 : 0)) { wq = m.wq; wsc = m.wsc; have = true; break; }
        if (!have) {
            MIRT(hipMalloc((void **)&wq, wq_bytes)); MIRT(hipMalloc((void **)&wsc, wsc_bytes)); mi_count_alloc(); mi_count_alloc();
            if (!wq || !wsc) mi_die("%s: no device memory for the prepared weights", who);
            MIRT(hipMemsetAsync(wq, 0, wq_bytes, 0)); MIRT(hipMemsetAsync(wsc, 0, wsc_bytes, 0));
            g_wmemo.push_back(wmemo_t{sp.wkey, w, fmt, cout, Ci, Cx, a.nbt, memoCB, nmt_all, dev, big ? MT : a.row ? 100 : s2d ? 200 : 0, wq, wsc});
        }
    } else { wq = (uint8_t *)mi_ws(MI_WS_WQ, wq_bytes); wsc = (uint8_t *)mi_ws(MI_WS_WSC, wsc_bytes); }
    if (!have) {
        const size_t nt = (size_t)npairs_all * nmt_all * 32;
        // 2-D fp4 weight scales (lp_set_w4_2d): the stride-1 e2m1 preps of more than 16 input channels, as src/lp_f4fwd.cuh:1163
        const int w2d = g_w2d_on() && fmt == 4 && stride == 1 && Ci > 16;
        if (fmt == 8) prep_w_k<8><<<nblk_(nt, 128), 128>>>(w, wq, (unsigned *)wsc, cout, Ci, Cx, CxP, a.nbt, a.CB, nmt_all, npairs_all, big ? MT : a.row ? -1 : s2d ? -2 : 0, 0);
        else prep_w_k<4><<<nblk_(nt, 128), 128>>>(w, wq, (unsigned *)wsc, cout, Ci, Cx, CxP, a.nbt, a.CB, nmt_all, npairs_all, big ? MT : a.row ? -1 : s2d ? -2 : 0, w2d);
        MICK();
    }
    a.wq = wq; a.wsc = wsc;
    a.stat_ch = osum && (cout / Go) % 4 ? 1 : 0;
    if (osum) a.part = (float *)mi_ws(MI_WS_MISC, (size_t)a.ntiles * (a.stat_ch ? 32 : a.row1 ? 64 : MT * 8) * 2 * sizeof(float));      // (row1: a record per wavefront, eight per tile)
    const bool epi = act != 0;
    const int out = ybf == 3 ? 8 : ybf == 4 ? 4 : 0;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    const bool ktime = g_ktime && !mi_ws_arena_on();
    if (ktime) { MIRT(hipEventCreate(&ev0)); MIRT(hipEventCreate(&ev1)); MIRT(hipEventRecord(ev0, 0)); }
    if (s2d) {
        const dim3 grid((unsigned)((s2runs + 3) / 4), (unsigned)a.ncs, (unsigned)N);
        if (fmt == 8) conv3s2_launch_f8(out, MT, a, grid, smem); else conv3s2_launch_f4(out, MT, a, grid, smem);
    } else if (fmt == 8) { if (out == 8) conv3_launch_f8_o8(stride, epi, MT, NT, a, smem); else if (out == 4) conv3_launch_f8_o4(stride, epi, MT, NT, a, smem); else conv3_launch_f8_o0(stride, epi, MT, NT, a, smem); }
    else { if (out == 8) conv3_launch_f4_o8(stride, epi, MT, NT, a, smem); else if (out == 4) conv3_launch_f4_o4(stride, epi, MT, NT, a, smem); else conv3_launch_f4_o0(stride, epi, MT, NT, a, smem); }
    if (ktime) { MIRT(hipEventRecord(ev1, 0)); ktime_push(ev0, ev1, 2.0 * 27 * Ci * (double)cout * N * Do * Ho * Wo); }
    if (osum) conv_stats_reduce(who, a, MT, sp, osum);
    return 0;
}

// the consumer-side transform of a conv input (GroupNorm + SiLU while staging, re-quantisation to the compute format) done once into an MX
// tensor of the same channels, for a tensor several convs read: they then take y as a plain input and stage it as stored. Channels a
// multiple of 32. The bits of the convs' results do not change (the same pre-pass runs inside a conv otherwise).
extern "C" int mi_conv_prestage(const void *x, int xdt, shape5 s, gnp_t gp, void *y, int ybits) {
    if ((ybits != 8 && ybits != 4) || s.c % 32 || xdt < 0 || xdt > 4 || (gp.G > 0 && s.c % gp.G)) return -1;
    const size_t hw = (size_t)s.h * s.w;
    gn_for_slabs("mi_conv_prestage", gp, s.h * s.w, 0, s.d, [&](int z0, int z1, gnp_t gs) { mi_restage_sub(x, xdt, s.n, s.c, (size_t)(z1 - z0) * hw, gs, s.c, 0, y, ybits, (size_t)s.d * hw, (size_t)z0 * hw); });
    return 0;
}
extern "C" int mi_conv_prestage2(const void *x, shape5 s, gnp_t gp, void *y8, void *y4) {
    if (s.c % 32 || (gp.G > 0 && s.c % gp.G) || !y8 || !y4) return -1;
    const size_t hw = (size_t)s.h * s.w;
    gn_for_slabs("mi_conv_prestage2", gp, s.h * s.w, 0, s.d, [&](int z0, int z1, gnp_t gs) { mi_restage_sub2(x, s.n, s.c, (size_t)(z1 - z0) * hw, gs, y8, y4, (size_t)s.d * hw, (size_t)z0 * hw); });
    return 0;
}
extern "C" int lp_conv_fwd_f8(const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp, double *osum, int Go, split_t sp) {
    return conv_dispatch("lp_conv_fwd_f8", 8, 1, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp, nullptr, nullptr, 0);
}
extern "C" int lp_conv_fwd_f4(const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp, double *osum, int Go, split_t sp) {
    return conv_dispatch("lp_conv_fwd_f4", 4, 1, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp, nullptr, nullptr, 0);
}
// prepared-weight memo id of the calling thread's next stride-2 conv, 3x3x3 or 2x2x2 (their signatures carry no split_t): 0 = prepare per call
static thread_local unsigned g_s2_wkey = 0;
extern "C" void mi_conv_s2_wkey(unsigned wkey) { g_s2_wkey = wkey; }
unsigned mi_take_s2_wkey(void) { const unsigned k = g_s2_wkey; g_s2_wkey = 0; return k; }      // (the 2x2x2 entries consume it too)
extern "C" void mi_conv_stem_zc(int zc) { g_stem_zc = zc; }
extern "C" int lp_conv_fwd_s2_f8(const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, shape5 ys, gnp_t gp) {
    const int Do = (xs.d - 1) / 2 + 1, Ho = (xs.h - 1) / 2 + 1, Wo = (xs.w - 1) / 2 + 1;
    if (ys.d != Do || ys.h != Ho || ys.w != Wo || ys.c != cout || ys.n != xs.n) mi_die("lp_conv_fwd_s2_f8: output shape %d x %d x %d x %d x %d does not match a stride-2 conv of the input", ys.n, ys.c, ys.d, ys.h, ys.w);
    split_t sp; memset(&sp, 0, sizeof sp);
    sp.wkey = g_s2_wkey; g_s2_wkey = 0;
    // compute format as the reference's dispatch (src/lp_s2.cu:647-754): fp4 only for an MX-fp4 32 -> <= 32 channel conv on even dims, else fp8
    const bool f4 = xbf == 4 && xs.c == 32 && cout <= 32 && !(xs.d & 1) && !(xs.h & 1) && !(xs.w & 1);
    conv_dispatch("lp_conv_fwd_s2_f8", f4 ? 4 : 8, 2, x, xbf, xs, w, b, cout, y, ybf, gp, nullptr, 0, sp, nullptr, nullptr, 0);
    return f4 ? 3 : 0;
}
extern "C" int mi_conv_fwd_gn(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp,
                              double *osum, int Go, split_t sp, float eps, float *omean, float *orstd) {
    if (bits != 8 && bits != 4) mi_die("mi_conv_fwd_gn: compute format %d (8 or 4)", bits);
    if (!osum || !omean || !orstd || Go <= 0) mi_die("mi_conv_fwd_gn: needs sum slots, mean and rstd buffers and groups");
    g_fin = gn_fin_t{omean, orstd, 0.0, eps};
    const int rc = conv_dispatch("mi_conv_fwd_gn", bits, 1, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp, nullptr, nullptr, 0);
    g_fin = gn_fin_t{nullptr, nullptr, 0.0, 0.f};
    return rc;
}
extern "C" int mi_conv_fwd_fused(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf,
                                 const float *ep_a, const float *ep_b, int act, gnp_t gp, double *osum, int Go, split_t sp) {
    if (bits != 8 && bits != 4) mi_die("mi_conv_fwd_fused: compute format %d (8 or 4)", bits);
    if (act < 0 || act > 3 || (!act && ep_a) || (!ep_a != !ep_b)) mi_die("mi_conv_fwd_fused: activation %d / affine arguments", act);
    return conv_dispatch("mi_conv_fwd_fused", bits, 1, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp, ep_a, ep_b, act);
}

// ---- the stride-1 convs for callers that cannot allocate (serving loops, harnesses that forbid hipMalloc) ----
// Every byte of device memory the conv needs beyond its inputs and outputs - prepared weights, re-staged operands, the coarse rows of a fused
// upsample, per-tile statistics partials, the constant page of out-of-volume rows - is carved from one file-scope device array. The array is a
// host-side stand-in by name: its device address is taken once per device and only that address is used from then on.
#define MI_STATIC_SCRATCH_BYTES ((size_t)64 << 20)
static __device__ __align__(256) unsigned char scratch[MI_STATIC_SCRATCH_BYTES];
static unsigned char *g_scratch_ptr[8];        // per device: the address of that device's copy of the array
static std::mutex g_scratch_mu;
extern "C" size_t mi_conv_static_scratch_bytes(void) { return MI_STATIC_SCRATCH_BYTES; }
// an upper bound of what conv_dispatch will request from mi_ws for this call, following its choices (every request rounded up to 256 bytes)
static size_t conv_scratch_bound(int fmt, const void *x2, int xbf, int ybf, shape5 xs, int cout, gnp_t gp, const double *osum, split_t sp) {
    auto al = [](size_t n) { return ((n + 255) & ~(size_t)255) + 256; };
    const int Ci = xs.c, Cx = x2 ? sp.c_split : Ci, C2 = Ci - Cx, N = xs.n, D = sp.Di ? sp.Di : xs.d;
    if (fmt == 4 && Ci <= 8) fmt = 8;
    const size_t S = (size_t)D * xs.h * xs.w, So = (size_t)xs.d * xs.h * xs.w;
    const int nmt_all = (cout + 31) / 32, fdt = fmt == 8 ? 3 : 4;
    const size_t tiles = (size_t)((xs.w + 15) / 16) * ((xs.h + 7) / 8) * xs.d * nmt_all * N;           // one-plane tiles of one channel tile: no launch has more
    size_t need = 256;                                              // the constant page
    if (Ci <= 16 && !x2 && fmt == 8) need += al((size_t)9 * nmt_all * 2048) + al((size_t)9 * nmt_all * 256);      // the tap-packed kernels' weights
    const int nbt = (Cx + 31) / 32 + (x2 ? (C2 + 31) / 32 : 0);
    need += al(((size_t)(27 * nbt + 1) / 2 + 2 * nbt + 16) * nmt_all * 2304) + al(((size_t)(27 * nbt + 1) / 2 + 2 * nbt + 16) * nmt_all * 256);      // (at most 15 pairs per block)
    // the tap-packed kernels read their input as stored and apply its GroupNorm while staging: nothing is re-staged (conv_dispatch's routing)
    const bool stem = fmt == 8 && !x2 && ((xbf == 0 || xbf >= 2) && Ci <= (xbf == 0 ? 16 : 8) || (xbf >= 2 && Ci <= 16)) && (xbf == ybf || ybf >= 3);
    const bool s2g = x2 && sp.gp2.G;
    for (int s = 0; s < (x2 ? 2 : 1) && !stem; s++) {
        const gnp_t g = s2g ? (s ? sp.gp2 : gp) : gp;
        const bool upseg = s == 0 && sp.up, direct = xbf == fdt && !(g.G > 0) && !upseg;
        const int C = s ? C2 : Cx;
        if (!direct) need += al((size_t)N * ((C + 31) / 32) * S * 33);
        if (upseg) need += al((size_t)N * ((C + 31) / 32) * (S / 8) * 33);
    }
    if (osum) need += al(tiles * 32 * 2 * sizeof(float));
    (void)So;
    return need;
}
// set-up, once per device with that device current: the array's address on this device, and the constant page at its head. mi_init calls it
// for the device it selects (a synchronous 128-byte copy: not something to meet for the first time inside a serving loop); the entry point
// repeats the call for a device nobody initialised through mi_init
int mi_conv_static_setup(const char *who) {
    int dv = 0; MIRT(hipGetDevice(&dv)); dv &= 7;
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (g_scratch_ptr[dv]) return 0;
    unsigned char *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) { fprintf(stderr, "%s: the fixed scratch has no address on device %d: %s\n", who, dv, hipGetErrorString(e)); return -2; }
    uint8_t init[128]; memset(init, 0, 64); memset(init + 64, 1, 64);
    if (hipMemcpy(ptr, init, 128, hipMemcpyHostToDevice) != hipSuccess) { fprintf(stderr, "%s: cannot initialise the fixed scratch on device %d\n", who, dv); return -2; }
    g_scratch_ptr[dv] = ptr;
    return 0;
}
static int conv_fwd_static(const char *who, int fmt, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp, double *osum, int Go, split_t sp) {
    int dv = 0; MIRT(hipGetDevice(&dv)); dv &= 7;
    if (!g_scratch_ptr[dv] && mi_conv_static_setup(who)) return -2;
    const size_t need = conv_scratch_bound(fmt, sp.x2, xbf, ybf, xs, cout, gp, osum, sp);
    if (need > MI_STATIC_SCRATCH_BYTES) {
        fprintf(stderr, "%s: this call needs up to %zu bytes of scratch (prepared weights, re-staged operands, statistics partials); the fixed scratch holds %zu. "
                        "Use lp_conv_fwd_f8 / lp_conv_fwd_f4, which allocate, or pass an input that is already in the compute format without GroupNorm\n", who, need, (size_t)MI_STATIC_SCRATCH_BYTES);
        return -1;
    }
    unsigned char *ptr = g_scratch_ptr[dv];
    g_static_zpage = ptr;                                          // bytes [0, 128): zero rows, then scale bytes of value 1
    mi_ws_arena(ptr + 256, MI_STATIC_SCRATCH_BYTES - 256);         // everything else is carved per call, and fully written before it is read
    const int rc = conv_dispatch(who, fmt, 1, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp, nullptr, nullptr, 0);
    mi_ws_arena(nullptr, 0);
    g_static_zpage = nullptr;
    return rc;
}
extern "C" int mi_conv_fwd_static(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp, double *osum, int Go, split_t sp) {
    if (bits != 8 && bits != 4) { fprintf(stderr, "mi_conv_fwd_static: compute format %d (8 or 4)\n", bits); return -1; }
    return conv_fwd_static("mi_conv_fwd_static", bits, x, xbf, xs, w, b, cout, y, ybf, gp, osum, Go, sp);
}
