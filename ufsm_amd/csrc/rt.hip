// Runtime shim of the library: device selection, memory, error latch, per-device scratch, events, GroupNorm finalize.
// These stand in for what the reference's lp_* units take from its op layer (src/nn.h:34-48, src/nn_core.cu:244-290, :751).
#include "mx_dev.hpp"
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <mutex>

static thread_local hipError_t g_err = hipSuccess;      // first error since the last lp_check (src/lp_common.cuh:35-38)
static thread_local char g_errmsg[256];
void mi_post_error(hipError_t e, const char *file, int line) {
    if (g_err != hipSuccess) return;
    g_err = e;
    snprintf(g_errmsg, sizeof g_errmsg, "%s (%s:%d)", hipGetErrorString(e), file, line);
}
[[noreturn]] void mi_die(const char *fmt, ...) {
    va_list ap; va_start(ap, fmt); vfprintf(stderr, fmt, ap); va_end(ap); fputc('\n', stderr); fflush(stderr);
    abort();
}
extern "C" const char *lp_check(void) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) mi_post_error(e, __FILE__, __LINE__);
    if (g_err == hipSuccess) return nullptr;
    g_err = hipSuccess;
    return g_errmsg;
}
extern "C" int mi_device_count(void) { int n = 0; if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return 0; } return n; }
int mi_conv_static_setup(const char *who);      // conv3.hip
extern "C" int mi_init(int device) {
    int n = mi_device_count();
    if (device < 0 || device >= n) { fprintf(stderr, "mi_init: no HIP device %d (%d visible): the MX kernels need a gfx950 GPU\n", device, n); return 1; }
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, device) != hipSuccess) return 2;
    if (strncmp(p.gcnArchName, "gfx950", 6) != 0) { fprintf(stderr, "mi_init: device %d is %s, this library is built for gfx950 only\n", device, p.gcnArchName); return 3; }
    if (hipSetDevice(device) != hipSuccess) return 4;
    return mi_conv_static_setup("mi_init") ? 5 : 0;             // the entry point that allocates nothing finds its fixed scratch addressed and its constant page written
}
extern "C" void *mi_malloc(size_t bytes) {
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes ? bytes : 1); mi_count_alloc();
    if (e != hipSuccess) mi_die("mi_malloc: %zu bytes: %s", bytes, hipGetErrorString(e));
    return p;
}
extern "C" void mi_free(void *p) { if (p) MIRT(hipFree(p)); }
__global__ void fill_u32_k(unsigned *p, size_t n, unsigned v) { size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; if (i < n) p[i] = v; }
extern "C" void mi_zero(void *p, size_t bytes) { MIRT(hipMemsetAsync(p, 0, bytes, 0)); }
extern "C" void mi_h2d(void *dst, const void *src, size_t bytes) { MIRT(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice)); }
// pinned host memory and a copy from it in stream order (the host does not wait), with a fence the host can wait on before it rewrites the source
extern "C" void *mi_host_alloc(size_t bytes) { void *p = nullptr; hipError_t e = hipHostMalloc(&p, bytes ? bytes : 1); if (e != hipSuccess) mi_die("mi_host_alloc: %zu bytes: %s", bytes, hipGetErrorString(e)); return p; }
extern "C" void mi_host_free(void *p) { if (p) MIRT(hipHostFree(p)); }
extern "C" void mi_h2d_async(void *dst, const void *src, size_t bytes) { if (bytes) MIRT(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, 0)); }
extern "C" void *mi_fence_new(void) { hipEvent_t e; MIRT(hipEventCreateWithFlags(&e, hipEventDisableTiming)); return (void *)e; }
extern "C" void mi_fence_set(void *f) { MIRT(hipEventRecord((hipEvent_t)f, 0)); }
extern "C" void mi_fence_wait(void *f) { MIRT(hipEventSynchronize((hipEvent_t)f)); }
extern "C" void mi_fence_free(void *f) { if (f) MIRT(hipEventDestroy((hipEvent_t)f)); }
extern "C" void mi_d2h(void *dst, const void *src, size_t bytes) { MIRT(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost)); }
extern "C" void mi_d2d(void *dst, const void *src, size_t bytes) { MIRT(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, 0)); }
// `rows` runs of `width` bytes, run r at dst + r * dpitch from src + r * spitch (a range of planes of every channel block of an MX tensor)
extern "C" void mi_d2d_rows(void *dst, size_t dpitch, const void *src, size_t spitch, size_t width, size_t rows) {
    if (width && rows) MIRT(hipMemcpy2DAsync(dst, dpitch, src, spitch, width, rows, hipMemcpyDeviceToDevice, 0));
}
extern "C" void mi_sync(void) { MIRT(hipDeviceSynchronize()); }

// per-device scratch: grow on demand, contents valid until the next request of the same slot on the same device
static void *g_ws[8][MI_WS_NSLOTS]; static size_t g_wscap[8][MI_WS_NSLOTS];
// device allocations this library has made so far (scratch growth, memo entries, mi_malloc): lets a caller check that a code path made none
static long g_nalloc = 0;
void mi_count_alloc(void) { __atomic_add_fetch(&g_nalloc, 1, __ATOMIC_RELAXED); }
extern "C" long mi_alloc_count(void) { return __atomic_load_n(&g_nalloc, __ATOMIC_RELAXED); }
// a fixed region the calling thread's scratch requests are carved from instead (the entry point that must not allocate): requests are
// handed out back to back, 256-byte aligned; one that does not fit ends the process with a message (the entry point checks its bound first)
static thread_local unsigned char *g_arena = nullptr; static thread_local size_t g_arena_off = 0, g_arena_cap = 0;
void mi_ws_arena(void *base, size_t cap) { g_arena = (unsigned char *)base; g_arena_off = 0; g_arena_cap = base ? cap : 0; }
bool mi_ws_arena_on(void) { return g_arena != nullptr; }
void *mi_ws(int slot, size_t bytes) {
    if (g_arena) {
        const size_t need = (bytes + 255) & ~(size_t)255;
        if (g_arena_off + need > g_arena_cap) mi_die("mi_ws: slot %d needs %zu bytes, %zu of the fixed scratch's %zu are taken", slot, need, g_arena_off, g_arena_cap);
        void *p = g_arena + g_arena_off; g_arena_off += need;
        return p;
    }
    int d = 0; MIRT(hipGetDevice(&d)); d &= 7;
    if (bytes > g_wscap[d][slot]) {
        if (g_ws[d][slot]) { MIRT(hipDeviceSynchronize()); MIRT(hipFree(g_ws[d][slot])); }
        const size_t cap = bytes + bytes / 8 + 4096;
        hipError_t e = hipMalloc(&g_ws[d][slot], cap); mi_count_alloc();
        if (e != hipSuccess) mi_die("mi_ws: slot %d, %zu bytes: %s", slot, cap, hipGetErrorString(e));
        g_wscap[d][slot] = cap;
    }
    return g_ws[d][slot];
}
extern "C" void mi_ws_release(void) {
    int d = 0; MIRT(hipGetDevice(&d)); d &= 7;
    MIRT(hipDeviceSynchronize());
    for (int s = 0; s < MI_WS_NSLOTS; s++) { if (g_ws[d][s]) MIRT(hipFree(g_ws[d][s])); g_ws[d][s] = nullptr; g_wscap[d][s] = 0; }
    lp_wmemo_clear();
}

// events on the null stream
extern "C" void *mi_event_create(void) { hipEvent_t e; if (hipEventCreate(&e) != hipSuccess) return nullptr; return (void *)e; }
extern "C" void mi_event_record(void *ev) { MIRT(hipEventRecord((hipEvent_t)ev, 0)); }
extern "C" float mi_event_elapsed_ms(void *ev0, void *ev1) { float ms = 0.f; MIRT(hipEventSynchronize((hipEvent_t)ev1)); MIRT(hipEventElapsedTime(&ms, (hipEvent_t)ev0, (hipEvent_t)ev1)); return ms; }
extern "C" void mi_event_destroy(void *ev) { if (ev) MIRT(hipEventDestroy((hipEvent_t)ev)); }

// ---- GroupNorm sum slots (src/gnacc.cuh): [lo: 2^-64 units][hi: integer part, two's complement][count of non-finite adds] ----
__device__ __forceinline__ double gn_slot_get(const double *b, size_t i) {
    const unsigned long long *w = (const unsigned long long *)b + 3 * i;
    if (w[2]) return __longlong_as_double(0x7ff8000000000000ll);
    return (double)(long long)w[1] + (double)w[0] * 5.42101086242752217e-20;
}
__global__ void gn_finalize_k(const double *sums, int NG, size_t len, float eps, float *mean, float *rstd) {   // src/nn_elem.cu:5-11
    const int ng = blockIdx.x * blockDim.x + threadIdx.x;
    if (ng >= NG) return;
    const double m = gn_slot_get(sums, 2 * ng) / (double)len, v = gn_slot_get(sums, 2 * ng + 1) / (double)len - m * m;
    mean[ng] = (float)m;
    rstd[ng] = (float)(1.0 / sqrt((v > 0 ? v : 0) + (double)eps));
}
extern "C" void mi_gn_finalize(const double *sums, int NG, size_t len, float eps, float *mean, float *rstd) {
    gn_finalize_k<<<nblk_(NG, 64), 64>>>(sums, NG, len, eps, mean, rstd); MICK();
}
__global__ void gn_get_k(const double *sums, int n, double *out) { const int i = blockIdx.x * blockDim.x + threadIdx.x; if (i < n) out[i] = gn_slot_get(sums, i); }
extern "C" void mi_gn_sums_get(const double *sums, int nslots, double *out) { gn_get_k<<<nblk_(nslots, 64), 64>>>(sums, nslots, out); MICK(); }
extern "C" void mi_gn_sums_zero(double *sums, int nslots) {
    const size_t n = (size_t)nslots * 6;   // 24 bytes = 6 words
    fill_u32_k<<<nblk_(n, 256), 256>>>((unsigned *)sums, n, 0u); MICK();
}
// ---- FiLM on GroupNorm affines (src/nn.h:494-504): a norm of C channels at offsets gam / bet of the parameter vector p, its K x C pairs A
// (scale) and D (shift) at fo, A first. cfg.film: K host codes c, fw gamma = gamma (1 + sum_k c_k A_kc), fw beta = beta + sum_k c_k D_kc.
// cfg.gfilm: the codes are a device vector (the attention stage's output averaged over the window's tokens) and the affine before is the one
// fw already holds (kept in g1). The sums are fused multiply-add chains from k = 0, as the reference's contracted loop ----
struct film_codes_t { float c[4]; };
__global__ void __launch_bounds__(64) film_affine_k(const float *__restrict__ p, float *__restrict__ fw, size_t gam, size_t bet, size_t fo, int C, int K, film_codes_t cc) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= C) return;
    const float *A = p + fo + c, *D = A + (size_t)K * C;
    float s = 0.f, t = 0.f;
    for (int k = 0; k < K; k++) { s = fmaf(cc.c[k], A[(size_t)k * C], s); t = fmaf(cc.c[k], D[(size_t)k * C], t); }
    const float one_s = 1.f + s;
    fw[gam + c] = p[gam + c] * one_s;
    fw[bet + c] = p[bet + c] + t;
}
extern "C" void nn_film_fwd(const float *p, float *fw, size_t gam, size_t bet, size_t fo, int C, int K, const float *codes) {
    if (C <= 0) return;
    if (K < 0 || K > 4) mi_die("nn_film_fwd: 0 .. 4 codes, not %d", K);
    film_codes_t cc = {{0.f, 0.f, 0.f, 0.f}};
    for (int k = 0; k < K; k++) cc.c[k] = codes[k];
    film_affine_k<<<(C + 63) / 64, 64>>>(p, fw, gam, bet, fo, C, K, cc); MICK();
}
// g[c] = mean over S of x[c S + s]: one workgroup of 256 per channel, fp64 partial sums of the strided elements, a halving tree over the 256
__global__ void __launch_bounds__(256) chan_mean_k(const float *__restrict__ x, long S, float *__restrict__ g) {
    __shared__ double part[256];
    const float *row = x + (size_t)blockIdx.x * S;
    double a = 0;
    for (long s = threadIdx.x; s < S; s += 256) a += (double)row[s];
    part[threadIdx.x] = a;
    __syncthreads();
    for (int h = 128; h; h >>= 1) { if ((int)threadIdx.x < h) part[threadIdx.x] += part[threadIdx.x + h]; __syncthreads(); }
    if (!threadIdx.x) g[blockIdx.x] = (float)(part[0] / (double)S);
}
extern "C" void nn_gfilm_pool(const float *x, int C, long S, float *g) { if (C > 0 && S > 0) { chan_mean_k<<<C, 256>>>(x, S, g); MICK(); } }
__global__ void __launch_bounds__(64) gfilm_affine_k(const float *__restrict__ p, float *__restrict__ fw, size_t gam, size_t bet, size_t fo, int C, int K, const float *__restrict__ gv, float *__restrict__ g1) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= C) return;
    const float *A = p + fo + c, *B = A + (size_t)K * C;
    float s = 0.f, t = 0.f;
    for (int k = 0; k < K; k++) { const float gk = gv[k]; s = fmaf(gk, A[(size_t)k * C], s); t = fmaf(gk, B[(size_t)k * C], t); }
    const float before = fw[gam + c], one_s = 1.f + s;
    g1[c] = before;
    fw[gam + c] = before * one_s;
    fw[bet + c] = fw[bet + c] + t;
}
extern "C" void nn_gfilm_fwd(const float *p, float *fw, size_t gam, size_t bet, size_t fo, int C, int K, const float *gv, float *g1) {
    if (C > 0) { gfilm_affine_k<<<(C + 63) / 64, 64>>>(p, fw, gam, bet, fo, C, K, gv, g1); MICK(); }
}
// ---- y += a x over n floats (nn_axpy, src/nn.h): the stem bias of a scale-conditioned net ----
// (a few dozen values in practice: one wavefront strides over them, one fused multiply-add each, as the reference's contracted a * x + y)
__global__ void __launch_bounds__(64) scaled_add_k(float *__restrict__ y, float a, const float *__restrict__ x, size_t n) {
    for (size_t i = blockIdx.x * 64 + threadIdx.x; i < n; i += (size_t)gridDim.x * 64) y[i] = fmaf(a, x[i], y[i]);
}
extern "C" void nn_axpy(float *y, float a, const float *x, size_t n) {
    if (n) { scaled_add_k<<<(unsigned)(n < 65536 ? (n + 63) / 64 : 1024), 64>>>(y, a, x, n); MICK(); }
}
// ---- constant GroupNorm statistics for N samples (src/nn.h:465-473, src/nn_l0norm.cu:10-20): run null: mean 0, rstd 1; else run = [mean G | var G] ----
__global__ void gn_const_k(float *mean, float *rstd, const float *run, int NG, int G, float eps) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= NG) return;
    const int g = i % G;
    mean[i] = run ? run[g] : 0.f;
    rstd[i] = run ? 1.f / sqrtf(run[G + g] + eps) : 1.f;
}
extern "C" void nn_gn_const_fill(float *mean, float *rstd, const float *run, int N, int G, float eps) {
    if (N * G > 0) { gn_const_k<<<nblk_((size_t)N * G, 64), 64>>>(mean, rstd, run, N * G, G, eps); MICK(); }
}
// ---- scaled weight standardisation (src/nn.h:477, src/nn_l0norm.cu:45-63): per output channel over its fan-in of n contiguous weights,
// wh = gain (w - mean) / (std sqrt(n) + eps), mean and population std in double. One wavefront per output channel (a fan-in is 108 .. a few
// thousand weights): a lane sums every 64th weight, the moments meet through lane exchanges ----
__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__global__ void __launch_bounds__(256) ws_fwd_k(float *wh, const float *w, int cout, int n, float gain, float eps) {
    const int o = blockIdx.x * 4 + (int)(threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (o >= cout) return;
    const float *wo = w + (size_t)o * n; float *ho = wh + (size_t)o * n;
    double s = 0.0;
    for (int i = lane; i < n; i += 64) s += (double)wo[i];
    const double mu = wave_sum_f64(s) / n;
    double v = 0.0;
    for (int i = lane; i < n; i += 64) { const double d = (double)wo[i] - mu; v += d * d; }
    const double sd = sqrt(wave_sum_f64(v) / n), sc = (double)gain / (sd * sqrt((double)n) + (double)eps);
    for (int i = lane; i < n; i += 64) ho[i] = (float)(((double)wo[i] - mu) * sc);
}
extern "C" void nn_ws_fwd(float *wh, const float *w, int cout, int n, float gain, float eps) {
    if (cout > 0 && n > 0) { ws_fwd_k<<<nblk_((size_t)cout, 4), 256>>>(wh, w, cout, n, gain, eps); MICK(); }
}

// ---- slab-local GroupNorm statistics (src/nn_lp.h:15-20, src/nn_fwd.cu:5-35): statistics arrays that hold one row per (sample, z-slab),
// [n][ns][G], and their geometry; every gnp_t made by gnp_mk from a registered mean array carries it. ns <= 0 removes mean's entry, a null
// mean clears the registry ----
static struct { const float *mean; int zs, zo, ns, zhw; } g_slab[32];
static int g_nslab = 0;
static std::mutex g_slab_mu;
extern "C" void lp_gn_slab_reg(const float *mean, int zs, int zo, int ns, int zhw) {
    std::lock_guard<std::mutex> lk(g_slab_mu);
    if (!mean) { g_nslab = 0; return; }
    int i = 0;
    while (i < g_nslab && g_slab[i].mean != mean) i++;
    if (ns <= 0) { if (i < g_nslab) g_slab[i] = g_slab[--g_nslab]; return; }
    if (zs <= 0 || zo < 0 || zo >= zs || zhw <= 0) mi_die("lp_gn_slab_reg: %d planes per slab, offset %d, %d voxels per plane", zs, zo, zhw);
    if (i == g_nslab) { if (g_nslab == 32) mi_die("lp_gn_slab_reg: more than 32 slab statistics arrays"); g_nslab++; }
    g_slab[i].mean = mean; g_slab[i].zs = zs; g_slab[i].zo = zo; g_slab[i].ns = ns; g_slab[i].zhw = zhw;
}
extern "C" int lp_gn_slab_any(void) { std::lock_guard<std::mutex> lk(g_slab_mu); return g_nslab > 0; }
extern "C" gnp_t gnp_mk(const float *gamma, const float *beta, const float *mean, const float *rstd, int G) {   // src/nn_lp.h:19
    gnp_t g; memset(&g, 0, sizeof g); g.gamma = gamma; g.beta = beta; g.mean = mean; g.rstd = rstd; g.G = G;
    if (G > 0 && mean) {
        std::lock_guard<std::mutex> lk(g_slab_mu);
        for (int i = 0; i < g_nslab; i++) if (g_slab[i].mean == mean) { g.zs = g_slab[i].zs; g.zo = g_slab[i].zo; g.ns = g_slab[i].ns; g.zhw = g_slab[i].zhw; break; }
    }
    return g;
}

// ---- the op layer's answers about masked convs and the z-window (src/nn_skip.cu:130-157, src/nn_bwd.cu:57): weak, so the reference's own
// definitions replace them when this library is linked into it; standing alone every conv is dense and no window is set ----
extern "C" __attribute__((weak)) skipm_t lp_skip_get(shape5, split_t, int) { skipm_t s; memset(&s, 0, sizeof s); return s; }
extern "C" __attribute__((weak)) int nn_skip_fwd_level(shape5, split_t) { return 0; }
extern "C" __attribute__((weak)) int nn_skip_masks(shape5, split_t) { return 0; }
extern "C" __attribute__((weak)) int zw_win(int, int *, int *) { return 0; }
