/* Op layer of the MX forward path (C23): storage registry, precision policy and the conv entry points that choose the kernel
   family, own the GroupNorm sum slots and finalize them. Restates what src/nn_bwd.cu:83-155, src/nn_wgrad.cu:103-145,
   src/nn_fusedgn.cu:22-70 and src/nn_core.cu:376-390 do around the lp_* kernels; no arithmetic happens here. */
#include "../../include/mi_unet.h"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#if __STDC_VERSION__ < 202311L      /* (this image's gcc 11 implements C2x without the nullptr constant) */
#define nullptr ((void *)0)
#endif

/* ---- storage registry: device ranges holding MX (or fp16) tensors (src/nn_core.cu:376-390) ---- */
typedef struct { const char *p; size_t bytes; int dt; } reg_t;
static reg_t *g_reg; static int g_nreg, g_capreg;
void nn_storage_forget(const void *p) {
    for (int i = 0; i < g_nreg; i++) if (g_reg[i].p == (const char *)p) { g_reg[i] = g_reg[--g_nreg]; return; }
}
void nn_set_storage(const void *p, size_t bytes, int dt) {
    nn_storage_forget(p);
    if (!dt || !p) return;
    if (g_nreg == g_capreg) { g_capreg = g_capreg ? 2 * g_capreg : 64; g_reg = realloc(g_reg, (size_t)g_capreg * sizeof *g_reg); if (!g_reg) { fprintf(stderr, "nn_set_storage: out of memory\n"); abort(); } }
    g_reg[g_nreg++] = (reg_t){(const char *)p, bytes, dt};
}
int nn_storage(const void *p) {
    for (int i = 0; i < g_nreg; i++) if ((const char *)p >= g_reg[i].p && (const char *)p < g_reg[i].p + g_reg[i].bytes) return g_reg[i].dt;
    return 0;
}
static int g_prec = 0, g_gn_stored = 0;
void nn_set_prec(int p) { g_prec = p; }
int nn_get_prec(void) { return g_prec; }
void nn_set_gn_stored(int on) { g_gn_stored = on; }
size_t nn_mx8_bytes(shape5 s) { return lp_mx8_bytes(s.n, s.c, (size_t)s.d * s.h * s.w); }
size_t nn_mx4_bytes(shape5 s) { return lp_mx4_bytes(s.n, s.c, (size_t)s.d * s.h * s.w); }
const char *nn_check(void) { return lp_check(); }

/* lp dtype code of a tensor (0 fp32, 2 fp16, 3 MX-fp8, 4 MX-fp4) from the registry (ISMX / MXDT, src/nn_common.cuh:118-127) */
static int lp_dt(const void *p) { const int dt = nn_storage(p); return dt == 8 ? 3 : dt == 4 ? 4 : dt == 2 ? 2 : 0; }

/* the GroupNorm sum slots of the conv in flight (gn_dsums, src/nn_elem.cu:12-17): one grow-only device buffer */
static double *g_sums; static size_t g_sums_cap;
static double *gn_dsums(size_t nslots) {
    if (nslots > g_sums_cap) { if (g_sums) mi_free(g_sums); g_sums = mi_malloc(nslots * MI_GN_SLOT_BYTES); g_sums_cap = nslots; }
    return g_sums;
}
/* statistics of the decoded stored output instead of the pre-quantisation values (gn_fused_stored, src/nn_bwd.cu:67-72) */
static int gn_fused_stored(int ydt, int cout) { return g_gn_stored && ydt >= 3 && cout >= 16; }

/* z-range (src/nn_bwd.cu:33-46): the next 3^3 stride-1 MX convs compute output planes [zo, zo + xs.d) of a depth-Do tensor, output plane z
   reading input plane z + zi0 of a depth-Di input; their output GroupNorm sums are zeroed only by the first slab's call and finalised
   (over all Do planes) only by the last's. Di 0 = off. With nn_set_zrange_out the MX outputs go straight to their planes of the depth-Do
   output tensor instead of a depth-xs.d one. Per host thread. */
static _Thread_local int g_zr_z0, g_zr_Di, g_zr_first, g_zr_last, g_zr_Do, g_zr_zo, g_zr_out;
void nn_set_zrange(int zi0, int Di, int first, int last, int Do, int zo) { g_zr_z0 = zi0; g_zr_Di = Di; g_zr_first = first; g_zr_last = last; g_zr_Do = Do; g_zr_zo = zo; }
void nn_set_zrange_out(int on) { g_zr_out = on; }

/* The kernel family of a 3^3 stride-1 conv, the reference's rule (conv_fwd_tc, src/nn_bwd.cu:97-119): with MX storage on either side, a 16-bit
   network input of <= 8 channels or an input whose MX format differs from the output's (<= 8 channels, or MX-fp8 in and MX-fp4 out: the
   independently quantised stem) runs the fp8 entry, an MX-fp4 input with fp32 planes out the fp4 entry (the reference's tests); otherwise input,
   second segment and output must share one MX format, and MX-fp4 storage or precision 3 runs the fp4 kernels, everything else fp8. Without MX
   storage precision 2 / 3 run the fp8 / fp4 entry on the planes as they are (no fused upsample there). Returns 8 or 4; anything else is a
   16-bit tensor-core conv, which this library does not hold: it says so and aborts, as the reference does for its unsupported combinations. */
static int conv_family(const char *who, int xdt, int ydt, int x2dt, int has_x2, int cin, int cout, int up) {
    if (xdt >= 3 || ydt >= 3) {
        if (xdt == 2 && ydt >= 3 && cin <= 8 && !has_x2) return 8;
        if (xdt >= 3 && ydt >= 3 && xdt != ydt && (cin <= 8 || (xdt == 3 && ydt == 4)) && !has_x2 && !up) return 8;
        if (xdt == 4 && ydt == 0) return 4;
        /* (one extension to the reference's one-format rule: under precision 3 an MX-fp8 conv may take its second segment as MX-fp4 rows - a skip the
           graph transformed once for two readers of different compute formats; the conv entry is told through mi_conv_x2_dt) */
        if (xdt < 3 || ydt != xdt || (has_x2 && x2dt != xdt && !(xdt == 3 && x2dt == 4 && g_prec == 3))) {
            fprintf(stderr, "%s: MX storage needs MX inputs and outputs of one format (x %d y %d x2 %d, %dx%d ch)\n", who, xdt, ydt, has_x2 ? x2dt : -1, cin, cout);
            abort();
        }
        return xdt == 4 || g_prec == 3 ? 4 : 8;
    }
    if (g_prec == 2 && !up) return 8;
    if (g_prec == 3 && !up) return 4;
    fprintf(stderr, "%s: neither MX storage nor precision 2 / 3 (precision %d): the 16-bit tensor-core convs are not part of this library\n", who, g_prec);
    abort();
}

/* one 3^3 stride-1 conv of the op layer: family by conv_family, the GroupNorm sum slots' lifecycle (zero, conv with fused sums, finalize;
   spread over the slab calls under a z-range), statistics of the stored output by a separate pass when nn_set_gn_stored asks for them and the
   epilogue cannot supply them (src/nn_wgrad.cu:103-124) */
static int conv_s1(const char *who, const float *x, shape5 xs, const float *w, const float *b, int cout, float *y, gnp_t gp, split_t sp,
                   int G_out, float eps, float *omean, float *orstd) {
    const int xdt = lp_dt(x), ydt = lp_dt(y), x2dt = sp.x2 ? lp_dt(sp.x2) : 0;
    const int fam = conv_family(who, xdt, ydt, x2dt, sp.x2 != nullptr, xs.c, cout, sp.up);
    int (*const conv)(const void *, int, shape5, const float *, const float *, int, void *, int, gnp_t, double *, int, split_t) = fam == 4 ? lp_conv_fwd_f4 : lp_conv_fwd_f8;
    sp.wkey = (unsigned)((uintptr_t)w >> 4) | 1u;                   /* inference: weights are prepared once per conv (keyed by the weight pointer) */
    if (sp.x2 && x2dt >= 3 && x2dt != xdt) mi_conv_x2_dt(x2dt);
    if (G_out > cout) G_out = cout;                                 /* GroupNorm uses min(G, C) groups (src/nn_wgrad.cu:105) */
    const int want = G_out > 0 && omean && orstd;
    const int fused = gn_fused_stored(ydt, cout);
    double *sums = nullptr;
    if (want && (!g_gn_stored || fused)) { sums = gn_dsums((size_t)2 * xs.n * G_out); sp.stored_stats = fused; }
    if (g_zr_Di) {                                                  /* a slab of the conv: zero / accumulate / finalize spread over the calls */
        if (xdt < 3 || ydt < 3) { fprintf(stderr, "%s: the z-range needs MX storage\n", who); return -1; }
        if (want && !sums) { fprintf(stderr, "%s: the z-range needs fused output statistics\n", who); abort(); }
        sp.zi0 = (int16_t)g_zr_z0; sp.Di = (int16_t)g_zr_Di;
        if (g_zr_out) { sp.yzo = (int16_t)g_zr_zo; sp.yD = (int16_t)g_zr_Do; }
        if (sums && g_zr_first) mi_gn_sums_zero(sums, 2 * xs.n * G_out);
        conv(x, xdt, xs, w, b, cout, y, ydt, gp, sums, sums ? G_out : 0, sp);
        if (sums && g_zr_last) mi_gn_finalize(sums, xs.n * G_out, (size_t)(cout / G_out) * g_zr_Do * xs.h * xs.w, eps, omean, orstd);
        return 0;
    }
    /* with output statistics: the conv's reduction sets the slots and finalizes them (the reference's zero / conv / finalize sequence,
       src/nn_bwd.cu:37-56, in one call) */
    if (sums) mi_conv_fwd_gn(fam, x, xdt, xs, w, b, cout, y, ydt, gp, sums, G_out, sp, eps, omean, orstd);
    else conv(x, xdt, xs, w, b, cout, y, ydt, gp, nullptr, 0, sp);
    if (want && !sums) { const shape5 ys = {xs.n, cout, xs.d, xs.h, xs.w}; return nn_gn_stats(y, ys, G_out, eps, omean, orstd); }
    return 0;
}

int nn_conv3d_fwd_x(const float *x, const nn_gn_t *gx, const float *x2, const nn_gn_t *gx2, int c_split, int up, shape5 xs,
                    const float *w, const float *b, int cout, int k, int stride, float *y, int G_out, float eps, float *omean, float *orstd) {
    const int xdt = lp_dt(x), ydt = lp_dt(y);
    if (x2 && lp_dt(x2) != xdt && !(xdt == 3 && lp_dt(x2) == 4 && g_prec == 3)) { fprintf(stderr, "nn_conv3d_fwd_x: x and x2 differ in storage\n"); return -1; }      /* (the exception: conv_family) */
    gnp_t gp = gx ? gnp_mk(gx->gamma, gx->beta, gx->mean, gx->rstd, gx->G) : gnp_mk(nullptr, nullptr, nullptr, nullptr, 0);
    if (k == 1) {                                                   /* the head: MX input, fp32 (or registered fp16) planes out (src/nn_fusedgn.cu:57-62) */
        if (xdt < 3 || x2 || stride != 1 || G_out) return -1;
        if (ydt == 2) lp_conv1_fwd_mx_h16(x, xdt, xs, w, b, cout, y, gp); else lp_conv1_fwd_mx(x, xdt, xs, w, b, cout, y, gp);
        return 0;
    }
    if (k != 3) return -1;
    if (stride == 2) {                                              /* down conv: no split, no output statistics (src/nn_bwd.cu:120-155) */
        if (x2 || G_out) return -1;
        if (xdt < 3 && !((g_prec == 2 || g_prec == 3) && ydt == xdt)) return -1;      /* planes: only under precision 2 / 3, same type out (src/nn_bwd.cu:129-130) */
        if (xdt >= 3 && ydt != xdt) { fprintf(stderr, "conv s2: MX storage needs MX input and output of one format\n"); abort(); }      /* src/nn_bwd.cu:123 */
        const shape5 ys = {xs.n, cout, (xs.d - 1) / 2 + 1, (xs.h - 1) / 2 + 1, (xs.w - 1) / 2 + 1};
        mi_conv_s2_wkey((unsigned)((uintptr_t)w >> 4) | 1u);        /* inference: prepared once per conv, as the stride-1 convs below */
        lp_conv_fwd_s2_f8(x, xdt, xs, w, b, cout, y, ydt, ys, gp);
        return 0;
    }
    if (stride != 1) return -1;
    split_t sp; memset(&sp, 0, sizeof sp);
    if (x2) { sp.x2 = x2; sp.c_split = c_split; sp.up = (int16_t)up; if (gx2) sp.gp2 = gnp_mk(gx2->gamma, gx2->beta, gx2->mean, gx2->rstd, gx2->G); }   /* (gx2->G -1: x2 without GroupNorm) */
    else if (up) return -1;
    return conv_s1("nn_conv3d_fwd_x", x, xs, w, b, cout, y, gp, sp, G_out, eps, omean, orstd);
}
int nn_conv3d_fwd_gn_stats(const float *x, shape5 xs, int G_in, const float *gamma, const float *beta, const float *mean, const float *rstd,
                           const float *w, const float *b, int cout, float *y, int G_out, float eps, float *omean, float *orstd) {
    if (G_in > xs.c) G_in = xs.c;                                   /* GroupNorm uses min(G, C) groups (src/nn_wgrad.cu:105) */
    const nn_gn_t g = {gamma, beta, mean, rstd, G_in};
    return nn_conv3d_fwd_x(x, G_in ? &g : nullptr, nullptr, nullptr, 0, 0, xs, w, b, cout, 3, 1, y, G_out, eps, omean, orstd);
}
shape5 nn_conv3d_out_shape(shape5 xs, int cout, int k, int stride) {   /* src/nn_bwd.cu:132-135 */
    const shape5 o = {xs.n, cout, (xs.d + 2 * (k / 2) - k) / stride + 1, (xs.h + 2 * (k / 2) - k) / stride + 1, (xs.w + 2 * (k / 2) - k) / stride + 1};
    return o;
}
/* the plain conv (src/nn.h:400, src/nn_bwd.cu:136-141): the 1^3 head of an MX tensor, the 3^3 stride-1 and stride-2 convs on MX storage or, under
   precision 2 / 3, on fp32 planes; no GroupNorm on either side. Unsupported combinations print and abort, as in the reference */
void nn_conv3d_fwd(const float *x, shape5 xs, const float *w, const float *b, int cout, int k, int stride, float *y) {
    if (nn_conv3d_fwd_x(x, nullptr, nullptr, nullptr, 0, 0, xs, w, b, cout, k, stride, y, 0, 0.f, nullptr, nullptr)) {
        fprintf(stderr, "nn_conv3d_fwd: unsupported k=%d stride=%d for this storage (x %d, y %d)\n", k, stride, lp_dt(x), lp_dt(y));
        abort();
    }
}
/* the conv of silu(gn(x)) without materialising the activation (src/nn.h:416, src/nn_wgrad.cu:93-102) */
int nn_conv3d_fwd_gn(const float *x, shape5 xs, int G, const float *gamma, const float *beta, const float *mean, const float *rstd,
                     const float *w, const float *b, int cout, float *y) {
    return nn_conv3d_fwd_gn_stats(x, xs, G, gamma, beta, mean, rstd, w, b, cout, y, 0, 0.f, nullptr, nullptr);
}
/* the conv of the channel concat [x, x2] (c_split = channels of x), one GroupNorm of G_in groups over all xs.c channels on the input side when
   G_in > 0, output statistics for G_out groups (src/nn.h:442, src/nn_wgrad.cu:125-145) */
int nn_conv3d_fwd_split(const float *x, const float *x2, int c_split, shape5 xs, int G_in, const float *gamma, const float *beta, const float *mean, const float *rstd,
                        const float *w, const float *b, int cout, float *y, int G_out, float eps, float *omean, float *orstd) {
    if (G_in > xs.c) G_in = xs.c;
    if (!x2) return -1;
    split_t sp; memset(&sp, 0, sizeof sp);
    sp.x2 = x2; sp.c_split = c_split;                               /* (gp2.G 0: gp spans both segments) */
    return conv_s1("nn_conv3d_fwd_split", x, xs, w, b, cout, y, gnp_mk(gamma, beta, mean, rstd, G_in), sp, G_out, eps, omean, orstd);
}
int nn_gn_stats(const float *x, shape5 s, int G, float eps, float *mean, float *rstd) {
    const int dt = lp_dt(x);
    if (dt < 3 || G <= 0 || s.c % G) return -1;
    const size_t S = (size_t)s.d * s.h * s.w;
    double *sums = gn_dsums((size_t)2 * s.n * G);
    mi_gn_sums_zero(sums, 2 * s.n * G);
    if (lp_gn_sums_mx(x, dt, s.n, s.c, G, S, sums, 0, S)) return -1;
    mi_gn_finalize(sums, s.n * G, (size_t)(s.c / G) * S, eps, mean, rstd);
    return 0;
}
