/* The U-Net inference graph (C23) over the op layer: two 3x3x3 convs per level with GroupNorm statistics fused into their
   epilogues and the GroupNorm + SiLU applied by the next reader while it stages its input (recompute mode: no activated tensor is
   ever stored), 3x3x3 stride-2 down convs, decoder conv1 reading [up2(coarse) | skip] without materialising either, 1x1x1 head.
   Parameter layout: src/unet.c:451-459 (unet_create); initialisation: src/unet.c:588-607 (unet_init); layer order: src/unet.c:2567-2636, :2939-3105 (block_fwd, unet_forward_x). */
#include "../../include/mi_unet.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#if __STDC_VERSION__ < 202311L      /* (this image's gcc 11 implements C2x without the nullptr constant) */
#define nullptr ((void *)0)
#endif

typedef struct { size_t w, b; int cin, cout, k; } convp;           /* offsets into the flat parameter vector */
typedef struct { size_t gamma, beta; int c; } gnpar;
typedef struct {
    convp c1, c2; gnpar n1, n2;
    shape5 xs, ys;                                                 /* conv1 input shape (all its channels), block output shape */
    void *a1, *a2;                                                 /* conv outputs (pre-norm, MX) */
    int single;                                                    /* cfg.dec_convs 1: one conv, its output is a2 with the statistics m2 / r2 and the norm n2 = n1; no c2, a1 unused (src/unet.c:69, :357-362) */
    float *m1, *r1, *m2, *r2;                                      /* their GroupNorm statistics [n * G] */
} block;
struct unet {
    unet_cfg cfg;
    /* the activations, built for one input shape and storage mode (rebuilt when either changes: src/unet.c:2876) */
    int built, act_dt, prec; shape5 in; shape5 ls[UNET_MAXLEV];
    /* cfg.l0_norm 1 .. 3 (src/unet.h:52-58): the level-0 GroupNorms on constant statistics: mean 0 / rstd 1 (none, ws) or the checkpoint's running
       statistics once its warm-up is over (ema: l0run = [live weights: 4 sites x (mean G | var G)][EMA weights: the same], device; l0_n updates so far) */
    float *l0run; long l0_n; int l0_warm; float l0_mom; float ws_gain;
    /* cfg.film (src/unet.h:108-111): K codes per forward scale and shift the output norms of the encoder blocks (level 0 up) and then of the decoder
       blocks (coarsest first): film_off = the first norm's K x C scale / shift pair, the pairs in that order; the effective affines live in the
       forward weight copy. cfg.gfilm (src/unet.h:60-64): the decoder blocks' output norms once more, by the attention stage's output averaged over
       the window's tokens (gf_K = widths[L-1] device codes gf_g); gf_g1 keeps the affines before */
    size_t film_off, gf_off; float film_c[4]; int film_ok, gf_K; float *gf_g, *gf_g1;
    size_t sc_w; float sc_c; float *stem_b;                        /* cfg.scale_cond (src/unet.h:24, src/unet.c:129): the conditioning vector's offset, the current code, the stem bias b + c v of a forward */
    /* cfg.gn_ema (src/unet.h:67-71): every GroupNorm (all levels, down norms, the attention stage's) on the checkpoint's running statistics:
       ge_run = [live weights: ge_ns values][EMA weights: the same], per site pair [mean G | var G] in the order of gn_sites (src/unet.c:5125-5135) */
    float *ge_run; size_t ge_ns; long ge_n; int ge_warm, ge_live; float ge_mom;
    int l0s_zs, l0s_ns;                /* cfg.l0_norm 4: planes per statistics slab and slabs of the current build (0: per-sample statistics) */
    int slab_ip, slab_nl, slab_s;      /* the build's in-place slab plan: on, and over how many levels (a level's tensors all live in enc[i].a2's buffer) */
    void *slab_tmp[2], *slab_carry[2]; /* per such level: one slab of output planes, and the plane that waits for the next slab */
    block enc[UNET_MAXLEV], dec[UNET_MAXLEV];
    block *rb[UNET_MAXLEV]; char (*rbn[UNET_MAXLEV])[2][16];      /* cfg.enc_blocks: residual blocks after encoder level i (src/unet.c:96, :461-465), the names of their convs */
    convp down[UNET_MAXLEV], head;
    convp ds[UNET_MAXLEV], eh;         /* cfg.ds_levels / cfg.emb_lev: the deep-supervision heads of decoder levels 1 .. ds_levels and the distillation head: training-time outputs, here only their place in the parameter vector (src/unet.c:467, :511) */
    void *downo[UNET_MAXLEV];
    void *skipst[UNET_MAXLEV];         /* silu(gn(enc[i].a2)) in the compute format, formed once for its two readers (down conv, decoder conv1); null: each reader transforms it */
    void *skipst4[UNET_MAXLEV];        /* precision 3 over MX-fp8 storage: the two readers compute in different formats (the stride-2 conv in e4m3, the decoder's in e2m1);
                                          the same pass writes the MX-fp4 rows here beside the MX-fp8 ones in skipst */
    gnpar dn[UNET_MAXLEV]; float *dm[UNET_MAXLEV], *dr[UNET_MAXLEV];   /* down_norm: GroupNorm after down[i], its statistics */
    size_t np; float *p, *ema, *params;                            /* device: live weights, EMA copy, the one the forward reads */
    float *src, *wm; int wm_ok;                                    /* cfg.w4_2d: the selected weights (p or ema), their forward copy with the fp4 convs' weights rounded per 32 x 32 block, whether it is current */
    void *xin;                                                     /* the network input as an MX tensor */
    float *logits;                                                 /* [n][cout][S], owned by the net */
    struct { const void *p; shape5 s; const char *name; const float *mean, *rstd; int G; } outs[64]; int nouts;
    /* the attention stage on the bottleneck (src/unet.c:470-509 set-up, :2795-2835 forward) */
    int tbn; at_dims tbd; at_bp tbp[16]; size_t reg_off; at_geom tbg; at_ws tbw;
    block tb;                                                      /* its output: a2 and the statistics m2 / r2 (the level's n2 affine) */
    size_t peg_w, peg_b;                                           /* cfg.attn_pe 0: the conv positional encoding's parameters */
    float *tb_vr; size_t vr_off;                                   /* cfg.attn_vres (src/unet.h:81): the first application's V rows; the lerps' offset */
    float *tb_cs, *tb_tok; void *tb_ws;                            /* fp32 planes [n][C][Sg]; token rows, one buffer per block + 1; block scratch */
    /* cfg.attn_axis 1 / attn_pe 3: the scroll geometry (src/unet.c:280-282). One device buffer tb_rb holds the ray table, lengths, axis dims, ray
       positions, stencil weight sums, the grid tokens' scroll coordinates and the per-plane frames; the host side of a plan; the axis records */
    at_rays tbr; float *tb_rb, *tb_gpos, *tb_cen, *tb_rayh, *tb_cenh, *tb_axb, *tb_axh; int *tb_lensh, *tb_adh;
    void *tb_pin[2], *tb_fence[2]; int tb_set;                     /* the plan's host tables: two pinned sets copied in stream order, each rewritten only after its copy ran */
    int tb_Q, tb_Nt, tb_Nr, tb_axn, tb_axs, tb_axdirty, tb_axwarn, tb_noax;
};

/* activation storage of the nets built from now on (src/unet.c:700-706): MX-fp8 unless MX-fp4 is asked for */
static int g_act_mx8 = 1, g_act_mx4 = 0;
void unet_set_act_mx8(int on) { g_act_mx8 = on != 0; }
void unet_set_act_mx4(int on) { g_act_mx4 = on != 0; }
int unet_act_mx(void) { return g_act_mx8 || g_act_mx4; }
static int act_dt_now(void) { return g_act_mx4 ? 4 : 8; }

static int G_of(const unet *u, int c) { return u->cfg.G < c ? u->cfg.G : c; }      /* src/unet.c:297 */
static size_t add_conv(convp *c, int cin, int cout, int k, size_t off) { c->cin = cin; c->cout = cout; c->k = k; c->w = off; off += (size_t)cout * cin * k * k * k; c->b = off; return off + cout; }
/* output channels of the block the decoder upsamples into level i - 1: cfg.dec_widths[i], 0 or the bottom level: the encoder's (src/unet.c:298-300) */
static int dw_of(const unet_cfg *c, int i) { return i >= c->nlev - 1 || !c->dec_widths[i] ? c->widths[i] : c->dec_widths[i]; }
static size_t add_gn(gnpar *g, int c, size_t off) { g->c = c; g->gamma = off; g->beta = off + c; return off + 2 * (size_t)c; }
static size_t act_bytes(const unet *u, shape5 s) { return u->act_dt == 4 ? nn_mx4_bytes(s) : nn_mx8_bytes(s); }
static void *act_new(const unet *u, shape5 s) { const size_t b = act_bytes(u, s); void *p = mi_malloc(b); mi_zero(p, b); nn_set_storage(p, b, u->act_dt); return p; }
static void act_del(void *p) { if (p) { nn_storage_forget(p); mi_free(p); } }
static float *f32_new(size_t n) { float *p = mi_malloc(n * 4); mi_zero(p, n * 4); return p; }

/* the attention stage reads the scroll axis (unet_cfg_axis, src/unet.h): radial attention or the scroll rotary embedding */
static int cfg_axis(const unet_cfg *c) { return c->attn_blocks > 0 && (c->attn_axis == 1 || c->attn_pe == 3); }
/* radial attention: rays per axis-normal plane / the grid's largest dim (the reference's environment knob UFSM_ATTN_RAY_MULT, default 2; src/unet.c:692-694) */
static float attn_ray_mult(void) { static float m = 0; if (m <= 0) { const char *e = getenv("UFSM_ATTN_RAY_MULT"); m = e && atof(e) > 0 ? (float)atof(e) : 2.f; } return m; }
static void tb_geom_free(unet *u) {
    if (u->tb_rb) mi_free(u->tb_rb);
    for (int k = 0; k < 2; k++) { if (u->tb_fence[k]) { mi_fence_wait(u->tb_fence[k]); mi_fence_free(u->tb_fence[k]); } if (u->tb_pin[k]) mi_host_free(u->tb_pin[k]); u->tb_pin[k] = u->tb_fence[k] = nullptr; }
    free(u->tb_axb);
    u->tb_rb = u->tb_gpos = u->tb_cen = u->tb_rayh = u->tb_cenh = u->tb_axb = nullptr; u->tb_lensh = u->tb_adh = nullptr;
    u->tbr = (at_rays){0}; u->tbg.rays = nullptr; u->tbg.pos = nullptr;
}

/* a field of the reference's configuration this build's graph does not run: named, so the caller knows which */
static const char *cfg_unsupported(const unet_cfg *c) {
    for (int i = 0; i < UNET_MAXLEV; i++) {
        /* decoder widths: at most the level's encoder width, and that width at level 0 (the head's input); the bottom level has no decoder (src/unet.c:452-455) */
        if (c->dec_widths[i] && (i >= c->nlev - 1 || c->dec_widths[i] > c->widths[i] || c->dec_widths[i] < 0 || (i == 0 && c->dec_widths[0] != c->widths[0]))) return "dec_widths";
        if (c->enc_blocks[i] < 0 || c->enc_blocks[i] > 64 || (c->enc_blocks[i] && (i == 0 || i >= c->nlev))) return "enc_blocks (levels 1 and deeper)";      /* (src/unet.c:462) */
        if (c->dec_convs[i] && c->dec_convs[i] != 2 && c->dec_convs[i] != 1) return "dec_convs";
    }
    if (c->ds_levels < 0 || (c->ds_levels > 0 && c->ds_levels > c->nlev - 2)) return "ds_levels (decoder levels 1 .. nlev - 2)";      /* (src/unet.c:466) */
    if (c->lat_guide || c->lat_nsub) return "lat_guide";
    if (c->l0_norm < 0 || c->l0_norm > 4) return "l0_norm (0 GroupNorm, 1 none, 2 ema, 3 ws, 4 slab)";
    if (c->l0_norm == 2 && (c->G < c->widths[0] ? c->G : c->widths[0]) > 64) return "l0_norm 2 with more than 64 groups";
    if (c->l0_norm == 4 && c->widths[0] > 32) return "l0_norm 4 with more than 32 level-0 channels";   /* (one MX channel block: a slab is a sample of the same layout) */
    if (c->l0_slab && c->l0_norm != 4) return "l0_slab without l0_norm 4";
    if (c->gfilm && (!c->attn_blocks || c->nlev < 2)) return "gfilm without the attention stage (src/unet.c:517)";
    if (c->gn_ema && c->l0_norm) return "gn_ema with l0_norm (src/unet.c:551)";
    if (c->attn_vres && !c->attn_blocks) return "attn_vres without attention blocks";
    if (c->attn_axis < 0 || c->attn_axis > 1 || (c->attn_axis && (!c->attn_blocks || c->attn_reg))) return "attn_axis (0 or 1; radial attention takes no register tokens, src/unet.c:471-472)";
    if (c->attn_repeat < 0 || (c->attn_repeat > 1 && (!c->attn_blocks || c->attn_blocks * c->attn_repeat > 64))) return "attn_repeat";
    if (c->attn_mem) return "attn_mem";
    if (c->view_P || c->view_patch) return "view_P";
    if (c->attn_deform || c->attn_dlev || c->attn_dco || c->attn_dinit) return "attn_deform";
    if (c->emb_lev < 0 || (c->emb_lev > 0 && (c->emb_lev > c->nlev - 2 || c->emb_ch <= 0)) || (!c->emb_lev && c->emb_ch)) return "emb_lev (decoder levels 1 .. nlev - 2, at least one channel)";      /* (src/unet.c:510) */
    if (c->film < 0 || c->film > 4) return "film (0 .. 4 codes, src/unet.c:512)";
    if (c->skip_thr || c->skip_margin || c->skip_nl) return "skip_empty";
    if (c->fstem || c->fstem_out) return "fstem";
    if (c->lat_dec || c->lat_dec_raw || c->lat_dec_ng || c->lat_dec_wq) return "lat_dec";
    return nullptr;
}

/* the GroupNorm statistics sites in the reference's order (gn_sites, src/unet.c:5125-5135): encoder blocks (conv1's, conv2's), down norms,
   decoder blocks from the coarsest, the attention stage's output; a site is a (mean, rstd) pair of g groups, its running statistics
   [mean g | var g] at offset off. Fills up to 192 entries when the arrays are given; returns the number of values. */
static size_t ge_sites(unet *u, float **mean, float **rstd, int *g, size_t *off) {
    size_t o = 0; int k = 0; const int L = u->cfg.nlev;
#define GE_SITE(m, r, gg) do { if (mean && k < 192) { mean[k] = (m); rstd[k] = (r); g[k] = (gg); off[k] = o; } k++; o += 2 * (size_t)(gg); } while (0)
    for (int i = 0; i < L; i++) { block *b = &u->enc[i]; GE_SITE(b->m1, b->r1, G_of(u, b->c1.cout)); GE_SITE(b->m2, b->r2, G_of(u, b->c2.cout)); }
    if (u->cfg.down_norm) for (int i = 0; i < L - 1; i++) GE_SITE(u->dm[i], u->dr[i], G_of(u, u->cfg.widths[i]));
    for (int i = L - 2; i >= 0; i--) { block *b = &u->dec[i]; GE_SITE(b->m1, b->r1, G_of(u, b->c1.cout)); GE_SITE(b->m2, b->r2, G_of(u, b->c2.cout)); }
    for (int i = 0; i < L; i++) for (int j = 0; j < u->cfg.enc_blocks[i]; j++) { block *b = &u->rb[i][j]; GE_SITE(b->m1, b->r1, G_of(u, b->c1.cout)); GE_SITE(b->m2, b->r2, G_of(u, b->c2.cout)); }
    if (u->tbn) GE_SITE(u->tb.m2, u->tb.r2, G_of(u, u->tbd.C));
#undef GE_SITE
    if (mean && k > 192) { fprintf(stderr, "unet: gn_ema: %d GroupNorm sites (at most 192)\n", k); abort(); }
    return o;
}
/* cfg.film's norms, j < 2 L - 1: the encoder blocks' output norms from level 0, then the decoder blocks' from the coarsest (src/unet.c:372-373) */
static const gnpar *film_norm(const unet *u, int j) { const int L = u->cfg.nlev; return j < L ? &u->enc[j].n2 : &u->dec[L - 2 - (j - L)].n2; }
unet *unet_create(const unet_cfg *cfg) {
    const int L = cfg->nlev;
    if (L < 1 || L > UNET_MAXLEV || cfg->cin < 1 || cfg->cout < 1 || cfg->G < 1) { fprintf(stderr, "unet_create: bad configuration (nlev %d, cin %d, cout %d, G %d)\n", L, cfg->cin, cfg->cout, cfg->G); return nullptr; }
    for (int i = 0; i < L; i++) if (cfg->widths[i] < 1) { fprintf(stderr, "unet_create: width %d of level %d\n", cfg->widths[i], i); return nullptr; }
    const char *bad = cfg_unsupported(cfg);
    if (bad) { fprintf(stderr, "unet_create: the configuration sets \"%s\", which this build's graph does not run\n", bad); return nullptr; }
    unet *u = calloc(1, sizeof *u);
    if (!u) return nullptr;
    u->cfg = *cfg;
    const int *w = cfg->widths;
    size_t off = 0;
    /* the layout of the reference's unet_create (src/unet.c:451-459): encoder blocks, down convs, decoder blocks from the coarsest, head, down norms, attention stage */
    for (int i = 0; i < L; i++) {
        block *b = &u->enc[i];
        off = add_conv(&b->c1, i ? w[i - 1] : cfg->cin, w[i], 3, off); off = add_gn(&b->n1, w[i], off);
        off = add_conv(&b->c2, w[i], w[i], 3, off); off = add_gn(&b->n2, w[i], off);
    }
    for (int i = 0; i < L - 1; i++) off = add_conv(&u->down[i], w[i], w[i], 3, off);         /* the down conv keeps its level's width (src/unet.c:2970) */
    for (int i = L - 2; i >= 0; i--) {                             /* the decoder blocks from the coarsest (src/unet.c:456); conv1 reads [up2(coarse: dw(i + 1)) | skip: w[i]] */
        block *b = &u->dec[i];
        const int d = dw_of(cfg, i);
        off = add_conv(&b->c1, dw_of(cfg, i + 1) + w[i], d, 3, off); off = add_gn(&b->n1, d, off);
        if (cfg->dec_convs[i] == 1) { b->c2 = b->c1; b->c2.cin = d; b->n2 = b->n1; b->single = 1; }      /* one conv: c2 / n2 alias c1 / n1 */
        else { off = add_conv(&b->c2, d, d, 3, off); off = add_gn(&b->n2, d, off); }
    }
    off = add_conv(&u->head, w[0], cfg->cout, 1, off);
    if (cfg->down_norm) for (int i = 0; i < L - 1; i++) off = add_gn(&u->dn[i], w[i], off);       /* (appended after the head, src/unet.c:459) */
    if (cfg->scale_cond) { u->sc_w = off; off += (size_t)w[0]; }  /* (src/unet.c:460) */
    for (int i = 0; i < L; i++) if (cfg->enc_blocks[i] > 0) {      /* residual blocks after encoder level i: parameters after everything older (src/unet.c:461-465) */
        u->rb[i] = calloc((size_t)cfg->enc_blocks[i], sizeof(block)); u->rbn[i] = calloc((size_t)cfg->enc_blocks[i], sizeof *u->rbn[i]);
        for (int k = 0; k < cfg->enc_blocks[i]; k++) {
            block *b = &u->rb[i][k];
            off = add_conv(&b->c1, w[i], w[i], 3, off); off = add_gn(&b->n1, w[i], off);
            off = add_conv(&b->c2, w[i], w[i], 3, off); off = add_gn(&b->n2, w[i], off);
            snprintf(u->rbn[i][k][0], 16, "rb%d.%d.c1", i, k); snprintf(u->rbn[i][k][1], 16, "rb%d.%d.c2", i, k);
        }
    }
    for (int j = 1; j <= cfg->ds_levels; j++) off = add_conv(&u->ds[j], dw_of(cfg, j), cfg->cout, 1, off);
    if (cfg->attn_blocks > 0) {                                   /* parameters last: registers, then the blocks (src/unet.c:490-499) */
        const int C = w[L - 1];
        if (C % AT_HD || cfg->attn_blocks > 16 || cfg->attn_pe < 0 || cfg->attn_pe > 3 || cfg->attn_reg < 0) {
            fprintf(stderr, "unet_create: attention blocks need a bottleneck width that is a multiple of %d (got %d), at most 16 blocks, attn_pe 0 (PEG), 1 (RoPE), 2 (none) or 3 (scroll RoPE)\n", AT_HD, C);
            free(u); return nullptr;
        }
        const int F = cfg->attn_mlp > 0 ? cfg->attn_mlp : (8 * C / 3 + 31) / 32 * 32;
        u->tbd = (at_dims){.C = C, .H = C / AT_HD, .F = F, .rope = cfg->attn_pe == 1 ? 1 : cfg->attn_pe == 3 ? 2 : 0, .nreg = cfg->attn_reg, .rope_base = 100.f};
        if (cfg->attn_pe == 0) { u->peg_w = off; off += (size_t)C * 27; u->peg_b = off; off += (size_t)C; }      /* the conv positional encoding's depthwise taps and bias, before the registers (src/unet.c:491) */
        u->reg_off = off; off += (size_t)cfg->attn_reg * C;
        for (int k = 0; k < cfg->attn_blocks; k++) off = at_block_layout(&u->tbd, &u->tbp[k], off);
        u->tbn = cfg->attn_blocks;
        if (cfg->attn_vres) { u->vr_off = off; off += (size_t)cfg->attn_blocks * (size_t)(C / AT_HD); }      /* the value residual's per-head lerps, a row per block (src/unet.c:504) */
    }
    if (cfg->emb_lev) off = add_conv(&u->eh, dw_of(cfg, cfg->emb_lev), cfg->emb_ch, 1, off);        /* (after the attention stage, src/unet.c:511) */
    if (cfg->film) { u->film_off = off; for (int j = 0; j < 2 * L - 1; j++) off += (size_t)2 * cfg->film * film_norm(u, j)->c; }      /* (src/unet.c:513) */
    if (cfg->gfilm) {                                              /* one pair per decoder block's output norm, the coarsest first (src/unet.c:516-520) */
        u->gf_K = w[L - 1]; u->gf_off = off;
        int cs = 0;
        for (int i = L - 2; i >= 0; i--) { off += (size_t)2 * u->gf_K * u->dec[i].n2.c; cs += u->dec[i].n2.c; }
        u->gf_g = f32_new((size_t)u->gf_K); u->gf_g1 = f32_new((size_t)cs);
    }
    u->np = off;
    u->p = f32_new(off); u->ema = f32_new(off); u->params = u->src = u->p;
    if (cfg->w4_2d || cfg->l0_norm == 3 || cfg->film || cfg->gfilm) { u->wm = f32_new(off); u->params = u->wm; }
    if (cfg->l0_norm == 3) {           /* 1 / std(silu(z)), z ~ N(0, 1): the gain of the convs that read a SiLU output (the quadrature of src/unet.c:543-547) */
        double s1 = 0, s2 = 0;
        for (int i = -24000; i <= 24000; i++) { const double z = i * 5e-4, p = exp(-0.5 * z * z) * 5e-4 / sqrt(2 * 3.14159265358979323846), y = z / (1 + exp(-z)); s1 += p * y; s2 += p * y * y; }
        u->ws_gain = (float)(1.0 / sqrt(s2 - s1 * s1));
    }
    u->l0_mom = 0.01f; u->l0_warm = 100;                          /* (src/unet.c:549) */
    if (cfg->l0_norm == 2) u->l0run = f32_new((size_t)16 * G_of(u, w[0]));
    if (cfg->gn_ema) {
        u->ge_ns = ge_sites(u, nullptr, nullptr, nullptr, nullptr);
        if (u->ge_ns > 4096) { fprintf(stderr, "unet_create: gn_ema: %zu statistics (at most 4096)\n", u->ge_ns); mi_free(u->p); mi_free(u->ema); if (u->wm) mi_free(u->wm); free(u); return nullptr; }
        u->ge_run = f32_new(2 * u->ge_ns); u->ge_mom = 0.01f; u->ge_warm = 500;      /* (src/unet.c:550) */
    }
    return u;
}
/* inference in z-slabs (src/unet.h:422-424, src/unet.c:2499-2550): the convs of level 0 (and of level 1 in nets of three or more levels,
   src/unet.c:1165) run slab by slab through the z-range; results are those of the whole-tensor convs.
   Direct form (the default, src/unet.c:216, :1167): each slab's planes go straight into the full-depth output tensor.
   In-place form (unet_set_slab_direct(0); src/unet.c:2435-2440): every tensor of such a level lives in one buffer X; a conv whose input is X
   writes its slab into a temp, whose planes but the last then go into X (the next slab still reads the old last plane); that last plane
   waits in a carry plane until the next slab is computed. One slab temp, one plane and X replace a1, a2, the decoder's a1 and a2 and the
   pre-staged skip of the level. */
static int g_infer_slab, g_slab_direct = 1;
void unet_set_infer_slab(int planes) { g_infer_slab = planes > 0 ? (planes + 3) / 4 * 4 : 0; }
void unet_set_slab_direct(int on) { g_slab_direct = on != 0; }
int mi_unet_infer_slab(void) { return g_infer_slab; }
static int slab_levels(const unet *u) {      /* how many of the finest levels run in slabs (UFSM_INFER_SLAB_L1=0: level 0 only) */
    if (!g_infer_slab) return 0;
    const char *e = getenv("UFSM_INFER_SLAB_L1");
    return u->cfg.nlev > 2 && !(e && atoi(e) == 0) ? 2 : 1;
}
static int slab_inplace_now(const unet *u) { return g_infer_slab && !g_slab_direct && u->cfg.nlev > 1; }

/* the activation buffers of the current build */
static void free_acts(unet *u) {
    if (!u->built) return;
    mi_sync();
    for (int i = 0; i < UNET_MAXLEV; i++) {
        for (int s = 0; s < 2; s++) {
            block *b = s ? &u->dec[i] : &u->enc[i];
            if (u->slab_ip && i < u->slab_nl) { if (s) b->a2 = nullptr; b->a1 = nullptr; }       /* (aliases of enc[i].a2) */
            if (i == 0 && u->l0s_ns) { if (b->m1) lp_gn_slab_reg(b->m1, 0, 0, 0, 0); if (b->m2) lp_gn_slab_reg(b->m2, 0, 0, 0, 0); }
            act_del(b->a1); act_del(b->a2); mi_free(b->m1); mi_free(b->r1); mi_free(b->m2); mi_free(b->r2);
            b->a1 = b->a2 = nullptr; b->m1 = b->r1 = b->m2 = b->r2 = nullptr;
        }
        for (int k = 0; k < u->cfg.enc_blocks[i]; k++) {
            block *b = &u->rb[i][k];
            act_del(b->a1); act_del(b->a2); mi_free(b->m1); mi_free(b->r1); mi_free(b->m2); mi_free(b->r2);
            b->a1 = b->a2 = nullptr; b->m1 = b->r1 = b->m2 = b->r2 = nullptr;
        }
        act_del(u->downo[i]); act_del(u->skipst[i]); act_del(u->skipst4[i]); mi_free(u->dm[i]); mi_free(u->dr[i]);
        u->downo[i] = u->skipst[i] = u->skipst4[i] = nullptr; u->dm[i] = u->dr[i] = nullptr;
    }
    if (u->tbn) { act_del(u->tb.a2); mi_free(u->tb.m2); mi_free(u->tb.r2); mi_free(u->tb_cs); mi_free(u->tb_tok); mi_free(u->tb_ws); if (u->tb_vr) mi_free(u->tb_vr); u->tb_vr = nullptr; tb_geom_free(u); u->tb.a2 = nullptr; u->tb.m2 = u->tb.r2 = nullptr; u->tb_cs = u->tb_tok = nullptr; u->tb_ws = nullptr; }
    for (int i = 0; i < 2; i++) { act_del(u->slab_tmp[i]); act_del(u->slab_carry[i]); u->slab_tmp[i] = u->slab_carry[i] = nullptr; }
    act_del(u->xin); u->xin = nullptr;
    mi_free(u->logits); u->logits = nullptr;
    u->built = 0; u->nouts = 0; u->slab_ip = u->slab_nl = u->slab_s = 0; u->l0s_zs = u->l0s_ns = 0;
}
/* (re)build for input shape `in` under the storage mode and precision policy in force (build_acts, src/unet.c:2876) */
static int build_acts(unet *u, shape5 in) {
    const unet_cfg *cfg = &u->cfg; const int L = cfg->nlev; const int *w = cfg->widths;
    if (in.n < 1 || in.c != cfg->cin || in.d < 1 || in.h < 1 || in.w < 1) { fprintf(stderr, "unet: input shape %d x %d x %d x %d x %d does not fit a net of %d input channels\n", in.n, in.c, in.d, in.h, in.w, cfg->cin); return -1; }
    if ((in.d | in.h | in.w) & ((1 << (L - 1)) - 1)) { fprintf(stderr, "unet: spatial size %dx%dx%d must be divisible by %d\n", in.d, in.h, in.w, 1 << (L - 1)); abort(); }   /* (src/unet.c:2875) */
    if (!unet_act_mx()) { fprintf(stderr, "unet: this build stores activations as MX-fp8 or MX-fp4 only (unet_set_act_mx8 / unet_set_act_mx4)\n"); return -1; }
    /* cfg.l0_norm 4: ceil(depth / slab) statistics slabs (src/unet.c:1004). Several slabs must be uniform; a window of at most one slab's depth has a
       single slab, which is the sample: nothing is registered and level 0 runs ordinary GroupNorm on the convs' own statistics (src/unet.c:2336, :2364) */
    const int l0_S = cfg->l0_norm == 4 ? (cfg->l0_slab > 0 ? cfg->l0_slab : 64) : 0, l0_ns = l0_S ? (in.d + l0_S - 1) / l0_S : 0;
    if (l0_ns > 1 && in.d % l0_S) { fprintf(stderr, "unet: l0_norm 4 needs a depth (%d) that is a multiple of the %d planes of a statistics slab (or at most one slab)\n", in.d, l0_S); return -1; }
    free_acts(u);
    u->in = in; u->act_dt = act_dt_now(); u->prec = nn_get_prec();
    /* cfg.l0_norm 4 (src/unet.h:52-59; the kernel path of src/unet.c:992-1003): the four GroupNorms of level 0 take their statistics per z-slab of
       l0_slab planes (0: 64). The statistics arrays hold [n][slab][G] and are registered with their geometry, which every reader's gnp_t then carries */
    u->l0s_ns = l0_ns > 1 ? l0_ns : 0; u->l0s_zs = u->l0s_ns ? l0_S : 0;
    u->slab_ip = slab_inplace_now(u); u->slab_nl = u->slab_ip ? slab_levels(u) : 0; u->slab_s = u->slab_ip ? g_infer_slab : 0;
    /* (a level shares one buffer only if its decoder block has the encoder's width and two convs: the reference's slab_w_ok / any_single
       conditions, src/unet.c:1163; the levels that do not qualify run the direct form) */
    for (int i = 0; i < u->slab_nl; i++) if (u->dec[i].c1.cout != w[i] || u->dec[i].single || cfg->enc_blocks[i]) u->slab_nl = i;
    for (int i = 0; i < L; i++) u->ls[i] = (shape5){in.n, w[i], in.d >> i, in.h >> i, in.w >> i};
    for (int i = 0; i < L; i++) {
        for (int s = 0; s < 2; s++) {
            block *b = s ? &u->dec[i] : &u->enc[i];
            if (s && i == L - 1) continue;
            b->ys = u->ls[i]; b->ys.c = b->c1.cout; b->xs = u->ls[i]; b->xs.c = b->c1.cin;
            if (i < u->slab_nl) { b->a2 = s ? u->enc[i].a2 : act_new(u, b->ys); b->a1 = b->a2; }
            else { b->a1 = b->single ? nullptr : act_new(u, b->ys); b->a2 = act_new(u, b->ys); }
            const size_t ng = (size_t)in.n * G_of(u, b->ys.c) * (i == 0 && u->l0s_ns ? u->l0s_ns : 1);
            b->m1 = f32_new(ng); b->r1 = f32_new(ng); b->m2 = f32_new(ng); b->r2 = f32_new(ng);
            if (i == 0 && u->l0s_ns) { lp_gn_slab_reg(b->m1, u->l0s_zs, 0, u->l0s_ns, in.h * in.w); lp_gn_slab_reg(b->m2, u->l0s_zs, 0, u->l0s_ns, in.h * in.w); }
        }
        for (int k = 0; k < cfg->enc_blocks[i]; k++) {
            block *b = &u->rb[i][k];
            b->ys = b->xs = u->ls[i];
            b->a1 = act_new(u, b->ys); b->a2 = act_new(u, b->ys);
            const size_t ng = (size_t)in.n * G_of(u, w[i]);
            b->m1 = f32_new(ng); b->r1 = f32_new(ng); b->m2 = f32_new(ng); b->r2 = f32_new(ng);
        }
        if (i < L - 1) {
            shape5 ds = u->ls[i + 1]; ds.c = w[i]; u->downo[i] = act_new(u, ds);
            /* both readers of the skip compute in e4m3 from MX-fp8 storage: one shared pre-stage (any other combination: the readers' formats differ) */
            static int skip2 = -1;                                 /* tuning knob MI_UNET_SKIP2=0: under precision 3 each reader transforms the skip itself */
            if (skip2 < 0) skip2 = getenv("MI_UNET_SKIP2") ? atoi(getenv("MI_UNET_SKIP2")) : 1;
            if (u->act_dt == 8 && (u->prec != 3 || skip2) && w[i] % 32 == 0 && i >= u->slab_nl) {
                u->skipst[i] = act_new(u, u->enc[i].ys);
                if (u->prec == 3) { const size_t b4 = nn_mx4_bytes(u->enc[i].ys); u->skipst4[i] = mi_malloc(b4); mi_zero(u->skipst4[i], b4); nn_set_storage(u->skipst4[i], b4, 4); }
            }
            if (cfg->down_norm) { const size_t ng = (size_t)in.n * G_of(u, w[i]); u->dm[i] = f32_new(ng); u->dr[i] = f32_new(ng); }
        }
    }
    for (int i = 0; i < u->slab_nl; i++) {
        shape5 t = u->ls[i]; if (u->slab_s < t.d) t.d = u->slab_s;
        u->slab_tmp[i] = act_new(u, t); t.d = 1; u->slab_carry[i] = act_new(u, t);
    }
    u->xin = act_new(u, in);
    u->logits = f32_new((size_t)in.n * cfg->cout * in.d * in.h * in.w);
    if (u->tbn) {
        const shape5 ys = u->ls[L - 1]; const long Sg = (long)ys.d * ys.h * ys.w, S = Sg + u->tbd.nreg, T = (long)ys.n * S; const int C = u->tbd.C;
        u->tbg = (at_geom){.nseq = ys.n, .S = (int)S, .D = ys.d, .Hh = ys.h, .W = ys.w};
        u->tb.ys = ys; u->tb.a2 = act_new(u, ys);
        const size_t ng = (size_t)in.n * G_of(u, C);
        u->tb.m2 = f32_new(ng); u->tb.r2 = f32_new(ng);
        if (u->cfg.attn_vres) u->tb_vr = f32_new((size_t)T * C);
        u->tb_cs = f32_new((size_t)ys.n * C * Sg); u->tb_tok = f32_new((size_t)3 * T * C);     /* the stage's input rows and two buffers the applications alternate between */
        long Tr = 0;
        if (cfg_axis(&u->cfg)) {                                  /* the scroll geometry's buffers; tb_geom fills them per forward (src/unet.c:1354-1375) */
            at_rays_dims(ys.d, ys.h, ys.w, attn_ray_mult(), &u->tb_Q, &u->tb_Nt, &u->tb_Nr);
            const int Pm = ys.d > ys.h ? (ys.d > ys.w ? ys.d : ys.w) : (ys.h > ys.w ? ys.h : ys.w);
            Tr = u->cfg.attn_axis == 1 ? (long)ys.n * u->tb_Q * u->tb_Nr : 0;
            const size_t nq = (size_t)ys.n * u->tb_Q, al = 64;
#define UP(v) (((size_t)(v) + al - 1) / al * al)
            const size_t o_ray = 0, o_len = o_ray + UP(nq * AT_RAY_F), o_ad = o_len + UP(nq), o_pos = o_ad + UP(ys.n), o_ws = o_pos + UP((size_t)Tr * 3),
                         o_gp = o_ws + UP((size_t)ys.n * Sg), o_cen = o_gp + UP((size_t)T * 3), o_end = o_cen + UP((size_t)ys.n * Pm * 4);
#undef UP
            u->tb_rb = f32_new(o_end);
            u->tbr = (at_rays){.n = ys.n, .Q = u->tb_Q, .Nt = u->tb_Nt, .Nr = u->tb_Nr, .D = ys.d, .Hh = ys.h, .W = ys.w, .ad = (const int *)(u->tb_rb + o_ad), .ray = u->tb_rb + o_ray,
                               .lens = (const int *)(u->tb_rb + o_len), .pos = u->tb_rb + o_pos, .wsum = u->tb_rb + o_ws};
            u->tb_gpos = u->tb_rb + o_gp; u->tb_cen = u->tb_rb + o_cen;
            for (int k = 0; k < 2; k++) { u->tb_pin[k] = mi_host_alloc((nq * AT_RAY_F + nq + (size_t)ys.n + (size_t)ys.n * Pm * 4) * 4); u->tb_fence[k] = mi_fence_new(); mi_fence_set(u->tb_fence[k]); }
            u->tb_set = 0;
            u->tb_axb = malloc((size_t)ys.n * AT_AXR(Pm) * sizeof(float));
            if (!u->tb_axb) { fprintf(stderr, "unet: no host memory for the ray plan\n"); abort(); }
            u->tb_axdirty = 1;
            if (u->cfg.attn_axis == 1) u->tbg.rays = &u->tbr; else u->tbg.pos = u->tb_gpos;
        }
        u->tb_ws = mi_malloc(at_ws_bytes_r(&u->tbd, T, Tr)); at_ws_carve_r(&u->tbw, &u->tbd, T, Tr, u->tb_ws);
    }
    u->built = 1;
    return 0;
}
static int ensure_built(unet *u, shape5 xs) {
    const int ip = slab_inplace_now(u);
    if (u->built && !memcmp(&u->in, &xs, sizeof xs) && u->act_dt == act_dt_now() && u->prec == nn_get_prec() && u->slab_ip == ip && (!ip || u->slab_s == g_infer_slab)) return 0;
    return build_acts(u, xs);
}
void unet_free(unet *u) {
    if (!u) return;
    mi_sync();
    free_acts(u);
    mi_free(u->p); mi_free(u->ema); if (u->wm) mi_free(u->wm); if (u->l0run) mi_free(u->l0run); if (u->ge_run) mi_free(u->ge_run);
    for (int i = 0; i < UNET_MAXLEV; i++) { free(u->rb[i]); free(u->rbn[i]); }
    if (u->stem_b) mi_free(u->stem_b);
    free(u->tb_axh);
    if (u->gf_g) { mi_free(u->gf_g); mi_free(u->gf_g1); }
    lp_wmemo_clear();
    free(u);
}
size_t unet_nparams(const unet *u) { return u->np; }
const unet_cfg *unet_cfg_of(const unet *u) { return &u->cfg; }
float *unet_param_ptr(unet *u) { return u->p; }
float *unet_ema_ptr(unet *u) { return u->ema; }
void unet_use_ema(unet *u, int on) {      /* (the prepared weights are keyed by pointer; dropped all the same) */
    float *w = on ? u->ema : u->p;
    if (w == u->src) return;
    u->src = w;
    if (u->wm) u->wm_ok = 0; else u->params = w;
    lp_wmemo_clear();
}
/* cfg.w4_2d (src/unet.h:47-51, src/unet.c:5292-5326): the forward reads a copy of the selected weights in which the stride-1 3^3 convs' weights
   (not the network input conv, not the down convs) are rounded to MX-fp4 values with one scale per 32 x 32 (output x input channel) block and tap.
   The reference forms the copy before every forward; here it is formed when the weights were replaced through this interface (set / load /
   EMA switch). A caller that writes through unet_param_ptr calls mi_unet_weights_changed. */
void mi_unet_weights_changed(unet *u) { u->wm_ok = 0; lp_wmemo_clear(); }
static void film_one(unet *u, int j) {                             /* norm j's effective affine of the current codes, from the selected weights into the copy */
    size_t fo = u->film_off;
    for (int k = 0; k < j; k++) fo += (size_t)2 * u->cfg.film * film_norm(u, k)->c;
    const gnpar *n = film_norm(u, j);
    nn_film_fwd(u->src, u->wm, n->gamma, n->beta, fo, n->c, u->cfg.film, u->film_c);
}
static void fw_refresh(unet *u) {
    if (!u->wm) return;
    if (u->wm_ok) {                                                /* the copy is current but for the codes' affines (src/unet.c:374-380) */
        if (u->cfg.film && !u->film_ok) { for (int j = 0; j < 2 * u->cfg.nlev - 1; j++) film_one(u, j); u->film_ok = 1; }
        return;
    }
    mi_d2d(u->wm, u->src, u->np * 4);
    const int L = u->cfg.nlev;
    if (u->cfg.l0_norm == 3) {         /* ws: the four level-0 3^3 convs standardised per output channel over its fan-in; the network input conv without the SiLU gain (src/unet.c:5298-5304, :5311-5318) */
        const convp *wc[4] = {&u->enc[0].c1, &u->enc[0].c2, &u->dec[0].c1, &u->dec[0].c2};
        for (int i = 0; i < (L > 1 ? (u->dec[0].single ? 3 : 4) : 2); i++) nn_ws_fwd(u->wm + wc[i]->w, u->src + wc[i]->w, wc[i]->cout, wc[i]->cin * 27, i ? u->ws_gain : 1.f, 1e-5f);
    }
    if (u->cfg.w4_2d) {
        const convp *cs[4 * UNET_MAXLEV]; int n = 0;
        for (int i = 0; i < L; i++) { if (i) cs[n++] = &u->enc[i].c1; cs[n++] = &u->enc[i].c2; }
        for (int i = 0; i < L - 1; i++) { cs[n++] = &u->dec[i].c1; if (!u->dec[i].single) cs[n++] = &u->dec[i].c2; }
        for (int i = 0; i < n; i++) nn_fakeq_w4_2d(u->wm + cs[i]->w, cs[i]->cout, cs[i]->cin, 27, 32);
        n = 0;
        for (int i = 0; i < L; i++) for (int k = 0; k < u->cfg.enc_blocks[i]; k++) { if (n + 2 > 4 * UNET_MAXLEV) { for (int j = 0; j < n; j++) nn_fakeq_w4_2d(u->wm + cs[j]->w, cs[j]->cout, cs[j]->cin, 27, 32); n = 0; } cs[n++] = &u->rb[i][k].c1; cs[n++] = &u->rb[i][k].c2; }      /* (src/unet.c:5338) */
        for (int i = 0; i < n; i++) nn_fakeq_w4_2d(u->wm + cs[i]->w, cs[i]->cout, cs[i]->cin, 27, 32);
    }
    if (u->cfg.film) { for (int j = 0; j < 2 * L - 1; j++) film_one(u, j); u->film_ok = 1; }
    lp_wmemo_clear();
    u->wm_ok = 1;
}
/* cfg.gfilm, after the attention stage (its output in tb_cs, fp32 [C][S], one window): the pooled tokens are the codes of the decoder blocks'
   output norms, applied to the affines the copy would hold without them: the selected weights' or cfg.film's (src/unet.c:386-398) */
static int gfilm_fwd(unet *u, long S) {
    if (u->tb.ys.n != 1) { fprintf(stderr, "unet: gfilm takes one window per forward (src/unet.c:390)\n"); return -1; }
    const int L = u->cfg.nlev, K = u->gf_K;
    nn_gfilm_pool(u->tb_cs, K, S, u->gf_g);
    size_t fo = u->gf_off; int co = 0;
    for (int i = L - 2; i >= 0; i--) {
        const gnpar *n = &u->dec[i].n2;
        if (u->cfg.film) film_one(u, L + (L - 2 - i));
        else { mi_d2d(u->wm + n->gamma, u->src + n->gamma, (size_t)n->c * 4); mi_d2d(u->wm + n->beta, u->src + n->beta, (size_t)n->c * 4); }
        nn_gfilm_fwd(u->src, u->wm, n->gamma, n->beta, fo, n->c, K, u->gf_g, u->gf_g1 + co);
        fo += (size_t)2 * K * n->c; co += n->c;
    }
    return 0;
}
void mi_unet_get_params(const unet *u, float *host) { mi_sync(); mi_d2h(host, u->p, u->np * 4); }
void mi_unet_set_params(unet *u, const float *host) { mi_h2d(u->p, host, u->np * 4); mi_h2d(u->ema, host, u->np * 4); u->wm_ok = 0; lp_wmemo_clear(); }
shape5 unet_out_shape(const unet *u, shape5 xs) { return (shape5){xs.n, u->cfg.cout, xs.d, xs.h, xs.w}; }

/* ---- initial weights ----
   Same seed, same network as the reference's unet_init, bit for bit (src/unet.c:584-644): a caller that trains or tests from unet_init(u, seed)
   starts from identical weights in either program, which is what lets logits, checkpoints and regression baselines be compared across the two.
   That fixes the generator (splitmix64, 53-bit uniforms, one Box-Muller cosine branch per pair of uniforms) and the order in which the
   parameter vector consumes it; the rest is this file's: the network is first described as a list of runs (a span of the parameter vector,
   how it is filled), then one loop fills the spans in list order. tests/test_gpu_unet.py::test_unet_init_matches_the_published_generator
   checks the weights against an independent statement of the generator. */
typedef struct { size_t off, n; double sd; float fill; int drop; } init_run;      /* sd > 0: N(0, sd^2) draws (drop: drawn, then stored as 0); else the constant */
typedef struct { init_run *r; int n, cap; } init_plan;
static void plan_add(init_plan *pl, size_t off, size_t n, double sd, float fill, int drop) {
    if (!n) return;
    if (pl->n == pl->cap) { pl->cap = pl->cap ? 2 * pl->cap : 128; pl->r = realloc(pl->r, (size_t)pl->cap * sizeof *pl->r); if (!pl->r) { fprintf(stderr, "unet_init: out of memory\n"); abort(); } }
    pl->r[pl->n++] = (init_run){off, n, sd, fill, drop};
}
static void plan_conv(init_plan *pl, const convp *c, float bias, int drop) {      /* Kaiming-normal weights, constant bias */
    const size_t fan = (size_t)c->cin * c->k * c->k * c->k;
    plan_add(pl, c->w, (size_t)c->cout * fan, sqrt(2.0 / (double)fan), 0.f, drop);
    plan_add(pl, c->b, (size_t)c->cout, 0.0, bias, 0);
}
static void plan_norm(init_plan *pl, const gnpar *g) { plan_add(pl, g->gamma, (size_t)g->c, 0.0, 1.f, 0); }      /* (beta: the vector starts zeroed) */
static uint64_t mix64(uint64_t *state) {                               /* splitmix64 */
    uint64_t z = (*state += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}
static double draw_normal(uint64_t *state) {
    const double u1 = (double)(mix64(state) >> 11) * 0x1.0p-53 + 1e-300, u2 = (double)(mix64(state) >> 11) * 0x1.0p-53;
    return sqrt(-2 * log(u1)) * cos(6.283185307179586 * u2);
}
void unet_init(unet *u, uint64_t seed) {
    init_plan pl = {nullptr, 0, 0};
    const int L = u->cfg.nlev;
    for (int i = 0; i < L; i++) { const block *b = &u->enc[i]; plan_conv(&pl, &b->c1, 0.f, 0); plan_norm(&pl, &b->n1); plan_conv(&pl, &b->c2, 0.f, 0); plan_norm(&pl, &b->n2); }
    for (int i = 0; i + 1 < L; i++) plan_conv(&pl, &u->down[i], 0.f, 0);
    for (int i = 0; i + 1 < L; i++) {
        const block *b = &u->dec[i];
        plan_conv(&pl, &b->c1, 0.f, 0); plan_norm(&pl, &b->n1);
        if (!b->single) { plan_conv(&pl, &b->c2, 0.f, 0); plan_norm(&pl, &b->n2); }
    }
    plan_conv(&pl, &u->head, -2.f, 0);
    const char *rbnz = getenv("UFSM_RB_NONZERO");
    const int rb_keep = rbnz && atoi(rbnz);
    for (int i = 0; i < L; i++) for (int k = 0; k < u->cfg.enc_blocks[i]; k++) {      /* residual blocks start as the identity: conv2's weights drawn, then zero (src/unet.c:606-610) */
        const block *b = &u->rb[i][k];
        plan_conv(&pl, &b->c1, 0.f, 0); plan_norm(&pl, &b->n1); plan_conv(&pl, &b->c2, 0.f, !rb_keep); plan_norm(&pl, &b->n2);
    }
    for (int j = 1; j <= u->cfg.ds_levels; j++) plan_conv(&pl, &u->ds[j], -2.f, 0);                     /* as the main head (src/unet.c:611-612) */
    if (u->cfg.emb_lev) plan_conv(&pl, &u->eh, 0.f, 0);
    if (u->cfg.down_norm) for (int i = 0; i + 1 < L; i++) plan_norm(&pl, &u->dn[i]);
    if (u->tbn) {   /* LayerNorm and QK-norm gains 1, QKV and MLP-in N(0, 1 / C), out projections and biases 0 (identity blocks), registers N(0, 0.02^2) (src/unet.c:612-642) */
        const size_t C = (size_t)u->tbd.C, F = (size_t)u->tbd.F; const double sd = 1.0 / sqrt((double)C);
        for (int k = 0; k < u->tbn; k++) {
            const at_bp *bp = &u->tbp[k];
            plan_add(&pl, bp->ln1g, C, 0.0, 1.f, 0); plan_add(&pl, bp->ln2g, C, 0.0, 1.f, 0); plan_add(&pl, bp->qg, C, 0.0, 1.f, 0); plan_add(&pl, bp->kg, C, 0.0, 1.f, 0);
            plan_add(&pl, bp->wqkv, 3 * C * C, sd, 0.f, 0);
            plan_add(&pl, bp->w1, 2 * F * C, sd, 0.f, 0);
        }
        plan_add(&pl, u->reg_off, (size_t)u->tbd.nreg * C, 0.02, 0.f, 0);
        if (u->cfg.attn_vres && u->tbn > 1) plan_add(&pl, u->vr_off + (size_t)u->tbd.H, (size_t)(u->tbn - 1) * u->tbd.H, 0.0, 0.5f, 0);      /* every application after the first (src/unet.c:644) */
    }
    float *h = calloc(u->np, 4);
    if (!h) { fprintf(stderr, "unet_init: out of memory\n"); abort(); }
    for (int r = 0; r < pl.n; r++) {
        const init_run *ir = &pl.r[r];
        float *dst = h + ir->off;
        if (ir->sd > 0) for (size_t i = 0; i < ir->n; i++) { const float v = (float)(ir->sd * draw_normal(&seed)); dst[i] = ir->drop ? 0.f : v; }
        else for (size_t i = 0; i < ir->n; i++) dst[i] = ir->fill;
    }
    free(pl.r);
    mi_unet_set_params(u, h);
    free(h);
}

#define P(u, off) ((u)->params + (off))
static void note(unet *u, const void *p, shape5 s, const char *name, const float *mean, const float *rstd, int G) {
    if (u->nouts < 64) { u->outs[u->nouts].p = p; u->outs[u->nouts].s = s; u->outs[u->nouts].name = name; u->outs[u->nouts].mean = mean; u->outs[u->nouts].rstd = rstd; u->outs[u->nouts].G = G; u->nouts++; }
}
/* the block whose output is level i's encoder output (skip, down-conv input, bottom): the last residual block, else enc[i] (src/unet.c:302-303) */
static block *stage_out(unet *u, int i) { return u->cfg.enc_blocks[i] > 0 ? &u->rb[i][u->cfg.enc_blocks[i] - 1] : &u->enc[i]; }
static nn_gn_t gn_out(const unet *u, const block *b) { return (nn_gn_t){P(u, b->n2.gamma), P(u, b->n2.beta), b->m2, b->r2, G_of(u, b->ys.c)}; }   /* silu(gn(a2)) for the block's readers */

/* planes [s0, s0 + n) of the MX tensor src (depth Ds) -> planes [d0, d0 + n) of dst (depth Dd), every sample and channel block: a block's
   element rows and its scales are each contiguous over a range of planes (mx_copy_planes, src/unet.c:2410-2422) */
static void copy_planes(const unet *u, void *dst, int Dd, int d0, const void *src, int Ds, int s0, int n, shape5 s) {
    if (n <= 0) return;
    const int bw = s.c <= 8 ? 8 : s.c <= 16 ? 16 : 32, nb = (s.c + bw - 1) / bw, rb = u->act_dt == 4 ? bw / 2 : bw;
    const size_t hw = (size_t)s.h * s.w, Sd = (size_t)Dd * hw, Ss = (size_t)Ds * hw, rows = (size_t)s.n * nb;
    mi_d2d_rows((char *)dst + (size_t)d0 * hw * rb, Sd * rb, (const char *)src + (size_t)s0 * hw * rb, Ss * rb, (size_t)n * hw * rb, rows);
    mi_d2d_rows((char *)dst + rows * Sd * rb + (size_t)d0 * hw, Sd, (const char *)src + rows * Ss * rb + (size_t)s0 * hw, Ss, (size_t)n * hw, rows);
}
/* cfg.l0_norm 1 / 3 always, 2 once the running statistics' warm-up is over (src/unet.c:2315): the level-0 GroupNorms read constant statistics,
   written at the start of every forward (src/unet.c:2318-2323) */
static int l0_const(const unet *u) { const int md = u->cfg.l0_norm; return md == 1 || md == 3 || (md == 2 && u->l0_n > 0 && u->l0_n >= u->l0_warm); }
/* cfg.gn_ema at inference (ge_begin, src/unet.c:2229-2250): once the running statistics have seen an update, every site reads them (unless
   unet_gn_ema_live asks for the window's own); no conv or statistics pass reduces anything */
static int ge_const(const unet *u) { return u->cfg.gn_ema && u->ge_n > 0 && !u->ge_live; }
void unet_gn_ema_live(unet *u, int on) { u->ge_live = on != 0; }
static void ge_const_fill(unet *u) {
    float *m[192], *r[192]; int g[192]; size_t off[192];
    ge_sites(u, m, r, g, off);
    size_t o = 0; int n = 0;
    while (o < u->ge_ns) { o = off[n] + 2 * (size_t)g[n]; n++; }
    const float *run = u->ge_run + (u->src == u->ema ? u->ge_ns : 0);                       /* (the EMA weights have their own) */
    for (int k = 0; k < n; k++) nn_gn_const_fill(m[k], r[k], run + off[k], u->in.n, g[k], 1e-5f);
}
static void l0_const_fill(unet *u) {
    const int G = G_of(u, u->cfg.widths[0]), N = u->in.n;
    for (int i = 0; i < (u->cfg.nlev > 1 ? 2 : 1); i++) for (int k = 1; k <= 2; k++) {
        block *b = i ? &u->dec[0] : &u->enc[0];
        if (k == 1 && b->single) continue;                         /* (src/unet.c:2320) */
        const float *run = u->cfg.l0_norm == 2 ? u->l0run + (u->src == u->ema ? (size_t)8 * G : 0) + (size_t)(2 * i + k - 1) * 2 * G : nullptr;      /* (the EMA weights have their own) */
        nn_gn_const_fill(k == 1 ? b->m1 : b->m2, k == 1 ? b->r1 : b->r2, run, N, G, 1e-5f);
    }
}
/* conv1 -> a1 (+ its statistics), conv2 reads silu(gn(a1)) while staging -> a2 (+ statistics) (src/unet.c:2567-2636); in z-slabs when asked for
   (slab_run, src/unet.c:2499-2545) */
static int block_fwd(unet *u, block *b, int level, const void *x, const nn_gn_t *gin, const void *xup, const nn_gn_t *gup, int c_split, const char *n1, const char *n2) {
    const int G = G_of(u, b->c1.cout), D = b->ys.d, ip = u->slab_ip && level < u->slab_nl;
    /* per-slab statistics (level 0 under cfg.l0_norm 4): the convs reduce nothing; a pass over the stored output, seen as n * slabs samples of
       l0_slab planes (one channel block: a slab is a sample of the same layout), fills the [n][slab][G] rows (src/unet.c:996-998) */
    const int l0s = level == 0 && u->l0s_ns, Gc = l0s || (level == 0 && l0_const(u)) || ge_const(u) ? 0 : G;       /* (constant statistics: nothing to reduce either) */
    const int s = level >= slab_levels(u) ? 0 : g_infer_slab < D ? g_infer_slab : ip ? D : 0;      /* (in place: a level of fewer planes is one slab) */
    void *tmp = ip ? u->slab_tmp[level] : nullptr, *carry = ip ? u->slab_carry[level] : nullptr;
    int r = 0;
    for (int conv = b->single ? 2 : 1; conv <= 2 && !r; conv++) {  /* (one-conv decoder block: its conv, with c1's weights, writes a2 and the statistics m2 / r2, src/unet.c:2581-2582) */
        void *y = conv == 1 ? b->a1 : b->a2;
        const int first = conv == 1 || b->single;                  /* this conv reads the block's input */
        const int over = ip && (!first || x == y);                 /* the conv reads the buffer it writes: through the temp */
        float *om = conv == 1 ? b->m1 : b->m2, *orr = conv == 1 ? b->r1 : b->r2;
        for (int z0 = 0, k = 0, sk; z0 < D && !r; z0 += sk, k++) {
            sk = s && D - z0 > s ? s : D - z0;
            const int last = z0 + sk >= D;
            shape5 xs = first ? b->xs : b->ys;
            if (s) { nn_set_zrange(z0, D, z0 == 0, last, D, z0); nn_set_zrange_out(!over); xs.d = sk; }
            void *o = over ? tmp : y;
            if (!first) r = nn_conv3d_fwd_gn_stats(b->a1, xs, G, P(u, b->n1.gamma), P(u, b->n1.beta), b->m1, b->r1, P(u, b->c2.w), P(u, b->c2.b), b->c2.cout, o, Gc, 1e-5f, om, orr);
            else if (xup) r = nn_conv3d_fwd_x(xup, gup, x, gin, c_split, 1, xs, P(u, b->c1.w), P(u, b->c1.b), b->c1.cout, 3, 1, o, Gc, 1e-5f, om, orr);   /* [up2(coarse) | skip] */
            else r = nn_conv3d_fwd_x(x, gin, nullptr, nullptr, 0, 0, xs, P(u, b->c1.w), b == &u->enc[0] && u->cfg.scale_cond ? u->stem_b : P(u, b->c1.b), b->c1.cout, 3, 1, o, Gc, 1e-5f, om, orr);
            if (s) { nn_set_zrange(0, 0, 0, 0, 0, 0); nn_set_zrange_out(0); }
            if (over && !r) {                                      /* planes below the next slab's first input plane are dead: the last one waits */
                if (k) copy_planes(u, y, D, z0 - 1, carry, 1, 0, 1, b->ys);
                copy_planes(u, y, D, z0, tmp, sk, 0, last ? sk : sk - 1, b->ys);
                if (!last) copy_planes(u, carry, 1, 0, tmp, sk, sk - 1, 1, b->ys);
            }
        }
        if (!r && l0s) {
            shape5 ps = b->ys; ps.n *= u->l0s_ns; ps.d = u->l0s_zs;
            if (nn_gn_stats(y, ps, G, 1e-5f, om, orr)) { fprintf(stderr, "unet: per-slab GroupNorm statistics unsupported for this storage\n"); r = -1; }
        }
        if (!r) note(u, y, b->ys, first ? n1 : n2, om, orr, G);    /* (a one-conv block's output goes by its conv's name) */
    }
    return r;
}
/* replaces unet_set_attn_axis (src/unet.h:470-474, src/unet.c:2732-2737): the scroll axis of every sample of the following forwards, n records of
   stride floats (UNET_AXR, host memory, copied); n 0 or a null pointer: no axis (rays along the grid rows, grid-index coordinates) */
void unet_set_attn_axis(unet *u, const float *rec, int n, int stride) {
    if (n <= 0 || stride < 4 || !rec) { u->tb_axn = 0; u->tb_axdirty = 1; return; }
    if ((size_t)n * stride > (size_t)u->tb_axn * u->tb_axs || !u->tb_axh) {
        free(u->tb_axh); u->tb_axh = malloc((size_t)n * stride * sizeof(float));
        if (!u->tb_axh) { fprintf(stderr, "unet: no memory for axis records\n"); abort(); }
    }
    memcpy(u->tb_axh, rec, (size_t)n * stride * sizeof(float));
    u->tb_axn = n; u->tb_axs = stride; u->tb_axdirty = 1;
}
/* the scroll geometry of this forward from the axis records (tb_geom, src/unet.c:2738-2782): each sample's window axis centres averaged over the
   window planes of a bottleneck plane and expressed in bottleneck voxels, then the ray plan, its device tables and the ray positions and
   stencil weight sums (radial attention) or the grid tokens' scroll coordinates (full attention). A record that does not describe this grid
   (another plane count) or says "no axis" leaves its sample without one */
static void tb_geom(unet *u) {
    if (!u->tb_rb || !u->tb_axdirty) return;
    const shape5 ys = u->tb.ys; const int n = ys.n, D = ys.d, Hh = ys.h, W = ys.w, Pm = D > Hh ? (D > W ? D : W) : (Hh > W ? Hh : W);
    const int fp = 1 << (u->cfg.nlev - 1), have = u->tb_axh && u->tb_axn == n;
    u->tb_noax = 0;
    if (!have && !u->tb_axwarn) { fprintf(stderr, "unet: the attention stage has no scroll axis records for %d samples (unet_set_attn_axis): rays along the grid rows\n", n); u->tb_axwarn = 1; }
    for (int b = 0; b < n; b++) {
        float *o = u->tb_axb + (size_t)b * AT_AXR(Pm);
        memset(o, 0, AT_AXR(Pm) * sizeof *o);
        if (!have) continue;
        const float *r = u->tb_axh + (size_t)b * u->tb_axs;
        const int ad = (int)r[0], np = (int)r[2], div = (int)r[3] > 0 ? (int)r[3] : 1, F = div * fp;
        if (ad < 0 || ad > 2) continue;
        const int Np = ad == 0 ? D : ad == 1 ? Hh : W;
        o[0] = (float)ad;
        if (r[1] == 0.f || np != Np * F || u->tb_axs < UNET_AXR(np)) { u->tb_noax++; continue; }
        o[1] = 1.f;
        for (int k = 0; k < Np; k++) {
            double su = 0, sv = 0;
            for (int z = k * F; z < (k + 1) * F; z++) { su += r[4 + 2 * z]; sv += r[5 + 2 * z]; }
            o[2 + 2 * k] = (float)((su / F + 0.5) / F - 0.5); o[3 + 2 * k] = (float)((sv / F + 0.5) / F - 0.5);      /* voxel centres at integers on both grids */
        }
    }
    /* the tables go to the device in stream order from pinned memory: the host does not wait for the forwards still queued (a synchronous copy
       would, and the device would then idle while the next forward is enqueued); a set is rewritten only once its own copy has run */
    const size_t nq = (size_t)n * u->tb_Q; const int set = u->tb_set; u->tb_set ^= 1;
    mi_fence_wait(u->tb_fence[set]);
    u->tb_rayh = u->tb_pin[set]; u->tb_lensh = (int *)(u->tb_rayh + nq * AT_RAY_F); u->tb_adh = u->tb_lensh + nq; u->tb_cenh = (float *)(u->tb_adh + n);
    at_rays_plan(n, D, Hh, W, attn_ray_mult(), u->tb_axb, u->tb_rayh, u->tb_lensh, u->tb_adh, u->tb_cenh);
    mi_h2d_async((void *)u->tbr.ray, u->tb_rayh, nq * AT_RAY_F * sizeof(float));
    mi_h2d_async((void *)u->tbr.lens, u->tb_lensh, nq * sizeof(int));
    mi_h2d_async((void *)u->tbr.ad, u->tb_adh, (size_t)n * sizeof(int));
    mi_h2d_async(u->tb_cen, u->tb_cenh, (size_t)n * Pm * 4 * sizeof(float));
    mi_fence_set(u->tb_fence[set]);
    if (u->cfg.attn_axis == 1) at_rays_setup(&u->tbr);
    else at_scroll_pos(n, u->tbd.nreg, D, Hh, W, u->tbr.ad, u->tb_cen, u->tb_gpos);
    u->tb_axdirty = 0;
}
/* replaces unet_attn_rays (src/unet.c:2783-2796): the ray set's sizes and, when asked, the share of grid tokens a ray sample touches; -1 without
   radial attention or before the first forward built the graph */
int unet_attn_rays(const unet *u, int *Q, int *Nr, double *coverage) {
    if (!u->tb_rb || u->cfg.attn_axis != 1) return -1;
    if (Q) *Q = u->tb_Q;
    if (Nr) *Nr = u->tb_Nr;
    if (coverage) {
        const size_t ng = (size_t)u->tbr.n * u->tbr.D * u->tbr.Hh * u->tbr.W; float *w = malloc(ng * sizeof *w); size_t c = 0;
        if (!w) return -1;
        mi_sync(); mi_d2h(w, u->tbr.wsum, ng * sizeof *w);
        for (size_t i = 0; i < ng; i++) c += w[i] > 0.f;
        *coverage = (double)c / (double)ng; free(w);
    }
    return 0;
}
/* the bottleneck's raw output -> fp32 planes -> token rows with the registers prepended -> blocks -> planes -> a new MX tensor with its
   GroupNorm statistics: the level's output for the decoder (src/unet.c:2795-2835; no PEG, memory, view or deformable paths) */
static int tb_fwd(unet *u) {
    const block *x = stage_out(u, u->cfg.nlev - 1); block *b = &u->tb;
    const shape5 ys = b->ys; const int C = u->tbd.C, nr = u->tbd.nreg; const size_t Sg = (size_t)ys.d * ys.h * ys.w, TC = (size_t)u->tbg.nseq * u->tbg.S * C;
    if (u->act_dt == 4) lp_mx4_to_f32(x->a2, ys.n, C, Sg, u->tb_cs); else lp_mx8_to_f32(x->a2, ys.n, C, Sg, u->tb_cs);
    at_cs_to_tok(u->tb_cs, u->tb_tok, P(u, u->reg_off), ys.n, C, (long)Sg, nr);
    tb_geom(u);
    at_set_mx(8);
    lp_mx_gemm_bmemo(1);                                           /* inference: the linears' weights are packed once (dropped when the weights change) */
    const int tba = u->tbn * (u->cfg.attn_repeat > 1 ? u->cfg.attn_repeat : 1);      /* application k runs block k % tbn (cfg.attn_repeat, src/unet.c:2816) */
    float *tin = u->tb_tok;
    if (u->cfg.attn_pe == 0) { at_peg_fwd(tin, u->tb_tok + 2 * TC, P(u, u->peg_w), P(u, u->peg_b), &u->tbg, nr, C); tin = u->tb_tok + 2 * TC; }      /* (src/unet.c:2805; the first block writes the other buffer) */
    for (int k = 0; k < tba; k++) {
        float *tout = u->tb_tok + (size_t)(1 + (k & 1)) * TC;
        if (u->tb_vr) { u->tbw.vr = k ? 2 : 1; u->tbw.v1 = u->tb_vr; u->tbw.own = nullptr; u->tbw.lam = P(u, u->vr_off + (size_t)(k % u->tbn) * (size_t)u->tbd.H); }      /* (tb_vr_set, src/unet.c:2699-2704) */
        if (at_block_fwd(&u->tbd, u->params, &u->tbp[k % u->tbn], tin, tout, &u->tbg, &u->tbw)) { lp_mx_gemm_bmemo(0); fprintf(stderr, "unet: attention block forward failed\n"); return -1; }
        tin = tout;
    }
    lp_mx_gemm_bmemo(0);
    at_tok_to_cs(tin, u->tb_cs, ys.n, C, (long)Sg, nr);
    if (u->cfg.gfilm && gfilm_fwd(u, (long)Sg)) return -1;        /* (src/unet.c:2827) */
    if (u->act_dt == 4) lp_f32_to_mx4(u->tb_cs, ys.n, C, Sg, b->a2); else lp_f32_to_mx8(u->tb_cs, ys.n, C, Sg, b->a2);
    const int G = G_of(u, C);
    if (!ge_const(u) && nn_gn_stats(b->a2, ys, G, 1e-5f, b->m2, b->r2)) { fprintf(stderr, "unet: attention stage GroupNorm statistics unsupported for this storage\n"); return -1; }
    note(u, b->a2, ys, "attn", b->m2, b->r2, G);
    return 0;
}
/* a residual block (rblock_fwd, src/unet.c:2656-2671): conv1 of silu(gn(prev's output)) with statistics, conv2 of silu(gn(a1)) without, the
   previous output added into it (MX: decode, add, re-quantise), then the statistics of the stored sum */
static int rblock_fwd(unet *u, block *b, block *prev, const char (*nm)[16]) {
    const int G = G_of(u, b->c1.cout), Gc = ge_const(u) ? 0 : G;
    const nn_gn_t gi = gn_out(u, prev);
    if (nn_conv3d_fwd_gn_stats(prev->a2, b->xs, gi.G, gi.gamma, gi.beta, gi.mean, gi.rstd, P(u, b->c1.w), P(u, b->c1.b), b->c1.cout, b->a1, Gc, 1e-5f, b->m1, b->r1)) return -1;
    note(u, b->a1, b->ys, nm[0], b->m1, b->r1, G);
    if (nn_conv3d_fwd_gn_stats(b->a1, b->ys, G, P(u, b->n1.gamma), P(u, b->n1.beta), b->m1, b->r1, P(u, b->c2.w), P(u, b->c2.b), b->c2.cout, b->a2, 0, 1e-5f, nullptr, nullptr)) return -1;
    lp_add_mx(b->a2, prev->a2, b->ys, u->act_dt, 0u);
    if (!ge_const(u) && nn_gn_stats(b->a2, b->ys, G, 1e-5f, b->m2, b->r2)) { fprintf(stderr, "unet: residual block GroupNorm statistics unsupported for this storage\n"); return -1; }
    note(u, b->a2, b->ys, nm[1], b->m2, b->r2, G);
    return 0;
}
/* the graph on the MX input tensor x (src/unet.c:2939-3105) */
static int graph_fwd(unet *u, const void *x) {
    static const char *en1[] = {"enc0.c1", "enc1.c1", "enc2.c1", "enc3.c1", "enc4.c1", "enc5.c1", "enc6.c1", "enc7.c1"}, *en2[] = {"enc0.c2", "enc1.c2", "enc2.c2", "enc3.c2", "enc4.c2", "enc5.c2", "enc6.c2", "enc7.c2"};
    static const char *dn1[] = {"dec0.c1", "dec1.c1", "dec2.c1", "dec3.c1", "dec4.c1", "dec5.c1", "dec6.c1"}, *dn2[] = {"dec0.c2", "dec1.c2", "dec2.c2", "dec3.c2", "dec4.c2", "dec5.c2", "dec6.c2"};
    static const char *dwn[] = {"down0", "down1", "down2", "down3", "down4", "down5", "down6"};
    const int L = u->cfg.nlev;
    u->nouts = 0;
    if (l0_const(u)) l0_const_fill(u);
    if (ge_const(u)) ge_const_fill(u);
    if (u->cfg.scale_cond) {                                       /* the stem bias of this forward: b + c v (src/unet.c:2880-2885) */
        const int c0 = u->enc[0].c1.cout;
        if (!u->stem_b) u->stem_b = f32_new((size_t)c0);
        mi_d2d(u->stem_b, P(u, u->enc[0].c1.b), (size_t)c0 * 4);
        nn_axpy(u->stem_b, u->sc_c, P(u, u->sc_w), (size_t)c0);
    }
    const void *cur = x;
    for (int i = 0; i < L; i++) {
        nn_gn_t gd; const nn_gn_t *gin = nullptr;                  /* down_norm: conv1 reads silu(gn(down conv output)) (src/unet.c:2593) */
        if (i && u->cfg.down_norm) { gd = (nn_gn_t){P(u, u->dn[i - 1].gamma), P(u, u->dn[i - 1].beta), u->dm[i - 1], u->dr[i - 1], G_of(u, u->cfg.widths[i - 1])}; gin = &gd; }
        if (block_fwd(u, &u->enc[i], i, cur, gin, nullptr, nullptr, 0, en1[i], en2[i])) return -1;
        for (int k = 0; k < u->cfg.enc_blocks[i]; k++) if (rblock_fwd(u, &u->rb[i][k], k ? &u->rb[i][k - 1] : &u->enc[i], u->rbn[i][k])) return -1;      /* (src/unet.c:2963) */
        if (i < L - 1) {                                           /* stride-2 down conv of silu(gn(a2)), width kept (src/unet.c:2970) */
            const block *so = stage_out(u, i);
            const nn_gn_t g = gn_out(u, so);
            const int pre = u->skipst[i] != nullptr;
            if (pre && (u->skipst4[i] ? mi_conv_prestage2(so->a2, so->ys, gnp_mk(g.gamma, g.beta, g.mean, g.rstd, g.G), u->skipst[i], u->skipst4[i])
                                      : mi_conv_prestage(so->a2, 3, so->ys, gnp_mk(g.gamma, g.beta, g.mean, g.rstd, g.G), u->skipst[i], 8))) return -1;
            if (nn_conv3d_fwd_x(pre ? u->skipst[i] : so->a2, pre ? nullptr : &g, nullptr, nullptr, 0, 0, so->ys, P(u, u->down[i].w), P(u, u->down[i].b), u->cfg.widths[i], 3, 2, u->downo[i], 0, 0.f, nullptr, nullptr)) return -1;
            shape5 ds = u->ls[i + 1]; ds.c = u->cfg.widths[i];
            if (u->cfg.down_norm) {                                /* statistics of the stored down-conv output now, the transform in the next conv1's staging (src/unet.c:2974-2979) */
                if (!ge_const(u) && nn_gn_stats(u->downo[i], ds, G_of(u, ds.c), 1e-5f, u->dm[i], u->dr[i])) { fprintf(stderr, "unet: down_norm GroupNorm statistics unsupported for this storage\n"); return -1; }
                note(u, u->downo[i], ds, dwn[i], u->dm[i], u->dr[i], G_of(u, ds.c));
            } else note(u, u->downo[i], ds, dwn[i], nullptr, nullptr, 0);
            cur = u->downo[i];
        }
    }
    if (u->tbn && tb_fwd(u)) return -1;
    for (int i = L - 2; i >= 0; i--) {                             /* decoder: nothing materialised (src/unet.c:3010-3013) */
        const block *coarse = i == L - 2 ? stage_out(u, L - 1) : &u->dec[i + 1], *skip = stage_out(u, i);
        nn_gn_t gc = gn_out(u, coarse); const nn_gn_t gs = gn_out(u, skip);
        if (i == L - 2 && u->tbn) { coarse = &u->tb; gc.mean = u->tb.m2; gc.rstd = u->tb.r2; }      /* the stage's output under the level's n2 affine (src/unet.c:508) */
        static const nn_gn_t none = {nullptr, nullptr, nullptr, nullptr, -1};          /* the pre-staged skip: no GroupNorm left to apply */
        const void *sk = u->skipst4[i] ? u->skipst4[i] : u->skipst[i];      /* (the decoder's conv computes in e2m1 under precision 3: its rows) */
        if (block_fwd(u, &u->dec[i], i, sk ? sk : skip->a2, sk ? &none : &gs, coarse->a2, &gc, coarse->ys.c, dn1[i], dn2[i])) return -1;
    }
    const block *last = L > 1 ? &u->dec[0] : &u->enc[0];
    const nn_gn_t g = gn_out(u, last);
    return nn_conv3d_fwd_x(last->a2, &g, nullptr, nullptr, 0, 0, last->ys, P(u, u->head.w), P(u, u->head.b), u->cfg.cout, 1, 1, u->logits, 0, 0.f, nullptr, nullptr);
}
/* every exit of a forward passes here: the caller's tensor leaves the storage registry again (a stale range would make a later allocation
   inside it look like MX storage) */
const float *mi_unet_forward_mx(unet *u, const void *xmx, shape5 xs) {
    if (ensure_built(u, xs)) return nullptr;
    fw_refresh(u);
    const int reg_here = xmx != u->xin && nn_storage(xmx) != u->act_dt;     /* the input is looked up by the convs like any activation */
    if (reg_here) nn_set_storage(xmx, act_bytes(u, u->in), u->act_dt);
    const int rc = graph_fwd(u, xmx);
    if (reg_here) nn_storage_forget(xmx);
    return rc ? nullptr : u->logits;
}
const float *unet_forward_x(unet *u, const void *x, shape5 xs, int train, int x_h16) {
    if (train) { fprintf(stderr, "unet_forward_x: this is an inference build (train must be 0)\n"); abort(); }
    if (ensure_built(u, xs)) return nullptr;
    const size_t S = (size_t)xs.d * xs.h * xs.w;
    /* the input conversion of src/unet.c:2909-2919: fp32 planes, or the 16-bit storage type read in place (fp16 here) -> the MX input tensor */
    if (x_h16) { if (u->act_dt == 4) lp_h16_to_mx4(x, 2, xs.n, xs.c, S, u->xin); else lp_h16_to_mx8(x, 2, xs.n, xs.c, S, u->xin); }
    else if (u->act_dt == 4) lp_f32_to_mx4(x, xs.n, xs.c, S, u->xin); else lp_f32_to_mx8(x, xs.n, xs.c, S, u->xin);
    return mi_unet_forward_mx(u, u->xin, xs);
}
const float *unet_forward(unet *u, const float *x, shape5 xs, int train) { return unet_forward_x(u, x, xs, train, 0); }
/* one forward over xs.n windows: window n's input rows go to sample n; logits [n][cout][voxels] */
const float *mi_unet_forward_ct_n(unet *u, const uint8_t *const *ct, float mean, float isd, const float *const *dyo, const float *const *dxo, int axis, shape5 xs, int h16) {
    if (xs.c != 4 || u->cfg.cin != 4 || xs.h != xs.w) { fprintf(stderr, "unet_forward_ct: needs square windows of 4 input channels\n"); return nullptr; }
    if (ensure_built(u, xs)) return nullptr;
    mi_pred_input_mx_batch(ct, xs.w, mean, isd, dyo, dxo, axis, 0, xs.d, u->xin, h16, u->act_dt == 4 ? 4 : 8, xs.n, 0, xs.n);
    return mi_unet_forward_mx(u, u->xin, xs);
}
const float *unet_forward_ct(unet *u, const uint8_t *ct, float mean, float isd, const float *dyo, const float *dxo, int axis, shape5 xs, int h16) {
    if (xs.n < 1 || xs.n > 64) { fprintf(stderr, "unet_forward_ct: %d windows per forward (1 .. 64)\n", xs.n); return nullptr; }
    const uint8_t *cts[64]; const float *dys[64], *dxs[64];
    const size_t w3 = (size_t)xs.d * xs.h * xs.w;
    for (int n = 0; n < xs.n; n++) { cts[n] = ct + (size_t)n * w3; dys[n] = dyo + (size_t)n * xs.d; dxs[n] = dxo + (size_t)n * xs.d; }
    return mi_unet_forward_ct_n(u, cts, mean, isd, dys, dxs, axis, xs, h16);
}
int mi_unet_layer_stats(const unet *u, int k, const float **mean, const float **rstd) {
    if (k < 0 || k >= u->nouts) return 0;
    *mean = u->outs[k].mean; *rstd = u->outs[k].rstd;
    return u->outs[k].G;
}
const void *mi_unet_layer_out(const unet *u, int k, shape5 *s, const char **name) {
    if (k < 0 || k >= u->nouts) return nullptr;
    if (s) *s = u->outs[k].s;
    if (name) *name = u->outs[k].name;
    return u->outs[k].p;
}


/* ---- checkpoints (the reference's file format: src/unet.c:5534-5650, :5650-5700, :5774-5800) ---- */
static char *header_line(FILE *f) {                                /* the first line without its newline (malloc'ed), the stream left after it */
    size_t cap = 1 << 16, n = 0; char *s = malloc(cap);
    for (int c; s && (c = fgetc(f)) != EOF;) {
        if (c == '\n') { s[n] = 0; return s; }
        if (n + 2 > cap) { if (cap >= (1u << 22)) break; cap *= 2; char *t = realloc(s, cap); if (!t) break; s = t; }
        s[n++] = (char)c;
    }
    free(s); return nullptr;
}
static int key_int(const char *line, const char *key, int dflt) { const char *p = strstr(line, key); return p ? atoi(p + strlen(key)) : dflt; }
/* the running level-0 statistics a checkpoint of cfg.l0_norm 2 carries (src/unet.c:5579-5584, :5737-5739): their state and 16 G values */
typedef struct { long n; int warm; float mom; int cnt; float run[1024]; long gn; int gwarm; float gmom; int gcnt; float grun[8192]; } l0_hdr;      /* (and cfg.gn_ema's: src/unet.c:5744-5751) */
static int read_header(const char *path, unet_cfg *cfg, size_t *nparams, int *step, l0_hdr *l0) {
    FILE *f = fopen(path, "rb");
    if (!f) return -1;
    char *line = header_line(f); fclose(f);
    if (!line || strncmp(line, "UFSM{", 5)) { free(line); return -1; }
    char *ex = strstr(line, ",\"extra\":"); if (ex) *ex = 0;       /* (the caller's object may repeat key names) */
    memset(cfg, 0, sizeof *cfg);
    cfg->nlev = key_int(line, "\"nlev\":", 0);
    const char *p = strstr(line, "\"widths\":[");
    if (cfg->nlev < 1 || cfg->nlev > UNET_MAXLEV || !p) { free(line); return -1; }
    p += 10;
    for (int i = 0; i < cfg->nlev; i++) { cfg->widths[i] = atoi(p); p = strchr(p, ','); if (!p) break; p++; }
    cfg->cin = key_int(line, "\"cin\":", 0); cfg->cout = key_int(line, "\"cout\":", 0); cfg->G = key_int(line, "\"G\":", 8);
    if ((p = strstr(line, "\"dec_widths\":["))) { p += 14; for (int i = 0; i < UNET_MAXLEV && *p && *p != ']'; i++) { char *e; cfg->dec_widths[i] = (int)strtol(p, &e, 10); p = e; if (*p == ',') p++; } }      /* (src/unet.c:5674) */
    if ((p = strstr(line, "\"enc_blocks\":["))) { p += 14; for (int i = 0; i < UNET_MAXLEV && *p && *p != ']'; i++) { char *e; cfg->enc_blocks[i] = (int)strtol(p, &e, 10); p = e; if (*p == ',') p++; } }      /* (src/unet.c:5675) */
    if ((p = strstr(line, "\"dec_convs\":["))) { p += 13; for (int i = 0; i < UNET_MAXLEV && *p && *p != ']'; i++) { char *e; cfg->dec_convs[i] = (int)strtol(p, &e, 10); p = e; if (*p == ',') p++; } }        /* (src/unet.c:5700) */
    cfg->down_norm = key_int(line, "\"down_norm\":", 0); cfg->w4_2d = key_int(line, "\"w4_2d\":", 0);
    cfg->l0_norm = key_int(line, "\"l0_norm\":", 0); cfg->l0_slab = key_int(line, "\"l0_slab\":", 0);      /* (src/unet.c:5726) */
    cfg->gn_ema = key_int(line, "\"gn_ema\":", 0);
    cfg->ds_levels = key_int(line, "\"ds_levels\":", 0); cfg->emb_lev = key_int(line, "\"emb_lev\":", 0); cfg->emb_ch = key_int(line, "\"emb_ch\":", 0);      /* (src/unet.c:5562-5563) */
    cfg->attn_blocks = key_int(line, "\"attn_blocks\":", 0); cfg->attn_pe = key_int(line, "\"attn_pe\":", 0);
    cfg->attn_reg = key_int(line, "\"attn_reg\":", 0); cfg->attn_mlp = key_int(line, "\"attn_mlp\":", 0);
    cfg->attn_repeat = key_int(line, "\"attn_repeat\":", 0); cfg->attn_vres = key_int(line, "\"attn_vres\":", 0);      /* (src/unet.c:5690) */
    cfg->attn_axis = key_int(line, "\"attn_axis\":", 0);                                                                  /* (src/unet.c:5691) */
    cfg->half_res = key_int(line, "\"half_res\":", 0); cfg->scan_norm = key_int(line, "\"scan_norm\":", 0);      /* (the caller's business: the graph does not use them) */
    if (nparams) { const char *q = strstr(line, "\"nparams\":"); *nparams = q ? (size_t)strtoull(q + 10, nullptr, 10) : 0; }
    if (step) *step = key_int(line, "\"step\":", 0);
    /* architecture features this build's graph does not have */
    static const char *const no[] = {"\"lat_guide\":", "\"lat_sub\":", "\"lat_c\":",
                                     "\"fstem\":", "\"lat_dec\":", "\"attn_mem\":", "\"view_P\":", "\"attn_deform\":",
                                     "\"skip_empty\":"};
    const char *bad = nullptr;
    for (size_t k = 0; k < sizeof no / sizeof *no && !bad; k++) if (strstr(line, no[k])) bad = no[k];
    cfg->scale_cond = key_int(line, "\"scale_cond\":", 0);
    cfg->film = key_int(line, "\"film\":", 0); cfg->gfilm = key_int(line, "\"gfilm\":", 0);      /* (src/unet.c:5683, :5742) */
    if (!bad && (cfg->film < 0 || cfg->film > 4)) bad = "\"film\":";
    if (!bad && (cfg->l0_norm < 0 || cfg->l0_norm > 4)) bad = "\"l0_norm\":";
    if (l0) {
        memset(l0, 0, sizeof *l0);
        l0->n = key_int(line, "\"l0_n\":", 0); l0->warm = key_int(line, "\"l0_warm\":", 100);
        const char *q = strstr(line, "\"l0_mom\":"); l0->mom = q ? strtof(q + 9, nullptr) : 0.01f;
        l0->gn = key_int(line, "\"ge_n\":", 0); l0->gwarm = key_int(line, "\"ge_warm\":", 500);
        q = strstr(line, "\"ge_mom\":"); l0->gmom = q ? strtof(q + 9, nullptr) : 0.01f;
        if ((q = strstr(line, "\"ge_run\":["))) { q += 10; while (l0->gcnt < 8192 && *q && *q != ']') { char *e; l0->grun[l0->gcnt] = strtof(q, &e); if (e == q) break; l0->gcnt++; q = e; if (*q == ',') q++; } }
        if ((q = strstr(line, "\"l0_run\":["))) { q += 10; while (l0->cnt < 1024 && *q && *q != ']') { char *e; l0->run[l0->cnt] = strtof(q, &e); if (e == q) break; l0->cnt++; q = e; if (*q == ',') q++; } }
    }
    /* weights the reference transforms after reading the same fp32 payload: 2:4 masks (unet_set_sparse24*) and packed fp8 / fp4 weight storage
       (unet_set_wq), src/unet.c:5703-5707, :5839-5840. Loading such a file as dense fp32 master weights would run another function */
    if (!bad && key_int(line, "\"sparse24\":", 0)) bad = "\"sparse24\": (2:4 sparse weights)";
    if (!bad && key_int(line, "\"wq\":", 0)) bad = "\"wq\": (packed fp8 / fp4 weight storage)";
    if (!bad && cfg->attn_blocks && (cfg->attn_pe < 0 || cfg->attn_pe > 3)) bad = "\"attn_pe\":";
    if (!bad && cfg->attn_blocks && (cfg->attn_axis < 0 || cfg->attn_axis > 1)) bad = "\"attn_axis\":";
    if (bad) { fprintf(stderr, "unet_peek: %s uses %s which this build does not run\n", path, bad); free(line); return -2; }
    free(line);
    return cfg->cin > 0 && cfg->cout > 0 ? 0 : -1;
}
int unet_peek(const char *path, unet_cfg *cfg, int *step) { return read_header(path, cfg, nullptr, step, nullptr); }      /* src/unet.c:5756 */
size_t mi_unet_peek_nparams(const char *path) { unet_cfg c; size_t np = 0; return read_header(path, &c, &np, nullptr, nullptr) == -1 ? 0 : np; }
/* weights and EMA weights into a net of the same architecture; the saved step, or -1 (src/unet.c:5774-5800) */
int unet_load(unet *u, const char *path) {
    unet_cfg c; size_t np = 0; int step = 0;
    static _Thread_local l0_hdr l0;
    const int r = read_header(path, &c, &np, &step, &l0);
    if (r) { if (r == -1) fprintf(stderr, "unet_load: %s: unreadable header\n", path); return -1; }
    const unet_cfg *m = &u->cfg; const char *bad = nullptr;
    if (c.nlev != m->nlev) bad = "nlev";
    for (int i = 0; !bad && i < m->nlev; i++) if (c.widths[i] != m->widths[i]) bad = "widths";
    if (!bad && c.cin != m->cin) bad = "cin";
    if (!bad && c.cout != m->cout) bad = "cout";
    if (!bad && c.attn_blocks != m->attn_blocks) bad = "attn_blocks";
    if (!bad && c.attn_blocks && c.attn_pe != m->attn_pe) bad = "attn_pe";      /* (RoPE and none have the same parameters and another function) */
    if (!bad && (c.attn_repeat > 1 ? c.attn_repeat : 1) != (m->attn_repeat > 1 ? m->attn_repeat : 1)) bad = "attn_repeat";
    if (!bad && (c.attn_vres != 0) != (m->attn_vres != 0)) bad = "attn_vres";
    if (!bad && c.down_norm != m->down_norm) bad = "down_norm";
    if (!bad && c.w4_2d != m->w4_2d) bad = "w4_2d";
    if (!bad && c.gn_ema != m->gn_ema) bad = "gn_ema";
    if (!bad && (c.scale_cond != 0) != (m->scale_cond != 0)) bad = "scale_cond";
    if (!bad && (c.film != m->film || (c.gfilm != 0) != (m->gfilm != 0))) bad = "film / gfilm";
    if (!bad && (c.ds_levels != m->ds_levels || c.emb_lev != m->emb_lev || c.emb_ch != m->emb_ch)) bad = "ds_levels / emb_lev";
    for (int i = 0; !bad && i < m->nlev; i++) if (c.enc_blocks[i] != m->enc_blocks[i]) bad = "enc_blocks";
    for (int i = 0; !bad && i < m->nlev - 1; i++) { if (dw_of(&c, i) != dw_of(m, i)) bad = "dec_widths"; if ((c.dec_convs[i] == 1) != (m->dec_convs[i] == 1)) bad = "dec_convs"; }
    if (!bad && (c.l0_norm != m->l0_norm || (c.l0_norm == 4 && (c.l0_slab > 0 ? c.l0_slab : 64) != (m->l0_slab > 0 ? m->l0_slab : 64)))) bad = "l0_norm / l0_slab";
    if (!bad && np != u->np) bad = "nparams";
    if (bad) { fprintf(stderr, "unet_load: %s: \"%s\" differs from this network's\n", path, bad); return -1; }
    FILE *f = fopen(path, "rb");
    if (!f) return -1;
    char *line = header_line(f); free(line);
    const long off = ftell(f);
    fseek(f, 0, SEEK_END);
    const long long have = (long long)ftell(f) - off, a = 4ll * (long long)np;
    if (have != 2 * a && have != 4 * a && have != 5 * a) {         /* weights + EMA, + AdamW moments, + Muon momentum (src/unet.c:5782-5790) */
        fprintf(stderr, "unet_load: %s: %lld payload bytes, the header (nparams %zu) needs 2, 4 or 5 arrays of %lld: truncated or not a checkpoint of this format\n", path, have, np, a);
        fclose(f); return -1;
    }
    float *h = malloc((size_t)a);
    int rc = -1;
    if (h && !fseek(f, off, SEEK_SET)) {
        rc = step;
        for (int which = 0; which < 2 && rc >= 0; which++) {       /* the weights, then their EMA copy */
            if (fread(h, 4, np, f) != np) { rc = -1; break; }
            size_t nbad = 0; for (size_t i = 0; i < np; i++) nbad += !isfinite(h[i]);
            if (nbad) { fprintf(stderr, "unet_load: %s: %zu non-finite values\n", path, nbad); rc = -1; break; }
            mi_h2d(which ? u->ema : u->p, h, (size_t)a); u->wm_ok = 0;
        }
        lp_wmemo_clear();
    }
    free(h); fclose(f);
    if (rc >= 0 && u->cfg.l0_norm == 2) {                          /* the running statistics; a checkpoint without them: a fresh warm-up on live statistics (src/unet.c:5841-5845) */
        const int n = 16 * G_of(u, u->cfg.widths[0]);
        if (l0.cnt == n) { mi_h2d(u->l0run, l0.run, (size_t)n * 4); u->l0_n = l0.n; u->l0_warm = l0.warm; u->l0_mom = l0.mom; }
        else { mi_zero(u->l0run, (size_t)n * 4); u->l0_n = 0; }
    }
    if (rc >= 0 && u->cfg.gn_ema) {
        /* The file holds two copies of the running statistics, the live weights' and the EMA weights'. A value that is not finite in one copy is
           taken from the other; only when some value is finite in neither, or the count does not fit the net, the statistics are dropped and the
           sites read the window's own until a trainer has made new ones (src/unet.c:5846-5860) */
        int ok = l0.gcnt == (int)(2 * u->ge_ns);
        if (ok) {
            const size_t ns = u->ge_ns; size_t bad = 0, mended = 0;
            for (size_t i = 0; i < ns; i++) {
                float *live = &l0.grun[i], *avg = &l0.grun[ns + i];
                const int fl = isfinite(*live), fa = isfinite(*avg);
                bad += !fl + !fa;
                if (!fl && fa) { *live = *avg; mended++; } else if (fl && !fa) { *avg = *live; mended++; }
            }
            if (bad) fprintf(stderr, "unet_load: gn_ema: %zu running statistics of %s are not finite, %zu taken from the other copy%s\n", bad, path, mended, mended < bad ? ": statistics dropped" : "");
            ok = mended == bad;
        }
        if (ok) { mi_h2d(u->ge_run, l0.grun, (size_t)l0.gcnt * 4); u->ge_n = l0.gn; u->ge_warm = l0.gwarm; u->ge_mom = l0.gmom; }
        else { mi_zero(u->ge_run, 2 * u->ge_ns * 4); u->ge_n = 0; }
    }
    return rc;
}
void unet_set_scale(unet *u, double um) { u->sc_c = um > 0 ? (float)log2(um / 4.8) : 0.f; }      /* the code of an input voxel size: log2(um / 4.8) (src/unet.h:141-144, src/unet.c:1943) */
void unet_set_film(unet *u, const float *codes, int k) {         /* cfg.film nets: the K codes of the following forwards (src/unet.h:148-149, src/unet.c:443) */
    float c[4];
    for (int i = 0; i < 4; i++) c[i] = i < k && codes ? codes[i] : 0.f;
    if (memcmp(c, u->film_c, sizeof c)) { memcpy(u->film_c, c, sizeof c); u->film_ok = 0; }
}
size_t unet_gfilm_off(const unet *u) { return u->gf_off; }      /* (src/unet.h:160) */
size_t mi_unet_film_off(const unet *u) { return u->film_off; }
const float *mi_unet_gfilm_codes(const unet *u) { return u->gf_g; }      /* cfg.gfilm: the last forward's pooled codes (device, widths[L-1] floats) */
void unet_set_cond(unet *u, float c) { u->sc_c = c; }             /* the code itself (src/unet.h:146-147) */
long unet_gn_ema_updates(const unet *u) { return u->ge_n; }       /* src/unet.h:280 */
long unet_l0_updates(const unet *u) { return u->l0_n; }           /* src/unet.h:314 */
int unet_save(const unet *u, const char *path, int step, const char *extra) {
    float *h = malloc(u->np * 4), *he = malloc(u->np * 4);
    if (!h || !he) { free(h); free(he); return -1; }
    mi_sync(); mi_d2h(h, u->p, u->np * 4); mi_d2h(he, u->ema, u->np * 4);
    if (nn_check()) { fprintf(stderr, "unet_save: a device error is latched: %s not written\n", path); free(h); free(he); return -1; }
    for (size_t i = 0; i < u->np; i++) if (!isfinite(h[i]) || !isfinite(he[i])) { fprintf(stderr, "unet_save: non-finite weights (first at parameter %zu): %s not written\n", i, path); free(h); free(he); return -2; }
    char tmp[1400]; snprintf(tmp, sizeof tmp, "%s.tmp", path);
    FILE *f = fopen(tmp, "wb");
    if (!f) { fprintf(stderr, "unet_save: cannot create %s\n", tmp); free(h); free(he); return -1; }
    fprintf(f, "UFSM{\"nlev\":%d,\"widths\":[", u->cfg.nlev);
    for (int i = 0; i < u->cfg.nlev; i++) fprintf(f, "%s%d", i ? "," : "", u->cfg.widths[i]);
    fputc(']', f);
    { int any = 0; for (int i = 0; i < u->cfg.nlev; i++) any |= u->cfg.dec_widths[i] != 0;       /* (only when set, src/unet.c:5549-5550) */
      if (any) { fputs(",\"dec_widths\":[", f); for (int i = 0; i < u->cfg.nlev; i++) fprintf(f, "%s%d", i ? "," : "", u->cfg.dec_widths[i]); fputc(']', f); } }
    { int any = 0; for (int i = 0; i < u->cfg.nlev; i++) any |= u->cfg.enc_blocks[i] != 0;       /* (src/unet.c:5551-5552) */
      if (any) { fputs(",\"enc_blocks\":[", f); for (int i = 0; i < u->cfg.nlev; i++) fprintf(f, "%s%d", i ? "," : "", u->cfg.enc_blocks[i]); fputc(']', f); } }
    /* (the reference's key order, src/unet.c:5561-5578: w4_2d, the attention keys, l0_norm / l0_slab, then cin) */
    if (u->cfg.w4_2d) fprintf(f, ",\"w4_2d\":%d", u->cfg.w4_2d);
    if (u->cfg.ds_levels) fprintf(f, ",\"ds_levels\":%d", u->cfg.ds_levels);
    if (u->cfg.emb_lev) fprintf(f, ",\"emb_lev\":%d,\"emb_ch\":%d", u->cfg.emb_lev, u->cfg.emb_ch);
    if (u->cfg.film) fprintf(f, ",\"film\":%d", u->cfg.film);     /* (src/unet.c:5564) */
    if (u->cfg.attn_blocks) fprintf(f, ",\"attn_blocks\":%d,\"attn_pe\":%d,\"attn_reg\":%d,\"attn_mlp\":%d", u->cfg.attn_blocks, u->cfg.attn_pe, u->cfg.attn_reg, u->tbd.F);
    if (u->cfg.attn_vres) fprintf(f, ",\"attn_vres\":%d", u->cfg.attn_vres);      /* (src/unet.c:5569) */
    if (u->cfg.attn_blocks && u->cfg.attn_axis) fprintf(f, ",\"attn_axis\":%d", u->cfg.attn_axis);      /* (src/unet.c:5570) */
    if (u->cfg.attn_blocks && u->cfg.attn_repeat > 1) fprintf(f, ",\"attn_repeat\":%d", u->cfg.attn_repeat);      /* (src/unet.c:5571) */
    if (u->cfg.l0_norm) fprintf(f, ",\"l0_norm\":%d", u->cfg.l0_norm);
    if (u->cfg.l0_norm == 4) fprintf(f, ",\"l0_slab\":%d", u->cfg.l0_slab);
    if (u->cfg.gfilm) fputs(",\"gfilm\":1", f);                    /* (src/unet.c:5588) */
    if (u->cfg.gn_ema) {                                           /* every site's running statistics and their state (src/unet.c:5587-5592; written after l0_norm's keys there too) */
        float *r = malloc(2 * u->ge_ns * 4);
        if (!r) { fprintf(stderr, "unet_save: out of memory for the running statistics: %s not written\n", path); fclose(f); remove(tmp); free(h); free(he); return -1; }      /* (a file without them would load as a fresh warm-up) */
        mi_d2h(r, u->ge_run, 2 * u->ge_ns * 4);
        fprintf(f, ",\"gn_ema\":1,\"ge_n\":%ld,\"ge_warm\":%d,\"ge_mom\":%.9g,\"ge_run\":[", u->ge_n, u->ge_warm, (double)u->ge_mom);
        for (size_t i = 0; i < 2 * u->ge_ns; i++) fprintf(f, "%s%.9g", i ? "," : "", (double)r[i]);
        fputc(']', f); free(r);
    }
    if (u->cfg.l0_norm == 2) {                                     /* the running statistics and their state (src/unet.c:5579-5584) */
        const int n = 16 * G_of(u, u->cfg.widths[0]); float r[1024];
        mi_d2h(r, u->l0run, (size_t)n * 4);
        fprintf(f, ",\"l0_n\":%ld,\"l0_warm\":%d,\"l0_mom\":%.9g,\"l0_run\":[", u->l0_n, u->l0_warm, (double)u->l0_mom);
        for (int i = 0; i < n; i++) fprintf(f, "%s%.9g", i ? "," : "", (double)r[i]);
        fputc(']', f);
    }
    { int any = 0; for (int i = 0; i < u->cfg.nlev; i++) any |= u->cfg.dec_convs[i] == 1;        /* (src/unet.c:5595-5596) */
      if (any) { fputs(",\"dec_convs\":[", f); for (int i = 0; i < u->cfg.nlev; i++) fprintf(f, "%s%d", i ? "," : "", u->cfg.dec_convs[i]); fputc(']', f); } }
    fprintf(f, ",\"cin\":%d,\"cout\":%d,\"G\":%d,\"down_norm\":%d,\"scale_cond\":%d,\"nparams\":%zu,\"step\":%d,\"sparse24\":0,\"wq\":0,\"muon_mom\":0", u->cfg.cin, u->cfg.cout, u->cfg.G,
            u->cfg.down_norm, u->cfg.scale_cond, u->np, step);
    fprintf(f, ",\"extra\":%s}\n", extra ? extra : "{}");
    int ok = fwrite(h, 4, u->np, f) == u->np && fwrite(he, 4, u->np, f) == u->np;      /* weights, EMA weights */
    ok = !fclose(f) && ok;
    free(h); free(he);
    if (!ok || rename(tmp, path)) { fprintf(stderr, "unet_save: write error on %s\n", tmp); remove(tmp); return -1; }
    return 0;
}
