// Host side of the 2x2x2 stride-2 conv and transposed conv (mi_conv_down2_fwd, mi_convt_up2_fwd): operand staging, weight preparation, launch.
#include "conv2_kernel.hpp"
#include "../../include/mi_lp.h"

bool mi_wmemo_other(unsigned key, const float *w, int fmt, int Co, int Ci, int nmt_all, int lay, size_t wq_bytes, size_t wsc_bytes, uint8_t **wq, uint8_t **wsc);     // conv3.hip
unsigned mi_take_s2_wkey(void);

// weights -> the MFMA's lane order, one tile per (K pair, channel tile) as the 3x3x3 kernels read them. down: w [Co][Ci][8], pair gp = units 2 gp,
// 2 gp + 1 of the tap-major (tap, block) order; up: w [Ci][Co][8], pair gp = (tap gp / npt, blocks 2 (gp % npt), + 1), a missing second block = zeros
template <int FMT>
__global__ void __launch_bounds__(128) prep_w2_k(const float *__restrict__ w, uint8_t *__restrict__ wq, unsigned *__restrict__ wsc, int Co, int Ci, int nb, int nmt_all, int npairs, int up) {
    constexpr int WTILE = fmt_t<FMT>::WTILE;
    const size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    const int Cop = nmt_all * 32;
    if (i >= (size_t)npairs * Cop) return;
    const int cop = (int)(i % Cop), gp = (int)(i / Cop), m = cop >> 5, r = cop & 31, npt = (nb + 1) >> 1, cw = (cop & ~31) + mi_row_chan(r);     // row r carries output channel cw
    uint8_t *tile = wq + ((size_t)gp * nmt_all + m) * WTILE;
    unsigned *tsc = wsc + ((size_t)gp * nmt_all + m) * 64;
#pragma unroll
    for (int side = 0; side < 2; side++) {
        int t, blk;
        if (up) { t = gp / npt; blk = 2 * (gp % npt) + side; } else { const int u = 2 * gp + side; t = u / nb; blk = u - t * nb; }
        float v[32];
#pragma unroll
        for (int k = 0; k < 32; k++) {
            const int ci = blk * 32 + k;
            v[k] = (blk < nb && cw < Co && ci < Ci) ? (up ? w[((size_t)ci * Co + cw) * 8 + t] : w[((size_t)cw * Ci + ci) * 8 + t]) : 0.f;
        }
        prep_store_unit<FMT>(tile, tsc, 1, side, r, v);
    }
}

static int conv2_dispatch(const char *who, int up, int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp) {
    const unsigned wkey = mi_take_s2_wkey();                 // (consumed by this call, whatever becomes of it)
    if (bits != 8 && bits != 4) { fprintf(stderr, "%s: compute format %d (8 or 4)\n", who, bits); return -1; }
    if (xbf != 3 && xbf != 4) { fprintf(stderr, "%s: the input must be an MX tensor (dtype %d)\n", who, xbf); return -1; }
    if (ybf != 0 && ybf != 2 && ybf != 3 && ybf != 4) { fprintf(stderr, "%s: output dtype %d\n", who, ybf); return -1; }
    const int N = xs.n, Ci = xs.c, D = xs.d, H = xs.h, W = xs.w;
    if (N <= 0 || Ci <= 0 || cout <= 0 || D <= 0 || H <= 0 || W <= 0 || N > 65535) { fprintf(stderr, "%s: shape\n", who); return -1; }
    if (!up && ((D | H | W) & 1)) { fprintf(stderr, "%s: the 2x2x2 stride-2 conv needs even dims (%d %d %d)\n", who, D, H, W); return -1; }
    if (gp.ns) mi_die("%s: slab-local GroupNorm (gnp_t.ns) is not supported", who);
    const int fmt = bits, fdt = fmt == 8 ? 3 : 4, RB = fmt == 8 ? 32 : 16, WTILE = fmt == 8 ? 2048 : 1024;
    const size_t S = (size_t)D * H * W;
    conv_args a;
    memset(&a, 0, sizeof a);
    const int nbp = (Ci + 31) / 32;
    if (xbf == fdt && !(gp.G > 0) && mx_bw(Ci) == 32) {      // the stored rows are the operand
        a.xq[0] = (const uint8_t *)x; a.xsc[0] = a.xq[0] + (size_t)N * nbp * S * RB;
    } else {                                                 // GroupNorm + SiLU and / or another format or row width: one re-quantising pass, as the 3x3x3 convs
        uint8_t *st = (uint8_t *)mi_ws(MI_WS_XSTAGE, (size_t)N * nbp * S * (RB + 1));
        mi_restage(x, xbf, N, Ci, S, gp, Ci, 0, st, fmt);
        a.xq[0] = st; a.xsc[0] = st + (size_t)N * nbp * S * RB;
    }
    a.nbs[0] = nbp; a.bws[0] = 32; a.nbt = nbp; a.wide = 1;
    a.N = N; a.D = D; a.H = H; a.W = W;
    a.Do = up ? 2 * D : D / 2; a.Ho = up ? 2 * H : H / 2; a.Wo = up ? 2 * W : W / 2;
    const int nmt_all = (cout + 31) / 32, npairs = up ? 8 * ((nbp + 1) / 2) : 4 * nbp;
    const int MT = nmt_all % 4 == 0 ? 4 : nmt_all % 2 == 0 ? 2 : 1;
    // prepared weights: per call into the scratch, or once under the memo id the calling thread set for this call (mi_conv_s2_wkey)
    const size_t wq_bytes = (size_t)npairs * nmt_all * WTILE, wsc_bytes = (size_t)npairs * nmt_all * 256;
    uint8_t *wq = nullptr, *wsc = nullptr; bool have = false;
    if (wkey && !mi_ws_arena_on()) have = mi_wmemo_other(wkey, w, fmt, cout, Ci, nmt_all, up ? 2 : 1, wq_bytes, wsc_bytes, &wq, &wsc);
    else { wq = (uint8_t *)mi_ws(MI_WS_WQ, wq_bytes); wsc = (uint8_t *)mi_ws(MI_WS_WSC, wsc_bytes); }
    if (!have) {
        const size_t nt = (size_t)npairs * nmt_all * 32;
        if (fmt == 8) prep_w2_k<8><<<nblk_(nt, 128), 128>>>(w, wq, (unsigned *)wsc, cout, Ci, nbp, nmt_all, npairs, up);
        else prep_w2_k<4><<<nblk_(nt, 128), 128>>>(w, wq, (unsigned *)wsc, cout, Ci, nbp, nmt_all, npairs, up);
        MICK();
    }
    a.wq = wq; a.wsc = wsc; a.nmt_all = nmt_all; a.ncs = nmt_all / MT;
    a.bias = b; a.Co = cout; a.y = y; a.ydt = ybf;
    a.zs0 = 0; a.zs1 = a.Do;
    a.epi_o = 0; a.red_o = (unsigned)((size_t)3 * MT * 32 * sizeof(float));
    const size_t smem = a.red_o + 1024;
    const long long Scol = up ? (long long)S : (long long)a.Do * a.Ho * a.Wo;
    const long long gx = ((Scol + 31) / 32 + 7) / 8;         // 4 wavefronts x 2 tiles of 32 columns per workgroup
    if (gx > 0x7fffffffLL || a.ncs > 8191) mi_die("%s: launch grid", who);
    const dim3 grid((unsigned)gx, (unsigned)(up ? 8 * a.ncs : a.ncs), (unsigned)N);      // (up: one tap per workgroup)
    const int out = ybf == 3 ? 8 : ybf == 4 ? 4 : 0;
    if (fmt == 8) conv2_launch_f8(out, up, MT, a, grid, smem); else conv2_launch_f4(out, up, MT, a, grid, smem);
    return 0;
}
extern "C" int mi_conv_down2_fwd(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp) {
    return conv2_dispatch("mi_conv_down2_fwd", 0, bits, x, xbf, xs, w, b, cout, y, ybf, gp);
}
extern "C" int mi_convt_up2_fwd(int bits, const void *x, int xbf, shape5 xs, const float *w, const float *b, int cout, void *y, int ybf, gnp_t gp) {
    return conv2_dispatch("mi_convt_up2_fwd", 1, bits, x, xbf, xs, w, b, cout, y, ybf, gp);
}
