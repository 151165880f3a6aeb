/* Sliding-window prediction of a device-resident volume: window iteration, placement and the feather blend
 * (the reference's `predict --feather` single pass: src/predict.c:282-333 blend, :2538-2545 window grid, :3420-3436 placement of E). */
#include <stdio.h>
#include <stdlib.h>
#include "../../include/mi_unet.h"
#include "../../include/mi_predict.h"

int mi_unet_predict_volume(unet *u, int window, int nbatch, const uint8_t *vol, const int64_t dims[3], int halo, int feather, float mean, float isd,
                           int axis, float cy, float cx, uint8_t *out, int64_t nwin[2]) {
    shape5 in = {nbatch, 4, window, window, window};
    const int W = in.w, S = W - 2 * halo, B = feather, En = S + B;
    if (in.n < 1 || in.n > 64 || in.d != W || in.h != W || halo < 0 || S <= 0 || B < 0 || B > halo || B > S || B > 1024) {
        fprintf(stderr, "mi_unet_predict_volume: needs cubic windows (1 .. 64 per forward), 0 <= feather <= halo, window - 2 halo > 0 and feather <= it (window %d x %d x %d, halo %d, feather %d)\n",
                in.d, in.h, in.w, halo, feather);
        return -1;
    }
    int64_t nss[3], total = 1;
    for (int d = 0; d < 3; d++) { if (dims[d] <= 0) return -1; nss[d] = (dims[d] + S - 1) / S; total *= nss[d]; }
    const size_t w3 = (size_t)W * W * W, e3 = (size_t)En * En * En;
    uint8_t *E = mi_malloc((size_t)total * e3), *ctw = mi_malloc((size_t)in.n * w3), *dpres = mi_malloc((size_t)total);
    const size_t lgn = (size_t)unet_cfg_of(u)->cout * w3;      /* logits of one window */
    float *doff = mi_malloc((size_t)total * 2 * W * sizeof(float));
    unsigned *dany = mi_malloc((size_t)total * sizeof(unsigned));
    uint8_t *present = calloc((size_t)total, 1);
    unsigned *hany = malloc((size_t)total * sizeof(unsigned));
    float *hoff = malloc((size_t)total * 2 * W * sizeof(float));
    int rc = present && hoff && hany ? 0 : -1;
    int64_t done = 0;
    const int iso = nn_get_pred_iso();
    /* Pass 1, no host round trip per window: every window's "holds a voxel >= iso in its interior" flag (air windows are not computed; their
     * neighbours renormalise) and the table of the window rows' / columns' offsets from the scroll axis, then one copy each way. The forwards
     * of pass 2 are then enqueued back to back and the GPU never waits for the host. */
    if (!rc) {
        mi_zero(dany, (size_t)total * sizeof(unsigned));
        mi_ct_flags(vol, dims[0], dims[1], dims[2], S, nss, iso, dany);       /* (a window's interior is cell (a, b, c) of the S grid: one read of the volume) */
        for (int64_t a = 0; a < nss[0]; a++) for (int64_t b = 0; b < nss[1]; b++) for (int64_t c = 0; c < nss[2]; c++) {
            const int64_t id = (a * nss[1] + b) * nss[2] + c, oy = b * S - halo, ox = c * S - halo;
            float *ho = hoff + (size_t)id * 2 * W;
            for (int z = 0; z < W; z++) { ho[z] = (float)oy - cy; ho[W + z] = (float)ox - cx; }
        }
        mi_d2h(hany, dany, (size_t)total * sizeof(unsigned));
        mi_h2d(doff, hoff, (size_t)total * 2 * W * sizeof(float));
    }
    /* Pass 2: the windows that hold material, in z-y-x order, in.n per forward (window j of a batch -> sample j; samples are independent, so a
     * window's prediction does not depend on its batch; a last, incomplete batch repeats its last window and places it once) */
    int64_t *list = malloc((size_t)(total ? total : 1) * sizeof(int64_t)), np = 0;
    /* a net whose attention stage reads the scroll axis (cfg.attn_axis radial / attn_pe scroll) gets every forward's windows' axis records:
     * the axis along window z, its centre per window plane = the negated row / column offsets (pred_axis, src/predict.c:1128-1141) */
    const unet_cfg *cf = unet_cfg_of(u);
    const int wants_axis = cf->attn_blocks > 0 && (cf->attn_axis == 1 || cf->attn_pe == 3);
    float *axrec = wants_axis ? malloc((size_t)64 * UNET_AXR(W) * sizeof(float)) : NULL;
    if (!list || (wants_axis && !axrec)) rc = -1;
    for (int64_t id = 0; id < total && !rc; id++) if (hany[id]) list[np++] = id;
    /* the windows are spread evenly over the forwards that nbatch windows per forward need: 726 windows at up to 64 per forward are 12 forwards
     * of 61 (6 samples repeat a window), not 11 of 64 and one of 22 padded to 64. The graph is (re)built for that sample count by the first forward */
    if (np > 0) { const int64_t nf = (np + in.n - 1) / in.n; in.n = (int)((np + nf - 1) / nf); }
    for (int64_t k = 0; k < np && !rc; k += in.n) {
        const uint8_t *cts[64]; const float *dyos[64], *dxos[64]; int64_t org[64 * 3], eoff[64];
        const int nreal = (int)(np - k < in.n ? np - k : in.n);
        for (int j = 0; j < in.n; j++) {
            const int64_t id = list[k + j < np ? k + j : np - 1], a = id / (nss[1] * nss[2]), b = (id / nss[2]) % nss[1], c = id % nss[2];
            org[3 * j] = a * S - halo; org[3 * j + 1] = b * S - halo; org[3 * j + 2] = c * S - halo;
            eoff[j] = id * (int64_t)e3;
            cts[j] = ctw + (size_t)j * w3; dyos[j] = doff + (size_t)id * 2 * W; dxos[j] = dyos[j] + W;
        }
        if (wants_axis) {
            for (int j = 0; j < in.n; j++) {
                float *r = axrec + (size_t)j * UNET_AXR(W);
                r[0] = 0.f; r[1] = axis ? 1.f : 0.f; r[2] = (float)W; r[3] = 1.f;
                for (int z = 0; z < W; z++) { r[4 + 2 * z] = cy - (float)org[3 * j + 1]; r[5 + 2 * z] = cx - (float)org[3 * j + 2]; }
            }
            unet_set_attn_axis(u, axrec, in.n, UNET_AXR(W));
        }
        mi_ct_windows(vol, dims[0], dims[1], dims[2], org, in.n, W, ctw, iso, halo, NULL);
        const float *lg = mi_unet_forward_ct_n(u, cts, mean, isd, dyos, dxos, axis, in, 2);      /* (fp16-rounded input values, as predict) */
        if (!lg) { rc = -1; break; }
        /* E: the interior and B voxels of the upper halo, window coordinates [halo, halo + S + B) -> [0, S + B) (src/predict.c:3426-3427) */
        mi_pred_place_n(lg, lgn, ctw, w3, nreal, eoff, W, W, halo - B, halo - B, -halo, -halo, -halo, En, En, En, En, E);
        for (int j = 0; j < nreal; j++) { present[list[k + j]] = 1; done++; }
    }
    free(list); free(axrec);
    if (!rc) {
        mi_h2d(dpres, present, (size_t)total);
        rc = mi_feather_blend(E, dpres, S, B, nss, dims, out);
        mi_sync();
        if (lp_check()) rc = -1;
    }
    if (nwin) { nwin[0] = total; nwin[1] = done; }
    mi_sync();
    mi_free(E); mi_free(ctw); mi_free(dpres); mi_free(doff); mi_free(dany);
    free(present); free(hoff); free(hany);
    return rc;
}
