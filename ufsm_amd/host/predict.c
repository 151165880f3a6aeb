/* Sliding-window prediction of a device-resident volume: window iteration, placement and the feather blend
 * (the reference's `predict --feather` single pass: src/predict.c:282-333 blend, :2538-2545 window grid, :3420-3436 placement of E). */
#include <stdio.h>
#include <stdlib.h>
#include "../../include/mi_unet.h"
#include "../../include/mi_predict.h"

int unet_predict_volume(unet *u, const uint8_t *vol, const int64_t dims[3], int halo, int feather, float mean, float isd,
                        int axis, float cy, float cx, uint8_t *out, int64_t nwin[2]) {
    const shape5 in = unet_in_shape(u);
    const int W = in.w, S = W - 2 * halo, B = feather, En = S + B;
    if (in.n != 1 || in.d != W || in.h != W || halo < 0 || S <= 0 || B < 0 || B > halo || B > S || B > 1024) {
        fprintf(stderr, "unet_predict_volume: needs one cubic window, 0 <= feather <= halo, window - 2 halo > 0 and feather <= it (window %d x %d x %d, halo %d, feather %d)\n",
                in.d, in.h, in.w, halo, feather);
        return -1;
    }
    int64_t nss[3], total = 1;
    for (int d = 0; d < 3; d++) { if (dims[d] <= 0) return -1; nss[d] = (dims[d] + S - 1) / S; total *= nss[d]; }
    const size_t w3 = (size_t)W * W * W, e3 = (size_t)En * En * En;
    uint8_t *E = mi_malloc((size_t)total * e3), *ctw = mi_malloc(w3), *dpres = mi_malloc((size_t)total);
    float *lg = mi_malloc((size_t)unet_config(u)->head_out * w3 * sizeof(float)), *doff = mi_malloc(2 * (size_t)W * sizeof(float));
    unsigned *dany = mi_malloc(sizeof(unsigned));
    uint8_t *present = calloc((size_t)total, 1);
    float *hoff = malloc(2 * (size_t)W * sizeof(float));
    int rc = present && hoff ? 0 : -1;
    int64_t done = 0;
    const int iso = nn_get_pred_iso();
    for (int64_t a = 0; a < nss[0] && !rc; a++) for (int64_t b = 0; b < nss[1] && !rc; b++) for (int64_t c = 0; c < nss[2] && !rc; c++) {
        const int64_t id = (a * nss[1] + b) * nss[2] + c, oz = a * S - halo, oy = b * S - halo, ox = c * S - halo;
        mi_zero(dany, sizeof(unsigned));
        mi_ct_window(vol, dims[0], dims[1], dims[2], oz, oy, ox, W, ctw, iso, halo, dany);
        unsigned any = 0; mi_d2h(&any, dany, sizeof any);
        if (!any) continue;                                 /* air: not computed; its neighbours renormalise */
        for (int z = 0; z < W; z++) { hoff[z] = (float)oy - cy; hoff[W + z] = (float)ox - cx; }      /* the window rows' / columns' offsets from the scroll axis, per plane */
        mi_h2d(doff, hoff, 2 * (size_t)W * sizeof(float));
        if (unet_forward_ct(u, ctw, mean, isd, doff, doff + W, axis, lg)) { rc = -1; break; }
        /* E: the interior and B voxels of the upper halo, window coordinates [halo, halo + S + B) -> [0, S + B) (src/predict.c:3426-3427) */
        nn_pred_place(lg, ctw, W, halo - B, -halo, -halo, -halo, En, En, En, En, E + (size_t)id * e3);
        present[id] = 1; done++;
    }
    if (!rc) {
        mi_h2d(dpres, present, (size_t)total);
        rc = mi_feather_blend(E, dpres, S, B, nss, dims, out);
        mi_sync();
        if (lp_check()) rc = -1;
    }
    if (nwin) { nwin[0] = total; nwin[1] = done; }
    mi_sync();
    mi_free(E); mi_free(ctw); mi_free(dpres); mi_free(lg); mi_free(doff); mi_free(dany);
    free(present); free(hoff);
    return rc;
}
