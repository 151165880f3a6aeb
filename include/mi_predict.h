/* Sliding-window prediction pieces for AMD MI355X (gfx950): the sigmoid -> uint8 placement of a window's logits, and the seam-free
 * feather blend of window borders. Device pointers everywhere, asynchronous on the null stream; errors are latched for lp_check().
 *
 * nn_pred_place / nn_pred_place_d / nn_set_pred_iso / nn_get_pred_iso keep the reference's declarations (src/nn.h, defined in
 * src/nn_elem.cu:1103-1130). The blend is the reference's host routine (src/predict.c:282-333) as one device kernel over the
 * whole output box: on a 288 GB device every window's prediction stays resident, so no spill slabs are kept on the host. */
#ifndef MI_PREDICT_H
#define MI_PREDICT_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* replaces nn_set_pred_iso / nn_get_pred_iso (src/nn_elem.cu:1103-1104): CT values below iso (>= 1) predict 0 */
void nn_set_pred_iso(int t);
int nn_get_pred_iso(void);
/* replaces nn_pred_place_d (src/nn_elem.cu:1122-1126): lg fp32 logits and ct uint8 of a D x W x W window; the voxels inside the window's
   interior ([hz, D - hz) x [halo, W - halo)^2) and inside the target box ([-o, e - o) per axis) are written to
   dsh[((oz + z) shard + oy + y) shard + ox + x] = ct >= iso ? (uint8)(255 sigmoid(lg) + .5) : 0 */
void nn_pred_place_d(const float *lg, const uint8_t *ct, int D, int W, int hz, int halo, int oz, int oy, int ox, int ez, int ey, int ex, int shard, uint8_t *dsh);
/* replaces nn_pred_place (src/nn_elem.cu:1127-1129): the cubic window, hz = halo */
void nn_pred_place(const float *lg, const uint8_t *ct, int W, int halo, int oz, int oy, int ox, int ez, int ey, int ex, int shard, uint8_t *dsh);
/* (no counterpart: the reference places one window per call) nn_pred_place_d for the n windows of one forward in one launch: window j's logits
   at lg + j lstride (floats), its CT at ct + j cstride (bytes), its target dsh + doff[j] (doff: n byte offsets on the host, or null for 0);
   one geometry for all. Each window's bytes are those of nn_pred_place_d on it. */
void mi_pred_place_n(const float *lg, size_t lstride, const uint8_t *ct, size_t cstride, int n, const int64_t *doff, int D, int W, int hz, int halo, int oz, int oy, int ox,
                     int ez, int ey, int ex, int shard, uint8_t *dsh);

/* (no counterpart: the reference reads windows from its volume store) a W^3 window of a device uint8 volume [Z][Y][X] with its origin at
   (oz, oy, ox), zero outside the volume; any[0] (device, zeroed by the caller or null) is set non-zero when a voxel >= iso lies inside the
   window's interior [halo, W - halo)^3 (the footprint it predicts: a window without one is air) */
void mi_ct_window(const uint8_t *vol, int64_t Z, int64_t Y, int64_t X, int64_t oz, int64_t oy, int64_t ox, int W, uint8_t *win, int iso, int halo, unsigned *any);
/* (no counterpart) mi_ct_window for n windows in one launch: window j's origin org[3 j .. 3 j + 2] (host, z-y-x), its bytes at win + j W^3, its flag
   any + j (any may be null) */
void mi_ct_windows(const uint8_t *vol, int64_t Z, int64_t Y, int64_t X, const int64_t *org, int n, int W, uint8_t *win, int iso, int halo, unsigned *any);
/* (no counterpart) the flags alone, for every window of a sliding grid, in one read of the volume: any[(a nss[1] + b) nss[2] + c] (device, zeroed by
   the caller) is set non-zero when a voxel >= iso lies in [a S, a S + S) x [b S, b S + S) x [c S, c S + S) clipped to the volume - the interior of the
   window whose origin is (a S - halo, b S - halo, c S - halo), i.e. what mi_ct_window reports for it */
void mi_ct_flags(const uint8_t *vol, int64_t Z, int64_t Y, int64_t X, int S, const int64_t nss[3], int iso, unsigned *any);
/* the feather blend of src/predict.c:282-333 over the whole output box. Windows of interior S lie on a grid nss[3] (z-y-x order), window
   k's prediction E + k (S + B)^3 covers [0, S + B)^3 from its interior origin (what nn_pred_place writes with halo - B, o = -halo,
   e = shard = S + B); present[k] != 0: computed. out: uint8 [bn0][bn1][bn2], the box from the grid origin (bn <= nss S). A voxel with every
   local coordinate >= B is the window's own byte; in the lower shell the present windows shifted back by delta in {0, 1}^3 blend with
   weights prod_d (delta_d ? 1 - u(v_d) : u(v_d)), u(j) = sin^2(pi/2 (j + .5) / B), normalised, summed in the reference's order.
   0 <= B <= S, B <= 1024 (0: no blend). Returns 0, or -1 for a bad geometry. */
int mi_feather_blend(const uint8_t *E, const uint8_t *present, int S, int B, const int64_t nss[3], const int64_t bn[3], uint8_t *out);

#ifdef __cplusplus
}
#endif
#endif
