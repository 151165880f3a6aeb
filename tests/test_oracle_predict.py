"""Pins of the oracle's sliding-window pieces (CPU only): placement box + sigmoid rounding, and the feather blend against the checks the
reference's own test makes (tests/test_predict_feather.c:95-121)."""
import numpy as np
import pytest

import orc


@pytest.mark.parametrize("o,e", [((-4, -4, -4), (24, 24, 24)), ((0, 3, -6), (10, 20, 9)), ((-20, 0, 0), (8, 8, 8))])
def test_place_box_and_rounding(o, e):
    rng = np.random.default_rng(1)
    D = W = 16; hz, halo, shard, iso = 2, 4, 24, 64
    lg = (3 * rng.standard_normal((D, W, W))).astype(np.float32); ct = rng.integers(0, 256, (D, W, W)).astype(np.uint8)
    got = orc.pred_place(lg, ct, D, W, hz, halo, o, e, shard, iso, dsh=np.full((shard,) * 3, 7, np.uint8))
    want = np.full((shard,) * 3, 7, np.uint8)                       # brute force: every window voxel tested against both boxes
    prob = np.floor(255.0 / (1.0 + np.exp(-lg.astype(np.float64))) + 0.5)
    for z in range(D):
        for y in range(W):
            for x in range(W):
                inside = hz <= z < D - hz and halo <= y < W - halo and halo <= x < W - halo
                g = (o[0] + z, o[1] + y, o[2] + x)
                if inside and all(0 <= g[k] < e[k] for k in range(3)):
                    want[g] = prob[z, y, x] if ct[z, y, x] >= iso else 0
    d = np.abs(got.astype(int) - want.astype(int))
    assert d.max() <= 1 and (d > 0).mean() < 1e-3                   # (fp32 sigmoid against fp64: a step of 1 at an exact .5 only)
    assert np.array_equal(got == 7, want == 7)                      # exactly the intersection is written


def u_of(B):
    s = np.sin(np.pi / 2 * (np.arange(B) + 0.5) / B)
    return s * s


def test_blend_core_first_window_and_z_shell():
    rng = np.random.default_rng(2)
    S, B = 12, 4; En = S + B
    nss = (2, 2, 2); bn = (24, 24, 24)
    E = rng.integers(0, 256, (8, En, En, En)).astype(np.uint8)
    out = orc.feather_blend(E, np.ones(8, np.uint8), S, B, nss, bn)
    u = u_of(B)
    for wid, (a, b, c) in enumerate(np.ndindex(2, 2, 2)):
        own = out[a * S:(a + 1) * S, b * S:(b + 1) * S, c * S:(c + 1) * S]
        assert np.array_equal(own[B:, B:, B:], E[wid][B:S, B:S, B:S])                                # core: the window's own bytes
    assert np.array_equal(out[:S, :S, :S], E[0][:S, :S, :S])                                         # the first window has nothing to blend with
    # z shell of window (1, 0, 0) away from the y / x shells: u(j) own + (1 - u(j)) lower window's spill, within 1 (the reference's gate)
    for j in range(B):
        want = u[j] * E[4][j, B:S, B:S].astype(float) + (1 - u[j]) * E[0][S + j, B:S, B:S].astype(float)
        assert np.abs(out[S + j, B:S, B:S] - want).max() <= 1.0
    # an edge of three windows (z and y shells of window (1, 1, 0)): normalised product weights over the four windows back by (dz, dy)
    z, y, x = 1, 2, 7
    w = {(0, 0): u[z] * u[y], (1, 0): (1 - u[z]) * u[y], (0, 1): u[z] * (1 - u[y]), (1, 1): (1 - u[z]) * (1 - u[y])}
    val = {(0, 0): E[6][z, y, x], (1, 0): E[2][z + S, y, x], (0, 1): E[4][z, y + S, x], (1, 1): E[0][z + S, y + S, x]}
    want = sum(w[k] * float(val[k]) for k in w) / sum(w.values())
    assert abs(float(out[S + z, S + y, x]) - want) <= 1.0


def test_blend_constant_field_and_absent_windows():
    S, B = 8, 8; En = S + B                                          # B = S: the whole interior is shell
    nss = (3, 1, 2); bn = (22, 8, 13)                               # the box ends inside the last windows
    E = np.zeros((6, En, En, En), np.uint8)
    for k in range(6):
        E[k] = 40 * k + 10
    present = np.array([1, 1, 0, 1, 1, 1], np.uint8)
    out = orc.feather_blend(E, present, S, B, nss, bn)
    assert out.shape == bn
    assert (out[8:16, :, 0:8] == 0).all()                            # window 2 = (1, 0, 0) was not computed: nothing is written there
    assert (out[0:8, :, 0:8] == 10).all()                            # first window: its own value
    # window 4 = (2, 0, 0): its z neighbour is absent, so the blend renormalises to its own value
    assert (out[16:22, :, 0:8] == 170).all()
    # window 1 = (0, 0, 1) blends with window 0 along x only: between the two constants, monotone from the neighbour's to its own
    row = out[3, 4, 8:13].astype(int)
    assert (np.diff(row) >= 0).all() and 10 <= row[0] < row[-1] <= 50
    Ec = np.full((6, En, En, En), 93, np.uint8)                      # a constant field is a fixed point whatever the weights
    o2 = orc.feather_blend(Ec, present, S, B, nss, bn)
    assert set(np.unique(o2)) == {0, 93}
