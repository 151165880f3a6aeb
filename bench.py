#!/usr/bin/env python3
"""Benchmark of the MX conv hot path on one MI355X.

Workload (BASELINE.json configs[1]): a stack of four 3x3x3 convolutions, Cin = Cout = 128, batch 2, 64^3 voxels, MX-fp8 (e4m3 + E8M0
per 32 channels) activations and weights, bias, GroupNorm(8) statistics fused into each conv's epilogue, the previous layer's
GroupNorm affine + SiLU applied to the conv's input, MX-fp8 re-quantised output: the reference's block structure (src/unet.c:2567-2636).
A step = one pass of the stack over one batch resident in HBM. Prints one JSON line."""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

METRIC = "U-Net infer voxels/s (128^3 patch, MX fp8) + 3x3x3 conv % of MFMA peak"
MFMA_PEAK_FP8_TFLOPS = 5033.0          # MI355X dense MXFP8 (2.5 PFLOP/s bf16 x 2)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="target seconds of CPU work for the cpu_baseline sample")
    ap.add_argument("--copy-probe", action="store_true", help="run 5 device-to-device copies of 1 GiB and exit: the known-size kernel that scales "
                    "rocprofv3's FETCH_SIZE / WRITE_SIZE counters")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (the path shards by windows / z-slabs, see DESIGN.md)" % a.gpus, file=sys.stderr)
        sys.exit(2)
    import numpy as np
    from ufsm_amd import lib, LP, shape5, gnp_t, split_t, DevBuf
    if lib.mi_init(0) != 0:
        print("bench.py: no gfx950 GPU: the HIP path cannot run (there is no CPU fallback)", file=sys.stderr)
        sys.exit(3)
    if a.copy_probe:
        nb = 1 << 30
        src, dst = DevBuf(nb), DevBuf(nb)
        lib.mi_zero(src.ptr, nb)
        for _ in range(5):
            lib.mi_d2d(dst.ptr, src.ptr, nb)
        lib.mi_sync(); LP.check()
        print(json.dumps({"copy_probe_bytes": nb, "copies": 5}))
        return
    N, Cc, D, L, G = 2, 128, 64, 4, 8
    S = D * D * D
    rng = np.random.default_rng(0)
    x = rng.standard_normal((N, Cc, S)).astype(np.float32)
    dx = DevBuf.from_numpy(x)
    act = [DevBuf(lib.lp_mx8_bytes(N, Cc, S)) for _ in range(2)]
    x0 = DevBuf(lib.lp_mx8_bytes(N, Cc, S))
    lib.lp_f32_to_mx8(dx.ptr, N, Cc, S, x0.ptr)
    ws, bs, gam, bet, mean, rstd, sums = [], [], [], [], [], [], []
    for l in range(L):
        w = (rng.standard_normal((Cc, Cc, 27)) * np.sqrt(2.0 / (Cc * 27))).astype(np.float32)
        ws.append(DevBuf.from_numpy(w)); bs.append(DevBuf.from_numpy((rng.standard_normal(Cc) * 0.1).astype(np.float32)))
        gam.append(DevBuf.from_numpy(np.ones(Cc, np.float32))); bet.append(DevBuf.from_numpy(np.zeros(Cc, np.float32)))
        mean.append(DevBuf(N * G * 4)); rstd.append(DevBuf(N * G * 4)); sums.append(DevBuf(N * G * 2 * 24))
    w_host_l0 = w
    xs = shape5(N, Cc, D, D, D)

    def step():
        src = x0
        for l in range(L):
            dst = act[l & 1]
            gp = gnp_t() if l == 0 else LP.gn(gam[l - 1], bet[l - 1], mean[l - 1], rstd[l - 1], G)
            sp = split_t(); sp.wkey = 100 + l            # weights are constant across steps: prepared once (inference)
            lib.mi_gn_sums_zero(sums[l].ptr, N * G * 2)
            lib.lp_conv_fwd_f8(src.ptr, 3, xs, ws[l].ptr, bs[l].ptr, Cc, dst.ptr, 3, gp, sums[l].ptr, G, sp)
            lib.mi_gn_finalize(sums[l].ptr, N * G, (Cc // G) * S, 1e-5, mean[l].ptr, rstd[l].ptr)
            src = dst

    for _ in range(a.warmup):
        step()
    LP.check()
    lib.mi_kernel_timing(1)
    lib.mi_sync()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    lib.mi_sync()
    t1 = time.perf_counter()
    LP.check()
    nl = C.c_long(0)
    kms = lib.mi_kernel_timing_read(C.byref(nl))
    lib.mi_kernel_timing(0)
    kernel = lib.mi_last_kernel().decode()
    ms_step = (t1 - t0) * 1e3 / a.steps
    vox_per_step = N * S
    flops_layer = 2.0 * 27 * Cc * Cc * N * S               # logical channels, all 27 taps (tests/bench_lp.c:46)
    k_ms = kms / max(nl.value, 1)
    achieved = flops_layer / (k_ms * 1e-3) / 1e12
    out = {
        "metric": METRIC, "value": vox_per_step / (ms_step * 1e-3), "unit": "voxels/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "mxfp8 (e4m3 x e4m3, fp32 accumulate)",
        "data": "synthetic",
        "config": {"workload": "configs[1]: 4 x (3x3x3 conv 128->128, N 2, 64^3, MX-fp8 in/out, bias + GroupNorm(8) stats, GN+SiLU on the input)",
                   "layers": L, "batch": N, "channels": Cc, "dims": [D, D, D]},
        "tflops": L * flops_layer / (ms_step * 1e-3) / 1e12,
        "roofline": {"bound": "mfma", "kernel": kernel, "achieved": achieved, "peak": MFMA_PEAK_FP8_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_PEAK_FP8_TFLOPS,
                     "launches": nl.value, "avg_launch_ms": k_ms, "flops_per_launch": flops_layer, "traffic": None},
    }
    if not a.no_cpu_baseline:
        import orc
        # the oracle (a port: the reference has no CPU MX conv) on a bounded z-slab of one layer of the same workload
        xq = x0.to_numpy(np.uint8)
        nthreads = orc.lib().orc_threads()
        t = time.perf_counter(); orc.conv3(xq, 3, N, Cc, D, D, D, w_host_l0, None, Cc, 3, z0=0, z1=1); dt1 = time.perf_counter() - t
        nz = int(max(1, min(D, a.cpu_seconds / max(dt1, 1e-3))))
        t = time.perf_counter(); orc.conv3(xq, 3, N, Cc, D, D, D, w_host_l0, None, Cc, 3, z0=D // 2 - nz // 2, z1=D // 2 - nz // 2 + nz); dt = time.perf_counter() - t
        layer_s = dt * D / nz                                   # a whole layer, extrapolated from the slab
        out["cpu_baseline"] = {"value": vox_per_step / (L * layer_s), "unit": "voxels/s", "cores": nthreads, "kind": "port",
                               "sample": "oracle orc_conv3 on %d of %d output z planes (both samples) of layer 0, scaled to the 4-layer stack" % (nz, D),
                               "gflops": flops_layer * nz / D / dt / 1e9}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
