"""Builds the HIP library (gfx950) and the CPU oracle in-tree. Used by __graft_entry__.build(); tests and the bench only load what is built."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ufsm_amd", "csrc")
LIB = os.path.join(ROOT, "ufsm_amd", "libufsm_lp.so")
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "liboracle.so")
HIP_SOURCES = ["rt.hip", "mx_elem.hip", "mx_gemm.hip", "attn8.hip", "attn_block.hip", "attn_ray.hip", "predict.hip", "conv3.hip", "conv3_stem.hip", "conv2.hip", "conv2_f8.hip", "conv2_f4.hip"] + ["conv3_f%d_o%d.hip" % (f, o) for f in (8, 4) for o in (8, 4, 0)]
HIPCC_FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-Wno-unused-value",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# per-file additions. attn8.hip: the attention core rescales its output accumulators on the vector pipe between two matrix products of every key
# tile; with the accumulators in ordinary vector registers (the kernel has room: one wavefront per SIMD) that is one multiply each instead of a
# read from and a write back to the accumulation registers around it
HIPCC_FILE_FLAGS = {"attn8.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def hipcc_cmd(src, obj):
    return ["hipcc"] + HIPCC_FLAGS + HIPCC_FILE_FLAGS.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj]


def _run(cmd, cwd=None):
    r = subprocess.run(cmd, cwd=cwd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_hip(verbose=False):
    objs = []
    procs = []
    for src in HIP_SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = hipcc_cmd(src, obj)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for cmd, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
        if verbose and out.strip():
            print(out)
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


HOST_LIB = os.path.join(ROOT, "ufsm_amd", "libufsm_host.so")


def build_host():
    """The C23 host layer (op dispatch + U-Net graph) over the C ABI of libufsm_lp.so."""
    src = [os.path.join(ROOT, "ufsm_amd", "host", f) for f in ("nn_host.c", "unet.c", "predict.c")]
    _run(["gcc", "-std=c2x", "-O2", "-Wall", "-Wextra", "-fPIC", "-shared", "-o", HOST_LIB] + src +
         ["-L" + os.path.dirname(LIB), "-lufsm_lp", "-Wl,-rpath,$ORIGIN", "-lm"])
    return HOST_LIB


def build_oracle():
    _run(["make", "-B", "liboracle.so"], cwd=ORACLE_DIR)
    return ORACLE_LIB


def build_all(verbose=False):
    build_oracle()
    build_hip(verbose)
    build_host()


if __name__ == "__main__":
    build_all(verbose=True)
    print("built", LIB, "and", ORACLE_LIB)
