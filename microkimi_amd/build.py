"""Builds libmk_hip.so (gfx950 code objects + the C-ABI host layer) in-tree with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmk_hip.so")
SOURCES = ["host.hip", "codec.hip", "gemv_mxfp4.hip", "gemv_q8.hip", "moe.hip", "moe_persist.hip", "mla.hip", "mla_heads.hip", "gemm_mxfp4.hip", "gemm_q8x.hip", "prefill.hip", "front.hip", "weights.hip", "vq1.hip", "quantize.hip"]


def hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    return "hipcc"


def build(verbose=False):
    """Compile every HIP source for gfx950 and link the shared library."""
    cmd = [hipcc(), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wno-unused-value", "-fno-strict-aliasing",
           # wrong results have been seen from compiler-formed packed-f32 ops on this target: keep them off
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-DMK_BUILD=1"]
    cmd += [os.path.join(CSRC, s) for s in SOURCES]
    cmd += ["-o", LIB]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
