"""Builds libcntk_amd_quantizer.so (HIP, gfx950) in-tree with hipcc. Run: python -m cntk_amd.build"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libcntk_amd_quantizer.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # the CPU reference never fuses multiply-add; bit-exact codes and residuals need the same here
    "-ffp-contract=off",
    # no packed fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build_library(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    src = os.path.join(HERE, "csrc", "quantizer_api.hip")
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", LIB_PATH, src]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature and says so; that warning is harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
