"""Builds libmrb.so (the HIP replay-buffer library) for gfx950 with hipcc, in-tree."""
import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB = os.path.join(CSRC, "libmrb.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # every float/double operation rounds once, in source order (bit-exact tree and weights)
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    # no packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wall",
]


def build(verbose=False):
    """Compile mindrl_amd/csrc/mrb.hip into mindrl_amd/csrc/libmrb.so. Returns the library path."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not os.path.exists(hipcc):
        hipcc = "hipcc"
    tmp = LIB + ".tmp"
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", tmp, os.path.join(CSRC, "mrb.hip")]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    noise = "is not a recognized feature for this target"
    out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
