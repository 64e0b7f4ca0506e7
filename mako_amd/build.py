"""Builds libmako_sampler.so (HIP, gfx950) in-tree with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "csrc", "mako_sampler.hip")
OUT = os.path.join(HERE, "libmako_sampler.so")

# Bit-exactness against the host toolchain needs: no FMA contraction, IEEE fp32
# division, subnormals kept.  Packed-fp32 instructions stay off.
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-gpu-flush-denormals-to-zero",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # every device function inlined into its kernel: no call stack, so the finishing kernels need no
    # scratch memory (kernels that use scratch run far fewer workgroups at a time on this chip)
    "-mllvm", "-amdgpu-function-calls=false",
    "-Wall",
    "-Wno-unused-command-line-argument",
]


def build(verbose=False, extra=()):
    cmd = ["hipcc", *FLAGS, *extra, SRC, "-o", OUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return OUT


if __name__ == "__main__":
    build(verbose=True, extra=sys.argv[1:])
