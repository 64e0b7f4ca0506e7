"""Builds libmako_sampler.so (HIP, gfx950) in-tree with hipcc."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
# the C ABI, and one translation unit per kernel family (a kernel's register allocation then does not depend on
# which other kernels exist; they also compile side by side)
SOURCES = ["mako_sampler.hip", "k_scan.hip", "k_finish.hip", "k_plan_alone.hip", "k_sort.hip", "k_sort_unsorted.hip", "k_tail.hip", "k_tail_unsorted.hip", "k_index.hip"]
OBJ_DIR = os.path.join(HERE, "csrc", "_obj")
OUT = os.path.join(HERE, "libmako_sampler.so")
# the same library with the kernels' index checks compiled in (-DMAKO_CHECKED): for the test that runs the workloads
# under it and expects no check to fail; never the library that is benchmarked
OUT_CHECKED = os.path.join(HERE, "libmako_sampler_checked.so")

# Bit-exactness against the host toolchain needs: no FMA contraction, IEEE fp32
# division, subnormals kept.  Packed-fp32 instructions stay off.
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-fno-gpu-flush-denormals-to-zero",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-command-line-argument",
]
# Every device function inlined into its kernel: no call stack, so the kernel needs no scratch memory (kernels
# that use scratch run far fewer workgroups at a time on this chip).
INLINE_ALL = ["-mllvm", "-amdgpu-function-calls=false"]
# Per source (a source listed here is compiled WITHOUT INLINE_ALL): code that only rare rows reach is called, not
# inlined, where it would cost a hot path registers and spills.  Such kernels use scratch memory for the calls, which
# slows down the start of their workgroups: not for kernels that many workgroups run (sort_kernel: +15 %).
RARE_CALLS = ["-DMAKO_RARE_CALL=__attribute__((noinline))", "-DMAKO_REAL_CALLS=1"]
SOURCE_FLAGS = {
    # the rare late rows (the whole-row path, second looks at a cut) out of line beside the tails and the top-k rows
    "k_tail.hip": ["-DMAKO_TOPK_GENERAL_SITE=0", *RARE_CALLS],
    "k_tail_unsorted.hip": ["-DMAKO_TOPK_GENERAL_SITE=0", *RARE_CALLS],
    "k_index.hip": ["-DMAKO_TOPK_GENERAL_SITE=0", *RARE_CALLS],
    # the whole-row path and the second look at a cut that is too close to call, out of line beside the top-k rows
    "k_plan_alone.hip": RARE_CALLS,
}


# and the checked library with plans that leave shares unsorted which they should not (-DMAKO_RASH_PLANS, only
# finish_kernel differs): for the test that expects the oracle's results all the same, through rows given up to the
# whole-row path
OUT_RASH = os.path.join(HERE, "libmako_sampler_rash.so")


def build(verbose=False, extra=(), jobs=8, checked=False, rash=False):
    """rash=True needs the checked build's objects (build(checked=True) first)."""
    from concurrent.futures import ThreadPoolExecutor
    os.makedirs(OBJ_DIR, exist_ok=True)
    if checked or rash:
        extra = (*extra, "-DMAKO_CHECKED=1")

    def compile_one(name):
        mine = rash and name == "k_finish.hip"
        suffix = "_rash.o" if mine else ("_checked.o" if checked or rash else ".o")
        obj = os.path.join(OBJ_DIR, os.path.splitext(name)[0] + suffix)
        if rash and not mine:
            return obj # (the checked build's)
        cmd = ["hipcc", *FLAGS, *SOURCE_FLAGS.get(name, INLINE_ALL), *extra, *(["-DMAKO_RASH_PLANS=1"] if mine else []), "-c",
               os.path.join(CSRC, name), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    out = OUT_RASH if rash else (OUT_CHECKED if checked else OUT)
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    build(verbose=True, extra=sys.argv[1:])
    build(verbose=True, extra=sys.argv[1:], checked=True)
    build(verbose=True, extra=sys.argv[1:], rash=True)
