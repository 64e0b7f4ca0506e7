// tail_kernel: top-p cut, exact total and draw of the wide rows.
#define MAKO_EMIT_TAIL_KERNEL
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
void launch_tail_unsorted(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t tail_cap);

void launch_tail(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t tail_cap, bool unsorted)
{
    if (unsorted)
        launch_tail_unsorted(st, d, sc, slices, tail_cap);
    else
        hipLaunchKernelGGL(tail_kernel, dim3(1, tail_cap + d.n_rows), dim3(kThreads), kTailLds, st, d, sc, slices, tail_cap);
}

hipError_t init_tail_unsorted();
hipError_t init_tail_kernels()
{
    const hipError_t e = hipFuncSetAttribute((const void*)tail_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kTailLds);
    return e != hipSuccess ? e : init_tail_unsorted();
}
} // namespace mako
