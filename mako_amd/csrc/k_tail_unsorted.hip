// tail_kernel for batches whose plans may have left shares unsorted (a translation unit of its own: the usual
// instance's code is then what it was without this one).
#define MAKO_EMIT_TAIL_KERNEL
#define MAKO_TAIL_UNSORTED
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
void launch_tail_unsorted(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t tail_cap)
{
    hipLaunchKernelGGL(tail_kernel_unsorted, dim3(1, tail_cap + d.n_rows), dim3(kThreads), kTailLds, st, d, sc, slices, tail_cap);
}

hipError_t init_tail_unsorted()
{
    return hipFuncSetAttribute((const void*)tail_kernel_unsorted, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kTailLds);
}
} // namespace mako
