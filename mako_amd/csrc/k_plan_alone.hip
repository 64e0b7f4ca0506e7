// plan_kernel: the last kernel of a batch without top_k == 0 or whole-row rows: a row that cannot be
// certified is given the whole-row path here.
#define MAKO_EMIT_PLAN_KERNEL
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
void launch_plan_alone(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices)
{
    hipLaunchKernelGGL(plan_kernel, dim3(1, d.n_rows), dim3(kThreads), kTailLds, st, d, sc, slices);
}

hipError_t init_plan_alone()
{
    return hipFuncSetAttribute((const void*)plan_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kTailLds);
}
} // namespace mako
