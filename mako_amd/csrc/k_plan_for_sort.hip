// plan_kernel<false>: the batch goes on to sort_kernel, which has the whole-row path.
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
void launch_plan_for_sort(hipStream_t st, const mako_sample_desc& d, const Scratch* sc, uint32_t slices)
{
    hipLaunchKernelGGL((plan_kernel<false>), dim3(1, d.n_rows), dim3(kThreads), kDynLds, st, d, sc, slices);
}

hipError_t init_plan_for_sort()
{
    return hipFuncSetAttribute((const void*)plan_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDynLds);
}
} // namespace mako
