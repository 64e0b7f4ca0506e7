// rows_kernel's two variants: the finishing launch of a batch without top_k == 0 rows.
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
void launch_rows(bool any_general, hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices)
{
    if (any_general)
        hipLaunchKernelGGL((rows_kernel<0>), dim3(d.n_rows), dim3(kThreads), kDynLds, st, d, sc, slices);
    else
        hipLaunchKernelGGL((rows_kernel<1>), dim3(d.n_rows), dim3(kThreads), kDynLds, st, d, sc, slices);
}

hipError_t init_rows_kernels()
{
    hipError_t e = hipFuncSetAttribute((const void*)rows_kernel<0>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDynLds);
    if (e == hipSuccess)
        e = hipFuncSetAttribute((const void*)rows_kernel<1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDynLds);
    return e;
}
} // namespace mako
