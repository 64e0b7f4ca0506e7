// sort_kernel for batches whose plans leave shares unsorted (a translation unit of its own: the usual instance's
// code is then what it was without this one).
#define MAKO_EMIT_SORT_KERNELS
#define MAKO_SORT_UNSORTED
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
void launch_sort_unsorted(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t grid_rows)
{
    // (the three regions of large_batch_lists() are sized by the batch's rows)
    (void)grid_rows;
    hipLaunchKernelGGL(sort_kernel_unsorted, dim3(kSortItemsPerRow, d.n_rows), dim3(kThreads), kSortLds, st, d, sc, slices);
}

hipError_t init_sort_unsorted()
{
    return hipFuncSetAttribute((const void*)sort_kernel_unsorted, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSortLds);
}
} // namespace mako
