// sort_kernel: the wide rows' shares sorted by their workers; narrow nuclei finished by one worker.
#define MAKO_EMIT_SORT_KERNELS
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
void launch_sort_unsorted(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t grid_rows);

void launch_sort(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices, uint32_t grid_rows, bool unsorted)
{
    if (unsorted)
        launch_sort_unsorted(st, d, sc, slices, grid_rows);
    else
        hipLaunchKernelGGL(sort_kernel, dim3(kWorkers, grid_rows), dim3(kThreads), kSortLds, st, d, sc, slices);
}

hipError_t init_sort_unsorted();
hipError_t init_sort_kernels()
{
    static_assert(kSortLds >= kTailLds, "sort_kernel's tail uses the finishing kernels' LDS layout");
    const hipError_t e = hipFuncSetAttribute((const void*)sort_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSortLds);
    return e != hipSuccess ? e : init_sort_unsorted();
}
} // namespace mako
