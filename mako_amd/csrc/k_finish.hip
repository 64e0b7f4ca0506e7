// finish_kernel's variants: the second pass over the top_k == 0 rows.
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
namespace {
template <bool VEC, int KH, bool UNSORTED>
void launch_one(uint32_t wgs, hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices)
{
    hipLaunchKernelGGL((finish_kernel<VEC, KH, UNSORTED>), dim3(1, wgs), dim3(kThreads), kDynLds, st, d, sc, slices);
}
template <bool VEC, bool UNSORTED>
void launch_vec(int kh, uint32_t wgs, hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices)
{
    if (kh == 2)
        launch_one<VEC, 2, UNSORTED>(wgs, st, d, sc, slices);
    else if (kh == 8)
        launch_one<VEC, 8, UNSORTED>(wgs, st, d, sc, slices);
    else
        launch_one<VEC, 0, UNSORTED>(wgs, st, d, sc, slices);
}
} // namespace

void launch_finish(bool vec, int kh, bool unsorted, uint32_t wgs, hipStream_t st, const mako_sample_desc& d, const Scratch& sc,
                   uint32_t slices)
{
    if (vec && unsorted)
        launch_vec<true, true>(kh, wgs, st, d, sc, slices);
    else if (vec)
        launch_vec<true, false>(kh, wgs, st, d, sc, slices);
    else if (unsorted)
        launch_vec<false, true>(kh, wgs, st, d, sc, slices);
    else
        launch_vec<false, false>(kh, wgs, st, d, sc, slices);
}

hipError_t init_finish_kernels()
{
    const void* kernels[] = {(const void*)finish_kernel<true, 0, false>, (const void*)finish_kernel<false, 0, false>,
                             (const void*)finish_kernel<true, 2, false>, (const void*)finish_kernel<false, 2, false>,
                             (const void*)finish_kernel<true, 8, false>, (const void*)finish_kernel<false, 8, false>,
                             (const void*)finish_kernel<true, 0, true>,  (const void*)finish_kernel<false, 0, true>,
                             (const void*)finish_kernel<true, 2, true>,  (const void*)finish_kernel<false, 2, true>,
                             (const void*)finish_kernel<true, 8, true>,  (const void*)finish_kernel<false, 8, true>};
    for (const void* k : kernels) {
        const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDynLds);
        if (e != hipSuccess)
            return e;
    }
    return hipSuccess;
}
} // namespace mako
