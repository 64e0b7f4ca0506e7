// scan_kernel's variants: the only kernels that stream the logits.
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
namespace {
template <bool VEC, int KH, bool ABOVE>
void launch_one(dim3 grid, size_t lds, hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slice_len,
                uint32_t cus)
{
    hipLaunchKernelGGL((scan_kernel<VEC, KH, ABOVE>), grid, dim3(kThreads), lds, st, d, sc, slice_len, cus);
}
template <bool VEC, int KH>
void launch_kh(bool above, dim3 grid, size_t lds, hipStream_t st, const mako_sample_desc& d, const Scratch& sc,
               uint32_t slice_len, uint32_t cus)
{
    if (above)
        launch_one<VEC, KH, true>(grid, lds, st, d, sc, slice_len, cus);
    else
        launch_one<VEC, KH, false>(grid, lds, st, d, sc, slice_len, cus);
}
template <bool VEC>
void launch_vec(int kh, bool above, dim3 grid, size_t lds, hipStream_t st, const mako_sample_desc& d, const Scratch& sc,
                uint32_t slice_len, uint32_t cus)
{
    if (kh == 2)
        launch_kh<VEC, 2>(above, grid, lds, st, d, sc, slice_len, cus);
    else if (kh == 8)
        launch_kh<VEC, 8>(above, grid, lds, st, d, sc, slice_len, cus);
    else
        launch_kh<VEC, 0>(above, grid, lds, st, d, sc, slice_len, cus);
}
} // namespace

void launch_scan(bool vec, int kh, bool above, dim3 grid, size_t lds, hipStream_t st, const mako_sample_desc& d,
                 const Scratch& sc, uint32_t slice_len, uint32_t cus)
{
    if (vec)
        launch_vec<true>(kh, above, grid, lds, st, d, sc, slice_len, cus);
    else
        launch_vec<false>(kh, above, grid, lds, st, d, sc, slice_len, cus);
}

hipError_t init_scan_kernels()
{
    const void* kernels[] = {(const void*)scan_kernel<true, 0, false>, (const void*)scan_kernel<false, 0, false>,
                             (const void*)scan_kernel<true, 2, false>, (const void*)scan_kernel<false, 2, false>,
                             (const void*)scan_kernel<true, 8, false>, (const void*)scan_kernel<false, 8, false>,
                             (const void*)scan_kernel<true, 0, true>,  (const void*)scan_kernel<false, 0, true>,
                             (const void*)scan_kernel<true, 2, true>,  (const void*)scan_kernel<false, 2, true>,
                             (const void*)scan_kernel<true, 8, true>,  (const void*)scan_kernel<false, 8, true>};
    for (const void* k : kernels) {
        const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDynLds);
        if (e != hipSuccess)
            return e;
    }
    return hipSuccess;
}
} // namespace mako
