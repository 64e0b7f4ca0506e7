// The kernels of the rows whose candidates stay in token order (index_rows.h): a translation unit of their own.
#define MAKO_EMIT_INDEX_KERNELS
#include "launch.h"
#include "sampler_kernels.h"

namespace mako {
namespace {
template <bool VEC>
void launch_weights(int kh, dim3 grid, hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices)
{
    if (kh == 2)
        hipLaunchKernelGGL((index_weights_kernel<VEC, 2>), grid, dim3(kThreads), kDynLds, st, d, sc, slices);
    else if (kh == 8)
        hipLaunchKernelGGL((index_weights_kernel<VEC, 8>), grid, dim3(kThreads), kDynLds, st, d, sc, slices);
    else
        hipLaunchKernelGGL((index_weights_kernel<VEC, 0>), grid, dim3(kThreads), kDynLds, st, d, sc, slices);
}
} // namespace

void launch_index_weights(bool vec, int kh, hipStream_t st, const mako_sample_desc& d, const Scratch& sc, uint32_t slices)
{
    const dim3 grid((d.n_vocab + kSliceMax - 1u) / kSliceMax, d.n_rows);
    if (vec)
        launch_weights<true>(kh, grid, st, d, sc, slices);
    else
        launch_weights<false>(kh, grid, st, d, sc, slices);
}

void launch_index_finish(hipStream_t st, const mako_sample_desc& d, const Scratch& sc, bool in_order_rows)
{
    // (the group records are for rows in token order only: a workgroup per 16 384 entries where the rows fill the chip
    // anyway, per 4 096 on a small batch)
    if (in_order_rows && (uint64_t)d.n_rows * ((d.n_vocab + kSliceMax - 1u) / kSliceMax) >= 256u)
        hipLaunchKernelGGL(index_groups_kernel<4u>, dim3((d.n_vocab + kSliceMax - 1u) / kSliceMax, d.n_rows), dim3(kThreads), 0, st, d, sc);
    else if (in_order_rows)
        hipLaunchKernelGGL(index_groups_kernel<1u>, dim3((d.n_vocab + kIndexBlock - 1u) / kIndexBlock, d.n_rows), dim3(kThreads), 0, st, d, sc);
    hipLaunchKernelGGL(index_tail_kernel, dim3(1, d.n_rows), dim3(kThreads), kTailLds, st, d, sc);
}

hipError_t init_index_kernels()
{
    const void* kernels[] = {(const void*)index_weights_kernel<true, 0>,  (const void*)index_weights_kernel<true, 2>,
                             (const void*)index_weights_kernel<true, 8>,  (const void*)index_weights_kernel<false, 0>,
                             (const void*)index_weights_kernel<false, 2>, (const void*)index_weights_kernel<false, 8>};
    for (const void* k : kernels) {
        const hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kDynLds);
        if (e != hipSuccess)
            return e;
    }
    return hipFuncSetAttribute((const void*)index_tail_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kTailLds);
}
} // namespace mako
