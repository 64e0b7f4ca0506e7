// The batch's top_k == 0 rows, listed for the kernels behind the scan.
#pragma once

#include "sampler_common.h"

namespace mako {

// The batch's top_k == 0 rows, in row order, go to `work_rows`; returns how many there are.  One wave of scan_kernel's
// first workgroup works them out from the rows' parameters.
__device__ __forceinline__ uint32_t nucleus_rows(const mako_sample_desc& d, uint32_t* work_rows)
{
    const unsigned long long lower = (1ull << lane_id()) - 1ull;
    uint32_t rows = 0;
    for (uint32_t base = 0; base < d.n_rows; base += kWave) {
        const uint32_t r = base + lane_id();
        const bool nucleus = r < d.n_rows && classify(d.params[r]) == kNucleus;
        const unsigned long long bal = __ballot(nucleus);
        if (nucleus)
            work_rows[rows + (uint32_t)__popcll(bal & lower)] = r;
        rows += (uint32_t)__popcll(bal);
    }
    return rows;
}

} // namespace mako
