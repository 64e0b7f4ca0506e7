// How the second pass over the top_k == 0 rows is cut into pieces, and the list of those rows.
#pragma once

#include "sampler_common.h"

namespace mako {

// The batch's top_k == 0 rows, in row order, go to `work_rows`; returns into how many pieces second_kernel cuts each
// of them and how long a piece is.  A piece is one to four blocks of 4096 logits (a slice is four): as few blocks
// as keep all the pieces of the batch, and the workgroups that finish the batch's other rows beside them, within
// one round of workgroups (`cus` of them run at a time, one per CU), since the pass is bound by instruction issue
// and more workgroups with less work each finish sooner.  Worked out
// from the rows' parameters by one wave of scan_kernel's first workgroup and left in Scratch::work_n.
__device__ __forceinline__ uint32_t second_pass_pieces(const mako_sample_desc& d, uint32_t slices, uint32_t slice_len,
                                                       uint32_t cus, uint32_t* work_rows, uint32_t& piece_len,
                                                       uint32_t& busy, uint32_t& rows)
{
    const unsigned long long lower = (1ull << lane_id()) - 1ull;
    rows = 0;
    for (uint32_t base = 0; base < d.n_rows; base += kWave) {
        const uint32_t r = base + lane_id();
        const bool nucleus = r < d.n_rows && classify(d.params[r]) == kNucleus;
        const unsigned long long bal = __ballot(nucleus);
        if (nucleus)
            work_rows[rows + (uint32_t)__popcll(bal & lower)] = r;
        rows += (uint32_t)__popcll(bal);
    }
    piece_len = slice_len;
    busy = rows * slices;
    for (uint32_t blocks = 1; blocks < 4u; ++blocks) {
        const uint32_t len = blocks * 4096u;
        const uint32_t n = (d.n_vocab + len - 1u) / len;
        if (len < slice_len && n <= kMaxSlices && rows * n + (d.n_rows - rows) <= cus) {
            piece_len = len;
            busy = rows * n;
            return n;
        }
    }
    return slices;
}

} // namespace mako
