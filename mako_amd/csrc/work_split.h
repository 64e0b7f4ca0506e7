// How the second pass over the top_k == 0 rows is cut into pieces, and which piece a workgroup serves.
#pragma once

#include "sampler_common.h"

namespace mako {

// Into how many pieces finish_kernel cuts each top_k == 0 row, and how long a piece is.  A piece is one to four
// blocks of 4096 logits (a slice is four): as few blocks as keep all the pieces of the batch within one round of
// workgroups (`cus` of them run at a time, one per CU), since the pass is bound by instruction issue and more
// workgroups with less work each finish sooner.  Worked out from the rows' parameters by one wave of scan_kernel's
// first workgroup and left in Scratch::work_n; batches of more than 64 rows take whole slices.
__device__ __forceinline__ uint32_t second_pass_pieces(const mako_sample_desc& d, uint32_t slices, uint32_t slice_len,
                                                       uint32_t cus, uint32_t& piece_len, uint32_t& busy)
{
    piece_len = slice_len;
    busy = d.n_rows * slices; // (no more than that)
    if (d.n_rows > (uint32_t)kWave)
        return slices;
    const uint32_t r = lane_id();
    const bool nucleus = r < d.n_rows && classify(d.params[r]) == kNucleus;
    const uint32_t rows = (uint32_t)__popcll(__ballot(nucleus));
    busy = rows * slices;
    for (uint32_t blocks = 1; blocks < 4u; ++blocks) {
        const uint32_t len = blocks * 4096u;
        const uint32_t n = (d.n_vocab + len - 1u) / len;
        if (len < slice_len && n <= kMaxSlices && rows * n <= cus) {
            piece_len = len;
            busy = rows * n;
            return n;
        }
    }
    return slices;
}

// Which piece of work does workgroup `piece` of finish_kernel (per_nucleus = slices, per_other = 1) or of plan_kernel
// (1, 0) serve?  Rows are taken in order, each contributing per_nucleus pieces if it is a top_k == 0 row and
// per_other otherwise.  Every workgroup works this out for itself from the rows' parameters (a few loads and one
// scan).  Returns false when there is no such piece; all threads receive the same answer.
__device__ bool find_piece(const mako_sample_desc& d, uint32_t piece, uint32_t per_nucleus, uint32_t per_other,
                           uint32_t& row, uint32_t& sub, BlockScratch& bs)
{
    const uint32_t tid = threadIdx.x;
    if (d.n_rows <= (uint32_t)kWave) {
        // up to 64 rows: every wave works it out for itself, one row per lane, without a barrier
        const uint32_t r = lane_id();
        uint32_t pieces = 0;
        if (r < d.n_rows)
            pieces = classify(d.params[r]) == kNucleus ? per_nucleus : per_other;
        const uint32_t upto = __ockl_wfscan_add_u32(pieces, true);
        const unsigned long long bal = __ballot(piece >= upto - pieces && piece < upto);
        if (bal == 0ull)
            return false;
        const int owner = __ffsll((long long)bal) - 1;
        row = (uint32_t)owner;
        sub = piece - (uint32_t)__builtin_amdgcn_readlane((int)(upto - pieces), owner);
        return true;
    }
    uint32_t before = 0;
    for (uint32_t base = 0; base < d.n_rows; base += kThreads) {
        const uint32_t r = base + tid;
        uint32_t pieces = 0;
        if (r < d.n_rows)
            pieces = classify(d.params[r]) == kNucleus ? per_nucleus : per_other;
        uint32_t tot;
        const uint32_t at = before + block_excl_scan_u32(pieces, tot, bs);
        if (piece >= at && piece < at + pieces)
            bs.bcast = ((unsigned long long)r << 32) | (unsigned long long)(piece - at);
        before += tot;
        if (piece < before) { // uniform
            __syncthreads();
            const unsigned long long v = bs.bcast;
            __syncthreads();
            row = (uint32_t)(v >> 32);
            sub = (uint32_t)v;
            return true;
        }
    }
    return false;
}

} // namespace mako
