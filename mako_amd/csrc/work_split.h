// How the second pass over the top_k == 0 rows is cut into pieces, and which piece a workgroup serves.
#pragma once

#include "sampler_common.h"

namespace mako {

// How finish_kernel cuts each top_k == 0 row into pieces, and how many workgroups share a row's pieces.  A piece is
// one to four blocks of 4096 logits (a slice is four): as few blocks as keep all the pieces of the batch within one
// round of workgroups (`cus` of them run at a time, one per CU), since the pass is bound by instruction issue and
// more workgroups with less work each finish sooner.  A batch with more pieces than that takes whole slices, and as
// many workgroups per row as keeps it to one round; each of them goes through its share of the row's pieces in turn
// (and builds the row's plan once, not once per piece).  Worked out from the rows' parameters by one wave of
// scan_kernel's first workgroup and left in Scratch::work_n.
struct SecondPassCut {
    uint32_t per_row;   // workgroups per top_k == 0 row
    uint32_t piece_len;
    uint32_t busy;      // workgroups with work
    uint32_t pieces;    // pieces per row: workgroup g of a row takes the pieces g, g + per_row, ...
};
// finish_grid: the workgroups finish_kernel is launched with (second_pass_grid()).
__device__ __forceinline__ SecondPassCut second_pass_cut(const mako_sample_desc& d, uint32_t slices, uint32_t slice_len,
                                                         uint32_t cus, uint32_t finish_grid)
{
    uint32_t rows = 0; // top_k == 0 rows of the batch (every lane ends up with the count)
    for (uint32_t base = 0; base < d.n_rows; base += (uint32_t)kWave) {
        const uint32_t r = base + (uint32_t)lane_id();
        rows += (uint32_t)__popcll(__ballot(r < d.n_rows && classify(d.params[r]) == kNucleus));
    }
    SecondPassCut cut;
    cut.piece_len = slice_len;
    cut.pieces = slices;
    for (uint32_t blocks = 1; blocks < 4u; ++blocks) {
        const uint32_t len = blocks * 4096u;
        const uint32_t n = (d.n_vocab + len - 1u) / len;
        if (len < slice_len && n <= kMaxSlices && rows * n <= cus) {
            cut.piece_len = len;
            cut.pieces = n;
            break;
        }
    }
    // (more pieces than one round of workgroups: as many workgroups per row as the grid allows when the rows are dealt
    // to the XCDs eight at a time, see finish_kernel)
    cut.per_row = rows * cut.pieces <= cus ? cut.pieces : min(cut.pieces, max(1u, finish_grid / ((max(rows, 1u) + 7u) & ~7u)));
    cut.busy = rows * cut.per_row;
    return cut;
}

// Workgroups finish_kernel is launched with (a multiple of eight, at least a workgroup per row): one round's worth, or
// two where the batch is expected to have more top_k == 0 rows than half a round: the CUs whose rows need little then
// take on the second halves of those that need much (a near-flat row takes twice as long as a peaked one).  On small
// batches the workgroups without work, which can only start once a CU is free, would lengthen the kernel instead.
__host__ __device__ inline uint32_t second_pass_grid(uint32_t n_rows, uint32_t nucleus_rows, uint32_t cus)
{
    const uint32_t rows8 = (n_rows + 7u) & ~7u, rounds = 2u * nucleus_rows >= cus ? 2u : 1u;
    return rows8 > rounds * cus ? rows8 : (rounds * cus + 7u) & ~7u;
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
