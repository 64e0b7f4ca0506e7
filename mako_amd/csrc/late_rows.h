// Rows that a batch with wide nuclei finishes in tail_kernel's launch, beside the tails and on CUs that would
// otherwise idle: top-k rows, rows for the whole-row path, and narrow nuclei that the candidate lists could not
// certify.  Rare or long-running code, kept out of the kernels that many workgroups run.
#pragma once

#include "row_records.h"
#include "sorted_tail.h"
#include "topk_candidates.h"
#include "whole_row.h"

namespace mako {

// Second look at a narrow nucleus (plan flag 4, left by sort_kernel): the row's weights at or above the plan's
// threshold, from its bits(q) array, sorted, cut and drawn from.
__device__ MAKO_RARE_CALL void narrow_second_look(const mako_sample_desc& d, const Scratch& sc, const mako_sampling_params& P,
                                                  uint32_t row, const FinishLds& L)
{
    FinishShared& sm = *L.sm;
    BigPlan* plan = sc.plan + row;
    const uint32_t n0 = min(plan->n0, d.n_vocab), thr_bits = plan->thr;
    double total = plan->total64;
    __syncthreads();
    if (threadIdx.x == 0)
        plan->flag = 0;
    const uint32_t* qk = reinterpret_cast<const uint32_t*>(sc.wbuf + (size_t)row * sc.vpad);
    uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
    uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
    uint32_t* key1 = sc.key[1] + (size_t)row * sc.vpad;
    uint32_t* idx1 = sc.idx[1] + (size_t)row * sc.vpad;
    gather_range(qk, d.n_vocab, thr_bits, 0x7f800001u, key0, idx0, n0, sm);
    sort_segment(key0, idx0, key1, idx1, n0, L);
    if (sorted_tail(d, row, P, key0, idx0, n0, true, total, MAKO_PATH_GENERAL, L))
        return;
    // too close to call: the reference's total decides (index order over the row's bits(q) array; the zeros of the
    // logits that are no candidates add nothing).  The list reaches far enough below the cut for it: plan_nucleus()
    // takes the band along.
    total = reference_total([=](uint32_t i) { return __uint_as_float(qk[i]); }, d.n_vocab, sm);
    sorted_tail_exact(d, row, P, key0, idx0, n0, total, MAKO_PATH_GENERAL, L);
}

// What plan_kernel<false> leaves of row `row`, by one workgroup (all threads call; sm.tab must hold the exp2 table).
__device__ MAKO_RARE_CALL void finish_late_row(const mako_sample_desc& d, const Scratch& sc, const mako_sampling_params& P,
                                               uint32_t row, uint32_t slices, const FinishLds& L)
{
    const RowClass cls = classify(P);
    if (cls == kGreedy)
        return;
    if (cls == kNucleus) {
        // (the flag is never set for a row whose token is forced: plan_kernel returns before planning)
        const uint32_t flag = sc.plan[row].flag;
        if (flag == 4) {
            narrow_second_look(d, sc, P, row, L);
        } else if (flag == 2) { // a nucleus too long for the workers' group records: the whole-row path
            const float m = (float)sc.plan[row].total64;
            const uint32_t argidx = sc.plan[row].n0;
            __syncthreads();
            if (threadIdx.x == 0)
                sc.plan[row].flag = 0;
            general_row<0>(d, sc, row, P, m, argidx, L);
        }
        return;
    }
    if (d.force_token || d.close_token) { // uniform
        int32_t ftok;
        uint32_t above;
        if (row_forced(d, sc, row, slices, ftok, above) != MAKO_FORCED_NONE)
            return;
    }
    CandSlots pre;
    const bool prefetched = cls == kTopK && !d.draft && slots_cover(slices); // uniform
    if (prefetched)
        fetch_candidate_slots(sc, row, slices, pre);
    float m;
    uint32_t argidx, n_cands, any_overflow;
    SliceStat lane_stat;
    row_summary(sc, row, slices, m, argidx, n_cands, any_overflow, &lane_stat);
    if (topk_takes_whole_row(cls, any_overflow, n_cands))
        general_row<0>(d, sc, row, P, m, argidx, L);
    else
        topk_row(d, sc, row, slices, P, m, argidx, n_cands, lane_stat, L, prefetched, pre);
}

} // namespace mako
