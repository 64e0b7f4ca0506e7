// Rows that a batch with wide nuclei finishes in tail_kernel's launch, beside the tails and on CUs that would
// otherwise idle: top-k rows, rows for the whole-row path, and narrow nuclei that the candidate lists could not
// certify.  Rare or long-running code, kept out of the kernels that many workgroups run.
#pragma once

#include "row_records.h"
#include "sorted_tail.h"
#include "topk_candidates.h"
#include "whole_row.h"

namespace mako {

// Second look at a narrow nucleus (plan flag 4, left by sort_kernel): the weights the second pass kept for the row
// (worker 0's share, unsorted) sorted, cut and drawn from; whatever that cannot settle goes to the whole-row path.
__device__ MAKO_RARE_CALL void narrow_second_look(const mako_sample_desc& d, const Scratch& sc, const mako_sampling_params& P,
                                                  uint32_t row, const FinishLds& L)
{
    assume_lds(L);
    BigPlan* plan = sc.plan + row;
    const uint32_t handed = plan->cursor[0], room = plan->cap[0], overflow = plan->overflow;
    const double total = plan->total64;
    const float m = plan->m;
    const uint32_t argidx = plan->argidx;
    __syncthreads();
    if (threadIdx.x == 0)
        plan->flag = 0;
    const uint32_t n0 = min(handed, d.n_vocab);
    if (handed <= room && !overflow) {
        if (n0 == 0) { // (nothing survived: sampler.cpp:36-38)
            fallback_row(d, row, argidx);
            return;
        }
        uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
        uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
        uint32_t* key1 = sc.key[1] + (size_t)row * sc.vpad;
        uint32_t* idx1 = sc.idx[1] + (size_t)row * sc.vpad;
        for (uint32_t i = threadIdx.x; i < n0; i += kThreads) {
            key0[i] = ~key1[i];
            idx0[i] = idx1[i];
        }
        __syncthreads();
        sort_segment(idx0, key0, idx1, key1, n0, L); // (stable sorts: token ids first, then the weights)
        sort_segment(key0, idx0, key1, idx1, n0, L);
        if (sorted_tail(d, row, P, key0, idx0, n0, true, total, MAKO_PATH_SORTED, L))
            return;
    }
    general_row<0>(d, sc, row, P, m, argidx, L);
}

// Rows that need no sampling: a forced token, the argmax of a greedy row.  Returns whether the row was one.  (Out of
// line: inlined beside the top-k rows' code it costs that code registers.)
__device__ MAKO_RARE_CALL bool late_plain_row(const mako_sample_desc& d, const Scratch& sc, RowClass cls, uint32_t row,
                                              uint32_t slices)
{
    if (d.force_token || d.close_token) { // uniform
        int32_t ftok;
        uint32_t above;
        const uint32_t kind = row_forced(d, sc, row, slices, ftok, above);
        if (threadIdx.x == 0 && d.out_above)
            d.out_above[row] = above;
        if (kind != MAKO_FORCED_NONE) {
            // a token >= 0 is taken instead of sampling, and a draft is kept only if it matches (session.hpp:43-45)
            if (threadIdx.x == 0) {
                RowOut o;
                o.token = ftok;
                o.n_cand = 0;
                o.total = 0.0f;
                o.q = 0.0f;
                o.path = MAKO_PATH_FORCED;
                o.accepted = d.draft ? (d.draft[row] == ftok) : 0u;
                o.forced = kind;
                write_row(d, row, o);
            }
            return true;
        }
    }
    if (cls == kGreedy) { // sampler.cpp:77-78, 88-92
        float m;
        uint32_t argidx, n_cands, any_overflow;
        row_summary(sc, row, slices, m, argidx, n_cands, any_overflow);
        if (threadIdx.x == 0) {
            RowOut o;
            o.token = (int32_t)argidx;
            o.n_cand = 0;
            o.total = 0.0f;
            o.q = 0.0f;
            o.path = MAKO_PATH_GREEDY;
            o.accepted = d.draft ? (d.draft[row] == (int32_t)argidx) : 0u;
            write_row(d, row, o);
        }
        return true;
    }
    return false;
}

// What the earlier kernels leave of row `row`, by one workgroup (all threads call; sm.tab must hold the exp2 table):
// rows whose token is forced, greedy rows, top-k rows, rows for the whole-row path, second looks.
__device__ MAKO_RARE_CALL void finish_late_row(const mako_sample_desc& d, const Scratch& sc, const mako_sampling_params& P,
                                               uint32_t row, uint32_t slices, const FinishLds& L)
{
    assume_lds(L);
    const RowClass cls = classify(P);
    if ((d.force_token || d.close_token || cls == kGreedy) && late_plain_row(d, sc, cls, row, slices))
        return;
    if (cls == kGeneral && sc.plan[row].flag == kIndexClaimed) // (a row in token order that the kernels of index_rows.h finish)
        return;
    if (cls == kNucleus) {
        // (the flag is never set for a row whose token is forced: the second pass leaves such a row alone)
        const uint32_t flag = sc.plan[row].flag;
        if (flag == 4) {
            narrow_second_look(d, sc, P, row, L);
        } else if (flag == 2) { // the whole-row path
            const float m = sc.plan[row].m;
            const uint32_t argidx = sc.plan[row].argidx;
            __syncthreads();
            if (threadIdx.x == 0)
                sc.plan[row].flag = 0;
            general_row<0>(d, sc, row, P, m, argidx, L);
        }
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
