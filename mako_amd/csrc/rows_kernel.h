// Rows that need no second pass: forced, greedy and top-k rows, finished by one workgroup each from the records
// scan_kernel left.
#pragma once

#include "topk_candidates.h"

namespace mako {

// One workgroup finishes row `row`: a forced token is written; a greedy row takes its argmax; a top-k row is
// resolved from the candidate lists.  A top_k == 0 row is only looked at for a forced token: its weights take the
// second pass and sort_kernel.  (sm.tab must hold the exp2 table; all threads call.)
// A row that needs the whole-row path is given it here (general_row<SITE>; SITE 1 leaves out the order of top-k without
// top-p, for batches whose host copy of the parameters shows a top-p on every sampled row).
#ifndef MAKO_ROWS_CALL
#define MAKO_ROWS_CALL __forceinline__
#endif
template <int SITE>
__device__ MAKO_ROWS_CALL void finish_row(const mako_sample_desc& d, const Scratch& sc, const mako_sampling_params& P,
                                           uint32_t row, uint32_t slices, const FinishLds& L)
{
    const uint32_t tid = threadIdx.x;
    const RowClass cls = classify(P);
    MAKO_STAMP(0);
    if (d.force_token || d.close_token) { // uniform
        int32_t ftok;
        uint32_t above;
        const uint32_t kind = row_forced(d, sc, row, slices, ftok, above);
        if (tid == 0 && d.out_above)
            d.out_above[row] = above;
        if (kind != MAKO_FORCED_NONE) {
            // a token >= 0 is taken instead of sampling, and a draft is kept only if it matches (session.hpp:43-45)
            if (tid == 0) {
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
            return;
        }
    }
    if (cls == kNucleus)
        return;
    // a top-k row's candidates are asked for together with the slices' records
    CandSlots pre;
    const bool prefetched = cls == kTopK && !d.draft && slots_cover(slices); // uniform
    if (prefetched)
        fetch_candidate_slots(sc, row, slices, pre);
    float m;
    uint32_t argidx, n_cands, any_overflow;
    SliceStat lane_stat;
    row_summary(sc, row, slices, m, argidx, n_cands, any_overflow, &lane_stat);
    MAKO_STAMP(1);
    if (cls == kGreedy) { // sampler.cpp:77-78, 88-92
        if (tid == 0) {
            RowOut o;
            o.token = (int32_t)argidx;
            o.n_cand = 0;
            o.total = 0.0f;
            o.q = 0.0f;
            o.path = MAKO_PATH_GREEDY;
            o.accepted = d.draft ? (d.draft[row] == (int32_t)argidx) : 0u;
            write_row(d, row, o);
        }
        return;
    }
    if (topk_takes_whole_row(cls, any_overflow, n_cands)) {
        general_row<SITE>(d, sc, row, P, m, argidx, L);
        return;
    }
    topk_row<SITE>(d, sc, row, slices, P, m, argidx, n_cands, lane_stat, L, prefetched, pre);
}

// grid = rows workgroups: batches without top_k == 0 rows (the host's copy of the parameters says so).
template <int SITE>
__global__ __launch_bounds__(kThreads) void rows_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    const Scratch& sc_arg = sc_val;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t row = blockIdx.x;
    const uint32_t tid = threadIdx.x;
#ifdef MAKO_TIMING_PLAN
    MAKO_WG_TIMER;
#endif
    MAKO_ROW(row);
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    stage_args(d_arg, sc_arg, row, s_args); // (its barrier publishes the table too)
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;
    L.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);
    finish_row<SITE>(s_args.d, s_args.sc, s_args.P, row, slices, L);
}

} // namespace mako
