// plan_kernel: one workgroup per row of a batch that needs neither the second pass nor the sort.
#pragma once

#include "topk_candidates.h"

namespace mako {

#ifdef MAKO_EMIT_PLAN_KERNEL // (not a template: defined by the one translation unit that launches it)
// grid = (1, rows), one workgroup per row, for a batch without top_k == 0 rows and without rows that need the
// whole-row path (the host saw none in its copy of the parameters): such a batch ends here.  Rows whose token is
// forced, greedy rows and top-k rows are finished from the records scan_kernel left; a row that turns out to need
// the whole-row path after all is given it here.
__global__ __launch_bounds__(kThreads) void plan_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    const Scratch& sc_arg = sc_val; // (by value: where the row's records are is known without a trip to memory)
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t row = blockIdx.y;
    const uint32_t tid = threadIdx.x;
#ifdef MAKO_TIMING_PLAN
    MAKO_WG_TIMER;
#endif
    MAKO_ROW(row);
    // Two trips to memory before the row's candidates are here, not three: the arguments' copy for LDS, the row's
    // parameters and the exp2 table go out first; the candidate slots and the slices' records as soon as the context's
    // record says where they are (whatever the row turns out to be: a greedy row's are never looked at); the copy is
    // put in LDS under them.
    const uint64_t tab_word = k_exp2_tab[tid & 31u];
    ArgWords arg_words;
    fetch_arg_words(d_arg, sc_arg, arg_words);
    fetch_param_words(d_arg, row, arg_words);
    CandSlots pre;
    const bool covered = slots_cover(slices); // uniform
    if (covered)
        fetch_candidate_slots(sc_arg, row, slices, pre);
    const SliceStat lane_stat = load_slice_stat(sc_arg.stats, (size_t)row * kMaxSlices + min((uint32_t)lane_id(), slices - 1u));
    place_arg_words(arg_words, s_args);
    if (tid < 32)
        sm.tab[tid] = tab_word;
    lds_barrier(); // (publishes the copy and the table; the loads above stay in flight)
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    const mako_sampling_params& P = s_args.P;
    const RowClass cls = classify(P);
    if (cls != kNucleus)
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
    const bool prefetched = covered && cls == kTopK && !d.draft; // uniform
    float m;
    uint32_t argidx, n_cands, any_overflow;
    row_summary_of(lane_stat, slices, m, argidx, n_cands, any_overflow);
    if (cls != kNucleus)
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

    // (a top_k == 0 row has no business here; should the host's copy of the parameters have hidden one, the whole-row
    // path serves it like any other)
    // (the views of the dynamic LDS block are made where they are handed on: those that a called function receives
    // by reference live in scratch memory, 32 bytes per thread, and only the rows that take the call should store them)
    if (cls == kNucleus || topk_takes_whole_row(cls, any_overflow, n_cands)) {
        const FinishLds views = finish_lds_views(sm, s_dyn64);
        general_row<1>(d, sc, row, P, m, argidx, views);
    } else {
        topk_row(d, sc, row, slices, P, m, argidx, n_cands, lane_stat, finish_lds_views(sm, s_dyn64), prefetched, pre);
    }
}
#endif // MAKO_EMIT_PLAN_KERNEL

} // namespace mako
