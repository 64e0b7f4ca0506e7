// tail_kernel: the wide rows' cut, total and draw.
#pragma once

#include "sorted_tail.h"
#include "late_rows.h"

namespace mako {

#ifdef MAKO_EMIT_TAIL_KERNEL
// grid = (1, rows).  Rows whose sorted list sort_kernel's workers have prepared: top-p cut, exact total, draw.
// (The context's record by value: with a pointer to it the first loads would have to wait for a trip to memory.  The
// list's length and this workgroup's entry are asked for together, then everything the row's plan holds.)
// Workgroups from tail_cap on: workgroup tail_cap + r finishes what the kernels before it left of row r, beside the
// few long tails, on CUs that would otherwise idle.  Top-k rows are finished in line; everything rarer
// (finish_late_row()) is called out of line: inlined as well, it made this kernel's chains compile to slower code.
// (With the top-k rows in line the compiler would make a called function of the wide rows' sorted tail instead,
// which costs them 2 us: that call is forced in line below.)
// UNSORTED: the instance for batches whose plans may have left shares unsorted (unsorted_shares.h; a translation unit of its
// own, k_tail_unsorted.hip).
template <bool UNSORTED>
__device__ __forceinline__ void tail_body(const mako_sample_desc& d_arg, const Scratch& sc_val, uint32_t slices, uint32_t tail_cap)
{
    const Scratch& sc_arg = sc_val;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
#ifdef MAKO_TIMING_TAIL
    MAKO_WG_TIMER;
#endif
    if (blockIdx.y >= tail_cap) {
        const uint32_t r = blockIdx.y - tail_cap;
        if (r >= d_arg.n_rows)
            return;
        MAKO_ROW(kNone);
        // (the arguments' copy for LDS, the row's parameters, the exp2 table, the candidate slots and the slices'
        // records are asked for before anything is waited for)
        const uint64_t tab_word = k_exp2_tab[threadIdx.x & 31u];
        ArgWords late_words;
        fetch_arg_words(d_arg, sc_arg, late_words);
        fetch_param_words(d_arg, r, late_words);
        // (a top_k == 0 row has no use for its candidate slots: a look at the row's top_k first, which costs the
        // others a trip they have time for beside the long tails)
        CandSlots pre;
        const bool covered = slots_cover(slices) && d_arg.params[r].top_k != 0u; // uniform
        if (covered)
            fetch_candidate_slots(sc_arg, r, slices, pre);
        const SliceStat lane_stat = load_slice_stat(sc_arg.stats, (size_t)r * kMaxSlices + min((uint32_t)lane_id(), slices - 1u));
        place_arg_words(late_words, s_args);
        if (threadIdx.x < 32)
            sm.tab[threadIdx.x] = tab_word;
        lds_barrier(); // (publishes the copy and the table; the loads above stay in flight)
        const RowClass late_cls = classify(s_args.P);
        const bool plain = d_arg.force_token || d_arg.close_token; // uniform
        // (a top_k == 0 row that the workers and the tail above take care of needs nothing here)
        if (late_cls == kNucleus && !plain) {
            const uint32_t late_flag = sc_arg.plan[r].flag;
            if (late_flag != 2 && late_flag != 4)
                return;
        }
        // A top-k row is finished here, in line: there are dozens of them beside a few long tails, and through the
        // call below (whose entry and the entries of what it calls store dozens of registers per thread) each took
        // longer than the longest tail.
        if (late_cls == kTopK && !plain && !d_arg.draft && covered) {
            float m;
            uint32_t argidx, n_cands, any_overflow;
            row_summary_of(lane_stat, slices, m, argidx, n_cands, any_overflow);
            if (!topk_takes_whole_row(late_cls, any_overflow, n_cands)) {
                topk_row(s_args.d, s_args.sc, r, slices, s_args.P, m, argidx, n_cands, lane_stat,
                         finish_lds_views(sm, s_dyn64), true, pre);
                return;
            }
        }
        // (the views handed on by reference live in scratch memory, 32 bytes per thread: made here, where only the
        // rows that take the call store them)
        const FinishLds late_views = finish_lds_views(sm, s_dyn64);
        finish_late_row(s_args.d, s_args.sc, s_args.P, r, slices, late_views);
        return;
    }
    // (two trips to memory before the list's records are asked for: the work list's entry with the arguments' copy
    // for LDS, then the row's plan with its parameters; the empty asm statements keep each trip's loads together)
    const uint32_t tid = threadIdx.x;
    ArgWords arg_words;
    fetch_arg_words(d_arg, sc_arg, arg_words);
    const uint32_t n_work = sc_arg.work_n[1];
    const uint32_t row = sc_arg.work_tail[blockIdx.y]; // (the list has room for every workgroup)
    asm volatile("" ::"s"(row), "s"(n_work), "v"(arg_words.d), "v"(arg_words.sc));
    if (blockIdx.y >= n_work)
        return;
    MAKO_ROW(row);
    const BigPlan* planned = sc_arg.plan + row;
    const uint32_t flag = planned->flag, plan_n0 = planned->n0, plan_groups = planned->groups;
    const double total64 = planned->total64;
    const float plan_m = planned->m;
    const uint32_t plan_argidx = planned->argidx;
    fetch_param_words(d_arg, row, arg_words);
    asm volatile("" ::"s"(flag), "s"(plan_n0), "s"(plan_groups), "v"(arg_words.p));
    if (flag != 1)
        return;
    place_arg_words(arg_words, s_args);
    __syncthreads();
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    BigPlan* plan = sc.plan + row;
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;
    L.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);
    const uint32_t n0 = min(plan_n0, d.n_vocab), groups = min(plan_groups, min(kMaxGroups, sc.g_cap));
    __syncthreads();
    if (tid == 0)
        plan->flag = 0;
    const uint32_t* kf = sc.key[0] + (size_t)row * sc.vpad;
    const uint32_t* jf = sc.idx[0] + (size_t)row * sc.vpad;
    // (in line whatever the compiler makes of the kernel's size: as a called function the wide rows' chains would
    // start by storing registers)
    MAKO_CHECK(sc, kCheckTailGroup, plan_n0 <= d.n_vocab && plan_groups <= min(kMaxGroups, sc.g_cap));
    bool done;
    [[clang::always_inline]] done = sorted_tail<true, false, false, UNSORTED>(d, row, s_args.P, kf, jf, n0, true, total64, MAKO_PATH_SORTED,
                                                                              L, false, 0.0f, sc.gt, (size_t)row * sc.g_cap, groups);
    if (done)
        return;
    // too close to call, or the list ends before the nucleus does: the whole-row path decides
    __syncthreads();
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    __syncthreads();
    general_row<0>(d, sc, row, s_args.P, plan_m, plan_argidx, L);
}
#ifdef MAKO_TAIL_UNSORTED
__global__ __launch_bounds__(kThreads) void tail_kernel_unsorted(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices, uint32_t tail_cap)
{
    tail_body<true>(d_arg, sc_val, slices, tail_cap);
}
#else
__global__ __launch_bounds__(kThreads) void tail_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices, uint32_t tail_cap)
{
    tail_body<false>(d_arg, sc_val, slices, tail_cap);
}
#endif
#endif // MAKO_EMIT_TAIL_KERNEL

} // namespace mako
