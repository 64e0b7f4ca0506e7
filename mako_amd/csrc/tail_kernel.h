// tail_kernel: the wide rows' cut, total and draw.
#pragma once

#include "sorted_tail.h"
#include "row_records.h"
#include "rows_kernel.h"
#include "whole_row.h"

namespace mako {

#ifdef MAKO_EMIT_TAIL_KERNEL
// grid = (1, rows).  The top_k == 0 rows, whose sorted lists sort_kernel's workers have prepared: top-p cut, exact
// total, draw.  The row's fp64 total of q is the sum of the second pass's pieces, added in piece order.
// (The batch's top-k rows were tried here too, beside the few long tails: this kernel's chains then compiled to
// slower code and lost twice what the other launch gained.)
// (The context's record by value: with a pointer to it the first loads would have to wait for a trip to memory.  The
// list's length and this workgroup's entry are asked for together, then everything known about the row.)
// Workgroups from tail_cap on: workgroup tail_cap + r finishes row r if it needs no second pass (finish_row(): forced,
// greedy and top-k rows), beside the few long tails, on CUs that would otherwise idle.  (That code is kept out of
// line: inlined, it made this kernel's chains compile to slower code.)
__global__ __launch_bounds__(kThreads) void tail_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices,
                                                        uint32_t tail_cap)
{
    const Scratch& sc_arg = sc_val;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t wg = blockIdx.x, tid = threadIdx.x;
    if (wg >= tail_cap) {
        const uint32_t r = wg - tail_cap;
        if (r >= d_arg.n_rows)
            return;
        if (tid < 32)
            sm.tab[tid] = k_exp2_tab[tid];
        stage_args(d_arg, sc_arg, r, s_args); // (its barrier publishes the table too)
        FinishLds Lr;
        Lr.sm = &sm;
        Lr.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
        Lr.sortk = s_dyn64;
        Lr.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);
        finish_row<0>(s_args.d, s_args.sc, s_args.P, r, slices, Lr);
        return;
    }
    const uint32_t n_work = sc_arg.work_n[1];
    const uint32_t pieces = min((d_arg.n_vocab + kPieceLen - 1u) / kPieceLen, sc_arg.pieces_cap);
    const uint32_t row = sc_arg.work_tail[wg]; // (the list has room for every workgroup below tail_cap)
    if (wg >= n_work || row >= d_arg.n_rows)
        return;
#ifdef MAKO_TIMING_TAIL
    MAKO_WG_TIMER;
#endif
    MAKO_ROW(row);
    const BigPlan* planned = sc_arg.plan + row;
    const uint32_t flag = planned->flag, plan_n0 = planned->n0, plan_groups = planned->groups, thr_bits = planned->thr;
    // (one piece per lane; the wave reduction adds them in a fixed order)
    const uint32_t pc = min((uint32_t)lane_id(), pieces - 1u); // pieces <= kMaxSlices = 64
    const double ps = sc_arg.piece_sum[(size_t)row * sc_arg.pieces_cap + pc];
    const uint32_t pn = sc_arg.piece_cnt[(size_t)row * sc_arg.pieces_cap + pc];
    if (flag != 1)
        return;
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid]; // (for the whole-row path; stage_args' barrier publishes it)
    const double total64 = __ockl_wfred_add_f64((uint32_t)lane_id() < pieces ? ps : 0.0);
    const uint32_t n_valid = __ockl_wfred_add_u32((uint32_t)lane_id() < pieces ? pn : 0u);
    stage_args(d_arg, sc_arg, row, s_args);
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
    if (n_valid == 0 || n0 == 0) { // no candidate survived (src/gen/sampler.cpp:37-38)
        float m;
        uint32_t argidx, nc, ov;
        row_summary(sc, row, slices, m, argidx, nc, ov);
        fallback_row(d, row, argidx);
        return;
    }
    // The list holds every weight with bits(q) >= thr_bits; when that is not every candidate the nucleus has to end
    // inside the list (it was kept on a guess: sample_plan()), else the row takes the whole-row path.
    const bool partial = n0 < n_valid; // uniform
    const float q_bound = thr_bits ? __uint_as_float(thr_bits - 1u) : 0.0f; // (no missing weight is heavier)
    if (sorted_tail<true>(d, row, s_args.P, sc.key[0] + (size_t)row * sc.vpad, sc.idx[0] + (size_t)row * sc.vpad, n0, true,
                          total64, MAKO_PATH_NUCLEUS, L, partial, q_bound, sc.gt, (size_t)row * sc.g_cap, groups))
        return;
    __syncthreads();
    {
        float m;
        uint32_t argidx, nc, ov;
        row_summary(sc, row, slices, m, argidx, nc, ov);
        general_row<0>(d, sc, row, s_args.P, m, argidx, L);
    }
}
#endif // MAKO_EMIT_TAIL_KERNEL

} // namespace mako
