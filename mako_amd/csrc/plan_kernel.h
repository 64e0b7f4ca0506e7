// plan_kernel: one workgroup per row between the second pass and the sort.
#pragma once

#include "topk_candidates.h"
#include "nucleus_plan.h"

namespace mako {

// grid = (1, rows), one workgroup per row.  Rows whose token is forced, greedy rows and (INLINE_GENERAL only: in a
// batch that goes on to sort_kernel and tail_kernel, top-k and whole-row rows are finished beside the tails) top-k
// rows are finished here from the records scan_kernel left; a top_k == 0 row's exact total, candidate count and weight histogram (from
// finish_kernel) are summed over its pieces and the row is planned: handed to sort_kernel's workers, or, when the
// nucleus is narrow enough to end inside the candidate lists, to its worker 0 alone.
// INLINE_GENERAL: sort_kernel will not be launched for this batch (the host saw no row that needs it), so a row
// that turns out to need the whole-row path after all is given it here.  (A variant of its own: the whole-row path
// costs the kernel registers that the usual batches should not pay for.)
template <bool INLINE_GENERAL>
__global__ __launch_bounds__(kThreads) void plan_kernel(mako_sample_desc d_arg, const Scratch* sc_dev, uint32_t slices)
{
    constexpr bool inline_general = INLINE_GENERAL;
    const Scratch& sc_arg = *sc_dev;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t row = blockIdx.y;
    const uint32_t tid = threadIdx.x;
#ifdef MAKO_TIMING_PLAN
    MAKO_WG_TIMER;
#endif
    MAKO_ROW(row);
    stage_args(d_arg, sc_arg, row, s_args);
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    const mako_sampling_params& P = s_args.P;
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;
    L.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);
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
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    __syncthreads();
    // a top-k row's candidates are asked for together with the slices' records
    CandSlots pre;
    const bool prefetched = inline_general && cls == kTopK && !d.draft && slots_cover(slices); // uniform
    if (prefetched)
        fetch_candidate_slots(sc, row, slices, pre);
    float m;
    uint32_t argidx, n_cands, any_overflow;
    SliceStat lane_stat;
    row_summary(sc, row, slices, m, argidx, n_cands, any_overflow, &lane_stat);
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

    if (cls != kNucleus) {
        // (in a batch that goes on to sort_kernel and tail_kernel, tail_kernel's launch finishes these rows beside the
        // tails: finish_late_row())
        if constexpr (inline_general) {
            if (topk_takes_whole_row(cls, any_overflow, n_cands))
                general_row<1>(d, sc, row, P, m, argidx, L);
            else
                topk_row(d, sc, row, slices, P, m, argidx, n_cands, lane_stat, L, prefetched, pre);
        }
        return;
    }

    MAKO_STAMP(2);
    const uint32_t pieces = uniform_u32(sc.work_n[4]);
    // this thread's two bins of the row's histogram (left zero for the next batch), the pieces' exact sums (one per
    // lane, added up in the wave reduction's fixed order)
    unsigned long long* bins = sc.bins + (size_t)row * kBins;
    const unsigned long long rec0 = bins[kBins - 1u - 2u * tid], rec1 = bins[kBins - 2u - 2u * tid];
    const uint32_t bin_c0 = (uint32_t)(rec0 >> kBinSumBits), bin_c1 = (uint32_t)(rec1 >> kBinSumBits);
    const unsigned long long bin_s0 = rec0 & ((1ull << kBinSumBits) - 1ull), bin_s1 = rec1 & ((1ull << kBinSumBits) - 1ull);
    const uint32_t pc = min((uint32_t)lane_id(), pieces - 1u); // pieces <= kMaxSlices = 64
    const double ps = sc.part_sum[(size_t)row * kMaxSlices + pc];
    const uint32_t pn = sc.part_n[(size_t)row * kMaxSlices + pc];
    const double row_total = __ockl_wfred_add_f64((uint32_t)lane_id() < pieces ? ps : 0.0);
    const uint32_t row_n0 = __ockl_wfred_add_u32((uint32_t)lane_id() < pieces ? pn : 0u);
    if (rec0)
        bins[kBins - 1u - 2u * tid] = 0;
    if (rec1)
        bins[kBins - 2u - 2u * tid] = 0;
    MAKO_STAMP(15);
    if (row_n0 == 0) {
        fallback_row(d, row, argidx);
        return;
    }
    uint32_t thr_bits = 0;
    const uint32_t n0 = plan_nucleus(P, row_total, bin_c0, bin_c1, bin_s0, bin_s1, sc.plan + row, sc.bin_worker + (size_t)row * kBins, L, thr_bits, d.n_vocab);
    MAKO_STAMP(16);
    const bool narrow = !d.draft && n0 <= kSmall && !any_overflow && n_cands <= kSortMax;
    // (a list too long for the workers' group records goes to the whole-row path)
    const bool fits = n0 <= kGroup * (kMaxGroups - kWorkers);
    if (tid == 0) {
        if (!fits) {
            sc.plan[row].total64 = (double)m;
            sc.plan[row].n0 = argidx;
        }
        sc.plan[row].thr = thr_bits;
        sc.plan[row].flag = !fits ? 2 : (narrow ? 3 : 1);
    }
    // the row's pieces of work for sort_kernel (all workers, or worker 0 alone) and tail_kernel; a row for the
    // whole-row path is finished in tail_kernel's launch from its flag alone (finish_late_row())
    if (!fits)
        return;
    const uint32_t work = !narrow ? kWorkers : 1u;
    if (tid == 0)
        sm.flag = atomicAdd(&sc.work_n[0], work);
    __syncthreads();
    if (tid < work)
        sc.work_sort[sm.flag + tid] = (row << 8) | tid;
    if (tid == 0 && !narrow)
        sc.work_tail[atomicAdd(&sc.work_n[1], 1u)] = row;
}

} // namespace mako
