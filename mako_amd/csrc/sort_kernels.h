// partition_kernel and sort_kernel.
#pragma once

#include "worker_sort.h"
#include "topk_candidates.h"

namespace mako {

#ifdef MAKO_EMIT_SORT_KERNELS // (not templates: defined by the one translation unit that launches them)
// grid = (kWorkers, rows) workgroups over the same work list as sort_kernel; only planned wide rows do anything.
// Piece c of a row reads the c-th part of the row's bits(q) array once and hands every weight the plan wants to
// the worker that will sort it: positions inside the workgroup from LDS counters, one global atomic per worker to
// reserve the workgroup's run in that worker's share.  (Without this step each of the 32 workers would sweep the
// whole row to find its own weights.)
__global__ __launch_bounds__(kThreads) void partition_kernel(mako_sample_desc d, Scratch sc_arg)
{
    // (the context's record by value, and loads asked for in groups: a workgroup here lives four microseconds, and
    // every dependent trip to memory is most of one)
    const Scratch& sc = sc_arg;
    __shared__ uint32_t s_count[kWorkers], s_base[kWorkers], s_off[kWorkers], s_cnt[kWorkers];
    __shared__ uint32_t s_table[kBins / 4];
    const uint32_t piece = blockIdx.y * gridDim.x + blockIdx.x;
    // first trip: the list's length and this workgroup's entry of it (the list has room for every workgroup of the
    // grid; what the entry says is looked at only if the length covers it)
    const uint32_t n_work = sc.work_n[0];
    const uint32_t item = sc.work_sort[piece];
    if (piece >= n_work)
        return;
    const uint32_t row = item >> 8, c = item & 255u, tid = threadIdx.x;
    MAKO_ROW(row);
    BigPlan* plan = sc.plan + row;
    const uint32_t V = d.n_vocab;
    const uint32_t* qk = reinterpret_cast<const uint32_t*>(sc.wbuf + (size_t)row * sc.vpad);
    uint32_t* kstage = sc.key[1] + (size_t)row * sc.vpad;
    uint32_t* istage = sc.idx[1] + (size_t)row * sc.vpad;
    const uint32_t part = (((V + kWorkers - 1u) / kWorkers) + 3u) & ~3u; // entries per piece, a multiple of 4
    const uint32_t lo = min(V, c * part), hi = min(V, lo + part);
    // second trip: the row's flag, the piece's first weights, the bin -> worker table and the workers' ranges
    const uint32_t flag = plan->flag;
    uint4 x = make_uint4(0, 0, 0, 0);
    {
        const uint32_t i = lo + tid * 4u;
        if (i < hi)
            x = *reinterpret_cast<const uint4*>(qk + i); // (the array is padded to a multiple of 1024 entries past V)
    }
    uint32_t table_word = 0, off_w = 0, cnt_w = 0;
    if (tid < kBins / 4)
        table_word = reinterpret_cast<const uint32_t*>(sc.bin_worker + (size_t)row * kBins)[tid];
    if (tid < kWorkers) {
        off_w = plan->off[tid];
        cnt_w = plan->cnt[tid];
    }
    if (flag != 1)
        return;
    if (tid < kBins / 4)
        s_table[tid] = table_word;
    if (tid < kWorkers) {
        s_count[tid] = 0;
        s_off[tid] = off_w;
        s_cnt[tid] = cnt_w;
    }
    __syncthreads();
    const uint8_t* table = reinterpret_cast<const uint8_t*>(s_table);
    for (uint32_t base = lo; base < hi; base += kThreads * 4u) {
        const uint32_t i = base + tid * 4u;
        if (base != lo) {
            x = make_uint4(0, 0, 0, 0);
            if (i < hi)
                x = *reinterpret_cast<const uint4*>(qk + i);
        }
        const uint32_t k[4] = {x.x, x.y, x.z, x.w};
        uint32_t dest[4], lpos[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            dest[j] = (i + j < hi && k[j] != 0) ? table[weight_bin(k[j])] : 0xffu;
            lpos[j] = 0;
            if (dest[j] < kWorkers)
                lpos[j] = atomicAdd(&s_count[dest[j]], 1u);
        }
        __syncthreads();
        if (tid < kWorkers) {
            s_base[tid] = s_count[tid] ? atomicAdd(&plan->cursor[tid], s_count[tid]) : 0u;
            s_count[tid] = 0;
        }
        __syncthreads();
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            if (dest[j] < kWorkers) {
                const uint32_t at = s_base[dest[j]] + lpos[j];
                if (at < s_cnt[dest[j]] && s_off[dest[j]] + at < V) { // (always, when the plan is sound)
                    kstage[s_off[dest[j]] + at] = k[j];
                    istage[s_off[dest[j]] + at] = i + j;
                }
            }
        __syncthreads();
    }
}

// grid = (kWorkers, rows) workgroups, of which workgroup i serves entry i of the work list.  Worker w gathers its range of weights from
// the row's bits(q) array, sorts it and stores it at its place in the row's sorted list; the last worker to
// finish cuts the nucleus and draws.
__global__ __launch_bounds__(kThreads) void sort_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    // (the context's record by value: its first loads, the list's length and this workgroup's entry, go out together
    // and at once; the list has room for every workgroup of the grid)
    const Scratch& sc_arg = sc_val;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t piece = blockIdx.y * gridDim.x + blockIdx.x;
    const uint32_t n_work = sc_arg.work_n[0];
    const uint32_t item = sc_arg.work_sort[piece];
    if (piece >= n_work)
        return;
#ifdef MAKO_TIMING_SORT
    MAKO_WG_TIMER;
#endif
    const uint32_t row = item >> 8, w = item & 255u, tid = threadIdx.x;
    MAKO_ROW(row);
    const uint32_t flag = sc_arg.plan[row].flag;
    if ((flag != 1 && flag != 3) || (flag == 3 && w != 0)) // (never: the list holds exactly the flagged rows' pieces)
        return;
    stage_args(d_arg, sc_arg, row, s_args);
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    BigPlan* plan = sc.plan + row;
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;
    L.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    const uint32_t* qk = reinterpret_cast<const uint32_t*>(sc.wbuf + (size_t)row * sc.vpad);
    uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
    uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
    uint32_t* key1 = sc.key[1] + (size_t)row * sc.vpad;
    uint32_t* idx1 = sc.idx[1] + (size_t)row * sc.vpad;
    const uint32_t n0 = min(plan->n0, d.n_vocab), groups = min(plan->groups, kMaxGroups);
    const double total64 = plan->total64;
    if (flag == 3) {
        // narrow nucleus: it should end inside the slices' candidate lists, strictly above everything they left out
        const uint32_t thr_bits = plan->thr;
        __syncthreads();
        if (tid == 0)
            plan->flag = 0;
        const mako_sampling_params& P = s_args.P;
        // (the candidate lists are asked for together with the slices' records, as for a top-k row)
        CandSlots pre;
        const bool prefetched = slots_cover(slices); // uniform
        if (prefetched)
            fetch_candidate_slots(sc, row, slices, pre);
        float m;
        uint32_t argidx, n_cands, any_overflow;
        SliceStat lane_stat;
        row_summary(sc, row, slices, m, argidx, n_cands, any_overflow, &lane_stat);
        const float inv_t = 1.0f / P.temperature;
        const float floor_q = (1.0f < P.min_p) ? 1.0f : P.min_p;
        const float q_bound = candidate_bound(lane_stat, slices, m, inv_t, floor_q, sm);
        MAKO_STAMP(3);
        uint32_t* kf = reinterpret_cast<uint32_t*>(L.sortk + kSortMax);
        uint32_t* jf = kf + kSortMax;
        uint32_t n_valid = 0;
        const uint32_t n_list =
            small_candidates(sc, row, slices, n_cands, m, inv_t, floor_q, 0u, thr_bits, kf, jf, n_valid, L, prefetched, pre);
        MAKO_STAMP(4);
        if (n_list != kNone && n_list > 0 &&
            sorted_tail(d, row, P, kf, jf, n_list, true, total64, MAKO_PATH_NUCLEUS, L, true, q_bound))
            return;
        // not certifiable from the candidates: tail_kernel's launch takes a second look (narrow_second_look())
        if (tid == 0)
            plan->flag = 4;
        return;
    }
    uint32_t cnt = plan->cnt[w];
    const uint32_t off = plan->off[w], gbase = plan->gbase[w];
    // (a sound plan never trips these; they keep every store of this worker inside the row's arrays)
    if (off > n0 || cnt > n0 - off || gbase + (cnt + kGroup - 1u) / kGroup > min(groups, sc.g_cap))
        cnt = 0;
    const size_t t_row = (size_t)row * sc.g_cap;
    if (cnt) {
        const uint32_t key_lo = plan->key_lo[w], key_hi = plan->key_hi[w];
        MAKO_STAMP(10);
        MAKO_COUNT(31, threadIdx.x == 0 && cnt > kSegCap ? 1 : 0);
        MAKO_COUNT(21, threadIdx.x == 0 ? cnt : 0);
        uint32_t* sorted_copy = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(s_dyn64) + kSortedCopyAt);
        const bool in_lds = cnt <= kSegCap; // uniform
        const bool sorted = in_lds
                                ? lds_sort_staged(key1 + off, idx1 + off, key_lo, key_hi, cnt, key0 + off, idx0 + off, s_dyn64, sm,
                                                  sorted_copy)
                                : lds_sort_staged_runs(key1 + off, idx1 + off, key_lo, key_hi, cnt, key0 + off, idx0 + off, s_dyn64, sm);
        if (cnt > kSegCap)
            MAKO_STAMP(18);
        if (!sorted) {
            MAKO_STAMP(17);
            MAKO_COUNT(23, threadIdx.x == 0 ? 1 : 0);
            gather_range(qk, d.n_vocab, key_lo, key_hi, key0 + off, idx0 + off, cnt, sm);
            sort_segment(key0 + off, idx0 + off, key1 + off, idx1 + off, cnt, L);
        }
        MAKO_STAMP(11);
        worker_groups(key0, off, cnt, t_row + gbase, plan->mass[w], sc.gt, L, (in_lds && sorted) ? sorted_copy : nullptr);
        MAKO_STAMP(12);
    }
}
#endif // MAKO_EMIT_SORT_KERNELS

} // namespace mako
