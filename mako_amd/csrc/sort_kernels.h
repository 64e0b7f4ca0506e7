// sort_kernel.
#pragma once

#include "worker_sort.h"
#include "topk_candidates.h"

namespace mako {

#ifdef MAKO_EMIT_SORT_KERNELS // (not templates: defined by the one translation unit that launches them)
// grid = (kWorkers, rows) workgroups, of which workgroup i serves entry i of the work list.  Worker w sorts the share
// of the row's weights that the second pass handed it and stores it at its place in the row's sorted list, with
// the group records tail_kernel works from; worker 0 of a narrow row finishes the row from the candidate lists.
// What the row's list looks like as a whole (the workers' counts, the exact total) every worker adds up for itself
// from what the second pass left; worker 0 stores it for tail_kernel.
// UNSORTED: the instance for batches whose plans leave shares unsorted (unsorted_shares.h; a translation unit of its own,
// k_sort_unsorted.hip): it knows the rows' collectors and that an unsorted share is one record.
template <bool UNSORTED>
__device__ __forceinline__ void sort_body(const mako_sample_desc& d_arg, const Scratch& sc_val, uint32_t slices)
{
    // (the context's record by value: its first loads, the list's length and this workgroup's entry, go out together
    // and at once; the list has room for every workgroup of the grid)
    const Scratch& sc_arg = sc_val;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t piece = blockIdx.y * gridDim.x + blockIdx.x, tid = threadIdx.x;
    // A workgroup's time here is a chain of round trips to device memory, and each one left out shortens it by half
    // a microsecond.  Three remain: the work list's entry (with the arguments' copy for LDS), everything of the row's
    // record (a worker per lane), the worker's share.  (The empty asm statements keep each trip's loads together:
    // the compiler would let those that only a later branch needs wait for that branch.)
    ArgWords arg_words;
    fetch_arg_words(d_arg, sc_arg, arg_words);
    const uint32_t n_work = sc_arg.work_n[0];
    const uint32_t pieces_raw = sc_arg.work_n[7];
    const uint32_t item = sc_arg.work_sort[piece];
    const uint64_t tab_word = k_exp2_tab[tid & 31u];
    if constexpr (UNSORTED) {
        // (two lists that meet at workgroup number sorted_at: large_batch_lists())
        const uint32_t n_collectors = sc_arg.work_n[3];
        asm volatile("" ::"s"(item), "s"(n_work), "s"(n_collectors), "s"(pieces_raw), "v"(arg_words.d), "v"(arg_words.sc), "v"(tab_word));
        const SortLists lists = large_batch_lists(d_arg.n_rows);
        const bool with_work = piece < lists.sorted_at ? lists.sorted_at - piece <= n_collectors : piece - lists.sorted_at < n_work;
        if (!with_work)
            return;
    } else {
        asm volatile("" ::"s"(item), "s"(n_work), "s"(pieces_raw), "v"(arg_words.d), "v"(arg_words.sc), "v"(tab_word));
        if (piece >= n_work)
            return;
    }
#ifdef MAKO_TIMING_SORT
    MAKO_WG_TIMER;
#endif
    const uint32_t row = item >> 8, w = item & 255u;
    MAKO_ROW(row);
    const uint32_t lane = (uint32_t)lane_id();
    const uint32_t wl = min(lane, kWorkers - 1u);
    const BigPlan* rec = sc_arg.plan + row;
    const uint32_t flag = rec->flag;
    const uint32_t overflow = rec->overflow;
    const uint32_t thr_bits = rec->thr;
    const double mass_all = rec->mass_all;
    const uint32_t opq_mask = UNSORTED ? rec->opq_mask : 0u; // workers whose shares stay unsorted (unsorted_shares.h)
    const uint32_t handed = rec->cursor[wl], room = rec->cap[wl];
    const uint32_t stage_l = rec->stage_off[wl], key_lo_l = rec->key_lo[wl];
    const double mass_l = rec->mass[wl];
    fetch_param_words(d_arg, row, arg_words);
    const double ps = sc_arg.part_sum[(size_t)row * kMaxSlices + lane]; // (kMaxSlices = 64 sums per row: one per lane)
    const float u_row = d_arg.u[row]; // (for the estimate of where the row's walk starts)
    asm volatile("" ::"s"(flag), "s"(overflow), "s"(thr_bits), "s"(opq_mask), "v"(handed), "v"(room), "v"(stage_l), "v"(key_lo_l),
                 "v"(mass_l), "v"(ps), "v"(arg_words.p));
    if ((flag != 1 && flag != 3) || (flag == 3 && w != 0)) // (never: the list holds exactly the flagged rows' pieces)
        return;
    // the worker's share sets out as soon as its place is known; the row's sums are added up under it
    const uint32_t cnt_l = lane < kWorkers ? min(handed, room) : 0u;
    const uint32_t cnt = flag == 1 ? (uint32_t)__builtin_amdgcn_readlane((int)cnt_l, (int)w) : 0u;
    MAKO_WG_TAG(cnt | (flag == 1 ? 0x80000000u : 0u));
    const uint32_t stage = (uint32_t)__builtin_amdgcn_readlane((int)stage_l, (int)w);
    const uint32_t key_lo = (uint32_t)__builtin_amdgcn_readlane((int)key_lo_l, (int)w);
    const uint32_t key_hi = w ? (uint32_t)__builtin_amdgcn_readlane((int)key_lo_l, (int)(w - 1u)) : 0x3f800001u; // (just above 1.0)
    uint32_t* key1 = sc_arg.key[1] + (size_t)row * sc_arg.vpad;
    uint32_t* idx1 = sc_arg.idx[1] + (size_t)row * sc_arg.vpad;
    StagedShare share;
    const bool in_lds = cnt <= kSegCap; // uniform
    if (cnt && in_lds)
        fetch_staged_share(key1 + stage, idx1 + stage, cnt, share);
    place_arg_words(arg_words, s_args);
    if (tid < 32)
        sm.tab[tid] = tab_word;
    lds_barrier(); // (not one that waits for the share)
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    BigPlan* plan = sc.plan + row;
    uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
    uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
    // the row's exact total: the pieces' sums, one per lane, added up in the wave reduction's fixed order; the workers'
    // counts, and from them this worker's place in the sorted list and in the group records
    const uint32_t pieces = uniform_u32(pieces_raw);
    const double total64 = __ockl_wfred_add_f64(lane < pieces ? ps : 0.0);
    // (a share that is left unsorted is one record, whatever it holds)
    const bool unsorted_l = UNSORTED && flag == 1 && lane < kWorkers && ((opq_mask >> lane) & 1u) != 0u;
    const uint32_t grp_l = unsorted_l ? 1u : (cnt_l + kGroup - 1u) / kGroup;
    const uint32_t cnt_upto = __ockl_wfscan_add_u32(cnt_l, true), grp_upto = __ockl_wfscan_add_u32(grp_l, true);
    const uint32_t n0 = (uint32_t)__builtin_amdgcn_readlane((int)cnt_upto, kWave - 1);
    const uint32_t groups = (uint32_t)__builtin_amdgcn_readlane((int)grp_upto, kWave - 1);
    const bool spilled = __ballot(lane < kWorkers && handed > room) != 0ull || overflow != 0u;
    MAKO_STAMP(3);
    if (flag == 3) {
        // narrow nucleus: it should end inside the slices' candidate lists, strictly above everything they left out
        __syncthreads();
        if (tid == 0)
            plan->flag = 0;
        const mako_sampling_params& P = s_args.P;
        const FinishLds L = finish_lds_views(sm, s_dyn64);
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
        if (tid == 0) {
            plan->total64 = total64;
            plan->flag = 4;
        }
        return;
    }
    // a share that did not fit its room, or a list too long for the group records: the row takes the whole-row path
    if (spilled || n0 > d.n_vocab || groups > min(kMaxGroups, sc.g_cap)) {
        __syncthreads();
        if (w == 0 && tid == 0)
            plan->flag = 2;
        return;
    }
    MAKO_CHECK(sc, kCheckShare, (uint64_t)stage + cnt <= sc.vpad && (uint64_t)(cnt_upto - cnt_l) + cnt_l <= sc.vpad && n0 <= d.n_vocab);
    MAKO_CHECK(sc, kCheckGroups, grp_upto <= sc.g_cap);
    if (w == 0 && tid == 0) {
        plan->n0 = n0;
        plan->groups = groups;
        plan->total64 = total64;
    }
    const uint32_t off = (uint32_t)__builtin_amdgcn_readlane((int)(cnt_upto - cnt_l), (int)w);
    const uint32_t gbase = (uint32_t)__builtin_amdgcn_readlane((int)(grp_upto - grp_l), (int)w);
    const size_t t_row = (size_t)row * sc.g_cap;
    if (UNSORTED && w >= kWorkers) {
        // One of the row's collectors: each of its waves takes one of the shares that are left unsorted (collector c the
        // shares 16 c .. 16 c + 15 of them) and leaves its record.  (The binades of the maps from the plan's estimates in
        // the exact total's units; any guess is safe, the tail tests what it applies.  A verification row has no such
        // shares.)
        MAKO_WG_TAG(0xc0000000u);
        const double r0_raw = (double)u_row * ((double)s_args.P.top_p * total64);
        const double r0 = r0_raw == r0_raw ? r0_raw : 0.0, scale = mass_all > 0.0 ? total64 / mass_all : 0.0;
        uint32_t* wave_lds = reinterpret_cast<uint32_t*>(s_dyn64) + (uint32_t)wave_id() * (kOpaqueLdsWords + 2u);
        const uint32_t mine = (w - kWorkers) * (uint32_t)kWaves + (uint32_t)wave_id();
        uint32_t rank = 0;
        for (uint32_t v = 0; v + 1u < kWorkers; ++v) { // (uniform)
            if (!((opq_mask >> v) & 1u) || rank++ != mine)
                continue;
            const uint32_t cnt_v = (uint32_t)__builtin_amdgcn_readlane((int)cnt_l, (int)v);
            const uint32_t stage_v = (uint32_t)__builtin_amdgcn_readlane((int)stage_l, (int)v);
            const uint32_t off_v = (uint32_t)__builtin_amdgcn_readlane((int)(cnt_upto - cnt_l), (int)v);
            const size_t t_at = t_row + (uint32_t)__builtin_amdgcn_readlane((int)(grp_upto - grp_l), (int)v);
            const double before = readlane_f64(mass_l, v) * scale, after_raw = readlane_f64(mass_l, v + 1u) * scale;
            bool same_tot, same_walk;
            const OpaqueGuess og = opaque_epochs(before, after_raw > before ? after_raw : before, r0, same_tot, same_walk);
            if (cnt_v == 0u) { // (nothing came: an empty group)
                if (lane == 0u) {
                    sc.gt.sum[t_at] = 0.0;
                    sc.gt.d0[t_at] = sc.gt.d1[t_at] = sc.gt.cmax[t_at] = 0u;
                    sc.gt.start[t_at] = off_v;
                    sc.gt.pack[t_at] = 0u;
                    sc.gt.walk[t_at] = make_uint4(0u, 0u, 0u, 0u);
                }
            } else {
                opaque_share(key1 + stage_v, cnt_v, off_v, og.e_tot, og.e_walk, t_at, sc.gt, wave_lds);
            }
        }
        MAKO_STAMP(12);
        return;
    }
    if (cnt) {
        MAKO_STAMP(10);
        MAKO_COUNT(31, threadIdx.x == 0 && cnt > kSegCap ? 1 : 0);
        MAKO_COUNT(21, threadIdx.x == 0 ? cnt : 0);
        uint32_t* sorted_copy = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(s_dyn64) + kSortedCopyAt);
        const FinishLds L = finish_lds_views(sm, s_dyn64);
        const bool sorted = in_lds
                                ? lds_sort_staged(share, key_lo, key_hi, cnt, key0 + off, idx0 + off, s_dyn64, sm, sorted_copy)
                                : lds_sort_staged_runs(key1 + stage, idx1 + stage, key_lo, key_hi, cnt, key0 + off, idx0 + off, s_dyn64, sm);
        if (cnt > kSegCap)
            MAKO_STAMP(18);
        if (!sorted) {
            // (crowded value buckets: the radix sort through device memory, on a copy of the share at its place in
            // the list, with the share's own room in the staging arrays as the second buffer; stable, so the token
            // ids are put in order first)
            MAKO_STAMP(17);
            MAKO_COUNT(23, threadIdx.x == 0 ? 1 : 0);
            for (uint32_t i = tid; i < cnt; i += kThreads) {
                key0[off + i] = ~key1[stage + i];
                idx0[off + i] = idx1[stage + i];
            }
            __syncthreads();
            sort_segment(idx0 + off, key0 + off, idx1 + stage, key1 + stage, cnt, L);
            sort_segment(key0 + off, idx0 + off, key1 + stage, idx1 + stage, cnt, L);
        }
        MAKO_STAMP(11);
        // (the guess of the running sum before the share: the plan's estimate, in the exact total's units)
        const double mass_w = readlane_f64(mass_l, w);
        // (the walk starts from u * (the nucleus' fp32 total), which is top_p * total64 and at most one weight more;
        // a verification row's walk is replayed by other code)
        const double r0 = d.draft ? 0.0 : (double)u_row * ((double)s_args.P.top_p * total64);
        worker_groups(key0, off, cnt, t_row + gbase, mass_all > 0.0 ? mass_w * (total64 / mass_all) : 0.0, sc.gt, L,
                      (in_lds && sorted) ? sorted_copy : nullptr, r0 == r0 ? r0 : 0.0);
        MAKO_STAMP(12);
    }
}
#ifdef MAKO_SORT_UNSORTED
__global__ __launch_bounds__(kThreads) void sort_kernel_unsorted(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    sort_body<true>(d_arg, sc_val, slices);
}
#else
__global__ __launch_bounds__(kThreads) void sort_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    sort_body<false>(d_arg, sc_val, slices);
}
#endif
#endif // MAKO_EMIT_SORT_KERNELS

} // namespace mako
