// finish_kernel: the second pass over the top_k == 0 rows.
#pragma once

#include "slice_load.h"
#include "work_split.h"
#include "row_records.h"
#include "coarse_plan.h"

namespace mako {

// A workgroup's share of a top_k == 0 row's pieces, one after the other.  Of each piece: the exact fp64 sum of q over
// it, and every weight the row's plan keeps handed to the share of the worker that will sort it.
// The summation order is fixed: each thread adds its logits in index order, then lanes, then waves.
// The plan (coarse_plan()) is built while the first piece's logits are on their way; every workgroup of the row
// arrives at the same one, and the one with the row's first piece stores it for the kernels that follow and enters
// the row in their lists.
// (PEN: the row has penalties to apply; a compile-time fact so that each case gets straight-line code of its own.)
// (`slices`: of scan_kernel, whose records give the row maximum)
// (PLANNING: the workgroup's first piece, with which the plan is built; returns false when the row leaves for the
// whole-row path and the pass has nothing more to do for it)
template <bool VEC, int KH, bool PEN, bool PLANNING, bool UNSORTED = false>
__device__ bool one_piece(const mako_sample_desc& d, const Scratch& sc, uint32_t row, uint32_t slice, uint32_t slice_len,
                          const mako_sampling_params& P, uint32_t hl, uint32_t slices, const FinishLds& L, CoarsePlan& pl,
                          float& m, uint32_t& argidx, uint32_t opaque_first = kNone)
{
    assume_lds(L);
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
    constexpr bool pen = PEN;
    BigPlan* plan = sc.plan + row;
    const uint32_t lo = slice * slice_len;
    const uint32_t hi = min(d.n_vocab, lo + slice_len);
    float wv[16];
    MAKO_STAMP(28);
    if constexpr (PLANNING) {
        PlanLoads pre;
        issue_plan_loads<UNSORTED>(d, sc, row, slices, pre);
        load_penalised<VEC, KH>(d, row, lo, hi, slice_len, P, hl, pen, L.cnt, wv, [&]() {
            uint32_t n_cands, any_overflow;
            row_summary_of(pre.st, slices, m, argidx, n_cands, any_overflow);
            coarse_plan(sc, row, slices, d.n_vocab, P, m, pre, !d.draft && !any_overflow && n_cands <= kSortMax, UNSORTED ? opaque_first : kNone, pl, sm.tab);
        });
    } else {
        load_penalised<VEC, KH>(d, row, lo, hi, slice_len, P, hl, pen, L.cnt, wv);
    }
    MAKO_STAMP(1);
    MAKO_STAMP(24);
    const uint32_t flag = pl.flag;
    if (PLANNING && slice == 0) {
        // the row's first piece stores the plan and enters the row in the lists of sort_kernel and tail_kernel
        if (tid < kWorkers) {
            plan->key_lo[tid] = pl.key_lo[tid];
            plan->stage_off[tid] = pl.stage_off[tid];
            plan->cap[tid] = pl.cap[tid];
            plan->mass[tid] = pl.mass_above[tid];
        }
        if (tid == 0) {
            plan->thr = pl.thr;
            plan->argidx = argidx;
            plan->m = m;
            plan->mass_all = pl.mass_all;
            plan->flag = flag;
            const uint32_t unsorted = (UNSORTED && flag == 1) ? pl.opq_mask : 0u;
            plan->opq_mask = unsorted;
            if (flag == 1 || flag == 3) {
                // sort_kernel's work: a workgroup per worker that sorts, and up to kCollectors whose waves take one of the
                // row's unsorted shares each (work items kWorkers + c)
                const uint32_t n_unsorted = (uint32_t)__popc(unsorted), collectors = (n_unsorted + (uint32_t)kWaves - 1u) / (uint32_t)kWaves;
                if constexpr (UNSORTED) {
                    // (two lists, the costly entries in front: large_batch_lists())
                    const SortLists lists = large_batch_lists(d.n_rows);
                    if (flag == 3) {
                        sc.work_sort[lists.sorted_at + atomicAdd(&sc.work_n[0], 1u)] = row << 8;
                    } else {
                        uint32_t at = lists.sorted_at - atomicAdd(&sc.work_n[3], collectors) - collectors;
                        for (uint32_t c = 0; c < collectors; ++c)
                            sc.work_sort[at++] = (row << 8) | (kWorkers + c);
                        at = lists.sorted_at + atomicAdd(&sc.work_n[0], kWorkers - n_unsorted);
                        for (uint32_t w = 0; w < kWorkers; ++w)
                            if (!((unsorted >> w) & 1u))
                                sc.work_sort[at++] = (row << 8) | w;
                    }
                } else {
                    const uint32_t work = flag == 1 ? kWorkers : 1u;
                    uint32_t at = atomicAdd(&sc.work_n[0], work);
                    for (uint32_t w = 0; w < work; ++w)
                        sc.work_sort[at++] = (row << 8) | w;
                }
                if (flag == 1)
                    sc.work_tail[atomicAdd(&sc.work_n[1], 1u)] = row;
            }
        }
    }
    if (flag == 2) // the whole-row path starts from the logits again
        return false;
    const float inv_t = 1.0f / P.temperature;
    const float floor_q = (1.0f < P.min_p) ? 1.0f : P.min_p;
    const uint32_t thr = pl.thr;
    const uint32_t edge7 = uniform_u32(pl.key_lo[7]), edge15 = uniform_u32(pl.key_lo[15]), edge23 = uniform_u32(pl.key_lo[23]);
    double sum = 0;
    uint32_t qb[16];   // bits(q), 0 where q is not a candidate
    uint32_t slot[16]; // kept weights: worker << 16 | position among this workgroup's entries for that worker
    // (a piece may be shorter than the sixteen logits per thread: whole blocks past its end are skipped; the test is
    // the same for every thread)
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j) {
        qb[j] = 0u;
        slot[j] = kNone;
        if (lo + (VEC ? (j / 4u) * 4096u : j * (uint32_t)kThreads) < hi) {
            // (the large batches' instance: a wave whose weights all underflow to zero, as those of a peaked row far
            // below its maximum do, skips the arithmetic that would tell it so; expf_glibc() returns 0 below that bound)
            float q = 0.0f;
            if (!UNSORTED || __ballot(!((wv[j] - m) * inv_t < -0x1.9fe368p6f)) != 0ull)
                q = weight_of(wv[j], m, inv_t, sm.tab);
            qb[j] = (q >= floor_q && q > 0.0f) ? __float_as_uint(q) : 0u;
            if (qb[j])
                sum += (double)q;
            if (qb[j] >= thr && qb[j]) {
                // the worker whose range of bits(q) holds the weight (equal weights always meet in one share): the
                // number of workers whose lower edge lies above it, by bisection over the edges
                // (the first two steps against edges held in scalar registers, the other three from LDS)
                static_assert(kWorkers == 32, "five steps");
                uint32_t w = qb[j] < edge15 ? 16u : 0u;
                w += qb[j] < (w ? edge23 : edge7) ? 8u : 0u;
#pragma unroll
                for (uint32_t step = 4u; step; step >>= 1)
                    w += qb[j] < pl.key_lo[w + step - 1u] ? step : 0u;
                slot[j] = (w << 16) | atomicAdd(&pl.count[w], 1u);
            }
        }
    }
    MAKO_STAMP(25);
    // the piece's sum: wave reductions, then the sixteen waves' results in order
    {
        const double sw = __ockl_wfred_add_f64(sum);
        if (lane_id() == 0)
            sm.bs.f64[wave_id()] = sw;
    }
    lds_barrier();
    MAKO_STAMP(26);
    // One run per worker in its share of the row's staging arrays, reserved with a single atomic.  The kept weights
    // are first put in LDS (the penalty table's block, free by now) in the order of their workers, so that the runs
    // go out as contiguous stores.
    // (the reservations' answers take a trip to device memory: the entries are put in LDS order under it)
    uint32_t mine = 0, lbase_mine = 0, base_mine = 0;
    if (wave_id() == 0) {
        mine = tid < kWorkers ? pl.count[tid] : 0u;
        const uint32_t upto = __ockl_wfscan_add_u32(mine, true);
        lbase_mine = upto - mine;
        if (tid < kWorkers) {
            pl.lbase[tid] = lbase_mine;
            if (mine)
                base_mine = __hip_atomic_fetch_add(as_global(&plan->cursor[tid]), mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (tid == kWorkers - 1u)
            pl.lbase[kWorkers] = upto;
    }
    lds_barrier(); // (not one that waits for the reservations)
    MAKO_STAMP(27);
    if (tid < kWorkers)
        pl.count[tid] = 0; // (for the workgroup's next piece)
    const global_ptr<uint32_t> kstage = as_global(sc.key[1]) + (size_t)row * sc.vpad;
    const global_ptr<uint32_t> istage = as_global(sc.idx[1]) + (size_t)row * sc.vpad;
    uint2* buf = reinterpret_cast<uint2*>(L.cnt); // [kSliceMax / 2] (weight, token id)
    constexpr uint32_t kHalf = kSliceMax / 2u;
    const uint32_t kept = pl.lbase[kWorkers];
    // (the entries' workers travel beside them, a byte each, in the plan's count arrays, which are done with)
    static_assert(offsetof(CoarsePlan, incl) == offsetof(CoarsePlan, cnt) + sizeof(uint32_t) * kLogBins && 2u * sizeof(uint32_t) * kLogBins >= kHalf &&
                      kSliceMax <= 0x10000u && kWorkers <= 256u,
                  "a byte per buffered entry; an entry's place fits sixteen bits beside its worker");
    uint8_t* wbuf = reinterpret_cast<uint8_t*>(pl.cnt);
    // (from here on: worker << 16 | the entry's place in the workgroup's order.  The runs' starts are read for all
    // sixteen at once, kept or not: behind sixteen branches each read would be a wait of its own.)
    {
        uint32_t start[16];
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j)
            start[j] = pl.lbase[(slot[j] >> 16) & (kWorkers - 1u)];
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j)
            if (slot[j] != kNone)
                slot[j] = (slot[j] & 0xffff0000u) | (start[j] + (slot[j] & 0xffffu));
    }
    bool dropped = false;
    const uint32_t unsorted_mask = UNSORTED ? uniform_u32(pl.opq_mask) : 0u;
    for (uint32_t from = 0; from < kept; from += kHalf) { // (what fits the buffer at a time: usually everything)
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j)
            if (slot[j] != kNone && (slot[j] & 0xffffu) - from < kHalf) {
                buf[(slot[j] & 0xffffu) - from] = make_uint2(qb[j], elem_index<VEC>(lo, tid, j));
                wbuf[(slot[j] & 0xffffu) - from] = (uint8_t)(slot[j] >> 16);
            }
        if (from == 0 && tid < kWorkers) { // (wave 0: where each worker's run goes and where its room ends, in the
                                           // workgroup's order)
            const uint32_t room = pl.cap[tid];
            pl.goff[tid] = pl.stage_off[tid] + base_mine - lbase_mine;
            pl.lim[tid] = lbase_mine + (room > base_mine ? room - base_mine : 0u);
        }
        lds_barrier();
#pragma unroll 4 // (fully unrolled, the unaligned variants spill dozens of registers for no gain)
        for (uint32_t t = 0; t < kHalf / kThreads; ++t) {
            const uint32_t e = from + t * kThreads + tid;
            if (e < kept) { // (uniform per wave but for the last one)
                const uint32_t w = wbuf[e - from];
                if (e < pl.lim[w]) {
                    const uint2 x = buf[e - from];
                    MAKO_CHECK(sc, kCheckStage, (uint64_t)(pl.goff[w] + e) < sc.vpad && pl.goff[w] + e >= pl.stage_off[w] &&
                                                    pl.goff[w] + e < pl.stage_off[w] + pl.cap[w]);
                    kstage[pl.goff[w] + e] = x.x;
                    if (!UNSORTED || !((unsorted_mask >> w) & 1u)) // (a share that is only summed has no use for the token ids)
                        istage[pl.goff[w] + e] = x.y;
                } else {
                    dropped = true;
                }
            }
        }
        lds_barrier();
    }
    MAKO_STAMP(29);
    if (dropped) // (more weights in a range than the counts promised: the row takes the whole-row path)
        plan->overflow = 1;
    if (tid == 0) {
        double total = 0;
        for (int w = 0; w < kWaves; ++w) // waves in order: the same inputs always give the same bits
            total += sm.bs.f64[w];
        as_global(sc.part_sum)[(size_t)row * kMaxSlices + slice] = total;
    }
    lds_barrier(); // (the waves' sums have been read before the next piece's replace them)
    MAKO_STAMP(30);
    return true;
}

template <bool VEC, int KH, bool PEN, bool UNSORTED>
__device__ void row_pieces(const mako_sample_desc& d, const Scratch& sc, uint32_t row, uint32_t first, uint32_t stride,
                           uint32_t n_pieces, uint32_t slice_len, const mako_sampling_params& P, uint32_t hl, uint32_t slices,
                           const FinishLds& L, CoarsePlan& pl, uint32_t opaque_first)
{
    assume_lds(L);
    // the workgroup's pieces in turn: first, first + stride, ...
    float m = 0.0f;
    uint32_t argidx = 0;
    if (first >= n_pieces || !one_piece<VEC, KH, PEN, true, UNSORTED>(d, sc, row, first, slice_len, P, hl, slices, L, pl, m, argidx, opaque_first))
        return;
    for (uint32_t slice = first + stride; slice < n_pieces; slice += stride)
        one_piece<VEC, KH, PEN, false, UNSORTED>(d, sc, row, slice, slice_len, P, hl, slices, L, pl, m, argidx);
}

// Second pass over the top_k == 0 rows.  grid = (most pieces a row can have, rows) workgroups, of which workgroup i
// serves the i-th share of a row's pieces in row order, SecondPassCut::per_row per top_k == 0 row (find_piece): the busy
// workgroups are then the first ones dispatched and land evenly on the XCDs, shader engines and CUs, whatever the
// mix of rows.
// (UNSORTED: the instance for batches of many such rows, whose plans leave shares unsorted: unsorted_shares.h)
template <bool VEC, int KH, bool UNSORTED>
__global__ __launch_bounds__(kThreads) void finish_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    const Scratch& sc_arg = sc_val; // (by value: the cut is one trip to memory away, not two)
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    __shared__ CoarsePlan s_plan;
#ifdef MAKO_TIMING_FINISH
    MAKO_WG_TIMER;
#endif
    // What the workgroup needs before it can ask for its logits is asked for in as few trips to memory as possible
    // (each costs most of a microsecond here, and the pass starts with nothing else to do): the rows' parameters
    // for find_piece() and the arguments' copy go out together with the cut, and the row's own parameters are then
    // taken from the lane that loaded them.
    uint32_t wg = blockIdx.y * gridDim.x + blockIdx.x;
    const uint32_t tid = threadIdx.x;
    const bool by_lane = d_arg.n_rows <= (uint32_t)kWave; // uniform
    mako_sampling_params P_lane = mako_sampling_params{};
    if (by_lane)
        P_lane = d_arg.params[min((uint32_t)lane_id(), d_arg.n_rows - 1u)];
    stage_args_only(d_arg, sc_arg, s_args);
    // (pieces per row, their length, workgroups with work: the others leave at once)
    const uint4 cut = *reinterpret_cast<const uint4*>(sc_arg.work_n + 4);
    // Workgroups go to the eight XCDs in turn.  The shares are dealt so that an XCD's workgroups serve consecutive
    // ones: the workgroups of a row then sit on one XCD (two where a row straddles), whose L2 fetches the row's
    // coarse counts and history once for all of them.  (Only if the grid holds every workgroup the deal names.)
    if (cut.x < cut.w) {
        // More pieces than one round of workgroups, so a row's workgroups go through several pieces each and rows that
        // need little are done long before rows that need much (a near-flat row takes twice as long as a peaked one).
        // The rows go round-robin to the XCDs (an XCD's workgroups are dispatched in order onto whichever of its CUs
        // is free, but which XCD a workgroup goes to is fixed by its number), a row's workgroups to one XCD.
        const uint32_t rowrank = (wg & 7u) + 8u * ((wg >> 3) / cut.x);
        wg = rowrank * cut.x + (wg >> 3) % cut.x;
        if (rowrank * cut.x >= cut.z)
            return;
    } else {
        const uint32_t per_xcd = (cut.z + 7u) / 8u;
        if (per_xcd * 8u <= gridDim.x * gridDim.y) {
            if ((wg >> 3) >= per_xcd)
                return;
            wg = (wg & 7u) * per_xcd + (wg >> 3);
        }
    }
    if (wg >= cut.z)
        return;
    const uint32_t pieces = cut.x, piece_len = cut.y, n_pieces = cut.w; // (pieces: workgroups per row)
    uint32_t row, piece;
    if (by_lane) {
        // find_piece() over the parameters already here: one row per lane, every wave for itself
        const uint32_t mine = ((uint32_t)lane_id() < d_arg.n_rows && classify(P_lane) == kNucleus) ? pieces : 0u;
        const uint32_t upto = __ockl_wfscan_add_u32(mine, true);
        const unsigned long long bal = __ballot(wg >= upto - mine && wg < upto);
        if (bal == 0ull)
            return;
        const int owner = __ffsll((long long)bal) - 1;
        row = (uint32_t)owner;
        piece = wg - (uint32_t)__builtin_amdgcn_readlane((int)(upto - mine), owner);
        mako_sampling_params P_row;
        uint32_t* dst = reinterpret_cast<uint32_t*>(&P_row);
        const uint32_t* src = reinterpret_cast<const uint32_t*>(&P_lane);
#pragma unroll
        for (uint32_t i = 0; i < sizeof(mako_sampling_params) / 4; ++i)
            dst[i] = (uint32_t)__builtin_amdgcn_readlane((int)src[i], owner);
        stage_params(P_row, s_args);
    } else {
        if (!find_piece(d_arg, wg, pieces, 0u, row, piece, sm.bs))
            return;
        stage_params(d_arg.params[row], s_args);
    }
    MAKO_ROW(row);
    MAKO_WG_TAG((row << 8) | piece | 0x80000000u);
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    __syncthreads(); // (publishes the arguments, the parameters and the table)
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;                                             // 32 KB
    L.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);    // next 16 KB
    const mako_sampling_params& P = s_args.P;
    MAKO_STAMP(0);
    if (d.force_token || d.close_token) { // a forced row needs no weights (plan_kernel writes its token)
        int32_t ftok;
        uint32_t above;
        if (row_forced(d, sc, row, slices, ftok, above) != MAKO_FORCED_NONE)
            return;
    }
    // (the history's length and, inside slice_partial, the history, the logits and the slices' records: one trip)
    const uint32_t hl = d.hist_tokens ? min(as_global(d.hist_len)[row], (uint32_t)d.hist_stride) : 0u;
    // (a row without history entries takes the penalising variant too when it has penalties: it finds nothing to
    // penalise, and nothing here waits for the length)
    // (shares may be left unsorted from the first position that the tail neither keeps in LDS nor writes out; never on
    // verification rows, whose replay reads the list itself)
    const uint32_t opaque_first = (UNSORTED && !d.draft) ? max(kHeadGroups * kGroup, (d.out_cand_idx && d.out_cand_q) ? d.cand_cap : 0u) : kNone;
    if (d.hist_tokens && !penalties_neutral(P))
        row_pieces<VEC, KH, true, UNSORTED>(d, sc, row, piece, pieces, n_pieces, piece_len, P, hl, slices, L, s_plan, opaque_first);
    else
        row_pieces<VEC, KH, false, UNSORTED>(d, sc, row, piece, pieces, n_pieces, piece_len, P, hl, slices, L, s_plan, opaque_first);
}

} // namespace mako
