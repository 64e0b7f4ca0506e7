// sort_kernel: the top_k == 0 rows planned, their nuclei sorted; rows on the whole-row list.
#pragma once

#include "worker_sort.h"
#include "topk_candidates.h"

namespace mako {

#ifdef MAKO_EMIT_SORT_KERNELS // (not a template: defined by the one translation unit that launches it)
// The row's kept weights of histogram bins [blo, bhi] (both inclusive), cnt of them by the row's histogram, collected
// from the second pass's pieces in any order: as pairs (bits(q), token id) into A (LDS) when A is given, else as
// ~bits(q) and token id into gk / gi (device memory).  Piece p keeps its weights ordered by bin from the heaviest
// down and a table of how many lie in bins >= b, so the wanted ones are one run per piece.  Returns false, having
// written nothing, when the pieces' tables do not add up to cnt (never, when the plan is sound).
__device__ bool gather_bins(const Scratch& sc, uint32_t row, uint32_t pieces, uint32_t piece_len, uint32_t blo, uint32_t bhi,
                            uint32_t cnt, uint2* A, uint32_t* gk, uint32_t* gi, FinishShared& sm)
{
    const uint32_t tid = threadIdx.x;
    uint32_t* base = sm.hist;  // [64] first output position of piece p's run
    uint32_t* start = sm.run;  // [64] first entry of the run inside the piece
    if (wave_id() == 0) {
        const uint32_t p = lane_id();
        uint32_t st = 0, len = 0;
        if (p < pieces && blo <= bhi && bhi < kBins) {
            const uint16_t* tab = sc.piece_tab + ((size_t)row * sc.pieces_cap + p) * (kBins + 1u);
            st = tab[bhi + 1u];
            const uint32_t end = tab[blo];
            len = end >= st ? end - st : 0u;
            if (st + len > piece_len) // (never: a table counts the piece's own weights)
                len = 0;
        }
        const uint32_t upto = __ockl_wfscan_add_u32(len, true);
        base[p] = upto - len;
        start[p] = st;
        if (p == (uint32_t)kWave - 1u)
            sm.ticket = upto;
    }
    __syncthreads();
    if (sm.ticket != cnt)
        return false;
    const uint32_t* pk = sc.key[1] + (size_t)row * sc.vpad;
    const uint16_t* pi = sc.piece_idx + (size_t)row * sc.vpad;
    constexpr uint32_t kTrip = 6; // loads in flight per thread
    for (uint32_t e0 = 0; e0 < cnt; e0 += kTrip * kThreads) {
        uint32_t k[kTrip], id[kTrip];
#pragma unroll
        for (uint32_t u = 0; u < kTrip; ++u) {
            const uint32_t e = min(e0 + u * kThreads + tid, cnt - 1u);
            uint32_t p = 0; // the last piece whose run starts at or before e (pieces without a run share a start
                            // with the next one that has)
#pragma unroll
            for (uint32_t step = 32; step; step >>= 1)
                if (base[p + step] <= e)
                    p += step;
            const uint32_t at = p * piece_len + start[p] + (e - base[p]);
            k[u] = pk[at];
            id[u] = p * piece_len + pi[at];
        }
#pragma unroll
        for (uint32_t u = 0; u < kTrip; ++u) {
            const uint32_t e = e0 + u * kThreads + tid;
            if (e < cnt) {
                if (A) {
                    A[e] = make_uint2(k[u], id[u]);
                } else {
                    gk[e] = ~k[u];
                    gi[e] = id[u];
                }
            }
        }
    }
    __syncthreads();
    return true;
}

// One worker's share sorted into kout / iout (cnt entries by (q desc, idx asc), as ~bits(q) and token id).
// sorted_lds: receives the sorted ~bits(q) too when the share fits one LDS sort (see lds_bucket_sort); the function
// returns whether it did.  tk / ti: a second buffer of cnt entries in device memory.
__device__ bool sort_share(const Scratch& sc, uint32_t row, uint32_t pieces, uint32_t piece_len, uint32_t blo, uint32_t bhi,
                           uint32_t key_lo, uint32_t key_hi, uint32_t cnt, uint32_t* kout, uint32_t* iout, uint32_t* tk,
                           uint32_t* ti, unsigned long long* dyn, uint32_t* sorted_lds, const FinishLds& L)
{
    FinishShared& sm = *L.sm;
    uint2* A = reinterpret_cast<uint2*>(dyn);
    uint16_t* B = reinterpret_cast<uint16_t*>(A + kSegCap);
    uint32_t* hist = reinterpret_cast<uint32_t*>(B + kSegCap);
    const uint32_t tid = threadIdx.x;
    bool in_lds = false;
    bool sorted = false;
    if (cnt <= kSegCap) {
        for (uint32_t b = tid; b <= kFine; b += kThreads)
            hist[b] = 0;
        if (tid == 0)
            sm.flag = 0;
        if (gather_bins(sc, row, pieces, piece_len, blo, bhi, cnt, A, nullptr, nullptr, sm)) {
            // (keys clamped into the worker's range: a bucket index is then always valid)
            for (uint32_t e = tid; e < cnt; e += kThreads)
                A[e].x = min(max(A[e].x, key_lo), key_hi - 1u);
            __syncthreads();
            sorted = lds_bucket_sort(cnt, key_lo, key_hi, kout, iout, dyn, sm, sorted_lds);
            in_lds = sorted;
        }
    } else if (gather_bins(sc, row, pieces, piece_len, blo, bhi, cnt, nullptr, tk, ti, sm)) {
        // (the staged form of the share holds bits(q), not their complement)
        for (uint32_t e = tid; e < cnt; e += kThreads)
            tk[e] = ~tk[e];
        __syncthreads();
        sorted = lds_sort_staged_runs(tk, ti, key_lo, key_hi, cnt, kout, iout, dyn, sm);
    }
    if (!sorted) {
        // crowded buckets (many equal weights): a radix sort of the share through device memory
        MAKO_STAMP(17);
        __syncthreads();
        if (gather_bins(sc, row, pieces, piece_len, blo, bhi, cnt, nullptr, kout, iout, sm))
            sort_segment_unordered(kout, iout, tk, ti, cnt, L);
    }
    return in_lds;
}

// A narrow nucleus (plan_row() found at most kSmall weights at or above the row's threshold): it should end inside
// the slices' candidate lists, strictly above everything they left out.  Returns true when that cannot be certified
// (a slice holds more of the nucleus than its list): the row then takes the whole-row path, with the row maximum and
// its first index.  All threads call.
__device__ __forceinline__ bool narrow_row(const mako_sample_desc& d, const Scratch& sc, const mako_sampling_params& P,
                                           uint32_t row, uint32_t slices, const FinishLds& L, float& whole_m,
                                           uint32_t& whole_argidx)
{
    FinishShared& sm = *L.sm;
    const BigPlan* gplan = sc.plan + row;
    const uint32_t thr_bits = gplan->thr;
    const double total64 = gplan->total64;
    // (the candidate lists are asked for together with the slices' records, as for a top-k row)
    CandSlots pre;
    const bool prefetched = slots_cover(slices); // uniform
    if (prefetched)
        fetch_candidate_slots(sc, row, slices, pre);
    uint32_t n_cands, any_overflow;
    SliceStat lane_stat;
    row_summary(sc, row, slices, whole_m, whole_argidx, n_cands, any_overflow, &lane_stat);
    const float m = whole_m;
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
        return false;
    __syncthreads();
    return true;
}

// Worker w of a wide nucleus: gathers its range of weights from the second pass's pieces, sorts it, stores it at its
// place in the row's sorted list and leaves the group records tail_kernel chains.  All threads call.
__device__ __forceinline__ void wide_worker(const Scratch& sc, uint32_t row, uint32_t w, uint32_t pieces, uint32_t piece_len,
                                            unsigned long long* s_dyn64, const FinishLds& L)
{
    const BigPlan* gplan = sc.plan + row;
    // (everything the worker needs of the plan in one trip; values every lane holds alike go to scalar registers:
    // the sort needs the vector registers)
    const uint32_t flag = gplan->flag;
    const uint32_t n0 = uniform_u32(gplan->n0), groups = uniform_u32(gplan->groups);
    uint32_t cnt = uniform_u32(gplan->cnt[w]);
    const uint32_t off = uniform_u32(gplan->off[w]), gbase = uniform_u32(gplan->gbase[w]);
    const uint32_t key_lo = uniform_u32(gplan->key_lo[w]), key_hi = uniform_u32(gplan->key_hi[w]);
    const uint32_t blo = uniform_u32(gplan->bin_lo[w]), bhi = uniform_u32(gplan->bin_hi[w]);
    const double mass = readlane_f64(gplan->mass[w], 0);
    if (flag != 1)
        return;
    // (a sound plan never trips these; they keep every store of this worker inside the row's arrays)
    if (off > n0 || cnt > n0 - off || gbase + (cnt + kGroup - 1u) / kGroup > min(groups, sc.g_cap) || key_lo >= key_hi)
        cnt = 0;
    if (cnt == 0)
        return;
    uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
    uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
    uint32_t* tk = reinterpret_cast<uint32_t*>(sc.wbuf + (size_t)row * sc.vpad);
    uint32_t* ti = sc.idx[1] + (size_t)row * sc.vpad;
    const size_t t_row = (size_t)row * sc.g_cap;
    MAKO_STAMP(10);
    uint32_t* sorted_copy = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(s_dyn64) + kSortedCopyAt);
    const bool in_lds = sort_share(sc, row, pieces, piece_len, blo, bhi, key_lo, key_hi, cnt, key0 + off, idx0 + off, tk + off,
                                   ti + off, s_dyn64, sorted_copy, L);
    MAKO_STAMP(11);
    worker_groups(key0, off, cnt, t_row + gbase, mass, sc.gt, L, in_lds ? sorted_copy : nullptr);
    MAKO_STAMP(12);
}

// Workgroup i serves entry i of the work list second_kernel left (Scratch::work_sort): a worker of a wide nucleus, a
// narrow nucleus, or a row on the whole-row path.  The busy workgroups are then the first ones dispatched and land
// evenly on the XCDs, shader engines and CUs, whatever the mix of rows.
__global__ __launch_bounds__(kThreads) void sort_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    // (the context's record by value: the first loads, the list's length and this workgroup's entry, go out together
    // and at once; the list has room for every workgroup of the grid)
    const Scratch& sc_arg = sc_val;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t wg = blockIdx.x, tid = threadIdx.x;
    const uint32_t n_work = sc_arg.work_n[0];
    const uint32_t item = sc_arg.work_sort[wg];
    const uint4 cut = *reinterpret_cast<const uint4*>(sc_arg.work_n + 4);
    if (wg >= n_work)
        return;
    const uint32_t row = item >> 8, code = item & 255u;
    if (row >= d_arg.n_rows)
        return;
    const uint32_t pieces = min(cut.x, sc_arg.pieces_cap), piece_len = cut.y;
#ifdef MAKO_TIMING_SORT
    MAKO_WG_TIMER;
#endif
    MAKO_ROW(row);
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    stage_args(d_arg, sc_arg, row, s_args); // (its barrier publishes the table too)
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    const mako_sampling_params& P = s_args.P;
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;
    L.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);
    if (code < kWorkers) {
        wide_worker(sc, row, code, pieces, piece_len, s_dyn64, L);
        return;
    }
    // (one call of the whole-row path for both kinds of rows that take it, at the end: the path is large, and a
    // second copy of it inside this kernel costs every other path registers)
    float whole_m = 0.0f;
    uint32_t whole_argidx = 0;
    if (code == kItemNarrow) {
        if (!narrow_row(d, sc, P, row, slices, L, whole_m, whole_argidx))
            return;
    } else {
        // top_k > 128, no top-p, a candidate list that could not be certified, a nucleus beyond the group records
        BigPlan* gplan = sc.plan + row;
        if (code != kItemWhole || gplan->flag != 2)
            return;
        whole_m = (float)gplan->total64;
        whole_argidx = gplan->n0;
        __syncthreads();
        if (tid == 0)
            gplan->flag = 0;
    }
    general_row<0>(d, sc, row, P, whole_m, whole_argidx, L);
}
#endif // MAKO_EMIT_SORT_KERNELS

} // namespace mako
