// sort_kernel: the top_k == 0 rows planned, their nuclei sorted; rows on the whole-row list.
#pragma once

#include "worker_sort.h"
#include "whole_row.h"
#include "row_records.h"

namespace mako {

#ifdef MAKO_EMIT_SORT_KERNELS // (not a template: defined by the one translation unit that launches it)
// Worker w's weights of the row, cnt of them, collected from the second pass's pieces in any order: as pairs
// (bits(q), token id) into A (LDS) when A is given, else as ~bits(q) and token id into gk / gi (device memory).
// Piece p keeps its weights ordered by worker and a table of where each worker's run starts.  Returns false,
// having written nothing, when the pieces' tables do not add up to cnt (never: cnt was summed from them).
__device__ bool gather_share(const Scratch& sc, uint32_t row, uint32_t pieces, uint32_t piece_len, uint32_t w, uint32_t cnt,
                             uint2* A, uint32_t* gk, uint32_t* gi, FinishShared& sm)
{
    const uint32_t tid = threadIdx.x;
    uint32_t* base = sm.hist;  // [64] first output position of piece p's run
    uint32_t* start = sm.run;  // [64] first entry of the run inside the piece
    if (wave_id() == 0) {
        const uint32_t p = lane_id();
        uint32_t st = 0, len = 0;
        if (p < pieces) {
            const uint32_t* tab = sc.piece_tab + ((size_t)row * sc.pieces_cap + p) * (kWorkers + 1u);
            st = tab[w];
            const uint32_t end = tab[w + 1u];
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

// Smallest and largest of n keys at keys[i * stride] (bits(q), or their complement when `inverted`), as the range
// [key_lo, key_hi) of bits(q) that holds them.  All threads call; all receive the result.
__device__ void share_key_range(const uint32_t* keys, uint32_t stride, uint32_t n, bool inverted, uint32_t& key_lo,
                                uint32_t& key_hi, FinishShared& sm)
{
    uint32_t lo = 0xffffffffu, hi = 0u;
    for (uint32_t e = threadIdx.x; e < n; e += kThreads) {
        const uint32_t k = inverted ? ~keys[(size_t)e * stride] : keys[(size_t)e * stride];
        lo = min(lo, k);
        hi = max(hi, k);
    }
    lo = __ockl_wfred_min_u32(lo);
    hi = __ockl_wfred_max_u32(hi);
    if (lane_id() == 0)
        sm.bs.u64[wave_id()] = ((unsigned long long)hi << 32) | lo;
    __syncthreads();
    lo = 0xffffffffu, hi = 0u;
    for (int w = 0; w < kWaves; ++w) {
        lo = min(lo, (uint32_t)sm.bs.u64[w]);
        hi = max(hi, (uint32_t)(sm.bs.u64[w] >> 32));
    }
    __syncthreads();
    key_lo = lo;
    key_hi = hi + 1u;
}

// One worker's share sorted into kout / iout (cnt entries by (q desc, idx asc), as ~bits(q) and token id).
// sorted_lds: receives the sorted ~bits(q) too when the share fits one LDS sort (see lds_bucket_sort); the function
// returns whether it did.  tk / ti: a second buffer of cnt entries in device memory.
__device__ bool sort_share(const Scratch& sc, uint32_t row, uint32_t pieces, uint32_t piece_len, uint32_t w, uint32_t cnt,
                           uint32_t* kout, uint32_t* iout, uint32_t* tk, uint32_t* ti, unsigned long long* dyn,
                           uint32_t* sorted_lds, const FinishLds& L)
{
    FinishShared& sm = *L.sm;
    uint2* A = reinterpret_cast<uint2*>(dyn);
    uint16_t* B = reinterpret_cast<uint16_t*>(A + kSegCap);
    uint32_t* hist = reinterpret_cast<uint32_t*>(B + kSegCap);
    const uint32_t tid = threadIdx.x;
    bool in_lds = false;
    bool sorted = false;
    uint32_t key_lo, key_hi;
    if (cnt <= kSegCap) {
        for (uint32_t b = tid; b <= kFine; b += kThreads)
            hist[b] = 0;
        if (tid == 0)
            sm.flag = 0;
        if (gather_share(sc, row, pieces, piece_len, w, cnt, A, nullptr, nullptr, sm)) {
            MAKO_STAMP(13);
            share_key_range(&A[0].x, 2u, cnt, false, key_lo, key_hi, sm);
            MAKO_STAMP(14);
            sorted = lds_bucket_sort(cnt, key_lo, key_hi, kout, iout, dyn, sm, sorted_lds);
            in_lds = sorted;
        }
    } else if (gather_share(sc, row, pieces, piece_len, w, cnt, nullptr, tk, ti, sm)) {
        // (the staged form of the share holds bits(q), not their complement)
        for (uint32_t e = tid; e < cnt; e += kThreads)
            tk[e] = ~tk[e];
        __syncthreads();
        share_key_range(tk, 1u, cnt, false, key_lo, key_hi, sm);
        sorted = lds_sort_staged_runs(tk, ti, key_lo, key_hi, cnt, kout, iout, dyn, sm);
    }
    if (!sorted) {
        // crowded buckets (many equal weights): a radix sort of the share through device memory
        MAKO_STAMP(17);
        __syncthreads();
        if (gather_share(sc, row, pieces, piece_len, w, cnt, nullptr, kout, iout, sm))
            sort_segment_unordered(kout, iout, tk, ti, cnt, L);
    }
    return in_lds;
}

// Worker w of a top_k == 0 row: gathers its share of the row's kept weights from the second pass's pieces, sorts it,
// stores it at its place in the row's sorted list and leaves the group records tail_kernel chains.  Where the share
// lies in the list, and the mass ahead of it (from which the running sum's binades are guessed), come from the
// pieces' tables.  All threads call.
__device__ __forceinline__ void wide_worker(const Scratch& sc, uint32_t row, uint32_t w, uint32_t pieces, uint32_t piece_len,
                                            unsigned long long* s_dyn64, const FinishLds& L)
{
    BigPlan* gplan = sc.plan + row;
    const uint32_t flag = gplan->flag;
    // lane v of every wave: the row's kept weights for workers below v (v <= kWorkers), and the mass handed to
    // worker v; every wave works the same numbers out for itself
    const uint32_t v = min((uint32_t)lane_id(), kWorkers);
    uint32_t below = 0;
    unsigned long long mass_v = 0;
    {
        const uint32_t* tabs = sc.piece_tab + (size_t)row * sc.pieces_cap * (kWorkers + 1u);
        const unsigned long long* masses = sc.piece_mass + (size_t)row * sc.pieces_cap * kWorkers;
        for (uint32_t p0 = 0; p0 < pieces; p0 += 8u) { // (eight pieces per trip to memory)
            uint32_t t[8];
            unsigned long long mm[8];
#pragma unroll
            for (uint32_t u = 0; u < 8u; ++u) {
                const uint32_t p = min(p0 + u, pieces - 1u);
                t[u] = tabs[p * (kWorkers + 1u) + v];
                mm[u] = masses[p * kWorkers + min(v, kWorkers - 1u)];
            }
#pragma unroll
            for (uint32_t u = 0; u < 8u; ++u)
                if (p0 + u < pieces) {
                    below += t[u];
                    mass_v += mm[u];
                }
        }
    }
    if (flag != 1)
        return;
    const uint32_t next = (uint32_t)__shfl_down((int)below, 1);
    const uint32_t cnt_v = (uint32_t)lane_id() < kWorkers ? next - below : 0u;
    const uint32_t groups_v = (cnt_v + kGroup - 1u) / kGroup;
    const uint32_t gincl = __ockl_wfscan_add_u32(groups_v, true);
    // (values every lane holds alike go to scalar registers: the sort needs the vector registers)
    const uint32_t n0 = (uint32_t)__builtin_amdgcn_readlane((int)below, kWorkers);
    const uint32_t groups = (uint32_t)__builtin_amdgcn_readlane((int)gincl, kWave - 1);
    const uint32_t off = (uint32_t)__builtin_amdgcn_readlane((int)below, w);
    uint32_t cnt = (uint32_t)__builtin_amdgcn_readlane((int)cnt_v, w);
    const uint32_t gbase = (uint32_t)__builtin_amdgcn_readlane((int)(gincl - groups_v), w);
    const unsigned long long mass_units = __ockl_wfred_add_u64((uint32_t)lane_id() < w ? mass_v : 0ull);
    const double mass = (double)mass_units * 0x1p-30;
    if (w == 0 && threadIdx.x == 0) { // what tail_kernel needs to know of the list
        gplan->n0 = n0;
        gplan->groups = groups;
    }
    // (sound tables never trip these; they keep every store of this worker inside the row's arrays)
    if (n0 > sc.vpad || groups > min(kMaxGroups, sc.g_cap) || off > n0 || cnt > n0 - off)
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
    const bool in_lds =
        sort_share(sc, row, pieces, piece_len, w, cnt, key0 + off, idx0 + off, tk + off, ti + off, s_dyn64, sorted_copy, L);
    MAKO_STAMP(11);
    worker_groups(key0, off, cnt, t_row + gbase, mass, sc.gt, L, in_lds ? sorted_copy : nullptr);
    MAKO_STAMP(12);
}

// Workgroup i serves entry i of the work list second_kernel left (Scratch::work_sort): a worker of a top_k == 0 row, or
// a row on the whole-row path.  The busy workgroups are then the first ones dispatched and land evenly on the XCDs,
// shader engines and CUs, whatever the mix of rows.
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
    const uint32_t item = sc_arg.work_sort[wg]; // (the list has room for every workgroup of the grid)
    if (wg >= n_work)
        return;
    const uint32_t row = item >> 8, code = item & 255u;
    if (row >= d_arg.n_rows)
        return;
    const uint32_t pieces = min((d_arg.n_vocab + kPieceLen - 1u) / kPieceLen, sc_arg.pieces_cap), piece_len = kPieceLen;
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
    // top_k > 128, no top-p, a candidate list that could not be certified, a row beyond the group records
    BigPlan* gplan = sc.plan + row;
    if (code != kItemWhole || gplan->flag != 2)
        return;
    const float whole_m = (float)gplan->total64;
    const uint32_t whole_argidx = gplan->n0;
    __syncthreads();
    if (tid == 0)
        gplan->flag = 0;
    general_row<0>(d, sc, row, P, whole_m, whole_argidx, L);
}
#endif // MAKO_EMIT_SORT_KERNELS

} // namespace mako
