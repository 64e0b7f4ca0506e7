// second_kernel: the second pass over the top_k == 0 rows, and beside it the rows that need none.
#pragma once

#include "slice_load.h"
#include "work_split.h"
#include "row_records.h"
#include "rows_kernel.h"
#include "nucleus_plan.h"

namespace mako {

// Exact fp64 sum of q over one slice, and the number of candidates in it (q > 0 and q >= min_p).
// The summation order is fixed: each thread adds its logits in index order, then lanes, then waves.
// (PEN: the row has penalties to apply; a compile-time fact so that each case gets straight-line code of its own.)
// (`slices`: of scan_kernel, whose records give the row maximum; they are asked for behind the piece's own loads)
// Returns true in the workgroup that finishes the row's last piece (`pieces` of them), which goes on to plan the row.
template <bool VEC, int KH, bool PEN>
__device__ bool slice_partial(const mako_sample_desc& d, const Scratch& sc, uint32_t row, uint32_t slice,
                              uint32_t slice_len, const mako_sampling_params& P, uint32_t hl, uint32_t slices,
                              uint32_t pieces, const FinishLds& L)
{
    FinishShared& sm = *L.sm;
    const uint32_t lo = slice * slice_len;
    const uint32_t hi = min(d.n_vocab, lo + slice_len);
    constexpr bool pen = PEN;
    float wv[16];
    float m = 0.0f;
    load_penalised<VEC, KH>(d, row, lo, hi, slice_len, P, hl, pen, L.cnt, wv, [&]() {
        uint32_t argidx, n_cands, any_overflow;
        row_summary(sc, row, slices, m, argidx, n_cands, any_overflow);
    });
    MAKO_STAMP(1);
    MAKO_STAMP(24);
    const float inv_t = 1.0f / P.temperature;
    const float floor_q = (1.0f < P.min_p) ? 1.0f : P.min_p;
    uint32_t qb[16]; // bits(q), 0 where q is not a candidate
    // (a piece may be shorter than the sixteen logits per thread: whole blocks past its end are skipped; the test is
    // the same for every thread)
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j) {
        qb[j] = 0u;
        if (lo + (VEC ? (j / 4u) * 4096u : j * (uint32_t)kThreads) < hi) {
            const float q = weight_of(wv[j], m, inv_t, sm.tab);
            qb[j] = (q >= floor_q && q > 0.0f) ? __float_as_uint(q) : 0u;
        }
    }
    MAKO_STAMP(25);
    // The piece's histogram (exact bin masses: the row's total comes from them), and the piece's weights ordered by
    // bin from the heaviest down: each weight's returning atomic also tells its place among the weights of its bin.
    // Bins below b_prune hold weights the nucleus cannot reach (prune_bin()): counted and summed like the others,
    // but not kept.  (The histogram was cleared by second_kernel before the loads; it lies outside the token counts.)
    char* dyn = reinterpret_cast<char*>(L.cnt);
    unsigned long long* hist = reinterpret_cast<unsigned long long*>(dyn + kSecondHistAt); // count << kBinSumBits | significands
    uint32_t* above = reinterpret_cast<uint32_t*>(dyn + kSecondAboveAt);   // [kBins] kept weights in higher bins
    uint32_t* skey = reinterpret_cast<uint32_t*>(dyn + kSecondKeysAt);     // [piece] kept weights in bin order
    uint16_t* sidx = reinterpret_cast<uint16_t*>(dyn + kSecondIdxAt);      // [piece] and their places in the piece
    MAKO_STAMP(26);
    const uint32_t b_prune = prune_bin(P, d.n_vocab);
    // one candidate and the significand of a positive float (subnormals: no hidden bit, as seqfp::split)
    auto record = [](uint32_t b) {
        return (1ull << kBinSumBits) | (unsigned long long)((b & 0x7fffffu) | ((b >> 23) ? 0x800000u : 0u));
    };
    uint32_t place[16]; // bin << 16 | place inside the bin (a piece holds at most 16384 weights); kNone: not kept
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j) {
        place[j] = kNone;
        if (qb[j]) {
            const uint32_t b = weight_bin(qb[j]);
            const unsigned long long old = atomicAdd(&hist[b], record(qb[j]));
            if (b >= b_prune)
                place[j] = (b << 16) | (uint32_t)(old >> kBinSumBits);
        }
    }
    lds_barrier(); // (the histogram is complete)
    MAKO_STAMP(27);
    // What the row's plan needs of this piece sets out first: its non-empty bins are added to the row's histogram (a
    // few hundred atomics per piece).  The planner reads them from another workgroup, so these are operations of
    // device scope, complete before this workgroup takes its ticket below.
    const uint32_t b0 = kBins - 1u - 2u * threadIdx.x, b1 = b0 - 1u; // thread t holds bins kBins - 1 - 2t and kBins - 2 - 2t
    const unsigned long long h0 = hist[b0], h1 = hist[b1];
    {
        unsigned long long* bins = sc.bins + (size_t)row * kBins;
        if (h0)
            atomicAdd(&bins[b0], h0);
        if (h1)
            atomicAdd(&bins[b1], h1);
    }
    // kept weights above each bin, from the top bin down (barriers that order LDS only)
    uint32_t kept = 0;
    {
        const uint32_t c0 = b0 >= b_prune ? (uint32_t)(h0 >> kBinSumBits) : 0u;
        const uint32_t c1 = b1 >= b_prune ? (uint32_t)(h1 >> kBinSumBits) : 0u;
        const uint32_t incl = __ockl_wfscan_add_u32(c0 + c1, true);
        if (lane_id() == kWave - 1)
            sm.hist[wave_id()] = incl;
        lds_barrier();
        uint32_t ex = incl - (c0 + c1);
        for (int w = 0; w < kWaves; ++w) {
            const uint32_t x = sm.hist[w];
            ex += w < wave_id() ? x : 0u;
            kept += x;
        }
        above[b0] = ex;
        above[b1] = ex + c0;
        // the piece's table: kept weights in bins >= b
        uint16_t* tab = sc.piece_tab + ((size_t)row * sc.pieces_cap + slice) * (kBins + 1u);
        tab[b0] = (uint16_t)(ex + c0);
        tab[b1] = (uint16_t)(ex + c0 + c1);
        if (threadIdx.x == 0)
            tab[kBins] = 0;
    }
    lds_barrier();
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j)
        if (place[j] != kNone) {
            const uint32_t at = above[place[j] >> 16] + (place[j] & 0xffffu);
            skey[at] = qb[j];
            sidx[at] = (uint16_t)(VEC ? (j >> 2) * 4096u + threadIdx.x * 4u + (j & 3u) : j * (uint32_t)kThreads + threadIdx.x);
        }
    lds_barrier();
    MAKO_STAMP(28);
    // out, four weights per store (a piece starts at a multiple of four; what lies past `kept` is never read)
    {
        const size_t at = (size_t)row * sc.vpad + lo;
        uint4* gk = reinterpret_cast<uint4*>(sc.key[1] + at);
        uint2* gi = reinterpret_cast<uint2*>(sc.piece_idx + at);
        const uint4* lk = reinterpret_cast<const uint4*>(skey);
        const uint2* li = reinterpret_cast<const uint2*>(sidx);
        for (uint32_t i = threadIdx.x; i * 4u < kept; i += kThreads) {
            gk[i] = lk[i];
            gi[i] = li[i];
        }
    }
    // (this barrier also waits for every wave's atomics and stores above: the piece's part of the row's histogram
    // is in place, and the ticket may be taken)
    __syncthreads();
    if (threadIdx.x == 0)
        sm.ticket = atomicAdd(&sc.row_ticket[row], 1u);
    __syncthreads();
    return sm.ticket == pieces - 1u;
}

// The row's plan, by the workgroup that finished the last piece of its second pass: the exact total and the histogram
// of the row's weights decide how far down the nucleus can reach; a narrow nucleus goes to sort_kernel as one piece
// of work, a wide one as kWorkers pieces with the workers' value ranges in the row's BigPlan.  The other pieces'
// bins were added by other workgroups, through other L2 caches: they are read with loads of device scope.
__device__ void plan_row(const mako_sample_desc& d, const Scratch& sc, const mako_sampling_params& P, uint32_t row,
                         uint32_t slices, uint32_t pieces, BigPlan& s_plan, const FinishLds& L)
{
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
    if (tid == 0)
        sc.row_ticket[row] = 0; // (for the next batch)
    const unsigned long long* bins = sc.bins + (size_t)row * kBins;
    const unsigned long long rec0 = __hip_atomic_load(&bins[kBins - 1u - 2u * tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned long long rec1 = __hip_atomic_load(&bins[kBins - 2u - 2u * tid], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    float m;
    uint32_t argidx, n_cands, any_overflow;
    row_summary(sc, row, slices, m, argidx, n_cands, any_overflow);
    const uint32_t bin_c0 = (uint32_t)(rec0 >> kBinSumBits), bin_c1 = (uint32_t)(rec1 >> kBinSumBits);
    const unsigned long long bin_s0 = rec0 & ((1ull << kBinSumBits) - 1ull), bin_s1 = rec1 & ((1ull << kBinSumBits) - 1ull);
    MAKO_STAMP(15);
    uint32_t thr_bits = 0, row_n0 = 0;
    double row_total = 0;
    const uint32_t n0_plan =
        plan_nucleus(P, bin_c0, bin_c1, bin_s0, bin_s1, prune_bin(P, d.n_vocab), &s_plan, L, thr_bits, row_total, row_n0);
    MAKO_STAMP(16);
    if (row_n0 == 0) { // (no candidate survived: sampler.cpp:37-38)
        fallback_row(d, row, argidx);
        return;
    }
    const uint32_t n0 = min(n0_plan, d.n_vocab);
    const bool narrow = !d.draft && n0 <= kSmall && !any_overflow && n_cands <= kSortMax;
    // (a list too long for the workers' group records goes to the whole-row path)
    const bool fits = n0 <= kGroup * (kMaxGroups - kWorkers);
    BigPlan* gplan = sc.plan + row;
    if (fits && !narrow) { // the workers' ranges
        static_assert(sizeof(BigPlan) % 4 == 0, "word copies");
        const uint32_t* src = reinterpret_cast<const uint32_t*>(&s_plan);
        uint32_t* dst = reinterpret_cast<uint32_t*>(gplan);
        for (uint32_t i = 8u + tid; i < sizeof(BigPlan) / 4u; i += kThreads) // (the record's head is written below)
            dst[i] = src[i];
    }
    const uint32_t work = (fits && !narrow) ? kWorkers : 1u;
    if (tid == 0) {
        gplan->n0 = fits ? n0 : argidx;                        // (the whole-row path is handed the row maximum and
        gplan->total64 = fits ? row_total : (double)m;         // its first index here)
        gplan->groups = min(s_plan.groups, kMaxGroups);
        gplan->thr = thr_bits;
        gplan->flag = !fits ? 2u : (narrow ? 3u : 1u);
        sm.flag = atomicAdd(&sc.work_n[0], work);
        if (fits && !narrow)
            sc.work_tail[atomicAdd(&sc.work_n[1], 1u)] = row;
    }
    __syncthreads();
    if (tid < work)
        sc.work_sort[sm.flag + tid] = (row << 8) | (!fits ? kItemWhole : (narrow ? kItemNarrow : tid));
}

// The launch behind scan_kernel.  Workgroups [0, busy) take the second pass over the top_k == 0 rows: workgroup i
// serves piece i % pieces of the (i / pieces)-th such row (the cut and the rows are scan_kernel's, Scratch::work_n and
// work_rows), so the busy workgroups are the first ones dispatched and land evenly on the XCDs, shader engines and
// CUs, whatever the mix of rows.  Workgroup busy + r then finishes row r if it needs no second pass (finish_row()).
template <bool VEC, int KH>
__global__ __launch_bounds__(kThreads) void second_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    const Scratch& sc_arg = sc_val;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    __shared__ BigPlan s_plan;
#ifdef MAKO_TIMING_FINISH
    MAKO_WG_TIMER;
#endif
    // What the workgroup needs before it can ask for its logits is asked for in as few trips to memory as possible
    // (each costs most of a microsecond here, and the pass starts with nothing else to do): the rows' parameters
    // and the arguments' copy go out together with the cut, and the row's own parameters are then taken from the
    // lane that loaded them.
    const uint32_t wg = blockIdx.x, tid = threadIdx.x;
    const bool by_lane = d_arg.n_rows <= (uint32_t)kWave; // uniform
    mako_sampling_params P_lane = mako_sampling_params{};
    uint32_t hl_lane = 0; // (the histories' lengths too: one trip less before the history can be asked for)
    if (by_lane) {
        P_lane = d_arg.params[min((uint32_t)lane_id(), d_arg.n_rows - 1u)];
        if (d_arg.hist_tokens)
            hl_lane = d_arg.hist_len[min((uint32_t)lane_id(), d_arg.n_rows - 1u)];
    }
    stage_args_only(d_arg, sc_arg, s_args);
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    // (pieces per row, their length, workgroups of the second pass, top_k == 0 rows)
    const uint4 cut = *reinterpret_cast<const uint4*>(sc_arg.work_n + 4);
    const uint32_t pieces = cut.x, piece_len = cut.y, busy = cut.z;
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;                                             // 32 KB
    L.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);    // next 16 KB
    if (wg >= busy) {
        const uint32_t row = wg - busy;
        if (row >= d_arg.n_rows)
            return;
        MAKO_ROW(row);
        stage_params(d_arg.params[row], s_args);
        __syncthreads(); // (publishes the arguments, the parameters and the table)
#ifndef K2_NO_ROWS
        finish_row<false>(s_args.d, s_args.sc, s_args.P, row, slices, L);
#endif
        return;
    }
    uint32_t row, piece, hl_row = 0;
    if (by_lane) {
        // one row per lane, every wave for itself: the lane whose row owns workgroup wg's piece
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
        hl_row = (uint32_t)__builtin_amdgcn_readlane((int)hl_lane, owner);
        stage_params(P_row, s_args);
    } else {
        row = min(sc_arg.work_rows[wg / pieces], d_arg.n_rows - 1u);
        piece = wg % pieces;
        stage_params(d_arg.params[row], s_args);
        if (d_arg.hist_tokens)
            hl_row = d_arg.hist_len[row];
    }
    MAKO_ROW(row);
    { // the piece's histogram starts empty (it lies outside the token counts, which the loading code clears)
        uint4* hz = reinterpret_cast<uint4*>(reinterpret_cast<char*>(s_dyn64) + kSecondHistAt);
        for (uint32_t i = tid; i < kBins * 8u / 16u; i += kThreads)
            hz[i] = make_uint4(0, 0, 0, 0);
    }
    __syncthreads(); // (publishes the arguments, the parameters, the table and the cleared histogram)
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    const mako_sampling_params& P = s_args.P;
    MAKO_STAMP(0);
    if (d.force_token || d.close_token) { // a forced row needs no weights (its token is written by finish_row())
        int32_t ftok;
        uint32_t above;
        if (row_forced(d, sc, row, slices, ftok, above) != MAKO_FORCED_NONE)
            return;
    }
    // (inside slice_partial the history, the logits and the slices' records: one trip)
    const uint32_t hl = d.hist_tokens ? min(hl_row, (uint32_t)d.hist_stride) : 0u;
    // (a row without history entries takes the penalising variant too when it has penalties: it finds nothing to
    // penalise, and nothing here waits for the length)
    bool last;
    if (d.hist_tokens && !penalties_neutral(P))
        last = slice_partial<VEC, KH, true>(d, sc, row, piece, piece_len, P, hl, slices, pieces, L);
    else
        last = slice_partial<VEC, KH, false>(d, sc, row, piece, piece_len, P, hl, slices, pieces, L);
#ifndef K2_NO_PLAN
    if (last)
        plan_row(d, sc, P, row, slices, pieces, s_plan, L);
#endif
}

} // namespace mako
