// finish_kernel: the second pass over the top_k == 0 rows.
#pragma once

#include "slice_load.h"
#include "work_split.h"
#include "row_records.h"

namespace mako {

// Exact fp64 sum of q over one slice, and the number of candidates in it (q > 0 and q >= min_p).
// The summation order is fixed: each thread adds its logits in index order, then lanes, then waves.
// (PEN: the row has penalties to apply; a compile-time fact so that each case gets straight-line code of its own.)
// (`slices`: of scan_kernel, whose records give the row maximum; they are asked for behind the piece's own loads)
template <bool VEC, int KH, bool PEN>
__device__ void slice_partial(const mako_sample_desc& d, const Scratch& sc, uint32_t row, uint32_t slice,
                              uint32_t slice_len, const mako_sampling_params& P, uint32_t hl, uint32_t slices,
                              const FinishLds& L)
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
    double sum = 0;
    uint32_t n = 0;
    uint32_t qb[16]; // bits(q), 0 where q is not a candidate
    // (a piece may be shorter than the sixteen logits per thread: whole blocks past its end are skipped; the test is
    // the same for every thread)
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j) {
        qb[j] = 0u;
        if (lo + (VEC ? (j / 4u) * 4096u : j * (uint32_t)kThreads) < hi) {
            const float q = weight_of(wv[j], m, inv_t, sm.tab);
            qb[j] = (q >= floor_q && q > 0.0f) ? __float_as_uint(q) : 0u;
            if (qb[j]) {
                sum += (double)q;
                ++n;
            }
        }
    }
    MAKO_STAMP(25);
    // the piece's sum and count: wave reductions, one exchange of the sixteen waves' results for both (the barrier
    // also retires every use of L.cnt above); they are stored at the very end, so that no barrier waits for the store
    {
        const double sw = __ockl_wfred_add_f64(sum);
        const uint32_t nw = __ockl_wfred_add_u32(n);
        if (lane_id() == 0) {
            sm.bs.f64[wave_id()] = sw;
            sm.bs.u64[wave_id()] = nw;
        }
    }
    lds_barrier();
    // bits(q) of every logit of the slice (0 = not a candidate) and their histogram, for nucleus_big_row()
    uint32_t* qk = reinterpret_cast<uint32_t*>(sc.wbuf + (size_t)row * sc.vpad);
    unsigned long long* hist = reinterpret_cast<unsigned long long*>(L.cnt); // count << kBinSumBits | significands
    for (uint32_t b = threadIdx.x; b < kBins; b += kThreads)
        hist[b] = 0;
    lds_barrier();
    MAKO_STAMP(26);
    // one candidate and the significand of a positive float (subnormals: no hidden bit, as seqfp::split)
    auto record = [](uint32_t b) {
        return (1ull << kBinSumBits) | (unsigned long long)((b & 0x7fffffu) | ((b >> 23) ? 0x800000u : 0u));
    };
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j)
        if (qb[j])
            atomicAdd(&hist[weight_bin(qb[j])], record(qb[j]));
    if (VEC) {
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint32_t i = lo + k * 4096u + threadIdx.x * 4u;
            if (i < hi)
                *reinterpret_cast<uint4*>(qk + i) = make_uint4(qb[4 * k], qb[4 * k + 1], qb[4 * k + 2], qb[4 * k + 3]);
        }
    } else {
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j) {
            const uint32_t i = lo + j * (uint32_t)kThreads + threadIdx.x;
            if (i < hi)
                qk[i] = qb[j];
        }
    }
    lds_barrier(); // (the histogram is complete; nobody waits for the stores above)
    MAKO_STAMP(27);
    // the slice's non-empty bins are added to the row's histogram (a few hundred atomics per slice, none waited for)
    unsigned long long* bins = sc.bins + (size_t)row * kBins;
    for (uint32_t b = threadIdx.x; b < kBins; b += kThreads)
        if (hist[b])
            atomicAdd(&bins[b], hist[b]);
    if (threadIdx.x == 0) {
        double total = 0;
        uint32_t count = 0;
        for (int w = 0; w < kWaves; ++w) { // waves in order: the same inputs always give the same bits
            total += sm.bs.f64[w];
            count += (uint32_t)sm.bs.u64[w];
        }
        sc.part_sum[(size_t)row * kMaxSlices + slice] = total;
        sc.part_n[(size_t)row * kMaxSlices + slice] = count;
    }
}

// Second pass over the top_k == 0 rows.  grid = (most pieces a row can have, rows) workgroups, of which workgroup i
// serves the i-th piece of work in row order, second_pass_pieces() per top_k == 0 row (find_piece): the busy
// workgroups are then the first ones dispatched and land evenly on the XCDs, shader engines and CUs, whatever the
// mix of rows.
template <bool VEC, int KH>
__global__ __launch_bounds__(kThreads) void finish_kernel(mako_sample_desc d_arg, const Scratch* sc_dev, uint32_t slices)
{
    const Scratch& sc_arg = *sc_dev;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
#ifdef MAKO_TIMING_FINISH
    MAKO_WG_TIMER;
#endif
    // What the workgroup needs before it can ask for its logits is asked for in as few trips to memory as possible
    // (each costs most of a microsecond here, and the pass starts with nothing else to do): the rows' parameters
    // for find_piece() and the arguments' copy go out together with the cut, and the row's own parameters are then
    // taken from the lane that loaded them.
    const uint32_t wg = blockIdx.y * gridDim.x + blockIdx.x, tid = threadIdx.x;
    const bool by_lane = d_arg.n_rows <= (uint32_t)kWave; // uniform
    mako_sampling_params P_lane = mako_sampling_params{};
    if (by_lane)
        P_lane = d_arg.params[min((uint32_t)lane_id(), d_arg.n_rows - 1u)];
    stage_args_only(d_arg, sc_arg, s_args);
    // (pieces per row, their length, workgroups with work: the others leave at once)
    const uint4 cut = *reinterpret_cast<const uint4*>(sc_arg.work_n + 4);
    if (wg >= cut.z)
        return;
    const uint32_t pieces = cut.x, piece_len = cut.y;
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
    const uint32_t hl = d.hist_tokens ? min(d.hist_len[row], (uint32_t)d.hist_stride) : 0u;
    // (a row without history entries takes the penalising variant too when it has penalties: it finds nothing to
    // penalise, and nothing here waits for the length)
    if (d.hist_tokens && !penalties_neutral(P))
        slice_partial<VEC, KH, true>(d, sc, row, piece, piece_len, P, hl, slices, L);
    else
        slice_partial<VEC, KH, false>(d, sc, row, piece, piece_len, P, hl, slices, L);
}

} // namespace mako
