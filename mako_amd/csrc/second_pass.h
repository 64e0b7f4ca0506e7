// second_kernel: the second pass over the top_k == 0 rows.
#pragma once

#include "slice_load.h"
#include "work_split.h"
#include "row_records.h"
#include "row_output.h"
#include "nucleus_plan.h"

namespace mako {

// One piece of the second pass over a top_k == 0 row: q of every logit of the piece, the piece's fp64 sum of q
// and its number of candidates (q > 0 and q >= min_p), and the piece's kept weights handed to the row's workers.
//
// Which weights are kept, and who gets them: every piece computes q of the same kSamples logits of the row, one per
// thread, and sample_plan() turns their histogram into the lowest bin kept (a guess of how far down the nucleus
// reaches, never below prune_bin(); the other weights are summed and counted, nothing else) and a bin -> worker
// table; a weight's place among its worker's weights comes from one returning LDS atomic per weight on a counter
// per worker and sixteenth of the lanes, which the split keeps evenly loaded.  The kept weights leave the workgroup ordered by worker, with a table of where each
// worker's run starts.
// The summation order of the piece's sum is fixed: each thread adds its logits in index order, then lanes, then waves.
// (PEN: the row has penalties to apply; a compile-time fact so that each case gets straight-line code of its own.)
// (`slices`: of scan_kernel, whose records give the row maximum; they are asked for behind the piece's own loads)
template <bool VEC, int KH, bool PEN>
__device__ void slice_partial(const mako_sample_desc& d, const Scratch& sc, uint32_t row, uint32_t slice,
                              uint32_t slice_len, const mako_sampling_params& P, uint32_t hl, uint32_t slices,
                              const FinishLds& L)
{
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
    const uint32_t lo = slice * slice_len;
    const uint32_t hi = min(d.n_vocab, lo + slice_len);
    constexpr bool pen = PEN;
    char* dyn = reinterpret_cast<char*>(L.cnt);
    uint32_t* skey = reinterpret_cast<uint32_t*>(dyn + kSecondKeysAt);   // [piece] kept weights, ordered by worker
    uint16_t* sidx = reinterpret_cast<uint16_t*>(dyn + kSecondIdxAt);    // [piece] and their places in the piece
    uint32_t* shist = reinterpret_cast<uint32_t*>(dyn + kSecondHistAt);  // [kBins] histogram of the sampled weights
    uint8_t* table = reinterpret_cast<uint8_t*>(dyn + kSecondTableAt);   // [kBins] bin -> worker
    // [kWorkers][16] weights handed over << kMassBits | their mass in units of 2^-30: a counter per worker and per
    // sixteenth of the lanes (lane & 15), so that the lanes of one atomic instruction rarely meet at one address
    unsigned long long* wcnt = reinterpret_cast<unsigned long long*>(dyn + kSecondCntAt);
    uint32_t* woff = reinterpret_cast<uint32_t*>(dyn + kSecondOffAt);    // [kWorkers][16] their first places
    uint32_t* cut = reinterpret_cast<uint32_t*>(dyn + kSecondCutAt);     // [kWorkers] cuts between the workers
    constexpr uint32_t kPer = 4u * kPieceBlocks; // logits per thread
    float wv[kPer];
    float m = 0.0f;
    float sample_raw = 0.0f;
    uint32_t sample_ok = 1u, argidx = 0;
    load_penalised<VEC, KH, kPieceBlocks>(d, row, lo, hi, slice_len, P, hl, pen, L.cnt, wv, [&]() {
        uint32_t n_cands, any_overflow;
        row_summary(sc, row, slices, m, argidx, n_cands, any_overflow);
        // this thread's sample of the row (the mask honoured, penalties ignored: the split need not be exact)
        const uint32_t si = min(d.n_vocab - 1u, (uint32_t)(((unsigned long long)tid * d.n_vocab + d.n_vocab / 2u) / kSamples));
        sample_raw = d.logits[(int64_t)row * d.logits_stride + si];
        if (d.mask)
            sample_ok = (d.mask[(int64_t)row * d.mask_stride + (si >> 5)] >> (si & 31u)) & 1u;
    });
    MAKO_STAMP(1);
    MAKO_STAMP(24);
    const float inv_t = 1.0f / P.temperature;
    const float floor_q = (1.0f < P.min_p) ? 1.0f : P.min_p;
    const uint32_t b_prune = prune_bin(P, d.n_vocab);
    {
        const float q = weight_of(sample_ok ? sample_raw : -INFINITY, m, inv_t, sm.tab);
        if (q >= floor_q && q > 0.0f) {
            const uint32_t b = weight_bin(min(__float_as_uint(q), 0x3f800000u));
            if (b >= b_prune)
                atomicAdd(&shist[b], 1u);
        }
    }
    lds_barrier();
    uint32_t b_keep;
    const uint32_t workers =
        sample_plan(shist, table, cut, d.n_vocab, P.top_p, b_prune, *reinterpret_cast<SamplePlanLds*>(sm.hist), b_keep);
    double sum = 0;
    uint32_t n = 0;
    uint32_t qb[kPer]; // bits(q), 0 where q is not a candidate
    // (the row's last piece may be shorter: whole blocks past its end are skipped; the test is the same for every
    // thread)
#pragma unroll
    for (uint32_t j = 0; j < kPer; ++j) {
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
    // the piece's sum and count: wave reductions, one exchange of the sixteen waves' results for both
    {
        const double sw = __ockl_wfred_add_f64(sum);
        const uint32_t nw = __ockl_wfred_add_u32(n);
        if (lane_id() == 0) {
            sm.bs.f64[wave_id()] = sw;
            sm.bs.u64[wave_id()] = nw;
        }
    }
    lds_barrier(); // (the table is in place; every use of the token counts above is over)
    MAKO_STAMP(26);
    double piece_total = 0;
    uint32_t piece_count = 0;
    if (tid == 0)
        for (int w = 0; w < kWaves; ++w) { // waves in order: the same inputs always give the same bits
            piece_total += sm.bs.f64[w];
            piece_count += (uint32_t)sm.bs.u64[w];
        }
    uint32_t place[kPer]; // worker << 16 | place among the weights of that worker's counter; kNone: not kept
    const uint32_t sub = threadIdx.x & 15u;
    {
        // in steps that keep eight LDS operations in flight each: the bins' first workers, the cuts below them
        // (a weight under the cut belongs to the next worker), then the counters
        uint32_t dest[kPer];
#pragma unroll
        for (uint32_t j = 0; j < kPer; ++j) {
            const uint32_t b = qb[j] ? weight_bin(qb[j]) : 0u;
            dest[j] = (qb[j] && b >= b_keep) ? (uint32_t)table[b] : kNone;
        }
#pragma unroll
        for (uint32_t step = 0; step < 2u; ++step) {
            uint32_t c[kPer];
#pragma unroll
            for (uint32_t j = 0; j < kPer; ++j)
                c[j] = cut[min(dest[j] + 1u, kWorkers - 1u)]; // (kNone + 1 = 0: a slot nobody compares against)
#pragma unroll
            for (uint32_t j = 0; j < kPer; ++j)
                if (dest[j] != kNone && dest[j] + 1u < workers && qb[j] < c[j])
                    ++dest[j];
        }
#pragma unroll
        for (uint32_t j = 0; j < kPer; ++j) {
            place[j] = kNone;
            if (dest[j] != kNone) {
                while (dest[j] + 1u < workers && qb[j] < cut[dest[j] + 1u]) // (more than two cuts inside one bin)
                    ++dest[j];
                // (one atomic for the place and the mass; mass below 2^-30 does not move a guess)
                const unsigned long long rec =
                    (1ull << kMassBits) | (unsigned long long)(uint32_t)(__uint_as_float(qb[j]) * 0x1p30f);
                place[j] = (dest[j] << 16) | (uint32_t)(atomicAdd(&wcnt[dest[j] * 16u + sub], rec) >> kMassBits);
            }
        }
    }
    lds_barrier();
    MAKO_STAMP(27);
    // first places, workers in order and within a worker its sixteen counters in order: thread t < 16 * kWorkers
    // takes counter t
    {
        const uint32_t dw = tid / 16u, ww = tid % 16u;
        const unsigned long long rec = tid < 16u * kWorkers ? wcnt[tid] : 0ull;
        const uint32_t v = (uint32_t)(rec >> kMassBits);
        // (the worker's mass over its sixteen counters: sixteen neighbouring lanes)
        unsigned long long wm = rec & ((1ull << kMassBits) - 1ull);
        for (int o = 1; o < 16; o <<= 1)
            wm += __shfl_xor(wm, o);
        if (tid < 16u * kWorkers && ww == 0)
            sc.piece_mass[((size_t)row * sc.pieces_cap + slice) * kWorkers + dw] = wm;
        const uint32_t incl = __ockl_wfscan_add_u32(v, true);
        if (lane_id() == kWave - 1)
            sm.hist[wave_id()] = incl;
        lds_barrier();
        uint32_t ex = incl - v, kept = 0;
        for (int w = 0; w < kWaves; ++w) {
            const uint32_t x = sm.hist[w];
            ex += w < wave_id() ? x : 0u;
            kept += x;
        }
        if (tid < 16u * kWorkers)
            woff[tid] = ex;
        // the piece's table: kept weights for workers below w
        uint32_t* tab = sc.piece_tab + ((size_t)row * sc.pieces_cap + slice) * (kWorkers + 1u);
        if (tid < 16u * kWorkers && ww == 0)
            tab[dw] = ex;
        if (tid == 0)
            tab[kWorkers] = kept;
        sm.run[0] = kept; // (every thread writes the same value)
    }
    lds_barrier();
    const uint32_t kept = sm.run[0];
#pragma unroll
    for (uint32_t j = 0; j < kPer; ++j)
        if (place[j] != kNone) {
            const uint32_t at = woff[(place[j] >> 16) * 16u + sub] + (place[j] & 0xffffu);
            skey[at] = qb[j];
            sidx[at] = (uint16_t)(VEC ? (j >> 2) * 4096u + tid * 4u + (j & 3u) : j * (uint32_t)kThreads + tid);
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
        for (uint32_t i = tid; i * 4u < kept; i += kThreads) {
            gk[i] = lk[i];
            gi[i] = li[i];
        }
    }
    if (tid == 0) {
        sc.piece_sum[(size_t)row * sc.pieces_cap + slice] = piece_total;
        sc.piece_cnt[(size_t)row * sc.pieces_cap + slice] = piece_count;
    }
    // the row's first piece puts the row's workers on sort_kernel's list and the row on tail_kernel's
    // (a row too long for the workers' group records takes the whole-row path)
    if (slice == 0) {
        const bool fits = d.n_vocab <= kGroup * (kMaxGroups - kWorkers);
        if (tid == 0) {
            BigPlan* gplan = sc.plan + row;
            gplan->workers = workers;
            gplan->thr = bin_lo_key(b_keep);
            gplan->flag = fits ? 1u : 2u;
            if (!fits) {
                gplan->total64 = (double)m; // carries the row maximum and its first index to the whole-row path
                gplan->n0 = argidx;
            }
            sm.flag = atomicAdd(&sc.work_n[0], fits ? workers : 1u);
            if (fits)
                sc.work_tail[atomicAdd(&sc.work_n[1], 1u)] = row;
        }
        __syncthreads();
        if (tid < (fits ? workers : 1u))
            sc.work_sort[sm.flag + tid] = (row << 8) | (fits ? tid : kItemWhole);
    }
}

// The second pass over the top_k == 0 rows, the launch behind scan_kernel: workgroup i serves piece i % pieces of the
// (i / pieces)-th such row (Scratch::work_rows, scan_kernel's list), pieces of kPieceLen logits.  Two workgroups share a
// CU (eight waves per SIMD: 64 vector registers; under 80 KB of LDS): one's waits are the other's work.
template <bool VEC, int KH>
__global__ __launch_bounds__(kThreads, 8) void second_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices,
                                                               uint32_t pieces)
{
    const Scratch& sc_arg = sc_val;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
#ifdef MAKO_TIMING_FINISH
    MAKO_WG_TIMER;
#endif
    // What the workgroup needs before it can ask for its logits is asked for in as few trips to memory as possible
    // (each costs most of a microsecond here, and the pass starts with nothing else to do): the list's length and
    // this workgroup's row go out together with the arguments' copy.
    const uint32_t wg = blockIdx.x, tid = threadIdx.x;
    const uint32_t n_nucleus = sc_arg.work_n[4];
    const uint32_t row = min(sc_arg.work_rows[min(wg / pieces, d_arg.n_rows - 1u)], d_arg.n_rows - 1u);
    const uint32_t piece = wg % pieces;
    stage_args_only(d_arg, sc_arg, s_args);
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    { // the sample histogram and the workers' counters start empty (they lie outside the token counts, which the
      // loading code clears)
        static_assert(kSecondTableAt == kSecondHistAt + kBins * 4u && kSecondLds % 16u == 0 && kSecondHistAt % 16u == 0,
                      "one run of 16-byte words from the histogram to the end of the block");
        uint4* hz = reinterpret_cast<uint4*>(reinterpret_cast<char*>(s_dyn64) + kSecondHistAt);
        for (uint32_t i = tid; i < (kSecondLds - kSecondHistAt) / 16u; i += kThreads)
            hz[i] = make_uint4(0, 0, 0, 0);
    }
    if (wg >= n_nucleus * pieces)
        return;
    // second trip: the row's parameters and the history's length
    const mako_sampling_params P_row = d_arg.params[row];
    const uint32_t hl_row = d_arg.hist_tokens ? d_arg.hist_len[row] : 0u;
    stage_params(P_row, s_args);
    MAKO_ROW(row);
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;
    L.wcount = nullptr;
    __syncthreads(); // (publishes the arguments, the parameters, the table and the cleared counters)
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
    if (d.hist_tokens && !penalties_neutral(P))
        slice_partial<VEC, KH, true>(d, sc, row, piece, kPieceLen, P, hl, slices, L);
    else
        slice_partial<VEC, KH, false>(d, sc, row, piece, kPieceLen, P, hl, slices, L);
}

} // namespace mako
