// Planning a top_k == 0 row from the exact histogram of its weights.
#pragma once

#include "workgroup_state.h"

namespace mako {

// Plans a top_k == 0 row from the histogram of its weights (weight_bin(), exact masses): finds the bin by
// which the nucleus must have ended and splits the weights above it over kWorkers workers by value.
// Thread t brings the counts (c0, c1) and significand sums (s0, s1) of bins kBins-1-2t and kBins-2-2t.
// Returns n0, the number of weights to sort; the plan is written to `plan` (flag left untouched).
__device__ uint32_t plan_nucleus(const mako_sampling_params& P, double total64, uint32_t c0, uint32_t c1,
                                 unsigned long long s0, unsigned long long s1, BigPlan* plan, uint8_t* bin_worker,
                                 const FinishLds& L, uint32_t& thr_bits, uint32_t n_vocab)
{
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
    const uint32_t b0 = kBins - 1u - 2u * tid, b1 = b0 - 1u;
    // exact mass of a bin: sum of significands times the bin's power of two (bins never straddle a binade)
    auto scale = [](uint32_t b) {
        const uint32_t e = max(bin_lo_key(b) >> 23, 1u); // biased exponent of the bin's weights (subnormals: 1)
        return __longlong_as_double((long long)(1023ull + e - 150ull) << 52);
    };
    const double m0 = (double)s0 * scale(b0), m1 = (double)s1 * scale(b1);
    // (what the reference's sums can make of `want`, at most: see order_band())
    const double want = (double)P.top_p * total64 + 2.0 * order_band(n_vocab, total64);
    uint32_t* w_hi = L.wcount;            // highest bin of each worker
    uint32_t* w_lo = L.wcount + kWorkers; // lowest bin
    uint32_t* w_off = L.wcount + 2 * kWorkers;
    uint32_t* w_cnt = L.wcount + 3 * kWorkers;
    if (tid < kWorkers) {
        w_hi[tid] = 0;
        w_lo[tid] = kNone;
        w_off[tid] = kNone;
        w_cnt[tid] = 0;
    }
    // running mass (inclusive) and candidates above each bin (exclusive), from the top bin down: wave scans, and
    // one exchange of the sixteen waves' totals for both
    const double mass_w = __ockl_wfscan_add_f64(m0 + m1, true);
    const uint32_t cnt_w = __ockl_wfscan_add_u32(c0 + c1, true);
    if (lane_id() == kWave - 1) {
        sm.bs.f64[wave_id()] = mass_w;
        sm.bs.u64[wave_id()] = cnt_w;
    }
    __syncthreads();
    double pre_m = 0;
    uint32_t pre_c = 0, count_all = 0;
    for (int w = 0; w < kWaves; ++w) {
        const double x = sm.bs.f64[w];
        const uint32_t y = (uint32_t)sm.bs.u64[w];
        if (w < wave_id()) {
            pre_m += x;
            pre_c += y;
        }
        count_all += y;
    }
    MAKO_STAMP(20);
    const double incl = pre_m + mass_w;
    const uint32_t above0 = pre_c + cnt_w - (c0 + c1), above1 = above0 + c0;
    // The nucleus ends by the first bin (from the top) at which the running mass reaches `want`: these sums
    // associate differently from the sorted prefix sums that make the final decision and from the reference's, and
    // `want` carries the band by which any of them can differ.
    const bool r0 = c0 && incl - m1 >= want, r1 = c1 && incl >= want;
    const uint32_t reached = (uint32_t)r0 + (uint32_t)r1;
    const uint32_t reached_w = __ockl_wfscan_add_u32(reached, true);
    if (lane_id() == kWave - 1)
        sm.hist[wave_id()] = reached_w;
    if (tid == 0) {
        sm.ticket = 0;        // the lowest bin taken; never reached: every candidate is kept
        sm.flag = count_all;  // the number of weights to sort
    }
    __syncthreads();
    uint32_t before = reached_w - reached;
    for (int w = 0; w < kWaves; ++w)
        before += w < wave_id() ? sm.hist[w] : 0u;
    if (r0 && before == 0) {
        sm.ticket = b0;
        sm.flag = above0 + c0;
    } else if (r1 && before + (uint32_t)r0 == 0) {
        sm.ticket = b1;
        sm.flag = above1 + c1;
    }
    __syncthreads();
    MAKO_STAMP(22);
    const uint32_t b_lo = sm.ticket;
    thr_bits = bin_lo_key(b_lo);
    const uint32_t n0 = sm.flag;
    auto worker_of = [&](uint32_t b, uint32_t c, uint32_t above) {
        return (c == 0 || b < b_lo) ? kNone : min(kWorkers - 1u, (uint32_t)(((unsigned long long)above * kWorkers) / n0));
    };
    const uint32_t wk0 = worker_of(b0, c0, above0), wk1 = worker_of(b1, c1, above1);
    if (wk0 != kNone) {
        atomicMax(&w_hi[wk0], b0);
        atomicMin(&w_lo[wk0], b0);
        atomicMin(&w_off[wk0], above0);
        atomicAdd(&w_cnt[wk0], c0);
    }
    if (wk1 != kNone) {
        atomicMax(&w_hi[wk1], b1);
        atomicMin(&w_lo[wk1], b1);
        atomicMin(&w_off[wk1], above1);
        atomicAdd(&w_cnt[wk1], c1);
    }
    __syncthreads();
    MAKO_STAMP(23);
    // the mass above a worker's range, known to the thread that holds the range's highest bin
    if (wk0 != kNone && w_hi[wk0] == b0)
        plan->mass[wk0] = incl - m0 - m1;
    if (wk1 != kNone && w_hi[wk1] == b1)
        plan->mass[wk1] = incl - m1;
    bin_worker[b0] = (uint8_t)wk0; // (kNone -> 0xff)
    bin_worker[b1] = (uint8_t)wk1;
    if (tid < kWorkers) {
        plan->cursor[tid] = 0;
        plan->key_lo[tid] = bin_lo_key(min(w_lo[tid], kBins - 1u));
        plan->key_hi[tid] = bin_hi_key(w_hi[tid]);
        plan->off[tid] = w_cnt[tid] ? w_off[tid] : 0u;
        plan->cnt[tid] = w_cnt[tid];
    }
    if (wave_id() == 0) { // the workers' first group records: a scan over their group counts
        const uint32_t mine = lane_id() < (int)kWorkers ? (w_cnt[lane_id()] + kGroup - 1u) / kGroup : 0u;
        const uint32_t upto = __ockl_wfscan_add_u32(mine, true);
        if (lane_id() < (int)kWorkers)
            plan->gbase[lane_id()] = upto - mine;
        if (lane_id() == kWave - 1) {
            plan->groups = upto;
            plan->n0 = n0;
            plan->total64 = total64;
        }
    }
    __syncthreads();
    return n0;
}

} // namespace mako
