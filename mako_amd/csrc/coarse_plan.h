// The second pass's plan for a top_k == 0 row, derived from scan_kernel's coarse counts before any weight exists.
#pragma once

#include "row_records.h"
#include "unsorted_shares.h"

namespace mako {

constexpr uint32_t kPlanSlices = 12; // slices whose counts are asked for ahead of the logits (the rest: one more trip)

// Every workgroup of a row builds the same plan (same inputs, same instructions); LDS of its own, beside the
// penalty table that the logits' loads work on meanwhile.
struct alignas(16) CoarsePlan {
    uint32_t cnt[kLogBins];          // logits per bin in the frame of the ROW's maximum (log_bin_in_frame())
    uint32_t incl[kLogBins];         // logits in bins [0, b]
    int32_t slice_top[kMaxSlices];   // unit of each slice's maximum
    float wave_mass[kWaves];
    uint32_t wave_cnt[kWaves];
    uint32_t wave_hit[kWaves];
    uint32_t first_bin[kWorkers + 1]; // worker w is expected to take the bins [first_bin[w], first_bin[w + 1])
    uint32_t key_lo[kWorkers];        // and takes the weights with bits(q) in [key_lo[w], key_lo[w - 1])
    uint32_t cap[kWorkers];
    uint32_t stage_off[kWorkers];
    double mass_above[kWorkers];
    double mass_all;
    uint32_t count[kWorkers]; // hand-over: this workgroup's entries for each worker
    uint32_t lbase[kWorkers + 1]; // where its run starts in the workgroup's own ordering of what it keeps
    uint32_t goff[kWorkers];      // entry e of that ordering, if worker w's, goes to goff[w] + e of the row's staging arrays
    uint32_t lim[kWorkers];       // if e < lim[w] (the share's room allows it)
    uint32_t flag, thr, n0_est;
    uint32_t opq_mask; // workers whose shares are left unsorted (opaque_guess())
};

// What coarse_plan() needs from device memory, asked for before the logits so that the plan can be built while they
// are on their way (loads return in the order they were issued).
struct PlanLoads {
    SliceStat st; // the record of slice min(lane, slices - 1)
    uint32_t v[kPlanSlices];
    float u; // the row's uniform draw (for the estimate of where its walk ends)
};
template <bool WITH_U>
__device__ __forceinline__ void issue_plan_loads(const mako_sample_desc& d, const Scratch& sc, uint32_t row, uint32_t slices, PlanLoads& pre)
{
    pre.u = WITH_U ? as_global(d.u)[row] : 0.0f;
    pre.st = load_slice_stat(sc.stats, (size_t)row * kMaxSlices + min((uint32_t)lane_id(), slices - 1u));
    const global_ptr<const uint16_t> lh = as_global(sc.log_hist) + (size_t)row * sc.slices_cap * kLogBins + threadIdx.x;
#pragma unroll
    for (uint32_t t = 0; t < kPlanSlices; ++t)
        pre.v[t] = lh[(size_t)min(t, slices - 1u) * kLogBins]; // (clamped, not skipped: no branch between the loads)
}

// Builds the row's plan in `pl` (all threads call; barriers order LDS only, the logits' loads stay in flight).
// `m`: the row's maximum.  narrow_ok: a narrow nucleus may be left to the candidate lists.
// The slices' counts are moved into the frame of the row's maximum (exactly: units are absolute), each bin's mass is
// estimated from the middle of the units it covers, and the threshold is put one bin below where the estimated mass
// under it falls to 1 - top_p of the estimated total, less a few percent.  The list that results is checked by the
// exact sums later: a plan that keeps too little costs a second look at the row, never a wrong answer.
// (Every instruction here is latency of the whole pass: a workgroup's sixteen waves share four SIMDs.)
// opaque_first: the first position of the list from which a share may be left unsorted (kNone: none may).
__device__ void coarse_plan(const Scratch& sc, uint32_t row, uint32_t slices, uint32_t n_vocab, const mako_sampling_params& P,
                            float m, const PlanLoads& pre, bool narrow_ok, uint32_t opaque_first, CoarsePlan& pl, const uint64_t* tab)
{
    const uint32_t tid = threadIdx.x, lane = (uint32_t)lane_id();
    MAKO_STAMP(10);
    const float scale = log_unit_scale(P);
    const float inv_t = 1.0f / P.temperature;
    constexpr float kPerUnit = -1.0f / (float)kLogUnitsPerOctave;
    const int32_t k_top = log_unit(m, scale);
    pl.cnt[tid] = 0;
    if (tid <= kWorkers)
        pl.first_bin[tid] = 0; // (0: no bin opens the worker; worker 0 starts at bin 0 anyway)
    if (tid < kWorkers)
        pl.count[tid] = 0;
    if (wave_id() == 0 && lane < slices)
        pl.slice_top[lane] = log_unit(pre.st.wmax, scale);
    lds_barrier();
    MAKO_STAMP(2);
    // a slice's bin (a unit, or a group of units: absolute either way) in the row's frame
    auto add = [&](uint32_t s, uint32_t v) {
        if (!v)
            return;
        // (the slice's maximum in a scalar register: what depends on it alone is scalar arithmetic)
        const uint32_t b = log_bin_moved(tid, (int32_t)__builtin_amdgcn_readfirstlane(pl.slice_top[s]), k_top);
        if (b < kLogBins - 1u)
            atomicAdd(&pl.cnt[b], v);
    };
#pragma unroll
    for (uint32_t t = 0; t < kPlanSlices; ++t)
        if (t < slices)
            add(t, pre.v[t]);
    for (uint32_t s = kPlanSlices; s < slices; ++s)
        add(s, as_global(sc.log_hist)[((size_t)row * sc.slices_cap + s) * kLogBins + tid]);
    lds_barrier();
    MAKO_STAMP(3);
    // Running mass and count from the LOWEST bin up (thread t takes bin kLogBins - 1 - t): the mass below a bin, which
    // is what the threshold is about, is then a sum of small terms and as accurate as they are, however close to one
    // top_p is.  Wave scans, then one scan of the sixteen waves' totals by every wave for itself.
    const uint32_t bin = kLogBins - 1u - tid;
    const uint32_t c = pl.cnt[bin];
    const float top_frac = fminf(fmaxf(m * scale, -1.0e9f), 1.0e9f) - (float)k_top; // the maximum inside its unit
    const float mass = (float)c * __builtin_amdgcn_exp2f((log_bin_middle(bin, k_top) + top_frac) * kPerUnit);
    const float mass_w = __ockl_wfscan_add_f32(mass, true);
    const uint32_t cnt_w = __ockl_wfscan_add_u32(c, true);
    if (lane == kWave - 1) {
        pl.wave_mass[wave_id()] = mass_w;
        pl.wave_cnt[wave_id()] = cnt_w;
    }
    lds_barrier();
    MAKO_STAMP(4);
    const float wm = lane < (uint32_t)kWaves ? pl.wave_mass[lane] : 0.0f;
    const uint32_t wc = lane < (uint32_t)kWaves ? pl.wave_cnt[lane] : 0u;
    const float wm_upto = __ockl_wfscan_add_f32(wm, true);
    const uint32_t wc_upto = __ockl_wfscan_add_u32(wc, true);
    const float all_m = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wm_upto), kWaves - 1));
    const uint32_t all_c = (uint32_t)__builtin_amdgcn_readlane((int)wc_upto, kWaves - 1);
    const float below_m = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wm_upto - wm), wave_id())) + mass_w - mass; // mass under the bin
    const uint32_t from_c = (uint32_t)__builtin_amdgcn_readlane((int)(wc_upto - wc), wave_id()) + cnt_w; // logits in it and under it
    const uint32_t excl_c = all_c - from_c, incl_c = excl_c + c; // logits above the bin; and with it
    pl.incl[bin] = incl_c;
    // the nucleus ends where what lies below it is 1 - top_p of the total; the estimates of both are good to a few
    // percent of themselves (the bins' widths), whatever top_p is
    // (what the bins do not cover, masked and far-off logits alike, is taken at the weight where the bins end)
    const float tail_allowed = (1.0f - P.top_p) * all_m * 0.9f -
                               (float)(n_vocab - min(all_c, n_vocab)) * __builtin_amdgcn_exp2f((log_bin_middle(kLogBins - 2u, k_top) + top_frac) * kPerUnit);
    {
        const unsigned long long bal = __ballot(c != 0 && below_m <= tail_allowed);
        if (lane == 0) // (the highest such bin: the last such thread)
            pl.wave_hit[wave_id()] = bal ? kLogBins - 1u - ((uint32_t)wave_id() * kWave + 63u - (uint32_t)__clzll((long long)bal)) : kNone;
    }
    lds_barrier();
    MAKO_STAMP(5);
    uint32_t hit_bin = lane < (uint32_t)kWaves ? pl.wave_hit[lane] : kNone;
    hit_bin = __ockl_wfred_min_u32(hit_bin);
    // weights of the bins below `bins_end` are kept
    const uint32_t bins_end = hit_bin == kNone ? kLogBins - 1u : min(hit_bin + 2u, kLogBins - 1u);
    const uint32_t n0_est = pl.incl[bins_end - 1u];
    const bool sane = scale > 0.0f && scale < INFINITY && m == m && fabsf(m) < INFINITY && all_m > 0.0f;
    uint32_t flag = 1;
    if (!sane)
        flag = 2;
    else if (narrow_ok && n0_est <= kSmall)
        flag = 3;
    else if (n0_est > kGroup * (kMaxGroups - kWorkers))
        flag = 2; // (a list too long for the workers' group records goes to the whole-row path)
    // shares of about equal counts (a monotone estimate is all that is needed)
    const float per_entry = flag == 1 ? (float)kWorkers / (float)max(n0_est, 1u) : 0.0f;
    auto worker_at = [&](uint32_t excl) { return min(kWorkers - 1u, (uint32_t)((float)excl * per_entry)); };
    const uint32_t wk = worker_at(excl_c);
    if (bin != 0 && bin < bins_end) {
        // the workers whose share starts with this bin
        const uint32_t c_prev = pl.cnt[bin - 1u];
        for (uint32_t w = worker_at(excl_c - c_prev) + 1u; w <= wk; ++w) {
            pl.first_bin[w] = bin;
            pl.mass_above[w] = (double)(all_m - below_m - mass);
        }
    }
    if (tid == 0)
        pl.mass_above[0] = 0.0;
    lds_barrier();
    MAKO_STAMP(6);
    if (wave_id() == 0) {
        const uint32_t w = lane;
        uint32_t fb = bins_end, nb = bins_end;
        if (w < kWorkers) {
            fb = (w == 0 || pl.first_bin[w]) ? pl.first_bin[w] : bins_end;
            nb = (w + 1u < kWorkers && pl.first_bin[w + 1u]) ? pl.first_bin[w + 1u] : bins_end;
        }
        // The lower edge of the worker's weights: the weight of the smallest logit whose unit lies above bin nb.
        // Found exactly (a division, then a few steps from float to float with the very function that made the
        // bins): the restated expf never falls as its argument rises, so every logit of the share's bins has a
        // weight at or above this one and every logit of the bins below a weight at or below it; what the bins
        // promised a worker and what its range of weights brings it then differ only by weights equal to an edge.
        const int32_t k_edge = log_bin_upper_edge(nb, k_top);
        float edge = (float)k_edge / scale;
        for (int i = 0; i < 6 && log_unit(edge, scale) < k_edge; ++i)
            edge = nextafterf(edge, INFINITY);
        for (int i = 0; i < 6; ++i) {
            const float below = nextafterf(edge, -INFINITY);
            if (log_unit(below, scale) < k_edge)
                break;
            edge = below;
        }
        const float qe = weight_of(edge, m, inv_t, tab);
        uint32_t key = qe == qe ? __float_as_uint(qe) : 0u; // (positive floats order like their bits)
        for (uint32_t o = 1; o < kWorkers; o <<= 1) { // the edges never rise from one worker to the next
            const uint32_t t = (uint32_t)__shfl_up((int)key, o);
            if (lane >= o)
                key = min(key, t);
        }
        // room: what the counts promise for the share's bins, and slack (weights within a rounding of an edge, and
        // equal weights of different logits, may fall on either side of it)
        const uint32_t expect = nb > fb ? pl.incl[nb - 1u] - (fb >= 1u ? pl.incl[fb - 1u] : 0u) : 0u;
        const uint32_t cap = w < kWorkers ? expect + expect / 64u + kStageSlack : 0u;
        const uint32_t upto = __ockl_wfscan_add_u32(cap, true);
        if (w < kWorkers) {
            pl.key_lo[w] = key;
            pl.cap[w] = cap;
            pl.stage_off[w] = upto - cap;
        }
        // which shares are left unsorted (positions from the counts the bins promise, with an eighth to spare: the
        // tail checks the records' real positions); and a valid mass for every worker
        const uint32_t expect_w = w < kWorkers ? expect : 0u;
        const unsigned long long filled = __ballot(expect_w != 0u);
        const unsigned long long above = w + 1u < (uint32_t)kWave ? filled >> (w + 1u) : 0ull;
        const uint32_t nx = above ? w + 1u + (uint32_t)__ffsll((long long)above) - 1u : kWorkers; // the next share with entries
        const double before = w < kWorkers ? pl.mass_above[w] : 0.0, after = nx < kWorkers ? pl.mass_above[nx] : -1.0;
        if (w > 0u && w < kWorkers && expect_w == 0u)
            pl.mass_above[w] = after; // (a worker without bins: the mass above the next one that has some, or none)
        bool unsorted = false;
        if (opaque_first != kNone) { // (uniform; only batches of many such rows)
            const uint32_t off_est = __ockl_wfscan_add_u32(expect_w, true) - expect_w;
            const uint32_t key_hi = w ? (uint32_t)__shfl_up((int)key, 1) : 0x3f800001u; // (just above 1.0)
            const double r0 = (double)pre.u * ((double)P.top_p * (double)all_m);
#ifdef MAKO_RASH_PLANS // (a test build: plans that leave unsorted what they should not; the results must not change)
            const uint32_t rash = 1u << (row & 3u);
#else
            constexpr uint32_t rash = 0u;
#endif
            unsorted = opaque_guess(flag == 1u && w < kWorkers && nx < kWorkers, expect_w, off_est, opaque_first + opaque_first / 8u,
                                    before, after, (double)all_m, P.top_p, r0, key_hi, rash);
        }
        const uint32_t opq_mask = (uint32_t)__ballot(unsorted);
        if (w == kWorkers - 1u) {
            pl.thr = key;
            pl.n0_est = n0_est;
            pl.mass_all = (double)all_m;
            pl.flag = (sane && upto > sc.vpad) ? 2u : flag;
            pl.opq_mask = opq_mask;
        }
    }
    lds_barrier();
    MAKO_STAMP(7);
}

} // namespace mako
