// Splitting a top_k == 0 row among the workers that sort its nucleus, from a sample of the row's weights.
#pragma once

#include "workgroup_state.h"

namespace mako {

// The whole workgroup turns the histogram of the row's sampled weights (shist[b]; only bins >= b_prune were counted)
// into (1) a guess of how far down the nucleus reaches and (2) the workers' value ranges.
//
// (1) Every sample stands for n_vocab / kSamples weights of about its size, except the eight heaviest, which stand for
// themselves (where the row's weights are sparse a sample has no neighbours, and counting it many times over would
// put the cut too high).  From the samples' masses (count x the bin's middle weight) the bin in which the running
// mass reaches top_p x total is found, and the row keeps the weights down to HALF the lower edge of that bin (never
// below b_prune).  This is a guess: the kept set is exactly the weights in bins >= b_keep, and tail_kernel checks that
// the nucleus ends inside it; a row whose nucleus does not takes the whole-row path instead.
// (2) The kept weights are cut by value into `workers` contiguous ranges, heaviest first, that hold about the same
// number of samples each.  A cut that falls inside a bin is placed by interpolation between the bin's edges, so a
// crowded bin is shared by several workers.
//   table[b]   the worker that takes the heaviest weights of bin b
//   cut[j]     (1 <= j < workers) bits(q) of the cut between workers j - 1 and j: weights with bits(q) below it go
//              to worker j or beyond; 0 where no cut was placed (cleared by the caller)
// `workers` is chosen so that a worker's share stays near kShareTarget.  Every piece of the row sees the same samples
// and arrives at the same answers; no result depends on them, only the work does.  Thread t holds bins
// kBins - 1 - 2t and kBins - 2 - 2t.  Three barriers inside (LDS only); the caller's next barrier publishes table and
// cut.  Returns the number of workers; b_keep receives the lowest bin kept.
struct SamplePlanLds {
    uint32_t wave_cnt[kWaves];
    float wave_mass[kWaves];
    uint32_t edge_bin;
    uint32_t kept_samples;
};
__device__ __forceinline__ uint32_t sample_plan(const uint32_t* shist, uint8_t* table, uint32_t* cut, uint32_t n_vocab,
                                                float top_p, uint32_t b_prune, SamplePlanLds& pl, uint32_t& b_keep)
{
    const uint32_t b0 = kBins - 1u - 2u * threadIdx.x, b1 = b0 - 1u;
    const uint32_t c0 = shist[b0], c1 = shist[b1];
    const uint32_t incl = __ockl_wfscan_add_u32(c0 + c1, true);
    if (lane_id() == kWave - 1)
        pl.wave_cnt[wave_id()] = incl;
    if (threadIdx.x == 0)
        pl.edge_bin = 0u; // (no bin reaches the cut: everything above b_prune is kept)
    lds_barrier();
    uint32_t above0 = incl - (c0 + c1);
    for (int w = 0; w < wave_id(); ++w)
        above0 += pl.wave_cnt[w];
    const uint32_t above1 = above0 + c0;
    // (1) masses: the samples ranked 0..7 count once, the others n_vocab / kSamples times
    const float each = fmaxf(1.0f, (float)n_vocab / (float)kSamples);
    auto weighted = [&](uint32_t above, uint32_t c) {
        const uint32_t solo = above < 8u ? min(c, 8u - above) : 0u;
        return (float)solo + (float)(c - solo) * each;
    };
    auto middle = [](uint32_t b) { return __uint_as_float((bin_lo_key(b) >> 1) + (bin_hi_key(b) >> 1)); };
    const float m0 = c0 ? weighted(above0, c0) * middle(b0) : 0.0f, m1 = c1 ? weighted(above1, c1) * middle(b1) : 0.0f;
    float mincl = m0 + m1; // inclusive scan over the wave, then the waves' totals
    for (int o = 1; o < kWave; o <<= 1) {
        const float t = __shfl_up(mincl, o);
        mincl += lane_id() >= o ? t : 0.0f;
    }
    if (lane_id() == kWave - 1)
        pl.wave_mass[wave_id()] = mincl;
    lds_barrier();
    float mabove0 = mincl - (m0 + m1), mtotal = 0.0f;
    for (int w = 0; w < kWaves; ++w) {
        const float x = pl.wave_mass[w];
        mabove0 += w < wave_id() ? x : 0.0f;
        mtotal += x;
    }
    const float want = top_p * mtotal;
    // the first bin (from the top) at which the running mass reaches `want` (the largest bin index among those that do)
    if (c0 && mabove0 + m0 >= want)
        atomicMax(&pl.edge_bin, b0);
    else if (c1 && mabove0 + m0 + m1 >= want)
        atomicMax(&pl.edge_bin, b1);
    lds_barrier();
    {
        const uint32_t edge = pl.edge_bin;
        uint32_t keep = b_prune;
        if (edge > 0u) {
            const uint32_t lo = bin_lo_key(edge);
            keep = max(b_prune, lo > (1u << 23) ? weight_bin(lo - (1u << 23)) : 0u); // (half the edge bin's lower edge)
        }
        b_keep = keep;
    }
    // samples kept: those in bins >= b_keep (the holder of bin b_keep knows)
    if (b0 == b_keep)
        pl.kept_samples = above0 + c0;
    else if (b1 == b_keep)
        pl.kept_samples = above1 + c1;
    lds_barrier();
    const uint32_t kept = pl.kept_samples;
    // (2) (samples * n_vocab stays below 2^32: kSamples = 2^10 samples, n_vocab below 2^20)
    const uint32_t est = (kept * n_vocab + kSamples - 1u) / kSamples;
    const uint32_t workers = min(kWorkers, max(1u, (est + kShareTarget - 1u) / kShareTarget));
    const float per = (float)max(kept, 1u) / (float)workers; // samples per worker
    const float inv_per = (float)workers / (float)max(kept, 1u);
    // cuts lie at sample counts j * per, j = 1 .. workers - 1: those at or before `above` lie in higher bins
    auto place = [&](uint32_t b, uint32_t above, uint32_t c) {
        const uint32_t j0 = min(workers - 1u, (uint32_t)((float)above * inv_per));
        table[b] = (uint8_t)j0;
        const uint32_t j1 = min(workers - 1u, (uint32_t)((float)(above + c) * inv_per));
        if (j1 > j0 && b >= b_keep) { // (few bins hold a cut)
            const uint32_t hi = bin_hi_key(b), lo = bin_lo_key(b);
            const float width = (float)(hi - lo), inv_c = 1.0f / (float)c;
            for (uint32_t j = j0 + 1u; j <= j1; ++j) {
                const float frac = ((float)j * per - (float)above) * inv_c; // from the bin's top down
                cut[j] = hi - min(hi - lo, (uint32_t)(fminf(fmaxf(frac, 0.0f), 1.0f) * width));
            }
        }
    };
    place(b0, above0, c0);
    place(b1, above1, c1);
    return workers;
}

// The worker that takes the weight with these bits(q), in bin b.
__device__ __forceinline__ uint32_t worker_of_weight(uint32_t bits, uint32_t b, const uint8_t* table, const uint32_t* cut,
                                                     uint32_t workers)
{
    uint32_t dest = table[b];
    while (dest + 1u < workers && bits < cut[dest + 1u])
        ++dest;
    return dest;
}

} // namespace mako
