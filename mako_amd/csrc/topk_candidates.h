// Top-k rows (and narrow nuclei) resolved from the candidate lists scan_kernel left.
#pragma once

#include "row_records.h"
#include "whole_row.h"

namespace mako {

// Bitonic sort, descending, of 1024 * ITEMS keys held ITEMS per thread: key[t] is element t * 1024 + tid.
// Partners 1024 or more apart are other registers of the same thread, partners less than 64 apart are lanes
// of the same wave (shuffles); only the strides in between go through LDS (two barriers each).
// (MAKO_TOPK_PART: __attribute__((noinline)) for a translation unit whose top-k code sits inside an out-of-line
// function: each part then has the register file to itself instead of spilling inside its loops.  No source sets it
// today: every kernel has its top-k rows in line.)
#ifndef MAKO_TOPK_PART
#define MAKO_TOPK_PART
#endif
template <int ITEMS>
__device__ void bitonic_sort_regs(unsigned long long (&key)[ITEMS], unsigned long long* lds)
{
    const uint32_t tid = threadIdx.x;
    for (uint32_t k = 2; k <= 1024u * ITEMS; k <<= 1)
        for (uint32_t j = k >> 1; j > 0; j >>= 1) {
            if (j >= 1024u) {
                // register-to-register stage; every index below is a compile-time constant so that key[]
                // stays in registers
#pragma unroll
                for (uint32_t dj = 1; dj < (uint32_t)ITEMS; dj <<= 1)
                    if (j == dj * 1024u) {
#pragma unroll
                        for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t)
                            if ((t & dj) == 0) {
                                const bool desc = ((t * 1024u + tid) & k) == 0;
                                const unsigned long long a = key[t], b = key[t | dj];
                                const bool swap = (a < b) == desc;
                                key[t] = swap ? b : a;
                                key[t | dj] = swap ? a : b;
                            }
                    }
            } else if (j >= (uint32_t)kWave) {
#pragma unroll
                for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t)
                    lds[t * 1024u + tid] = key[t];
                __syncthreads();
#pragma unroll
                for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t) {
                    const unsigned long long other = lds[t * 1024u + (tid ^ j)];
                    const bool keep_max = ((tid & j) == 0) == (((t * 1024u + tid) & k) == 0);
                    key[t] = keep_max ? (key[t] > other ? key[t] : other) : (key[t] < other ? key[t] : other);
                }
                __syncthreads();
            } else {
#pragma unroll
                for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t) {
                    const unsigned long long other = __shfl_xor(key[t], (int)j);
                    const bool keep_max = ((tid & j) == 0) == (((t * 1024u + tid) & k) == 0);
                    key[t] = keep_max ? (key[t] > other ? key[t] : other) : (key[t] < other ? key[t] : other);
                }
            }
        }
}

// Keys (bits(q) << 32 | ~token id, 0 = not a candidate) of candidates t * 1024 + tid of the row's flattened
// candidate list (all slices; sm.soff holds the slices' offsets), t < ITEMS.  Positions first, then every load
// from a clamped position with no branch in between (a branch around each load would make it wait for the one
// before), then the weights of the candidates that exist.
template <int ITEMS>
__device__ __forceinline__ void candidate_keys(const Scratch& sc, uint32_t row, uint32_t slices, uint32_t n_cands, float m,
                                               float inv_t, float floor_q, const FinishShared& sm,
                                               unsigned long long (&key)[ITEMS])
{
    const uint32_t tid = threadIdx.x;
    size_t at[ITEMS];
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t) {
        const uint32_t c = t * 1024u + tid < n_cands ? t * 1024u + tid : 0u; // (past the end: candidate 0, a short search)
        uint32_t s = 0;
        while (s + 1 < slices && c >= sm.soff[s + 1]) // slice holding candidate c
            ++s;
        at[t] = ((size_t)row * sc.slices_cap + s) * kCap + (c - sm.soff[s]);
    }
    float w[ITEMS];
    uint32_t id[ITEMS];
    const global_ptr<const float> cand_w = as_global(sc.cand_w);
    const global_ptr<const uint32_t> cand_i = as_global(sc.cand_i);
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t)
        w[t] = cand_w[at[t]];
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t)
        id[t] = cand_i[at[t]];
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t) {
        key[t] = 0;
        if (t * 1024u < n_cands) { // uniform: whole trips past the end of the list are skipped
            const float q = weight_of(w[t], m, inv_t, sm.tab);
            if (t * 1024u + tid < n_cands && q >= floor_q && q > 0.0f)
                key[t] = ((unsigned long long)__float_as_uint(q) << 32) | (unsigned long long)(kNone - id[t]);
        }
    }
}

// The same keys from the candidate lists read as SLOTS: thread tid takes entries (tid % 128) + 128 t, t < 4, of slice
// tid / 128, whether or not the slice emitted that many.  Where the lists end is not needed to ask for them, so the
// loads go out together with the loads of the slices' records instead of one trip to memory behind them; and
// since every slice's list starts at t = 0, the trips past the longest list are skipped by whole waves.
// For rows of at most eight slices.
constexpr int kPrefetchItems = 4;
struct CandSlots {
    float w[kPrefetchItems];
    uint32_t id[kPrefetchItems];
};
__device__ __forceinline__ bool slots_cover(uint32_t slices) { return slices <= 8u; }
__device__ __forceinline__ void fetch_candidate_slots(const Scratch& sc, uint32_t row, uint32_t slices, CandSlots& c)
{
    static_assert(kCap == (uint32_t)kPrefetchItems * 128u && kThreads == 1024, "eight slices of 128 threads, four entries each");
    const uint32_t sl = min(threadIdx.x >> 7, slices - 1u), i0 = threadIdx.x & 127u;
    const size_t base = ((size_t)row * sc.slices_cap + sl) * kCap + i0;
    const global_ptr<const float> cand_w = as_global(sc.cand_w);
    const global_ptr<const uint32_t> cand_i = as_global(sc.cand_i);
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)kPrefetchItems; ++t) {
        c.w[t] = cand_w[base + 128u * t];
        c.id[t] = cand_i[base + 128u * t];
    }
}
// (sm.soff as candidate_bound() leaves it)
__device__ __forceinline__ void keys_from_slots(const CandSlots& c, uint32_t slices, float m, float inv_t, float floor_q,
                                                const FinishShared& sm, unsigned long long (&key)[kPrefetchItems])
{
    const uint32_t sl = min(threadIdx.x >> 7, slices - 1u), i0 = threadIdx.x & 127u;
    const uint32_t emitted = (threadIdx.x >> 7) < slices ? sm.soff[sl + 1] - sm.soff[sl] : 0u;
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)kPrefetchItems; ++t) {
        key[t] = 0;
        if (i0 + 128u * t < emitted) {
            const float q = weight_of(c.w[t], m, inv_t, sm.tab);
            if (q >= floor_q && q > 0.0f)
                key[t] = ((unsigned long long)__float_as_uint(q) << 32) | (unsigned long long)(kNone - c.id[t]);
        }
    }
}

// The row's candidates (all slices) weighted, sorted by (q desc, idx asc) and left in LDS as kf[i] = ~bits(q_i),
// jf[i] = token id, invalid ones (q not a candidate) last.  Returns the number of valid candidates.
template <int ITEMS>
__device__ MAKO_TOPK_PART uint32_t sort_candidates(const Scratch& sc, uint32_t row, uint32_t slices, uint32_t n_cands, float m, float inv_t,
                                    float floor_q, uint32_t* kf, uint32_t* jf, const FinishLds& L)
{
    assume_lds(L);
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
    unsigned long long key[ITEMS];
    candidate_keys<ITEMS>(sc, row, slices, n_cands, m, inv_t, floor_q, sm, key);
    bitonic_sort_regs<ITEMS>(key, L.sortk);
    uint32_t nv = 0;
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t) {
        kf[t * 1024u + tid] = ~(uint32_t)(key[t] >> 32);
        jf[t * 1024u + tid] = kNone - (uint32_t)key[t];
        nv += key[t] != 0;
    }
    return block_sum_u32(nv, sm.bs); // (its barriers publish kf / jf)
}


// Fast route for rows that need only a few of their candidates.  Every thread weights up to four candidates;
// those at or above a weight threshold (at most kSmall of them) are ordered by (q desc, idx asc) by counting, for
// each, the entries that precede it, and left in LDS as kf[i] = ~bits(q_i), jf[i] = token id.
//   top_k > 0:  the threshold is the lower edge of the quarter-binade bin that holds the top_k-th largest weight
//               (one histogram over bits(q) >> 21), so the list is a superset of the row's top_k candidates.
//   top_k == 0: the threshold is thr_bits, below which the nucleus cannot reach (from the row's histogram).
// Returns the number of entries in the list, or kNone when they exceed kSmall (nothing is written then);
// n_valid receives the number of candidates that have a weight at all.
// `pre` (when have_pre): the row's candidate slots as fetch_candidate_slots() loaded them.
__device__ MAKO_TOPK_PART uint32_t small_candidates(const Scratch& sc, uint32_t row, uint32_t slices, uint32_t n_cands, float m, float inv_t,
                                     float floor_q, uint32_t top_k, uint32_t thr_bits, uint32_t* kf, uint32_t* jf,
                                     uint32_t& n_valid, const FinishLds& L, bool have_pre = false,
                                     const CandSlots& pre = CandSlots{})
{
    assume_lds(L);
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
    uint32_t* hist = reinterpret_cast<uint32_t*>(L.sortk);             // [512]
    unsigned long long* sel = L.sortk + 256;                           // [kSmall]
    uint32_t* rank = reinterpret_cast<uint32_t*>(L.sortk + 256 + kSmall); // [kSmall]
    uint32_t* counter = rank + kSmall;
    // (cleared before the candidates are fetched: the barrier behind their weights then covers this too)
    if (tid < 512)
        hist[tid] = 0;
    if (tid < kSmall)
        rank[tid] = 0;
    if (tid == 0)
        *counter = 0;
    unsigned long long key[4];
    static_assert(kPrefetchItems == 4, "one key array for both routes");
    if (have_pre) // uniform
        keys_from_slots(pre, slices, m, inv_t, floor_q, sm, key);
    else
        candidate_keys<4>(sc, row, slices, n_cands, m, inv_t, floor_q, sm, key);
    MAKO_STAMP(17);
    lds_barrier();
    uint32_t n_list;
    if (top_k > 0) {
#pragma unroll
        for (uint32_t t = 0; t < 4; ++t)
            if (key[t])
                atomicAdd(&hist[min((uint32_t)(key[t] >> 53), 511u)], 1u);
        lds_barrier();
        if (wave_id() == 0) {
            // one wave finds the bin of the top_k-th weight: eight bins per lane from the top down, a scan over the
            // lanes' counts, then the lane that holds the bin goes through its eight
            uint32_t c[8], mine = 0;
#pragma unroll
            for (uint32_t j = 0; j < 8; ++j) {
                c[j] = hist[511u - (lane_id() * 8u + j)];
                mine += c[j];
            }
            const uint32_t upto = __ockl_wfscan_add_u32(mine, true);
            const uint32_t total = (uint32_t)__builtin_amdgcn_readlane((int)upto, kWave - 1);
            uint32_t above = upto - mine, bits = 0, taken = 0;
#pragma unroll
            for (uint32_t j = 0; j < 8; ++j) {
                if (above < top_k && top_k <= above + c[j]) {
                    bits = (511u - (lane_id() * 8u + j)) << 21;
                    taken = above + c[j];
                }
                above += c[j];
            }
            const unsigned long long hit = __ballot(taken != 0);
            const int owner = hit ? __ffsll((long long)hit) - 1 : 0;
            if (lane_id() == owner) {
                sm.flag = hit ? bits : 0u; // 0 when the row has fewer than top_k candidates
                sm.ticket = hit ? taken : 0u;
                sm.aux = total;
            }
        }
        lds_barrier();
        n_valid = sm.aux;
        thr_bits = sm.flag;
        n_list = n_valid < top_k ? n_valid : sm.ticket;
    } else {
        uint32_t mine = 0, ge = 0;
#pragma unroll
        for (uint32_t t = 0; t < 4; ++t) {
            mine += key[t] != 0;
            ge += key[t] != 0 && (uint32_t)(key[t] >> 32) >= thr_bits;
        }
        const uint32_t both = block_sum_u32((mine << 16) | ge, sm.bs); // each below 65536
        n_valid = both >> 16;
        n_list = both & 0xffffu;
    }
    MAKO_STAMP(18);
    if (n_list > kSmall)
        return kNone;
    // compaction in any order: the keys are distinct, the ranks below put them in place
    const unsigned long long lower = (1ull << lane_id()) - 1ull;
#pragma unroll
    for (uint32_t t = 0; t < 4; ++t) {
        const bool keep = key[t] != 0 && (uint32_t)(key[t] >> 32) >= thr_bits;
        const unsigned long long bal = __ballot(keep);
        if (bal) {
            uint32_t base = 0;
            if (lane_id() == (uint32_t)__ffsll((long long)bal) - 1u)
                base = atomicAdd(counter, (uint32_t)__popcll(bal));
            base = (uint32_t)__builtin_amdgcn_readlane((int)base, __ffsll((long long)bal) - 1);
            if (keep)
                sel[base + (uint32_t)__popcll(bal & lower)] = key[t];
        }
    }
    __syncthreads();
    MAKO_STAMP(19);
    {
        const uint32_t e = tid & (kSmall - 1u), part = tid / kSmall; // four threads share the comparisons of an entry
        const unsigned long long my = e < n_list ? sel[e] : ~0ull;
        // each of the four takes a quarter of the list; waves whose entries lie past its end have nothing to count
        const uint32_t chunk = (n_list + 3u) / 4u, jb = part * chunk, je = min(n_list, jb + chunk);
        uint32_t r = 0;
        if ((e & ~(kWave - 1u)) < n_list) {
#pragma unroll 4
            for (uint32_t j = jb; j < je; ++j)
                r += sel[j] > my;
        }
        if (r)
            atomicAdd(&rank[e], r);
        __syncthreads();
        if (tid < n_list) {
            const uint32_t at = rank[tid];
            kf[at] = ~(uint32_t)(my >> 32);
            jf[at] = kNone - (uint32_t)my;
        }
    }
    __syncthreads();
    return n_list;
}

// A top-k row (top_k <= kTopKFast) from the candidates scan_kernel left: weights of the candidates, the top_k-th
// weight's neighbourhood ordered by (q desc, idx asc) in LDS, the certificate that nothing left behind in a slice can
// reach the top_k-th weight, then top-p, total and draw by one wave.  A row that cannot be certified takes the
// whole-row path: here and now (INLINE_GENERAL), or through sort_kernel's work list.
#ifndef MAKO_TOPK_GENERAL_SITE
#define MAKO_TOPK_GENERAL_SITE 1 // (the general_row instance a top-k row falls back to: 0 where one exists anyway)
#endif
__device__ __forceinline__ void topk_row(const mako_sample_desc& d, const Scratch& sc, uint32_t row, uint32_t slices,
                                         const mako_sampling_params& P, float m, uint32_t argidx, uint32_t n_cands,
                                         const SliceStat& lane_stat, const FinishLds& L, bool have_pre = false,
                                         const CandSlots& pre = CandSlots{})
{
    assume_lds(L);
    FinishShared& sm = *L.sm;
    // ---- top-k rows: weights of the row's candidates, sorted by (q desc, idx asc) in LDS ----
    const float inv_t = 1.0f / P.temperature;
    const float floor_q = (1.0f < P.min_p) ? 1.0f : P.min_p;
    const float q_bound = candidate_bound(lane_stat, slices, m, inv_t, floor_q, sm);
    MAKO_STAMP(3);
    uint32_t* kf = reinterpret_cast<uint32_t*>(L.sortk + kSortMax); // upper half of the dynamic block
    uint32_t* jf = kf + kSortMax;
    uint32_t n_valid = 0;
    uint32_t n_list = kNone;
    if (!d.draft) // the top_k-th weight's neighbourhood only
        n_list = small_candidates(sc, row, slices, n_cands, m, inv_t, floor_q, P.top_k, 0u, kf, jf, n_valid, L, have_pre, pre);
    if (n_list == kNone)
        n_valid = n_cands <= 1024u ? sort_candidates<1>(sc, row, slices, n_cands, m, inv_t, floor_q, kf, jf, L)
                                   : sort_candidates<4>(sc, row, slices, n_cands, m, inv_t, floor_q, kf, jf, L);
    MAKO_STAMP(4);
    // top-k of the row = top-k of the candidates, provided nothing left behind can tie with or beat the k-th
    bool ok = n_valid >= P.top_k ? q_bound < __uint_as_float(~kf[P.top_k - 1]) : q_bound == 0.0f;
    if (ok && n_valid == 0) {
        fallback_row(d, row, argidx);
        return;
    }
    // (sampler.cpp:40-43; at most top_k <= kTopKFast <= kGroup entries.  A top-p cut too close to call is left to the
    // whole-row path, which can sum in the reference's order.)
    static_assert(kTopKFast <= kGroup, "top-k rows end in sorted_tail's short-list path");
    if (ok && sorted_tail<false, true>(d, row, P, kf, jf, min(P.top_k, n_valid), false, 0.0, MAKO_PATH_TOPK, L))
        return;
    __syncthreads(); // (the lists in LDS are done with)
    // (where the whole-row path is a called function the views it receives by reference live in scratch memory: a copy
    // made here, so that only the rows that come this way store one)
    const FinishLds views = L;
    general_row<MAKO_TOPK_GENERAL_SITE>(d, sc, row, P, m, argidx, views);
}

} // namespace mako
