// The workers' LDS sorts of their shares of a wide nucleus, and the group records they leave for the tail.
#pragma once

#include "sorted_tail.h"
#include "whole_row.h"
#include "unsorted_shares.h"

namespace mako {

__device__ bool lds_bucket_sort(uint32_t n, uint32_t key_lo, uint32_t key_hi, uint32_t* kout, uint32_t* iout,
                                unsigned long long* dyn, FinishShared& sm, uint32_t* sorted_lds = nullptr);

// The workers' sort in LDS: the n entries (bits(q), idx) in LDS at A, all with key_lo <= bits(q) < key_hi,
// are dropped into kFine value buckets (descending), and every entry finds its place by counting the entries of its
// own bucket that precede it under (q desc, idx asc); they go to kout / iout as ~bits(q) and token id.  Returns false
// when a bucket is too crowded to be ranked by counting.  hist must be zero and sm.flag 0 on entry.
// sorted_lds (optional, n words of LDS outside the sort's own): receives the sorted ~bits(q) as well, and the
// function then returns behind a barrier that orders LDS only: the caller goes on from the copy instead of waiting
// for the stores to kout and reading them back.
__device__ bool lds_bucket_sort(uint32_t n, uint32_t key_lo, uint32_t key_hi, uint32_t* kout, uint32_t* iout,
                                unsigned long long* dyn, FinishShared& sm, uint32_t* sorted_lds)
{
    uint2* A = reinterpret_cast<uint2*>(dyn);
    uint2* A2 = A + kSegCap; // the entries again, bucket after bucket (any order inside a bucket)
    uint32_t* hist = reinterpret_cast<uint32_t*>(A2 + kSegCap);
    const uint32_t tid = threadIdx.x;
    // 2. buckets by value, heaviest first
    const uint32_t range = key_hi - key_lo; // > 0
    const uint32_t shift = range > kFine ? 32u - (uint32_t)__clz((range - 1u) >> 11) : 0u; // (range - 1) >> shift < kFine
    constexpr uint32_t kPer = kSegCap / kThreads;
    uint32_t bucket[kPer], pib[kPer];
#pragma unroll
    for (uint32_t t = 0; t < kPer; ++t) {
        const uint32_t e = t * kThreads + tid;
        bucket[t] = kNone;
        pib[t] = 0;
        if (e < n) {
            bucket[t] = (key_hi - 1u - A[e].x) >> shift;
            pib[t] = atomicAdd(&hist[bucket[t]], 1u);
        }
    }
    __syncthreads();
    {
        const uint32_t c0 = hist[2u * tid], c1 = hist[2u * tid + 1u];
        if (max(c0, c1) > 64u)
            sm.flag = 1;
        uint32_t total;
        const uint32_t ex = block_excl_scan_u32(c0 + c1, total, sm.bs); // (barriers: all counts are read before)
        hist[2u * tid] = ex;
        hist[2u * tid + 1u] = ex + c0;
        if (tid == 0)
            hist[kFine] = total;
    }
    __syncthreads();
    MAKO_STAMP(14);
    if (sm.flag)
        return false;
    // (the entries themselves move, not their numbers: whoever ranks an entry reads its bucket's entries in one
    // trip to LDS each instead of two)
#pragma unroll
    for (uint32_t t = 0; t < kPer; ++t)
        if (bucket[t] != kNone)
            A2[hist[bucket[t]] + pib[t]] = A[t * kThreads + tid];
    __syncthreads();
    MAKO_STAMP(15);
    // 3. rank inside the bucket, and out
#pragma unroll
    for (uint32_t t = 0; t < kPer; ++t) {
        const uint32_t s = t * kThreads + tid;
        if (s < n) {
            const uint2 me = A2[s];
            const uint32_t b = (key_hi - 1u - me.x) >> shift;
            const uint32_t lo = hist[b], hi = hist[b + 1u];
            // (four of the bucket's entries per trip, from clamped positions: a bucket rarely holds more)
            uint32_t r = 0;
            for (uint32_t x = lo; x < hi; x += 4u) {
                uint2 o[4];
#pragma unroll
                for (uint32_t u = 0; u < 4; ++u)
                    o[u] = A2[min(x + u, hi - 1u)];
#pragma unroll
                for (uint32_t u = 0; u < 4; ++u)
                    r += (x + u < hi && ((o[u].x > me.x) || (o[u].x == me.x && o[u].y < me.y))) ? 1u : 0u;
            }
            kout[lo + r] = ~me.x;
            iout[lo + r] = me.y;
            if (sorted_lds)
                sorted_lds[lo + r] = ~me.x;
        }
    }
    if (sorted_lds) // uniform
        lds_barrier();
    else
        __syncthreads();
    return true;
}

// The worker's share as the second pass left it (cnt <= kSegCap entries, bits(q) in ks and token ids in is, any
// order): asked for with fetch_staged_share() (the loads stay in flight while the caller goes on), sorted into
// kout / iout by lds_sort_staged().
struct StagedShare {
    uint32_t k[kSegCap / kThreads], id[kSegCap / kThreads];
};
__device__ __forceinline__ void fetch_staged_share(const uint32_t* ks, const uint32_t* is, uint32_t cnt, StagedShare& s)
{
    const GlobalKeys gk{ks}, gi{is};
#pragma unroll
    for (uint32_t t = 0; t < kSegCap / kThreads; ++t) { // (all loads first, from clamped positions; cnt > 0)
        const uint32_t e = min(t * kThreads + threadIdx.x, cnt - 1u);
        s.k[t] = gk[e];
        s.id[t] = gi[e];
    }
}
__device__ __forceinline__ bool lds_sort_staged(const StagedShare& s, uint32_t key_lo, uint32_t key_hi, uint32_t cnt,
                                                uint32_t* kout, uint32_t* iout, unsigned long long* dyn, FinishShared& sm,
                                                uint32_t* sorted_lds = nullptr)
{
    uint2* A = reinterpret_cast<uint2*>(dyn);
    uint32_t* hist = reinterpret_cast<uint32_t*>(A + 2u * kSegCap); // (behind lds_bucket_sort()'s second copy)
    const uint32_t tid = threadIdx.x;
    for (uint32_t b = tid; b <= kFine; b += kThreads)
        hist[b] = 0;
    if (tid == 0)
        sm.flag = 0;
#pragma unroll
    for (uint32_t t = 0; t < kSegCap / kThreads; ++t) {
        const uint32_t e = t * kThreads + tid;
        uint32_t k = s.k[t];
        asm volatile("" : "+v"(k)); // (used here and not before: the loads are to be waited for no earlier)
        if (e < cnt)
            A[e] = make_uint2(min(max(k, key_lo), key_hi - 1u), s.id[t]); // (clamped: a bucket index is always valid)
    }
    __syncthreads();
    MAKO_STAMP(13);
    return lds_bucket_sort(cnt, key_lo, key_hi, kout, iout, dyn, sm, sorted_lds);
}

// A share too large for one LDS sort is cut by value into runs that fit: one counting sweep over the share (the
// same kFine buckets as the sort uses) finds run boundaries at bucket edges, then each run is collected from the
// share and sorted on its own.  Returns false (the caller falls back to the radix sort through global memory)
// when a single bucket holds more than fits.
__device__ bool lds_sort_staged_runs(const uint32_t* ks, const uint32_t* is, uint32_t key_lo, uint32_t key_hi, uint32_t cnt,
                                     uint32_t* kout, uint32_t* iout, unsigned long long* dyn, FinishShared& sm)
{
    uint2* A = reinterpret_cast<uint2*>(dyn);
    uint32_t* hist = reinterpret_cast<uint32_t*>(A + 2u * kSegCap); // (behind lds_bucket_sort()'s second copy) // [kFine + 1]
    const uint32_t tid = threadIdx.x, lane = lane_id();
    const uint32_t range = key_hi - key_lo;
    const uint32_t shift = range > kFine ? 32u - (uint32_t)__clz((range - 1u) >> 11) : 0u;
    for (uint32_t b = tid; b <= kFine; b += kThreads)
        hist[b] = 0;
    __syncthreads();
    constexpr uint32_t kTrip = 8; // loads in flight per thread: the sweeps below are bound by memory latency
    for (uint32_t base = 0; base < cnt; base += kTrip * kThreads) {
        uint32_t k[kTrip];
#pragma unroll
        for (uint32_t u = 0; u < kTrip; ++u)
            k[u] = ks[min(base + u * kThreads + tid, cnt - 1u)];
#pragma unroll
        for (uint32_t u = 0; u < kTrip; ++u)
            if (base + u * kThreads + tid < cnt)
                atomicAdd(&hist[(key_hi - 1u - min(max(k[u], key_lo), key_hi - 1u)) >> shift], 1u);
    }
    __syncthreads();
    // bucket starts (exclusive scan), kept in sm.hist / sm.run as run boundaries below
    uint32_t total;
    const uint32_t c0 = hist[2u * tid], c1 = hist[2u * tid + 1u];
    const uint32_t ex = block_excl_scan_u32(c0 + c1, total, sm.bs);
    __syncthreads();
    hist[2u * tid] = ex;
    hist[2u * tid + 1u] = ex + c0;
    if (tid == 0) {
        hist[kFine] = total;
        sm.flag = 0;
    }
    __syncthreads();
    // runs: greedily as many whole buckets as fit (thread 0; a handful of runs).  Run r covers buckets
    // [sm.hist[r], sm.hist[64 + r]) = entries [sm.run[r], sm.run[r] + sm.run[64 + r]) of the sorted share.
    if (tid == 0) {
        uint32_t runs = 0, b0 = 0;
        while (b0 < kFine && runs < 64u) {
            uint32_t b1 = b0 + 1u;
            if (hist[b1] - hist[b0] > kSegCap) { // one bucket alone is too much
                runs = 0xffffffffu;
                break;
            }
            { // the last bucket edge within reach: the bucket starts never decrease, so bisect
                uint32_t lo = b1, hi = kFine;
                while (lo < hi) {
                    const uint32_t mid = (lo + hi + 1u) / 2u;
                    if (hist[mid] - hist[b0] <= kSegCap)
                        lo = mid;
                    else
                        hi = mid - 1u;
                }
                b1 = lo;
            }
            if (hist[b1] != hist[b0]) {
                sm.hist[runs] = b0;
                sm.hist[64u + runs] = b1;
                sm.run[runs] = hist[b0];
                sm.run[64u + runs] = hist[b1] - hist[b0];
                ++runs;
            }
            b0 = b1;
        }
        if (runs != 0xffffffffu && b0 < kFine)
            runs = 0xffffffffu;
        sm.ticket = runs;
    }
    __syncthreads();
    const uint32_t runs = sm.ticket;
    if (runs == 0xffffffffu)
        return false;
    for (uint32_t r = 0; r < runs; ++r) {
        const uint32_t b0 = sm.hist[r], b1 = sm.hist[64u + r];
        const uint32_t at = sm.run[r], n = sm.run[64u + r];
        // keys of buckets [b0, b1): (key_hi - 1 - k) >> shift in [b0, b1)
        const uint32_t hi_r = key_hi - (b0 << shift);
        const uint32_t lo_r = ((unsigned long long)b1 << shift) >= range ? key_lo : key_hi - (b1 << shift);
        __syncthreads();
        for (uint32_t b = tid; b <= kFine; b += kThreads)
            hist[b] = 0;
        if (tid == 0) {
            sm.ticket = 0;
            sm.flag = 0;
        }
        __syncthreads();
        const unsigned long long lower = (1ull << lane) - 1ull;
        for (uint32_t base = 0; base < cnt; base += kTrip * kThreads) {
            uint32_t k[kTrip], id[kTrip];
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u) {
                const uint32_t e = min(base + u * kThreads + tid, cnt - 1u);
                k[u] = ks[e];
                id[u] = is[e];
            }
            // slots for the whole trip from one LDS atomic per wave
            bool mine[kTrip];
            uint32_t before = 0, wave_total = 0;
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u) {
                k[u] = min(max(k[u], key_lo), key_hi - 1u);
                mine[u] = base + u * kThreads + tid < cnt && k[u] >= lo_r && k[u] < hi_r;
                const unsigned long long bal = __ballot(mine[u]);
                before += (uint32_t)__popcll(bal & lower);
                wave_total += (uint32_t)__popcll(bal);
            }
            if (wave_total) { // uniform
                uint32_t slot = 0;
                if (lane == 0)
                    slot = atomicAdd(&sm.ticket, wave_total);
                slot = uniform_u32(slot) + before;
#pragma unroll
                for (uint32_t u = 0; u < kTrip; ++u)
                    if (mine[u]) {
                        if (slot < kSegCap)
                            A[slot] = make_uint2(k[u], id[u]);
                        ++slot;
                    }
            }
        }
        __syncthreads();
        if (sm.ticket != n) // (cannot happen: the same keys were counted above)
            return false;
        if (!lds_bucket_sort(n, lo_r, hi_r, kout + at, iout + at, dyn, sm))
            return false; // (a crowded bucket: ties)
    }
    return true;
}

// ---- shares that need no sorting (unsorted_shares.h) ---------------------------------------------------------------
//
// The record of an unsorted share, by ONE wave (a collector workgroup's sixteen waves take a share each: no barrier,
// nothing shared).  ks: the share's cnt weights as bits(q), in device memory, any order.  `lds`: kOpaqueLdsWords words
// of LDS of the wave's own.  The share is streamed once (sixteen loads per lane in flight): its fp64 sum, its largest
// weight, the sums of the increments of the weights that are no exact ties, and the ties themselves (kept apart, up
// to kOpaqueTies of either kind); only a share with ties is streamed again, for the sums between neighbouring ties.
constexpr uint32_t kOpaqueLdsWords = 4u * kOpaqueTies + 4u * (kOpaqueTies + 1u);
__device__ void opaque_share(const uint32_t* ks, uint32_t cnt, uint32_t off, int e_tot, int e_walk, size_t t_at,
                             const GroupTable& T, uint32_t* lds)
{
    using namespace seqfp;
    constexpr uint32_t kTrip = 16, kSegs = kOpaqueTies + 1u;
    uint32_t* tie_key = lds;                          // [2][kOpaqueTies] as found
    uint32_t* tie_sorted = lds + 2u * kOpaqueTies;    // [2][kOpaqueTies] heaviest first
    unsigned long long* seg = reinterpret_cast<unsigned long long*>(lds + 4u * kOpaqueTies); // [2][kSegs]
    const GlobalKeys gk{ks};
    const uint32_t lane = (uint32_t)lane_id();
    const unsigned long long lower = (1ull << lane) - 1ull;
    double sum = 0.0;
    uint32_t kmax = 0u, n_t = 0u, n_w = 0u; // (the counts: uniform)
    uint32_t acc_t = 0u, acc_w = 0u;        // a lane's increments: at most 250 of them, 2^24 at most each
    const bool sat = cnt > (250u << 6);     // (more than that many per lane: no map)
    for (uint32_t base = 0; base < cnt; base += kTrip * kWave) {
        uint32_t k[kTrip];
#pragma unroll
        for (uint32_t u = 0; u < kTrip; ++u)
            k[u] = gk[min(base + u * kWave + lane, cnt - 1u)];
#pragma unroll
        for (uint32_t u = 0; u < kTrip; ++u) {
            const bool valid = base + u * kWave + lane < cnt;
            const uint32_t kv = valid ? k[u] : 0u;
            const float q = __uint_as_float(kv);
            sum += (double)q;
            kmax = max(kmax, kv);
            const Step32 st = step32_fp(q, e_tot); // (the weights of such a share lie binades below the epochs: never the mark)
            const bool tie_t = valid && st.d0 != st.d1;
            acc_t += (valid && !tie_t) ? min(st.d0, 1u << 24) : 0u;
            const unsigned long long bal_t = __ballot(tie_t);
            if (bal_t) { // (uniform, rare)
                const uint32_t slot = n_t + (uint32_t)__popcll(bal_t & lower);
                if (tie_t && slot < kOpaqueTies)
                    tie_key[slot] = kv;
                n_t += (uint32_t)__popcll(bal_t);
            }
            if (e_walk > 0) { // uniform
                const Step32 sw = step32_fp(q, e_walk);
                const bool tie_w = valid && sw.d0 != sw.d1;
                acc_w += (valid && !tie_w) ? min(sw.d0, 1u << 24) : 0u;
                const unsigned long long bal_w = __ballot(tie_w);
                if (bal_w) {
                    const uint32_t slot = n_w + (uint32_t)__popcll(bal_w & lower);
                    if (tie_w && slot < kOpaqueTies)
                        tie_key[kOpaqueTies + slot] = kv;
                    n_w += (uint32_t)__popcll(bal_w);
                }
            }
        }
    }
    const double sum64 = __ockl_wfred_add_f64(sum);
    kmax = __ockl_wfred_max_u32(kmax);
    // (a sum of 64 numbers below 2^31: in two halves)
    auto wave_total = [](uint32_t v) {
        return ((unsigned long long)__ockl_wfred_add_u32(v >> 16) << 16) + (unsigned long long)__ockl_wfred_add_u32(v & 0xffffu);
    };
    // One kind of map: the sums of the increments between neighbouring ties (heaviest first), with each tie's own
    // two-valued step composed in at its place.
    auto share_map = [&](uint32_t which, uint32_t n_raw, int e, uint32_t acc) {
        Step32 v = Step32{kSat, kSat, 0u};
        if (e > 0 && n_raw <= kOpaqueTies && !sat) { // uniform
            const uint32_t n = n_raw;
            if (n == 0u) {
                const unsigned long long S = wave_total(acc);
                const uint32_t add = S < (1ull << 24) ? (uint32_t)S : kSat;
                v = Step32{add, add, 0u};
            } else {
                // the ties by weight, heaviest first (equal ones in any order: they are the same step)
                __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): the wave's own writes of the ties
                const uint32_t mine = lane < n ? tie_key[which * kOpaqueTies + lane] : 0u;
                uint32_t rank = 0;
                for (uint32_t j = 0; j < n; ++j) {
                    const uint32_t other = (uint32_t)__builtin_amdgcn_readlane((int)mine, (int)j);
                    rank += (other > mine || (other == mine && j < lane)) ? 1u : 0u;
                }
                if (lane < n)
                    tie_sorted[which * kOpaqueTies + rank] = mine;
                if (lane <= n)
                    seg[which * kSegs + lane] = 0ull;
                __builtin_amdgcn_s_waitcnt(0xc07f);
                // the share again: a weight's segment is the number of ties heavier than it
                for (uint32_t base = 0; base < cnt; base += kTrip * kWave) {
                    uint32_t k[kTrip], sg[kTrip], dv[kTrip];
#pragma unroll
                    for (uint32_t u = 0; u < kTrip; ++u)
                        k[u] = gk[min(base + u * kWave + lane, cnt - 1u)];
#pragma unroll
                    for (uint32_t u = 0; u < kTrip; ++u) {
                        const bool valid = base + u * kWave + lane < cnt;
                        const Step32 st = step32_fp(__uint_as_float(k[u]), e);
                        dv[u] = (valid && st.d0 == st.d1) ? min(st.d0, 1u << 24) : 0u;
                        sg[u] = 0u;
                    }
                    for (uint32_t i = 0; i < n; ++i) {
                        const uint32_t tk = uniform_u32(tie_sorted[which * kOpaqueTies + i]);
#pragma unroll
                        for (uint32_t u = 0; u < kTrip; ++u)
                            sg[u] += tk > k[u] ? 1u : 0u;
                    }
                    for (uint32_t s = 0; s <= n; ++s) {
                        uint32_t part = 0u; // (sixteen increments below 2^24 + 1 each: below 2^29)
#pragma unroll
                        for (uint32_t u = 0; u < kTrip; ++u)
                            part += sg[u] == s ? dv[u] : 0u;
                        const unsigned long long all = wave_total(part);
                        if (lane == 0u && all)
                            seg[which * kSegs + s] += all;
                    }
                }
                __builtin_amdgcn_s_waitcnt(0xc07f);
                v = identity32();
                for (uint32_t s = 0; s <= n; ++s) {
                    const unsigned long long S = seg[which * kSegs + s];
                    const uint32_t add = S < (1ull << 24) ? (uint32_t)S : kSat;
                    v = compose32(v, Step32{add, add, 0u});
                    if (s < n)
                        v = compose32(v, step32_flat(__uint_as_float(tie_sorted[which * kOpaqueTies + s]), e));
                }
            }
        }
        v.cmax = e > 0 ? step32_flat(__uint_as_float(kmax), e).cmax : kSat; // (a weight's step never grows as the weight falls)
        return v;
    };
    const Step32 m0 = share_map(0u, n_t, e_tot, acc_t);
    const Step32 m1 = e_walk > 0 ? share_map(1u, n_w, e_walk, acc_w) : Step32{kSat, kSat, kSat};
    if (lane == 0u) {
        T.sum[t_at] = sum64;
        T.d0[t_at] = m0.d0;
        T.d1[t_at] = m0.d1;
        T.cmax[t_at] = m0.cmax;
        T.start[t_at] = off;
        T.pack[t_at] = kOpaque | ((uint32_t)e_tot << 16);
        T.walk[t_at] = e_walk > 0 ? make_uint4(m1.d0, m1.d1, walk_need(__uint_as_float(kmax), e_walk, m1.cmax), (uint32_t)e_walk)
                                  : make_uint4(0u, 0u, 0u, 0u);
    }
}

// Group records of a worker's sorted range (cnt entries from position off of the list kf): fp64 sums, and the
// maps of the running fp32 sum for the epoch guessed from the mass above the range plus the sums before the group.
// kf_lds (optional): the worker's cnt sorted weights in LDS (outside L.sortk's first 16 KB), read instead of kf + off.
// r0: the estimate of where the walk starts, u * top_p * (the row's total): the groups that r can reach also get their
// map for the walk, for the epoch guessed from r0 less the mass before the group (0 or less: none).
// (UNORDERED: the entries are in any order, e.g. a stretch of a row in token order: see span_map)
template <bool UNORDERED = false>
__device__ void worker_groups(const uint32_t* kf, uint32_t off, uint32_t cnt, size_t t_at, double mass, const GroupTable& T,
                              const FinishLds L, const uint32_t* kf_lds = nullptr, double r0 = 0.0)
{
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
    const uint32_t* src = kf_lds ? kf_lds : kf + off; // uniform
    double* gs = reinterpret_cast<double*>(L.sortk); // [groups] estimate of the sum before each group
    double* ge = gs + kMaxGroups;                    // [groups] and after it
    const uint32_t groups = (cnt + kGroup - 1u) / kGroup;
    if (kf_lds) // uniform: the copy is in place (its writers' barrier), nothing in device memory is waited for
        lds_barrier();
    else
        __syncthreads();
    for (uint32_t g = wave_id(); g < groups; g += kWaves) {
        float q[4];
        load_span(src, g * kGroup, min(kGroup, cnt - g * kGroup), q);
        const double s = __ockl_wfred_add_f64((((double)q[0] + (double)q[1]) + (double)q[2]) + (double)q[3]);
        if (lane_id() == 0)
            gs[g] = s;
    }
    MAKO_STAMP(16);
    // the sums before and after each group.  Up to a wave's worth of groups, every wave scans them for itself (the
    // values are those of the workgroup's scan, whose first wave adds them up the same way) and goes on at once.
    const bool few = groups <= (uint32_t)kWave; // uniform
    double before_l = 0, after_l = 0; // (few: lane g holds group g's)
    if (few) {
        if (kf_lds)
            lds_barrier();
        else
            __syncthreads();
        const uint32_t gq = (uint32_t)lane_id();
        const double v = gq < groups ? gs[gq] : 0.0;
        const double incl = __ockl_wfscan_add_f64(v, true);
        if (wave_id() == 0 && gq < groups)
            T.sum[t_at + gq] = v;
        before_l = mass + (incl - v);
        after_l = mass + incl;
    } else {
        __syncthreads();
        for (uint32_t g0 = 0; g0 < groups; g0 += kThreads) {
            const uint32_t g = g0 + tid;
            const double v = g < groups ? gs[g] : 0.0;
            double all;
            const double incl = block_incl_scan_f64(v, all, sm.bs);
            if (g < groups) {
                T.sum[t_at + g] = v;
                gs[g] = mass + (incl - v);
                ge[g] = mass + incl;
            }
            mass += all;
        }
        __syncthreads();
    }
    MAKO_STAMP(19);
    for (uint32_t g = wave_id(); g < groups; g += kWaves) {
        const uint32_t len = min(kGroup, cnt - g * kGroup);
        float q[4];
        load_span(src, g * kGroup, len, q);
        const double guess = few ? readlane_f64(before_l, g) : gs[g];
        const int eg = guess > 0 ? exponent_of((float)guess) : 0;
        const seqfp::Step32 st = span_map<UNORDERED>(q, len, eg);
        // the sum is expected to change binade inside the group (or starts at zero): records for its quarters
        const double at_end = few ? readlane_f64(after_l, g) : ge[g];
        const bool split4 = uniform_u32((uint32_t)(eg == 0 || exponent_of((float)at_end) != eg)) != 0;
        if (split4)
            build_quarters(q, len, guess, T.quarters + (t_at + g) * 4u);
        // the walk's map, where the walk is expected to pass the group without changing binade in it
        const double r_here = r0 - guess, r_after = r0 - at_end;
        const int ew = (r0 > 0.0 && r_after > 0.0) ? exponent_of((float)r_here) : 0;
        uint4 wrec = make_uint4(0u, 0u, 0u, 0u);
        if (ew > 0 && uniform_u32((uint32_t)(exponent_of((float)r_after) == ew)) != 0) {
            const seqfp::Step32 sw = span_map<UNORDERED>(q, len, ew);
            float q_top = q[0]; // (lane 0: the group's first, largest weight)
            if constexpr (UNORDERED)
                q_top = __uint_as_float(__ockl_wfred_max_u32(max(max(__float_as_uint(q[0]), __float_as_uint(q[1])), max(__float_as_uint(q[2]), __float_as_uint(q[3])))));
            wrec = make_uint4(sw.d0, sw.d1, walk_need(q_top, ew, sw.cmax), (uint32_t)ew);
        }
        if (lane_id() == 0) {
            T.d0[t_at + g] = st.d0;
            T.d1[t_at + g] = st.d1;
            T.cmax[t_at + g] = st.cmax;
            T.start[t_at + g] = off + g * kGroup;
            T.pack[t_at + g] = len | ((uint32_t)eg << 16) | (split4 ? kHasQuarters : 0u);
            T.walk[t_at + g] = wrec;
        }
    }
}

} // namespace mako
