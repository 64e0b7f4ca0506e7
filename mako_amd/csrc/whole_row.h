// The whole-row path: exact for every parameter combination, one workgroup per row.
#pragma once

#include "sorted_tail.h"

namespace mako {

// Lanes of this wave whose `digit` equals mine, restricted to `valid` lanes.
__device__ __forceinline__ unsigned long long match_digit(uint32_t digit, bool valid)
{
    unsigned long long m = __ballot(valid);
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const bool bit = (digit >> b) & 1u;
        const unsigned long long bal = __ballot(bit);
        m &= bit ? bal : ~bal;
    }
    return m;
}

// One stable counting-sort pass on bits [shift, shift + 8) of the keys, ascending, by one workgroup.
// Wave w owns the contiguous chunk [w * C, (w + 1) * C) of the input and walks it 64 pairs at a time: lanes
// with equal digits find each other with ballots (match_digit), so ranks inside a group need no atomics, and
// the wave's running output offsets per digit live in its private row of LDS.  Three barriers per pass.
// Returns false (and moves nothing) when every key has the same digit.
__device__ bool radix_pass(const uint32_t* ksrc, const uint32_t* isrc, uint32_t* kdst, uint32_t* idst, uint32_t n,
                           uint32_t shift, const FinishLds& L)
{
    assume_lds(L);
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x, lane = lane_id(), wave = wave_id();
    const uint32_t chunk = ((n + kThreads - 1u) / kThreads) * kWave; // per wave, a multiple of 64
    const uint32_t beg = min(n, wave * chunk), end = min(n, beg + chunk);
    uint32_t* woff = L.wcount + wave * 256u;
    for (uint32_t j = lane; j < 256u; j += kWave)
        woff[j] = 0;
    if (tid == 0)
        sm.flag = 0;
    const unsigned long long lower = (1ull << lane) - 1ull;
    // per-wave digit counts (the row is private to the wave: in-order LDS, no barrier needed).  Four groups
    // are fetched per trip, from clamped positions, so that their latencies overlap.
    for (uint32_t base = beg; base < end; base += 4u * kWave) {
        uint32_t key[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u)
            key[u] = ksrc[min(base + u * kWave + lane, end - 1u)];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const bool valid = base + u * kWave + lane < end;
            const uint32_t dg = valid ? ((key[u] >> shift) & 255u) : 0u;
            const unsigned long long mm = match_digit(dg, valid);
            if (valid && (mm & lower) == 0)
                woff[dg] += (uint32_t)__popcll(mm);
        }
    }
    __syncthreads();
    // digit totals -> global offsets; wave rows become each wave's first output position per digit
    uint32_t mine = 0;
    if (tid < 256)
        for (int w = 0; w < kWaves; ++w)
            mine += L.wcount[w * 256 + tid];
    if (tid < 256 && mine == n)
        sm.flag = 1;
    uint32_t tot;
    uint32_t acc = block_excl_scan_u32(mine, tot, sm.bs); // its barriers publish sm.flag
    if (sm.flag)
        return false;
    if (tid < 256)
        for (int w = 0; w < kWaves; ++w) {
            const uint32_t t = L.wcount[w * 256 + tid];
            L.wcount[w * 256 + tid] = acc;
            acc += t;
        }
    __syncthreads();
    for (uint32_t base = beg; base < end; base += 4u * kWave) {
        uint32_t key[4], id[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint32_t i = min(base + u * kWave + lane, end - 1u);
            key[u] = ksrc[i];
            id[u] = isrc[i];
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const bool valid = base + u * kWave + lane < end;
            const uint32_t dg = valid ? ((key[u] >> shift) & 255u) : 0u;
            const unsigned long long mm = match_digit(dg, valid);
            const uint32_t off = woff[dg];
            if (valid) {
                const uint32_t pos = off + (uint32_t)__popcll(mm & lower);
                kdst[pos] = key[u];
                idst[pos] = id[u];
                if ((mm & lower) == 0)
                    woff[dg] = off + (uint32_t)__popcll(mm);
            }
        }
    }
    __syncthreads();
    return true;
}

__device__ void sort_segment(uint32_t* k0, uint32_t* i0, uint32_t* k1, uint32_t* i1, uint32_t n, const FinishLds& L);

// libstdc++'s __heap_select(first, nth + 1, last) followed by iter_swap(first, nth) (bits/stl_algo.h:1956-1960,
// stl_heap.h): where introselect ends up when its depth limit is spent.  The arrangement it leaves is the library's,
// entry for entry, but the time is bounded:
//  * __make_heap sifts the parents from the last one down to the root.  A sift only touches the subtree of its
//    node and the subtrees of one level are disjoint, so a level's sifts run side by side, one thread each, level
//    after level from the bottom: the heap's depth in rounds instead of its size in dependent steps.
//  * the sweep `for (i = middle; i < last; ++i) if (comp(i, first)) __pop_heap(...)` is done by one wave, 64 entries
//    per ballot against the current root: entries that do not beat the root cost nothing, the first that does is
//    popped in (a sequential sift from the root), the lanes behind it are asked again (the root only ever moves
//    towards the heavy end, so whoever failed before fails again).
//  * the heap's first `cache_cap` entries (its upper levels, or all of it) live in LDS while this runs.
// get / put: the range in device memory or LDS, as introselect_rounds() has it.  cache: room for cache_cap values in
// LDS (0: the range is in LDS already).  All threads call.
template <typename Get, typename Put>
__device__ void heap_select_rest(Get get, Put put, uint32_t first, uint32_t last, uint32_t nth, unsigned long long* cache,
                                 uint32_t cache_cap)
{
    typedef unsigned long long u64;
    const uint32_t tid = threadIdx.x, lane = lane_id();
    const uint32_t middle = nth + 1u - first, len = last - first;
    const uint32_t cached = min(middle, cache_cap);
    for (uint32_t i = tid; i < cached; i += kThreads)
        cache[i] = get(first + i);
    __syncthreads();
    auto hget = [&](uint32_t j) -> u64 { return j < cached ? cache[j] : get(first + j); };
    auto hput = [&](uint32_t j, u64 v) {
        if (j < cached)
            cache[j] = v;
        else
            put(first + j, v);
    };
    auto sift = [&](uint32_t hole, u64 v) { // __adjust_heap: the hole sinks to a leaf, v rises from there
        const uint32_t top = hole;
        uint32_t child = hole;
        while (child < (middle - 1u) / 2u) {
            child = 2u * (child + 1u);
            if (hget(child) < hget(child - 1u))
                --child;
            hput(hole, hget(child));
            hole = child;
        }
        if ((middle & 1u) == 0 && middle >= 2u && child == (middle - 2u) / 2u) {
            child = 2u * (child + 1u);
            hput(hole, hget(child - 1u));
            hole = child - 1u;
        }
        while (hole > top) {
            const uint32_t parent = (hole - 1u) / 2u;
            if (!(hget(parent) < v))
                break;
            hput(hole, hget(parent));
            hole = parent;
        }
        hput(hole, v);
    };
    if (middle >= 2u) {
        const uint32_t last_parent = (middle - 2u) / 2u;
        // (node p sits on level floor(log2(p + 1)), which holds the nodes 2^level - 1 .. 2^(level + 1) - 2)
        for (int level = 31 - __clz((int)(last_parent + 1u)); level >= 0; --level) {
            const uint32_t lo = (1u << level) - 1u, hi = min(last_parent, (2u << level) - 2u);
            for (uint32_t p = lo + tid; p <= hi; p += kThreads)
                sift(p, hget(p));
            __syncthreads();
        }
    }
    if (wave_id() == 0 && middle < len) {
        constexpr uint32_t kTrip = 4;
        u64 root = hget(0u); // (the same in every lane)
        for (uint32_t base = middle; base < len; base += kWave * kTrip) {
            u64 v[kTrip];
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u)
                v[u] = get(first + min(base + u * kWave + lane, len - 1u));
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u) {
                const bool in = base + u * kWave + lane < len;
                u64 bal = __ballot(in && v[u] < root);
                while (bal) { // uniform
                    const int l = __ffsll((long long)bal) - 1;
                    const u64 hit = ((u64)(uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v[u] >> 32), l) << 32) |
                                    (u64)(uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v[u], l);
                    // __pop_heap(first, middle, i): the root goes to the entry's place, the entry sinks in from the root
                    // (every lane does the same stores and loads: each then reads back what it wrote itself)
                    put(first + base + u * kWave + (uint32_t)l, root);
                    sift(0u, hit);
                    root = hget(0u);
                    bal = __ballot(in && v[u] < root) & ~((2ull << l) - 1ull);
                }
            }
        }
    }
    __syncthreads();
    for (uint32_t i = tid; i < cached; i += kThreads)
        put(first + i, cache[i]);
    __syncthreads();
    if (tid == 0) {
        const u64 a = get(first), b = get(nth);
        put(first, b);
        put(nth, a);
    }
    __syncthreads();
}

// std::ranges::nth_element(cand, cand + nth, desc) of src/gen/sampler.cpp:41 as libstdc++ 11 runs it (introselect,
// bits/stl_algo.h:1964), leaving the first nth candidates in exactly the arrangement that library leaves: the
// reference keeps those (sampler.cpp:42) and sums and walks them in that order when no top-p follows.  What lies behind
// a cut that the rounds leave behind them is not kept up.  key/idx hold n candidates (~bits(q), token id); `desc` is
// the order of the 64-bit values key << 32 | idx, all distinct.
// One round = median of three to the front, then the unguarded Hoare partition of the rest around it.  That
// partition swaps the t-th entry from the left that belongs right with the t-th entry from the right that belongs
// left for as long as the former lies before the latter, and cuts behind the entries that belong left: the two
// position lists come from ballots (wave w owns the w-th sixteenth of the range), the swaps are independent.
// The depth limit's heap select is heap_select_rest() above; the last insertion sort (at most three entries) is one
// thread's.
//
// introselect_rounds runs the rounds on [first, last) through get(i) / get_key(i) (the high half alone) / put(i, v)
// until the range is no longer than `until` (3 = to the end, insertion sort included).  lsta / lstb: room for
// last - first positions each.  cache / cache_cap: LDS for heap_select_rest().  Returns true when nothing is left to
// do.
template <typename Get, typename GetKey, typename Put>
__device__ bool introselect_rounds(Get get, GetKey get_key, Put put, uint32_t& first, uint32_t& last, uint32_t nth, uint32_t& depth,
                                   uint32_t until, uint32_t* lsta, uint32_t* lstb, FinishShared& sm,
                                   unsigned long long* cache, uint32_t cache_cap)
{
    typedef unsigned long long u64;
    const uint32_t tid = threadIdx.x, lane = lane_id(), wave = wave_id();
    while (last - first > until) {
        if (depth == 0) {
            heap_select_rest(get, put, first, last, nth, cache, cache_cap);
            return true;
        }
        --depth;
        if (tid == 0) { // __move_median_to_first(first, first + 1, mid, last - 1)
            const uint32_t ix = first + 1u, iy = first + (last - first) / 2u, iz = last - 1u;
            const u64 x = get(ix), y = get(iy), z = get(iz), r = get(first); // (one trip to memory)
            uint32_t im;
            u64 med;
            if (x < y) {
                im = y < z ? iy : (x < z ? iz : ix);
                med = y < z ? y : (x < z ? z : x);
            } else {
                im = x < z ? ix : (y < z ? iz : iy);
                med = x < z ? x : (y < z ? z : y);
            }
            put(first, med);
            put(im, r);
            sm.bs.f64[0] = __longlong_as_double((long long)med); // (the pivot, for everyone)
            sm.bs.bcast = 0;                                     // the pairs that change places, counted below
        }
        __syncthreads();
        const u64 pivot = (u64)__double_as_longlong(sm.bs.f64[0]);
        // (scalars, like all of a wave's bounds and counts below)
        const uint32_t lo0 = uniform_u32(first + 1u), last_s = uniform_u32(last), len = last_s - lo0;
        const uint32_t chunk = ((len + kThreads - 1u) / kThreads) * kWave; // per wave, a multiple of 64
        const uint32_t beg = uniform_u32(min(last_s, lo0 + wave * chunk)), end = min(last_s, beg + chunk);
        // entries of the wave's chunk that belong left of the cut
        // (kTrip loads in flight per lane: a trip costs one round trip to memory, not kTrip; the high halves decide
        // but for an entry whose weight is the pivot's; one workgroup's instruction issue bounds these passes, so they
        // keep what they can in wave masks: per entry one compare, the masks' scalar arithmetic, and for an entry
        // that is listed its rank among the mask's lanes)
        constexpr uint32_t kTrip = 8;
        const uint32_t pivot_key = uniform_u32((uint32_t)(pivot >> 32));
        // left[u] / in[u]: the lanes whose entry base + 64 u + lane belongs left / lies in the chunk
        auto trip_masks = [&](uint32_t base, u64 (&left)[kTrip], u64 (&in)[kTrip]) {
            uint32_t k[kTrip];
            u64 ties = 0;
            if (base + kWave * kTrip <= end) { // (uniform)
                const size_t at = (size_t)base + lane;
#pragma unroll
                for (uint32_t u = 0; u < kTrip; ++u)
                    k[u] = get_key(at + u * kWave);
#pragma unroll
                for (uint32_t u = 0; u < kTrip; ++u) {
                    in[u] = ~0ull;
                    left[u] = __builtin_amdgcn_ballot_w64(k[u] < pivot_key);
                    ties |= __builtin_amdgcn_ballot_w64(k[u] == pivot_key);
                }
            } else {
                // (the chunk's last trip: only its loads that reach into the chunk, which on the short ranges of the
                // rounds in LDS is one in eight; scalar branches)
#pragma unroll
                for (uint32_t u = 0; u < kTrip; ++u) {
                    k[u] = 0u;
                    if (base + u * kWave < end)
                        k[u] = get_key((size_t)min(base + u * kWave + lane, last_s - 1u));
                }
#pragma unroll
                for (uint32_t u = 0; u < kTrip; ++u) {
                    in[u] = left[u] = 0ull;
                    if (base + u * kWave < end) {
                        in[u] = __builtin_amdgcn_ballot_w64(base + u * kWave + lane < end);
                        left[u] = __builtin_amdgcn_ballot_w64(k[u] < pivot_key) & in[u];
                        ties |= __builtin_amdgcn_ballot_w64(k[u] == pivot_key) & in[u];
                    }
                }
            }
            if (ties) { // (rare)
#pragma unroll
                for (uint32_t u = 0; u < kTrip; ++u) {
                    if (!in[u])
                        continue;
                    const uint32_t pos = base + u * kWave + lane;
                    bool l = false;
                    if (pos < end && k[u] == pivot_key)
                        l = get(pos) < pivot;
                    left[u] |= __builtin_amdgcn_ballot_w64(l);
                }
            }
        };
        auto rank_in = [](u64 m) { return __builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u)); };
        uint32_t mine = 0;
        for (uint32_t base = beg; base < end; base += kWave * kTrip) {
            u64 left[kTrip], in[kTrip];
            trip_masks(base, left, in);
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u)
                mine += (uint32_t)__popcll(left[u]);
        }
        if (lane == 0)
            sm.bs.u64[wave] = mine;
        __syncthreads();
        uint32_t small_before = 0, smalls = 0;
        for (int w = 0; w < kWaves; ++w) {
            const uint32_t x = (uint32_t)sm.bs.u64[w];
            if (w < (int)wave)
                small_before += x;
            smalls += x;
        }
        small_before = uniform_u32(small_before);
        smalls = uniform_u32(smalls);
        const uint32_t cut = lo0 + smalls;
        // Only the big entries before the cut and the small ones behind it change places, the t-th of the former
        // with the t-th of the latter counted from the right: as many of one kind as of the other.  When the rounds go
        // on in the left part (cut > nth), what lies behind the cut is never read again (nth_element's caller keeps the
        // first nth entries only): the big entries need not be moved there.
        const bool right_kept = cut <= nth;
        uint32_t big_before = (beg - lo0) - small_before;
        // position lists: lsta[t] = the t-th big entry from the left (those before the cut), lstb[t] = the t-th small
        // entry from the left (those behind it)
        uint32_t moving = 0; // big entries of the wave's chunk before the cut
        for (uint32_t base = beg; base < end; base += kWave * kTrip) {
            u64 left[kTrip], in[kTrip];
            trip_masks(base, left, in);
            if (base + kWave * kTrip <= cut) { // (uniform; all but one of the chunks' trips lie on one side of the cut)
#pragma unroll
                for (uint32_t u = 0; u < kTrip; ++u) {
                    if (!in[u]) // (scalar: a trip's part beyond the chunk)
                        continue;
                    const u64 big = in[u] & ~left[u];
                    if ((big >> lane) & 1ull)
                        lsta[big_before + rank_in(big)] = base + u * kWave + lane;
                    const uint32_t nb = (uint32_t)__popcll(big);
                    big_before += nb;
                    moving += nb;
                    small_before += (uint32_t)__popcll(left[u]);
                }
            } else if (base >= cut) {
#pragma unroll
                for (uint32_t u = 0; u < kTrip; ++u) {
                    if (!left[u])
                        continue;
                    if ((left[u] >> lane) & 1ull)
                        lstb[small_before + rank_in(left[u])] = base + u * kWave + lane;
                    small_before += (uint32_t)__popcll(left[u]);
                }
            } else {
#pragma unroll
                for (uint32_t u = 0; u < kTrip; ++u) {
                    if (!in[u])
                        continue;
                    const uint32_t pos = base + u * kWave + lane;
                    const u64 big = in[u] & ~left[u];
                    const u64 before = __builtin_amdgcn_ballot_w64(pos < cut);
                    if ((left[u] >> lane) & 1ull) {
                        if (pos >= cut)
                            lstb[small_before + rank_in(left[u])] = pos;
                    } else if (((big >> lane) & 1ull) && pos < cut)
                        lsta[big_before + rank_in(big)] = pos;
                    big_before += (uint32_t)__popcll(big);
                    moving += (uint32_t)__popcll(big & before);
                    small_before += (uint32_t)__popcll(left[u]);
                }
            }
        }
        if (lane == 0 && moving)
            atomicAdd(&sm.bs.bcast, (u64)moving);
        __syncthreads();
        const uint32_t pairs = (uint32_t)sm.bs.bcast;
        for (uint32_t t = tid; t < pairs; t += kThreads) {
            const uint32_t a = lsta[t], b = lstb[smalls - 1u - t];
            const u64 vb = get(b);
            if (right_kept)
                put(b, get(a));
            put(a, vb);
        }
        __syncthreads();
        if (right_kept)
            first = cut;
        else
            last = cut;
    }
    if (last - first > 3u)
        return false;
    if (tid == 0) // __insertion_sort(first, last)
        for (uint32_t i = first + 1u; i < last; ++i) {
            const u64 v = get(i);
            uint32_t j = i;
            if (v < get(first)) {
                for (; j > first; --j)
                    put(j, get(j - 1u));
            } else {
                for (; v < get(j - 1u); --j)
                    put(j, get(j - 1u));
            }
            put(j, v);
        }
    __syncthreads();
    return true;
}

// The row's candidates in device memory (key[i], idx[i]; lsta / lstb: room for n positions each).  The rounds run on
// device memory, ten or so dependent trips to memory each, until the range fits the dynamic LDS block (kSortMax
// entries and two position lists); the remaining dozen rounds run on a copy there.
__device__ void nth_element_row(uint32_t* key, uint32_t* idx, uint32_t n, uint32_t nth, uint32_t* lsta, uint32_t* lstb,
                                const FinishLds& L)
{
    assume_lds(L);
    typedef unsigned long long u64;
    const uint32_t tid = threadIdx.x;
    if (n == 0 || nth >= n)
        return;
    uint32_t first = 0, last = n;
    uint32_t depth = 2u * (31u - (uint32_t)__clz((int)n));
    __syncthreads();
    auto get = [=](uint32_t i) { return ((u64)key[i] << 32) | (u64)idx[i]; };
    auto put = [=](uint32_t i, u64 v) {
        key[i] = (uint32_t)(v >> 32);
        idx[i] = (uint32_t)v;
    };
    // (the rounds in device memory use no LDS of their own: the whole block holds the heap's upper levels if the
    // depth limit is reached here)
    if (introselect_rounds(get, [=](size_t i) { return key[i]; }, put, first, last, nth, depth, kSortMax, lsta, lstb, *L.sm, L.sortk,
                           kDynLds / 8u))
        return;
    u64* lds = L.sortk;
    uint32_t* la = reinterpret_cast<uint32_t*>(L.sortk + kSortMax);
    uint32_t* lb = la + kSortMax;
    static_assert(kSortMax * 16u <= kDynLds, "the range and its two position lists fit the dynamic LDS block");
    const uint32_t base = first, len = last - first;
    for (uint32_t i = tid; i < len; i += kThreads)
        lds[i] = get(base + i);
    __syncthreads();
    introselect_rounds([=](uint32_t i) { return lds[i - base]; }, [=](size_t i) { return (uint32_t)(lds[i - base] >> 32); },
                       [=](uint32_t i, u64 v) { lds[i - base] = v; }, first, last, nth, depth, 3u, la, lb, *L.sm, nullptr, 0u);
    for (uint32_t i = tid; i < len; i += kThreads)
        put(base + i, lds[i]);
    __syncthreads();
}

// key0 / idx0 <- the row's candidates in index order (~bits(q), token id), from its bits(q) array qb[0 .. V) (bits(q)
// of every candidate at its index, 0 elsewhere), as general_row() first leaves them.  All threads call.  (Only for
// the rare second look at a row: one entry per lane and round.)
__device__ MAKO_RARE_CALL void compact_candidates(const uint32_t* qb, uint32_t V, uint32_t* key0, uint32_t* idx0, FinishShared& sm)
{
    const uint32_t lane = lane_id(), wave = wave_id();
    const uint32_t chunk = (V + kWaves - 1u) / kWaves;
    const uint32_t beg = min(V, wave * chunk), end = min(V, beg + chunk);
    uint32_t mine = 0;
    for (uint32_t i = beg + lane; i < end; i += kWave)
        mine += qb[i] ? 1u : 0u;
    mine = __ockl_wfred_add_u32(mine);
    __syncthreads();
    if (lane == 0)
        sm.bs.u64[wave] = mine;
    __syncthreads();
    uint32_t at = 0;
    for (uint32_t w = 0; w < wave; ++w)
        at += (uint32_t)sm.bs.u64[w];
    for (uint32_t base = beg; base < end; base += kWave) {
        const uint32_t i = base + lane;
        const uint32_t k = i < end ? qb[i] : 0u;
        const unsigned long long bal = __ballot(k != 0u);
        if (k) {
            const uint32_t pos = at + (uint32_t)__popcll(bal & ((1ull << lane) - 1ull));
            key0[pos] = ~k;
            idx0[pos] = i;
        }
        at += (uint32_t)__popcll(bal);
    }
    __syncthreads();
}

// Common tail of the whole-row paths.  key[0]/idx[0] of the row hold n0 candidates (~bits(q), token id) in index
// order.  Sorts them by (q desc, idx asc) when top-k or top-p is active, truncates (src/gen/sampler.cpp:39-61)
// and draws.  `total64` (when have_total) is the fp64 sum of q over all candidates of the row, of which the list
// may be only the heaviest part; otherwise it is summed from the list.  The row's bits(q) array (sc.wbuf: bits(q) of
// every candidate at its index, 0 elsewhere) must be in place.
// (TOPK_ALONE = false leaves the top-k-without-top-p branch out of the instance inside plan_kernel: that kernel is
// only launched for batches whose host copy of the parameters shows a top-p on every sampled row, and the branch's
// registers would be spilled around the top-k rows' fast path, +3.5 us on a 256-row batch.)
template <bool TOPK_ALONE>
__device__ void sort_truncate_draw(const mako_sample_desc& d, const Scratch& sc, uint32_t row, const mako_sampling_params& P,
                                   uint32_t n0, bool have_total, double total64, uint32_t path, const FinishLds& L)
{
    assume_lds(L);
    FinishShared& sm = *L.sm;
    uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
    uint32_t* key1 = sc.key[1] + (size_t)row * sc.vpad;
    uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
    uint32_t* idx1 = sc.idx[1] + (size_t)row * sc.vpad;

    // order by (q desc, idx asc): stable LSD radix sort of ~bits(q), ascending
    const bool topk_active = P.top_k > 0 && P.top_k < n0;
    const bool topp_active = P.top_p < 1.0f;
    // top-k alone: the survivors stay in the order nth_element leaves them (sampler.cpp:39-43, then :79-83)
    const bool nth_order = TOPK_ALONE && topk_active && !topp_active;
    if (nth_order)
        nth_element_row(key0, idx0, n0, P.top_k, key1, idx1, L);
    else if (topk_active) {
        // a top-p follows: the survivors are sorted, so only which candidates they are matters, and `desc` is a total
        // order: nth_element's first top_k entries are the top_k first of the sorted list, in some order.  The
        // partitions and a sort of top_k entries cost a quarter of the sort of all candidates.
        nth_element_row(key0, idx0, n0, P.top_k, key1, idx1, L);
        sort_segment(idx0, key0, idx1, key1, P.top_k, L); // (stable sorts: token ids first, then the weights)
        sort_segment(key0, idx0, key1, idx1, P.top_k, L);
    } else if (topp_active)
        sort_segment(key0, idx0, key1, idx1, n0, L);
    const uint32_t *ks = key0, *is = idx0;
    MAKO_STAMP(12);
    const uint32_t n1 = topk_active ? P.top_k : n0; // sampler.cpp:40-43
    // (sorted_tail's one-wave path for lists of up to kGroup entries adds and walks them in the order given, whatever
    // it is, and without a top-p it cuts nothing: nth_element's survivors take it too)
    if (nth_order ? (!d.draft && n1 <= kGroup) : (topk_active || topp_active)) {
        if (sorted_tail(d, row, P, ks, is, n1, have_total, total64, path, L))
            return;
        // Too close to call (top-p rows only): the reference's total decides, summed in the order its candidates have
        // at that point (sampler.cpp:40-48).
        if (topk_active) {
            // the order nth_element leaves the survivors in: from the candidates in index order again
            compact_candidates(reinterpret_cast<const uint32_t*>(sc.wbuf + (size_t)row * sc.vpad), d.n_vocab, key0, idx0, sm);
            nth_element_row(key0, idx0, n0, P.top_k, key1, idx1, L);
            total64 = reference_total([=](uint32_t i) { return __uint_as_float(~key0[i]); }, n1, sm);
            sort_segment(idx0, key0, idx1, key1, n1, L); // (equal weights by token id, as in the list of all candidates)
            sort_segment(key0, idx0, key1, idx1, n1, L);
        } else {
            // index order: the row's bits(q) array (the zeros of the logits that are no candidates add nothing)
            const uint32_t* qk = reinterpret_cast<const uint32_t*>(sc.wbuf + (size_t)row * sc.vpad);
            total64 = reference_total([=](uint32_t i) { return __uint_as_float(qk[i]); }, d.n_vocab, sm);
        }
        sorted_tail_exact(d, row, P, ks, is, n1, total64, path, L);
        return;
    }
    // nth_element's order (long lists, verification), or neither top-k nor top-p: the candidates stay in index order
    const uint32_t* kf = ks;
    const uint32_t* jf = is;
    draw_from_list(
        d, row, [=](uint32_t i) { return __uint_as_float(~kf[i]); }, [=](uint32_t i) { return jf[i]; }, n1, path, sm);
}

// Sorts n (key, id) pairs at (k0, i0) by key ascending, stably, with (k1, i1) as the second buffer; the result
// ends in (k0, i0).
__device__ void sort_segment(uint32_t* k0, uint32_t* i0, uint32_t* k1, uint32_t* i1, uint32_t n, const FinishLds& L)
{
    assume_lds(L);
    if (n < 2)
        return;
    uint32_t *ks = k0, *is = i0, *kd = k1, *id = i1;
    for (uint32_t shift = 0; shift < 32; shift += 8) {
        if (radix_pass(ks, is, kd, id, n, shift, L)) {
            uint32_t* t = ks;
            ks = kd;
            kd = t;
            t = is;
            is = id;
            id = t;
        }
        __syncthreads();
    }
    if (ks != k0) {
        for (uint32_t i = threadIdx.x; i < n; i += kThreads) {
            k0[i] = ks[i];
            i0[i] = is[i];
        }
        __syncthreads();
    }
}

// Whole-row path: exact for every parameter combination.  One workgroup rebuilds the penalised
// row in scratch, keeps the candidates, sorts them by (q desc, idx asc) when top-k or top-p is
// active, truncates, and draws.  src/gen/sampler.cpp:20-62.
// (SITE: sort_kernel, its usual place, has an instance to itself, so that the compiler treats that kernel the same
// whether or not the instances inside plan_kernel exist.)
template <int SITE>
__device__ MAKO_RARE_CALL void general_row(const mako_sample_desc& d, const Scratch& sc, uint32_t row, const mako_sampling_params& P,
                            float m, uint32_t argidx, const FinishLds& L)
{
    assume_lds(L);
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
    const uint32_t V = d.n_vocab;
    float* wbuf = sc.wbuf + (size_t)row * sc.vpad;
    uint32_t* cnt = sc.cnt + (size_t)row * sc.vpad;
    uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
    uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
    const float* lrow = d.logits + (int64_t)row * d.logits_stride;
    const uint32_t* mrow = d.mask ? d.mask + (int64_t)row * d.mask_stride : nullptr;

    // 1. masked copy, then the penalties once per distinct history token
    for (uint32_t i = tid; i < V; i += kThreads) {
        float v = lrow[i];
        if (mrow && !((mrow[i >> 5] >> (i & 31u)) & 1u))
            v = -INFINITY;
        wbuf[i] = v;
    }
    __syncthreads();
    const uint32_t hl = d.hist_tokens ? d.hist_len[row] : 0u;
    if (hl > 0 && !penalties_neutral(P)) {
        const int32_t* ht = d.hist_tokens + (int64_t)row * d.hist_stride;
        const uint32_t* hc = d.hist_counts ? d.hist_counts + (int64_t)row * d.hist_stride : nullptr;
        for (uint32_t h = tid; h < hl; h += kThreads) {
            const uint32_t t = (uint32_t)ht[h];
            if (t < V)
                atomicAdd(&cnt[t], hc ? hc[h] : 1u);
        }
        __syncthreads();
        for (uint32_t h = tid; h < hl; h += kThreads) {
            const uint32_t t = (uint32_t)ht[h];
            if (t < V) {
                const uint32_t c = atomicExch(&cnt[t], 0u); // claims the token and restores the zero
                if (c)
                    wbuf[t] = penalize(wbuf[t], c, P.repetition_penalty, P.presence_penalty, P.frequency_penalty);
            }
        }
        __syncthreads();
    }

    // 2. weights and the min_p / q > 0 filter, compacted in index order (sampler.cpp:29-36).  Wave w owns the w-th
    // sixteenth of the row (a multiple of 256 logits, lane l entries 4l..4l+3 of each 256): a sweep that leaves bits(q)
    // of every candidate (0 otherwise) in place of the logit and counts them, one exchange of the waves' totals, and
    // a sweep in which every lane reads back what it wrote and a wave scan ranks it.  No barrier inside the sweeps.
    const float inv_t = 1.0f / P.temperature;
    const float floor_q = (1.0f < P.min_p) ? 1.0f : P.min_p; // std::min(min_p, 1.0f)
    uint32_t* qb = reinterpret_cast<uint32_t*>(wbuf);
    const uint32_t lane = lane_id(), wave = wave_id();
    const uint32_t chunk = ((V + kThreads * 4u - 1u) / (kThreads * 4u)) * kGroup;
    const uint32_t beg = min(V, wave * chunk), end = min(V, beg + chunk);
    uint32_t mine = 0;
    for (uint32_t base = beg; base < end; base += kGroup) {
        const uint32_t i = base + lane * 4u;
        float w[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        const bool whole = i + 3u < end;
        if (whole) {
            const float4 x = *reinterpret_cast<const float4*>(wbuf + i);
            w[0] = x.x, w[1] = x.y, w[2] = x.z, w[3] = x.w;
        } else {
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                if (i + j < end)
                    w[j] = wbuf[i + j];
        }
        uint32_t k[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const float q = weight_of(w[j], m, inv_t, sm.tab);
            k[j] = (i + j < end && q >= floor_q && q > 0.0f) ? __float_as_uint(q) : 0u;
            mine += k[j] ? 1u : 0u;
        }
        if (whole) {
            *reinterpret_cast<uint4*>(qb + i) = make_uint4(k[0], k[1], k[2], k[3]);
        } else {
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                if (i + j < end)
                    qb[i + j] = k[j];
        }
    }
    mine = __ockl_wfred_add_u32(mine);
    if (lane == 0)
        sm.bs.u64[wave] = mine;
    __syncthreads();
    uint32_t n0 = 0, at = 0;
    for (int w = 0; w < kWaves; ++w) {
        const uint32_t x = (uint32_t)sm.bs.u64[w];
        if (w < (int)wave)
            at += x;
        n0 += x;
    }
    for (uint32_t base = beg; base < end; base += kGroup) {
        const uint32_t i = base + lane * 4u;
        uint32_t k[4] = {0u, 0u, 0u, 0u};
        if (i + 3u < end) {
            const uint4 x = *reinterpret_cast<const uint4*>(qb + i);
            k[0] = x.x, k[1] = x.y, k[2] = x.z, k[3] = x.w;
        } else {
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                if (i + j < end)
                    k[j] = qb[i + j];
        }
        const uint32_t c = (k[0] ? 1u : 0u) + (k[1] ? 1u : 0u) + (k[2] ? 1u : 0u) + (k[3] ? 1u : 0u);
        const uint32_t incl = __ockl_wfscan_add_u32(c, true);
        uint32_t pos = at + incl - c;
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            if (k[j]) {
                MAKO_CHECK(sc, kCheckCompact, pos < n0 && (uint64_t)pos < sc.vpad);
                key0[pos] = ~k[j];
                idx0[pos] = i + j;
                ++pos;
            }
        at += (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
    }
    __syncthreads();

    if (n0 == 0) {
        fallback_row(d, row, argidx);
        return;
    }
    sort_truncate_draw<SITE == 0>(d, sc, row, P, n0, false, 0.0, MAKO_PATH_GENERAL, L);
}

// The whole-row path for a row whose weights are already in place: sc.wbuf of the row holds bits(q) of every candidate at
// its index and 0 elsewhere, as general_row()'s first sweep leaves it (index_weights_kernel writes the same array with a
// workgroup per 16 384 logits instead of one for the row).  Counts and compacts the candidates in index order and goes
// on like general_row().  All threads call; `argidx`: the row's first maximum, for a row without candidates.
// `listed`: true when that kernel found every logit a candidate (no mask, no floor, no underflow: the usual row) and
// has left the list itself as well, (~bits(q), i) at i in key[0] / idx[0] of the row: nothing to count or to compact.
template <int SITE>
__device__ MAKO_RARE_CALL void general_row_from_weights(const mako_sample_desc& d, const Scratch& sc, uint32_t row,
                                                        const mako_sampling_params& P, uint32_t argidx, bool listed,
                                                        const FinishLds& L)
{
    assume_lds(L);
    FinishShared& sm = *L.sm;
    const uint32_t V = d.n_vocab;
    if (listed) { // uniform
        sort_truncate_draw<SITE == 0>(d, sc, row, P, V, false, 0.0, MAKO_PATH_GENERAL, L);
        return;
    }
    const uint32_t* qb = reinterpret_cast<const uint32_t*>(sc.wbuf + (size_t)row * sc.vpad);
    uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
    uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
    const uint32_t lane = lane_id(), wave = wave_id();
    // (wave w owns the w-th sixteenth of the row, a multiple of 256 logits, lane l entries 4l..4l+3 of each 256; eight
    // such blocks' loads are in flight per trip, from clamped addresses and masked afterwards: one round trip to memory
    // per 2 048 entries of the wave instead of one per 256)
    const uint32_t chunk = ((V + kThreads * 4u - 1u) / (kThreads * 4u)) * kGroup;
    const uint32_t beg = min(V, wave * chunk), end = min(V, beg + chunk);
    const uint32_t last_vec = (uint32_t)sc.vpad - 4u; // (vpad is a multiple of 1024)
    constexpr uint32_t kTrip = 8;
    auto load_trip = [&](uint32_t base, uint32_t (&k)[kTrip][4]) {
        uint4 x[kTrip];
#pragma unroll
        for (uint32_t u = 0; u < kTrip; ++u)
            x[u] = *reinterpret_cast<const uint4*>(qb + min(base + u * kGroup + lane * 4u, last_vec));
#pragma unroll
        for (uint32_t u = 0; u < kTrip; ++u) {
            const uint32_t i = base + u * kGroup + lane * 4u;
            k[u][0] = i < end ? x[u].x : 0u;
            k[u][1] = i + 1u < end ? x[u].y : 0u;
            k[u][2] = i + 2u < end ? x[u].z : 0u;
            k[u][3] = i + 3u < end ? x[u].w : 0u;
        }
    };
    uint32_t mine = 0;
    for (uint32_t base = beg; base < end; base += kGroup * kTrip) {
        uint32_t k[kTrip][4];
        load_trip(base, k);
#pragma unroll
        for (uint32_t u = 0; u < kTrip; ++u)
            mine += (k[u][0] ? 1u : 0u) + (k[u][1] ? 1u : 0u) + (k[u][2] ? 1u : 0u) + (k[u][3] ? 1u : 0u);
    }
    mine = __ockl_wfred_add_u32(mine);
    __syncthreads();
    if (lane == 0)
        sm.bs.u64[wave] = mine;
    __syncthreads();
    uint32_t n0 = 0, at = 0;
    for (int w = 0; w < kWaves; ++w) {
        const uint32_t x = (uint32_t)sm.bs.u64[w];
        if (w < (int)wave)
            at += x;
        n0 += x;
    }
    if (n0 == V) {
        // every logit is a candidate (no mask, no floor, no underflow: the usual row): the list is the array itself,
        // written four entries per lane and store
        for (uint32_t base = beg; base < end; base += kGroup * kTrip) {
            uint32_t k[kTrip][4];
            load_trip(base, k);
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u) {
                const uint32_t i = base + u * kGroup + lane * 4u;
                if (i + 3u < end) {
                    *reinterpret_cast<uint4*>(key0 + i) = make_uint4(~k[u][0], ~k[u][1], ~k[u][2], ~k[u][3]);
                    *reinterpret_cast<uint4*>(idx0 + i) = make_uint4(i, i + 1u, i + 2u, i + 3u);
                } else {
#pragma unroll
                    for (uint32_t j = 0; j < 4; ++j)
                        if (i + j < end) {
                            key0[i + j] = ~k[u][j];
                            idx0[i + j] = i + j;
                        }
                }
            }
        }
    } else {
        for (uint32_t base = beg; base < end; base += kGroup * kTrip) {
            uint32_t k[kTrip][4];
            load_trip(base, k);
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u) {
                const uint32_t i = base + u * kGroup + lane * 4u;
                const uint32_t c = (k[u][0] ? 1u : 0u) + (k[u][1] ? 1u : 0u) + (k[u][2] ? 1u : 0u) + (k[u][3] ? 1u : 0u);
                const uint32_t incl = __ockl_wfscan_add_u32(c, true);
                uint32_t pos = at + incl - c;
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j)
                    if (k[u][j]) {
                        MAKO_CHECK(sc, kCheckCompact, pos < n0 && (uint64_t)pos < sc.vpad);
                        key0[pos] = ~k[u][j];
                        idx0[pos] = i + j;
                        ++pos;
                    }
                at += (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
            }
        }
    }
    __syncthreads();
    if (n0 == 0) {
        fallback_row(d, row, argidx);
        return;
    }
    sort_truncate_draw<SITE == 0>(d, sc, row, P, n0, false, 0.0, MAKO_PATH_GENERAL, L);
}


} // namespace mako
