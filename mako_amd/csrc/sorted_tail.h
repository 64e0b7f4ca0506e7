// Sorted candidate lists: top-p cut, exact fp32 total and walk in groups of 256 entries.
#pragma once

#include "generic_replay.h"
#include "unsorted_shares.h"

namespace mako {

constexpr uint32_t kWalkSeqGroups = 8; // leading groups in which the running sum may be added entry by entry from LDS
// (a walk expected to end within kHeadGroups groups goes entry by entry from LDS: two nanoseconds an entry, where a
// group that is walked by its map costs the chain a fraction of that but every binade r falls through a microsecond)
struct GroupLds { // carved from the dynamic LDS block once sorting is over; one pointer, the rest is offsets
    unsigned long long* base;
    __device__ __forceinline__ double* pg() const { return reinterpret_cast<double*>(base); } // [kMaxGroups + 2] fp64 sum of the entries before each group
    __device__ __forceinline__ uint32_t* d0() const { return reinterpret_cast<uint32_t*>(base + kMaxGroups + 2); } // [kMaxGroups] the group's map for the guessed epoch
    __device__ __forceinline__ uint32_t* d1() const { return d0() + kMaxGroups; }
    __device__ __forceinline__ uint32_t* cmax() const { return d1() + kMaxGroups; }
    __device__ __forceinline__ uint32_t* start() const { return cmax() + kMaxGroups; } // first entry of the group
    // entries (bits 0-8) | quarter-record slot + 1 (bits 9-15) | guessed exponent << 16
    __device__ __forceinline__ uint32_t* pack() const { return start() + kMaxGroups; }
    __device__ __forceinline__ uint32_t* misc() const { return pack() + kMaxGroups; } // [8]; misc[3] (and [4]: QuarterSlots) count the quarter-record slots in use
    // [kQuarterSlots][4], in the upper half of the dynamic LDS block
    __device__ __forceinline__ uint4* quarters() const { return reinterpret_cast<uint4*>(base + kSortMax); }
    // the walk's maps, bounds and packs ([kMaxGroups] each, behind the quarter records): built while the running
    // sum is still being chained, so they cannot share the arrays above
    __device__ __forceinline__ uint32_t* w_d0() const { return reinterpret_cast<uint32_t*>(base + kSortMax) + 1536; }
    __device__ __forceinline__ uint32_t* w_d1() const { return w_d0() + kMaxGroups; }
    __device__ __forceinline__ uint32_t* w_need() const { return w_d1() + kMaxGroups; }
    __device__ __forceinline__ uint32_t* w_pack() const { return w_need() + kMaxGroups; }
    // [kHeadGroups * kGroup + kWave] the head of the list as floats, for a walk that ends within it
    __device__ __forceinline__ float* head() const { return reinterpret_cast<float*>(w_pack() + kMaxGroups); }
};
constexpr uint32_t kLenMask = 0x1ffu;
constexpr uint32_t kHasQuarters = 1u << 31;
constexpr uint32_t kQuarterSlots = 96;
// Where a builder of group maps takes its quarter-record slots from: G.misc()[counter] counts those handed out of
// [first, first + slots).  (All of them from one counter, or, for long lists whose maps for the walk are built a block
// of groups ahead of the walk, the two halves in turn.)
struct QuarterSlots {
    uint32_t counter = 3, first = 0, slots = kQuarterSlots;
};
constexpr uint32_t kQuarter = kGroup / 4;
#ifndef MAKO_WALK_PASSED
#define MAKO_WALK_PASSED 1u
#endif
constexpr uint32_t kSeqMax = 1024; // sorted lists up to this long get their total and walk entry by entry

__device__ __forceinline__ GroupLds group_lds(const FinishLds& L)
{
    assume_lds(L);
    static_assert((kMaxGroups + 2) * 8 + 5 * kMaxGroups * 4 + 32 <= kSortMax * 8, "group records fit below the LDS lists");
    static_assert(kQuarterSlots * 16 == 1536 &&
                      kSortMax * 8 + 1536 * 4 + 4 * kMaxGroups * 4 + (kHeadGroups * kGroup + kWave) * 4 <= kTailLds,
                  "the walk's records sit behind the quarter records and fit the dynamic LDS block");
    return GroupLds{L.sortk};
}

// Values every lane of the wave holds alike, moved to scalar registers so that loops and branches on them
// compile to scalar control flow.
// A double from a lane whose number is the same for the whole wave.
__device__ __forceinline__ double readlane_f64(double v, uint32_t lane)
{
    const long long b = __double_as_longlong(v);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)b, (int)lane);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(b >> 32), (int)lane);
    return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

__device__ __forceinline__ uint32_t uniform_u32(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)v);
}

// Cross-lane moves on the VALU data path (DPP) instead of through the LDS crossbar: a dependent chain of six
// of them costs tens of cycles, not hundreds.  Lanes without a source lane receive 0.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_or_zero(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
}

// Inclusive scan, in lane order, of the 64 lanes' maps under composition (cmax is not touched).
__device__ __forceinline__ void wave_scan_maps(uint32_t& d0, uint32_t& d1)
{
    using seqfp::Step32;
#define MAKO_SCAN_STEP(CTRL, ROW_MASK)                                                                               \
    {                                                                                                                \
        const Step32 t = Step32{dpp_or_zero<CTRL, ROW_MASK>(d0), dpp_or_zero<CTRL, ROW_MASK>(d1), 0u};               \
        const Step32 r = seqfp::compose32(t, Step32{d0, d1, 0u}); /* earlier lanes first; {0, 0} is the identity */  \
        d0 = r.d0;                                                                                                   \
        d1 = r.d1;                                                                                                   \
    }
    MAKO_SCAN_STEP(0x111, 0xf) // row_shr:1
    MAKO_SCAN_STEP(0x112, 0xf) // row_shr:2
    MAKO_SCAN_STEP(0x114, 0xf) // row_shr:4
    MAKO_SCAN_STEP(0x118, 0xf) // row_shr:8
    MAKO_SCAN_STEP(0x142, 0xa) // row_bcast:15 into rows 1 and 3
    MAKO_SCAN_STEP(0x143, 0xc) // row_bcast:31 into rows 2 and 3
#undef MAKO_SCAN_STEP
}

__device__ __forceinline__ int exponent_of(float x)
{
    uint32_t M;
    int e;
    seqfp::split(x, M, e);
    return e;
}

// A sorted list's keys, wherever they are (LDS or device memory: loads through a generic pointer, which the
// hardware completes in no particular order, so that the code has to wait for all of them at once) ...
struct AnyKeys {
    const uint32_t* p;
    __device__ __forceinline__ uint32_t operator[](uint32_t i) const { return p[i]; }
    __device__ __forceinline__ uint4 vec(uint32_t i) const { return *reinterpret_cast<const uint4*>(p + i); }
};
// ... or known to be in device memory: plain global loads, which can be left in flight and waited for one by one.
struct GlobalKeys {
    const uint32_t* p;
    __device__ __forceinline__ uint32_t operator[](uint32_t i) const
    {
        return ((const __attribute__((address_space(1))) uint32_t*)p)[i];
    }
    __device__ __forceinline__ uint4 vec(uint32_t i) const
    {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 v = *((const __attribute__((address_space(1))) u32x4*)(p + i));
        return make_uint4(v.x, v.y, v.z, v.w);
    }
};

// The four weights a lane owns in the span of `len` (<= kGroup) entries that starts at kf[start]: entries
// 4 * lane .. 4 * lane + 3, 0.0f past the end.  kf itself is 16-byte aligned.
template <typename Keys>
__device__ __forceinline__ void load_span(Keys kf, uint32_t start, uint32_t len, float (&q)[4])
{
    const uint32_t i = lane_id() * 4u;
    uint32_t k[4] = {0u, 0u, 0u, 0u}; // bits(0.0f)
    if ((start & 3u) == 0 && i + 3 < len) {
        const uint4 x = kf.vec(start + i);
        k[0] = ~x.x;
        k[1] = ~x.y;
        k[2] = ~x.z;
        k[3] = ~x.w;
    } else if (len) {
        // (every load from a position inside the span, and what lies past the end masked with an AND: a select
        // would be turned into a branch around each load, and each would wait for the one before)
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            k[j] = ~kf[start + min(i + j, len - 1u)] & (i + j < len ? 0xffffffffu : 0u);
    }
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j)
        q[j] = __uint_as_float(k[j]);
}
__device__ __forceinline__ void load_span(const uint32_t* kf, uint32_t start, uint32_t len, float (&q)[4])
{
    load_span(AnyKeys{kf}, start, len, q);
}

// The map of one span OF A DESCENDING LIST for the epoch with exponent eg (eg == 0: no usable guess, the map is marked
// unusable).
// An entry's map depends on the parity of the state only when the entry is an exact tie (its bits below the epoch's
// last place are exactly one half), which is rare once the running value is far above the entries.  A span without
// ties is a span of constant increments, and their composition is their sum (saturated like compose32()): one wave
// reduction of one number instead of a six-step scan of two.  The largest single step is the first entry's (a weight's
// step never grows as the weight falls): no reduction at all.
// (UNORDERED: the span's entries come in any order, as those of a list in token order do: the composition is the same,
// in the order given, but the largest single step has to be looked for.)
template <bool UNORDERED = false>
__device__ __forceinline__ seqfp::Step32 span_map(const float (&q)[4], uint32_t len, int eg)
{
    using namespace seqfp;
    Step32 st = Step32{kSat, kSat, kSat};
    if (eg > 0) { // uniform per wave
        Step32 e[4];
        bool tie = false;
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            // (the step from the adder itself, half the instructions of the integer form; it marks a weight of 2^23 units
            // or more unusable, which a map that holds one is anyway)
            e[j] = lane_id() * 4u + j < len ? step32_fp(q[j], eg) : identity32();
            tie |= e[j].d0 != e[j].d1;
        }
        uint32_t cmax;
        if constexpr (UNORDERED)
            cmax = __ockl_wfred_max_u32(max(max(e[0].cmax, e[1].cmax), max(e[2].cmax, e[3].cmax)));
        else
            cmax = (uint32_t)__builtin_amdgcn_readfirstlane((int)e[0].cmax);
        if (__ballot(tie) == 0ull) {
            // (a lane's four increments: below 2^26, or marked unusable; clamped so that 64 of them cannot wrap)
            const uint32_t mine = min(e[0].d0 + e[1].d0 + e[2].d0 + e[3].d0, 1u << 25);
            // (a total of 2^24 or more can never be applied, whatever its value: marked like an unusable map)
            const uint32_t all = __ockl_wfred_add_u32(mine);
            st.d0 = st.d1 = all < (1u << 24) ? all : kSat;
            st.cmax = cmax;
            return st;
        }
        st = identity32();
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            st = compose32(st, e[j]);
        wave_scan_maps(st.d0, st.d1);
        st.d0 = (uint32_t)__builtin_amdgcn_readlane((int)st.d0, kWave - 1);
        st.d1 = (uint32_t)__builtin_amdgcn_readlane((int)st.d1, kWave - 1);
        st.cmax = cmax;
    }
    return st;
}

// Sums and maxima inside the rows of sixteen lanes (a group's quarters), on the VALU data path: lane 15 of each row
// ends up with its row's result (inclusive scans: row_shr 1, 2, 4, 8; lanes without a source lane add 0).
__device__ __forceinline__ double row_scan_add_f64(double v)
{
#define MAKO_ROW_ADD(CTRL)                                                                                           \
    {                                                                                                                \
        const unsigned long long b = (unsigned long long)__double_as_longlong(v);                                    \
        const unsigned long long t = ((unsigned long long)dpp_or_zero<CTRL, 0xf>((uint32_t)(b >> 32)) << 32) |       \
                                     (unsigned long long)dpp_or_zero<CTRL, 0xf>((uint32_t)b);                        \
        v += __longlong_as_double((long long)t);                                                                     \
    }
    MAKO_ROW_ADD(0x111)
    MAKO_ROW_ADD(0x112)
    MAKO_ROW_ADD(0x114)
    MAKO_ROW_ADD(0x118)
#undef MAKO_ROW_ADD
    return v;
}
__device__ __forceinline__ uint32_t row_scan_max_u32(uint32_t v)
{
    v = max(v, dpp_or_zero<0x111, 0xf>(v));
    v = max(v, dpp_or_zero<0x112, 0xf>(v));
    v = max(v, dpp_or_zero<0x114, 0xf>(v));
    v = max(v, dpp_or_zero<0x118, 0xf>(v));
    return v;
}
// The estimate of the sum in front of each quarter of a group (quarter k = the 16 lanes of row k, four entries per lane):
// every lane receives its own quarter's.
__device__ __forceinline__ double sum_before_quarter(const float (&q)[4])
{
    const double rs = row_scan_add_f64((((double)q[0] + (double)q[1]) + (double)q[2]) + (double)q[3]);
    const double s0 = readlane_f64(rs, 15), s1 = readlane_f64(rs, 31), s2 = readlane_f64(rs, 47);
    const uint32_t quarter = lane_id() >> 4;
    return quarter == 0 ? 0.0 : (quarter == 1 ? s0 : (quarter == 2 ? s0 + s1 : (s0 + s1) + s2));
}

// A group inside which the running sum is expected to change binade cannot be applied as one map.  Its four
// quarters (64 entries = the 16 lanes of one DPP row each) get maps of their own, each for the binade guessed from
// the fp64 sum up to ITS first entry: the chain then replays only the quarter in which the change happens.
// `at_start` is the estimate of the sum at the group's first entry.  One wave; the four records (d0, d1, cmax,
// exponent) go to out[0..3].  (No trip through LDS: the waves that meet such a group are the ones everybody waits for.)
__device__ void build_quarters(const float (&q)[4], uint32_t len, double at_start, uint4* out)
{
    using namespace seqfp;
    const uint32_t lane = lane_id(), quarter = lane >> 4;
    const double guess = at_start + sum_before_quarter(q);
    const int eg = guess > 0 ? exponent_of((float)guess) : 0;
    Step32 v = Step32{kSat, kSat, kSat};
    if (eg > 0) {
        v = identity32();
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            if (lane * 4u + j < len)
                v = compose32(v, step32_flat(q[j], eg));
    }
    const uint32_t cm = row_scan_max_u32(v.cmax);
    // inclusive scan inside the row of 16 lanes
#define MAKO_ROW_STEP(CTRL)                                                                                          \
    {                                                                                                                \
        const Step32 t = Step32{dpp_or_zero<CTRL, 0xf>(v.d0), dpp_or_zero<CTRL, 0xf>(v.d1), 0u};                     \
        const Step32 r = compose32(t, Step32{v.d0, v.d1, 0u});                                                       \
        v.d0 = r.d0;                                                                                                 \
        v.d1 = r.d1;                                                                                                 \
    }
    MAKO_ROW_STEP(0x111)
    MAKO_ROW_STEP(0x112)
    MAKO_ROW_STEP(0x114)
    MAKO_ROW_STEP(0x118)
#undef MAKO_ROW_STEP
    if ((lane & 15u) == 15u)
        out[quarter] = make_uint4(v.d0, v.d1, cm, (uint32_t)eg);
}

// The same for the walk: a group inside which r is expected to change binade gets a record per quarter, each for
// the binade guessed from r at the group's first entry minus the fp64 sum up to ITS first entry: (d0, d1, need,
// exponent), `need` being the bound of group_sub_ok as one number (the state after the quarter must be at least the
// quarter's first, largest weight, and inside the binade with room for one more decrement).  One wave.
template <bool UNORDERED = false>
__device__ void build_walk_quarters(const float (&q)[4], uint32_t len, double r_start, uint4* out)
{
    using namespace seqfp;
    const uint32_t lane = lane_id(), quarter = lane >> 4;
    const double guess = r_start - sum_before_quarter(q);
    const int eg = guess > 0 ? exponent_of((float)guess) : 0;
    Step32 v = Step32{kSat, kSat, kSat};
    if (eg > 0) {
        v = identity32();
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            if (lane * 4u + j < len)
                v = compose32(v, step32_flat(q[j], eg));
    }
    const uint32_t cm = row_scan_max_u32(v.cmax);
#define MAKO_ROW_STEP(CTRL)                                                                                          \
    {                                                                                                                \
        const Step32 t = Step32{dpp_or_zero<CTRL, 0xf>(v.d0), dpp_or_zero<CTRL, 0xf>(v.d1), 0u};                     \
        const Step32 r = compose32(t, Step32{v.d0, v.d1, 0u});                                                       \
        v.d0 = r.d0;                                                                                                 \
        v.d1 = r.d1;                                                                                                 \
    }
    MAKO_ROW_STEP(0x111)
    MAKO_ROW_STEP(0x112)
    MAKO_ROW_STEP(0x114)
    MAKO_ROW_STEP(0x118)
#undef MAKO_ROW_STEP
    // the quarter's first, largest weight (lane 16 * quarter's first entry), wanted by the row's last lane
    const uint32_t qb = __float_as_uint(q[0]);
    const uint32_t f0 = (uint32_t)__builtin_amdgcn_readlane((int)qb, 0), f1 = (uint32_t)__builtin_amdgcn_readlane((int)qb, 16);
    const uint32_t f2 = (uint32_t)__builtin_amdgcn_readlane((int)qb, 32), f3 = (uint32_t)__builtin_amdgcn_readlane((int)qb, 48);
    float q_first = __uint_as_float(quarter == 0 ? f0 : (quarter == 1 ? f1 : (quarter == 2 ? f2 : f3)));
    if constexpr (UNORDERED) // (the quarter's largest weight, wherever it is: positive floats order like their bits)
        q_first = __uint_as_float(row_scan_max_u32(max(max(__float_as_uint(q[0]), __float_as_uint(q[1])), max(__float_as_uint(q[2]), __float_as_uint(q[3])))));
    uint32_t Mq;
    int eq;
    split(q_first, Mq, eq);
    const int dl = eg - eq;
    uint32_t need = 1u;
    if (dl < 0)
        need = 1u << 31;
    else if (dl <= 25)
        need = max(1u, (uint32_t)(((unsigned long long)Mq + (1ull << dl) - 1ull) >> dl));
    if (eg > 1)
        need = max(need, min(cm, 1u << 30) + (1u << 23) + 1u);
    if (eg <= 0)
        need = 1u << 31; // (no usable guess: the quarter is replayed)
    if ((lane & 15u) == 15u)
        out[quarter] = make_uint4(v.d0, v.d1, need, (uint32_t)eg);
}

// group_sub_ok() as one bound, for a span of a descending list whose first (largest) weight is q_first and whose map
// for the epoch with exponent eg has the largest single step cmax: the state after the span must be at least the
// bound, which keeps it inside the binade with room for one more decrement and at or above that weight, so that
// nothing in the span stopped the walk.
__device__ __forceinline__ uint32_t walk_need(float q_first, int eg, uint32_t cmax)
{
    uint32_t Mq;
    int eq;
    seqfp::split(q_first, Mq, eq);
    const int dl = eg - eq;
    uint32_t need = 1u;
    if (dl < 0)
        need = 1u << 31;
    else if (dl <= 25)
        need = max(1u, (uint32_t)(((unsigned long long)Mq + (1ull << dl) - 1ull) >> dl));
    if (eg > 1)
        need = max(need, min(cmax, 1u << 30) + (1u << 23) + 1u);
    return need;
}

// Group maps of groups [g_begin, groups) for epochs guessed from pg: of the running sum (walk == false, into G.d0 /
// d1 / cmax / pack) or of the walk (into G.w_d0 / w_d1 / w_need / w_pack; r0 - pg[g] is the estimate of r at group
// g).  The calling wave is number `part` of `parts` that share the work.
// (UNSORTED: the list may hold records of unsorted shares, see unsorted_shares.h)
// (UNORDERED: a list in any order; see span_map)
// (LEAVE: G.misc()[5] may name a group that is to be left alone)
template <bool UNSORTED = false, bool UNORDERED = false, bool LEAVE = false, typename Keys>
__device__ void build_group_maps(Keys kf, uint32_t groups, bool walk, double r0, const GroupLds G,
                                 uint32_t part = wave_id(), uint32_t parts = kWaves, uint32_t g_begin = 0,
                                 const QuarterSlots qs = QuarterSlots{})
{
    using namespace seqfp;
    uint32_t* const o_d0 = walk ? G.w_d0() : G.d0();
    uint32_t* const o_d1 = walk ? G.w_d1() : G.d1();
    uint32_t* const o_c = walk ? G.w_need() : G.cmax();
    uint32_t* const o_pack = walk ? G.w_pack() : G.pack();
    // Up to four groups per trip and wave, their loads issued together; a wave's groups lie `parts` apart, so that a
    // short list is spread over all the waves (a map costs a wave about a microsecond).
    for (uint32_t g0 = g_begin + part; g0 < groups; g0 += parts * 4u) {
        float q[4][4];
        uint32_t len[4];
        double guess[4];
        int eg[4];
        bool crossing[4], keep[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint32_t g = min(g0 + u * parts, groups - 1u);
            guess[u] = walk ? r0 - G.pg()[g] : G.pg()[g];
            eg[u] = guess[u] > 0 ? exponent_of((float)guess[u]) : 0;
            // a group in which the running sum (or r) is expected to change binade, or which starts from zero, gets
            // quarter records
            const double at_end = walk ? r0 - G.pg()[g + 1] : G.pg()[g + 1];
            const int e_end = at_end > 0 ? exponent_of((float)at_end) : 0;
            crossing[u] = uniform_u32((uint32_t)(e_end != eg[u])) != 0 || (!walk && g == 0);
            // (a walk's map that a worker of sort_kernel has left for this very epoch is the map built here: kept)
            // (and so is the record of a share that was left unsorted, whatever it is for: there is nothing to build from)
            if constexpr (UNSORTED)
                keep[u] = walk && ((!crossing[u] && eg[u] > 0 && (uniform_u32(o_pack[g] >> 16) & 0xffu) == (uint32_t)eg[u]) ||
                                   (uniform_u32(o_pack[g]) & kOpaque) != 0u);
            else
                keep[u] = walk && !crossing[u] && eg[u] > 0 && uniform_u32(o_pack[g] >> 16) == (uint32_t)eg[u];
            if constexpr (LEAVE) // (the group of a rejected draft during its redraw: it has no map, see sorted_tail)
                keep[u] = keep[u] || g == uniform_u32(G.misc()[5]);
            len[u] = uniform_u32(G.pack()[g] & kLenMask);
            load_span(kf, uniform_u32(G.start()[g]), keep[u] ? 0u : len[u], q[u]);
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint32_t g = g0 + u * parts;
            if (g >= groups) // uniform
                break;
            MAKO_COUNT(walk ? 23 : 24, 1);
            if (keep[u]) // uniform
                continue;
            MAKO_COUNT(walk ? 27 : 28, 1);
            const Step32 st = span_map<UNORDERED>(q[u], len[u], eg[u]);
            uint32_t slot = 0;
            if (crossing[u]) {
                if (lane_id() == 0)
                    slot = atomicAdd(&G.misc()[(UNSORTED || UNORDERED) ? qs.counter : 3u], 1u) + 1u;
                slot = uniform_u32(slot);
                if constexpr (UNSORTED || UNORDERED) // (the instances whose walk builds its maps a block ahead)
                    slot = slot > qs.slots ? kQuarterSlots + 1u : slot + qs.first;
                if (slot > kQuarterSlots)
                    slot = 0;
                else if (walk)
                    build_walk_quarters<UNORDERED>(q[u], len[u], guess[u], G.quarters() + (slot - 1u) * 4u);
                else
                    build_quarters(q[u], len[u], G.pg()[g], G.quarters() + (slot - 1u) * 4u);
            }
            float q_top = q[u][0]; // (lane 0 holds the group's first, largest weight)
            if constexpr (UNORDERED)
                q_top = __uint_as_float(__ockl_wfred_max_u32(max(max(__float_as_uint(q[u][0]), __float_as_uint(q[u][1])),
                                                                 max(__float_as_uint(q[u][2]), __float_as_uint(q[u][3])))));
            if (lane_id() == 0) {
                o_d0[g] = st.d0;
                o_d1[g] = st.d1;
                o_c[g] = walk ? walk_need(q_top, eg[u], st.cmax) : st.cmax;
                o_pack[g] = len[u] | (slot << 9) | ((uint32_t)eg[u] << 16);
            }
        }
    }
}

// The entries of one span (at most 256), one per lane and register: x[j] of lane l is entry 64 * j + l, 0.0f past
// the end.
template <typename Keys>
__device__ __forceinline__ void load_span_lanes(Keys kf, uint32_t start, uint32_t len, float (&x)[4])
{
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        const uint32_t i = j * kWave + lane_id();
        // (every lane loads, from inside the span; masked with an AND, as in load_span)
        x[j] = __uint_as_float(~kf[start + min(i, len - 1u)] & (i < len ? 0xffffffffu : 0u));
    }
}
// The same in two steps, for loads that are to stay in flight while other work goes on: the words as loaded
// (nothing touches them here), and their conversion once they are wanted.
template <typename Keys>
__device__ __forceinline__ void fetch_span_lanes(Keys kf, uint32_t start, uint32_t len, uint32_t (&raw)[4])
{
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j)
        raw[j] = kf[start + min(j * kWave + lane_id(), len - 1u)];
}
__device__ __forceinline__ void take_span_lanes(const uint32_t (&raw)[4], uint32_t len, float (&x)[4])
{
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j)
        x[j] = __uint_as_float(~raw[j] & (j * kWave + lane_id() < len ? 0xffffffffu : 0u));
}

// One step of a chain that travels across the lanes: every lane takes the value of the lane below it (lane 0:
// of lane 63) and subtracts / adds its own entry.  Started from a uniform value, lane t holds after t + 1 steps
// the value a sequential loop would hold after entries 0..t; the other lanes hold values nobody reads.  One
// dependent instruction per entry, where a broadcast per entry costs three.
__device__ __forceinline__ float ror_sub(float v, float x)
{
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), 0x13C /* wave_ror:1 */,
                                                                 0xf, 0xf, false)) - x;
}
__device__ __forceinline__ float ror_add(float v, float x)
{
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), 0x13C /* wave_ror:1 */,
                                                                 0xf, 0xf, false)) + x;
}

// S plus the entries of one span (len in 1..256), added one by one in fp32 (src/gen/sampler.cpp:80-82).  One wave.
template <typename Keys>
__device__ float exact_span_sum(Keys kf, uint32_t start, uint32_t len, float S)
{
    float x[4];
    const uint32_t n = uniform_u32(len);
    if (n == 0)
        return S;
    load_span_lanes(kf, uniform_u32(start), n, x);
    float v = S; // uniform
    for (uint32_t base = 0; base < n; base += kWave) {
        const float cur = x[0];
        for (uint32_t b = 0; b < kWave && base + b < n; b += 16u) {
#pragma unroll
            for (uint32_t k = 0; k < 16; ++k)
                v = ror_add(v, cur);
        }
        x[0] = x[1];
        x[1] = x[2];
        x[2] = x[3];
    }
    // entries past the end added 0.0f: the lane of the last step holds the sum
    const uint32_t steps = (n + 15u) & ~15u;
    return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), (steps - 1u) & 63u));
}

// The entries of one span (n in 1..256, in registers as load_span_lanes() leaves them; the span starts at entry
// `beg` of the list) subtracted from r one by one (src/gen/sampler.cpp:67-71).  Returns true and the entry's
// position in the list when the walk stops inside the span, else false and the new r.  One wave.
//
// The walk stops at the first entry with r < x, which is the first entry whose subtraction turns r negative (x != r
// gives a nonzero difference, denormals kept), and a negative r stays negative under every later subtraction of a
// weight.  So 64 entries are subtracted without looking; only a block that ends negative is gone through again,
// sixteen entries at a time, and the sixteen that turn r negative one by one.
__device__ __forceinline__ bool walk_lanes(float (&x)[4], uint32_t n, uint32_t beg, float& r, uint32_t& pos)
{
    float v = r;    // uniform
    float r_in = r; // the walk's value in front of the current block
    for (uint32_t base = 0; base < n; base += kWave) {
        const float cur = x[0];
        const bool whole = n - base > 48u; // (a short rest goes sixteen at a time straight away)
        uint32_t out = 0x80000000u;
        if (whole) {
#pragma unroll
            for (uint32_t k = 0; k < kWave; ++k)
                v = ror_sub(v, cur);
            out = (uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), kWave - 1);
        }
        if (out >> 31) {
            v = r_in;
            for (uint32_t b = 0; b < kWave && base + b < n; b += 16u) {
#pragma unroll
                for (uint32_t k = 0; k < 16; ++k)
                    v = ror_sub(v, cur);
                const uint32_t o16 = (uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), (b + 15u) & 63u);
                if (o16 >> 31) {
                    float rr = r_in;
                    for (uint32_t l = b; l < b + 16u; ++l) {
                        const float xv =
                            __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(cur), l & 63u));
                        if (__ballot(rr < xv) != 0ull) {
                            pos = beg + base + l;
                            return true;
                        }
                        rr -= xv;
                    }
                }
                r_in = __uint_as_float(o16);
            }
        }
        if (whole)
            r_in = __uint_as_float(out);
        x[0] = x[1];
        x[1] = x[2];
        x[2] = x[3];
    }
    r = r_in;
    return false;
}

template <typename Keys>
__device__ bool exact_span_walk(Keys kf, uint32_t start, uint32_t len, float& r, uint32_t& pos)
{
    float x[4];
    const uint32_t n = uniform_u32(len);
    const uint32_t beg = uniform_u32(start);
    if (n == 0)
        return false;
    load_span_lanes(kf, beg, n, x);
    return walk_lanes(x, n, beg, r, pos);
}

// The walk over the first `n` entries of the list, staged in LDS as floats (16-byte aligned): every lane of the
// wave reads the same four entries with one broadcast load and subtracts them in turn, two nanoseconds an entry
// (the travelling chain of walk_lanes() takes five).  Blocks of 64 blind, then of 16, then entry by entry, as there.
// Returns true and the position when the walk stops, else false and the new r.
// (The list is read as LDS, not through the generic pointer: generic loads wait for one another in full, and the
// first subtraction of a block would wait for the block's last entry.)
typedef __attribute__((address_space(3))) const float LdsFloat;
typedef float LdsFloat4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bool walk_lds(const float* sx_any, uint32_t n, float& r, uint32_t& pos)
{
    LdsFloat* sx = (LdsFloat*)sx_any;
    typedef const __attribute__((address_space(3))) LdsFloat4* Vec4Ptr;
    float v = r;
    uint32_t base = 0;
    // Blocks of 64 in two halves, each half's loads issued while the other half is subtracted (the scheduling
    // barriers keep the loads where they are written: the compiler would otherwise issue each only just before its
    // use, to save registers, and every fourth subtraction would wait for LDS).  The loads run up to 32 entries past
    // the block; the staged list has a wave's worth of room behind it.
    LdsFloat4 xa[8], xb[8];
    if (kWave <= n) {
#pragma unroll
        for (uint32_t i = 0; i < 8u; ++i)
            xa[i] = ((Vec4Ptr)sx)[i];
    }
    for (; base + kWave <= n; base += kWave) {
        Vec4Ptr p = (Vec4Ptr)(sx + base);
#pragma unroll
        for (uint32_t i = 0; i < 8u; ++i)
            xb[i] = p[8u + i];
        __builtin_amdgcn_sched_barrier(0);
        float t = v;
#pragma unroll
        for (uint32_t i = 0; i < 8u; ++i) {
            t -= xa[i].x;
            t -= xa[i].y;
            t -= xa[i].z;
            t -= xa[i].w;
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (uint32_t i = 0; i < 8u; ++i)
            xa[i] = p[16u + i];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (uint32_t i = 0; i < 8u; ++i) {
            t -= xb[i].x;
            t -= xb[i].y;
            t -= xb[i].z;
            t -= xb[i].w;
        }
        __builtin_amdgcn_sched_barrier(0);
        if (__ballot(t < 0.0f) != 0ull)
            break; // the walk stops in this block: found below
        v = t;
    }
    for (; base + 16u <= n; base += 16u) {
        const __attribute__((address_space(3))) LdsFloat4* p = (const __attribute__((address_space(3))) LdsFloat4*)(sx + base);
        float t = v;
#pragma unroll
        for (uint32_t i = 0; i < 4u; ++i) {
            const LdsFloat4 x = p[i];
            t -= x.x;
            t -= x.y;
            t -= x.z;
            t -= x.w;
        }
        if (__ballot(t < 0.0f) != 0ull)
            break;
        v = t;
    }
    for (const uint32_t end = min(n, base + 16u); base < end; ++base) {
        const float x = sx[base];
        if (__ballot(v < x) != 0ull) {
            pos = base;
            return true;
        }
        v -= x;
    }
    r = v;
    return false;
}

// S plus the first `n` entries of a list staged in LDS as for walk_lds(), added one by one in fp32.
__device__ __forceinline__ float sum_lds(const float* sx_any, uint32_t n, float S)
{
    LdsFloat* sx = (LdsFloat*)sx_any;
    typedef const __attribute__((address_space(3))) LdsFloat4* Vec4Ptr;
    uint32_t base = 0;
    // (blocks of 64 in two halves, loads and additions interleaved as in walk_lds())
    LdsFloat4 xa[8], xb[8];
    if (kWave <= n) {
#pragma unroll
        for (uint32_t i = 0; i < 8u; ++i)
            xa[i] = ((Vec4Ptr)sx)[i];
    }
    for (; base + kWave <= n; base += kWave) {
        Vec4Ptr p = (Vec4Ptr)(sx + base);
#pragma unroll
        for (uint32_t i = 0; i < 8u; ++i)
            xb[i] = p[8u + i];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (uint32_t i = 0; i < 8u; ++i) {
            S += xa[i].x;
            S += xa[i].y;
            S += xa[i].z;
            S += xa[i].w;
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (uint32_t i = 0; i < 8u; ++i)
            xa[i] = p[16u + i];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (uint32_t i = 0; i < 8u; ++i) {
            S += xb[i].x;
            S += xb[i].y;
            S += xb[i].z;
            S += xb[i].w;
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    for (; base + 16u <= n; base += 16u) {
        Vec4Ptr p = (Vec4Ptr)(sx + base);
#pragma unroll
        for (uint32_t i = 0; i < 4u; ++i) {
            const LdsFloat4 x = p[i];
            S += x.x;
            S += x.y;
            S += x.z;
            S += x.w;
        }
    }
    for (; base < n; ++base)
        S += sx[base];
    return S;
}

// State of a chain between groups: significand and exponent of the running value, and where the walk stopped.
struct ChainState {
    uint32_t M;
    int e;
    uint32_t pos; // kNone while the walk goes on
};

// One group applied to the running sum quarter by quarter (records at `rec`), replaying only the quarters whose
// map does not apply.  One wave.  (State by value: the chain keeps it in scalar registers.)
template <typename Keys>
__device__ __forceinline__ ChainState sum_by_quarters(Keys kf, uint32_t st, uint32_t len, const uint4* rec, ChainState c)
{
    using namespace seqfp;
#pragma unroll 1
    for (uint32_t k = 0; k < 4u; ++k) {
        if (k * kQuarter < len) { // uniform
            const uint4 r = rec[k];
            const uint32_t d0 = uniform_u32(r.x), d1 = uniform_u32(r.y), cm = uniform_u32(r.z), eg = uniform_u32(r.w);
            const uint32_t dd = (c.M & 1u) ? d1 : d0;
            const uint32_t lim = cm >= (1u << 24) - 1u ? 0u : (1u << 24) - 1u - cm;
            if ((uint32_t)c.e == eg && c.M + dd < lim) {
                c.M += dd;
            } else {
                const float S = exact_span_sum(kf, st + k * kQuarter, min(kQuarter, len - k * kQuarter), join(c.M, c.e));
                uint32_t Mv;
                int ev;
                split(S, Mv, ev);
                c.M = uniform_u32(Mv);
                c.e = (int)uniform_u32((uint32_t)ev);
            }
        }
    }
    return c;
}

// One block of at most 64 entries (x of lane l = entry l of the block, 0.0f past its end; the block starts at entry
// `beg` of the list) subtracted from r one by one.  Returns true and the position when the walk stops inside the
// block, else false and the new r.  One wave.  (walk_lanes() for a single block.)
__device__ __forceinline__ bool walk_block(float cur, uint32_t n, uint32_t beg, float& r, uint32_t& pos)
{
    float v = r;
    float r_in = r;
    for (uint32_t b = 0; b < kWave && b < n; b += 16u) {
#pragma unroll
        for (uint32_t k = 0; k < 16; ++k)
            v = ror_sub(v, cur);
        const uint32_t o16 = (uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), (b + 15u) & 63u);
        if (o16 >> 31) {
            float rr = r_in;
            for (uint32_t l = b; l < b + 16u; ++l) {
                const float xv = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(cur), l & 63u));
                if (__ballot(rr < xv) != 0ull) {
                    pos = beg + l;
                    return true;
                }
                rr -= xv;
            }
        }
        r_in = __uint_as_float(o16);
    }
    r = r_in;
    return false;
}

// One group of the walk quarter by quarter (records at `rec`, see build_walk_quarters(); the group's entries in x as
// load_span_lanes() leaves them: x[k] of lane l is entry l of quarter k), replaying only the quarters whose map
// does not apply.  Returns true (and c.pos) when the walk stops inside the group.  One wave.
__device__ __forceinline__ bool walk_by_quarters(const float (&x)[4], uint32_t st, uint32_t len, const uint4* rec, ChainState& c)
{
    using namespace seqfp;
#pragma unroll
    for (uint32_t k = 0; k < 4u; ++k) {
        if (k * kQuarter < len) { // uniform
            const uint4 r = rec[k];
            const uint32_t d0 = uniform_u32(r.x), d1 = uniform_u32(r.y), need = uniform_u32(r.z), eg = uniform_u32(r.w);
            const uint32_t dd = (c.M & 1u) ? d1 : d0;
            if ((uint32_t)c.e == eg && dd <= c.M && c.M - dd >= need) {
                c.M -= dd;
            } else {
                float rr = join(c.M, c.e);
                uint32_t at = 0;
                if (walk_block(x[k], min(kQuarter, len - k * kQuarter), st + k * kQuarter, rr, at)) {
                    c.pos = at;
                    return true;
                }
                uint32_t Mv;
                int ev;
                split(rr, Mv, ev);
                c.M = uniform_u32(Mv);
                c.e = (int)uniform_u32((uint32_t)ev);
            }
        }
    }
    return false;
}

// The band for a top-p cut in a sorted list of n weights q_at(0 .. n).  When total64 is the sum of
// exactly these weights and the lightest one's last bit still lies within 53 bits of the total's first, no fp64
// addition of any of these sums can round, whatever the order: all of them are exact, the reference's too, and the
// comparison with `want` is the reference's (band 0).
template <typename Get>
__device__ __forceinline__ double cut_band(bool have_total, uint32_t n_vocab, uint32_t n, Get q_at, double total64)
{
    if (have_total)
        return order_band(n_vocab, total64);
    return total64 <= (double)q_at(n - 1u) * 0x1p29 ? 0.0 : order_band(n, total64);
}

// q_at(0) + q_at(1) + ... as the reference's loop adds them: one wave, one fp64 addition after the other, 256
// entries per round (lane l brings entries 4l .. 4l+3, handed round lane by lane).  Stops after the round in which
// the sum reaches `want` and returns in n_added how many entries the reference's `while (n < k && sum < want)` adds
// (n, if the sum stays below `want`; pass +inf for a plain total).  Every lane returns the sum.  One wave calls it.
template <typename Get>
__device__ MAKO_RARE_CALL double wave_sequential_sum(Get q_at, uint32_t n, double want, uint32_t& n_added)
{
    double cum = 0.0;
    n_added = n;
    for (uint32_t base = 0; base < n; base += 4u * kWave) {
        float q[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const uint32_t i = base + lane_id() * 4u + j;
            q[j] = i < n ? q_at(i) : 0.0f;
        }
        const double before = cum;
        for (uint32_t l = 0; l < kWave; ++l) {
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                cum += (double)__uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(q[j]), l));
        }
        if (cum >= want) { // (uniform) the reference stopped inside this round: again, entry by entry
            cum = before;
            uint32_t k = 0;
            for (; k < 4u * kWave && base + k < n && cum < want; ++k)
                cum += (double)__uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(q[k & 3u]), k >> 2));
            n_added = base + k;
            break;
        }
    }
    return cum;
}

// The reference's `total` (src/gen/sampler.cpp:46-48) over n weights in the order q_at gives them.  All threads call,
// all get it.
template <typename Get>
__device__ MAKO_RARE_CALL double reference_total(Get q_at, uint32_t n, FinishShared& sm)
{
    __syncthreads();
    if (wave_id() == 0) {
        uint32_t added;
        const double t = wave_sequential_sum(q_at, n, (double)INFINITY, added);
        if (lane_id() == 0)
            sm.bs.f64[0] = t;
    }
    __syncthreads();
    const double t = sm.bs.f64[0];
    __syncthreads();
    return t;
}

// Tail of every path that ends with a list sorted by (q desc, idx asc): kf[i] = ~bits(q_i), jf[i] = token id,
// n1 entries (already cut to top_k).  Applies top-p (src/gen/sampler.cpp:44-61) against total64 (the fp64 sum over
// the row's candidates; summed from the list when !have_total), then the exact fp32 total (:80-82) and walk
// (:64-73).  All 1024 threads must call it.
//
// When `need_cut` the list is only the heaviest part of the row's candidates and every candidate missing from
// it weighs at most q_bound: the nucleus must then end inside the list, at an entry strictly heavier than
// q_bound.  If it does not, nothing is written and false is returned (the caller widens the list).
//
// A cut that the sums here cannot tell from its neighbour with certainty (see order_band) is not made: nothing is
// written and false is returned.  The caller then either widens (need_cut) or calls the EXACT instance with, as
// total64, the reference's own total (reference_total() over the candidates in the reference's order): the cut is
// then made by the reference's running sum, entry by entry.  EXACT on a whole list always succeeds.  (An instance of
// its own, so that the usual one carries none of its code: sorted_tail_exact().)
//
// `T` (with `t_groups` records at `t_base`) describes a list whose groups were prepared by sort_kernel's workers;
// without it the list is cut into groups of kGroup here.
// SHORT_ONLY: the caller's lists never exceed kGroup entries; the code for longer ones is left out.
// UNSORTED (with PLANNED): some of the workers' shares may have been left unsorted, as one record each
// (unsorted_shares.h); a row whose records of that kind cannot all be applied is given up (false).
// UNORDERED (with PLANNED, without a top-p): the list is in token order, not sorted (a row that is neither cut to a
// top-k nor to a nucleus: src/gen/sampler.cpp:79-83 and :64-72 over the candidates as they come); nothing here needs
// the order except the bounds that stand for "the largest weight of a span", which are then looked for.
// VERIFY (with UNORDERED): the instance for verification (d.draft given); the plain one is then never asked to verify.
template <bool PLANNED = false, bool SHORT_ONLY = false, bool EXACT = false, bool UNSORTED = false, bool UNORDERED = false, bool VERIFY = false>
__device__ bool sorted_tail(const mako_sample_desc& d, uint32_t row, const mako_sampling_params& P, const uint32_t* kf_ptr,
                            const uint32_t* jf, uint32_t n1_arg, bool have_total, double total64, uint32_t path,
                            const FinishLds& L, bool need_cut = false, float q_bound = 0.0f, const GroupTable& T = GroupTable{},
                            size_t t_base = 0, uint32_t t_groups = 0)
{
    assume_lds(L);
    constexpr bool exact = EXACT;
    using namespace seqfp;
    // (a planned row's list is in device memory; the other callers may hand over a list in LDS)
    const typename std::conditional<PLANNED, GlobalKeys, AnyKeys>::type kf{kf_ptr};
    const float u_row = d.u[row]; // (asked for here, wanted much later)
    const uint32_t n1 = uniform_u32(n1_arg);
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
    auto qat = [=](uint32_t i) { return __uint_as_float(~kf[i]); };
    // (UNORDERED: a list in token order, whose entry i is token i: jf is not read)
    auto idat = [=](uint32_t i) {
        if constexpr (UNORDERED)
            return i;
        else
            return jf[i];
    };
    const GroupLds G = group_lds(L);
    const bool topp_active = P.top_p < 1.0f;
    constexpr uint32_t kEpochBits = UNSORTED ? 0xffu : ~0u; // (of a pack's upper half)
    // (UNORDERED: verification takes the running sum's chain below and, only if the draft is rejected, the generic walk)
    if ((d.draft && !UNORDERED) || (!PLANNED && n1 > kGroup * kMaxGroups)) {
        // verification and oversized lists take the generic windowed replay
        uint32_t n = n1;
        if (topp_active) {
            if (!have_total) {
                double part = 0;
                for (uint32_t i = tid; i < n; i += kThreads)
                    part += (double)qat(i);
                total64 = block_sum_f64(part, sm.bs);
            }
            const double want = (double)P.top_p * total64;
            uint32_t keep = kNone;
            if (exact) {
                if (wave_id() == 0) {
                    uint32_t added;
                    const double cum = wave_sequential_sum(qat, n, want, added);
                    if (lane_id() == 0)
                        sm.aux = cum >= want ? added : kNone;
                }
                __syncthreads();
                keep = sm.aux;
            } else {
                const double band = cut_band(have_total, d.n_vocab, n, qat, total64);
                double carry = 0;
                if (tid == 0)
                    sm.aux = 0; // set: the cut is too close to `want` to call
                for (uint32_t base = 0; base < n; base += kThreads) {
                    const uint32_t i = base + tid;
                    const double q = i < n ? (double)qat(i) : 0.0;
                    double tile;
                    const double incl = carry + block_incl_scan_f64(q, tile, sm.bs);
                    const uint32_t hit = (i < n && incl >= want) ? i : kNone;
                    const uint32_t first = block_min_u32(hit, sm.bs);
                    if (first != kNone) {
                        keep = first + 1;
                        if (i == first && P.top_p > 0.0f && band != 0.0 && !(incl - want > band && want - (incl - q) > band))
                            sm.aux = 1;
                        break;
                    }
                    carry += tile;
                }
                __syncthreads();
                if (sm.aux || keep == kNone) // (a list that never reaches `want`: the reference's sum might)
                    return false;
            }
            if (need_cut && keep == kNone)
                return false;
            n = keep == kNone ? n : keep;
        }
        if (need_cut && !(q_bound < qat(n - 1)))
            return false;
        draw_from_list(d, row, qat, idat, n, path, sm);
        return true;
    }

    if (!PLANNED && n1 <= kGroup) {
        // short list: one wave does everything, the chain of fp32 roundings replayed with real additions
        MAKO_STAMP(5);
        __syncthreads(); // the list is published; sm.flag is free
        if (wave_id() == 0) {
            float q[4];
            load_span(kf, 0, n1, q);
            double p[4];
            p[0] = (double)q[0];
            p[1] = p[0] + (double)q[1];
            p[2] = p[1] + (double)q[2];
            p[3] = p[2] + (double)q[3];
            const double incl = __ockl_wfscan_add_f64(p[3], true);
            if (!have_total)
                total64 = readlane_f64(incl, kWave - 1);
            uint32_t n = n1;
            bool ok = true;
            if (topp_active && exact) {
                const double want = (double)P.top_p * total64;
                uint32_t added;
                const double cum = wave_sequential_sum(qat, n1, want, added);
                if (cum >= want)
                    n = max(added, 1u); // (sampler.cpp:58: never fewer than one)
                else
                    ok = !need_cut;
            } else if (topp_active) {
                const double want = (double)P.top_p * total64;
                const double band = cut_band(have_total, d.n_vocab, n1, qat, total64);
                const double base = incl - p[3];
                uint32_t hit = kNone;
                bool clear = true; // both neighbours of the cut clear `want` by more than the band
#pragma unroll
                for (int j = 3; j >= 0; --j)
                    if (base + p[j] >= want) {
                        hit = lane_id() * 4u + (uint32_t)j;
                        clear = !(P.top_p > 0.0f) || band == 0.0 || (base + p[j] - want > band && want - (j ? base + p[j - 1] : base) > band);
                    }
                const unsigned long long bal = __ballot(hit != kNone && hit < n1);
                if (bal) {
                    const int src = __ffsll((long long)bal) - 1;
                    n = (uint32_t)__builtin_amdgcn_readlane((int)hit, src) + 1u;
                    ok = __builtin_amdgcn_readlane((int)clear, src) != 0;
                } else {
                    ok = false; // (a list that never reaches `want`: the reference's sum might)
                }
            }
            if (ok && need_cut && !(q_bound < qat(n - 1)))
                ok = false;
            if (ok) {
                const float total = exact_span_sum(kf, 0, n, 0.0f);
                const float span = total - 0.0f;
                const float prod = u_row * span;
                float r = prod + 0.0f;
                uint32_t pos = n - 1;
                if (r < 0.0f)
                    pos = 0;
                else if (r == r && r != INFINITY)
                    exact_span_walk(kf, 0, n, r, pos);
                if (d.out_cand_idx && d.out_cand_q)
                    for (uint32_t j = lane_id(); j < n && j < d.cand_cap; j += kWave) {
                        d.out_cand_idx[(size_t)row * d.cand_cap + j] = (int32_t)idat(j);
                        d.out_cand_q[(size_t)row * d.cand_cap + j] = qat(j);
                    }
                if (lane_id() == 0) {
                    RowOut o;
                    o.token = (int32_t)idat(pos);
                    o.n_cand = n;
                    o.total = total;
                    o.q = qat(pos);
                    o.path = path;
                    o.accepted = 0;
                    write_row(d, row, o);
                }
            }
            if (lane_id() == 0)
                sm.flag = ok;
        }
        __syncthreads();
        MAKO_STAMP(9);
        return sm.flag != 0;
    }
    if constexpr (SHORT_ONLY)
        return false; // (not reached)

    // group records: fp64 sums (and, from the workers, the maps of the running sum)
    MAKO_STAMP(5);
    const uint32_t groups1 = PLANNED ? t_groups : (n1 + kGroup - 1) / kGroup;
    // (UNSORTED: the running sum and the walk's first block of groups share the first half of the quarter-record slots;
    // the other half is for the maps of the walk's second block, built while the first is walked)
    constexpr bool kAhead = UNSORTED || UNORDERED; // (the instances for lists of hundreds of groups)
    constexpr uint32_t kFirstSlots = kAhead ? kQuarterSlots / 2u : kQuarterSlots;
    if (tid == 0) {
        G.misc()[3] = 0;
        if (kAhead)
            G.misc()[4] = 0;
        if (UNORDERED && VERIFY)
            G.misc()[5] = kNone; // (set: the group that is to get no map for the walk)
        if (UNSORTED) {
            sm.ticket = 0; // set: a record of an unsorted share where the code below needs the list itself
            sm.flag = 0;   // set: the list has such records
        }
    }
    // The head of the list as floats in LDS (loads set out now, wanted after the cut): where the running sum and
    // the walk change binade every few entries, both go through it entry by entry.
    constexpr uint32_t kHead = kHeadGroups * kGroup;
    float* const head = G.head();
    uint32_t raw[kHead / kThreads];
#pragma unroll
    for (uint32_t t = 0; t < kHead / kThreads; ++t)
        raw[t] = kf[min(t * kThreads + tid, n1 - 1u)];
    // (a planned list's group records are asked for in the same trip to memory: nothing below waits for the head's
    // loads before these are out)
    double r_sum = 0.0;
    uint32_t r_d0 = 0, r_d1 = 0, r_cm = 0, r_st = 0, r_pk = 0;
    uint4 qr0 = make_uint4(0, 0, 0, 0), qr1 = qr0, qr2 = qr0, qr3 = qr0, r_walk = qr0;
    if constexpr (PLANNED) {
        if (tid < groups1) {
            r_walk = T.walk[t_base + tid];
            r_sum = T.sum[t_base + tid];
            r_d0 = T.d0[t_base + tid];
            r_d1 = T.d1[t_base + tid];
            r_cm = T.cmax[t_base + tid];
            r_st = T.start[t_base + tid];
            r_pk = T.pack[t_base + tid];
            // (the quarter records are asked for together with the rest, whether or not the group has any: asking
            // only once `pk` is known would be one more trip to memory for every row)
            const uint4* tq = T.quarters + (t_base + tid) * 4u;
            qr0 = tq[0], qr1 = tq[1], qr2 = tq[2], qr3 = tq[3];
        }
        lds_barrier(); // (misc[3] is published; the loads stay in flight)
    } else {
        __syncthreads();
    }
#pragma unroll
    for (uint32_t t = 0; t < kHead / kThreads; ++t)
        head[t * kThreads + tid] = __uint_as_float(~raw[t] & (t * kThreads + tid < n1 ? 0xffffffffu : 0u));
    if (tid < kWave)
        head[kHead + tid] = 0.0f;
    if constexpr (PLANNED) {
        if (tid < groups1) {
            G.pg()[tid + 1] = r_sum;
            G.d0()[tid] = r_d0;
            G.d1()[tid] = r_d1;
            G.cmax()[tid] = r_cm;
            // (clamped into the list: a record is only ever read, never trusted for addressing)
            const uint32_t st = min(r_st, n1), pk = r_pk;
            uint32_t slot = 0;
            if (pk & kHasQuarters) {
                slot = atomicAdd(&G.misc()[3], 1u) + 1u;
                if (slot > kFirstSlots)
                    slot = 0;
            }
            if (slot) {
                uint4* gq = G.quarters() + (slot - 1u) * 4u;
                gq[0] = qr0;
                gq[1] = qr1;
                gq[2] = qr2;
                gq[3] = qr3;
            }
            G.start()[tid] = st;
            const uint32_t len = min(pk & kLenMask, min(kGroup, n1 - st));
            G.pack()[tid] = len | (slot << 9) | (pk & (0x00ff0000u | (UNSORTED ? kOpaque : 0u)));
            // (the worker's map for the walk, if it was made for the length the group has here: with its exponent;
            // the cut takes the exponent away again from the group it shortens, and the walk builds what is missing)
            G.w_d0()[tid] = r_walk.x;
            G.w_d1()[tid] = r_walk.y;
            G.w_need()[tid] = r_walk.z;
            G.w_pack()[tid] = ((pk & kLenMask) == len ? (len | ((r_walk.w & 0xffu) << 16)) : len) | (UNSORTED ? pk & kOpaque : 0u);
            // (the staged head and the candidates written out are read entry by entry: no unsorted share may lie there,
            // wherever the plan expected it to lie)
            if (UNSORTED && (pk & kOpaque)) {
                sm.flag = 1;
                if (tid < kHeadGroups || st < kHead || (d.out_cand_idx && d.out_cand_q && st < d.cand_cap))
                    sm.ticket = 1;
            }
        }
    } else {
        if (tid < groups1) {
            G.start()[tid] = tid * kGroup;
            G.pack()[tid] = min(kGroup, n1 - tid * kGroup);
            G.w_pack()[tid] = min(kGroup, n1 - tid * kGroup); // (no exponent: the walk's maps are built when it gets there)
        }
        for (uint32_t g0 = wave_id() * 4u; g0 < groups1; g0 += kWaves * 4u) {
            float q[4][4];
#pragma unroll
            for (uint32_t u = 0; u < 4; ++u) {
                const uint32_t g = min(g0 + u, groups1 - 1u);
                load_span(kf, g * kGroup, min(kGroup, n1 - g * kGroup), q[u]);
            }
#pragma unroll
            for (uint32_t u = 0; u < 4; ++u) {
                const double s = __ockl_wfred_add_f64((((double)q[u][0] + (double)q[u][1]) + (double)q[u][2]) + (double)q[u][3]);
                if (lane_id() == 0 && g0 + u < groups1)
                    G.pg()[g0 + u + 1] = s;
            }
        }
    }
    __syncthreads();
    if (UNSORTED && sm.ticket)
        return false;
    const uint32_t path_out = (UNSORTED && path == MAKO_PATH_SORTED && sm.flag) ? MAKO_PATH_SUMMED : path;
    {
        const double v = tid < groups1 ? G.pg()[tid + 1] : 0.0;
        double all;
        const double incl = block_incl_scan_f64(v, all, sm.bs);
        if (tid < groups1)
            G.pg()[tid + 1] = incl;
        if (tid == 0)
            G.pg()[0] = 0.0;
        if (!have_total)
            total64 = all;
    }
    __syncthreads();

    // top-p: first entry at which the running fp64 sum reaches top_p * total
    MAKO_STAMP(6);
    uint32_t n = n1, groups = uniform_u32(groups1);
    if (topp_active) {
        const double want = (double)P.top_p * total64;
        uint32_t hitg = (tid < groups1 && G.pg()[tid + 1] >= want) ? tid : kNone;
        if (exact) {
            // the reference's own running sum decides; the group it ends in follows from the entry
            if (wave_id() == 0) {
                uint32_t added;
                const double cum = wave_sequential_sum(qat, n1, want, added);
                if (lane_id() == 0)
                    G.misc()[0] = cum >= want ? max(added, 1u) : kNone;
            }
            __syncthreads();
            const uint32_t n_ref = G.misc()[0];
            hitg = kNone;
            if (n_ref != kNone && tid < groups1) {
                const uint32_t st = G.start()[tid], len = G.pack()[tid] & kLenMask;
                if (st < n_ref && n_ref <= st + len)
                    hitg = tid;
            }
            __syncthreads();
        }
        const uint32_t gs = block_min_u32(hitg, sm.bs);
        if (gs == kNone && (need_cut || !exact))
            return false; // (a list that never reaches `want`: a partial one is widened, a whole one decided exactly)
        if (UNSORTED && gs != kNone && (G.pack()[gs] & kOpaque))
            return false; // (the cut falls into a share that was left unsorted)
        if (gs != kNone && exact) {
            const uint32_t st = G.start()[gs], len = G.pack()[gs] & kLenMask, keep = G.misc()[0] - st;
            __syncthreads();
            if (tid == 0 && keep != len) {
                G.pack()[gs] = keep;
                G.w_pack()[gs] = keep;
            }
            __syncthreads();
            n = uniform_u32(G.misc()[0]);
            groups = uniform_u32(gs + 1u);
        } else if (gs != kNone) {
            const double band = cut_band(have_total, d.n_vocab, n1, qat, total64);
            if (wave_id() == 0) {
                const uint32_t st = G.start()[gs], len = G.pack()[gs] & kLenMask;
                float q[4];
                load_span(kf, st, len, q);
                double p[4];
                p[0] = (double)q[0];
                p[1] = p[0] + (double)q[1];
                p[2] = p[1] + (double)q[2];
                p[3] = p[2] + (double)q[3];
                const double incl = __ockl_wfscan_add_f64(p[3], true);
                const double base = G.pg()[gs] + (incl - p[3]);
                uint32_t hit = kNone;
                bool clear = true; // both neighbours of the cut clear `want` by more than the band
#pragma unroll
                for (int j = 3; j >= 0; --j)
                    if (base + p[j] >= want) {
                        hit = lane_id() * 4u + (uint32_t)j;
                        clear = !(P.top_p > 0.0f) || band == 0.0 || (base + p[j] - want > band && want - (j ? base + p[j - 1] : base) > band);
                    }
                const unsigned long long bal = __ballot(hit != kNone && hit < len);
                uint32_t keep = len;
                bool ok = false; // (no entry of the group reaches `want` although its sum does: too close to call)
                if (bal) {
                    const int src = __ffsll((long long)bal) - 1;
                    keep = (uint32_t)__builtin_amdgcn_readlane((int)hit, src) + 1u;
                    ok = __builtin_amdgcn_readlane((int)clear, src) != 0;
                }
                // (the shortened group's map for the running sum is made again from the entries at hand, for the binade
                // its old map was for: the chain then need not add its entries one by one; the walk's is not, exponent 0)
                const uint32_t eg_cut = PLANNED ? (uniform_u32(G.pack()[gs]) >> 16) & 0xffu : 0u;
                Step32 cut_map = Step32{kSat, kSat, kSat};
                if (ok && keep != len && eg_cut) // uniform
                    cut_map = span_map(q, keep, (int)eg_cut);
                if (lane_id() == 0) {
                    G.misc()[0] = ok ? st + keep : kNone;
                    if (ok && keep != len) {
                        G.pack()[gs] = keep | (eg_cut << 16);
                        G.w_pack()[gs] = keep;
                        if (eg_cut) {
                            G.d0()[gs] = cut_map.d0;
                            G.d1()[gs] = cut_map.d1;
                            G.cmax()[gs] = cut_map.cmax;
                        }
                    }
                }
            }
            __syncthreads();
            if (G.misc()[0] == kNone)
                return false;
            n = uniform_u32(G.misc()[0]);
            groups = uniform_u32(gs + 1u);
        }
    }
    if (n < 1)
        n = 1;
    // (values merged over branches the compiler cannot see as uniform: back to scalar registers)
    n = uniform_u32(n);
    groups = uniform_u32(groups);
    if (need_cut && !(q_bound < qat(n - 1)))
        return false;
    __syncthreads();

    // candidates and the row's results, once total and position are known
    auto emit = [&](float total, uint32_t pos) {
        if (d.out_cand_idx && d.out_cand_q)
            for (uint32_t j = tid; j < n && j < d.cand_cap; j += kThreads) {
                d.out_cand_idx[(size_t)row * d.cand_cap + j] = (int32_t)idat(j);
                d.out_cand_q[(size_t)row * d.cand_cap + j] = qat(j);
            }
        if (tid == 0) {
            RowOut o;
            o.token = (int32_t)idat(pos);
            o.n_cand = n;
            o.total = total;
            o.q = qat(pos);
            o.path = path_out;
            o.accepted = 0;
            write_row(d, row, o);
        }
    };

    MAKO_STAMP(7);
    if (n <= kSeqMax && !(UNORDERED && VERIFY)) {
        // A nucleus this short is copied to LDS and gone through entry by entry, once for the total and once for the
        // walk (two nanoseconds an entry each way): the group maps below only pay on longer lists.
        if (wave_id() == 0) {
            const float S = sum_lds(head, n, 0.0f);
            const float span = S - 0.0f;
            const float prod = u_row * span;
            const float r0 = prod + 0.0f;
            uint32_t at = n - 1;
            if (r0 < 0.0f) {
                at = 0;
            } else if (r0 == r0 && r0 != INFINITY) {
                float r = r0;
                walk_lds(head, n, r, at);
            }
            if (lane_id() == 0) {
                G.misc()[1] = __float_as_uint(S);
                G.misc()[2] = at;
            }
        }
        __syncthreads();
        MAKO_STAMP(9);
        emit(__uint_as_float(G.misc()[1]), G.misc()[2]);
        return true;
    }

    // exact fp32 total: group maps in parallel (here, or already by the workers), then one wave chains them
    if (!PLANNED) {
        build_group_maps(kf, groups, false, 0.0, G);
        __syncthreads();
    }
    MAKO_STAMP(13);
    // While one wave chains the running sum, the others already prepare the walk: its maps only need the binade r is
    // expected to be in at each group, and the fp64 sums give that (a wrong guess costs a replay, never the result).
    // Groups that start after the mass r0 could have is used up get no map.  (Every wave finds that group for itself,
    // 64 groups per ballot: no barrier stands between the cut and the chain.)
    const double r0_guess = (double)u_row * G.pg()[groups];
    uint32_t reach = groups;
    for (uint32_t g0 = 0; g0 < groups; g0 += kWave) {
        const uint32_t g = g0 + lane_id();
        const unsigned long long beyond = __ballot(g < groups && !(r0_guess * 1.001 - G.pg()[min(g, groups - 1u)] > 0));
        if (beyond) { // uniform
            reach = g0 + (uint32_t)__ffsll((long long)beyond) - 1u;
            break;
        }
    }
    // A walk that will end within a few groups goes through them entry by entry, from a copy in LDS: faster than
    // the groups' maps would be to build.
    bool head_walk = reach <= kHeadGroups; // uniform
    const uint32_t head_n = !head_walk ? 0u : (reach == groups ? n : uniform_u32(G.start()[reach]));
    if (UNSORTED) // (no unsorted share lies in front of an entry of the staged head: see kOpaque)
        head_walk = head_walk && head_n <= kHead;
    if (wave_id() != 0 && r0_guess == r0_guess && !head_walk && !(UNORDERED && VERIFY)) {
        // (all the other waves: with more than kHeadGroups maps to build they take longer than the chain, even
        // though three of them share its SIMD)
        if constexpr (kAhead)
            build_group_maps<UNSORTED, UNORDERED>(kf, min(reach, (uint32_t)kWave), true, r0_guess, G, (uint32_t)wave_id() - 1u, (uint32_t)kWaves - 1u, 0u,
                                       QuarterSlots{3u, 0u, kFirstSlots});
        else
            build_group_maps<false, UNORDERED>(kf, min(reach, (uint32_t)kWave), true, r0_guess, G, (uint32_t)wave_id() - 1u, (uint32_t)kWaves - 1u);
    }
    if (wave_id() == 0) {
        // 64 groups at a time, one per lane.  A scan composes the lanes' maps; every lane then knows the state after
        // its group, provided all groups so far share the running epoch and stay inside the binade.  The run up to the
        // first group that cannot promise this is applied in one step, that group is replayed entry by entry, and
        // the scan resumes behind it.  The state (significand M, exponent e) lives in scalar registers.
        uint32_t M = 0;
        int e = 1; // 0.0f
        // The sum changes binade every few entries at first.  The leading groups, up to the last of the first few in
        // which the fp64 sums expect a change, are added entry by entry from the copy in LDS.
        uint32_t first = 0;
        MAKO_TIC(0);
        {
            const uint32_t gq = min((uint32_t)lane_id(), groups - 1u);
            const bool cross = (uint32_t)lane_id() < min(groups, kWalkSeqGroups) &&
                               (lane_id() == 0 || exponent_of((float)G.pg()[gq]) != exponent_of((float)G.pg()[gq + 1u]));
            const unsigned long long bal = __ballot(cross);
            first = bal ? 64u - (uint32_t)__clzll((long long)bal) : 0u;
            if (first) {
                const uint32_t hs = first == groups ? n : uniform_u32(G.start()[min(first, groups - 1u)]);
                const float S = sum_lds(head, min(hs, kHead), 0.0f);
                uint32_t Mv;
                int ev;
                split(S, Mv, ev);
                M = uniform_u32(Mv);
                e = (int)uniform_u32((uint32_t)ev);
            }
        }
        MAKO_TOC(0, 17);
        MAKO_TIC(1);
        bool gave_up = false;
        for (uint32_t base = 0; base < groups && !(UNSORTED && gave_up); base += kWave) {
            const uint32_t gl = min(base + lane_id(), groups - 1u);
            const uint32_t pk_l = G.pack()[gl], st_l = G.start()[gl];
            const uint32_t d0_l = G.d0()[gl], d1_l = G.d1()[gl], cm_l = G.cmax()[gl];
            const uint32_t cnt = min((uint32_t)kWave, groups - base);
            uint32_t done = base == 0 ? first : 0u; // (first <= kWalkSeqGroups)
            while (done < cnt) {
                const bool live = lane_id() >= done && lane_id() < cnt;
                const bool same = live && ((pk_l >> 16) & kEpochBits) == (uint32_t)e;
                Step32 v = lane_id() < done ? identity32() : (same ? Step32{d0_l, d1_l, 0u} : Step32{kSat, kSat, 0u});
                wave_scan_maps(v.d0, v.d1);
                const uint32_t after = M + ((M & 1u) ? v.d1 : v.d0); // < 2^29: no wrap
                const bool ok = same && after + cm_l + 1u < (1u << 24); // group_add_ok for every group so far
                const unsigned long long bad = __ballot(live && !ok);
                const uint32_t f = bad ? (uint32_t)__ffsll((long long)bad) - 1u : cnt;
                if (f > done)
                    M = (uint32_t)__builtin_amdgcn_readlane((int)after, (int)f - 1);
                if (f < cnt) {
                    const uint32_t st = (uint32_t)__builtin_amdgcn_readlane((int)st_l, f);
                    const uint32_t pk = (uint32_t)__builtin_amdgcn_readlane((int)pk_l, f);
                    const uint32_t slot = (pk >> 9) & 0x7fu;
                    if (UNSORTED && (pk & kOpaque)) { // (a share left unsorted whose record does not apply: the row is given up)
                        gave_up = true;
                        break;
                    }
                    if (slot) {
                        const ChainState c = sum_by_quarters(kf, st, pk & kLenMask, G.quarters() + (slot - 1u) * 4u,
                                                             ChainState{M, e, kNone});
                        M = c.M;
                        e = c.e;
                    } else {
                        const float S = exact_span_sum(kf, st, pk & kLenMask, join(M, e));
                        uint32_t Mv;
                        int ev;
                        split(S, Mv, ev);
                        M = uniform_u32(Mv);
                        e = (int)uniform_u32((uint32_t)ev);
                    }
                }
                done = f + 1u;
            }
        }
        MAKO_TOC(1, 18);
        if (lane_id() == 0)
            G.misc()[1] = (UNSORTED && gave_up) ? 0xffffffffu : __float_as_uint(join(M, e)); // (a sum of weights is never a NaN)
    }
    __syncthreads();
    MAKO_STAMP(8);
    if (UNSORTED && G.misc()[1] == 0xffffffffu)
        return false;
    const float total = __uint_as_float(G.misc()[1]);
    const float span = total - 0.0f;
    const float prod = u_row * span;
    const float r0 = prod + 0.0f;
    __syncthreads();

    // What the walk starts from (other than r0, the maps' reach and the staged head only when a rejected draft is redrawn)
    float r_begin = r0;
    uint32_t reach_w = reach, head_n_w = head_n;
    bool head_walk_w = head_walk;
    uint32_t redraw_g = kNone, redraw_at = kNone; // the rejected draft's group and position
    float redraw_q = 0.0f;
    if constexpr (UNORDERED && VERIFY) {
        {
            // Verification (src/gen/sampler.cpp:93-106) of a row in token order: entry i is token i, so the draft's weight is
            // read off the list (0.0f if it is no candidate).  A rejected draft leaves the list for the redraw: as a weight of
            // 0.0f it can neither stop the walk nor change r.  Its group gets no map (it is gone through entry by entry,
            // the draft's entry zeroed in the registers), the staged head and the fp64 sums behind it lose its weight,
            // and the first block's maps are built now, from the redraw's own r.  Only where the reference's walk would
            // run off its list onto the last candidate, and that was the draft, the last one before it is looked for.
            const uint32_t dr = (uint32_t)d.draft[row];
            const float q_draft = dr < n ? qat(dr) : 0.0f;
            if (r0 < q_draft) { // accepted
                if (d.out_cand_idx && d.out_cand_q)
                    for (uint32_t j = tid; j < n && j < d.cand_cap; j += kThreads) {
                        d.out_cand_idx[(size_t)row * d.cand_cap + j] = (int32_t)idat(j);
                        d.out_cand_q[(size_t)row * d.cand_cap + j] = qat(j);
                    }
                if (tid == 0) {
                    RowOut o;
                    o.token = (int32_t)dr;
                    o.n_cand = n;
                    o.total = total;
                    o.q = q_draft;
                    o.path = path_out;
                    o.accepted = 1;
                    write_row(d, row, o);
                }
                return true;
            }
            const float rest = total - q_draft;
            const float span2 = rest - 0.0f;
            const float prod2 = d.u2[row] * span2;
            r_begin = prod2 + 0.0f;
            if (q_draft > 0.0f) { // (the draft is a candidate, at dr < n)
                redraw_at = dr;
                redraw_q = q_draft;
                redraw_g = dr / kGroup; // (a list in token order: every group but the last holds kGroup entries)
                for (uint32_t g = redraw_g + 1u + tid; g <= groups; g += kThreads)
                    G.pg()[g] -= (double)q_draft;
                if (tid == 0) {
                    G.misc()[5] = redraw_g;
                    G.w_pack()[redraw_g] = G.w_pack()[redraw_g] & kLenMask; // (no binade, no quarter records)
                    if (dr < kHead)
                        head[dr] = 0.0f;
                }
            }
            __syncthreads();
            const double rg = (double)r_begin;
            reach_w = groups;
            for (uint32_t g0 = 0; g0 < groups; g0 += kWave) {
                const uint32_t g = g0 + lane_id();
                const unsigned long long beyond = __ballot(g < groups && !(rg * 1.001 - G.pg()[min(g, groups - 1u)] > 0));
                if (beyond) { // uniform
                    reach_w = g0 + (uint32_t)__ffsll((long long)beyond) - 1u;
                    break;
                }
            }
            head_walk_w = reach_w <= kHeadGroups;
            head_n_w = !head_walk_w ? 0u : (reach_w == groups ? n : uniform_u32(G.start()[reach_w]));
            head_walk_w = head_walk_w && head_n_w <= kHead;
            if (rg == rg && !head_walk_w)
                build_group_maps<false, true, true>(kf, min(reach_w, (uint32_t)kWave), true, rg, G, wave_id(), kWaves, 0u,
                                                    QuarterSlots{3u, 0u, kFirstSlots});
            __syncthreads();
        }
    }

    // exact walk
    uint32_t pos = n - 1;
    if (r_begin < 0.0f) {
        pos = 0;
    } else if (r_begin == r_begin && r_begin != INFINITY) {
        MAKO_STAMP(14);
        // The state of the walk (wave 0's, in scalar registers; between blocks of 64 groups in LDS).
        uint32_t M = 0;
        int e = 1;
        uint32_t at = n - 1;
        bool stopped = false;
        uint32_t first = 0; // groups already walked
        if (wave_id() == 0) {
            {
                uint32_t Mv;
                int ev;
                split(r_begin, Mv, ev);
                M = uniform_u32(Mv);
                e = (int)uniform_u32((uint32_t)ev);
            }
            if (head_walk_w && head_n_w) {
                float r = r_begin;
                stopped = walk_lds(head, head_n_w, r, at);
                uint32_t Mv;
                int ev;
                split(r, Mv, ev);
                M = uniform_u32(Mv);
                e = (int)uniform_u32((uint32_t)ev);
                first = reach_w;
            }
        }
        // The groups are walked 64 at a time.  The first block's maps were built beside the running sum, for the
        // binades guessed from u * (fp64 total); deep into a list r is a small difference of large numbers and
        // that guess is worthless (every group would then go entry by entry: 140 us for a 245-group list at
        // u = 0.999), so every later block's maps are built, by all the waves, when the walk gets there, from the
        // exact r at the block's first group.
        // (UNSORTED and UNORDERED, the instances for lists of hundreds of groups: the maps of the NEXT block are built by the other
        // waves while wave 0 walks this one, from the exact r at this block's first group less the fp64 sums up to the
        // group, which is as good a guess as the exact r at the next block's first group unless the walk is about to
        // end; then nothing is built, so that a walk that has ended does not wait for maps nobody needs.  The two
        // blocks' quarter records take the halves of the slots in turn.)
        for (uint32_t base = 0; base < groups; base += kWave) {
            if constexpr (!kAhead) {
                if (base > 0) {
                    if (wave_id() == 0 && lane_id() == 0) {
                        G.misc()[0] = M;
                        G.misc()[1] = (uint32_t)e;
                        sm.aux = stopped ? 1u : 0u;
                    }
                    __syncthreads();
                    if (sm.aux) // uniform
                        break;
                    const double r_here = (double)join(G.misc()[0], (int)G.misc()[1]);
                    if (tid == 0)
                        G.misc()[3] = 0; // (the quarter records so far are done with: their slots start over)
                    __syncthreads();
                    MAKO_TIC(2);
                    build_group_maps<false, UNORDERED>(kf, min(groups, base + (uint32_t)kWave), true, r_here + G.pg()[base], G, wave_id(), kWaves, base);
                    __syncthreads();
                    if (wave_id() == 0) {
                        MAKO_TOC(2, 25);
                        MAKO_COUNT(26, 1);
                    }
                }
            } else {
                double r_here = (double)r_begin;
                if (base > 0) {
                    if (wave_id() == 0 && lane_id() == 0) {
                        G.misc()[0] = M;
                        G.misc()[1] = (uint32_t)e;
                        sm.aux = stopped ? 1u : 0u;
                        // (the slots of the block before this one are done with: the next block's start over)
                        G.misc()[3u + (((base / (uint32_t)kWave) + 1u) & 1u)] = 0;
                    }
                    __syncthreads();
                    if (sm.aux) // uniform
                        break;
                    r_here = (double)join(G.misc()[0], (int)G.misc()[1]);
                }
                const uint32_t next = base + (uint32_t)kWave;
                if (wave_id() != 0 && next < groups && r_here - (G.pg()[next] - G.pg()[base]) > r_here * -0x1p-6) { // uniform
                    const uint32_t half = ((next / (uint32_t)kWave) & 1u);
                    build_group_maps<UNSORTED, UNORDERED, UNORDERED && VERIFY>(kf, min(groups, next + (uint32_t)kWave), true, r_here + G.pg()[base], G, (uint32_t)wave_id() - 1u,
                                               (uint32_t)kWaves - 1u, next, QuarterSlots{3u + half, half * (kQuarterSlots / 2u), kQuarterSlots / 2u});
                }
            }
            if (wave_id() == 0 && !stopped) {
                const uint32_t gl = min(base + lane_id(), groups - 1u);
                const uint32_t pk_l = G.w_pack()[gl], st_l = G.start()[gl];
                const uint32_t d0_l = G.w_d0()[gl], d1_l = G.w_d1()[gl], need_l = G.w_need()[gl]; // (the bound, see build_group_maps)
                const uint32_t cnt = min((uint32_t)kWave, groups - base);
                uint32_t done = base == 0 ? first : 0u; // (first <= kWalkSeqGroups)
                while (done < cnt) {
                    MAKO_COUNT(30, 1);
                    const bool live = lane_id() >= done && lane_id() < cnt;
                    const bool same = live && ((pk_l >> 16) & kEpochBits) == (uint32_t)e;
                    Step32 v = lane_id() < done ? identity32() : (same ? Step32{d0_l, d1_l, 0u} : Step32{kSat, kSat, 0u});
                    wave_scan_maps(v.d0, v.d1);
                    const uint32_t dd = (M & 1u) ? v.d1 : v.d0;
                    const bool ok = same && dd <= M && M - dd >= need_l; // group_sub_ok for every group so far
                    const unsigned long long bad = __ballot(live && !ok);
                    const uint32_t f = bad ? (uint32_t)__ffsll((long long)bad) - 1u : cnt;
                    if (f > done)
                        M = (uint32_t)__builtin_amdgcn_readlane((int)(M - dd), (int)f - 1);
                    if (f >= cnt)
                        break;
                    // Group f goes entry by entry.  Where one group does, its neighbours tend to follow (r is down
                    // among the weights and changes binade every few entries), so the groups behind it are tried one
                    // at a time with a few scalar operations each, the next one's entries already on their way,
                    // and the scan takes over again as soon as one has gone through as a map.
                    uint32_t g = f, passed = 0;
                    uint32_t raw[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu}; // the entries of group g
                    {
                        const uint32_t st = (uint32_t)__builtin_amdgcn_readlane((int)st_l, g);
                        const uint32_t pk = (uint32_t)__builtin_amdgcn_readlane((int)pk_l, g);
                        if (pk & kLenMask)
                            fetch_span_lanes(kf, st, pk & kLenMask, raw);
                    }
                    while (g < cnt && passed < MAKO_WALK_PASSED) {
                        const uint32_t st = (uint32_t)__builtin_amdgcn_readlane((int)st_l, g);
                        const uint32_t pk = (uint32_t)__builtin_amdgcn_readlane((int)pk_l, g);
                        float xa[4];
                        take_span_lanes(raw, pk & kLenMask, xa);
                        if constexpr (UNORDERED && VERIFY) {
                            if (base + g == redraw_g) { // (the rejected draft's own entry, out of the list: entry 64 j + lane is xa[j])
                                const uint32_t in_g = redraw_at % kGroup;
                                if ((uint32_t)lane_id() == (in_g & 63u)) {
                                    xa[0] = (in_g >> 6) == 0u ? 0.0f : xa[0];
                                    xa[1] = (in_g >> 6) == 1u ? 0.0f : xa[1];
                                    xa[2] = (in_g >> 6) == 2u ? 0.0f : xa[2];
                                    xa[3] = (in_g >> 6) == 3u ? 0.0f : xa[3];
                                }
                            }
                        }
                        // (the next group's entries set out now; they are used only if that group is replayed too)
                        const uint32_t g1 = min(g + 1u, cnt - 1u);
                        const uint32_t st1 = (uint32_t)__builtin_amdgcn_readlane((int)st_l, g1);
                        const uint32_t pk1 = (uint32_t)__builtin_amdgcn_readlane((int)pk_l, g1);
                        if (pk1 & kLenMask)
                            fetch_span_lanes(kf, st1, pk1 & kLenMask, raw);
                        bool by_map = false;
                        if (g != f && ((pk >> 16) & kEpochBits) == (uint32_t)e) {
                            const uint32_t d0 = (uint32_t)__builtin_amdgcn_readlane((int)d0_l, g);
                            const uint32_t d1 = (uint32_t)__builtin_amdgcn_readlane((int)d1_l, g);
                            const uint32_t need = (uint32_t)__builtin_amdgcn_readlane((int)need_l, g);
                            const uint32_t d1g = (M & 1u) ? d1 : d0;
                            if (d1g <= M && M - d1g >= need) { // group_sub_ok
                                M -= d1g;
                                by_map = true;
                            }
                        }
                        if (by_map) {
                            ++passed;
                        } else if (UNSORTED && (pk & kOpaque)) {
                            // (a share left unsorted whose record does not apply: the row is given up)
                            at = kNone;
                            stopped = true;
                            break;
                        } else {
                            MAKO_COUNT(22, 1);
                            passed = 0;
                            const uint32_t slot = (pk >> 9) & 0x7fu;
                            if (slot && (pk & kLenMask)) {
                                ChainState c{M, e, kNone};
                                if (walk_by_quarters(xa, st, pk & kLenMask, G.quarters() + (slot - 1u) * 4u, c)) {
                                    at = c.pos;
                                    stopped = true;
                                    break;
                                }
                                M = c.M;
                                e = c.e;
                            } else {
                                float r = join(M, e);
                                if ((pk & kLenMask) && walk_lanes(xa, pk & kLenMask, st, r, at)) {
                                    stopped = true;
                                    break;
                                }
                                uint32_t Mv;
                                int ev;
                                split(r, Mv, ev);
                                M = uniform_u32(Mv);
                                e = (int)uniform_u32((uint32_t)ev);
                            }
                        }
                        ++g;
                    }
                    if (stopped)
                        break;
                    done = g;
                }
            }
        }
        if (wave_id() == 0 && lane_id() == 0)
            G.misc()[2] = at;
        __syncthreads();
        pos = G.misc()[2];
        if (UNSORTED && pos == kNone)
            return false;
    }
    if constexpr (UNORDERED && VERIFY) {
        if (pos == redraw_at) { // (only as the end of the list: a weight of 0.0f stops nothing)
            uint32_t before = 0; // (index + 1 of the last candidate in front of it)
            for (uint32_t i = tid; i < redraw_at; i += kThreads)
                before = qat(i) > 0.0f ? i + 1u : before;
            before = kNone - block_min_u32(kNone - before, sm.bs);
            pos = before ? before - 1u : redraw_at; // (no other candidate: the draft, src/gen/sampler.cpp:104-105)
        }
    }

    MAKO_STAMP(9);
    emit(total, pos);
    return true;
}

// The EXACT instance, out of line where the source is compiled for it (see MAKO_RARE_CALL).
template <bool PLANNED = false>
__device__ MAKO_RARE_CALL void sorted_tail_exact(const mako_sample_desc& d, uint32_t row, const mako_sampling_params& P,
                                                 const uint32_t* kf, const uint32_t* jf, uint32_t n1, double total64,
                                                 uint32_t path, const FinishLds& L, const GroupTable& T = GroupTable{},
                                                 size_t t_base = 0, uint32_t t_groups = 0)
{
    assume_lds(L);
    sorted_tail<PLANNED, false, true>(d, row, P, kf, jf, n1, true, total64, path, L, false, 0.0f, T, t_base, t_groups);
}

} // namespace mako
