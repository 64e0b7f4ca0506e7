// MI355X (gfx950) token sampler kernels.
//
// Pipeline per batch (rows are independent, src/gen/session.cpp:416):
//   scan_kernel    one workgroup per (row, slice): a single coalesced pass over the fp32 logits.  The
//                  token mask and the history penalties are applied in registers; the slice's maximum
//                  and its largest logits (a superset of what top-k / the nucleus can need) go to scratch.
//   finish_kernel  greedy rows: argmax.  top-k rows: the row's candidates are weighted with
//                  q = expf((w - m) / T), sorted by (q desc, idx asc) in LDS, truncated, and drawn from
//                  with the reference's exact fp32 rounding order.  top_k == 0 rows first take a second,
//                  cache-resident pass that sums q exactly over the whole row (all slices in parallel, the
//                  last one to finish continues).  Whatever the candidate lists cannot certify falls to a
//                  whole-row sort path that is exact for every parameter combination.
#pragma once

#include <hip/hip_runtime.h>

#include <math.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/mako_sampler.h"
#include "block_prims.h"
#include "device_math.h"
#include "seqfp.h"

namespace mako {

constexpr uint32_t kNone = 0xffffffffu;

// Optional stage timestamps of row 0 (thread 0), for tuning builds only.
#ifdef MAKO_TIMING
__device__ unsigned long long g_mako_stamp[32];
__shared__ uint32_t s_mako_row; // the row this workgroup serves (set by MAKO_ROW at kernel entry)
#define MAKO_ROW(r)                                                                                                  \
    do {                                                                                                             \
        if (threadIdx.x == 0)                                                                                        \
            s_mako_row = (r);                                                                                        \
    } while (0)
#define MAKO_STAMP(i)                                                                                                \
    do {                                                                                                             \
        if (threadIdx.x == 0 && s_mako_row == 0)                                                                     \
            g_mako_stamp[i] = wall_clock64();                                                                        \
    } while (0)
__device__ unsigned long long g_mako_wg[2][4096];
struct WgTimer {
    __device__ WgTimer()
    {
        if (threadIdx.x == 0)
            g_mako_wg[0][(blockIdx.y * gridDim.x + blockIdx.x) & 4095] = wall_clock64();
    }
    __device__ ~WgTimer()
    {
        if (threadIdx.x == 0)
            g_mako_wg[1][(blockIdx.y * gridDim.x + blockIdx.x) & 4095] = wall_clock64();
    }
};
#define MAKO_WG_TIMER WgTimer wg_timer_
} // namespace mako
// (readers of the above for the tuning scripts; one translation unit at a time is built with MAKO_TIMING)
extern "C" int mako_sampler_debug_wg(unsigned long long* out8192)
{
    return hipMemcpyFromSymbol(out8192, HIP_SYMBOL(mako::g_mako_wg), 8192 * sizeof(unsigned long long)) == hipSuccess
               ? MAKO_OK : MAKO_ERR_HIP;
}
extern "C" int mako_sampler_debug_stamps(unsigned long long* out32)
{
    return hipMemcpyFromSymbol(out32, HIP_SYMBOL(mako::g_mako_stamp), 32 * sizeof(unsigned long long)) == hipSuccess
               ? MAKO_OK : MAKO_ERR_HIP;
}
namespace mako {
#define MAKO_TIC(k)                                                                                                  \
    __builtin_amdgcn_s_waitcnt(0);                                                                                   \
    const unsigned long long tic_##k = wall_clock64()
#define MAKO_TOC(k, i)                                                                                               \
    do {                                                                                                             \
        __builtin_amdgcn_s_waitcnt(0);                                                                               \
        if (lane_id() == 0)                                                                                          \
            g_mako_stamp[i] += wall_clock64() - tic_##k;                                                             \
    } while (0)
#ifdef MAKO_TIMING_COUNTS // event counters: each costs a global round trip, so never together with timestamps
#define MAKO_COUNT(i, v)                                                                                             \
    do {                                                                                                             \
        if (lane_id() == 0)                                                                                          \
            g_mako_stamp[i] += (v);                                                                                  \
    } while (0)
#else
#define MAKO_COUNT(i, v) ((void)0)
#endif
#else
#define MAKO_STAMP(i) ((void)0)
#define MAKO_ROW(r) ((void)0)
#define MAKO_COUNT(i, v) ((void)0)
#define MAKO_WG_TIMER ((void)0)
#define MAKO_TIC(k) ((void)0)
#define MAKO_TOC(k, i) ((void)0)
#endif

constexpr uint32_t kSliceMax = 16384; // elements per slice: 16 per thread
constexpr uint32_t kMaxSlices = 64;
constexpr uint32_t kCap = 512;       // candidates kept per slice
constexpr uint32_t kTopKFast = 128;  // largest top_k resolved from the per-slice candidates
constexpr uint32_t kSortMax = 4096;  // candidates the finisher sorts in LDS
constexpr uint32_t kDynLds = 65536;  // dynamic LDS of both kernels
constexpr uint32_t kBins = 2048;     // weight histogram of top_k == 0 rows, see weight_bin()
constexpr uint32_t kBinSumBits = 44; // a bin's record: count << 44 | sum of 24-bit significands

// Histogram bin of a weight q in (0, 1], by its bits: 128 bins per binade for the eight binades below 1.0 (bins
// 1024..2047) and 8 per binade for everything smaller, subnormals included (bins 71..1023; bins below 71 stay
// empty).  Bin edges include every binade boundary, so all weights of a bin share their exponent and the bin's
// mass is exactly (sum of 24-bit significands) * 2^(exponent - 150).  The fine bins keep near-flat rows, whose
// weights all lie within a factor of two, spread over all workers.
constexpr uint32_t kFineFrom = 0x3b810000u; // bits(2^-8) + 0x10000: the top fine bin holds 1.0 alone
constexpr uint32_t kCoarseShift = 20;       // 8 bins per binade
constexpr uint32_t kCoarseBase = 1023u - ((kFineFrom - 1u) >> kCoarseShift); // 71
__device__ __forceinline__ uint32_t weight_bin(uint32_t bits)
{
    return bits >= kFineFrom ? min(1024u + ((bits - kFineFrom) >> 16), kBins - 1u) : (bits >> kCoarseShift) + kCoarseBase;
}
// Smallest bits(q) of a bin, and one past the largest.
__device__ __forceinline__ uint32_t bin_lo_key(uint32_t b)
{
    if (b >= 1024u)
        return kFineFrom + ((b - 1024u) << 16);
    return b > kCoarseBase ? (b - kCoarseBase) << kCoarseShift : 0u;
}
__device__ __forceinline__ uint32_t bin_hi_key(uint32_t b)
{
    return b + 1u < kBins ? bin_lo_key(b + 1u) : kFineFrom + (1024u << 16); // (just above bits(1.0f))
}

constexpr uint32_t kFlagFirstNan = 1u; // element 0 of the row is NaN (slice 0 only)
constexpr uint32_t kFlagOverflow = 2u; // more than kCap logits reached the slice's threshold
constexpr uint32_t kFlagComplete = 4u; // every logit above -inf was emitted

struct SliceStat {
    float wmax;       // max of the slice's penalised logits (-inf if none compares greater)
    uint32_t argidx;  // first index holding it, kNone if nothing exceeded -inf
    uint32_t flags;
    uint32_t n_emit;  // candidates written for this slice
    uint32_t tau_key; // order key of the emission threshold: every logit with key >= tau_key was emitted
    uint32_t above;   // logits of the slice strictly above the row's close_token logit (0 without one)
    uint32_t pad[2];
};

constexpr uint32_t kWorkers = 32;  // workgroups that share the sort of one wide-nucleus row
constexpr uint32_t kGroup = 256;      // a sorted list is processed in groups of one wave x four entries per lane
constexpr uint32_t kMaxGroups = 1024; // groups per list
constexpr uint32_t kSegCap = 6144;    // entries a worker sorts in LDS
constexpr uint32_t kFine = 2048;      // value buckets of that sort
// dynamic LDS of sort_kernel: the entries, their order, the buckets, and a copy of the sorted weights for the group
// records
constexpr uint32_t kSortLds = kSegCap * 8u + kSegCap * 2u + (kFine + 4u) * 4u + kSegCap * 4u;
constexpr uint32_t kSortedCopyAt = kSegCap * 8u + kSegCap * 2u + (kFine + 4u) * 4u; // byte offset of that copy

// Work order for a top_k == 0 row whose nucleus is too wide for the per-slice candidate lists: the weights
// with bits(q) >= key_lo (n0 of them) are split by value into kWorkers contiguous ranges of about equal size.
struct BigPlan {
    uint32_t flag;   // 1: the row waits for sort_kernel's workers; 2: for its whole-row path (worker 0 alone);
                     // 3: a narrow nucleus, finished by worker 0 from the candidate lists
    uint32_t n0;     // entries to sort
    uint32_t pad0;
    uint32_t groups; // groups of the whole list: each worker's range is cut into groups of kGroup on its own
    double total64;  // exact fp64 sum of q over the row's candidates
    uint32_t thr;    // bits(q) below which the nucleus cannot reach
    uint32_t pad;
    uint32_t key_lo[kWorkers]; // worker w takes bits(q) in [key_lo[w], key_hi[w])
    uint32_t key_hi[kWorkers];
    uint32_t off[kWorkers];    // and writes them from position off[w] of the sorted list
    uint32_t cnt[kWorkers];
    uint32_t gbase[kWorkers];  // first group of worker w
    uint32_t cursor[kWorkers]; // entries partition_kernel has handed to worker w so far
    double mass[kWorkers];     // sum of the weights above worker w's range
};

// Per-group records of a planned row's sorted list, written by the workers and read by the last of them.
struct GroupTable {
    double* sum;     // fp64 sum of the group's weights
    uint32_t* d0;    // the group's map for the running fp32 sum in the epoch guessed from the mass before it
    uint32_t* d1;
    uint32_t* cmax;
    uint32_t* start; // first entry of the group in the sorted list
    uint32_t* pack;  // entries | guessed exponent << 16 | kHasQuarters if `quarters` holds records for the group
    uint4* quarters; // [4] per group: the maps of the group's four quarters (see build_quarters)
};

struct Scratch {
    SliceStat* stats;  // [max_rows][kMaxSlices]
    float* cand_w;     // [max_rows][slices_cap][kCap] penalised logits of the slice's candidates
    uint32_t* cand_i;  // [max_rows][slices_cap][kCap] their token ids
    double* part_sum;  // [max_rows][kMaxSlices] exact fp64 sum of q over the slice (top_k == 0 rows)
    uint32_t* part_n;  // [max_rows][kMaxSlices] candidates (q > 0, q >= min_p) in the slice
    BigPlan* plan;     // [max_rows]; flag zero between calls
    unsigned long long* bins; // [max_rows][kBins] weight histogram of top_k == 0 rows: candidates in the bin << 44 |
                              // sum of their 24-bit significands (kBinSumBits: at most 2^20 - 1 logits per row).
                              // A bin's exact mass is that sum * 2^(e - 150), e being the bin's exponent.  The
                              // slices add with one atomic per non-empty bin; plan_kernel reads the row's bins
                              // and leaves them zero
    float* wbuf;       // [max_rows][vpad] penalised logits of rows on the whole-row path; top_k == 0 rows keep
                       // bits(q) of every logit here instead (0 where q is not a candidate)
    uint32_t* cnt;     // [max_rows][vpad] token counts; all zero between calls
    uint32_t* key[2];  // [max_rows][vpad] candidate keys (~bits(q)), ping-pong; [1] also takes the workers' unsorted
                       // shares (bits(q)) from partition_kernel
    uint32_t* idx[2];  // [max_rows][vpad] candidate token ids, likewise
    uint8_t* bin_worker; // [max_rows][kBins] the worker that takes the weights of each histogram bin (0xff: none)
    GroupTable gt;     // [max_rows][g_cap] each
    // Work lists.  sort_kernel and tail_kernel are launched with one workgroup per POSSIBLE piece of work, but
    // workgroup i serves entry i of its kernel's list and exits if there is none: the busy workgroups are then the
    // first ones dispatched and land evenly on the XCDs, shader engines and CUs, whatever the mix of rows.
    // (finish_kernel and plan_kernel get the same effect from find_piece().)
    uint32_t* work_n;      // [8] entries in work_sort, work_tail (zeroed by scan_kernel); then, 16-byte aligned at [4],
                           // the second pass's pieces per top_k == 0 row, their length and the number of workgroups
                           // with work (scan_kernel's first workgroup decides, see second_pass_pieces())
    uint32_t* work_sort;   // [max_rows * kWorkers] row << 8 | worker; appended by finish_kernel and plan_kernel
    uint32_t* work_tail;   // [max_rows] row; appended by plan_kernel
    uint64_t vpad;
    uint32_t slices_cap;
    uint32_t g_cap;    // vpad / kGroup + kWorkers
};

// Total order on floats as unsigned keys: -inf < ... < -0 = +0 < ... < +inf.  Never called on NaN.
__device__ __forceinline__ uint32_t order_key(float f)
{
    const uint32_t b = __float_as_uint(f + 0.0f); // -0 -> +0
    return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}
__device__ __forceinline__ float order_unkey(uint32_t k)
{
    const uint32_t b = (k & 0x80000000u) ? (k ^ 0x80000000u) : ~k;
    return __uint_as_float(b);
}
constexpr uint32_t kKeyNegInf = 0x007fffffu; // order_key(-inf)

enum RowClass { kGreedy = 0, kTopK = 1, kNucleus = 2, kGeneral = 3 };

__host__ __device__ __forceinline__ RowClass classify(const mako_sampling_params& p)
{
    if (p.temperature <= 0.0f) // Sampler::greedy, src/gen/sampler.hpp:26
        return kGreedy;
    if (!(p.top_p < 1.0f)) // no top-p: the candidate order is not the sorted one (sampler.cpp:44)
        return kGeneral;
    if (p.top_k == 0)
        return kNucleus;
    return p.top_k <= kTopKFast ? kTopK : kGeneral;
}

__device__ __forceinline__ bool penalties_neutral(const mako_sampling_params& p)
{
    return p.repetition_penalty == 1.0f && p.presence_penalty == 0.0f && p.frequency_penalty == 0.0f;
}

// ---------------------------------------------------------------------------------------------
// slice loading, shared by both kernels
// ---------------------------------------------------------------------------------------------

// Thread t of a slice owns 16 logits: for k = 0..3 the four consecutive ones at lo + k * 4096 + 4 * t
// (VEC), or lo + j * 1024 + t for j = 0..15 (scalar).  Either way a wavefront's loads are contiguous and
// each logit is read once.
template <bool VEC>
__device__ __forceinline__ uint32_t elem_index(uint32_t lo, uint32_t tid, uint32_t j)
{
    return VEC ? lo + (j >> 2) * 4096u + tid * 4u + (j & 3u) : lo + j * (uint32_t)kThreads + tid;
}

// accept() history -> per-token counts for [lo, hi) in LDS (src/gen/sampler.cpp:15-18); generic form used
// when a row's history is too long for the register-resident scheme of load_penalised().
__device__ __forceinline__ void build_counts(const mako_sample_desc& d, uint32_t row, uint32_t hl, uint32_t lo,
                                             uint32_t hi, uint32_t slice_len, uint32_t* s_cnt)
{
    const uint32_t tid = threadIdx.x;
    uint4* z = reinterpret_cast<uint4*>(s_cnt); // slice_len is a multiple of 4
    for (uint32_t i = tid; i < slice_len / 4; i += kThreads)
        z[i] = make_uint4(0, 0, 0, 0);
    __syncthreads();
    const int32_t* ht = d.hist_tokens + (int64_t)row * d.hist_stride;
    const uint32_t* hc = d.hist_counts ? d.hist_counts + (int64_t)row * d.hist_stride : nullptr;
    for (uint32_t h = tid; h < hl; h += kThreads) {
        const uint32_t t = (uint32_t)ht[h];
        if (t >= lo && t < hi)
            atomicAdd(&s_cnt[t - lo], hc ? hc[h] : 1u);
    }
    __syncthreads();
}

// The thread's 16 logits, raw, plus the mask bits of each group of four (VEC) or of each logit (scalar).
// Issued before anything else so that the HBM latency overlaps the LDS work that follows.
template <bool VEC>
struct RawSlice {
    float4 v[4];
    uint32_t bits[4]; // VEC: bit c of bits[k] = logit 4k+c allowed; scalar: bit j of bits[0] = logit j allowed
};

template <bool VEC>
__device__ __forceinline__ void load_raw(const mako_sample_desc& d, uint32_t row, uint32_t lo, uint32_t hi, RawSlice<VEC>& r)
{
    const uint32_t tid = threadIdx.x;
    const float* lrow = d.logits + (int64_t)row * d.logits_stride;
    const uint32_t* mrow = d.mask ? d.mask + (int64_t)row * d.mask_stride : nullptr;
    const float nan = __uint_as_float(0x7fc00000u);
    if (VEC) {
        // all four loads go out back to back, from clamped addresses and without a branch between them (a branch
        // would make the compiler wait for each load before the next); what lies past the slice is dropped after
        uint32_t at[4];
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint32_t i = lo + k * 4096u + tid * 4u;
            at[k] = i < hi ? i : hi - 4u; // hi - lo is a positive multiple of 4 in this mode
            r.v[k] = *reinterpret_cast<const float4*>(lrow + at[k]);
        }
        if (mrow) {
#pragma unroll
            for (uint32_t k = 0; k < 4; ++k)
                r.bits[k] = mrow[at[k] >> 5] >> (at[k] & 31u);
        }
        if (!mrow) {
#pragma unroll
            for (uint32_t k = 0; k < 4; ++k)
                r.bits[k] = 0xfu;
        }
        // (finish_slice() replaces what was read past the slice: nothing here touches the loaded values, so the
        // loads stay in flight while the caller goes on)
    } else {
        float* f = reinterpret_cast<float*>(r.v);
        uint32_t allowed = 0xffffu;
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j) {
            const uint32_t i = lo + j * (uint32_t)kThreads + tid;
            f[j] = nan;
            if (i < hi) {
                f[j] = lrow[i];
                if (mrow && !((mrow[i >> 5] >> (i & 31u)) & 1u))
                    allowed &= ~(1u << j);
            }
        }
        r.bits[0] = allowed;
    }
}

// How many of the thread's logits (as the sampler is given them: a token the mask clears is -inf) are strictly
// greater than v: the count of ReasoningBudget::forced, src/server/openai.cpp:599-602.
template <bool VEC>
__device__ __forceinline__ uint32_t count_above(const RawSlice<VEC>& r, uint32_t lo, uint32_t hi, float v)
{
    const uint32_t tid = threadIdx.x;
    uint32_t c = 0;
    if (VEC) {
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            if (lo + k * 4096u + tid * 4u < hi) {
                c += ((r.bits[k] & 1u) && r.v[k].x > v) ? 1u : 0u;
                c += ((r.bits[k] & 2u) && r.v[k].y > v) ? 1u : 0u;
                c += ((r.bits[k] & 4u) && r.v[k].z > v) ? 1u : 0u;
                c += ((r.bits[k] & 8u) && r.v[k].w > v) ? 1u : 0u;
            }
        }
    } else {
        const float* f = reinterpret_cast<const float*>(r.v);
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j)
            c += (lo + j * (uint32_t)kThreads + tid < hi && ((r.bits[0] >> j) & 1u) && f[j] > v) ? 1u : 0u;
    }
    return c;
}

// Mask and penalties (src/gen/sampler.cpp:22-28) applied to the raw logits; slots past the end of the
// slice hold NaN, which never wins a comparison and never becomes a candidate.
template <bool VEC>
__device__ __forceinline__ void finish_slice(const RawSlice<VEC>& r, uint32_t lo, uint32_t hi, const mako_sampling_params& P,
                                             bool pen, const uint32_t* s_cnt, float (&wv)[16], bool masked)
{
    const uint32_t tid = threadIdx.x;
    if (VEC && !masked) { // uniform: no mask, nothing to clear
        const float nan = __uint_as_float(0x7fc00000u);
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const bool inside = lo + k * 4096u + tid * 4u < hi;
            wv[4 * k + 0] = !inside ? nan : r.v[k].x;
            wv[4 * k + 1] = !inside ? nan : r.v[k].y;
            wv[4 * k + 2] = !inside ? nan : r.v[k].z;
            wv[4 * k + 3] = !inside ? nan : r.v[k].w;
        }
    } else if (VEC) {
        const float nan = __uint_as_float(0x7fc00000u);
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const bool inside = lo + k * 4096u + tid * 4u < hi;
            wv[4 * k + 0] = !inside ? nan : ((r.bits[k] & 1u) ? r.v[k].x : -INFINITY);
            wv[4 * k + 1] = !inside ? nan : ((r.bits[k] & 2u) ? r.v[k].y : -INFINITY);
            wv[4 * k + 2] = !inside ? nan : ((r.bits[k] & 4u) ? r.v[k].z : -INFINITY);
            wv[4 * k + 3] = !inside ? nan : ((r.bits[k] & 8u) ? r.v[k].w : -INFINITY);
        }
    } else {
        const float* f = reinterpret_cast<const float*>(r.v);
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j)
            wv[j] = ((r.bits[0] >> j) & 1u) ? f[j] : -INFINITY;
    }
    if (pen) {
        if (VEC) {
#pragma unroll
            for (uint32_t k = 0; k < 4; ++k) {
                const uint32_t i = lo + k * 4096u + tid * 4u;
                if (i < hi) {
                    const uint4 n = *reinterpret_cast<const uint4*>(s_cnt + (i - lo));
                    if (n.x | n.y | n.z | n.w) {
                        if (n.x)
                            wv[4 * k + 0] = penalize(wv[4 * k + 0], n.x, P.repetition_penalty, P.presence_penalty, P.frequency_penalty);
                        if (n.y)
                            wv[4 * k + 1] = penalize(wv[4 * k + 1], n.y, P.repetition_penalty, P.presence_penalty, P.frequency_penalty);
                        if (n.z)
                            wv[4 * k + 2] = penalize(wv[4 * k + 2], n.z, P.repetition_penalty, P.presence_penalty, P.frequency_penalty);
                        if (n.w)
                            wv[4 * k + 3] = penalize(wv[4 * k + 3], n.w, P.repetition_penalty, P.presence_penalty, P.frequency_penalty);
                    }
                }
            }
        } else {
#pragma unroll
            for (uint32_t j = 0; j < 16; ++j) {
                const uint32_t i = lo + j * (uint32_t)kThreads + tid;
                if (i < hi) {
                    const uint32_t n = s_cnt[i - lo];
                    if (n)
                        wv[j] = penalize(wv[j], n, P.repetition_penalty, P.presence_penalty, P.frequency_penalty);
                }
            }
        }
    }
}

// The thread's logits after the mask and the penalties (src/gen/sampler.cpp:22-28): wv[16] in the slice layout.
//
// KH > 0 (histories of at most KH * 1024 entries): thread t handles history entries t, t + 1024, ...  The
// per-token counts are accumulated in LDS; for every distinct token of the slice the thread holding its first
// entry (an election, so that each token is handled once) computes the penalised logit: one IEEE division per
// history entry instead of one per logit slot.  The logit travels through the token's slot of the LDS table:
// its owner puts the masked raw value there, the elected thread replaces it by the penalised one, the owner
// takes it back.  (A gather from device memory instead would return behind every streaming load in flight, and
// costs the slices that hold most of a Zipf history a microsecond more.)
// KH == 0: any history length; counts in LDS, every owner penalises its own logits.
struct NoOverlap {
    __device__ __forceinline__ void operator()() const {}
};

// `overlap` runs right after the slice's loads have been issued: work that does not depend on them hides
// behind their latency.  It must be reached by the whole workgroup or by none of it.
template <bool VEC, int KH, typename Overlap = NoOverlap>
__device__ __forceinline__ void load_penalised(const mako_sample_desc& d, uint32_t row, uint32_t lo, uint32_t hi,
                                               uint32_t slice_len, const mako_sampling_params& P, uint32_t hl, bool pen,
                                               uint32_t* s_cnt, float (&wv)[16], Overlap overlap = Overlap(),
                                               bool want_above = false, float close_v = 0.0f, uint32_t* above = nullptr)
{
    const uint32_t tid = threadIdx.x;
    // My history entries go first: loads return in the order they were issued, so whatever waits for these does not
    // wait for the logits behind them, and the counting in LDS below runs while the logits are still on their way.
    // (Loads from clamped positions, issued without branches between them; what was not wanted is dropped
    // afterwards: a branch around each load would make every load wait for the one before.)
    // Whether they are asked for depends on the kernel's arguments alone, not on the row's parameters or its history
    // length (`hl`, `pen`): a caller may still be waiting for those when these loads and the logits' go out.
    const bool may_penalise = KH > 0 && d.hist_tokens != nullptr && d.hist_stride > 0; // uniform
    const int32_t* ht = d.hist_tokens + (int64_t)row * d.hist_stride;
    const uint32_t* hc = d.hist_counts ? d.hist_counts + (int64_t)row * d.hist_stride : nullptr;
    uint32_t tok[KH > 0 ? KH : 1], cnt[KH > 0 ? KH : 1];
    bool have[KH > 0 ? KH : 1];
    if (may_penalise) {
        const uint32_t last = (uint32_t)d.hist_stride - 1u; // (entries past the row's length are read and dropped)
#pragma unroll
        for (int k = 0; k < KH; ++k)
            tok[k] = (uint32_t)ht[min(tid + (uint32_t)k * kThreads, last)];
        if (hc) {
#pragma unroll
            for (int k = 0; k < KH; ++k)
                cnt[k] = hc[min(tid + (uint32_t)k * kThreads, last)];
        }
    }
    RawSlice<VEC> raw;
    load_raw<VEC>(d, row, lo, hi, raw);
    overlap();
    if (want_above) // uniform
        *above = count_above<VEC>(raw, lo, hi, close_v);
    if (!pen) {
        finish_slice<VEC>(raw, lo, hi, P, false, s_cnt, wv, d.mask != nullptr);
        return;
    }
    if (KH == 0) {
        build_counts(d, row, hl, lo, hi, slice_len, s_cnt);
        finish_slice<VEC>(raw, lo, hi, P, true, s_cnt, wv, d.mask != nullptr);
        return;
    }
#pragma unroll
    for (int k = 0; k < KH; ++k) {
        if (!hc)
            cnt[k] = 1;
        // (an entry that counts no occurrence is no entry: the reference's table holds what accept() has seen)
        have[k] = tid + (uint32_t)k * kThreads < hl;
        if (!(have[k] && tok[k] >= lo && tok[k] < hi && cnt[k] != 0u)) {
            tok[k] = kNone;
            cnt[k] = 0;
        }
    }
    // (barriers that order LDS traffic only: the logits stay in flight)
    MAKO_STAMP(20);
    uint4* z = reinterpret_cast<uint4*>(s_cnt); // slice_len is a multiple of 4
    for (uint32_t i = tid; i < slice_len / 4; i += kThreads)
        z[i] = make_uint4(0, 0, 0, 0);
    lds_barrier();
    MAKO_STAMP(21);
    // every entry adds its occurrences to its token's slot; the entry that finds the slot empty speaks for the
    // token from here on (which of a token's entries that is does not matter: it only carries the logit through
    // penalize() once)
    bool elected[KH > 0 ? KH : 1];
#pragma unroll
    for (int k = 0; k < KH; ++k) {
        elected[k] = false;
        if (tok[k] != kNone)
            elected[k] = atomicAdd(&s_cnt[tok[k] - lo], cnt[k]) == 0u;
    }
    lds_barrier();
#pragma unroll
    for (int k = 0; k < KH; ++k)
        if (elected[k])
            cnt[k] = s_cnt[tok[k] - lo]; // occurrences of the token in the whole history
    lds_barrier(); // (the slots are about to be overwritten)
    MAKO_STAMP(22);
    finish_slice<VEC>(raw, lo, hi, P, false, s_cnt, wv, d.mask != nullptr);
    MAKO_STAMP(23);
    // owners: a logit whose slot is taken goes into the slot (its bits); `moved` remembers which of the sixteen
    uint32_t moved = 0;
    if (VEC) {
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint32_t i = lo + k * 4096u + tid * 4u;
            if (i < hi) {
                uint4* slot = reinterpret_cast<uint4*>(s_cnt + (i - lo));
                const uint4 n = *slot;
                if (n.x | n.y | n.z | n.w) {
                    *slot = make_uint4(n.x ? __float_as_uint(wv[4 * k + 0]) : 0u, n.y ? __float_as_uint(wv[4 * k + 1]) : 0u,
                                       n.z ? __float_as_uint(wv[4 * k + 2]) : 0u, n.w ? __float_as_uint(wv[4 * k + 3]) : 0u);
                    moved |= ((n.x ? 1u : 0u) | (n.y ? 2u : 0u) | (n.z ? 4u : 0u) | (n.w ? 8u : 0u)) << (4u * k);
                }
            }
        }
    } else {
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j) {
            const uint32_t i = lo + j * (uint32_t)kThreads + tid;
            if (i < hi && s_cnt[i - lo]) {
                s_cnt[i - lo] = __float_as_uint(wv[j]);
                moved |= 1u << j;
            }
        }
    }
    lds_barrier();
#pragma unroll
    for (int k = 0; k < KH; ++k)
        if (elected[k]) {
            const float rv = __uint_as_float(s_cnt[tok[k] - lo]); // (already -inf where the mask clears the token)
            s_cnt[tok[k] - lo] =
                __float_as_uint(penalize(rv, cnt[k], P.repetition_penalty, P.presence_penalty, P.frequency_penalty));
        }
    lds_barrier();
    if (moved) {
        if (VEC) {
#pragma unroll
            for (uint32_t k = 0; k < 4; ++k)
                if ((moved >> (4u * k)) & 0xfu) {
                    const uint4 v = *reinterpret_cast<const uint4*>(s_cnt + (lo + k * 4096u + tid * 4u - lo));
                    wv[4 * k + 0] = (moved >> (4u * k)) & 1u ? __uint_as_float(v.x) : wv[4 * k + 0];
                    wv[4 * k + 1] = (moved >> (4u * k)) & 2u ? __uint_as_float(v.y) : wv[4 * k + 1];
                    wv[4 * k + 2] = (moved >> (4u * k)) & 4u ? __uint_as_float(v.z) : wv[4 * k + 2];
                    wv[4 * k + 3] = (moved >> (4u * k)) & 8u ? __uint_as_float(v.w) : wv[4 * k + 3];
                }
        } else {
#pragma unroll
            for (uint32_t j = 0; j < 16; ++j)
                if ((moved >> j) & 1u)
                    wv[j] = __uint_as_float(s_cnt[j * (uint32_t)kThreads + tid]);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// scan_kernel
// ---------------------------------------------------------------------------------------------

struct alignas(16) ScanShared {
    uint32_t wave_max[kWaves]; // order keys
    uint32_t wave_kth[kWaves];
    uint32_t wave_above[kWaves];
    uint32_t argidx;
    uint32_t emit_n;
    uint32_t emit_flags;
    float cw[kCap];
    uint32_t ci[kCap];
};

// Into how many pieces finish_kernel cuts each top_k == 0 row, and how long a piece is.  A piece is one to four
// blocks of 4096 logits (a slice is four): as few blocks as keep all the pieces of the batch within one round of
// workgroups (`cus` of them run at a time, one per CU), since the pass is bound by instruction issue and more
// workgroups with less work each finish sooner.  Worked out from the rows' parameters by one wave of scan_kernel's
// first workgroup and left in Scratch::work_n; batches of more than 64 rows take whole slices.
__device__ __forceinline__ uint32_t second_pass_pieces(const mako_sample_desc& d, uint32_t slices, uint32_t slice_len,
                                                       uint32_t cus, uint32_t& piece_len, uint32_t& busy)
{
    piece_len = slice_len;
    busy = d.n_rows * slices; // (no more than that)
    if (d.n_rows > (uint32_t)kWave)
        return slices;
    const uint32_t r = lane_id();
    const bool nucleus = r < d.n_rows && classify(d.params[r]) == kNucleus;
    const uint32_t rows = (uint32_t)__popcll(__ballot(nucleus));
    busy = rows * slices;
    for (uint32_t blocks = 1; blocks < 4u; ++blocks) {
        const uint32_t len = blocks * 4096u;
        const uint32_t n = (d.n_vocab + len - 1u) / len;
        if (len < slice_len && n <= kMaxSlices && rows * n <= cus) {
            piece_len = len;
            busy = rows * n;
            return n;
        }
    }
    return slices;
}

// Which piece of work does workgroup `piece` of finish_kernel (per_nucleus = slices, per_other = 1) or of plan_kernel
// (1, 0) serve?  Rows are taken in order, each contributing per_nucleus pieces if it is a top_k == 0 row and
// per_other otherwise.  Every workgroup works this out for itself from the rows' parameters (a few loads and one
// scan).  Returns false when there is no such piece; all threads receive the same answer.
__device__ bool find_piece(const mako_sample_desc& d, uint32_t piece, uint32_t per_nucleus, uint32_t per_other,
                           uint32_t& row, uint32_t& sub, BlockScratch& bs)
{
    const uint32_t tid = threadIdx.x;
    if (d.n_rows <= (uint32_t)kWave) {
        // up to 64 rows: every wave works it out for itself, one row per lane, without a barrier
        const uint32_t r = lane_id();
        uint32_t pieces = 0;
        if (r < d.n_rows)
            pieces = classify(d.params[r]) == kNucleus ? per_nucleus : per_other;
        const uint32_t upto = __ockl_wfscan_add_u32(pieces, true);
        const unsigned long long bal = __ballot(piece >= upto - pieces && piece < upto);
        if (bal == 0ull)
            return false;
        const int owner = __ffsll((long long)bal) - 1;
        row = (uint32_t)owner;
        sub = piece - (uint32_t)__builtin_amdgcn_readlane((int)(upto - pieces), owner);
        return true;
    }
    uint32_t before = 0;
    for (uint32_t base = 0; base < d.n_rows; base += kThreads) {
        const uint32_t r = base + tid;
        uint32_t pieces = 0;
        if (r < d.n_rows)
            pieces = classify(d.params[r]) == kNucleus ? per_nucleus : per_other;
        uint32_t tot;
        const uint32_t at = before + block_excl_scan_u32(pieces, tot, bs);
        if (piece >= at && piece < at + pieces)
            bs.bcast = ((unsigned long long)r << 32) | (unsigned long long)(piece - at);
        before += tot;
        if (piece < before) { // uniform
            __syncthreads();
            const unsigned long long v = bs.bcast;
            __syncthreads();
            row = (uint32_t)(v >> 32);
            sub = (uint32_t)v;
            return true;
        }
    }
    return false;
}

// A lower bound, tight to 2^-9 relative, of the j-th largest of the wavefront's 64 order keys (j >= 1): the largest
// v with at least j keys >= v, built bit by bit from the top down to bit 14 (the low fourteen bits stay zero: whoever
// uses the result as a threshold keeps at least j keys, and a handful more at most).  One vector compare per bit;
// the rest is scalar.
__device__ __forceinline__ uint32_t wave_kth_largest(uint32_t key, uint32_t j)
{
    uint32_t prefix = 0;
#pragma unroll
    for (int b = 31; b >= 14; --b) {
        const uint32_t cand = prefix | (1u << b);
        const uint32_t c = (uint32_t)__popcll(__ballot(key >= cand));
        prefix = c >= j ? cand : prefix;
    }
    return prefix;
}

// grid = (slices, rows).
// (ABOVE: the batch has close tokens, whose logits' ranks are counted on the way; a variant of its own because the
// count takes sixteen more registers, up to the limit for two workgroups per CU, which no other batch should pay)
template <bool VEC, int KH, bool ABOVE = false>
__global__ __launch_bounds__(kThreads) void scan_kernel(mako_sample_desc d, Scratch sc_arg, uint32_t slice_len,
                                                        uint32_t cus)
{
    // (scan_kernel takes the context's record by value: its first loads then need no trip to memory for a pointer)
    const Scratch& sc = sc_arg;
    MAKO_ROW(blockIdx.y);
#ifdef MAKO_TIMING_SCAN
    MAKO_WG_TIMER;
#endif
    // (16-byte alignment: the table is cleared and read with 128-bit LDS operations, which crawl when misaligned)
    extern __shared__ __align__(16) uint32_t s_dyn[]; // [slice_len] token counts when the row has penalties
    __shared__ ScanShared sm;

    const uint32_t row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x;
    MAKO_STAMP(28);
    const uint32_t lo = slice * slice_len;
    const uint32_t hi = min(d.n_vocab, lo + slice_len);
    // (the history's length is asked for whatever the parameters say: its load then leaves together with theirs)
    const uint32_t hl_row = d.hist_tokens ? min(d.hist_len[row], (uint32_t)d.hist_stride) : 0u;
    const mako_sampling_params P = d.params[row];
    const RowClass cls = classify(P);
    // Greedy rows ignore the penalties (src/gen/sampler.cpp:77-78).
    const uint32_t hl = cls != kGreedy ? hl_row : 0u;
    const bool pen = hl > 0 && !penalties_neutral(P);
    if (tid == 0) {
        sm.argidx = kNone;
        sm.emit_n = 0;
        sm.emit_flags = 0;
        if (row == 0 && slice == 0) { // the lists finish_kernel and plan_kernel append to start empty
            sc.work_n[0] = 0;
            sc.work_n[1] = 0;
        }
    }
    if (row == 0 && slice == 0 && wave_id() == 1) { // how the second pass will be cut up
        uint32_t piece_len, busy;
        const uint32_t pieces = second_pass_pieces(d, gridDim.x, slice_len, cus, piece_len, busy);
        if (lane_id() == 0)
            *reinterpret_cast<uint4*>(sc.work_n + 4) = make_uint4(pieces, piece_len, busy, 0u);
    }
    // ReasoningBudget::forced's question (src/server/openai.cpp:598-602), answered in the same pass over the logits
    bool want_above = false;
    float close_v = 0.0f;
    if (ABOVE && d.close_token) {
        const int32_t ct = d.close_token[row];
        if (ct >= 0 && (uint32_t)ct < d.n_vocab &&
            (!d.mask || ((d.mask[(int64_t)row * d.mask_stride + ((uint32_t)ct >> 5)] >> ((uint32_t)ct & 31u)) & 1u))) {
            want_above = true;
            close_v = d.logits[(int64_t)row * d.logits_stride + ct];
        }
    }
    uint32_t above = 0;
    float wv[16];
    if (ABOVE) {
        load_penalised<VEC, KH>(d, row, lo, hi, slice_len, P, hl, pen, s_dyn, wv, NoOverlap(), want_above, close_v, &above);
        if (want_above) // uniform
            above = __ockl_wfred_add_u32(above);
    } else {
        load_penalised<VEC, KH>(d, row, lo, hi, slice_len, P, hl, pen, s_dyn, wv);
    }

    MAKO_STAMP(29);
    // maximum of the thread's logits (NaNs ignored), then of the wave, then of the slice
    float best = -INFINITY;
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j)
        best = fmaxf(best, wv[j]);
    const uint32_t bkey = order_key(best);
    const bool emits = cls == kTopK || cls == kNucleus;
    const uint32_t wmax = __ockl_wfred_max_u32(bkey);
    uint32_t wkth = 0;
    if (emits) {
        // Every logit that can be among the row's K largest is among this slice's K largest.  Each wave
        // takes the ceil(K/16)-th largest of its per-thread maxima; at least K logits of the slice are >= the
        // smallest of those 16 values, which becomes the emission threshold.
        const uint32_t K = cls == kTopK ? P.top_k : kTopKFast;
        wkth = wave_kth_largest(bkey, (K + kWaves - 1) / kWaves);
    }
    if (lane_id() == 0) {
        sm.wave_max[wave_id()] = wmax;
        sm.wave_kth[wave_id()] = wkth;
        if (ABOVE)
            sm.wave_above[wave_id()] = above;
    }
    __syncthreads();
    MAKO_STAMP(30);
    uint32_t mkey = 0, tau_key = 0xffffffffu, above_slice = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        mkey = max(mkey, sm.wave_max[w]);
        tau_key = min(tau_key, sm.wave_kth[w]);
        if (ABOVE)
            above_slice += sm.wave_above[w];
    }
    // first index holding the maximum
    if (bkey == mkey) {
        const float M = order_unkey(mkey);
        uint32_t first = kNone;
#pragma unroll
        for (int j = 15; j >= 0; --j)
            if (wv[j] == M)
                first = elem_index<VEC>(lo, tid, (uint32_t)j);
        if (first != kNone)
            atomicMin(&sm.argidx, first);
    }

    SliceStat st;
    st.wmax = order_unkey(mkey);
    st.flags = 0;
    st.n_emit = 0;
    st.tau_key = 0;
    st.above = above_slice;
    st.pad[0] = st.pad[1] = 0;
    // element 0 of the row is NaN: its holder raises the flag
    const bool first_nan = slice == 0 && tid == 0 && wv[0] != wv[0];
    if (first_nan)
        atomicOr(&sm.emit_flags, kFlagFirstNan);

    if (emits) {
        if (tau_key <= kKeyNegInf) {
            tau_key = kKeyNegInf;
            st.flags |= kFlagComplete;
        }
        // w >= tau and w > -inf in one compare: -inf itself is below the most negative finite float
        const float tau = fmaxf(order_unkey(tau_key), -3.402823466e38f);
        // slots in the slice's list: the wave counts its candidates, one lane reserves the wave's run with a single
        // LDS atomic, and every thread fills its part of the run (one atomic per candidate cost a round trip each)
        uint32_t mine = 0;
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j)
            mine += wv[j] >= tau ? 1u : 0u;
        const uint32_t upto = __ockl_wfscan_add_u32(mine, true);
        const uint32_t wave_total = (uint32_t)__builtin_amdgcn_readlane((int)upto, kWave - 1);
        if (wave_total) { // uniform
            uint32_t base = 0;
            if (lane_id() == 0)
                base = atomicAdd(&sm.emit_n, wave_total);
            uint32_t pos = (uint32_t)__builtin_amdgcn_readfirstlane((int)base) + upto - mine;
#pragma unroll
            for (uint32_t j = 0; j < 16; ++j) {
                const float w = wv[j];
                const bool take = w >= tau;
                if (take && pos < kCap) {
                    sm.cw[pos] = w;
                    sm.ci[pos] = elem_index<VEC>(lo, tid, j);
                }
                pos += take ? 1u : 0u;
            }
        }
    }
    __syncthreads();
    MAKO_STAMP(31);
    if (emits) {
        const uint32_t n = sm.emit_n;
        if (n > kCap)
            st.flags |= kFlagOverflow;
        st.n_emit = min(n, kCap);
        st.tau_key = tau_key;
        const size_t base = ((size_t)row * sc.slices_cap + slice) * kCap;
        if (tid < st.n_emit) {
            sc.cand_w[base + tid] = sm.cw[tid];
            sc.cand_i[base + tid] = sm.ci[tid];
        }
    }
    if (tid == 0) {
        st.argidx = sm.argidx;
        st.flags |= sm.emit_flags;
        sc.stats[(size_t)row * kMaxSlices + slice] = st;
    }
    MAKO_STAMP(27);
}

// ---------------------------------------------------------------------------------------------
// finish_kernel
// ---------------------------------------------------------------------------------------------

struct alignas(16) FinishShared {
    BlockScratch bs;
    uint64_t tab[32];
    uint32_t hist[256];
    uint32_t run[256];
    uint32_t flag;
    uint32_t ticket;
    uint32_t aux;
    uint32_t soff[kMaxSlices + 1]; // first candidate of each slice in the row's flattened candidate list
};

// Views into the 64 KB dynamic LDS block; `cnt` (first pass) overlaps the two others (second pass).
struct FinishLds {
    FinishShared* sm;
    uint32_t* cnt;              // [kSliceMax]
    unsigned long long* sortk;  // [kSortMax]
    uint32_t* wcount;           // [kWaves * 256]
};

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

// fp32 running sum of q(0..n) in order, bit-identical to `for (...) total += q` (src/gen/sampler.cpp:80-82).
template <typename QAt>
__device__ float emulate_sum(QAt qat, uint32_t n, FinishShared& sm)
{
    using namespace seqfp;
    const uint32_t tid = threadIdx.x;
    float S = qat(0);
    uint32_t i0 = 1;
    uint32_t L = 1;
    while (i0 < n) {
        uint32_t M;
        int e;
        split(S, M, e);
        const long long m = M;
        const uint32_t W = min(n - i0, (uint32_t)kThreads * L);
        const uint32_t jb = min(i0 + tid * L, i0 + W), je = min(jb + L, i0 + W);
        Step f = identity();
        for (uint32_t j = jb; j < je; ++j)
            f = compose(f, add_step(qat(j), e));
        Step total;
        const Step pre = block_excl_scan_step(f, total, sm.bs);
        long long mm = m + ((m & 1) ? pre.d1 : pre.d0);
        uint32_t hit = kNone;
        for (uint32_t j = jb; j < je; ++j) {
            const float q = qat(j);
            if (add_event(mm, q, e)) {
                hit = j;
                break;
            }
            mm = add_apply(mm, q, e);
        }
        const uint32_t first = block_min_u32(hit, sm.bs);
        if (first == kNone) {
            const long long m_end = m + ((m & 1) ? total.d1 : total.d0);
            S = join((uint32_t)m_end, e);
            i0 += W;
            L = min(L * 2u, 16u);
        } else {
            if (hit == first)
                sm.bs.bcast = (unsigned long long)mm;
            __syncthreads();
            const long long mf = (long long)sm.bs.bcast;
            __syncthreads();
            S = join((uint32_t)mf, e) + qat(first);
            i0 = first + 1;
        }
    }
    return S;
}

// Index returned by the walk of src/gen/sampler.cpp:67-72 started at r, bit-identical to the
// sequential fp32 `if (r < q) return; r -= q;` loop.
template <typename QAt>
__device__ uint32_t emulate_walk(QAt qat, uint32_t n, float r, FinishShared& sm)
{
    using namespace seqfp;
    const uint32_t tid = threadIdx.x;
    if (r < 0.0f)
        return 0;
    if (!(r == r) || r == INFINITY)
        return n - 1; // never below any q: falls through to the last candidate
    uint32_t i0 = 0;
    uint32_t L = 1;
    for (;;) {
        if (i0 >= n)
            return n - 1;
        uint32_t M;
        int e;
        split(r, M, e);
        const long long m = M;
        const uint32_t W = min(n - i0, (uint32_t)kThreads * L);
        const uint32_t jb = min(i0 + tid * L, i0 + W), je = min(jb + L, i0 + W);
        Step f = identity();
        for (uint32_t j = jb; j < je; ++j)
            f = compose(f, sub_step(qat(j), e));
        Step total;
        const Step pre = block_excl_scan_step(f, total, sm.bs);
        long long mm = m - ((m & 1) ? pre.d1 : pre.d0);
        uint32_t hit = kNone;
        bool stop = false;
        for (uint32_t j = jb; j < je; ++j) {
            const float q = qat(j);
            if (walk_stop(mm, q, e)) {
                hit = j;
                stop = true;
                break;
            }
            if (sub_event(mm, q, e)) {
                hit = j;
                break;
            }
            mm = sub_apply(mm, q, e);
        }
        const uint32_t first = block_min_u32(hit, sm.bs);
        if (first == kNone) {
            const long long m_end = m - ((m & 1) ? total.d1 : total.d0);
            r = join((uint32_t)m_end, e);
            i0 += W;
            L = min(L * 2u, 16u);
        } else {
            if (hit == first)
                sm.bs.bcast = ((unsigned long long)mm << 1) | (stop ? 1ull : 0ull);
            __syncthreads();
            const unsigned long long bc = sm.bs.bcast;
            __syncthreads();
            if (bc & 1ull)
                return first;
            r = join((uint32_t)(bc >> 1), e) - qat(first);
            i0 = first + 1;
        }
    }
}

struct RowOut {
    int32_t token;
    uint32_t n_cand;
    float total;
    float q;
    uint32_t path;
    uint32_t accepted;
    uint32_t forced = MAKO_FORCED_NONE;
};

// The row's results; with append_history also Sampler::accept of the token (src/gen/session.cpp:419-421).  Called
// once per row, by one thread, after everything that reads the row's history in this batch.
__device__ __forceinline__ void write_row(const mako_sample_desc& d, uint32_t row, const RowOut& o)
{
    d.out_tokens[row] = o.token;
    if (d.out_forced)
        d.out_forced[row] = (uint8_t)o.forced;
    if (d.append_history) {
        uint32_t* hl = const_cast<uint32_t*>(d.hist_len);
        const uint32_t len = hl[row];
        if (len < (uint32_t)d.hist_stride) {
            const_cast<int32_t*>(d.hist_tokens)[(int64_t)row * d.hist_stride + len] = o.token;
            hl[row] = len + 1u;
        }
    }
    if (d.out_n_cand)
        d.out_n_cand[row] = o.n_cand;
    if (d.out_total)
        d.out_total[row] = o.total;
    if (d.out_q)
        d.out_q[row] = o.q;
    if (d.out_path)
        d.out_path[row] = (uint8_t)o.path;
    if (d.out_accepted)
        d.out_accepted[row] = (uint8_t)o.accepted;
}

// No candidate survived (src/gen/sampler.cpp:37-38): the single candidate (1.0f, first max).
__device__ void fallback_row(const mako_sample_desc& d, uint32_t row, uint32_t argidx)
{
    if (threadIdx.x != 0)
        return;
    RowOut o;
    o.token = (int32_t)argidx;
    o.n_cand = 1;
    o.total = 1.0f;
    o.q = 1.0f;
    o.path = MAKO_PATH_FALLBACK;
    // verifying: u * 1 < 1 accepts the draft iff it is that candidate; otherwise it is the only one left
    o.accepted = d.draft ? (d.draft[row] == (int32_t)argidx) : 0u;
    if (d.out_cand_idx && d.out_cand_q && d.cand_cap) {
        d.out_cand_idx[(size_t)row * d.cand_cap] = (int32_t)argidx;
        d.out_cand_q[(size_t)row * d.cand_cap] = 1.0f;
    }
    write_row(d, row, o);
}

// The draw (and, when verifying, the accept/reject step) over the final candidate list of n entries with
// weights qat(i) and token ids idat(i).  src/gen/sampler.cpp:64-73, 79-83, 93-106.
template <typename QAt, typename IdAt>
__device__ void draw_from_list(const mako_sample_desc& d, uint32_t row, QAt qat, IdAt idat, uint32_t n, uint32_t path,
                               FinishShared& sm)
{
    const uint32_t tid = threadIdx.x;
    const float total = emulate_sum(qat, n, sm);
    const float u = d.u[row];
    RowOut o;
    o.n_cand = n;
    o.total = total;
    o.path = path;
    o.accepted = 0;
    if (d.out_cand_idx && d.out_cand_q)
        for (uint32_t j = tid; j < n && j < d.cand_cap; j += kThreads) {
            d.out_cand_idx[(size_t)row * d.cand_cap + j] = (int32_t)idat(j);
            d.out_cand_q[(size_t)row * d.cand_cap + j] = qat(j);
        }
    if (!d.draft) {
        const float span = total - 0.0f;
        const float prod = u * span;
        const uint32_t pos = emulate_walk(qat, n, prod + 0.0f, sm);
        o.token = (int32_t)idat(pos);
        o.q = qat(pos);
    } else {
        // position of the draft in the list, if it survived the truncation
        const int32_t draft = d.draft[row];
        uint32_t pd = kNone;
        for (uint32_t j = tid; j < n; j += kThreads)
            if ((int32_t)idat(j) == draft)
                pd = j;
        pd = block_min_u32(pd, sm.bs);
        const float q_draft = pd == kNone ? 0.0f : qat(pd);
        const float span = total - 0.0f;
        const float prod = u * span;
        const float r1 = prod + 0.0f;
        o.accepted = r1 < q_draft;
        o.token = draft;
        o.q = q_draft;
        const uint32_t n2 = pd == kNone ? n : n - 1;
        if (!o.accepted && n2 > 0) {
            auto qat2 = [&](uint32_t i) { return qat(i + (i >= pd ? 1u : 0u)); };
            const float rest = total - q_draft;
            const float span2 = rest - 0.0f;
            const float prod2 = d.u2[row] * span2;
            const uint32_t pos = emulate_walk(qat2, n2, prod2 + 0.0f, sm);
            const uint32_t at = pos + (pos >= pd ? 1u : 0u);
            o.token = (int32_t)idat(at);
            o.q = qat(at);
        }
    }
    if (tid == 0)
        write_row(d, row, o);
}

// ---------------------------------------------------------------------------------------------
// sorted lists: top-p cut, exact fp32 total and walk, in groups of 256 (see seqfp.h, "groups")
// ---------------------------------------------------------------------------------------------

constexpr uint32_t kWalkSeqGroups = 8; // a walk expected to end within this many groups goes entry by entry from LDS
struct GroupLds { // carved from the dynamic LDS block once sorting is over; one pointer, the rest is offsets
    unsigned long long* base;
    __device__ __forceinline__ double* pg() const { return reinterpret_cast<double*>(base); } // [kMaxGroups + 2] fp64 sum of the entries before each group
    __device__ __forceinline__ uint32_t* d0() const { return reinterpret_cast<uint32_t*>(base + kMaxGroups + 2); } // [kMaxGroups] the group's map for the guessed epoch
    __device__ __forceinline__ uint32_t* d1() const { return d0() + kMaxGroups; }
    __device__ __forceinline__ uint32_t* cmax() const { return d1() + kMaxGroups; }
    __device__ __forceinline__ uint32_t* start() const { return cmax() + kMaxGroups; } // first entry of the group
    // entries (bits 0-8) | quarter-record slot + 1 (bits 9-15) | guessed exponent << 16
    __device__ __forceinline__ uint32_t* pack() const { return start() + kMaxGroups; }
    __device__ __forceinline__ uint32_t* misc() const { return pack() + kMaxGroups; } // [4]; misc[3] counts the quarter-record slots in use
    // [kQuarterSlots][4], in the upper half of the dynamic LDS block
    __device__ __forceinline__ uint4* quarters() const { return reinterpret_cast<uint4*>(base + kSortMax); }
    // the walk's maps, bounds and packs ([kMaxGroups] each, behind the quarter records): built while the running
    // sum is still being chained, so they cannot share the arrays above
    __device__ __forceinline__ uint32_t* w_d0() const { return reinterpret_cast<uint32_t*>(base + kSortMax) + 1536; }
    __device__ __forceinline__ uint32_t* w_d1() const { return w_d0() + kMaxGroups; }
    __device__ __forceinline__ uint32_t* w_need() const { return w_d1() + kMaxGroups; }
    __device__ __forceinline__ uint32_t* w_pack() const { return w_need() + kMaxGroups; }
    // [kWalkSeqGroups * kGroup + kWave] the head of the list as floats, for a walk that ends within it
    __device__ __forceinline__ float* head() const { return reinterpret_cast<float*>(w_pack() + kMaxGroups); }
};
constexpr uint32_t kLenMask = 0x1ffu;
constexpr uint32_t kHasQuarters = 1u << 31;
constexpr uint32_t kQuarterSlots = 96;
constexpr uint32_t kQuarter = kGroup / 4;
constexpr uint32_t kSeqMax = 1024; // sorted lists up to this long get their total and walk entry by entry

__device__ __forceinline__ GroupLds group_lds(const FinishLds& L)
{
    static_assert((kMaxGroups + 2) * 8 + 5 * kMaxGroups * 4 + 16 <= kSortMax * 8, "group records fit below the LDS lists");
    static_assert(kQuarterSlots * 16 == 1536 &&
                      kSortMax * 8 + 1536 * 4 + 4 * kMaxGroups * 4 + (kWalkSeqGroups * kGroup + kWave) * 4 <= kDynLds,
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

// Composition of the 64 lanes' maps in lane order; every lane receives the result.
__device__ __forceinline__ seqfp::Step32 wave_compose_step32(seqfp::Step32 v)
{
    wave_scan_maps(v.d0, v.d1);
    seqfp::Step32 r;
    r.d0 = (uint32_t)__builtin_amdgcn_readlane((int)v.d0, kWave - 1);
    r.d1 = (uint32_t)__builtin_amdgcn_readlane((int)v.d1, kWave - 1);
    r.cmax = __ockl_wfred_max_u32(v.cmax);
    return r;
}

// The map of one span for the epoch with exponent eg (eg == 0: no usable guess, the map is marked unusable).
__device__ __forceinline__ seqfp::Step32 span_map(const float (&q)[4], uint32_t len, int eg)
{
    using namespace seqfp;
    Step32 st = Step32{kSat, kSat, kSat};
    if (eg > 0) { // uniform per wave
        st = identity32();
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            if (lane_id() * 4u + j < len)
                st = compose32(st, step32(q[j], eg));
        st = wave_compose_step32(st);
    }
    return st;
}

// A group inside which the running sum is expected to change binade cannot be applied as one map.  Its four
// quarters (64 entries = the 16 lanes of one DPP row each) get maps of their own, each for the binade guessed from
// the fp64 sum up to ITS first entry: the chain then replays only the quarter in which the change happens.
// `at_start` is the estimate of the sum at the group's first entry.  One wave; the four records (d0, d1, cmax,
// exponent) go to out[0..3].
__device__ void build_quarters(const float (&q)[4], uint32_t len, double at_start, uint4* out)
{
    using namespace seqfp;
    const uint32_t lane = lane_id(), quarter = lane >> 4;
    double rs = (((double)q[0] + (double)q[1]) + (double)q[2]) + (double)q[3];
    for (int o = 1; o < 16; o <<= 1)
        rs += __shfl_xor(rs, o);
    const double s0 = __shfl(rs, 0), s1 = __shfl(rs, 16), s2 = __shfl(rs, 32);
    const double before = quarter == 0 ? 0.0 : (quarter == 1 ? s0 : (quarter == 2 ? s0 + s1 : (s0 + s1) + s2));
    const double guess = at_start + before;
    const int eg = guess > 0 ? exponent_of((float)guess) : 0;
    Step32 v = Step32{kSat, kSat, kSat};
    if (eg > 0) {
        v = identity32();
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            if (lane * 4u + j < len)
                v = compose32(v, step32(q[j], eg));
    }
    uint32_t cm = v.cmax;
    for (int o = 1; o < 16; o <<= 1)
        cm = max(cm, (uint32_t)__shfl_xor((int)cm, o));
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

// Group maps of groups [0, groups) for epochs guessed from pg: of the running sum (walk == false, into G.d0 / d1 /
// cmax / pack) or of the walk from r0 (into G.w_d0 / w_d1 / w_need / w_pack).  The calling wave is number `part` of
// `parts` that share the work.
template <typename Keys>
__device__ void build_group_maps(Keys kf, uint32_t groups, bool walk, double r0, const GroupLds G,
                                 uint32_t part = wave_id(), uint32_t parts = kWaves)
{
    using namespace seqfp;
    uint32_t* const o_d0 = walk ? G.w_d0() : G.d0();
    uint32_t* const o_d1 = walk ? G.w_d1() : G.d1();
    uint32_t* const o_c = walk ? G.w_need() : G.cmax();
    uint32_t* const o_pack = walk ? G.w_pack() : G.pack();
    // Up to four groups per trip and wave, their loads issued together; a wave's groups lie `parts` apart, so that a
    // short list is spread over all the waves (a map costs a wave about a microsecond).
    for (uint32_t g0 = part; g0 < groups; g0 += parts * 4u) {
        float q[4][4];
        uint32_t len[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint32_t g = min(g0 + u * parts, groups - 1u);
            len[u] = uniform_u32(G.pack()[g] & kLenMask);
            load_span(kf, uniform_u32(G.start()[g]), len[u], q[u]);
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint32_t g = g0 + u * parts;
            if (g >= groups) // uniform
                break;
            const double guess = g < groups ? (walk ? r0 - G.pg()[g] : G.pg()[g]) : 0.0;
            const int eg = guess > 0 ? exponent_of((float)guess) : 0;
            const Step32 st = span_map(q[u], len[u], eg);
            // a group in which the running sum is expected to change binade (or starts from zero) gets quarter
            // records; the walk replays such groups whole
            uint32_t slot = 0;
            if (!walk && g < groups) { // uniform
                const double at_end = G.pg()[g + 1];
                const int e_end = at_end > 0 ? exponent_of((float)at_end) : 0;
                if (uniform_u32((uint32_t)(e_end != eg)) || g == 0) {
                    if (lane_id() == 0)
                        slot = atomicAdd(&G.misc()[3], 1u) + 1u;
                    slot = uniform_u32(slot);
                    if (slot > kQuarterSlots)
                        slot = 0;
                    else
                        build_quarters(q[u], len[u], G.pg()[g], G.quarters() + (slot - 1u) * 4u);
                }
            }
            if (lane_id() == 0 && g < groups) {
                uint32_t third = st.cmax;
                if (walk) {
                    // group_sub_ok as one bound (lane 0 holds the group's first, largest weight): the state after
                    // the group must be at least `third`, which keeps it inside the binade with room for one
                    // more decrement and at or above that weight, so that nothing in the group stopped the walk
                    uint32_t Mq;
                    int eq;
                    split(q[u][0], Mq, eq);
                    const int dl = eg - eq;
                    third = 1u;
                    if (dl < 0)
                        third = 1u << 31;
                    else if (dl <= 25)
                        third = max(1u, (uint32_t)(((unsigned long long)Mq + (1ull << dl) - 1ull) >> dl));
                    if (eg > 1)
                        third = max(third, min(st.cmax, 1u << 30) + (1u << 23) + 1u);
                }
                o_d0[g] = st.d0;
                o_d1[g] = st.d1;
                o_c[g] = third;
                o_pack[g] = len[u] | (slot << 9) | ((uint32_t)eg << 16);
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
// wave reads the same four entries with one broadcast load and subtracts them in turn, three nanoseconds an entry
// (the travelling chain of walk_lanes() takes five).  Blocks of 64 blind, then of 16, then entry by entry, as there.
// Returns true and the position when the walk stops, else false and the new r.
__device__ __forceinline__ bool walk_lds(const float* sx, uint32_t n, float& r, uint32_t& pos)
{
    float v = r;
    uint32_t base = 0;
    for (; base + kWave <= n; base += kWave) {
        const float4* p = reinterpret_cast<const float4*>(sx + base);
        float t = v;
#pragma unroll
        for (uint32_t i = 0; i < kWave / 4u; ++i) {
            const float4 x = p[i];
            t -= x.x;
            t -= x.y;
            t -= x.z;
            t -= x.w;
        }
        if (__ballot(t < 0.0f) != 0ull)
            break; // the walk stops in this block: found below
        v = t;
    }
    for (; base + 16u <= n; base += 16u) {
        const float4* p = reinterpret_cast<const float4*>(sx + base);
        float t = v;
#pragma unroll
        for (uint32_t i = 0; i < 4u; ++i) {
            const float4 x = p[i];
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
__device__ __forceinline__ float sum_lds(const float* sx, uint32_t n, float S)
{
    uint32_t base = 0;
    for (; base + 16u <= n; base += 16u) {
        const float4* p = reinterpret_cast<const float4*>(sx + base);
#pragma unroll
        for (uint32_t i = 0; i < 4u; ++i) {
            const float4 x = p[i];
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

// Tail of every path that ends with a list sorted by (q desc, idx asc): kf[i] = ~bits(q_i), jf[i] = token id,
// n1 entries (already cut to top_k).  Applies top-p (src/gen/sampler.cpp:44-61) against total64 (the fp64 sum over
// the row's candidates; summed from the list when !have_total), then the exact fp32 total (:80-82) and walk
// (:64-73).  All 1024 threads must call it.
//
// When `need_cut` the list is only the heaviest part of the row's candidates and every candidate missing from
// it weighs at most q_bound: the nucleus must then end inside the list, at an entry strictly heavier than
// q_bound.  If it does not, nothing is written and false is returned (the caller widens the list).
//
// `T` (with `t_groups` records at `t_base`) describes a list whose groups were prepared by sort_kernel's workers;
// without it the list is cut into groups of kGroup here.
// SHORT_ONLY: the caller's lists never exceed kGroup entries; the code for longer ones is left out.
template <bool PLANNED = false, bool SHORT_ONLY = false>
__device__ bool sorted_tail(const mako_sample_desc& d, uint32_t row, const mako_sampling_params& P, const uint32_t* kf_ptr,
                            const uint32_t* jf, uint32_t n1_arg, bool have_total, double total64, uint32_t path,
                            const FinishLds& L, bool need_cut = false, float q_bound = 0.0f, const GroupTable& T = GroupTable{},
                            size_t t_base = 0, uint32_t t_groups = 0)
{
    using namespace seqfp;
    // (a planned row's list is in device memory; the other callers may hand over a list in LDS)
    const typename std::conditional<PLANNED, GlobalKeys, AnyKeys>::type kf{kf_ptr};
    const float u_row = d.u[row]; // (asked for here, wanted much later)
    const uint32_t n1 = uniform_u32(n1_arg);
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
    auto qat = [=](uint32_t i) { return __uint_as_float(~kf[i]); };
    auto idat = [=](uint32_t i) { return jf[i]; };
    const GroupLds G = group_lds(L);
    const bool topp_active = P.top_p < 1.0f;
    if (d.draft || (!PLANNED && n1 > kGroup * kMaxGroups)) {
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
            double carry = 0;
            uint32_t keep = kNone;
            for (uint32_t base = 0; base < n; base += kThreads) {
                const uint32_t i = base + tid;
                const double q = i < n ? (double)qat(i) : 0.0;
                double tile;
                const double incl = carry + block_incl_scan_f64(q, tile, sm.bs);
                const uint32_t hit = (i < n && incl >= want) ? i : kNone;
                const uint32_t first = block_min_u32(hit, sm.bs);
                if (first != kNone) {
                    keep = first + 1;
                    break;
                }
                carry += tile;
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
            if (topp_active) {
                const double want = (double)P.top_p * total64;
                const double base = incl - p[3];
                uint32_t hit = kNone;
#pragma unroll
                for (int j = 3; j >= 0; --j)
                    if (base + p[j] >= want)
                        hit = lane_id() * 4u + (uint32_t)j;
                const unsigned long long bal = __ballot(hit != kNone && hit < n1);
                if (bal)
                    n = (uint32_t)__builtin_amdgcn_readlane((int)hit, __ffsll((long long)bal) - 1) + 1u;
                else
                    ok = !need_cut;
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
    if (tid == 0)
        G.misc()[3] = 0;
    // The head of the list as floats in LDS (loads set out now, wanted after the cut): where the running sum and
    // the walk change binade every few entries, both go through it entry by entry.
    constexpr uint32_t kHead = kWalkSeqGroups * kGroup;
    {
        uint32_t raw[kHead / kThreads];
#pragma unroll
        for (uint32_t t = 0; t < kHead / kThreads; ++t)
            raw[t] = kf[min(t * kThreads + tid, n1 - 1u)];
#pragma unroll
        for (uint32_t t = 0; t < kHead / kThreads; ++t)
            G.head()[t * kThreads + tid] = __uint_as_float(~raw[t] & (t * kThreads + tid < n1 ? 0xffffffffu : 0u));
        if (tid < kWave)
            G.head()[kHead + tid] = 0.0f;
    }
    __syncthreads();
    if constexpr (PLANNED) {
        if (tid < groups1) {
            G.pg()[tid + 1] = T.sum[t_base + tid];
            G.d0()[tid] = T.d0[t_base + tid];
            G.d1()[tid] = T.d1[t_base + tid];
            G.cmax()[tid] = T.cmax[t_base + tid];
            // (clamped into the list: a record is only ever read, never trusted for addressing)
            const uint32_t st = min(T.start[t_base + tid], n1), pk = T.pack[t_base + tid];
            // (the quarter records are asked for together with the rest, whether or not the group has any: asking
            // only once `pk` is known would be one more trip to memory for every row)
            const uint4* tq = T.quarters + (t_base + tid) * 4u;
            const uint4 qr0 = tq[0], qr1 = tq[1], qr2 = tq[2], qr3 = tq[3];
            uint32_t slot = 0;
            if (pk & kHasQuarters) {
                slot = atomicAdd(&G.misc()[3], 1u) + 1u;
                if (slot > kQuarterSlots)
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
            G.pack()[tid] = min(pk & kLenMask, min(kGroup, n1 - st)) | (slot << 9) | (pk & 0x00ff0000u);
        }
    } else {
        if (tid < groups1) {
            G.start()[tid] = tid * kGroup;
            G.pack()[tid] = min(kGroup, n1 - tid * kGroup);
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
        const uint32_t hitg = (tid < groups1 && G.pg()[tid + 1] >= want) ? tid : kNone;
        const uint32_t gs = block_min_u32(hitg, sm.bs);
        if (need_cut && gs == kNone)
            return false;
        if (gs != kNone) {
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
#pragma unroll
                for (int j = 3; j >= 0; --j)
                    if (base + p[j] >= want)
                        hit = lane_id() * 4u + (uint32_t)j;
                const unsigned long long bal = __ballot(hit != kNone && hit < len);
                uint32_t keep = len;
                if (bal)
                    keep = (uint32_t)__builtin_amdgcn_readlane((int)hit, __ffsll((long long)bal) - 1) + 1u;
                if (lane_id() == 0) {
                    G.misc()[0] = st + keep;
                    if (keep != len)
                        G.pack()[gs] = keep; // shortened: the prepared map no longer applies (exponent 0)
                }
            }
            __syncthreads();
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
            o.path = path;
            o.accepted = 0;
            write_row(d, row, o);
        }
    };

    MAKO_STAMP(7);
    if (n <= kSeqMax) {
        // A nucleus this short is copied to LDS and gone through entry by entry, once for the total and once for the
        // walk (three nanoseconds an entry each way): the group maps below only pay on longer lists.
        if (wave_id() == 0) {
            const float S = sum_lds(G.head(), n, 0.0f);
            const float span = S - 0.0f;
            const float prod = u_row * span;
            const float r0 = prod + 0.0f;
            uint32_t at = n - 1;
            if (r0 < 0.0f) {
                at = 0;
            } else if (r0 == r0 && r0 != INFINITY) {
                float r = r0;
                walk_lds(G.head(), n, r, at);
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
    if (!PLANNED)
        build_group_maps(kf, groups, false, 0.0, G);
    __syncthreads();
    MAKO_STAMP(13);
    // While one wave chains the running sum, the others already prepare the walk: its maps only need the binade r is
    // expected to be in at each group, and the fp64 sums give that (a wrong guess costs a replay, never the result).
    // Groups that start after the mass r0 could have is used up get no map.
    const double r0_guess = (double)u_row * G.pg()[groups];
    uint32_t reach;
    {
        const uint32_t beyond = (tid < groups && !(r0_guess * 1.001 - G.pg()[tid] > 0)) ? tid : kNone;
        reach = min(groups, block_min_u32(beyond, sm.bs));
        if (tid < groups)
            G.w_pack()[tid] = G.pack()[tid] & kLenMask;
        __syncthreads();
    }
#ifdef MAKO_TIMING
    if (tid == 0 && s_mako_row == 0) {
        g_mako_stamp[20] = groups;
        g_mako_stamp[21] = reach;
        g_mako_stamp[22] = n;
    }
    const unsigned long long tb0 = wall_clock64();
#endif
    // A walk that will end within a few groups goes through them entry by entry, from a copy in LDS: faster than
    // the groups' maps would be to build.
    const bool head_walk = reach <= kWalkSeqGroups; // uniform
    const uint32_t head_n = !head_walk ? 0u : (reach == groups ? n : uniform_u32(G.start()[reach]));
    if (wave_id() != 0 && (wave_id() & 3) != 0 && r0_guess == r0_guess && !head_walk) {
        // (the waves that do not share a SIMD with the chaining wave: 1, 2, 3, 5, 6, 7, ...)
        build_group_maps(kf, reach, true, r0_guess, G, (uint32_t)(wave_id() >> 2) * 3u + (uint32_t)(wave_id() & 3) - 1u,
                         3u * kWaves / 4u);
#ifdef MAKO_TIMING
        if (tid == 64 && s_mako_row == 0)
            g_mako_stamp[23] = wall_clock64() - tb0;
#endif
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
                const float S = sum_lds(G.head(), min(hs, kHead), 0.0f);
                uint32_t Mv;
                int ev;
                split(S, Mv, ev);
                M = uniform_u32(Mv);
                e = (int)uniform_u32((uint32_t)ev);
            }
        }
        MAKO_TOC(0, 17);
#ifdef MAKO_TIMING
        if (lane_id() == 0)
            g_mako_stamp[19] = first;
#endif
        MAKO_TIC(1);
        for (uint32_t base = 0; base < groups; base += kWave) {
            const uint32_t gl = min(base + lane_id(), groups - 1u);
            const uint32_t pk_l = G.pack()[gl], st_l = G.start()[gl];
            const uint32_t d0_l = G.d0()[gl], d1_l = G.d1()[gl], cm_l = G.cmax()[gl];
            const uint32_t cnt = min((uint32_t)kWave, groups - base);
            uint32_t done = base == 0 ? first : 0u; // (first <= kWalkSeqGroups)
            while (done < cnt) {
                const bool live = lane_id() >= done && lane_id() < cnt;
                const bool same = live && (pk_l >> 16) == (uint32_t)e;
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
#ifdef MAKO_TIMING
                    if (lane_id() == 0)
                        g_mako_stamp[21] += 1;
#endif
                    const uint32_t slot = (pk >> 9) & 0x7fu;
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
            G.misc()[1] = __float_as_uint(join(M, e));
    }
    __syncthreads();
    MAKO_STAMP(8);
    const float total = __uint_as_float(G.misc()[1]);
    const float span = total - 0.0f;
    const float prod = u_row * span;
    const float r0 = prod + 0.0f;
    __syncthreads();

    // exact walk
    uint32_t pos = n - 1;
    if (r0 < 0.0f) {
        pos = 0;
    } else if (r0 == r0 && r0 != INFINITY) {
        MAKO_STAMP(14);
        if (wave_id() == 0) {
            uint32_t M;
            int e;
            {
                uint32_t Mv;
                int ev;
                split(r0, Mv, ev);
                M = uniform_u32(Mv);
                e = (int)uniform_u32((uint32_t)ev);
            }
            uint32_t at = n - 1;
            bool stopped = false;
            uint32_t first = 0; // groups already walked
            if (head_walk && head_n) {
                float r = r0;
                stopped = walk_lds(G.head(), head_n, r, at);
                uint32_t Mv;
                int ev;
                split(r, Mv, ev);
                M = uniform_u32(Mv);
                e = (int)uniform_u32((uint32_t)ev);
                first = reach;
            }
            for (uint32_t base = 0; base < groups && !stopped; base += kWave) {
                const uint32_t gl = min(base + lane_id(), groups - 1u);
                const uint32_t pk_l = G.w_pack()[gl], st_l = G.start()[gl];
                const uint32_t d0_l = G.w_d0()[gl], d1_l = G.w_d1()[gl], need_l = G.w_need()[gl]; // (the bound, see build_group_maps)
                const uint32_t cnt = min((uint32_t)kWave, groups - base);
                uint32_t done = base == 0 ? first : 0u; // (first <= kWalkSeqGroups)
                while (done < cnt) {
                    MAKO_COUNT(30, 1);
                    const bool live = lane_id() >= done && lane_id() < cnt;
                    const bool same = live && (pk_l >> 16) == (uint32_t)e;
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
                    // and the scan takes over again once four in a row have gone through as maps.
                    uint32_t g = f, passed = 0;
                    uint32_t raw[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu}; // the entries of group g
                    {
                        const uint32_t st = (uint32_t)__builtin_amdgcn_readlane((int)st_l, g);
                        const uint32_t pk = (uint32_t)__builtin_amdgcn_readlane((int)pk_l, g);
                        if (pk & kLenMask)
                            fetch_span_lanes(kf, st, pk & kLenMask, raw);
                    }
                    while (g < cnt && passed < 4u) {
                        const uint32_t st = (uint32_t)__builtin_amdgcn_readlane((int)st_l, g);
                        const uint32_t pk = (uint32_t)__builtin_amdgcn_readlane((int)pk_l, g);
                        float xa[4];
                        take_span_lanes(raw, pk & kLenMask, xa);
                        // (the next group's entries set out now; they are used only if that group is replayed too)
                        const uint32_t g1 = min(g + 1u, cnt - 1u);
                        const uint32_t st1 = (uint32_t)__builtin_amdgcn_readlane((int)st_l, g1);
                        const uint32_t pk1 = (uint32_t)__builtin_amdgcn_readlane((int)pk_l, g1);
                        if (pk1 & kLenMask)
                            fetch_span_lanes(kf, st1, pk1 & kLenMask, raw);
                        bool by_map = false;
                        if (g != f && (pk >> 16) == (uint32_t)e) {
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
                        } else {
                            MAKO_COUNT(22, 1);
                            passed = 0;
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
                        ++g;
                    }
                    if (stopped)
                        break;
                    done = g;
                }
            }
            if (lane_id() == 0)
                G.misc()[2] = at;
        }
        __syncthreads();
        pos = G.misc()[2];
    }

    MAKO_STAMP(9);
    emit(total, pos);
    return true;
}

__device__ void sort_segment(uint32_t* k0, uint32_t* i0, uint32_t* k1, uint32_t* i1, uint32_t n, const FinishLds& L);

// std::ranges::nth_element(cand, cand + nth, desc) of src/gen/sampler.cpp:41 as libstdc++ 11 runs it (introselect,
// bits/stl_algo.h:1964), leaving the candidates in exactly the arrangement that library leaves: the reference sums
// and walks the top_k survivors in that order when no top-p follows.  key/idx hold n candidates (~bits(q), token
// id); `desc` is the order of the 64-bit values key << 32 | idx, all distinct.
// One round = median of three to the front, then the unguarded Hoare partition of the rest around it.  That
// partition swaps the t-th entry from the left that belongs right with the t-th entry from the right that belongs
// left for as long as the former lies before the latter, and cuts behind the entries that belong left: the two
// position lists come from ballots (wave w owns the w-th sixteenth of the range), the swaps are independent.
// The depth limit's heap select and the last insertion sort (at most three entries) are sequential code on one
// thread.
//
// introselect_rounds runs the rounds on [first, last) through get(i) / put(i, v) until the range is no longer than
// `until` (3 = to the end, insertion sort included).  lsta / lstb: room for last - first positions each.  Returns
// true when nothing is left to do.
template <typename Get, typename Put>
__device__ bool introselect_rounds(Get get, Put put, uint32_t& first, uint32_t& last, uint32_t nth, uint32_t& depth,
                                   uint32_t until, uint32_t* lsta, uint32_t* lstb, FinishShared& sm)
{
    typedef unsigned long long u64;
    const uint32_t tid = threadIdx.x, lane = lane_id(), wave = wave_id();
    while (last - first > until) {
        if (depth == 0) {
            // __heap_select(first, nth + 1, last) and iter_swap(first, nth): bits/stl_algo.h:1956-1960, stl_heap.h
            if (tid == 0) {
                const uint32_t middle = nth + 1u - first, len = last - first;
                auto sift = [&](uint32_t hole, u64 v) { // __adjust_heap: the hole sinks to a leaf, v rises from there
                    const uint32_t top = hole;
                    uint32_t child = hole;
                    while (child < (middle - 1u) / 2u) {
                        child = 2u * (child + 1u);
                        if (get(first + child) < get(first + child - 1u))
                            --child;
                        put(first + hole, get(first + child));
                        hole = child;
                    }
                    if ((middle & 1u) == 0 && middle >= 2u && child == (middle - 2u) / 2u) {
                        child = 2u * (child + 1u);
                        put(first + hole, get(first + child - 1u));
                        hole = child - 1u;
                    }
                    while (hole > top) {
                        const uint32_t parent = (hole - 1u) / 2u;
                        if (!(get(first + parent) < v))
                            break;
                        put(first + hole, get(first + parent));
                        hole = parent;
                    }
                    put(first + hole, v);
                };
                if (middle >= 2u)
                    for (uint32_t parent = (middle - 2u) / 2u;; --parent) {
                        sift(parent, get(first + parent));
                        if (parent == 0)
                            break;
                    }
                for (uint32_t i = middle; i < len; ++i) {
                    const u64 v = get(first + i);
                    if (v < get(first)) {
                        put(first + i, get(first));
                        sift(0u, v);
                    }
                }
                const u64 a = get(first), b = get(nth);
                put(first, b);
                put(nth, a);
            }
            __syncthreads();
            return true;
        }
        --depth;
        if (tid == 0) { // __move_median_to_first(first, first + 1, mid, last - 1)
            const uint32_t ix = first + 1u, iy = first + (last - first) / 2u, iz = last - 1u;
            const u64 x = get(ix), y = get(iy), z = get(iz);
            uint32_t im;
            if (x < y)
                im = y < z ? iy : (x < z ? iz : ix);
            else
                im = x < z ? ix : (y < z ? iz : iy);
            const u64 r = get(first), med = get(im);
            put(first, med);
            put(im, r);
        }
        __syncthreads();
        const u64 pivot = get(first);
        const uint32_t lo0 = first + 1u, len = last - lo0;
        const uint32_t chunk = ((len + kThreads - 1u) / kThreads) * kWave; // per wave, a multiple of 64
        const uint32_t beg = min(last, lo0 + wave * chunk), end = min(last, beg + chunk);
        // entries of the wave's chunk that belong left of the cut
        // (kTrip loads in flight per lane: a trip costs one round trip to memory, not kTrip)
        constexpr uint32_t kTrip = 4;
        uint32_t mine = 0;
        for (uint32_t base = beg; base < end; base += kWave * kTrip) {
            u64 v[kTrip];
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u)
                v[u] = get(min(base + u * kWave + lane, last - 1u));
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u)
                mine += (uint32_t)__popcll(__ballot(base + u * kWave + lane < end && v[u] < pivot));
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
        const uint32_t bigs = len - smalls;
        uint32_t big_before = (beg - lo0) - small_before;
        // position lists: lsta[t] = the t-th big entry from the left, lstb[t] = the t-th small entry from the left
        const u64 lower = (1ull << lane) - 1ull;
        for (uint32_t base = beg; base < end; base += kWave * kTrip) {
            u64 v[kTrip];
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u)
                v[u] = get(min(base + u * kWave + lane, last - 1u));
#pragma unroll
            for (uint32_t u = 0; u < kTrip; ++u) {
                const uint32_t pos = base + u * kWave + lane;
                const bool in = pos < end;
                const bool small = in && v[u] < pivot;
                const u64 bs = __ballot(small), bb = __ballot(in && !small);
                if (small)
                    lstb[small_before + (uint32_t)__popcll(bs & lower)] = pos;
                else if (in)
                    lsta[big_before + (uint32_t)__popcll(bb & lower)] = pos;
                small_before += (uint32_t)__popcll(bs);
                big_before += (uint32_t)__popcll(bb);
            }
        }
        __syncthreads();
        const uint32_t pairs = min(bigs, smalls);
        for (uint32_t t = tid; t < pairs; t += kThreads) {
            const uint32_t a = lsta[t], b = lstb[smalls - 1u - t];
            if (a < b) {
                const u64 va = get(a), vb = get(b);
                put(a, vb);
                put(b, va);
            }
        }
        __syncthreads();
        const uint32_t cut = lo0 + smalls;
        if (cut <= nth)
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
    if (introselect_rounds(get, put, first, last, nth, depth, kSortMax, lsta, lstb, *L.sm))
        return;
    u64* lds = L.sortk;
    uint32_t* la = reinterpret_cast<uint32_t*>(L.sortk + kSortMax);
    uint32_t* lb = la + kSortMax;
    static_assert(kSortMax * 16u <= kDynLds, "the range and its two position lists fit the dynamic LDS block");
    const uint32_t base = first, len = last - first;
    for (uint32_t i = tid; i < len; i += kThreads)
        lds[i] = get(base + i);
    __syncthreads();
    introselect_rounds([=](uint32_t i) { return lds[i - base]; }, [=](uint32_t i, u64 v) { lds[i - base] = v; }, first, last,
                       nth, depth, 3u, la, lb, *L.sm);
    for (uint32_t i = tid; i < len; i += kThreads)
        put(base + i, lds[i]);
    __syncthreads();
}

// Common tail of the whole-row paths.  key[0]/idx[0] of the row hold n0 candidates (~bits(q), token id) in index
// order.  Sorts them by (q desc, idx asc) when top-k or top-p is active, truncates (src/gen/sampler.cpp:39-61)
// and draws.  `total64` (when have_total) is the fp64 sum of q over all candidates of the row, of which the list
// may be only the heaviest part; otherwise it is summed from the list.
// (TOPK_ALONE = false leaves the top-k-without-top-p branch out of the instance inside plan_kernel<true>: that kernel is
// only launched for batches whose host copy of the parameters shows a top-p on every sampled row, and the branch's
// registers would be spilled around the top-k rows' fast path, +3.5 us on a 256-row batch.)
template <bool TOPK_ALONE>
__device__ void sort_truncate_draw(const mako_sample_desc& d, const Scratch& sc, uint32_t row, const mako_sampling_params& P,
                                   uint32_t n0, bool have_total, double total64, uint32_t path, const FinishLds& L)
{
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
    else if (topk_active || topp_active)
        sort_segment(key0, idx0, key1, idx1, n0, L);
    const uint32_t *ks = key0, *is = idx0;
    MAKO_STAMP(12);
    const uint32_t n1 = topk_active ? P.top_k : n0; // sampler.cpp:40-43
    // (sorted_tail's one-wave path for lists of up to kGroup entries adds and walks them in the order given, whatever
    // it is, and without a top-p it cuts nothing: nth_element's survivors take it too)
    if (nth_order ? (!d.draft && n1 <= kGroup) : (topk_active || topp_active)) {
        sorted_tail(d, row, P, ks, is, n1, have_total, total64, path, L);
        return;
    }
    // nth_element's order (long lists, verification), or neither top-k nor top-p: the candidates stay in index order
    const uint32_t* kf = ks;
    const uint32_t* jf = is;
    draw_from_list(
        d, row, [=](uint32_t i) { return __uint_as_float(~kf[i]); }, [=](uint32_t i) { return jf[i]; }, n1, path, sm);
}

// Plans a top_k == 0 row from the histogram of its weights (weight_bin(), exact masses): finds the bin by
// which the nucleus must have ended and splits the weights above it over kWorkers workers by value.
// Thread t brings the counts (c0, c1) and significand sums (s0, s1) of bins kBins-1-2t and kBins-2-2t.
// Returns n0, the number of weights to sort; the plan is written to `plan` (flag left untouched).
__device__ uint32_t plan_nucleus(const mako_sampling_params& P, double total64, uint32_t c0, uint32_t c1,
                                 unsigned long long s0, unsigned long long s1, BigPlan* plan, uint8_t* bin_worker,
                                 const FinishLds& L, uint32_t& thr_bits)
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
    const double want = (double)P.top_p * total64;
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
    // The nucleus ends in the first bin (from the top) at which the running mass reaches `want`.  These sums
    // associate differently from the sorted prefix sums that make the final decision, so one more non-empty
    // bin is taken along: the list stops at the SECOND bin that satisfies the test.
    const bool r0 = c0 && incl - m1 >= want, r1 = c1 && incl >= want;
    const uint32_t reached = (uint32_t)r0 + (uint32_t)r1;
    const uint32_t reached_w = __ockl_wfscan_add_u32(reached, true);
    if (lane_id() == kWave - 1)
        sm.hist[wave_id()] = reached_w;
    if (tid == 0) {
        sm.ticket = 0;        // the lowest bin taken; not reached twice: every candidate is kept
        sm.flag = count_all;  // the number of weights to sort
    }
    __syncthreads();
    uint32_t before = reached_w - reached;
    for (int w = 0; w < kWaves; ++w)
        before += w < wave_id() ? sm.hist[w] : 0u;
    if (r0 && before + 1 == 2) {
        sm.ticket = b0;
        sm.flag = above0 + c0;
    } else if (r1 && before + (uint32_t)r0 + 1 == 2) {
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

// Copies the weights of the row with key_lo <= bits(q) < key_hi, in index order, to kout / iout (as ~bits(q) and
// token id).  Wave w owns a contiguous chunk of the row: a counting sweep, one exchange of the 16 wave totals,
// then a writing sweep in which ranks come from ballots.  Lane l holds entries 4l..4l+3 of each 256-entry group.
// Returns the number of entries written.
__device__ uint32_t gather_range(const uint32_t* qk, uint32_t V, uint32_t key_lo, uint32_t key_hi, uint32_t* kout,
                                 uint32_t* iout, uint32_t cap, FinishShared& sm)
{
    const uint32_t lane = lane_id(), wave = wave_id();
    const uint32_t chunk = ((V + kThreads * 4u - 1u) / (kThreads * 4u)) * kGroup; // per wave, a multiple of 256
    const uint32_t beg = min(V, wave * chunk), end = min(V, beg + chunk);
    auto fetch = [&](uint32_t i, uint32_t (&k)[4]) {
        if (i + 3 < end) {
            const uint4 x = *reinterpret_cast<const uint4*>(qk + i);
            k[0] = x.x;
            k[1] = x.y;
            k[2] = x.z;
            k[3] = x.w;
        } else {
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                k[j] = i + j < end ? qk[i + j] : 0u;
        }
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            if (k[j] < key_lo || k[j] >= key_hi)
                k[j] = 0;
    };
    uint32_t mine = 0;
    for (uint32_t base = beg; base < end; base += 4u * kGroup) {
        uint32_t k[4][4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u)
            fetch(base + u * kGroup + lane * 4u, k[u]);
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u)
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                mine += k[u][j] != 0;
    }
    mine = __ockl_wfred_add_u32(mine);
    __syncthreads();
    if (lane == 0)
        sm.bs.u64[wave] = mine;
    __syncthreads();
    uint32_t out = 0, n0 = 0;
    for (int w = 0; w < kWaves; ++w) {
        const uint32_t x = (uint32_t)sm.bs.u64[w];
        if (w < (int)wave)
            out += x;
        n0 += x;
    }
    const unsigned long long lower = (1ull << lane) - 1ull;
    for (uint32_t base = beg; base < end; base += 2u * kGroup) {
        uint32_t k[2][4];
        fetch(base + lane * 4u, k[0]);
        fetch(base + kGroup + lane * 4u, k[1]);
#pragma unroll
        for (uint32_t u = 0; u < 2; ++u) {
            uint32_t before = 0, total = 0;
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
                const unsigned long long bal = __ballot(k[u][j] != 0);
                before += (uint32_t)__popcll(bal & lower);
                total += (uint32_t)__popcll(bal);
            }
            uint32_t pos = out + before;
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j)
                if (k[u][j]) {
                    if (pos < cap) { // (the caller's count of the range; never exceeded when the plan is sound)
                        kout[pos] = ~k[u][j];
                        iout[pos] = base + u * kGroup + lane * 4u + j;
                    }
                    ++pos;
                }
            out += total;
        }
    }
    __syncthreads();
    return n0;
}

// Sorts n (key, id) pairs at (k0, i0) by key ascending, stably, with (k1, i1) as the second buffer; the result
// ends in (k0, i0).
__device__ void sort_segment(uint32_t* k0, uint32_t* i0, uint32_t* k1, uint32_t* i1, uint32_t n, const FinishLds& L)
{
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

__device__ bool lds_bucket_sort(uint32_t n, uint32_t key_lo, uint32_t key_hi, uint32_t* kout, uint32_t* iout,
                                unsigned long long* dyn, FinishShared& sm, uint32_t* sorted_lds = nullptr);

// Worker's sort, LDS-resident: the weights of the row with key_lo <= bits(q) < key_hi (at most kSegCap of them)
// are collected from the row's bits(q) array in one sweep, dropped into kFine value buckets (descending), and
// every entry then finds its place by counting the entries of its own bucket that precede it under
// (q desc, idx asc).  The sorted range is written to kout / iout as ~bits(q) and token id.  Returns false, having
// written nothing, when the range does not fit or a bucket is too crowded to be ranked by counting.
__device__ bool lds_sort_range(const uint32_t* qk, uint32_t V, uint32_t key_lo, uint32_t key_hi, uint32_t cnt, uint32_t* kout,
                               uint32_t* iout, unsigned long long* dyn, FinishShared& sm)
{
    uint2* A = reinterpret_cast<uint2*>(dyn);                       // [kSegCap] (bits(q), idx), any order
    uint16_t* B = reinterpret_cast<uint16_t*>(A + kSegCap);         // [kSegCap] entry of A at each bucket-ordered slot
    uint32_t* hist = reinterpret_cast<uint32_t*>(B + kSegCap);      // [kFine + 1] bucket counts, then bucket starts
    const uint32_t tid = threadIdx.x, lane = lane_id();
    if (cnt > kSegCap)
        return false;
    for (uint32_t b = tid; b <= kFine; b += kThreads)
        hist[b] = 0;
    if (tid == 0) {
        sm.ticket = 0;
        sm.flag = 0;
    }
    __syncthreads();
    // 1. collect: a slot range per wave and trip from one LDS atomic
    for (uint32_t base = 0; base < V; base += 4u * kThreads * 4u) {
        uint32_t k[4][4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint32_t i = base + u * kThreads * 4u + tid * 4u;
            if (i + 3 < V) {
                const uint4 x = *reinterpret_cast<const uint4*>(qk + i);
                k[u][0] = x.x;
                k[u][1] = x.y;
                k[u][2] = x.z;
                k[u][3] = x.w;
            } else {
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j)
                    k[u][j] = i + j < V ? qk[i + j] : 0u;
            }
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            // ranks inside the wave from ballots (any order will do), one LDS atomic per wave for the slots
            uint32_t before = 0, wave_total = 0;
            const unsigned long long lower = (1ull << lane) - 1ull;
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
                if (k[u][j] < key_lo || k[u][j] >= key_hi)
                    k[u][j] = 0; // 0 is never a candidate's weight
                const unsigned long long bal = __ballot(k[u][j] != 0);
                before += (uint32_t)__popcll(bal & lower);
                wave_total += (uint32_t)__popcll(bal);
            }
            if (wave_total) { // uniform
                uint32_t slot = 0;
                if (lane == 0)
                    slot = atomicAdd(&sm.ticket, wave_total);
                slot = uniform_u32(slot) + before;
                const uint32_t i = base + u * kThreads * 4u + tid * 4u;
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j)
                    if (k[u][j]) {
                        if (slot < kSegCap)
                            A[slot] = make_uint2(k[u][j], i + j);
                        ++slot;
                    }
            }
        }
    }
    __syncthreads();
    if (sm.ticket != cnt) // (cannot happen: the plan counted the same array)
        return false;
    return lds_bucket_sort(cnt, key_lo, key_hi, kout, iout, dyn, sm);
}

// Second half of the workers' sort: the n entries (bits(q), idx) in LDS at A, all with key_lo <= bits(q) < key_hi,
// go to kout / iout ordered by (q desc, idx asc).  hist must be zero and sm.flag 0 on entry.
// sorted_lds (optional, n words of LDS outside the sort's own): receives the sorted ~bits(q) as well, and the
// function then returns behind a barrier that orders LDS only: the caller goes on from the copy instead of waiting
// for the stores to kout and reading them back.
__device__ bool lds_bucket_sort(uint32_t n, uint32_t key_lo, uint32_t key_hi, uint32_t* kout, uint32_t* iout,
                                unsigned long long* dyn, FinishShared& sm, uint32_t* sorted_lds)
{
    uint2* A = reinterpret_cast<uint2*>(dyn);
    uint16_t* B = reinterpret_cast<uint16_t*>(A + kSegCap);
    uint32_t* hist = reinterpret_cast<uint32_t*>(B + kSegCap);
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
    if (sm.flag)
        return false;
#pragma unroll
    for (uint32_t t = 0; t < kPer; ++t)
        if (bucket[t] != kNone)
            B[hist[bucket[t]] + pib[t]] = (uint16_t)(t * kThreads + tid);
    __syncthreads();
    // 3. rank inside the bucket, and out
#pragma unroll
    for (uint32_t t = 0; t < kPer; ++t) {
        const uint32_t s = t * kThreads + tid;
        if (s < n) {
            const uint2 me = A[B[s]];
            const uint32_t b = (key_hi - 1u - me.x) >> shift;
            const uint32_t lo = hist[b], hi = hist[b + 1u];
            uint32_t r = 0;
            for (uint32_t x = lo; x < hi; ++x) {
                const uint2 o = A[B[x]];
                r += (o.x > me.x) || (o.x == me.x && o.y < me.y);
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

// The worker's share as partition_kernel left it (cnt <= kSegCap entries, bits(q) in ks and token ids in is, any
// order), sorted into kout / iout.
__device__ bool lds_sort_staged(const uint32_t* ks, const uint32_t* is, uint32_t key_lo, uint32_t key_hi, uint32_t cnt,
                                uint32_t* kout, uint32_t* iout, unsigned long long* dyn, FinishShared& sm,
                                uint32_t* sorted_lds = nullptr)
{
    uint2* A = reinterpret_cast<uint2*>(dyn);
    uint16_t* B = reinterpret_cast<uint16_t*>(A + kSegCap);
    uint32_t* hist = reinterpret_cast<uint32_t*>(B + kSegCap);
    const uint32_t tid = threadIdx.x;
    for (uint32_t b = tid; b <= kFine; b += kThreads)
        hist[b] = 0;
    if (tid == 0)
        sm.flag = 0;
    constexpr uint32_t kPer = kSegCap / kThreads;
    uint32_t k[kPer], id[kPer];
#pragma unroll
    for (uint32_t t = 0; t < kPer; ++t) { // (all loads first, from clamped positions)
        const uint32_t e = min(t * kThreads + tid, cnt - 1u);
        k[t] = ks[e];
        id[t] = is[e];
    }
#pragma unroll
    for (uint32_t t = 0; t < kPer; ++t) {
        const uint32_t e = t * kThreads + tid;
        if (e < cnt)
            A[e] = make_uint2(min(max(k[t], key_lo), key_hi - 1u), id[t]); // (clamped: a bucket index is always valid)
    }
    __syncthreads();
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
    uint16_t* B = reinterpret_cast<uint16_t*>(A + kSegCap);
    uint32_t* hist = reinterpret_cast<uint32_t*>(B + kSegCap); // [kFine + 1]
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

// Group records of a worker's sorted range (cnt entries from position off of the list kf): fp64 sums, and the
// maps of the running fp32 sum for the epoch guessed from the mass above the range plus the sums before the group.
// kf_lds (optional): the worker's cnt sorted weights in LDS (outside L.sortk's first 16 KB), read instead of kf + off.
__device__ void worker_groups(const uint32_t* kf, uint32_t off, uint32_t cnt, size_t t_at, double mass, const GroupTable& T,
                              const FinishLds& L, const uint32_t* kf_lds = nullptr)
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
    __syncthreads();
    for (uint32_t g0 = 0; g0 < groups; g0 += kThreads) { // (one trip unless the range is the fallback's)
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
    for (uint32_t g = wave_id(); g < groups; g += kWaves) {
        const uint32_t len = min(kGroup, cnt - g * kGroup);
        float q[4];
        load_span(src, g * kGroup, len, q);
        const double guess = gs[g];
        const int eg = guess > 0 ? exponent_of((float)guess) : 0;
        const seqfp::Step32 st = span_map(q, len, eg);
        // the sum is expected to change binade inside the group (or starts at zero): records for its quarters
        const double at_end = ge[g];
        const bool split4 = uniform_u32((uint32_t)(eg == 0 || exponent_of((float)at_end) != eg)) != 0;
        if (split4)
            build_quarters(q, len, guess, T.quarters + (t_at + g) * 4u);
        if (lane_id() == 0) {
            T.d0[t_at + g] = st.d0;
            T.d1[t_at + g] = st.d1;
            T.cmax[t_at + g] = st.cmax;
            T.start[t_at + g] = off + g * kGroup;
            T.pack[t_at + g] = len | ((uint32_t)eg << 16) | (split4 ? kHasQuarters : 0u);
        }
    }
}

// Whole-row path: exact for every parameter combination.  One workgroup rebuilds the penalised
// row in scratch, keeps the candidates, sorts them by (q desc, idx asc) when top-k or top-p is
// active, truncates, and draws.  src/gen/sampler.cpp:20-62.
// (SITE: sort_kernel, its usual place, has an instance to itself, so that the compiler treats that kernel the same
// whether or not the instances inside plan_kernel exist.)
template <int SITE>
__device__ void general_row(const mako_sample_desc& d, const Scratch& sc, uint32_t row, const mako_sampling_params& P,
                            float m, uint32_t argidx, const FinishLds& L)
{
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

// Bitonic sort, descending, of 1024 * ITEMS keys held ITEMS per thread: key[t] is element t * 1024 + tid.
// Partners 1024 or more apart are other registers of the same thread, partners less than 64 apart are lanes
// of the same wave (shuffles); only the strides in between go through LDS (two barriers each).
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
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t)
        w[t] = sc.cand_w[at[t]];
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)ITEMS; ++t)
        id[t] = sc.cand_i[at[t]];
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
#pragma unroll
    for (uint32_t t = 0; t < (uint32_t)kPrefetchItems; ++t) {
        c.w[t] = sc.cand_w[base + 128u * t];
        c.id[t] = sc.cand_i[base + 128u * t];
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
__device__ uint32_t sort_candidates(const Scratch& sc, uint32_t row, uint32_t slices, uint32_t n_cands, float m, float inv_t,
                                    float floor_q, uint32_t* kf, uint32_t* jf, const FinishLds& L)
{
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

constexpr uint32_t kSmall = 256; // lists of up to this many entries are ordered by counting ranks

// Fast route for rows that need only a few of their candidates.  Every thread weights up to four candidates;
// those at or above a weight threshold (at most kSmall of them) are ordered by (q desc, idx asc) by counting, for
// each, the entries that precede it, and left in LDS as kf[i] = ~bits(q_i), jf[i] = token id.
//   top_k > 0:  the threshold is the lower edge of the quarter-binade bin that holds the top_k-th largest weight
//               (one histogram over bits(q) >> 21), so the list is a superset of the row's top_k candidates.
//   top_k == 0: the threshold is thr_bits, below which the nucleus cannot reach (from the row's histogram).
// Returns the number of entries in the list, or kNone when they exceed kSmall (nothing is written then);
// n_valid receives the number of candidates that have a weight at all.
// `pre` (when have_pre): the row's candidate slots as fetch_candidate_slots() loaded them.
__device__ uint32_t small_candidates(const Scratch& sc, uint32_t row, uint32_t slices, uint32_t n_cands, float m, float inv_t,
                                     float floor_q, uint32_t top_k, uint32_t thr_bits, uint32_t* kf, uint32_t* jf,
                                     uint32_t& n_valid, const FinishLds& L, bool have_pre = false,
                                     const CandSlots& pre = CandSlots{})
{
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

__device__ __forceinline__ void row_summary(const Scratch& sc, uint32_t row, uint32_t slices, float& m, uint32_t& argidx,
                                            uint32_t& n_cands, uint32_t& any_overflow, SliceStat* lane_stat = nullptr);

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

// Kernel arguments that are handed on by reference to out-of-line device functions would be spilled to scratch
// memory (a microsecond per access); the two finishing kernels keep their copies in LDS instead.
struct alignas(16) ArgsLds {
    mako_sample_desc d;
    Scratch sc;
    mako_sampling_params P; // the row's parameters
};

// The same in two steps for a kernel that learns its row late: the arguments first (no barrier), the row's parameters
// (already in registers, the same in every lane) afterwards; the caller's next barrier publishes both.
__device__ __forceinline__ void stage_args_only(const mako_sample_desc& d_arg, const Scratch& sc_arg, ArgsLds& a)
{
    const uint32_t* src_d = reinterpret_cast<const uint32_t*>(&d_arg);
    const uint32_t* src_s = reinterpret_cast<const uint32_t*>(&sc_arg);
    uint32_t* dst_d = reinterpret_cast<uint32_t*>(&a.d);
    uint32_t* dst_s = reinterpret_cast<uint32_t*>(&a.sc);
    for (uint32_t i = threadIdx.x; i < sizeof(mako_sample_desc) / 4; i += kThreads)
        dst_d[i] = src_d[i];
    for (uint32_t i = threadIdx.x; i < sizeof(Scratch) / 4; i += kThreads)
        dst_s[i] = src_s[i];
}
__device__ __forceinline__ void stage_params(const mako_sampling_params& P, ArgsLds& a)
{
    if (threadIdx.x == 0)
        a.P = P;
}

__device__ __forceinline__ void stage_args(const mako_sample_desc& d_arg, const Scratch& sc_arg, uint32_t row, ArgsLds& a)
{
    static_assert(sizeof(mako_sample_desc) % 4 == 0 && sizeof(Scratch) % 4 == 0, "word copies");
    const uint32_t* src_d = reinterpret_cast<const uint32_t*>(&d_arg);
    const uint32_t* src_s = reinterpret_cast<const uint32_t*>(&sc_arg);
    uint32_t* dst_d = reinterpret_cast<uint32_t*>(&a.d);
    uint32_t* dst_s = reinterpret_cast<uint32_t*>(&a.sc);
    for (uint32_t i = threadIdx.x; i < sizeof(mako_sample_desc) / 4; i += kThreads)
        dst_d[i] = src_d[i];
    for (uint32_t i = threadIdx.x; i < sizeof(Scratch) / 4; i += kThreads)
        dst_s[i] = src_s[i];
    const uint32_t* src_p = reinterpret_cast<const uint32_t*>(d_arg.params + row);
    uint32_t* dst_p = reinterpret_cast<uint32_t*>(&a.P);
    if (threadIdx.x < sizeof(mako_sampling_params) / 4)
        dst_p[threadIdx.x] = src_p[threadIdx.x];
    __syncthreads();
}

// First maximum of the row (std::max_element semantics, NaNs never win unless at index 0) and the totals of the
// slices' candidate lists, from the records scan_kernel left.
__device__ __forceinline__ void row_summary(const Scratch& sc, uint32_t row, uint32_t slices, float& m, uint32_t& argidx,
                                            uint32_t& n_cands, uint32_t& any_overflow, SliceStat* lane_stat)
{
    // lane s of every wave takes slice s (at most kMaxSlices = 64 of them): one load each, then wave reductions
    const uint32_t s = min((uint32_t)lane_id(), slices - 1u);
    const SliceStat st = sc.stats[(size_t)row * kMaxSlices + s];
    if (lane_stat)
        *lane_stat = st;
    const bool mine = (uint32_t)lane_id() < slices;
    const unsigned long long p =
        mine ? ((unsigned long long)order_key(st.wmax) << 32) | (unsigned long long)(kNone - st.argidx) : 0ull;
    const unsigned long long top = __ockl_wfred_max_u64(p);
    n_cands = __ockl_wfred_add_u32(mine ? st.n_emit : 0u);
    any_overflow = __ballot(mine && (st.flags & kFlagOverflow)) != 0ull ? kFlagOverflow : 0u;
    const bool first_nan = __ballot(lane_id() == 0 && (st.flags & kFlagFirstNan)) != 0ull;
    m = order_unkey((uint32_t)(top >> 32));
    argidx = kNone - (uint32_t)top;
    if (argidx == kNone)
        argidx = 0;
    if (first_nan) {
        m = __uint_as_float(0x7fc00000u);
        argidx = 0;
    }
}

// Where each slice's candidates start in the row's flattened candidate list (sm.soff), and the largest weight a
// logit that was NOT emitted can have over all slices (0 if none can be a candidate): everything left behind
// has an order key below its slice's tau_key.
__device__ float candidate_bound(const SliceStat& st, uint32_t slices, float m, float inv_t, float floor_q, FinishShared& sm)
{
    // `st`: the record of slice min(lane, slices - 1), as row_summary() hands it out; one wave leaves the offsets in LDS
    const bool mine = (uint32_t)lane_id() < slices;
    uint32_t qbits = 0;
    if (mine && !(st.flags & kFlagComplete)) {
        const float qb = weight_of(order_unkey(st.tau_key - 1u), m, inv_t, sm.tab);
        if (qb >= floor_q && qb > 0.0f)
            qbits = __float_as_uint(qb); // positive floats order like their bits
    }
    const float q_bound = __uint_as_float(__ockl_wfred_max_u32(qbits));
    const uint32_t emitted = mine ? st.n_emit : 0u;
    const uint32_t upto = __ockl_wfscan_add_u32(emitted, true);
    if (wave_id() == 0) {
        if (mine)
            sm.soff[lane_id() + 1] = upto;
        if (lane_id() == 0)
            sm.soff[0] = 0;
    }
    __syncthreads();
    return q_bound;
}

// Is the row's token decided without sampling (Session's `forced` callback, src/gen/session.cpp:441-443)?  Returns
// MAKO_FORCED_* and the token; `above` receives the logits strictly above the close_token's (kNone without one).
// The same answer in every thread and in every workgroup that asks.
__device__ __forceinline__ uint32_t row_forced(const mako_sample_desc& d, const Scratch& sc, uint32_t row, uint32_t slices,
                                               int32_t& token, uint32_t& above)
{
    uint32_t kind = MAKO_FORCED_NONE;
    above = kNone;
    token = -1;
    if (d.close_token) {
        const int32_t ct = d.close_token[row];
        if (ct >= 0 && (uint32_t)ct < d.n_vocab &&
            (!d.mask || ((d.mask[(int64_t)row * d.mask_stride + ((uint32_t)ct >> 5)] >> ((uint32_t)ct & 31u)) & 1u))) {
            uint32_t a = 0;
            for (uint32_t s = 0; s < slices; ++s)
                a += sc.stats[(size_t)row * kMaxSlices + s].above;
            above = a;
            if (a < d.close_max_above) { // src/server/openai.cpp:600-603
                kind = MAKO_FORCED_CLOSE;
                token = ct;
            }
        }
    }
    if (d.force_token) {
        const int32_t ft = d.force_token[row];
        if (ft >= 0) {
            kind = MAKO_FORCED_TOKEN;
            token = ft;
        }
    }
    return kind;
}

// Rows other than top_k == 0 rows whose candidate lists cannot serve: top_k > kTopKFast, no truncation at all, a slice
// that had to drop candidates.  They take the whole-row path.
__device__ __forceinline__ bool topk_takes_whole_row(RowClass cls, uint32_t any_overflow, uint32_t n_cands)
{
    return cls == kGeneral || any_overflow || n_cands > kSortMax;
}

// A top-k row (top_k <= kTopKFast) from the candidates scan_kernel left: weights of the candidates, the top_k-th
// weight's neighbourhood ordered by (q desc, idx asc) in LDS, the certificate that nothing left behind in a slice can
// reach the top_k-th weight, then top-p, total and draw by one wave.  A row that cannot be certified takes the
// whole-row path: here and now (INLINE_GENERAL), or through sort_kernel's work list.
template <bool INLINE_GENERAL>
__device__ __forceinline__ void topk_row(const mako_sample_desc& d, const Scratch& sc, uint32_t row, uint32_t slices,
                                         const mako_sampling_params& P, float m, uint32_t argidx, uint32_t n_cands,
                                         const SliceStat& lane_stat, const FinishLds& L, bool have_pre = false,
                                         const CandSlots& pre = CandSlots{})
{
    constexpr bool inline_general = INLINE_GENERAL;
    FinishShared& sm = *L.sm;
    const uint32_t tid = threadIdx.x;
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
    const bool ok = n_valid >= P.top_k ? q_bound < __uint_as_float(~kf[P.top_k - 1]) : q_bound == 0.0f;
    if (!ok) {
        if constexpr (inline_general) {
            __syncthreads(); // (the lists in LDS are done with)
            general_row<1>(d, sc, row, P, m, argidx, L);
            return;
        } else {
            if (tid == 0) {
                sc.plan[row].total64 = (double)m;
                sc.plan[row].n0 = argidx;
                sc.plan[row].flag = 2;
                sc.work_sort[atomicAdd(&sc.work_n[0], 1u)] = row << 8;
            }
            return;
        }
    }
    if (n_valid == 0) {
        fallback_row(d, row, argidx);
        return;
    }
    // (sampler.cpp:40-43; at most top_k <= kTopKFast <= kGroup entries)
    static_assert(kTopKFast <= kGroup, "top-k rows end in sorted_tail's short-list path");
    sorted_tail<false, true>(d, row, P, kf, jf, min(P.top_k, n_valid), false, 0.0, MAKO_PATH_TOPK, L);
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

// grid = (1, rows), one workgroup per row.  Rows whose token is forced, greedy rows and top-k rows are finished here
// from the records scan_kernel left; a top_k == 0 row's exact total, candidate count and weight histogram (from
// finish_kernel) are summed over its pieces and the row is planned: handed to sort_kernel's workers, or, when the
// nucleus is narrow enough to end inside the candidate lists, to its worker 0 alone.
// INLINE_GENERAL: sort_kernel will not be launched for this batch (the host saw no row that needs it), so a row
// that turns out to need the whole-row path after all is given it here.  (A variant of its own: the whole-row path
// costs the kernel registers that the usual batches should not pay for.)
template <bool INLINE_GENERAL>
__global__ __launch_bounds__(kThreads) void plan_kernel(mako_sample_desc d_arg, const Scratch* sc_dev, uint32_t slices)
{
    constexpr bool inline_general = INLINE_GENERAL;
    const Scratch& sc_arg = *sc_dev;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t row = blockIdx.y;
    const uint32_t tid = threadIdx.x;
#ifdef MAKO_TIMING_PLAN
    MAKO_WG_TIMER;
#endif
    MAKO_ROW(row);
    stage_args(d_arg, sc_arg, row, s_args);
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    const mako_sampling_params& P = s_args.P;
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;
    L.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);
    const RowClass cls = classify(P);
    if (cls != kNucleus)
        MAKO_STAMP(0);
    if (d.force_token || d.close_token) { // uniform
        int32_t ftok;
        uint32_t above;
        const uint32_t kind = row_forced(d, sc, row, slices, ftok, above);
        if (tid == 0 && d.out_above)
            d.out_above[row] = above;
        if (kind != MAKO_FORCED_NONE) {
            // a token >= 0 is taken instead of sampling, and a draft is kept only if it matches (session.hpp:43-45)
            if (tid == 0) {
                RowOut o;
                o.token = ftok;
                o.n_cand = 0;
                o.total = 0.0f;
                o.q = 0.0f;
                o.path = MAKO_PATH_FORCED;
                o.accepted = d.draft ? (d.draft[row] == ftok) : 0u;
                o.forced = kind;
                write_row(d, row, o);
            }
            return;
        }
    }
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    __syncthreads();
    // a top-k row's candidates are asked for together with the slices' records
    CandSlots pre;
    const bool prefetched = cls == kTopK && !d.draft && slots_cover(slices); // uniform
    if (prefetched)
        fetch_candidate_slots(sc, row, slices, pre);
    float m;
    uint32_t argidx, n_cands, any_overflow;
    SliceStat lane_stat;
    row_summary(sc, row, slices, m, argidx, n_cands, any_overflow, &lane_stat);
    if (cls != kNucleus)
        MAKO_STAMP(1);
    if (cls == kGreedy) { // sampler.cpp:77-78, 88-92
        if (tid == 0) {
            RowOut o;
            o.token = (int32_t)argidx;
            o.n_cand = 0;
            o.total = 0.0f;
            o.q = 0.0f;
            o.path = MAKO_PATH_GREEDY;
            o.accepted = d.draft ? (d.draft[row] == (int32_t)argidx) : 0u;
            write_row(d, row, o);
        }
        return;
    }

    if (cls != kNucleus) {
        if (topk_takes_whole_row(cls, any_overflow, n_cands)) {
            if constexpr (inline_general) {
                general_row<1>(d, sc, row, P, m, argidx, L);
                return;
            }
            if (tid == 0) {
                sc.plan[row].total64 = (double)m; // carries the row maximum and its first index to the whole-row path
                sc.plan[row].n0 = argidx;
                sc.plan[row].flag = 2;
                sc.work_sort[atomicAdd(&sc.work_n[0], 1u)] = row << 8;
            }
            return;
        }

        topk_row<inline_general>(d, sc, row, slices, P, m, argidx, n_cands, lane_stat, L, prefetched, pre);
        return;
    }

    MAKO_STAMP(2);
    const uint32_t pieces = uniform_u32(sc.work_n[4]);
    // this thread's two bins of the row's histogram (left zero for the next batch), the pieces' exact sums (one per
    // lane, added up in the wave reduction's fixed order)
    unsigned long long* bins = sc.bins + (size_t)row * kBins;
    const unsigned long long rec0 = bins[kBins - 1u - 2u * tid], rec1 = bins[kBins - 2u - 2u * tid];
    const uint32_t bin_c0 = (uint32_t)(rec0 >> kBinSumBits), bin_c1 = (uint32_t)(rec1 >> kBinSumBits);
    const unsigned long long bin_s0 = rec0 & ((1ull << kBinSumBits) - 1ull), bin_s1 = rec1 & ((1ull << kBinSumBits) - 1ull);
    const uint32_t pc = min((uint32_t)lane_id(), pieces - 1u); // pieces <= kMaxSlices = 64
    const double ps = sc.part_sum[(size_t)row * kMaxSlices + pc];
    const uint32_t pn = sc.part_n[(size_t)row * kMaxSlices + pc];
    const double row_total = __ockl_wfred_add_f64((uint32_t)lane_id() < pieces ? ps : 0.0);
    const uint32_t row_n0 = __ockl_wfred_add_u32((uint32_t)lane_id() < pieces ? pn : 0u);
    if (rec0)
        bins[kBins - 1u - 2u * tid] = 0;
    if (rec1)
        bins[kBins - 2u - 2u * tid] = 0;
    MAKO_STAMP(15);
    if (row_n0 == 0) {
        fallback_row(d, row, argidx);
        return;
    }
    uint32_t thr_bits = 0;
    const uint32_t n0 = plan_nucleus(P, row_total, bin_c0, bin_c1, bin_s0, bin_s1, sc.plan + row, sc.bin_worker + (size_t)row * kBins, L, thr_bits);
    MAKO_STAMP(16);
    const bool narrow = !d.draft && n0 <= kSmall && !any_overflow && n_cands <= kSortMax;
    // (a list too long for the workers' group records goes to the whole-row path)
    const bool fits = n0 <= kGroup * (kMaxGroups - kWorkers);
    if (tid == 0) {
        if (!fits) {
            sc.plan[row].total64 = (double)m;
            sc.plan[row].n0 = argidx;
        }
        sc.plan[row].thr = thr_bits;
        sc.plan[row].flag = !fits ? 2 : (narrow ? 3 : 1);
    }
    // the row's pieces of work for sort_kernel (all workers, or worker 0 alone) and tail_kernel
    const uint32_t work = (fits && !narrow) ? kWorkers : 1u;
    if (tid == 0)
        sm.flag = atomicAdd(&sc.work_n[0], work);
    __syncthreads();
    if (tid < work)
        sc.work_sort[sm.flag + tid] = (row << 8) | tid;
    if (tid == 0 && fits && !narrow)
        sc.work_tail[atomicAdd(&sc.work_n[1], 1u)] = row;
}

#ifdef MAKO_EMIT_SORT_KERNELS // (not templates: defined by the one translation unit that launches them)
// grid = (kWorkers, rows) workgroups over the same work list as sort_kernel; only planned wide rows do anything.
// Piece c of a row reads the c-th part of the row's bits(q) array once and hands every weight the plan wants to
// the worker that will sort it: positions inside the workgroup from LDS counters, one global atomic per worker to
// reserve the workgroup's run in that worker's share.  (Without this step each of the 32 workers would sweep the
// whole row to find its own weights.)
__global__ __launch_bounds__(kThreads) void partition_kernel(mako_sample_desc d, Scratch sc_arg)
{
    // (the context's record by value, and loads asked for in groups: a workgroup here lives four microseconds, and
    // every dependent trip to memory is most of one)
    const Scratch& sc = sc_arg;
    __shared__ uint32_t s_count[kWorkers], s_base[kWorkers], s_off[kWorkers], s_cnt[kWorkers];
    __shared__ uint32_t s_table[kBins / 4];
    const uint32_t piece = blockIdx.y * gridDim.x + blockIdx.x;
    // first trip: the list's length and this workgroup's entry of it (the list has room for every workgroup of the
    // grid; what the entry says is looked at only if the length covers it)
    const uint32_t n_work = sc.work_n[0];
    const uint32_t item = sc.work_sort[piece];
    if (piece >= n_work)
        return;
    const uint32_t row = item >> 8, c = item & 255u, tid = threadIdx.x;
    MAKO_ROW(row);
    BigPlan* plan = sc.plan + row;
    const uint32_t V = d.n_vocab;
    const uint32_t* qk = reinterpret_cast<const uint32_t*>(sc.wbuf + (size_t)row * sc.vpad);
    uint32_t* kstage = sc.key[1] + (size_t)row * sc.vpad;
    uint32_t* istage = sc.idx[1] + (size_t)row * sc.vpad;
    const uint32_t part = (((V + kWorkers - 1u) / kWorkers) + 3u) & ~3u; // entries per piece, a multiple of 4
    const uint32_t lo = min(V, c * part), hi = min(V, lo + part);
    // second trip: the row's flag, the piece's first weights, the bin -> worker table and the workers' ranges
    const uint32_t flag = plan->flag;
    uint4 x = make_uint4(0, 0, 0, 0);
    {
        const uint32_t i = lo + tid * 4u;
        if (i < hi)
            x = *reinterpret_cast<const uint4*>(qk + i); // (the array is padded to a multiple of 1024 entries past V)
    }
    uint32_t table_word = 0, off_w = 0, cnt_w = 0;
    if (tid < kBins / 4)
        table_word = reinterpret_cast<const uint32_t*>(sc.bin_worker + (size_t)row * kBins)[tid];
    if (tid < kWorkers) {
        off_w = plan->off[tid];
        cnt_w = plan->cnt[tid];
    }
    if (flag != 1)
        return;
    if (tid < kBins / 4)
        s_table[tid] = table_word;
    if (tid < kWorkers) {
        s_count[tid] = 0;
        s_off[tid] = off_w;
        s_cnt[tid] = cnt_w;
    }
    __syncthreads();
    const uint8_t* table = reinterpret_cast<const uint8_t*>(s_table);
    for (uint32_t base = lo; base < hi; base += kThreads * 4u) {
        const uint32_t i = base + tid * 4u;
        if (base != lo) {
            x = make_uint4(0, 0, 0, 0);
            if (i < hi)
                x = *reinterpret_cast<const uint4*>(qk + i);
        }
        const uint32_t k[4] = {x.x, x.y, x.z, x.w};
        uint32_t dest[4], lpos[4];
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            dest[j] = (i + j < hi && k[j] != 0) ? table[weight_bin(k[j])] : 0xffu;
            lpos[j] = 0;
            if (dest[j] < kWorkers)
                lpos[j] = atomicAdd(&s_count[dest[j]], 1u);
        }
        __syncthreads();
        if (tid < kWorkers) {
            s_base[tid] = s_count[tid] ? atomicAdd(&plan->cursor[tid], s_count[tid]) : 0u;
            s_count[tid] = 0;
        }
        __syncthreads();
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            if (dest[j] < kWorkers) {
                const uint32_t at = s_base[dest[j]] + lpos[j];
                if (at < s_cnt[dest[j]] && s_off[dest[j]] + at < V) { // (always, when the plan is sound)
                    kstage[s_off[dest[j]] + at] = k[j];
                    istage[s_off[dest[j]] + at] = i + j;
                }
            }
        __syncthreads();
    }
}

// grid = (kWorkers, rows) workgroups, of which workgroup i serves entry i of the work list.  Worker w gathers its range of weights from
// the row's bits(q) array, sorts it and stores it at its place in the row's sorted list; the last worker to
// finish cuts the nucleus and draws.
__global__ __launch_bounds__(kThreads) void sort_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    // (the context's record by value: its first loads, the list's length and this workgroup's entry, go out together
    // and at once; the list has room for every workgroup of the grid)
    const Scratch& sc_arg = sc_val;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t piece = blockIdx.y * gridDim.x + blockIdx.x;
    const uint32_t n_work = sc_arg.work_n[0];
    const uint32_t item = sc_arg.work_sort[piece];
    if (piece >= n_work)
        return;
#ifdef MAKO_TIMING_SORT
    MAKO_WG_TIMER;
#endif
    const uint32_t row = item >> 8, w = item & 255u, tid = threadIdx.x;
    MAKO_ROW(row);
    const uint32_t flag = sc_arg.plan[row].flag;
    if (flag == 0 || (flag != 1 && w != 0)) // (never: the list holds exactly the flagged rows' pieces)
        return;
    stage_args(d_arg, sc_arg, row, s_args);
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    BigPlan* plan = sc.plan + row;
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;
    L.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    if (flag == 2) {
        // top_k > 128, no top-p, or a candidate list that could not be certified: the whole-row path
        const float m = (float)plan->total64;
        const uint32_t argidx = plan->n0;
        __syncthreads();
        if (tid == 0)
            plan->flag = 0;
        general_row<0>(d, sc, row, s_args.P, m, argidx, L);
        return;
    }
    const uint32_t* qk = reinterpret_cast<const uint32_t*>(sc.wbuf + (size_t)row * sc.vpad);
    uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
    uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
    uint32_t* key1 = sc.key[1] + (size_t)row * sc.vpad;
    uint32_t* idx1 = sc.idx[1] + (size_t)row * sc.vpad;
    const uint32_t n0 = min(plan->n0, d.n_vocab), groups = min(plan->groups, kMaxGroups);
    const double total64 = plan->total64;
    if (flag == 3) {
        // narrow nucleus: it should end inside the slices' candidate lists, strictly above everything they left out
        const uint32_t thr_bits = plan->thr;
        __syncthreads();
        if (tid == 0)
            plan->flag = 0;
        const mako_sampling_params& P = s_args.P;
        // (the candidate lists are asked for together with the slices' records, as for a top-k row)
        CandSlots pre;
        const bool prefetched = slots_cover(slices); // uniform
        if (prefetched)
            fetch_candidate_slots(sc, row, slices, pre);
        float m;
        uint32_t argidx, n_cands, any_overflow;
        SliceStat lane_stat;
        row_summary(sc, row, slices, m, argidx, n_cands, any_overflow, &lane_stat);
        const float inv_t = 1.0f / P.temperature;
        const float floor_q = (1.0f < P.min_p) ? 1.0f : P.min_p;
        const float q_bound = candidate_bound(lane_stat, slices, m, inv_t, floor_q, sm);
        MAKO_STAMP(3);
        uint32_t* kf = reinterpret_cast<uint32_t*>(L.sortk + kSortMax);
        uint32_t* jf = kf + kSortMax;
        uint32_t n_valid = 0;
        const uint32_t n_list =
            small_candidates(sc, row, slices, n_cands, m, inv_t, floor_q, 0u, thr_bits, kf, jf, n_valid, L, prefetched, pre);
        MAKO_STAMP(4);
        if (n_list != kNone && n_list > 0 &&
            sorted_tail(d, row, P, kf, jf, n_list, true, total64, MAKO_PATH_NUCLEUS, L, true, q_bound))
            return;
        // not certifiable from the candidates: the row's weights at or above the threshold, from its bits(q) array
        if (!lds_sort_range(qk, d.n_vocab, thr_bits, 0x7f800001u, n0, key0, idx0, s_dyn64, sm)) {
            gather_range(qk, d.n_vocab, thr_bits, 0x7f800001u, key0, idx0, n0, sm);
            sort_segment(key0, idx0, key1, idx1, n0, L);
        }
        sorted_tail(d, row, P, key0, idx0, n0, true, total64, MAKO_PATH_GENERAL, L);
        return;
    }
    uint32_t cnt = plan->cnt[w];
    const uint32_t off = plan->off[w], gbase = plan->gbase[w];
    // (a sound plan never trips these; they keep every store of this worker inside the row's arrays)
    if (off > n0 || cnt > n0 - off || gbase + (cnt + kGroup - 1u) / kGroup > min(groups, sc.g_cap))
        cnt = 0;
    const size_t t_row = (size_t)row * sc.g_cap;
    if (cnt) {
        const uint32_t key_lo = plan->key_lo[w], key_hi = plan->key_hi[w];
        MAKO_STAMP(10);
        MAKO_COUNT(31, threadIdx.x == 0 && cnt > kSegCap ? 1 : 0);
        MAKO_COUNT(21, threadIdx.x == 0 ? cnt : 0);
        uint32_t* sorted_copy = reinterpret_cast<uint32_t*>(reinterpret_cast<char*>(s_dyn64) + kSortedCopyAt);
        const bool in_lds = cnt <= kSegCap; // uniform
        const bool sorted = in_lds
                                ? lds_sort_staged(key1 + off, idx1 + off, key_lo, key_hi, cnt, key0 + off, idx0 + off, s_dyn64, sm,
                                                  sorted_copy)
                                : lds_sort_staged_runs(key1 + off, idx1 + off, key_lo, key_hi, cnt, key0 + off, idx0 + off, s_dyn64, sm);
        if (cnt > kSegCap)
            MAKO_STAMP(18);
        if (!sorted) {
            MAKO_STAMP(17);
            MAKO_COUNT(23, threadIdx.x == 0 ? 1 : 0);
            gather_range(qk, d.n_vocab, key_lo, key_hi, key0 + off, idx0 + off, cnt, sm);
            sort_segment(key0 + off, idx0 + off, key1 + off, idx1 + off, cnt, L);
        }
        MAKO_STAMP(11);
        worker_groups(key0, off, cnt, t_row + gbase, plan->mass[w], sc.gt, L, (in_lds && sorted) ? sorted_copy : nullptr);
        MAKO_STAMP(12);
    }
}
#endif // MAKO_EMIT_SORT_KERNELS

#ifdef MAKO_EMIT_TAIL_KERNEL
// grid = (1, rows).  Rows whose sorted list sort_kernel's workers have prepared: top-p cut, exact total, draw.
// (The batch's top-k rows were tried here too, beside the few long tails instead of ahead of the planning in
// plan_kernel: 2.3 us less there, but this kernel's chains then compiled to slower code and lost twice that.)
// (The context's record by value: with a pointer to it the first loads would have to wait for a trip to memory.  The
// list's length and this workgroup's entry are asked for together, then everything the row's plan holds.)
__global__ __launch_bounds__(kThreads) void tail_kernel(mako_sample_desc d_arg, Scratch sc_val)
{
    const Scratch& sc_arg = sc_val;
    extern __shared__ __align__(16) unsigned long long s_dyn64[]; // (128-bit LDS operations need the alignment)
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t n_work = sc_arg.work_n[1];
    const uint32_t row = sc_arg.work_tail[blockIdx.y], tid = threadIdx.x; // (the list has room for every workgroup)
    if (blockIdx.y >= n_work)
        return;
#ifdef MAKO_TIMING_TAIL
    MAKO_WG_TIMER;
#endif
    MAKO_ROW(row);
    const BigPlan* planned = sc_arg.plan + row;
    const uint32_t flag = planned->flag, plan_n0 = planned->n0, plan_groups = planned->groups;
    const double total64 = planned->total64;
    if (flag != 1)
        return;
    stage_args(d_arg, sc_arg, row, s_args);
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    BigPlan* plan = sc.plan + row;
    FinishLds L;
    L.sm = &sm;
    L.cnt = reinterpret_cast<uint32_t*>(s_dyn64);
    L.sortk = s_dyn64;
    L.wcount = reinterpret_cast<uint32_t*>(s_dyn64 + kSortMax);
    const uint32_t n0 = min(plan_n0, d.n_vocab), groups = min(plan_groups, min(kMaxGroups, sc.g_cap));
    __syncthreads();
    if (tid == 0)
        plan->flag = 0;
    sorted_tail<true>(d, row, s_args.P, sc.key[0] + (size_t)row * sc.vpad, sc.idx[0] + (size_t)row * sc.vpad, n0, true,
                      total64, MAKO_PATH_GENERAL, L, false, 0.0f, sc.gt, (size_t)row * sc.g_cap, groups);
}
#endif // MAKO_EMIT_TAIL_KERNEL

} // namespace mako
