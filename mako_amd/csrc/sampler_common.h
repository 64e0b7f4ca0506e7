// Constants, the context's scratch layout, order keys and the classification of rows: shared by every kernel
// of the sampler.
#pragma once

#include <hip/hip_runtime.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <type_traits>
#include "../../include/mako_sampler.h"
#include "block_prims.h"
#include "device_math.h"
#include "seqfp.h"
#include "log_bins.h"
#include "tuning_stamps.h"

namespace mako {

constexpr uint32_t kNone = 0xffffffffu;

constexpr uint32_t kSliceMax = 16384; // elements per slice: 16 per thread
constexpr uint32_t kMaxSlices = 64;
constexpr uint32_t kCap = 512;       // candidates kept per slice
constexpr uint32_t kTopKFast = 128;  // largest top_k resolved from the per-slice candidates
constexpr uint32_t kSortMax = 4096;  // candidates the finisher sorts in LDS
constexpr uint32_t kSmall = 256;     // lists of up to this many entries are ordered by counting ranks
constexpr uint32_t kDynLds = 65536;  // dynamic LDS of the second pass (and the most scan_kernel takes)
constexpr uint32_t kHeadGroups = 32; // groups at the head of a sorted list that tail code keeps in LDS as floats
constexpr uint32_t kTailLds = kDynLds + (kHeadGroups - 8u) * 1024u; // dynamic LDS of the kernels that cut and draw
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

// A slice's record from device memory (two 128-bit loads through a pointer typed as device memory, see as_global()).
__device__ __forceinline__ SliceStat load_slice_stat(const SliceStat* stats, size_t i)
{
    static_assert(sizeof(SliceStat) == 32, "two 128-bit loads");
    const global_ptr<const u32x4> sp = (global_ptr<const u32x4>)(as_global(stats) + i);
    const u32x4 s0 = sp[0], s1 = sp[1];
    SliceStat st;
    st.wmax = __uint_as_float(s0.x);
    st.argidx = s0.y;
    st.flags = s0.z;
    st.n_emit = s0.w;
    st.tau_key = s1.x;
    st.above = s1.y;
    st.pad[0] = st.pad[1] = 0;
    return st;
}

// A logit's unit for the coarse counts of log_bins.h.
__device__ __forceinline__ float log_unit_scale(const mako_sampling_params& P)
{
    return (1.0f / P.temperature) * (1.4426950408889634f * (float)kLogUnitsPerOctave);
}
__device__ __forceinline__ int32_t log_unit(float logit, float scale)
{
    // floor and conversion in one instruction that saturates at the limits and turns NaN into 0: the same for every
    // kernel that asks, which is all that matters here
    int32_t k;
    asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(k) : "v"(logit * scale));
    return k;
}

constexpr uint32_t kWorkers = 32;  // workgroups that share the sort of one wide-nucleus row
constexpr uint32_t kStageSlack = 64; // room a worker's share of the staging arrays gets beyond what the coarse counts
                                     // promise (and 1/64 of that count); the rows' arrays are sized to hold it
constexpr uint32_t kGroup = 256;      // a sorted list is processed in groups of one wave x four entries per lane
constexpr uint32_t kMaxGroups = 1024; // groups per list
constexpr uint32_t kSegCap = 6144;    // entries a worker sorts in LDS
constexpr uint32_t kFine = 2048;      // value buckets of that sort
// dynamic LDS of sort_kernel: the entries, the entries again in the order of their buckets, the buckets, and a copy
// of the sorted weights for the group records
constexpr uint32_t kSortLds = kSegCap * 8u + kSegCap * 8u + (kFine + 4u) * 4u + kSegCap * 4u;
constexpr uint32_t kSortedCopyAt = kSegCap * 8u + kSegCap * 8u + (kFine + 4u) * 4u; // byte offset of that copy

// Work order for a top_k == 0 row, written by the second pass (every workgroup of the row derives the same one from
// scan_kernel's coarse counts, see coarse_plan(); the row's first piece stores it): the weights with bits(q) >= thr
// are split by value into kWorkers contiguous ranges of about equal size, handed to the workers' shares as they are
// computed, sorted by sort_kernel and cut and drawn from by tail_kernel.
struct BigPlan {
    uint32_t flag;   // 1: the row waits for sort_kernel's workers and tail_kernel; 2: for the whole-row path (in
                     // tail_kernel's launch); 3: a narrow nucleus, finished by worker 0 from the candidate lists;
                     // 4: one that the lists could not certify (second look in tail_kernel's launch)
    uint32_t n0;     // entries of the sorted list (sort_kernel's worker 0 adds up what the workers were handed)
    uint32_t overflow; // set by the second pass when a worker's share did not fit its room (then flag 2 follows)
    uint32_t groups; // groups of the whole list: each worker's range is cut into groups of kGroup on its own
    double total64;  // exact fp64 sum of q over the row's candidates (worker 0)
    uint32_t thr;    // bits(q) from which weights are kept
    uint32_t argidx; // first index of the row's maximum, and the maximum (for the whole-row path)
    float m;
    uint32_t opq_mask; // workers whose shares are left unsorted, as one record each (unsorted_shares.h)
    double mass_all; // the plan's estimate of the row's total, in the units of mass[]
    uint32_t key_lo[kWorkers];    // worker w takes bits(q) in [key_lo[w], key_lo[w - 1]) (worker 0: up to 1.0)
    uint32_t stage_off[kWorkers]; // where its share starts in the row's staging arrays (Scratch::key[1], idx[1])
    uint32_t cap[kWorkers];       // and how many entries it has room for
    uint32_t cursor[kWorkers];    // entries handed to worker w so far (zeroed by scan_kernel)
    double mass[kWorkers];        // estimated sum of the weights above worker w's range
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
    uint4* walk;     // the group's map for the walk (d0, d1, the bound of group_sub_ok, exponent) in the epoch guessed
                     // for r at the group; exponent 0: none
};

// The large batches' work lists of sort_kernel.  Workgroups are dispatched in the order of their numbers, to the XCDs
// in turn, and the next one waits for a CU of ITS XCD: with entries of unequal cost in row order the XCDs fall out of
// step and CUs idle (a quarter of the time on config 4).  So the costliest entries, the collectors of unsorted shares
// (up to two per row, ~19 us), come first and together, then the workers that sort (~13 us) and the narrow rows
// (~10 us).  A workgroup without an entry costs nothing behind the last one with work, but between two of them it
// waits for a CU like any other: the collectors' list is filled from its end backwards (work_n[3] of them, the last at
// workgroup number sorted_at - 1), the others' forwards from sorted_at (work_n[0]), so that no gap lies between.
constexpr uint32_t kSortItemsPerRow = kWorkers + 2u;
struct SortLists {
    uint32_t sorted_at; // first workgroup number (= entry of work_sort) of the workers that sort and the narrow rows
};
__host__ __device__ inline SortLists large_batch_lists(uint32_t n_rows)
{
    return SortLists{2u * n_rows};
}

struct Scratch {
    SliceStat* stats;  // [max_rows][kMaxSlices]
    float* cand_w;     // [max_rows][slices_cap][kCap] penalised logits of the slice's candidates
    uint32_t* cand_i;  // [max_rows][slices_cap][kCap] their token ids
    double* part_sum;  // [max_rows][kMaxSlices] exact fp64 sum of q over the slice (top_k == 0 rows)
    BigPlan* plan;     // [max_rows]; flag zero between calls
    float* wbuf;       // [max_rows][vpad] penalised logits of rows on the whole-row path, then bits(q) of every logit
                       // (0 where q is not a candidate)
    uint32_t* cnt;     // [max_rows][vpad] token counts; all zero between calls
    uint32_t* key[2];  // [max_rows][vpad] candidate keys (~bits(q)), ping-pong; [1] also takes the workers' unsorted
                       // shares (bits(q)) from the second pass
    uint32_t* idx[2];  // [max_rows][vpad] candidate token ids, likewise
    uint16_t* log_hist;  // [max_rows][slices_cap][kLogBins] top_k == 0 rows: logits of the slice per bin of the slice's
                         // own frame (log_bin_in_frame(); a slice holds 16384 logits at most)
    GroupTable gt;     // [max_rows][g_cap] each
                       // (kept at a multiple of 16 bytes: the kernels' LDS copies of this record are read with
                       // 128-bit operations, which stall on anything less)
    // Work lists.  sort_kernel and tail_kernel are launched with one workgroup per POSSIBLE piece of work, but
    // workgroup i serves entry i of its kernel's list and exits if there is none: the busy workgroups are then the
    // first ones dispatched and land evenly on the XCDs, shader engines and CUs, whatever the mix of rows.
    // (finish_kernel and plan_kernel get the same effect from find_piece().)
    uint32_t* work_n;      // [8] entries in work_sort, work_tail (zeroed by scan_kernel); [3]: the large batches' collectors; [2]: failed checks of a checked
                           // build (MAKO_CHECK); then, 16-byte aligned at [4], how the second pass is cut up
                           // (SecondPassCut; scan_kernel's first workgroup decides)
    uint32_t* work_sort;   // [max_rows * kSortItemsPerRow] row << 8 | worker; appended by finish_kernel.  The large batches'
                           // instances keep two lists in it that meet, the costliest entries in front (large_batch_lists())
    uint32_t* work_tail;   // [max_rows] row; appended by finish_kernel
    uint64_t vpad;
    uint32_t slices_cap;
    uint32_t g_cap;    // vpad / kGroup + kWorkers
};

static_assert(offsetof(Scratch, gt) % 16 == 0 && sizeof(mako_sample_desc) % 16 == 0, "128-bit LDS reads of the staged records");

// Checked builds (-DMAKO_CHECKED, libmako_sampler_checked.so): every index a kernel computes into the context's scratch
// arrays from counts that other kernels left is compared with the array's bound before it is used, and a failed
// comparison sets a bit of Scratch::work_n[2] (nothing traps; mako_sampler_debug_checks() reads and clears the word).
// The shipped library compiles the checks to nothing: its hot code clamps where it must and assumes the rest.
enum CheckBit {
    kCheckCandSlot = 0,   // scan_kernel: a candidate's slot in its slice's list
    kCheckStage = 1,      // second pass: an entry's place in the row's staging arrays
    kCheckShare = 2,      // sort_kernel: a worker's share and its place in the sorted list
    kCheckGroups = 3,     // sort_kernel: a worker's group records
    kCheckTailGroup = 4,  // tail_kernel: the list's length and group count as sort_kernel left them
    kCheckCompact = 5,    // the whole-row path: a candidate's place in the compacted list
    kCheckAlive = 31,     // set by every batch of a checked build: the checks are compiled in and their word is read
};
#ifdef MAKO_CHECKED
#define MAKO_CHECK(sc, bit, cond)                                                                                    \
    do {                                                                                                             \
        if (!(cond))                                                                                                 \
            atomicOr(&(sc).work_n[2], 1u << (bit));                                                                  \
    } while (0)
#else
#define MAKO_CHECK(sc, bit, cond) ((void)0)
#endif

// Device functions that only rare rows reach (the whole-row path, the second look at a cut that is too close to
// call).  The sources whose kernels have a hot path beside them are compiled with MAKO_RARE_CALL=__attribute__((noinline)):
// inlined, such code costs the hot path registers and spills.
#ifndef MAKO_RARE_CALL
#define MAKO_RARE_CALL
#endif

// The reference adds a row's weights one after the other in fp64 (src/gen/sampler.cpp:46-48 in candidate order,
// :55-56 in sorted order); the sums here associate differently (per thread, wave and workgroup; bin masses).  An
// fp64 sum of n fp32 addends in ANY order lies within n * 2^-53 * total of the exact sum, so two orders differ by at
// most twice that; order_band() is that bound with room for the roundings of the product top_p * total and of the
// tree sums themselves.  A cut whose two neighbouring prefix sums both clear `want` by more than the band is the
// reference's cut; any other is decided by wave_sequential_sum() on the reference's own order.
__device__ __forceinline__ double order_band(uint32_t n_addends, double total64)
{
    return (double)(n_addends + 64u) * 0x1p-51 * total64;
}

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

// Rows that are cut neither to a top-k nor to a nucleus: their candidates stay in token order.  With the caller's host
// copy of the parameters such rows get kernels of their own (index_rows.h), which hand a row on through BigPlan::flag:
__host__ __device__ __forceinline__ bool index_order_row(const mako_sampling_params& p)
{
    return p.temperature > 0.0f && !(p.top_p < 1.0f) && p.top_k == 0u;
}
constexpr uint32_t kIndexClaimed = 6; // index_weights_kernel has the row: the kernels that finish late rows leave it alone
constexpr uint32_t kIndexReady = 7;   // the group records are in place
constexpr uint32_t kIndexWhole = 8;   // the whole-row path is wanted (candidates to be written out from a list with gaps)
constexpr uint32_t kIndexEmpty = 9;   // no candidate survived
// (BigPlan::n0 of a claimed row of another kind, from index_weights_kernel to index_tail_kernel: the whole-row path's
// list was written beside the weights, and is the row's list of candidates if every logit turns out to be one)
constexpr uint32_t kIndexListed = 1;

__device__ __forceinline__ bool penalties_neutral(const mako_sampling_params& p)
{
    return p.repetition_penalty == 1.0f && p.presence_penalty == 0.0f && p.frequency_penalty == 0.0f;
}

} // namespace mako
