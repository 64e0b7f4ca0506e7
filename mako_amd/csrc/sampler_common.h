// Constants, the context's scratch layout, order keys and the classification of rows: shared by every kernel
// of the sampler.
#pragma once

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <type_traits>
#include "../../include/mako_sampler.h"
#include "block_prims.h"
#include "device_math.h"
#include "seqfp.h"
#include "tuning_stamps.h"

namespace mako {

constexpr uint32_t kNone = 0xffffffffu;

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

// Weights of a top_k == 0 row that its nucleus cannot reach, as a histogram bin: every weight in a bin below the
// returned one is smaller than (1 - top_p) / (2 top_p V).  Why such a weight x lies outside: the row's maximum
// weighs 1, so the weights ahead of x in the sorted order sum to A >= 1, the row's total is below A + V x, and
// top_p * total < top_p A + (1 - top_p) / 2 <= A - (1 - top_p) A / 2: the running sum has passed the cut before x
// is reached (src/gen/sampler.cpp:46-58), by a margin far above any rounding.  0 = nothing is left out.
__device__ __forceinline__ uint32_t prune_bin(const mako_sampling_params& P, uint32_t n_vocab)
{
    const float p = P.top_p;
    if (!(p > 0.0f && p < 1.0f))
        return 0u;
    const float q = ((1.0f - p) / (p * (float)n_vocab)) * 0.5f;
    if (!(q > 0.0f))
        return 0u;
    return weight_bin(min(__float_as_uint(q), 0x7f800000u));
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
// entries of sort_kernel's work list: row << 8 | worker (below kWorkers), or
constexpr uint32_t kItemWhole = 65u;  // a row (of any class) on the whole-row path
constexpr uint32_t kGroup = 256;      // a sorted list is processed in groups of one wave x four entries per lane
constexpr uint32_t kMaxGroups = 1024; // groups per list
constexpr uint32_t kSegCap = 6144;    // entries a worker sorts in LDS
constexpr uint32_t kFine = 2048;      // value buckets of that sort
// dynamic LDS of sort_kernel: the entries, their order, the buckets, and a copy of the sorted weights for the group
// records
constexpr uint32_t kSortLds = kSegCap * 8u + kSegCap * 2u + (kFine + 4u) * 4u + kSegCap * 4u;
constexpr uint32_t kSortedCopyAt = kSegCap * 8u + kSegCap * 2u + (kFine + 4u) * 4u; // byte offset of that copy
// A piece of the second pass over a top_k == 0 row: kPieceBlocks blocks of 4096 logits, eight logits per thread.
constexpr int kPieceBlocks = 2;
constexpr uint32_t kPieceLen = kPieceBlocks * 4096u;
// dynamic LDS of second_kernel: the piece's staged weights and their indices inside the piece (kPieceLen x (4 + 2)
// bytes; the token counts of the penalties, kPieceLen x 4, lie over the front of them earlier in the pass), the
// histogram of the row's sampled weights (kBins x 4), the bin -> worker table (kBins x 1), per wave and worker the
// weights handed over with their mass (kWaves x kWorkers x 8) and their first places (kWaves x kWorkers x 4), and
// the cuts between the workers (kWorkers x 4)
constexpr uint32_t kSamples = 1024; // weights of the row every piece looks at to split the row among its workers
constexpr uint32_t kSecondKeysAt = 0u;
constexpr uint32_t kSecondIdxAt = kSecondKeysAt + kPieceLen * 4u;
constexpr uint32_t kSecondHistAt = kSecondIdxAt + kPieceLen * 2u;
constexpr uint32_t kSecondTableAt = kSecondHistAt + kBins * 4u;
constexpr uint32_t kSecondCntAt = kSecondTableAt + kBins;
constexpr uint32_t kSecondOffAt = kSecondCntAt + 16u * kWorkers * 8u;
constexpr uint32_t kSecondCutAt = kSecondOffAt + 16u * kWorkers * 4u;
constexpr uint32_t kSecondLds = kSecondCutAt + kWorkers * 4u;
// a (wave, worker) counter of the second pass: weights handed over << kMassBits | their mass in units of 2^-30
constexpr uint32_t kMassBits = 48;
constexpr uint32_t kShareTarget = 3072; // weights per worker the split aims at (a worker sorts up to kSegCap in LDS)

// What the kernels behind the second pass hand each other about a top_k == 0 row.
struct BigPlan {
    uint32_t flag;    // 1: tail_kernel finishes the row from the workers' sorted list; 2: a row (of any class) that
                      // waits for sort_kernel's whole-row path
    uint32_t n0;      // entries of the sorted list (sort_kernel's worker 0); for flag 2: first index of the row maximum
    uint32_t workers; // workers that share the row (second_kernel)
    uint32_t groups;  // groups of the whole list: each worker's range is cut into groups of kGroup on its own
    double total64;   // for flag 2: the row maximum
    uint32_t thr;     // bits(q) of the lightest weight the second pass kept: the list holds every weight >= it
    uint32_t pad;
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
    BigPlan* plan;     // [max_rows]; flag zero between calls
    float* wbuf;       // [max_rows][vpad] penalised logits of rows on the whole-row path; also the second buffer
                       // (with idx[1]) of a worker whose share does not fit one LDS sort
    uint32_t* cnt;     // [max_rows][vpad] token counts; all zero between calls
    uint32_t* key[2];  // [max_rows][vpad] candidate keys (~bits(q)), ping-pong.  For top_k == 0 rows [1] holds the
                       // second pass's pieces instead: piece p's kept weights (bits(q)), ordered by the worker they
                       // are for, from position p * piece length
    uint32_t* idx[2];  // [max_rows][vpad] candidate token ids, likewise
    uint16_t* piece_idx; // [max_rows][vpad] beside key[1]: each kept weight's index inside its piece
    uint32_t* piece_tab; // [max_rows][pieces_cap][kWorkers + 1] kept weights of the piece for workers below w, every w
    unsigned long long* piece_mass; // [max_rows][pieces_cap][kWorkers] sum of the piece's weights for worker w, in
                                    // units of 2^-30 (what the workers guess the running sum's binade from)
    double* piece_sum;   // [max_rows][pieces_cap] fp64 sum of q over the piece's candidates, in a fixed order
    uint32_t* piece_cnt; // [max_rows][pieces_cap] candidates (q > 0, q >= min_p) in the piece
    GroupTable gt;     // [max_rows][g_cap] each
    // Work lists.  sort_kernel and tail_kernel are launched with one workgroup per POSSIBLE piece of work, but
    // workgroup i serves entry i of its kernel's list and exits if there is none: the busy workgroups are then the
    // first ones dispatched and land evenly on the XCDs, shader engines and CUs, whatever the mix of rows.
    // (finish_kernel and plan_kernel get the same effect from find_piece().)
    uint32_t* work_n;      // [8] entries in work_sort, work_tail (zeroed by scan_kernel); at [4] the number of top_k == 0
                           // rows (scan_kernel's first workgroup, see nucleus_rows())
    uint32_t* work_rows;   // [max_rows] the batch's top_k == 0 rows, in row order (scan_kernel's first workgroup)
    uint32_t* work_sort;   // [max_rows * kWorkers] sort_kernel's work: row << 8 | worker (a top_k == 0 row) or
                           // kItemWhole; appended by second_kernel / rows_kernel
    uint32_t* work_tail;   // [max_rows] rows whose workers leave a sorted list; appended by second_kernel
    uint64_t vpad;
    uint32_t slices_cap;
    uint32_t pieces_cap;   // pieces of kPieceLen logits a row of max_vocab logits has
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

} // namespace mako
