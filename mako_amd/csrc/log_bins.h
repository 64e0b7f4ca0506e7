// Coarse bins of a top_k == 0 row's logits by the weight they will have: the integer arithmetic, shared by
// scan_kernel (which counts), the second pass (which plans from the counts) and a host unit test.
//
// A logit's `unit` is floor(logit * scale) with scale = kLogUnitsPerOctave * log2(e) / T: one unit is
// 1/kLogUnitsPerOctave of a factor of two of the weight the logit will have, and the unit is a function of the logit
// and the row's temperature alone.  scan_kernel counts each slice's penalised logits by unit, in the frame of the
// slice's own maximum: one bin per unit for the kLogFine units at and below the maximum's (near-flat rows, whose
// weights all lie within a factor of two, still spread over hundreds of bins), one bin per aligned group of
// 2^kLogCoarseShift units below that (34 octaves in all; what lies further down is not counted).  Units and groups
// are absolute, so the second pass can move every slice's counts into the frame of the row's maximum with integer
// arithmetic alone, exactly, and size its work from them before it has computed a single weight.  Nothing exact is
// ever decided from these counts: they balance work and size buffers, and every list built from them is checked
// against the exact sums afterwards.
//
// This header is plain C++ so that the host test and the HIP kernels share one implementation.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define LOGBINS_HD __host__ __device__ __forceinline__
#else
#define LOGBINS_HD inline
#endif

namespace mako {

constexpr uint32_t kLogBins = 1024;
constexpr uint32_t kLogUnitsPerOctave = 256;
constexpr uint32_t kLogFine = 512;
constexpr uint32_t kLogCoarseShift = 4;
constexpr uint32_t kLogNotCounted = kLogBins; // what log_bin_in_frame() answers for a unit outside the bins

// (arithmetic shift of a possibly negative unit: floor division by the group size)
LOGBINS_HD int32_t log_group(int32_t k)
{
    return k >> kLogCoarseShift;
}
// The group of the first coarse bin in the frame of a maximum whose unit is k_top.
LOGBINS_HD int32_t log_first_group(int32_t k_top)
{
    return log_group((int32_t)((uint32_t)k_top - kLogFine));
}

// Bin of unit k in the frame of a maximum whose unit is k_top: bins 0 .. kLogBins - 2, or kLogNotCounted.
// (unsigned arithmetic: units at the limits wrap instead of overflowing, and end up "not counted")
LOGBINS_HD uint32_t log_bin_in_frame(int32_t k, int32_t k_top)
{
    const uint32_t d = (uint32_t)k_top - (uint32_t)k;
    const uint32_t c = (uint32_t)(log_first_group(k_top) - log_group(k));
    return d < kLogFine ? d : (c < kLogBins - 1u - kLogFine ? kLogFine + c : kLogNotCounted);
}

// The same for counting in a table of kLogBins slots followed by spare ones: a unit outside the bins lands in slot
// kLogBins - 1 (which is no bin) or in a spare slot, never beyond slot `spare_end` (>= kLogBins - 1); two operations
// fewer per logit than a test and a choice.
LOGBINS_HD uint32_t log_slot_in_frame(int32_t k, int32_t k_top, uint32_t spare_end)
{
    const uint32_t d = (uint32_t)k_top - (uint32_t)k;
    const uint32_t c = (uint32_t)(log_first_group(k_top) + (int32_t)kLogFine - log_group(k)); // kLogFine + coarse bin
    return d < kLogFine ? d : (c < spare_end ? c : spare_end);
}

// A unit of bin b of the frame of k_top (the bin's only one if the bin is fine, the lowest of its group otherwise):
// log_bin_in_frame() of it, in the frame of any maximum at or above k_top, is where the bin's logits belong there.
LOGBINS_HD int32_t log_bin_unit(uint32_t b, int32_t k_top)
{
    return b < kLogFine ? (int32_t)((uint32_t)k_top - b)
                        : (int32_t)((uint32_t)(log_first_group(k_top) - (int32_t)(b - kLogFine)) << kLogCoarseShift);
}

// Where the logits of bin b of a slice's frame (maximum k_slice) belong in the frame of the row's maximum k_top
// (>= k_slice): log_bin_in_frame(log_bin_unit(b, k_slice), k_top) with less arithmetic.  A coarse bin is a group of
// units and stays one: only its number changes, by the distance between the two frames' first groups.
// (Equal to that composition for units within +-2^30, which is what the host test checks; beyond, where the units
// of log_unit() saturate anyway, the two may name different bins, which costs balance and nothing else.)
LOGBINS_HD uint32_t log_bin_moved(uint32_t b, int32_t k_slice, int32_t k_top)
{
    if (b >= kLogFine) {
        const uint32_t c = b + (uint32_t)(log_first_group(k_top) - log_first_group(k_slice));
        return c < kLogBins - 1u ? c : kLogNotCounted;
    }
    return log_bin_in_frame((int32_t)((uint32_t)k_slice - b), k_top);
}

// The lowest unit that lies above every unit of bin b (b >= 1) in the frame of k_top: logits whose unit is at
// least this one are in the bins before b.
LOGBINS_HD int32_t log_bin_upper_edge(uint32_t b, int32_t k_top)
{
    return b <= kLogFine ? (int32_t)((uint32_t)k_top - b + 1u)
                         : (int32_t)((uint32_t)(log_first_group(k_top) - (int32_t)(b - kLogFine) + 1) << kLogCoarseShift);
}

// How far below the maximum (its unit k_top) the middle of bin b lies, in units, counted from the lower edge of the
// maximum's unit.
LOGBINS_HD float log_bin_middle(uint32_t b, int32_t k_top)
{
    if (b < kLogFine)
        return (float)b - 0.5f;
    const int32_t g = log_first_group(k_top) - (int32_t)(b - kLogFine);
    const int32_t lowest = (int32_t)((uint32_t)k_top - ((uint32_t)g << kLogCoarseShift)); // distance of the group's lowest unit
    if (b == kLogFine) // (the first group's upper units belong to the fine bins)
        return 0.5f * (float)((int32_t)kLogFine - 1 + lowest);
    return (float)(lowest - (1 << (kLogCoarseShift - 1)));
}

} // namespace mako
