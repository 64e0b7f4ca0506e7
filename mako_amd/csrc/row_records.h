// What scan_kernel's slice records say about a row: maximum, candidate totals, forced tokens.
#pragma once

#include "workgroup_state.h"

namespace mako {

// First maximum of the row (std::max_element semantics, NaNs never win unless at index 0) and the totals of the
// slices' candidate lists, from the records scan_kernel left.
// (`st`: the record of slice min(lane, slices - 1), already loaded)
__device__ __forceinline__ void row_summary_of(const SliceStat& st, uint32_t slices, float& m, uint32_t& argidx,
                                               uint32_t& n_cands, uint32_t& any_overflow)
{
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
__device__ __forceinline__ void row_summary(const Scratch& sc, uint32_t row, uint32_t slices, float& m, uint32_t& argidx,
                                            uint32_t& n_cands, uint32_t& any_overflow, SliceStat* lane_stat = nullptr)
{
    // lane s of every wave takes slice s (at most kMaxSlices = 64 of them): one load each, then wave reductions
    const SliceStat st = load_slice_stat(sc.stats, (size_t)row * kMaxSlices + min((uint32_t)lane_id(), slices - 1u));
    if (lane_stat)
        *lane_stat = st;
    row_summary_of(st, slices, m, argidx, n_cands, any_overflow);
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

} // namespace mako
