// scan_kernel: the single pass over the logits in device memory.
#pragma once

#include "slice_load.h"
#include "work_split.h"

namespace mako {

struct alignas(16) ScanShared {
    uint32_t wave_max[kWaves]; // order keys
    uint32_t wave_kth[kWaves];
    uint32_t wave_above[kWaves];
    uint32_t argidx;
    uint32_t emit_n;
    uint32_t emit_flags;
    float cw[kCap];
    uint32_t ci[kCap];
    uint32_t log_hist[kLogBins + kWave]; // top_k == 0 rows (and one slot per lane for what is not counted)
};

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

// (ABOVE: the batch has close tokens, whose logits' ranks are counted on the way; a variant of its own because the
// count takes sixteen more registers, up to the limit for two workgroups per CU, which no other batch should pay)
// (amdgpu_waves_per_eu: the vectorised variants are held to the 64 registers that let two workgroups share a CU)
template <bool VEC, int KH, bool ABOVE = false>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(VEC ? 8 : 4))) void scan_kernel(mako_sample_desc d, Scratch sc_arg, uint32_t slice_len,
                                                        uint32_t cus_and_grid)
{
    // (cus_and_grid: the CUs of the device, and in the upper half an eighth of finish_kernel's grid: second_pass_cut())
    // (scan_kernel takes the context's record by value: its first loads then need no trip to memory for a pointer)
    const Scratch& sc = sc_arg;
    MAKO_ROW(d.hist_tokens ? blockIdx.x : blockIdx.y);
#ifdef MAKO_TIMING_SCAN
    MAKO_WG_TIMER;
#endif
    // (16-byte alignment: the table is cleared and read with 128-bit LDS operations, which crawl when misaligned)
    extern __shared__ __align__(16) uint32_t s_dyn[]; // [slice_len] token counts when the row has penalties
    __shared__ ScanShared sm;

    // grid = (slices, rows), or, for a batch with histories, (rows rounded up to a multiple of 8, slices):
    // workgroups go to the eight XCDs in turn, so with the row in x all slices of a row run on one XCD and its L2
    // fetches the row's history from memory once, not eight times (-10 % of the kernel's fetches on a decode batch
    // with 2048-token histories).  Without histories the first form is 2-4 % faster on batches of 256 rows.
    const bool row_in_x = d.hist_tokens != nullptr; // uniform
    const uint32_t row = row_in_x ? blockIdx.x : blockIdx.y, slice = row_in_x ? blockIdx.y : blockIdx.x, tid = threadIdx.x;
    const uint32_t n_slices = row_in_x ? gridDim.y : gridDim.x;
    if (row >= d.n_rows)
        return;
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
            sc.work_n[3] = 0;
            MAKO_CHECK(sc, kCheckAlive, false);
        }
    }
    static_assert(kLogBins == (uint32_t)kThreads, "one bin per thread");
    if (cls == kNucleus) {
        sm.log_hist[tid] = 0;
        if (slice == 0) { // what the second pass adds to starts at zero
            if (tid < kWorkers)
                sc.plan[row].cursor[tid] = 0;
            if (tid == 0)
                sc.plan[row].overflow = 0;
        }
    }
    if (row == 0 && slice == 0 && wave_id() == 1) { // how the second pass will be cut up
        const SecondPassCut cut = second_pass_cut(d, n_slices, slice_len, cus_and_grid & 0xffffu, (cus_and_grid >> 16) * 8u);
        if (lane_id() == 0)
            *reinterpret_cast<uint4*>(sc.work_n + 4) = make_uint4(cut.per_row, cut.piece_len, cut.busy, cut.pieces);
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
        // Slots in the slice's list.  Candidates are few (a percent or three of the logits): for each of the sixteen
        // positions j a ballot says which lanes hold one, the counts add up in scalar registers, one lane reserves
        // the wave's run with a single LDS atomic, and only the positions with a candidate in some lane cost vector
        // instructions at all (a lane's slot: the run's start, the candidates of earlier positions, and the set
        // bits below the lane).  The order inside the list is by position, then lane; nobody depends on it.
        unsigned long long takes[16];
        uint32_t wave_total = 0;
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j) {
            takes[j] = __ballot(wv[j] >= tau);
            wave_total += (uint32_t)__popcll(takes[j]);
        }
        if (wave_total) { // uniform
            uint32_t base = 0;
            if (lane_id() == 0)
                base = atomicAdd(&sm.emit_n, wave_total);
            uint32_t run = (uint32_t)__builtin_amdgcn_readfirstlane((int)base);
#pragma unroll
            for (uint32_t j = 0; j < 16; ++j) {
                if (takes[j]) { // uniform
                    const uint32_t pos =
                        run + __builtin_amdgcn_mbcnt_hi((uint32_t)(takes[j] >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)takes[j], 0u));
                    const float w = wv[j];
                    if (w >= tau && pos < kCap) {
                        sm.cw[pos] = w;
                        sm.ci[pos] = elem_index<VEC>(lo, tid, j);
                    }
                    run += (uint32_t)__popcll(takes[j]);
                }
            }
        }
    }
    if (cls == kNucleus) {
        // the slice's logits by unit, in the frame of the slice's maximum (log_slot_in_frame()); what the bins do not
        // cover (and NaN) goes to slot kLogBins - 1, which is no bin, or to one of the spare slots up to the lane's own
        const float scale = log_unit_scale(P);
        const int32_t k_top = log_unit(st.wmax, scale);
        const uint32_t spare_end = kLogBins + (uint32_t)lane_id();
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j)
            atomicAdd(&sm.log_hist[log_slot_in_frame(log_unit(wv[j], scale), k_top, spare_end)], 1u);
    }
    __syncthreads();
    MAKO_STAMP(31);
    if (cls == kNucleus && tid < kLogBins / 2u) { // (two 16-bit counts per store)
        static_assert(kSliceMax < 65536u, "a bin's count fits sixteen bits");
        // (slot kLogBins - 1 took logits that no bin covers: it is stored as zero)
        reinterpret_cast<uint32_t*>(sc.log_hist + ((size_t)row * sc.slices_cap + slice) * kLogBins)[tid] =
            sm.log_hist[2u * tid] | (2u * tid + 1u < kLogBins - 1u ? sm.log_hist[2u * tid + 1u] << 16 : 0u);
    }
    if (emits) {
        const uint32_t n = sm.emit_n;
        if (n > kCap)
            st.flags |= kFlagOverflow;
        st.n_emit = min(n, kCap);
        st.tau_key = tau_key;
        const size_t base = ((size_t)row * sc.slices_cap + slice) * kCap;
        MAKO_CHECK(sc, kCheckCandSlot, st.n_emit <= kCap && slice < sc.slices_cap);
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

} // namespace mako
