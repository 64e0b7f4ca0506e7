// A thread's sixteen logits of a slice: loaded, masked and penalised (src/gen/sampler.cpp:22-28).
#pragma once

#include "sampler_common.h"

namespace mako {

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
    const global_ptr<const int32_t> ht = as_global(d.hist_tokens) + (int64_t)row * d.hist_stride;
    const global_ptr<const uint32_t> hc = d.hist_counts ? as_global(d.hist_counts) + (int64_t)row * d.hist_stride : nullptr;
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
    const global_ptr<const float> lrow = as_global(d.logits) + (int64_t)row * d.logits_stride;
    const global_ptr<const uint32_t> mrow = d.mask ? as_global(d.mask) + (int64_t)row * d.mask_stride : nullptr;
    const float nan = __uint_as_float(0x7fc00000u);
    if (VEC) {
        // all four loads go out back to back, from clamped addresses and without a branch between them (a branch
        // would make the compiler wait for each load before the next); what lies past the slice is dropped after
        uint32_t at[4];
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint32_t i = lo + k * 4096u + tid * 4u;
            at[k] = i < hi ? i : hi - 4u; // hi - lo is a positive multiple of 4 in this mode
            const f32x4 x = *(global_ptr<const f32x4>)(lrow + at[k]);
            r.v[k] = make_float4(x.x, x.y, x.z, x.w);
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
        // (a mask bit spread over a word, then one bit-field insert: the logit where the bit is set, -inf elsewhere)
        const float nan = __uint_as_float(0x7fc00000u);
        auto pick = [](uint32_t bits, uint32_t c, float v) {
            const uint32_t m = (uint32_t)((int32_t)(bits << (31u - c)) >> 31); // all ones if bit c is set
            return __uint_as_float((__float_as_uint(v) & m) | (0xff800000u & ~m));
        };
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const bool inside = lo + k * 4096u + tid * 4u < hi;
            wv[4 * k + 0] = !inside ? nan : pick(r.bits[k], 0, r.v[k].x);
            wv[4 * k + 1] = !inside ? nan : pick(r.bits[k], 1, r.v[k].y);
            wv[4 * k + 2] = !inside ? nan : pick(r.bits[k], 2, r.v[k].z);
            wv[4 * k + 3] = !inside ? nan : pick(r.bits[k], 3, r.v[k].w);
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
    const global_ptr<const int32_t> ht = as_global(d.hist_tokens) + (int64_t)row * d.hist_stride;
    const global_ptr<const uint32_t> hc = d.hist_counts ? as_global(d.hist_counts) + (int64_t)row * d.hist_stride : nullptr;
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

} // namespace mako
