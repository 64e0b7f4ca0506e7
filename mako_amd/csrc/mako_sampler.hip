// MI355X (gfx950) token sampler: HIP kernels and the C ABI of include/mako_sampler.h.
//
// Pipeline per batch (rows are independent, src/gen/session.cpp:416):
//   scan_kernel    one workgroup per (row, slice): a single coalesced pass over the fp32 logits that
//                  applies the token mask and the history penalties in registers and leaves per-slice
//                  maxima (and, for the fast paths, per-slice candidate lists) in scratch.
//   finish_kernel  one workgroup per row: greedy argmax, or weights q = expf((w - m) / T), top-k,
//                  top-p and the categorical draw with the reference's exact fp32 rounding order.
#include <hip/hip_runtime.h>

#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <new>
#include <string>

#include "../../include/mako_sampler.h"
#include "block_prims.h"
#include "device_math.h"
#include "seqfp.h"

namespace mako {

constexpr uint32_t kNone = 0xffffffffu;
constexpr uint32_t kSliceMax = 16384; // elements per slice: 16 per thread
constexpr uint32_t kMaxSlices = 64;

struct SliceStat {
    float wmax;      // max of the slice's penalised logits (-inf if none compares greater)
    uint32_t argidx; // first index holding it, kNone if nothing exceeded -inf
    uint32_t flags;  // bit 0: element 0 of the row is NaN (slice 0 only)
    uint32_t pad;
};

struct Scratch {
    SliceStat* stats; // [max_rows][kMaxSlices]
    float* wbuf;      // [max_rows][vpad] penalised logits of rows on the general path
    uint32_t* cnt;    // [max_rows][vpad] token counts; all zero between calls
    uint32_t* key[2]; // [max_rows][vpad] candidate keys (~bits(q)), ping-pong
    uint32_t* idx[2]; // [max_rows][vpad] candidate token ids, ping-pong
    uint64_t vpad;
};

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

__device__ __forceinline__ bool greedy_row(const mako_sampling_params& p)
{
    return p.temperature <= 0.0f; // Sampler::greedy, src/gen/sampler.hpp:26
}

__device__ __forceinline__ bool penalties_neutral(const mako_sampling_params& p)
{
    return p.repetition_penalty == 1.0f && p.presence_penalty == 0.0f && p.frequency_penalty == 0.0f;
}

// ---------------------------------------------------------------------------------------------
// scan_kernel
// ---------------------------------------------------------------------------------------------

// grid = (slices, rows).  Thread t of slice s owns, for k = 0..3, the four consecutive logits at
// lo + k * 4096 + 4 * t (VEC) or the logits lo + j * 1024 + t (scalar): every load is coalesced
// and each logit is read from HBM exactly once.
template <bool VEC>
__global__ __launch_bounds__(kThreads) void scan_kernel(mako_sample_desc d, Scratch sc, uint32_t slice_len)
{
    extern __shared__ uint32_t s_cnt[]; // [slice_len] when the batch carries histories
    __shared__ BlockScratch bs;

    const uint32_t row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x;
    const uint32_t V = d.n_vocab;
    const uint32_t lo = slice * slice_len;
    const uint32_t hi = min(V, lo + slice_len);
    const mako_sampling_params P = d.params[row];
    const bool greedy = greedy_row(P);

    // accept() history -> per-token counts for this slice (src/gen/sampler.cpp:15-18, 23-28).
    // Greedy rows ignore the penalties (src/gen/sampler.cpp:77-78).
    const uint32_t hl = (d.hist_tokens && !greedy) ? d.hist_len[row] : 0u;
    const bool pen = hl > 0 && !penalties_neutral(P);
    if (pen) {
        for (uint32_t i = tid; i < slice_len; i += kThreads)
            s_cnt[i] = 0;
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

    const float* lrow = d.logits + (int64_t)row * d.logits_stride;
    const uint32_t* mrow = d.mask ? d.mask + (int64_t)row * d.mask_stride : nullptr;

    float best = -INFINITY;
    uint32_t bidx = kNone;
    bool first_nan = false;
    auto visit = [&](uint32_t i, float v, bool allowed) {
        if (!allowed)
            v = -INFINITY;
        if (pen) {
            const uint32_t n = s_cnt[i - lo];
            if (n)
                v = penalize(v, n, P.repetition_penalty, P.presence_penalty, P.frequency_penalty);
        }
        if (i == 0)
            first_nan = v != v;
        if (v > best) {
            best = v;
            bidx = i;
        }
    };

    if (VEC) {
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint32_t i = lo + k * 4096u + tid * 4u;
            if (i < hi) { // hi - lo is a multiple of 4 in this mode
                const float4 v = *reinterpret_cast<const float4*>(lrow + i);
                uint32_t bits = 0xfu;
                if (mrow)
                    bits = mrow[i >> 5] >> (i & 31u);
                visit(i, v.x, bits & 1u);
                visit(i + 1, v.y, bits & 2u);
                visit(i + 2, v.z, bits & 4u);
                visit(i + 3, v.w, bits & 8u);
            }
        }
    } else {
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j) {
            const uint32_t i = lo + j * kThreads + tid;
            if (i < hi) {
                const float v = lrow[i];
                const bool allowed = mrow ? ((mrow[i >> 5] >> (i & 31u)) & 1u) : true;
                visit(i, v, allowed);
            }
        }
    }

    const unsigned long long packed = ((unsigned long long)order_key(best) << 32) | (unsigned long long)(kNone - bidx);
    const unsigned long long top = block_max_u64(packed, bs);
    if (tid == 0) {
        SliceStat st;
        st.wmax = order_unkey((uint32_t)(top >> 32));
        st.argidx = kNone - (uint32_t)top;
        st.flags = (slice == 0 && first_nan) ? 1u : 0u;
        st.pad = 0;
        sc.stats[(size_t)row * kMaxSlices + slice] = st;
    }
}

// ---------------------------------------------------------------------------------------------
// finish_kernel
// ---------------------------------------------------------------------------------------------

struct FinishShared {
    BlockScratch bs;
    uint64_t tab[32];
    uint32_t hist[256];
    uint32_t run[256];
    uint32_t wcount[kWaves * 256];
    uint32_t flag;
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

// One stable counting-sort pass on bits [shift, shift + 8) of the keys, ascending.
// Returns false (and moves nothing) when every key has the same digit.
__device__ bool radix_pass(const uint32_t* ksrc, const uint32_t* isrc, uint32_t* kdst, uint32_t* idst, uint32_t n,
                           uint32_t shift, FinishShared& sm)
{
    const uint32_t tid = threadIdx.x;
    if (tid < 256)
        sm.hist[tid] = 0;
    if (tid == 0)
        sm.flag = 0;
    __syncthreads();
    for (uint32_t base = 0; base < n; base += kThreads) {
        const uint32_t i = base + tid;
        const bool valid = i < n;
        const uint32_t dg = valid ? ((ksrc[i] >> shift) & 255u) : 0u;
        const unsigned long long mm = match_digit(dg, valid);
        const unsigned long long below = mm & ((1ull << lane_id()) - 1ull);
        if (valid && below == 0)
            atomicAdd(&sm.hist[dg], (uint32_t)__popcll(mm));
    }
    __syncthreads();
    uint32_t mine = tid < 256 ? sm.hist[tid] : 0u;
    if (mine == n)
        sm.flag = 1;
    uint32_t tot;
    const uint32_t excl = block_excl_scan_u32(mine, tot, sm.bs); // barriers inside publish sm.flag
    if (sm.flag)
        return false;
    if (tid < 256)
        sm.run[tid] = excl;
    __syncthreads();
    for (uint32_t base = 0; base < n; base += kThreads) {
        for (uint32_t j = tid; j < kWaves * 256; j += kThreads)
            sm.wcount[j] = 0;
        __syncthreads();
        const uint32_t i = base + tid;
        const bool valid = i < n;
        const uint32_t key = valid ? ksrc[i] : 0u;
        const uint32_t dg = (key >> shift) & 255u;
        const unsigned long long mm = match_digit(dg, valid);
        const uint32_t rank = (uint32_t)__popcll(mm & ((1ull << lane_id()) - 1ull));
        if (valid && rank == 0)
            sm.wcount[wave_id() * 256 + dg] = (uint32_t)__popcll(mm);
        __syncthreads();
        if (tid < 256) {
            uint32_t acc = sm.run[tid];
            for (int w = 0; w < kWaves; ++w) {
                const uint32_t t = sm.wcount[w * 256 + tid];
                sm.wcount[w * 256 + tid] = acc;
                acc += t;
            }
            sm.run[tid] = acc;
        }
        __syncthreads();
        if (valid) {
            const uint32_t pos = sm.wcount[wave_id() * 256 + dg] + rank;
            kdst[pos] = key;
            idst[pos] = isrc[i];
        }
        __syncthreads();
    }
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
};

__device__ void write_row(const mako_sample_desc& d, uint32_t row, const RowOut& o)
{
    d.out_tokens[row] = o.token;
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

// The draw (and, when verifying, the accept/reject step) over the final candidate list
// key[0..n), idx[0..n): keys are ~bits(q).  src/gen/sampler.cpp:64-73, 79-83, 93-106.
__device__ void draw_from_list(const mako_sample_desc& d, uint32_t row, const uint32_t* key, const uint32_t* idx,
                               uint32_t n, uint32_t path, FinishShared& sm)
{
    const uint32_t tid = threadIdx.x;
    auto qat = [&](uint32_t i) { return __uint_as_float(~key[i]); };
    const float total = emulate_sum(qat, n, sm);
    const float u = d.u[row];
    RowOut o;
    o.n_cand = n;
    o.total = total;
    o.path = path;
    o.accepted = 0;
    if (d.out_cand_idx && d.out_cand_q)
        for (uint32_t j = tid; j < n && j < d.cand_cap; j += kThreads) {
            d.out_cand_idx[(size_t)row * d.cand_cap + j] = (int32_t)idx[j];
            d.out_cand_q[(size_t)row * d.cand_cap + j] = qat(j);
        }
    if (!d.draft) {
        const float span = total - 0.0f;
        const float prod = u * span;
        const uint32_t pos = emulate_walk(qat, n, prod + 0.0f, sm);
        o.token = (int32_t)idx[pos];
        o.q = qat(pos);
    } else {
        // position of the draft in the list, if it survived the truncation
        const int32_t draft = d.draft[row];
        uint32_t pd = kNone;
        for (uint32_t j = tid; j < n; j += kThreads)
            if ((int32_t)idx[j] == draft)
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
            auto qat2 = [&](uint32_t i) { return __uint_as_float(~key[i + (i >= pd ? 1u : 0u)]); };
            const float rest = total - q_draft;
            const float span2 = rest - 0.0f;
            const float prod2 = d.u2[row] * span2;
            const uint32_t pos = emulate_walk(qat2, n2, prod2 + 0.0f, sm);
            const uint32_t at = pos + (pos >= pd ? 1u : 0u);
            o.token = (int32_t)idx[at];
            o.q = qat(at);
        }
    }
    if (tid == 0)
        write_row(d, row, o);
}

// Whole-row path: exact for every parameter combination.  One workgroup rebuilds the penalised
// row in scratch, keeps the candidates, sorts them by (q desc, idx asc) when top-k or top-p is
// active, truncates, and draws.  src/gen/sampler.cpp:20-62.
__device__ void general_row(const mako_sample_desc& d, const Scratch& sc, uint32_t row, const mako_sampling_params& P,
                            float m, uint32_t argidx, FinishShared& sm)
{
    const uint32_t tid = threadIdx.x;
    const uint32_t V = d.n_vocab;
    float* wbuf = sc.wbuf + (size_t)row * sc.vpad;
    uint32_t* cnt = sc.cnt + (size_t)row * sc.vpad;
    uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
    uint32_t* key1 = sc.key[1] + (size_t)row * sc.vpad;
    uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
    uint32_t* idx1 = sc.idx[1] + (size_t)row * sc.vpad;
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

    // 2. weights and the min_p / q > 0 filter, compacted in index order (sampler.cpp:29-36)
    const float inv_t = 1.0f / P.temperature;
    const float floor_q = (1.0f < P.min_p) ? 1.0f : P.min_p; // std::min(min_p, 1.0f)
    uint32_t n0 = 0;
    for (uint32_t base = 0; base < V; base += kThreads * 4u) {
        const uint32_t i = base + tid * 4u;
        uint32_t k[4];
        uint32_t c = 0;
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            k[j] = 0;
            if (i + j < V) {
                const float q = weight_of(wbuf[i + j], m, inv_t, sm.tab);
                if (q >= floor_q && q > 0.0f) {
                    k[j] = __float_as_uint(q);
                    ++c;
                }
            }
        }
        uint32_t tot;
        uint32_t pos = n0 + block_excl_scan_u32(c, tot, sm.bs);
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j)
            if (k[j]) {
                key0[pos] = ~k[j];
                idx0[pos] = i + j;
                ++pos;
            }
        n0 += tot;
    }
    __syncthreads();

    if (n0 == 0) { // sampler.cpp:37-38
        RowOut o;
        o.token = (int32_t)argidx;
        o.n_cand = 1;
        o.total = 1.0f;
        o.q = 1.0f;
        o.path = MAKO_PATH_FALLBACK;
        o.accepted = 0;
        if (d.draft) {
            // one candidate (1.0f, argidx): accepted iff it is the draft (u * 1 < 1), else it is drawn
            o.accepted = d.draft[row] == (int32_t)argidx;
        }
        if (d.out_cand_idx && d.out_cand_q && d.cand_cap && tid == 0) {
            d.out_cand_idx[(size_t)row * d.cand_cap] = (int32_t)argidx;
            d.out_cand_q[(size_t)row * d.cand_cap] = 1.0f;
        }
        if (tid == 0)
            write_row(d, row, o);
        return;
    }

    // 3. order by (q desc, idx asc): stable LSD radix sort of ~bits(q), ascending
    const bool topk_active = P.top_k > 0 && P.top_k < n0;
    const bool topp_active = P.top_p < 1.0f;
    uint32_t *ks = key0, *is = idx0, *kd = key1, *id = idx1;
    if (topk_active || topp_active) {
        for (uint32_t shift = 0; shift < 32; shift += 8) {
            if (radix_pass(ks, is, kd, id, n0, shift, sm)) {
                uint32_t* t = ks;
                ks = kd;
                kd = t;
                t = is;
                is = id;
                id = t;
            }
            __syncthreads();
        }
    }
    uint32_t n = topk_active ? P.top_k : n0; // sampler.cpp:40-43

    // 4. top-p: shortest sorted prefix whose fp64 running sum reaches top_p * total (sampler.cpp:44-61)
    if (topp_active) {
        double part = 0;
        for (uint32_t i = tid; i < n; i += kThreads)
            part += (double)__uint_as_float(~ks[i]);
        const double total64 = block_sum_f64(part, sm.bs);
        const double want = (double)P.top_p * total64;
        double carry = 0;
        uint32_t keep = n;
        for (uint32_t base = 0; base < n; base += kThreads) {
            const uint32_t i = base + tid;
            const double q = i < n ? (double)__uint_as_float(~ks[i]) : 0.0;
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
        n = keep;
    }

    draw_from_list(d, row, ks, is, n, MAKO_PATH_GENERAL, sm);
}

// grid = rows.
__global__ __launch_bounds__(kThreads) void finish_kernel(mako_sample_desc d, Scratch sc, uint32_t slices)
{
    __shared__ FinishShared sm;
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    __syncthreads();

    const mako_sampling_params P = d.params[row];
    // first maximum of the row (std::max_element semantics, NaNs never win unless at index 0)
    unsigned long long top = 0;
    for (uint32_t s = 0; s < slices; ++s) {
        const SliceStat st = sc.stats[(size_t)row * kMaxSlices + s];
        const unsigned long long p = ((unsigned long long)order_key(st.wmax) << 32) | (unsigned long long)(kNone - st.argidx);
        top = p > top ? p : top;
    }
    const bool first_nan = sc.stats[(size_t)row * kMaxSlices].flags & 1u;
    float m = order_unkey((uint32_t)(top >> 32));
    uint32_t argidx = kNone - (uint32_t)top;
    if (argidx == kNone)
        argidx = 0;
    if (first_nan) {
        m = __uint_as_float(0x7fc00000u);
        argidx = 0;
    }

    if (greedy_row(P)) { // sampler.cpp:77-78, 88-92
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
    general_row(d, sc, row, P, m, argidx, sm);
}

__global__ void debug_expf_kernel(const float* x, float* y, uint32_t n)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        y[i] = expf_glibc(x[i], k_exp2_tab);
}

__global__ void debug_div_kernel(const float* a, const float* b, float* y, uint32_t n)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        y[i] = a[i] / b[i];
}

} // namespace mako

// ---------------------------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------------------------

struct mako_sampler_ctx {
    int device = 0;
    uint32_t max_rows = 0, max_vocab = 0, max_hist = 0;
    mako::Scratch sc{};
    // staging for the host-pointer call
    float* st_logits = nullptr;
    mako_sampling_params* st_params = nullptr;
    float* st_u = nullptr;
    float* st_u2 = nullptr;
    uint32_t* st_mask = nullptr;
    int32_t* st_hist = nullptr;
    uint32_t* st_hcnt = nullptr;
    uint32_t* st_hlen = nullptr;
    int32_t* st_draft = nullptr;
    int32_t* st_tokens = nullptr;
    uint8_t* st_acc = nullptr;
    std::string err = "";
};

namespace {

int fail(mako_sampler_ctx* ctx, int code, const std::string& what)
{
    if (ctx)
        ctx->err = what;
    return code;
}

#define MAKO_HIP(ctx, call)                                                                                        \
    do {                                                                                                           \
        hipError_t e_ = (call);                                                                                    \
        if (e_ != hipSuccess)                                                                                      \
            return fail(ctx, MAKO_ERR_HIP, std::string(#call) + ": " + hipGetErrorString(e_));                     \
    } while (0)

template <typename T>
hipError_t dev_alloc(T** p, size_t count)
{
    return hipMalloc(reinterpret_cast<void**>(p), count * sizeof(T));
}

uint32_t slice_len_for(uint32_t n_vocab, uint32_t slices)
{
    uint32_t len = (n_vocab + slices - 1) / slices;
    return (len + 3u) & ~3u;
}

} // namespace

extern "C" {

uint32_t mako_sampler_slices(uint32_t n_vocab)
{
    const uint32_t s = (n_vocab + mako::kSliceMax - 1) / mako::kSliceMax;
    return s ? s : 1;
}

int mako_sampler_create(mako_sampler_ctx** out, int device, uint32_t max_rows, uint32_t max_vocab, uint32_t max_hist)
{
    if (!out || max_rows == 0 || max_vocab == 0)
        return MAKO_ERR_INVALID_ARG;
    if (mako_sampler_slices(max_vocab) > mako::kMaxSlices)
        return MAKO_ERR_INVALID_ARG;
    mako_sampler_ctx* ctx = new (std::nothrow) mako_sampler_ctx;
    if (!ctx)
        return MAKO_ERR_NO_MEMORY;
    *out = ctx;
    ctx->device = device;
    ctx->max_rows = max_rows;
    ctx->max_vocab = max_vocab;
    ctx->max_hist = max_hist;
    MAKO_HIP(ctx, hipSetDevice(device));
    mako::Scratch& sc = ctx->sc;
    sc.vpad = ((uint64_t)max_vocab + 1023u) & ~1023ull;
    const size_t rv = (size_t)max_rows * sc.vpad;
    MAKO_HIP(ctx, dev_alloc(&sc.stats, (size_t)max_rows * mako::kMaxSlices));
    MAKO_HIP(ctx, dev_alloc(&sc.wbuf, rv));
    MAKO_HIP(ctx, dev_alloc(&sc.cnt, rv));
    MAKO_HIP(ctx, dev_alloc(&sc.key[0], rv));
    MAKO_HIP(ctx, dev_alloc(&sc.key[1], rv));
    MAKO_HIP(ctx, dev_alloc(&sc.idx[0], rv));
    MAKO_HIP(ctx, dev_alloc(&sc.idx[1], rv));
    MAKO_HIP(ctx, hipMemset(sc.cnt, 0, rv * sizeof(uint32_t)));
    MAKO_HIP(ctx, hipDeviceSynchronize());
    return MAKO_OK;
}

void mako_sampler_destroy(mako_sampler_ctx* ctx)
{
    if (!ctx)
        return;
    (void)hipSetDevice(ctx->device);
    mako::Scratch& sc = ctx->sc;
    void* ptrs[] = {sc.stats,      sc.wbuf,      sc.cnt,        sc.key[0],     sc.key[1],     sc.idx[0],
                    sc.idx[1],     ctx->st_logits, ctx->st_params, ctx->st_u,   ctx->st_u2,    ctx->st_mask,
                    ctx->st_hist,  ctx->st_hcnt, ctx->st_hlen,  ctx->st_draft, ctx->st_tokens, ctx->st_acc};
    for (void* p : ptrs)
        if (p)
            (void)hipFree(p);
    delete ctx;
}

const char* mako_sampler_last_error(const mako_sampler_ctx* ctx)
{
    return ctx ? ctx->err.c_str() : "null context";
}

int mako_sampler_sample_batch(mako_sampler_ctx* ctx, const mako_sample_desc* desc, void* stream)
{
    if (!ctx || !desc)
        return MAKO_ERR_INVALID_ARG;
    const mako_sample_desc& d = *desc;
    if (d.n_vocab == 0)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: empty vocabulary"); // sampler.cpp:11-12
    if (d.n_rows == 0)
        return MAKO_OK;
    if (!d.logits || !d.params || !d.u || !d.out_tokens)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: logits, params, u and out_tokens are required");
    if (d.n_rows > ctx->max_rows || d.n_vocab > ctx->max_vocab)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: batch exceeds the context's max_rows/max_vocab");
    if (d.logits_stride < (int64_t)d.n_vocab)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: logits_stride < n_vocab");
    if (d.mask && d.mask_stride < (int64_t)((d.n_vocab + 31) / 32))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: mask_stride < ceil(n_vocab / 32)");
    if (d.hist_tokens && (!d.hist_len || d.hist_stride < 0))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: hist_tokens needs hist_len and a stride");
    if ((d.draft != nullptr) != (d.u2 != nullptr) || (d.draft != nullptr) != (d.out_accepted != nullptr))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: draft, u2 and out_accepted go together");
    if ((d.out_cand_idx != nullptr) != (d.out_cand_q != nullptr))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: out_cand_idx and out_cand_q go together");

    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t slices = mako_sampler_slices(d.n_vocab);
    const uint32_t slice_len = slice_len_for(d.n_vocab, slices);
    const bool vec = d.n_vocab % 4 == 0 && d.logits_stride % 4 == 0 && (reinterpret_cast<uintptr_t>(d.logits) & 15u) == 0;
    const size_t lds = d.hist_tokens ? (size_t)slice_len * sizeof(uint32_t) : 0;
    const dim3 grid(slices, d.n_rows);
    if (vec)
        hipLaunchKernelGGL(mako::scan_kernel<true>, grid, dim3(mako::kThreads), lds, st, d, ctx->sc, slice_len);
    else
        hipLaunchKernelGGL(mako::scan_kernel<false>, grid, dim3(mako::kThreads), lds, st, d, ctx->sc, slice_len);
    hipLaunchKernelGGL(mako::finish_kernel, dim3(d.n_rows), dim3(mako::kThreads), 0, st, d, ctx->sc, slices);
    MAKO_HIP(ctx, hipGetLastError());
    return MAKO_OK;
}

int mako_sampler_sample_host(mako_sampler_ctx* ctx, const float* logits, int64_t logits_stride, uint32_t n_rows,
                             uint32_t n_vocab, const mako_sampling_params* params, const float* u,
                             const uint32_t* mask, int64_t mask_stride, const int32_t* hist_tokens,
                             const uint32_t* hist_counts, int64_t hist_stride, const uint32_t* hist_len,
                             const int32_t* draft, const float* u2, uint8_t* out_accepted, int32_t* out_tokens)
{
    if (!ctx)
        return MAKO_ERR_INVALID_ARG;
    if (n_vocab == 0)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: empty vocabulary");
    if (n_rows == 0)
        return MAKO_OK;
    if (!logits || !params || !u || !out_tokens || n_rows > ctx->max_rows || n_vocab > ctx->max_vocab)
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: bad host arguments");
    if (hist_tokens && (!hist_len || hist_stride < 0 || (uint64_t)hist_stride > ctx->max_hist))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: history exceeds the context's max_hist");
    if ((draft != nullptr) != (u2 != nullptr) || (draft != nullptr) != (out_accepted != nullptr))
        return fail(ctx, MAKO_ERR_INVALID_ARG, "sampler: draft, u2 and out_accepted go together");
    MAKO_HIP(ctx, hipSetDevice(ctx->device));
    const size_t R = ctx->max_rows;
    const size_t mwords = ((size_t)ctx->max_vocab + 31) / 32;
    // staging buffers are created on first use and kept
    if (!ctx->st_logits) {
        MAKO_HIP(ctx, dev_alloc(&ctx->st_logits, R * ctx->sc.vpad));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_params, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_u, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_u2, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_mask, R * mwords));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_hist, R * (size_t)(ctx->max_hist ? ctx->max_hist : 1)));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_hcnt, R * (size_t)(ctx->max_hist ? ctx->max_hist : 1)));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_hlen, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_draft, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_tokens, R));
        MAKO_HIP(ctx, dev_alloc(&ctx->st_acc, R));
    }
    const size_t vp = ctx->sc.vpad;
    MAKO_HIP(ctx, hipMemcpy2D(ctx->st_logits, vp * sizeof(float), logits, (size_t)logits_stride * sizeof(float),
                              (size_t)n_vocab * sizeof(float), n_rows, hipMemcpyHostToDevice));
    MAKO_HIP(ctx, hipMemcpy(ctx->st_params, params, n_rows * sizeof(*params), hipMemcpyHostToDevice));
    MAKO_HIP(ctx, hipMemcpy(ctx->st_u, u, n_rows * sizeof(float), hipMemcpyHostToDevice));
    mako_sample_desc d;
    memset(&d, 0, sizeof d);
    d.logits = ctx->st_logits;
    d.logits_stride = (int64_t)vp;
    d.n_rows = n_rows;
    d.n_vocab = n_vocab;
    d.params = ctx->st_params;
    d.u = ctx->st_u;
    if (mask) {
        const size_t w = ((size_t)n_vocab + 31) / 32;
        MAKO_HIP(ctx, hipMemcpy2D(ctx->st_mask, mwords * 4, mask, (size_t)mask_stride * 4, w * 4, n_rows,
                                  hipMemcpyHostToDevice));
        d.mask = ctx->st_mask;
        d.mask_stride = (int64_t)mwords;
    }
    if (hist_tokens && hist_stride > 0) {
        const size_t hs = ctx->max_hist;
        MAKO_HIP(ctx, hipMemcpy2D(ctx->st_hist, hs * 4, hist_tokens, (size_t)hist_stride * 4, (size_t)hist_stride * 4,
                                  n_rows, hipMemcpyHostToDevice));
        if (hist_counts) {
            MAKO_HIP(ctx, hipMemcpy2D(ctx->st_hcnt, hs * 4, hist_counts, (size_t)hist_stride * 4,
                                      (size_t)hist_stride * 4, n_rows, hipMemcpyHostToDevice));
            d.hist_counts = ctx->st_hcnt;
        }
        MAKO_HIP(ctx, hipMemcpy(ctx->st_hlen, hist_len, n_rows * 4, hipMemcpyHostToDevice));
        d.hist_tokens = ctx->st_hist;
        d.hist_stride = (int64_t)hs;
        d.hist_len = ctx->st_hlen;
    }
    if (draft) {
        MAKO_HIP(ctx, hipMemcpy(ctx->st_draft, draft, n_rows * 4, hipMemcpyHostToDevice));
        MAKO_HIP(ctx, hipMemcpy(ctx->st_u2, u2, n_rows * 4, hipMemcpyHostToDevice));
        d.draft = ctx->st_draft;
        d.u2 = ctx->st_u2;
        d.out_accepted = ctx->st_acc;
    }
    d.out_tokens = ctx->st_tokens;
    const int rc = mako_sampler_sample_batch(ctx, &d, nullptr);
    if (rc != MAKO_OK)
        return rc;
    MAKO_HIP(ctx, hipMemcpy(out_tokens, ctx->st_tokens, n_rows * 4, hipMemcpyDeviceToHost));
    if (draft)
        MAKO_HIP(ctx, hipMemcpy(out_accepted, ctx->st_acc, n_rows, hipMemcpyDeviceToHost));
    return MAKO_OK;
}

int mako_sampler_debug_expf(const float* x_dev, float* y_dev, uint32_t n, void* stream)
{
    if (!x_dev || !y_dev)
        return MAKO_ERR_INVALID_ARG;
    if (n)
        hipLaunchKernelGGL(mako::debug_expf_kernel, dim3((n + 255) / 256), dim3(256), 0,
                           static_cast<hipStream_t>(stream), x_dev, y_dev, n);
    return hipGetLastError() == hipSuccess ? MAKO_OK : MAKO_ERR_HIP;
}

int mako_sampler_debug_div(const float* a_dev, const float* b_dev, float* y_dev, uint32_t n, void* stream)
{
    if (!a_dev || !b_dev || !y_dev)
        return MAKO_ERR_INVALID_ARG;
    if (n)
        hipLaunchKernelGGL(mako::debug_div_kernel, dim3((n + 255) / 256), dim3(256), 0,
                           static_cast<hipStream_t>(stream), a_dev, b_dev, y_dev, n);
    return hipGetLastError() == hipSuccess ? MAKO_OK : MAKO_ERR_HIP;
}

} // extern "C"
