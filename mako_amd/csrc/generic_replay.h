// The exact fp32 running sum and walk over any candidate list, by the whole workgroup (windows of maps), and the
// draw / verification built on them.
#pragma once

#include "workgroup_state.h"
#include "row_output.h"

namespace mako {

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

} // namespace mako
