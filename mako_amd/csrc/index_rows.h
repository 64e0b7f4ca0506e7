// Rows that are cut neither to a top-k nor to a nucleus (top_k == 0, top_p >= 1, temperature > 0): the reference adds
// up and walks the candidates in token order (src/gen/sampler.cpp:29-36, :79-83, :64-72), so nothing is sorted.  With
// the caller's host copy of the parameters the library knows that a batch has such rows and gives them three launches
// of their own instead of one workgroup per row on the whole-row path:
//   index_weights_kernel  a workgroup per 16 384 logits: masks and penalties as everywhere, q = expf((w - m) / T), and
//                         ~bits(q) (0.0f for a logit that is no candidate) stored at the token's own position;
//   index_groups_kernel   a workgroup per 4 096 entries: the group records of its sixteen groups of 256 (fp64 sums, the
//                         maps of the running fp32 sum and of the walk for the binades guessed from the sums before
//                         them), as sort_kernel's workers leave them for a sorted list;
//   index_tail_kernel     a workgroup per row: the exact fp32 total and the walk over the group records
//                         (sorted_tail's planned instance for lists in any order).
// A logit that is no candidate stays in the list as a weight of 0.0f: adding it changes no sum, and the walk's
// `r < q` is never true for it.  The list ends behind the row's last candidate, which is where the reference's walk
// ends when it runs off its list.
#pragma once

#include "sorted_tail.h"
#include "worker_sort.h"
#include "whole_row.h"

namespace mako {

constexpr uint32_t kIndexBlock = 4096;                       // entries per workgroup of index_groups_kernel
constexpr uint32_t kIndexMaxVocab = kMaxSlices * kIndexBlock; // a sum per block in Scratch::part_sum's row
static_assert(kIndexMaxVocab <= kMaxGroups * kGroup && kSliceMax == 4u * kIndexBlock && kIndexBlock % kGroup == 0, "blocks, groups");
#ifdef MAKO_EMIT_INDEX_KERNELS
// grid = (ceil(V / 16384), rows); rows of other kinds leave at once.  V % 4 == 0 and aligned rows (the host checks).
template <int KH>
__global__ __launch_bounds__(kThreads) void index_weights_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    extern __shared__ __align__(16) unsigned long long s_dyn64[];
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t row = blockIdx.y, piece = blockIdx.x, tid = threadIdx.x;
    const mako_sampling_params P0 = d_arg.params[row];
    if (!index_order_row(P0)) // uniform
        return;
    stage_args_only(d_arg, sc_val, s_args);
    stage_params(P0, s_args);
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    __syncthreads();
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    const mako_sampling_params& P = s_args.P;
    float m;
    uint32_t argidx, n_cands, any_overflow;
    row_summary(sc, row, slices, m, argidx, n_cands, any_overflow);
    const uint32_t hl = d.hist_tokens ? min(as_global(d.hist_len)[row], (uint32_t)d.hist_stride) : 0u;
    const bool pen = d.hist_tokens && !penalties_neutral(P);
    const uint32_t lo = piece * kSliceMax, hi = min(d.n_vocab, lo + kSliceMax);
    float wv[16];
    load_penalised<true, KH>(d, row, lo, hi, kSliceMax, P, hl, pen, reinterpret_cast<uint32_t*>(s_dyn64), wv);
    const float inv_t = 1.0f / P.temperature;
    const float floor_q = (1.0f < P.min_p) ? 1.0f : P.min_p;
    uint32_t* key0 = sc.key[0] + (size_t)row * sc.vpad;
    uint32_t* idx0 = sc.idx[0] + (size_t)row * sc.vpad;
    uint32_t cnt = 0, last = 0;
    double bsum[4];
#pragma unroll
    for (uint32_t b = 0; b < 4; ++b) {
        bsum[b] = 0.0;
        const uint32_t base = lo + b * kIndexBlock + tid * 4u;
        if (lo + b * kIndexBlock < hi) { // uniform
            uint32_t k[4];
#pragma unroll
            for (uint32_t c = 0; c < 4; ++c) {
                const float q = weight_of(wv[4u * b + c], m, inv_t, sm.tab);
                const bool ok = base + c < hi && q >= floor_q && q > 0.0f; // src/gen/sampler.cpp:34-35
                k[c] = ok ? __float_as_uint(q) : 0u;
                cnt += ok ? 1u : 0u;
                last = ok ? base + c + 1u : last;
                bsum[b] += ok ? (double)q : 0.0;
            }
            if (base + 3u < hi) {
                *reinterpret_cast<uint4*>(key0 + base) = make_uint4(~k[0], ~k[1], ~k[2], ~k[3]);
                *reinterpret_cast<uint4*>(idx0 + base) = make_uint4(base, base + 1u, base + 2u, base + 3u);
            } else {
#pragma unroll
                for (uint32_t c = 0; c < 4; ++c)
                    if (base + c < hi) {
                        key0[base + c] = ~k[c];
                        idx0[base + c] = base + c;
                    }
            }
        }
    }
    // the blocks' fp64 sums (estimates for the binades only: any order of addition will do), the piece's candidates
    // and its last one
    double* wsum = reinterpret_cast<double*>(s_dyn64); // [4][kWaves] (the penalty table is done with)
    uint32_t* wcnt = reinterpret_cast<uint32_t*>(wsum + 4 * kWaves);
    __syncthreads();
#pragma unroll
    for (uint32_t b = 0; b < 4; ++b) {
        const double s = __ockl_wfred_add_f64(bsum[b]);
        if (lane_id() == 0)
            wsum[b * kWaves + wave_id()] = s;
    }
    cnt = __ockl_wfred_add_u32(cnt);
    last = __ockl_wfred_max_u32(last);
    if (lane_id() == 0) {
        wcnt[wave_id()] = cnt;
        wcnt[kWaves + wave_id()] = last;
    }
    __syncthreads();
    if (tid < 4 && lo + tid * kIndexBlock < hi) {
        double s = 0.0;
        for (int w = 0; w < kWaves; ++w)
            s += wsum[tid * kWaves + w];
        sc.part_sum[(size_t)row * kMaxSlices + piece * 4u + tid] = s;
    }
    if (tid == 0) {
        uint32_t c = 0, l = 0;
        for (int w = 0; w < kWaves; ++w) {
            c += wcnt[w];
            l = max(l, wcnt[kWaves + w]);
        }
        BigPlan* plan = sc.plan + row;
        plan->cursor[piece] = c; // (the pieces' counts and last candidates travel in the plan's per-worker words)
        plan->key_lo[piece] = l;
        if (piece == 0) {
            plan->flag = kIndexClaimed;
            plan->m = m;
            plan->argidx = argidx;
        }
    }
}

// grid = (ceil(V / 4096), rows).
__global__ __launch_bounds__(kThreads) void index_groups_kernel(mako_sample_desc d_arg, Scratch sc_val)
{
    extern __shared__ __align__(16) unsigned long long s_dyn64[];
    __shared__ FinishShared sm;
    const uint32_t row = blockIdx.y, b = blockIdx.x, tid = threadIdx.x, lane = lane_id();
    const mako_sampling_params P0 = d_arg.params[row];
    if (!index_order_row(P0)) // uniform
        return;
    BigPlan* plan = sc_val.plan + row;
    const uint32_t pieces = (d_arg.n_vocab + kSliceMax - 1u) / kSliceMax, blocks = (d_arg.n_vocab + kIndexBlock - 1u) / kIndexBlock;
    const uint32_t cnt_l = lane < pieces ? plan->cursor[min(lane, kWorkers - 1u)] : 0u;
    const uint32_t last_l = lane < pieces ? plan->key_lo[min(lane, kWorkers - 1u)] : 0u;
    const double ps = lane < blocks ? sc_val.part_sum[(size_t)row * kMaxSlices + lane] : 0.0;
    const float u_row = d_arg.u[row];
    const uint32_t n_cand = __ockl_wfred_add_u32(cnt_l), n_list = __ockl_wfred_max_u32(last_l);
    const double incl = __ockl_wfscan_add_f64(ps, true);
    const double total64 = readlane_f64(incl, kWave - 1), mass = readlane_f64(incl - ps, b);
    if (b == 0 && tid == 0) {
        plan->n0 = n_list;
        plan->groups = (n_list + kGroup - 1u) / kGroup;
        plan->total64 = total64;
        plan->thr = n_cand;
        const bool gaps_matter = n_cand < n_list && d_arg.out_cand_idx && d_arg.out_cand_q && d_arg.cand_cap;
        plan->flag = n_cand == 0u ? kIndexEmpty : (gaps_matter ? kIndexWhole : kIndexReady);
    }
    if (n_cand == 0u || b * kIndexBlock >= n_list) // uniform
        return;
    const FinishLds L = finish_lds_views(sm, s_dyn64);
    const double r0_raw = (double)u_row * total64;
    const uint32_t* key0 = sc_val.key[0] + (size_t)row * sc_val.vpad;
    worker_groups<true>(key0, b * kIndexBlock, min(kIndexBlock, n_list - b * kIndexBlock),
                        (size_t)row * sc_val.g_cap + b * (kIndexBlock / kGroup), mass, sc_val.gt, L, nullptr, r0_raw == r0_raw ? r0_raw : 0.0);
}

// grid = (1, rows).
__global__ __launch_bounds__(kThreads) void index_tail_kernel(mako_sample_desc d_arg, Scratch sc_val)
{
    extern __shared__ __align__(16) unsigned long long s_dyn64[];
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t row = blockIdx.y, tid = threadIdx.x;
    if (!index_order_row(d_arg.params[row])) // uniform
        return;
    const BigPlan* planned = sc_val.plan + row;
    const uint32_t flag = planned->flag, n0 = min(planned->n0, d_arg.n_vocab), n_cand = planned->thr;
    const uint32_t groups = min(planned->groups, min(kMaxGroups, sc_val.g_cap));
    const double total64 = planned->total64;
    const float m = planned->m;
    const uint32_t argidx = planned->argidx;
    stage_args(d_arg, sc_val, row, s_args); // (with a barrier: the plan has been read)
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    if (tid == 0)
        sc.plan[row].flag = 0;
    if (flag != kIndexReady && flag != kIndexWhole && flag != kIndexEmpty) // (never)
        return;
    const FinishLds L = finish_lds_views(sm, s_dyn64);
    if (flag == kIndexEmpty) {
        fallback_row(d, row, argidx);
        return;
    }
    if (flag == kIndexReady) {
        const uint32_t* kf = sc.key[0] + (size_t)row * sc.vpad;
        const uint32_t* jf = sc.idx[0] + (size_t)row * sc.vpad;
        if (sorted_tail<true, false, false, false, true>(d, row, s_args.P, kf, jf, n0, true, total64, MAKO_PATH_INDEXED, L, false, 0.0f,
                                                         sc.gt, (size_t)row * sc.g_cap, groups)) {
            // (the list's length counts the gaps; the candidates are what the reference counts)
            if (tid == 0 && d.out_n_cand)
                d.out_n_cand[row] = n_cand;
            return;
        }
    }
    __syncthreads();
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    __syncthreads();
    general_row<0>(d, sc, row, s_args.P, m, argidx, L);
}
#endif // MAKO_EMIT_INDEX_KERNELS

} // namespace mako
