// Rows that are cut neither to a top-k nor to a nucleus (top_k == 0, top_p >= 1, temperature > 0): the reference adds
// up and walks the candidates in token order (src/gen/sampler.cpp:29-36, :79-83, :64-72), so nothing is sorted.  With
// the caller's host copy of the parameters the library knows that a batch has such rows and gives them three launches
// of their own instead of one workgroup per row on the whole-row path:
//   index_weights_kernel  a workgroup per 16 384 logits: masks and penalties as everywhere, q = expf((w - m) / T), and
//                         ~bits(q) (0.0f for a logit that is no candidate) stored at the token's own position (entry i
//                         of the list is token i: no array of token ids);
//   index_groups_kernel   a workgroup per 16 384 entries: the group records of its 64 groups of 256 (fp64 sums, the maps
//                         of the running fp32 sum and of the walk for the binades guessed from the sums before them),
//                         as sort_kernel's workers leave them for a sorted list;
//   index_tail_kernel     a workgroup per row: the exact fp32 total and the walk over the group records
//                         (sorted_tail's planned instance for lists in any order).
// A logit that is no candidate stays in the list as a weight of 0.0f: adding it changes no sum, and the walk's
// `r < q` is never true for it.  The list ends behind the row's last candidate, which is where the reference's walk
// ends when it runs off its list.  Verification works on the same list: the draft's weight is entry `draft`, and a
// rejected draft is redrawn with that entry taken as 0.0f (sorted_tail's UNORDERED instance).
// The other rows of the whole-row class (top-k without top-p, top-k beyond the candidate lists) only get their weights
// here (index_weights_kernel, into the array general_row_from_weights() starts from) and one workgroup each in
// index_tail_kernel's launch for the rest of the whole-row path.
#pragma once

#include "sorted_tail.h"
#include "worker_sort.h"
#include "whole_row.h"

namespace mako {

constexpr uint32_t kIndexBlock = 4096;                   // entries whose fp64 sum index_weights_kernel leaves as one number
constexpr uint32_t kIndexMaxVocab = kMaxGroups * kGroup; // the group records of a row
static_assert(kIndexMaxVocab / kSliceMax <= kWorkers && kIndexMaxVocab / kIndexBlock <= kMaxSlices && kIndexMaxVocab / kIndexBlock <= (uint32_t)kWave &&
                  kSliceMax == 4u * kIndexBlock && kIndexBlock == (uint32_t)kWaves * kGroup,
              "a piece's count and last candidate travel in the plan's per-worker words, the blocks' sums in the row's part_sum, a lane each");
#ifdef MAKO_EMIT_INDEX_KERNELS
// grid = (ceil(V / 16384), rows); rows of other kinds leave at once.  (VEC: V % 4 == 0 and 16-byte aligned rows, whose
// logits are loaded four at a time; the layout of a thread's sixteen logits is slice_load.h's either way.)
template <bool VEC, int KH>
__global__ __launch_bounds__(kThreads) void index_weights_kernel(mako_sample_desc d_arg, Scratch sc_val, uint32_t slices)
{
    extern __shared__ __align__(16) unsigned long long s_dyn64[];
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t row = blockIdx.y, piece = blockIdx.x, tid = threadIdx.x;
    const mako_sampling_params P0 = d_arg.params[row];
    if (classify(P0) != kGeneral) // uniform
        return;
    // (a row that is cut to a top-k without a top-p, or to a top-k beyond the candidate lists, is still finished by one
    // workgroup on the whole-row path, in index_tail_kernel's launch; its weights, a third of that path's time, are left
    // here where general_row_from_weights() expects them)
    const bool in_order = index_order_row(P0);
    stage_args_only(d_arg, sc_val, s_args);
    stage_params(P0, s_args);
    if (tid < 32)
        sm.tab[tid] = k_exp2_tab[tid];
    __syncthreads();
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    const mako_sampling_params& P = s_args.P;
    if (d.force_token || d.close_token) { // a forced row needs no weights: it is not claimed, and the launch that
                                          // finishes the late rows writes its token
        int32_t ftok;
        uint32_t above;
        if (row_forced(d, sc, row, slices, ftok, above) != MAKO_FORCED_NONE)
            return;
    }
    float m;
    uint32_t argidx, n_cands, any_overflow;
    row_summary(sc, row, slices, m, argidx, n_cands, any_overflow);
    const uint32_t hl = d.hist_tokens ? min(as_global(d.hist_len)[row], (uint32_t)d.hist_stride) : 0u;
    const bool pen = d.hist_tokens && !penalties_neutral(P);
    const uint32_t lo = piece * kSliceMax, hi = min(d.n_vocab, lo + kSliceMax);
    float wv[16];
    load_penalised<VEC, KH>(d, row, lo, hi, kSliceMax, P, hl, pen, reinterpret_cast<uint32_t*>(s_dyn64), wv);
    const float inv_t = 1.0f / P.temperature;
    const float floor_q = (1.0f < P.min_p) ? 1.0f : P.min_p;
    // (~bits(q) into the row's list, or bits(q) into the whole-row path's array)
    uint32_t* key0 = in_order ? sc.key[0] + (size_t)row * sc.vpad : reinterpret_cast<uint32_t*>(sc.wbuf + (size_t)row * sc.vpad);
    const uint32_t flip = in_order ? ~0u : 0u;
    MAKO_CHECK(sc, kCheckStage, (uint64_t)hi <= sc.vpad);
    uint32_t cnt = 0, last = 0;
    double bsum[4];
#pragma unroll
    for (uint32_t b = 0; b < 4; ++b) {
        bsum[b] = 0.0;
        // (the thread's logits 4b .. 4b+3 lie in the piece's b-th 4 096: four in a row, or 1 024 apart)
        const uint32_t base = elem_index<VEC>(lo, tid, 4u * b);
        if (lo + b * kIndexBlock < hi) { // uniform
            uint32_t k[4];
#pragma unroll
            for (uint32_t c = 0; c < 4; ++c) {
                const uint32_t at = elem_index<VEC>(lo, tid, 4u * b + c);
                const float q = weight_of(wv[4u * b + c], m, inv_t, sm.tab);
                const bool ok = at < hi && q >= floor_q && q > 0.0f; // src/gen/sampler.cpp:34-35
                k[c] = ok ? __float_as_uint(q) : 0u;
                cnt += ok ? 1u : 0u;
                last = ok ? max(last, at + 1u) : last;
                bsum[b] += ok ? (double)q : 0.0;
            }
            if (VEC && base + 3u < hi) {
                *reinterpret_cast<uint4*>(key0 + base) = make_uint4(k[0] ^ flip, k[1] ^ flip, k[2] ^ flip, k[3] ^ flip);
            } else {
#pragma unroll
                for (uint32_t c = 0; c < 4; ++c)
                    if (elem_index<VEC>(lo, tid, 4u * b + c) < hi)
                        key0[elem_index<VEC>(lo, tid, 4u * b + c)] = k[c] ^ flip;
            }
            if (VEC && !in_order) { // uniform
                // the whole-row path's list as well, (~bits(q), token) at the token's position: it is the row's list
                // of candidates when every logit turns out to be one, as the pieces' counts will tell.  (Not from
                // the instances for rows that are loaded a logit at a time: they would need more registers than
                // two workgroups on a CU have.)
                uint32_t* lk = sc.key[0] + (size_t)row * sc.vpad;
                uint32_t* li = sc.idx[0] + (size_t)row * sc.vpad;
                if (base + 3u < hi) {
                    *reinterpret_cast<uint4*>(lk + base) = make_uint4(~k[0], ~k[1], ~k[2], ~k[3]);
                    *reinterpret_cast<uint4*>(li + base) = make_uint4(base, base + 1u, base + 2u, base + 3u);
                } else {
#pragma unroll
                    for (uint32_t c = 0; c < 4; ++c)
                        if (base + c < hi) {
                            lk[base + c] = ~k[c];
                            li[base + c] = base + c;
                        }
                }
            }
        }
        // (four weights at a time: with all sixteen in flight the kernel needs twice the registers, and two workgroups
        // no longer share a CU)
        __builtin_amdgcn_sched_barrier(0);
    }
    // the piece's fp64 sum (an estimate for the binades only: any order of addition will do), its candidates and its
    // last one
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
    if (tid < 4u && lo + tid * kIndexBlock < hi) { // (a sum per 4 096 entries: index_groups_kernel's workgroups may be that small)
        double s = 0.0;
        for (int w = 0; w < kWaves; ++w)
            s += wsum[tid * kWaves + w];
        sc.part_sum[(size_t)row * kMaxSlices + piece * 4u + tid] = s;
    }
    if (tid == 0) {
        cnt = last = 0;
        for (int w = 0; w < kWaves; ++w) {
            cnt += wcnt[w];
            last = max(last, wcnt[kWaves + w]);
        }
    }
    if (tid == 0) {
        BigPlan* plan = sc.plan + row;
        plan->cursor[piece] = cnt; // (the pieces' counts and last candidates travel in the plan's per-worker words)
        plan->key_lo[piece] = last;
        if (piece == 0) {
            plan->flag = kIndexClaimed;
            plan->m = m;
            plan->argidx = argidx;
            plan->n0 = VEC && !in_order ? kIndexListed : 0u;
        }
    }
}

// grid = (ceil(V / (4096 GPW)), rows): workgroup p leaves the records of the groups of its 4096 GPW entries.  Wave w
// takes the groups w, w + 16, ... (GPW of them): their entries in one trip to memory, their fp64 sums to LDS, and once
// every wave has the sums before each group, the maps from the entries it still holds.  (GPW = 4 where there are rows
// enough to fill the chip, 1 on a small batch, which waits for one workgroup's chain of dependent steps.)
template <uint32_t GPW>
__global__ __launch_bounds__(kThreads) void index_groups_kernel(mako_sample_desc d_arg, Scratch sc_val)
{
    __shared__ double s_gs[kWave];
    constexpr uint32_t kSpan = kIndexBlock * GPW; // entries per workgroup
    const uint32_t row = blockIdx.y, p = blockIdx.x, tid = threadIdx.x, lane = lane_id(), wave = wave_id();
    const mako_sampling_params P0 = d_arg.params[row];
    if (!index_order_row(P0)) // uniform
        return;
    BigPlan* plan = sc_val.plan + row;
    // (zero: index_weights_kernel left the row alone, its token is forced; a workgroup that starts late may already see
    // what this kernel's first workgroup has made of the flag)
    if (plan->flag == 0u) // uniform
        return;
    const uint32_t pieces = (d_arg.n_vocab + kSliceMax - 1u) / kSliceMax, blocks = (d_arg.n_vocab + kIndexBlock - 1u) / kIndexBlock;
    const uint32_t cnt_l = lane < pieces ? plan->cursor[min(lane, kWorkers - 1u)] : 0u;
    const uint32_t last_l = lane < pieces ? plan->key_lo[min(lane, kWorkers - 1u)] : 0u;
    const double ps = lane < blocks ? sc_val.part_sum[(size_t)row * kMaxSlices + lane] : 0.0;
    const float u_row = d_arg.u[row];
    const uint32_t n_cand = __ockl_wfred_add_u32(cnt_l), n_list = __ockl_wfred_max_u32(last_l);
    const double incl = __ockl_wfscan_add_f64(ps, true);
    const double total64 = readlane_f64(incl, kWave - 1), mass = readlane_f64(incl - ps, p * GPW);
    if (p == 0 && tid == 0) {
        plan->n0 = n_list;
        plan->groups = (n_list + kGroup - 1u) / kGroup;
        plan->total64 = total64;
        plan->thr = n_cand;
        const bool gaps_matter = n_cand < n_list && d_arg.out_cand_idx && d_arg.out_cand_q && d_arg.cand_cap;
        plan->flag = n_cand == 0u ? kIndexEmpty : (gaps_matter ? kIndexWhole : kIndexReady);
    }
    if (n_cand == 0u || p * kSpan >= n_list) // uniform
        return;
    const uint32_t off = p * kSpan, cnt = min(kSpan, n_list - off);
    const uint32_t groups = (cnt + kGroup - 1u) / kGroup; // <= 16 GPW <= 64
    const GlobalKeys kf{sc_val.key[0] + (size_t)row * sc_val.vpad};
    const GroupTable& T = sc_val.gt;
    const size_t t_at = (size_t)row * sc_val.g_cap + p * (kSpan / kGroup);
    MAKO_CHECK(sc_val, kCheckGroups, p * (kSpan / kGroup) + groups <= sc_val.g_cap && (uint64_t)off + cnt <= sc_val.vpad);
    float q[GPW][4];
    uint32_t len[GPW];
#pragma unroll
    for (uint32_t k = 0; k < GPW; ++k) {
        const uint32_t g = wave + k * (uint32_t)kWaves;
        len[k] = g < groups ? min(kGroup, cnt - g * kGroup) : 0u; // uniform per wave
        load_span(kf, off + min(g, groups - 1u) * kGroup, len[k], q[k]);
    }
    if (GPW < 4u && tid < (uint32_t)kWave)
        s_gs[tid] = 0.0;
    if (GPW < 4u)
        __syncthreads();
#pragma unroll
    for (uint32_t k = 0; k < GPW; ++k) {
        const double s = __ockl_wfred_add_f64((((double)q[k][0] + (double)q[k][1]) + (double)q[k][2]) + (double)q[k][3]);
        if (lane == 0)
            s_gs[wave + k * (uint32_t)kWaves] = len[k] ? s : 0.0;
    }
    __syncthreads();
    // the sums before and behind each group: lane g holds group g's
    const double v = s_gs[lane];
    const double upto = __ockl_wfscan_add_f64(v, true);
    const double before_l = mass + (upto - v), after_l = mass + upto;
    const double r0_raw = (double)u_row * total64, r0 = r0_raw == r0_raw ? r0_raw : 0.0;
#pragma unroll
    for (uint32_t k = 0; k < GPW; ++k) {
        const uint32_t g = uniform_u32(wave + k * (uint32_t)kWaves);
        if (g >= groups) // uniform per wave
            break;
        const double guess = readlane_f64(before_l, g), at_end = readlane_f64(after_l, g);
        const int eg = guess > 0 ? exponent_of((float)guess) : 0;
        const seqfp::Step32 st = span_map<true>(q[k], len[k], eg);
        // the sum is expected to change binade inside the group (or starts at zero): records for its quarters
        const bool split4 = uniform_u32((uint32_t)(eg == 0 || exponent_of((float)at_end) != eg)) != 0;
        if (split4)
            build_quarters(q[k], len[k], guess, T.quarters + (t_at + g) * 4u);
        // the walk's map, where the walk is expected to pass the group without changing binade in it
        const double r_here = r0 - guess, r_after = r0 - at_end;
        const int ew = (r0 > 0.0 && r_after > 0.0) ? exponent_of((float)r_here) : 0;
        uint4 wrec = make_uint4(0u, 0u, 0u, 0u);
        if (ew > 0 && uniform_u32((uint32_t)(exponent_of((float)r_after) == ew)) != 0) {
            const seqfp::Step32 sw = span_map<true>(q[k], len[k], ew);
            const float q_top = __uint_as_float(__ockl_wfred_max_u32(max(max(__float_as_uint(q[k][0]), __float_as_uint(q[k][1])),
                                                                         max(__float_as_uint(q[k][2]), __float_as_uint(q[k][3])))));
            wrec = make_uint4(sw.d0, sw.d1, walk_need(q_top, ew, sw.cmax), (uint32_t)ew);
        }
        if (lane == 0) {
            T.sum[t_at + g] = s_gs[g];
            T.d0[t_at + g] = st.d0;
            T.d1[t_at + g] = st.d1;
            T.cmax[t_at + g] = st.cmax;
            T.start[t_at + g] = off + g * kGroup;
            T.pack[t_at + g] = len[k] | ((uint32_t)eg << 16) | (split4 ? kHasQuarters : 0u);
            T.walk[t_at + g] = wrec;
        }
    }
}

// grid = (1, rows).
__global__ __launch_bounds__(kThreads) void index_tail_kernel(mako_sample_desc d_arg, Scratch sc_val)
{
    extern __shared__ __align__(16) unsigned long long s_dyn64[];
    __shared__ FinishShared sm;
    __shared__ ArgsLds s_args;
    const uint32_t row = blockIdx.y, tid = threadIdx.x;
    const mako_sampling_params P0 = d_arg.params[row];
    if (classify(P0) != kGeneral) // uniform
        return;
    const bool in_order = index_order_row(P0);
    const BigPlan* planned = sc_val.plan + row;
    const uint32_t flag = planned->flag, n0 = min(planned->n0, d_arg.n_vocab), n_cand = planned->thr;
    const uint32_t groups = min(planned->groups, min(kMaxGroups, sc_val.g_cap));
    const double total64 = planned->total64;
    const float m = planned->m;
    const uint32_t argidx = planned->argidx;
    MAKO_ROW(row);
    stage_args(d_arg, sc_val, row, s_args); // (with a barrier: the plan has been read)
    const mako_sample_desc& d = s_args.d;
    const Scratch& sc = s_args.sc;
    if (tid == 0)
        sc.plan[row].flag = 0;
    const FinishLds L = finish_lds_views(sm, s_dyn64);
    if (!in_order) {
        // the whole-row path from the weights index_weights_kernel left (the group records' kernel has not touched the row)
        if (flag != kIndexClaimed) // (never)
            return;
        __syncthreads();
        if (tid < 32)
            sm.tab[tid] = k_exp2_tab[tid];
        __syncthreads();
        // (the pieces' counts of candidates: when every logit is one, index_weights_kernel's list is the row's list)
        const uint32_t pieces = (d.n_vocab + kSliceMax - 1u) / kSliceMax;
        uint32_t counted = 0;
        for (uint32_t p = 0; p < pieces; ++p)
            counted += sc.plan[row].cursor[p];
        general_row_from_weights<0>(d, sc, row, s_args.P, argidx, sc.plan[row].n0 == kIndexListed && uniform_u32(counted) == d.n_vocab, L);
        return;
    }
    if (flag != kIndexReady && flag != kIndexWhole && flag != kIndexEmpty) // (never)
        return;
    if (flag == kIndexEmpty) {
        fallback_row(d, row, argidx);
        return;
    }
    if (flag == kIndexReady) {
        const uint32_t* kf = sc.key[0] + (size_t)row * sc.vpad;
        // (entry i of the list is token i: no array of token ids)
        // (verification has an instance of its own: its code costs the plain one registers)
        const bool done = d.draft ? sorted_tail<true, false, false, false, true, true>(d, row, s_args.P, kf, nullptr, n0, true, total64, MAKO_PATH_INDEXED,
                                                                                        L, false, 0.0f, sc.gt, (size_t)row * sc.g_cap, groups)
                                  : sorted_tail<true, false, false, false, true, false>(d, row, s_args.P, kf, nullptr, n0, true, total64, MAKO_PATH_INDEXED,
                                                                                         L, false, 0.0f, sc.gt, (size_t)row * sc.g_cap, groups);
        if (done) {
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
