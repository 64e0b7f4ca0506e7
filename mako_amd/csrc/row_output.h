// A row's results, written in one place.
#pragma once

#include "sampler_common.h"

namespace mako {

struct RowOut {
    int32_t token;
    uint32_t n_cand;
    float total;
    float q;
    uint32_t path;
    uint32_t accepted;
    uint32_t forced = MAKO_FORCED_NONE;
};

// The row's results; with append_history also Sampler::accept of the token (src/gen/session.cpp:419-421).  Called
// once per row, by one thread, after everything that reads the row's history in this batch.
__device__ __forceinline__ void write_row(const mako_sample_desc& d, uint32_t row, const RowOut& o)
{
    d.out_tokens[row] = o.token;
    if (d.out_forced)
        d.out_forced[row] = (uint8_t)o.forced;
    if (d.append_history) {
        uint32_t* hl = const_cast<uint32_t*>(d.hist_len);
        const uint32_t len = hl[row];
        if (len < (uint32_t)d.hist_stride) {
            const_cast<int32_t*>(d.hist_tokens)[(int64_t)row * d.hist_stride + len] = o.token;
            hl[row] = len + 1u;
        }
    }
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

// No candidate survived (src/gen/sampler.cpp:37-38): the single candidate (1.0f, first max).
__device__ void fallback_row(const mako_sample_desc& d, uint32_t row, uint32_t argidx)
{
    if (threadIdx.x != 0)
        return;
    RowOut o;
    o.token = (int32_t)argidx;
    o.n_cand = 1;
    o.total = 1.0f;
    o.q = 1.0f;
    o.path = MAKO_PATH_FALLBACK;
    // verifying: u * 1 < 1 accepts the draft iff it is that candidate; otherwise it is the only one left
    o.accepted = d.draft ? (d.draft[row] == (int32_t)argidx) : 0u;
    if (d.out_cand_idx && d.out_cand_q && d.cand_cap) {
        d.out_cand_idx[(size_t)row * d.cand_cap] = (int32_t)argidx;
        d.out_cand_q[(size_t)row * d.cand_cap] = 1.0f;
    }
    write_row(d, row, o);
}

} // namespace mako
