// C entry points around the UNMODIFIED reference sampler, compiled from where it
// lies under /root/reference (src/gen/sampler.cpp + src/gen/sampler.hpp) -- TEST
// INFRASTRUCTURE ONLY.  The build output goes to oracle/_ref/ and is never part
// of the shipped library.  It pins the oracle restatement and serves as the
// timed CPU baseline.
//
// The reference keeps its candidate list private; the shim reads it after a
// call to report the candidate ids and weights the reference itself computed.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <random>
#include <thread>
#include <vector>

#define private public
#include "gen/sampler.hpp"
#undef private

using mako::gen::Sampler;
using mako::gen::SamplingParams;

extern "C" {

struct ref_params { // same field order as SamplingParams, src/gen/sampler.hpp:11-20
    float temperature;
    uint32_t top_k;
    float top_p, min_p, presence_penalty, frequency_penalty, repetition_penalty;
};

static SamplingParams to_params(const ref_params& p)
{
    SamplingParams s;
    s.temperature = p.temperature;
    s.top_k = p.top_k;
    s.top_p = p.top_p;
    s.min_p = p.min_p;
    s.presence_penalty = p.presence_penalty;
    s.frequency_penalty = p.frequency_penalty;
    s.repetition_penalty = p.repetition_penalty;
    return s;
}

static void apply_mask(std::vector<float>& row, const uint32_t* mask)
{
    if (!mask)
        return;
    for (size_t i = 0; i < row.size(); ++i)
        if (!((mask[i >> 5] >> (i & 31)) & 1u))
            row[i] = -INFINITY;
}

// The uniforms a Sampler seeded with `seed` consumes: draw d is
// uniform_real_distribution<float>(0, 1)(rng), i.e. generate_canonical<float,24>.
void ref_uniforms(uint64_t seed, uint32_t n, float* out)
{
    std::mt19937_64 rng(seed);
    for (uint32_t i = 0; i < n; ++i)
        out[i] = std::generate_canonical<float, 24>(rng);
}

// Fresh Sampler(p, n_vocab, seed); accept() every history token; one sample().
// cand_idx/cand_q (optional, capacity cap) receive the reference's candidate list.
int32_t ref_sample(const float* logits, uint32_t n_vocab, const ref_params* p, const int32_t* hist, uint32_t n_hist,
                   const uint32_t* mask, uint64_t seed, uint32_t* n_cand, int32_t* cand_idx, float* cand_q,
                   uint32_t cap)
{
    std::vector<float> row(logits, logits + n_vocab);
    apply_mask(row, mask);
    Sampler s(to_params(*p), n_vocab, seed);
    for (uint32_t h = 0; h < n_hist; ++h)
        s.accept(hist[h]);
    const int32_t t = s.sample(row.data());
    if (n_cand)
        *n_cand = s.greedy() ? 0 : uint32_t(s.cand_.size());
    if (!s.greedy() && cand_idx && cand_q)
        for (size_t i = 0; i < s.cand_.size() && i < cap; ++i) {
            cand_idx[i] = s.cand_[i].second;
            cand_q[i] = s.cand_[i].first;
        }
    return t;
}

int32_t ref_verify(const float* logits, uint32_t n_vocab, const ref_params* p, const int32_t* hist, uint32_t n_hist,
                   const uint32_t* mask, uint64_t seed, int32_t draft, int* accepted)
{
    std::vector<float> row(logits, logits + n_vocab);
    apply_mask(row, mask);
    Sampler s(to_params(*p), n_vocab, seed);
    for (uint32_t h = 0; h < n_hist; ++h)
        s.accept(hist[h]);
    bool acc = false;
    const int32_t t = s.verify(row.data(), draft, acc);
    *accepted = acc;
    return t;
}

// std::nth_element under the reference's comparator (sampler.cpp:39), for the
// pin of the oracle's restated introselect.
void ref_nth_element(float* q, int32_t* idx, uint32_t n, uint32_t nth)
{
    std::vector<std::pair<float, int32_t>> v(n);
    for (uint32_t i = 0; i < n; ++i)
        v[i] = {q[i], idx[i]};
    auto desc = [](const auto& a, const auto& b) { return a.first > b.first || (a.first == b.first && a.second < b.second); };
    std::ranges::nth_element(v, v.begin() + nth, desc);
    for (uint32_t i = 0; i < n; ++i) {
        q[i] = v[i].first;
        idx[i] = v[i].second;
    }
}

float ref_libm_expf(float x) { return std::exp(x); }

// A worst-case input for libstdc++'s nth_element (McIlroy's adversary, "A Killer Adversary for
// Quicksort", 1999): the comparator decides the values lazily so that every pivot is bad, which drives
// __introselect into its depth limit and its heap-select branch.  q_out[i] is the weight of item i such
// that ordering by (q desc, idx asc) replays the same comparisons.  Returns the comparisons made.
long ref_make_nth_killer(uint32_t n, uint32_t nth, float* q_out)
{
    std::vector<int> val(n, int(n) - 1), items(n);
    const int gas = int(n) - 1;
    int nsolid = 0, candidate = 0;
    long ncmp = 0;
    for (uint32_t i = 0; i < n; ++i)
        items[i] = int(i);
    auto less = [&](int x, int y) {
        ++ncmp;
        if (val[x] == gas && val[y] == gas) {
            if (x == candidate)
                val[x] = nsolid++;
            else
                val[y] = nsolid++;
        }
        if (val[x] == gas)
            candidate = x;
        else if (val[y] == gas)
            candidate = y;
        return val[x] < val[y] || (val[x] == val[y] && x < y);
    };
    std::nth_element(items.begin(), items.begin() + nth, items.end(), less);
    for (uint32_t i = 0; i < n; ++i)
        q_out[i] = float(int(n) - val[i]);
    return ncmp;
}

// Timed CPU baseline: one fresh Sampler per row, history replayed through
// accept() (untimed), then sample() timed.  Rows are split statically over
// n_threads threads.  Masks are applied to a private copy before timing.
// Returns the wall-clock seconds of the slowest thread's sample() calls.
double ref_sample_batch_timed(const float* logits, int64_t row_stride, uint32_t n_rows, uint32_t n_vocab,
                              const ref_params* params, const int32_t* hist, int64_t hist_stride,
                              const uint32_t* hist_len, const uint32_t* mask, int64_t mask_stride,
                              const uint64_t* seeds, uint32_t n_threads, int32_t* out_tokens)
{
    if (n_threads == 0)
        n_threads = 1;
    std::vector<double> secs(n_threads, 0.0);
    auto work = [&](uint32_t tid) {
        std::vector<float> row;
        double acc = 0;
        for (uint32_t r = tid; r < n_rows; r += n_threads) {
            const float* src = logits + int64_t(r) * row_stride;
            Sampler s(to_params(params[r]), n_vocab, seeds[r]);
            if (hist && hist_len)
                for (uint32_t h = 0; h < hist_len[r]; ++h)
                    s.accept(hist[int64_t(r) * hist_stride + h]);
            if (mask) {
                row.assign(src, src + n_vocab);
                apply_mask(row, mask + int64_t(r) * mask_stride);
                src = row.data();
            }
            const auto t0 = std::chrono::steady_clock::now();
            out_tokens[r] = s.sample(src);
            acc += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        }
        secs[tid] = acc;
    };
    std::vector<std::thread> th;
    for (uint32_t t = 1; t < n_threads; ++t)
        th.emplace_back(work, t);
    work(0);
    for (auto& t : th)
        t.join();
    return *std::max_element(secs.begin(), secs.end());
}

} // extern "C"
