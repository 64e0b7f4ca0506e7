// mako::gen::Sampler on an MI355X: the reference's C++ call surface
// (src/gen/sampler.hpp:11-45) over the C ABI of mako_sampler.h.
//
// Same constructor, greedy(), sample(), verify() and accept() as the reference
// class, same SamplingParams, same exception on an empty vocabulary
// (src/gen/sampler.cpp:11-12).  Like the reference it keeps the accept()
// counts in a host map and owns a std::mt19937_64 seeded by the caller; every
// uniform the reference would draw through uniform_real_distribution<float> is
// drawn here with generate_canonical<float, 24> and handed to the device, so
// with the same standard library the token stream is the reference's.
// Logits are host pointers, as in src/gen/session.cpp:443 (device-resident
// logits go through mako_sampler_sample_batch of the C ABI instead).  Link with
// libmako_sampler.so.
#pragma once

#include <cstdint>
#include <limits>
#include <random>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "../mako_sampler.h"

namespace mako::gen {

// Applied in this order: penalties, temperature, min_p, top_k, top_p.
struct SamplingParams {
    float temperature = 1.0f; // <= 0: greedy
    uint32_t top_k = 0;       // 0: no limit
    float top_p = 1.0f;
    float min_p = 0.0f;
    float presence_penalty = 0.0f, frequency_penalty = 0.0f;
    float repetition_penalty = 1.0f;
};

class Sampler {
public:
    Sampler(const SamplingParams& p, uint32_t n_vocab, uint64_t seed, int device = 0)
        : p_(p), n_vocab_(n_vocab), device_(device), rng_(seed)
    {
        if (n_vocab == 0)
            throw std::invalid_argument("sampler: empty vocabulary");
    }
    ~Sampler()
    {
        if (ctx_)
            mako_sampler_destroy(ctx_);
    }
    Sampler(const Sampler&) = delete;
    Sampler& operator=(const Sampler&) = delete;

    bool greedy() const { return p_.temperature <= 0.0f; }

    int32_t sample(const float* logits)
    {
        const float u = greedy() ? 0.0f : std::generate_canonical<float, 24>(rng_);
        int32_t token = 0;
        run(logits, u, nullptr, 0.0f, nullptr, &token);
        return token;
    }

    // Speculative verification (src/gen/sampler.cpp:86-107): one uniform for the acceptance test, a second
    // one only when the draft is rejected.
    int32_t verify(const float* logits, int32_t draft, bool& accepted)
    {
        std::mt19937_64 ahead = rng_;
        float u1 = 0.0f, u2 = 0.0f;
        if (!greedy()) {
            u1 = std::generate_canonical<float, 24>(ahead);
            u2 = std::generate_canonical<float, 24>(ahead);
        }
        int32_t token = 0;
        uint8_t acc = 0;
        run(logits, u1, &draft, u2, &acc, &token);
        accepted = acc != 0;
        if (!greedy()) {
            rng_.discard(1);
            // the reference redraws unless the draft was accepted or was the only candidate (sampler.cpp:103-106)
            // (a rejected draft that is returned anyway held all the weight: no second draw happened)
            if (!accepted && token != draft)
                rng_.discard(1);
        }
        return token;
    }

    // Records a generated token (for the penalties).
    void accept(int32_t token)
    {
        ++counts_[token];
        dirty_ = true;
    }

private:
    void ensure(uint32_t hist)
    {
        if (ctx_ && hist <= max_hist_)
            return;
        if (ctx_)
            mako_sampler_destroy(ctx_);
        ctx_ = nullptr;
        max_hist_ = hist < 256 ? 256 : hist * 2;
        if (mako_sampler_create(&ctx_, device_, 1, n_vocab_, max_hist_) != MAKO_OK) {
            const std::string why = ctx_ ? mako_sampler_last_error(ctx_) : "invalid argument";
            if (ctx_)
                mako_sampler_destroy(ctx_);
            ctx_ = nullptr;
            throw std::runtime_error("sampler: " + why);
        }
    }

    void run(const float* logits, float u, const int32_t* draft, float u2, uint8_t* acc, int32_t* token)
    {
        if (dirty_) { // counts_ as (id, count) pairs
            ids_.clear();
            cnts_.clear();
            for (const auto& [t, n] : counts_) {
                ids_.push_back(t);
                cnts_.push_back(n);
            }
            dirty_ = false;
        }
        const uint32_t hl = uint32_t(ids_.size());
        ensure(hl);
        mako_sampling_params mp{p_.temperature,      p_.top_k,           p_.top_p,           p_.min_p,
                                p_.presence_penalty, p_.frequency_penalty, p_.repetition_penalty};
        const int rc = mako_sampler_sample_host(ctx_, logits, n_vocab_, 1, n_vocab_, &mp, &u, nullptr, 0,
                                                hl ? ids_.data() : nullptr, hl ? cnts_.data() : nullptr, hl,
                                                hl ? &hl : nullptr, draft, draft ? &u2 : nullptr, acc, token);
        if (rc == MAKO_ERR_INVALID_ARG)
            throw std::invalid_argument(mako_sampler_last_error(ctx_));
        if (rc != MAKO_OK)
            throw std::runtime_error(mako_sampler_last_error(ctx_));
    }

    SamplingParams p_;
    uint32_t n_vocab_;
    int device_;
    std::mt19937_64 rng_;
    std::unordered_map<int32_t, uint32_t> counts_;
    std::vector<int32_t> ids_;
    std::vector<uint32_t> cnts_;
    bool dirty_ = false;
    mako_sampler_ctx* ctx_ = nullptr;
    uint32_t max_hist_ = 0;
};

} // namespace mako::gen
