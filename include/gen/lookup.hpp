// mako::gen::LookupDrafter with the reference's interface (src/gen/lookup.hpp:19-44): drafts taken from the context
// itself, host-side integer logic of the speculative decode loop (the drafts are what the sampler's verify rows then
// accept or reject).  When the tokens being written repeat an earlier stretch of the context, the tokens that
// followed that stretch are proposed.
//
// Behaviour follows src/gen/lookup.cpp:9-101: every trigram of the context remembers the last four positions it
// ended at; the earlier occurrence of the current trigram with the longest backward match (capped at 64, ties to
// the most recent) is taken if the match reaches min_match; 3 drafts for a match of 4-5, 5 for 6-7, 7 from 8, never
// past the current position; per match-length bucket an exponential average (0.2) of "the first draft was kept"
// gates the offers: below 0.55 only every eighth proposal goes out, as a single probe, and a kept probe lifts the
// average back to 0.55.  The index here is keyed by the trigram itself, not by a hash of it.
#pragma once

#include <algorithm>
#include <array>
#include <cstddef>
#include <cstdint>
#include <unordered_map>
#include <vector>

namespace mako::gen {

class LookupDrafter {
public:
    static constexpr uint32_t kMaxDrafts = 7; // with the verified token, the 8 rows an engine verifies at most

    // The tokens likely to follow `next`, which comes after ctx[0..n).  Empty: no match of min_match (>= 3) tokens,
    // or offers of that match length are gated off.  Pointer + length stand in for the reference's std::span.
    std::vector<int32_t> propose(const int32_t* ctx, size_t n, int32_t next, uint32_t min_match,
                                 uint32_t max_drafts = kMaxDrafts)
    {
        offered_bucket_ = -1;
        min_match = std::max<uint32_t>(min_match, 3);
        if (n < min_match)
            return {};
        follow(ctx, n);
        const uint32_t here = uint32_t(text_.size()); // `next` would be text_[here]
        const auto found = ends_.find(Trigram{text_[here - 2], text_[here - 1], next});
        if (found == ends_.end())
            return {};
        uint32_t at = 0, length = 0;
        const Recent& recent = found->second;
        for (uint32_t r = 0; r < recent.count; ++r) { // oldest first: of equal matches the most recent stays
            const uint32_t j = recent.at[(recent.first + r) % kKept];
            uint32_t m = 3;
            while (m < kLongestMatch && m <= j && text_[j - m] == text_[here - m])
                ++m;
            if (m >= length) {
                length = m;
                at = j;
            }
        }
        if (length < min_match || at + 1 >= here)
            return {};
        const uint32_t bucket = bucket_of(length);
        uint32_t drafts = std::min({bucket == 2 ? 7u : bucket == 1 ? 5u : 3u, max_drafts, here - 1 - at});
        if (kept_share_[bucket] < kOpenAbove) {
            if (++held_back_[bucket] % kProbeEvery != 0)
                return {};
            drafts = 1; // a probe
        }
        offered_bucket_ = int(bucket);
        return std::vector<int32_t>(text_.begin() + at + 1, text_.begin() + at + 1 + drafts);
    }
    std::vector<int32_t> propose(const std::vector<int32_t>& ctx, int32_t next, uint32_t min_match,
                                 uint32_t max_drafts = kMaxDrafts)
    {
        return propose(ctx.data(), ctx.size(), next, min_match, max_drafts);
    }

    // How many of the last proposal's drafts were kept, for the gate.
    void outcome(uint32_t kept)
    {
        if (offered_bucket_ < 0)
            return;
        double& share = kept_share_[offered_bucket_];
        share = share * (1.0 - kAverage) + (kept > 0 ? kAverage : 0.0);
        if (kept > 0 && share < kOpenAbove)
            share = kOpenAbove; // a kept probe reopens the bucket; one rejection closes it again
        offered_bucket_ = -1;
    }

    // Drops the index (a parked session); the next propose() rebuilds it.
    void clear()
    {
        text_.clear();
        ends_.clear();
    }

    // The share of first drafts kept, per bucket (match 4-5, 6-7, 8 and more).
    double acceptance(uint32_t bucket) const { return bucket < 3 ? kept_share_[bucket] : 0.0; }

private:
    static constexpr uint32_t kKept = 4;          // most recent occurrences remembered per trigram
    static constexpr uint32_t kLongestMatch = 64; // a backward match is not extended further
    static constexpr double kOpenAbove = 0.55;
    static constexpr double kAverage = 0.2;
    static constexpr uint32_t kProbeEvery = 8;

    using Trigram = std::array<int32_t, 3>;
    struct TrigramHash {
        size_t operator()(const Trigram& t) const
        {
            uint64_t h = 0x9e3779b97f4a7c15ull;
            for (int32_t x : t) {
                h ^= uint64_t(uint32_t(x)) + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2);
                h *= 0xff51afd7ed558ccdull;
            }
            return size_t(h ^ (h >> 32));
        }
    };
    struct Recent { // a ring of the last kKept positions the trigram ended at
        uint32_t at[kKept];
        uint32_t first = 0, count = 0;
        void add(uint32_t pos)
        {
            if (count < kKept) {
                at[(first + count++) % kKept] = pos;
            } else {
                at[first] = pos;
                first = (first + 1) % kKept;
            }
        }
    };

    static uint32_t bucket_of(uint32_t match) { return match >= 8 ? 2 : match >= 6 ? 1 : 0; }

    // The index follows ctx: extended when the indexed text is a prefix of it (judged by its last eight tokens),
    // rebuilt otherwise (the context was cut back).
    void follow(const int32_t* ctx, size_t n)
    {
        const size_t have = text_.size();
        bool prefix = have <= n;
        for (size_t i = have > 8 ? have - 8 : 0; prefix && i < have; ++i)
            prefix = text_[i] == ctx[i];
        if (!prefix)
            clear();
        const size_t from = text_.size();
        text_.insert(text_.end(), ctx + from, ctx + n);
        for (size_t pos = std::max<size_t>(from, 2); pos < text_.size(); ++pos)
            ends_[Trigram{text_[pos - 2], text_[pos - 1], text_[pos]}].add(uint32_t(pos));
    }

    std::vector<int32_t> text_;
    std::unordered_map<Trigram, Recent, TrigramHash> ends_;
    double kept_share_[3] = {0.8, 0.8, 0.8};
    uint32_t held_back_[3] = {0, 0, 0};
    int offered_bucket_ = -1;
};

} // namespace mako::gen
