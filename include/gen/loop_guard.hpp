// mako::gen::LoopGuard with the reference's interface (src/gen/loop_guard.hpp:15-33): host-side integer logic of
// the decode loop, no device work.  A generation is "in a loop" when the tokens so far end in a stretch that
// repeats with some period p in 1..max_period at least four times: either exactly, over at least min_tokens
// positions (and at least 3 p of them), or nearly, with at least 90 % of the last 2 * min_tokens positions equal to
// the token p places earlier (a loop with a counter in it).  Cost per token: one comparison per period.
//
// Behaviour follows src/gen/loop_guard.cpp:17-55 (which period wins, where the loop is said to start); the state is
// kept differently: one record per period and a bit ring per period packed into 64-bit words.
#pragma once

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <vector>

namespace mako::gen {

class LoopGuard {
public:
    explicit LoopGuard(uint32_t min_tokens, uint32_t max_period = 512)
        : min_tokens_(min_tokens), max_period_(std::max<uint32_t>(1, max_period)), window_(2 * min_tokens),
          words_((window_ + 63) / 64)
    {
        reset();
    }

    // Forgets the tokens so far.
    void reset()
    {
        history_.clear();
        periods_.assign(max_period_ + 1, Period{});
        ring_.assign(size_t(max_period_ + 1) * words_, 0);
        start_ = 0;
        period_ = 0;
    }

    // Takes the next token; true when the tokens so far end in a loop (start() and period() then say where).
    bool push(int32_t token)
    {
        history_.push_back(token);
        if (min_tokens_ == 0)
            return false; // off
        const size_t n = history_.size();
        const size_t slot = (n - 1) % window_;
        const uint64_t slot_bit = uint64_t(1) << (slot & 63);
        bool reported = false;
        const uint32_t last_period = uint32_t(std::min<size_t>(max_period_, n - 1));
        for (uint32_t p = 1; p <= last_period; ++p) {
            Period& st = periods_[p];
            const bool equal = token == history_[n - 1 - p];
            st.run = equal ? st.run + 1 : 0;
            // the ring holds, for the last window_ positions, whether each equalled the token p before it
            uint64_t& word = ring_[size_t(p) * words_ + (slot >> 6)];
            if (word & slot_bit)
                --st.hits;
            if (equal) {
                ++st.hits;
                word |= slot_bit;
            } else {
                word &= ~slot_bit;
            }
            if (reported)
                continue; // the smallest period that qualifies is the one reported; the others are only kept current
            if (st.run >= std::max(min_tokens_, 3 * p)) {
                // exactly periodic over run + p tokens: at least four periods
                start_ = n - st.run - p;
                period_ = p;
                reported = true;
            } else if (4 * p <= window_ && n >= size_t(window_) + p && 10ull * st.hits >= 9ull * window_) {
                // nearly periodic: the loop is taken to start one period before the window's first match
                size_t k = n - window_;
                while (history_[k] != history_[k - p])
                    ++k;
                start_ = k - p;
                period_ = p;
                reported = true;
            }
        }
        return reported;
    }

    // Index (in tokens pushed since the last reset) of the loop's first token, and its period.
    size_t start() const { return start_; }
    uint32_t period() const { return period_; }

private:
    struct Period {
        uint32_t run = 0;  // trailing positions equal to the token `p` before
        uint32_t hits = 0; // such positions among the last window_
    };
    uint32_t min_tokens_, max_period_, window_, words_;
    std::vector<int32_t> history_;
    std::vector<Period> periods_;
    std::vector<uint64_t> ring_;
    size_t start_ = 0;
    uint32_t period_ = 0;
};

} // namespace mako::gen
