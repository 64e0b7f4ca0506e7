// TEST INFRASTRUCTURE ONLY: this build's LoopGuard and LookupDrafter (include/gen/) against the UNMODIFIED reference
// classes, compiled from where they lie under /root/reference (src/gen/loop_guard.cpp, src/gen/lookup.cpp), on
// random token streams rich in repeats.  Built into oracle/_ref/ by the Makefile where the reference tree is mounted.
// Prints "N differences" last.
#include <algorithm>
#include <array>
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <random>
#include <span>
#include <unordered_map>
#include <vector>

#include "gen/lookup.hpp"     // the reference's (-I$(REF)/src)
#include "gen/loop_guard.hpp" // the reference's

namespace mine { // (the standard headers above are already in: only the classes land in here)
#include "../include/gen/lookup.hpp"
#include "../include/gen/loop_guard.hpp"
} // namespace mine

int main()
{
    std::mt19937_64 rng(2024);
    long differences = 0, steps = 0, fired = 0, proposals = 0;
    // LoopGuard: text that alternates between noise, exact loops and loops with a changing token
    for (int round = 0; round < 60; ++round) {
        const uint32_t min_tokens = 8 + uint32_t(rng() % 120), max_period = 1 + uint32_t(rng() % 200);
        mako::gen::LoopGuard ref(min_tokens, max_period);
        mine::mako::gen::LoopGuard own(min_tokens, max_period);
        std::vector<int32_t> para;
        for (int i = 0; i < 4000; ++i) {
            const int phase = (i / 500) % 4;
            if (i % 500 == 0) {
                para.resize(1 + rng() % 90);
                for (int32_t& t : para)
                    t = int32_t(rng() % 50);
            }
            int32_t t;
            if (phase == 0)
                t = int32_t(rng() % 6);
            else if (phase == 1)
                t = para[size_t(i) % para.size()];
            else if (phase == 2)
                t = (size_t(i) % para.size() == 2) ? int32_t(1000 + i / para.size()) : para[size_t(i) % para.size()];
            else
                t = int32_t(rng() % 100000);
            if (rng() % 1500 == 0) {
                ref.reset();
                own.reset();
            }
            const bool a = ref.push(t), b = own.push(t);
            ++steps;
            fired += a;
            if (a != b || (a && (ref.start() != own.start() || ref.period() != own.period())))
                ++differences;
        }
    }
    // LookupDrafter: a growing context with copied stretches, cuts, random outcomes
    for (int round = 0; round < 40; ++round) {
        mako::gen::LookupDrafter ref;
        mine::mako::gen::LookupDrafter own;
        std::vector<int32_t> ctx;
        for (int i = 0; i < 3000; ++i) {
            int32_t next;
            if (ctx.size() > 40 && rng() % 3 != 0) {
                const size_t from = rng() % (ctx.size() - 20);
                const size_t len = 1 + rng() % 30;
                for (size_t k = 0; k < len; ++k)
                    ctx.push_back(ctx[from + k]);
                next = ctx[from + len];
            } else {
                ctx.push_back(int32_t(rng() % 40));
                next = int32_t(rng() % 40);
            }
            if (rng() % 400 == 0 && ctx.size() > 30)
                ctx.resize(ctx.size() - 1 - rng() % 25); // the context is cut back
            if (rng() % 700 == 0) {
                ref.clear();
                own.clear();
            }
            const uint32_t min_match = 2 + uint32_t(rng() % 6), max_drafts = 1 + uint32_t(rng() % 7);
            const std::vector<int32_t> a = ref.propose(std::span<const int32_t>(ctx), next, min_match, max_drafts);
            const std::vector<int32_t> b = own.propose(ctx, next, min_match, max_drafts);
            ++steps;
            proposals += !a.empty();
            if (a != b)
                ++differences;
            const uint32_t kept = uint32_t(rng() % (a.size() + 1)) * uint32_t(rng() % 3 != 0);
            ref.outcome(kept);
            own.outcome(kept);
            for (uint32_t bk = 0; bk < 3; ++bk)
                if (ref.acceptance(bk) != own.acceptance(bk))
                    ++differences;
            ctx.push_back(next);
        }
    }
    std::printf("%ld steps, %ld loops reported, %ld proposals\n%ld differences\n", steps, fired, proposals, differences);
    return differences ? 1 : 0;
}
