// Host helpers of the decode loop: LoopGuard and LookupDrafter (include/gen/loop_guard.hpp, include/gen/lookup.hpp)
// on the scenarios and expected numbers of the reference's own tests (tests/loop_guard_test.cpp:48-108,
// tests/lookup_test.cpp:29-91).  Prints "N failures" last.
#include <cstdint>
#include <cstdio>
#include <random>
#include <vector>

#include "gen/lookup.hpp"
#include "gen/loop_guard.hpp"

using mako::gen::LookupDrafter;
using mako::gen::LoopGuard;

static int failures = 0;
static void expect(bool ok, const char* what)
{
    std::printf("%s %s\n", ok ? "ok  " : "FAIL", what);
    failures += !ok;
}

static std::mt19937 gen(7);
static std::vector<int32_t> varied(size_t n)
{
    std::uniform_int_distribution<int32_t> d(0, 150000);
    std::vector<int32_t> v(n);
    for (int32_t& t : v)
        t = d(gen);
    return v;
}
// tokens pushed when the guard first fires, 0 if never
static size_t fires_at(LoopGuard& g, const std::vector<int32_t>& v)
{
    for (size_t i = 0; i < v.size(); ++i)
        if (g.push(v[i]))
            return i + 1;
    return 0;
}
static void append(std::vector<int32_t>& to, const std::vector<int32_t>& what, size_t n)
{
    to.insert(to.end(), what.begin(), what.begin() + n);
}

static void loop_guard()
{
    {
        LoopGuard g(256);
        expect(fires_at(g, varied(20000)) == 0, "loop guard: 20000 varied tokens, no loop (loop_guard_test.cpp:50-51)");
    }
    {
        std::vector<int32_t> v = varied(100);
        const std::vector<int32_t> para = varied(60);
        for (int i = 0; i < 20; ++i)
            append(v, para, 60);
        LoopGuard g(256);
        const size_t at = fires_at(g, v);
        expect(at == 100 + 60 + 256 && g.start() == 100 && g.period() == 60,
               "loop guard: a repeated 60-token paragraph is found after 100 + 60 + 256 tokens, from 100 (:54-64)");
    }
    {
        std::vector<int32_t> v = varied(100), para = varied(60);
        for (int i = 0; i < 20; ++i) {
            para[5] = 1000 + i; // a counter
            append(v, para, 60);
        }
        LoopGuard g(256);
        const size_t at = fires_at(g, v);
        expect(at > 0 && at <= 100 + 60 * 11 && g.period() == 60 && g.start() == 100,
               "loop guard: the paragraph with a counter is found within 11 repeats, from 100 (:66-78)");
    }
    {
        std::vector<int32_t> v;
        const std::vector<int32_t> row = varied(10);
        for (int i = 0; i < 300; ++i) {
            std::vector<int32_t> r = row;
            for (int j : {1, 4, 7})
                r[size_t(j)] = int32_t(gen() % 150000);
            append(v, r, 10);
        }
        LoopGuard g(256);
        expect(fires_at(g, v) == 0, "loop guard: table rows differing in 3 of 10 tokens are no loop (:80-91)");
    }
    {
        LoopGuard g(256);
        const size_t at = fires_at(g, std::vector<int32_t>(400, 42));
        expect(at == 257 && g.period() == 1 && g.start() == 0, "loop guard: one token repeated fires at 257 (:93-96)");
    }
    {
        std::vector<int32_t> v = varied(50);
        const std::vector<int32_t> para = varied(60), head = v;
        for (int i = 0; i < 3; ++i)
            append(v, para, 60);
        append(v, head, 50);
        LoopGuard g(256);
        expect(fires_at(g, v) == 0, "loop guard: three repeats are fewer than four (:98-105)");
    }
    {
        LoopGuard g(256);
        fires_at(g, std::vector<int32_t>(200, 42));
        g.reset();
        expect(fires_at(g, std::vector<int32_t>(200, 42)) == 0, "loop guard: reset forgets the run (:107-111)");
        LoopGuard off(0);
        expect(fires_at(off, std::vector<int32_t>(5000, 42)) == 0, "loop guard: min_tokens 0 switches it off (:112-113)");
    }
    {
        // the packed bit ring against a plain restatement of the rule, token by token, on loop-rich text
        std::vector<int32_t> v;
        std::uniform_int_distribution<int32_t> small(0, 3);
        for (int i = 0; i < 6000; ++i)
            v.push_back(i % 700 < 350 ? small(gen) : int32_t(i % 37));
        LoopGuard g(40, 64);
        const uint32_t mn = 40, window = 80, maxp = 64;
        std::vector<int32_t> t;
        bool same = true;
        for (int32_t x : v) {
            const bool got = g.push(x);
            t.push_back(x);
            const size_t n = t.size();
            bool want = false;
            size_t ws = 0;
            uint32_t wp = 0;
            for (uint32_t p = 1; p <= maxp && p < n && !want; ++p) {
                uint32_t run = 0;
                while (run + p < n && t[n - 1 - run] == t[n - 1 - run - p])
                    ++run;
                uint32_t hits = 0;
                for (size_t k = n > window ? n - window : 0; k < n; ++k)
                    hits += k >= p && t[k] == t[k - p];
                if (run >= std::max(mn, 3 * p)) {
                    want = true, ws = n - run - p, wp = p;
                } else if (4 * p <= window && n >= window + p && 10ull * hits >= 9ull * window) {
                    size_t k = n - window;
                    while (t[k] != t[k - p])
                        ++k;
                    want = true, ws = k - p, wp = p;
                }
            }
            if (got != want || (got && (g.start() != ws || g.period() != wp)))
                same = false;
        }
        expect(same, "loop guard: equals a brute-force restatement of the rule on 6000 tokens");
    }
}

static void lookup_drafter()
{
    std::vector<int32_t> passage;
    for (int32_t t = 100; t < 120; ++t)
        passage.push_back(t);
    std::vector<int32_t> ctx = passage;
    for (int32_t t : {7, 8, 9, 10, 11, 12})
        ctx.push_back(t);
    append(ctx, passage, 9);
    using V = std::vector<int32_t>;
    {
        LookupDrafter d;
        expect(d.propose(ctx, 109, 4) == V({110, 111, 112, 113, 114, 115, 116}),
               "lookup: a match of 10 proposes the 7 tokens that followed (lookup_test.cpp:40-42)");
        expect(d.propose(ctx, 50, 4).empty(), "lookup: an unseen trigram proposes nothing (:43)");
    }
    {
        const V c{1, 2, 3, 4, 5, 6, 7, 8, 2, 3};
        LookupDrafter d;
        expect(d.propose(c, 4, 4).empty(), "lookup: a 3-token match is below min_match 4 (:47-49)");
        expect(d.propose(c, 4, 3) == V({5, 6, 7}), "lookup: at min_match 3 it proposes 3 (:50)");
    }
    {
        V c{1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 1, 2, 3, 4};
        LookupDrafter d;
        expect(d.propose(c, 5, 4) == V({6, 7, 8}), "lookup: a match of 5 proposes 3 (:54-56)");
        c.push_back(5);
        expect(d.propose(c, 6, 4) == V({7, 8, 9, 10, 1}), "lookup: a match of 6 proposes 5 (:57-58)");
        const V tail{1, 2, 3, 1, 2, 3, 1, 2};
        expect(d.propose(tail, 3, 4) == V({1, 2}), "lookup: drafts stop before the current position (:60-61)");
    }
    {
        LookupDrafter d;
        int offered = 0, probes = 0;
        for (int r = 0; r < 40; ++r) {
            const V got = d.propose(ctx, 109, 4);
            offered += got.size() == 7;
            probes += got.size() == 1;
            d.outcome(0);
        }
        expect(offered >= 2 && offered <= 4 && probes >= 3, "lookup: rejections close the bucket, probes one in eight (:64-76)");
        int reopened = 0;
        for (int r = 0; r < 40; ++r) {
            const V got = d.propose(ctx, 109, 4);
            reopened += got.size() == 7;
            d.outcome(uint32_t(got.size()));
        }
        expect(reopened >= 28, "lookup: a kept probe reopens the bucket (:77-83)");
    }
    {
        LookupDrafter d;
        d.propose(ctx, 109, 4);
        V cut(ctx.begin(), ctx.begin() + 22);
        for (int32_t t : {40, 41, 42, 43, 44, 45, 40, 41, 42, 43})
            cut.push_back(t);
        expect(d.propose(cut, 44, 4) == V({45, 40, 41}), "lookup: after a cut the index is rebuilt (:86-90)");
        expect(d.propose(cut, 109, 4).empty(), "lookup: the old continuation past the cut is gone (:91)");
    }
}

int main()
{
    loop_guard();
    lookup_drafter();
    std::printf("%d failures\n", failures);
    return failures ? 1 : 0;
}
