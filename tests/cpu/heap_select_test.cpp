// Host restatement of heap_select_rest() (mako_amd/csrc/whole_row.h), the depth-limit branch of the sampler's
// nth_element: libstdc++'s __heap_select(first, nth + 1, last) + iter_swap(first, nth) done (a) with __make_heap's
// sifts grouped by heap level (the device runs a level's sifts side by side; here they are run in the OPPOSITE order
// within a level, which only gives the same heap if they really are independent) and (b) with the sweep over the rest
// taken 64 entries per "ballot" against the current root, re-asked behind every pop.
//
// Checks, against the library routine itself (std::__heap_select is what std::nth_element calls, bits/stl_algo.h:1956):
// the arrangement is identical on random, sorted, reversed, constant and few-valued inputs of many sizes; and counts
// the dependent steps the device version makes on a whole 129 280-entry row in the worst orders, to show that the time
// is bounded by ballots + pops x heap depth, not by one dependent memory access per entry.
//
//   g++ -O2 -std=c++17 heap_select_test.cpp -o heap_select_test && ./heap_select_test
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <numeric>
#include <random>
#include <vector>

typedef unsigned long long u64;

struct Counts {
    long levels = 0, level_rounds = 0, longest_sift = 0, ballots = 0, pops = 0, pop_steps = 0;
};

// The device algorithm on a[first, last): names as in whole_row.h.
static void heap_select_rest(std::vector<u64>& a, uint32_t first, uint32_t last, uint32_t nth, Counts& c)
{
    const uint32_t middle = nth + 1u - first, len = last - first;
    long steps = 0;
    auto hget = [&](uint32_t j) { return a[first + j]; };
    auto hput = [&](uint32_t j, u64 v) { a[first + j] = v; };
    auto sift = [&](uint32_t hole, u64 v) {
        const uint32_t top = hole;
        uint32_t child = hole;
        while (child < (middle - 1u) / 2u) {
            child = 2u * (child + 1u);
            if (hget(child) < hget(child - 1u))
                --child;
            hput(hole, hget(child));
            hole = child;
            ++steps;
        }
        if ((middle & 1u) == 0 && middle >= 2u && child == (middle - 2u) / 2u) {
            child = 2u * (child + 1u);
            hput(hole, hget(child - 1u));
            hole = child - 1u;
            ++steps;
        }
        while (hole > top) {
            const uint32_t parent = (hole - 1u) / 2u;
            if (!(hget(parent) < v))
                break;
            hput(hole, hget(parent));
            hole = parent;
            ++steps;
        }
        hput(hole, v);
    };
    if (middle >= 2u) {
        const uint32_t last_parent = (middle - 2u) / 2u;
        int top_level = 0;
        while ((2u << top_level) - 1u <= last_parent)
            ++top_level;
        for (int level = top_level; level >= 0; --level) {
            const uint32_t lo = (1u << level) - 1u, hi = std::min(last_parent, (2u << level) - 2u);
            long longest = 0;
            for (uint32_t p = lo; p <= hi; ++p) { // (left to right: libstdc++ goes right to left)
                steps = 0;
                sift(p, hget(p));
                longest = std::max(longest, steps);
            }
            ++c.levels;
            c.level_rounds += (hi - lo) / 1024 + 1; // rounds of 1024 threads
            c.longest_sift = std::max(c.longest_sift, longest);
        }
    }
    u64 root = hget(0);
    for (uint32_t base = middle; base < len; base += 64) {
        const uint32_t cnt = std::min(64u, len - base);
        u64 v[64];
        for (uint32_t l = 0; l < cnt; ++l)
            v[l] = a[first + base + l];
        u64 bal = 0;
        for (uint32_t l = 0; l < cnt; ++l)
            bal |= (u64)(v[l] < root) << l;
        ++c.ballots;
        while (bal) {
            const int l = __builtin_ctzll(bal);
            a[first + base + l] = root;
            steps = 0;
            sift(0u, v[l]);
            ++c.pops;
            c.pop_steps += steps;
            root = hget(0);
            bal = 0;
            for (uint32_t k = l + 1; k < cnt; ++k)
                bal |= (u64)(v[k] < root) << k;
            ++c.ballots;
        }
    }
    std::swap(a[first], a[nth]);
}

static void library(std::vector<u64>& a, uint32_t first, uint32_t last, uint32_t nth)
{
    std::__heap_select(a.begin() + first, a.begin() + nth + 1, a.begin() + last, __gnu_cxx::__ops::__iter_less_iter());
    std::iter_swap(a.begin() + first, a.begin() + nth);
}

static int failures = 0;
static Counts check(const char* what, const std::vector<u64>& in, uint32_t first, uint32_t last, uint32_t nth, bool say = false)
{
    std::vector<u64> a = in, b = in;
    Counts c;
    heap_select_rest(a, first, last, nth, c);
    library(b, first, last, nth);
    if (a != b) {
        ++failures;
        printf("FAIL %s: n %zu first %u last %u nth %u\n", what, in.size(), first, last, nth);
    }
    if (say)
        printf("%-28s heap %6u of %6u: %2ld levels in %3ld rounds (longest sift %2ld steps), %6ld ballots, %6ld pops, "
               "%7ld sift steps in pops\n", what, nth + 1 - first, last - first, c.levels, c.level_rounds, c.longest_sift,
               c.ballots, c.pops, c.pop_steps);
    return c;
}

int main()
{
    std::mt19937_64 rng(12345);
    // distinct 64-bit values, as the device's key << 32 | idx are
    auto random_values = [&](uint32_t n, uint32_t distinct_keys) {
        std::vector<u64> a(n);
        for (uint32_t i = 0; i < n; ++i)
            a[i] = ((u64)(rng() % distinct_keys) << 32) | i;
        return a;
    };
    int cases = 0;
    for (uint32_t n : {1u, 2u, 3u, 4u, 5u, 7u, 8u, 9u, 31u, 64u, 65u, 100u, 127u, 128u, 129u, 1000u, 4097u, 20000u})
        for (uint32_t keys : {1u, 2u, 7u, 1000000u})
            for (int rep = 0; rep < 6; ++rep) {
                std::vector<u64> a = random_values(n, keys);
                if (rep == 1)
                    std::sort(a.begin(), a.end());
                if (rep == 2)
                    std::sort(a.begin(), a.end(), std::greater<u64>());
                const uint32_t first = n > 4 ? (uint32_t)(rng() % (n / 4)) : 0u;
                const uint32_t last = n - (n > 4 ? (uint32_t)(rng() % (n / 4)) : 0u);
                if (last - first < 1)
                    continue;
                const uint32_t nth = first + (uint32_t)(rng() % (last - first));
                check("random", a, first, last, nth);
                check("nth = first", a, first, last, first);
                check("nth = last - 1", a, first, last, last - 1);
                cases += 3;
            }
    printf("%d cases against std::__heap_select: %d failures\n", cases, failures);

    // the device's worst cases on a whole row: a descending range (in the heap's order every entry of the rest beats
    // the root: one pop per entry) and an ascending one (none does), heaps that fit LDS and one that does not
    const uint32_t V = 129280;
    std::vector<u64> desc(V), asc(V), rnd = random_values(V, 1u << 30);
    for (uint32_t i = 0; i < V; ++i) {
        desc[i] = ((u64)(V - i) << 32) | i;
        asc[i] = ((u64)i << 32) | i;
    }
    for (uint32_t nth : {40u, 3000u, 8191u, 20000u, 100000u}) {
        check("every entry pops", desc, 0, V, nth, true);
        check("no entry pops", asc, 0, V, nth, true);
        check("random order", rnd, 0, V, nth, true);
    }
    // the bound the kernel's time follows from: ballots <= entries / 64 + pops, pops <= entries, and a pop's sift is at
    // most 2 x the heap's depth steps; nothing is proportional to entries x memory latency
    {
        Counts c = check("every entry pops", desc, 0, V, 8191u);
        const long depth = 13;
        if (c.pops > (long)V || c.pop_steps > c.pops * 2 * depth || c.ballots > (long)V / 64 + 1 + c.pops || c.levels > depth + 1) {
            ++failures;
            printf("FAIL: step counts beyond the stated bounds\n");
        }
    }
    printf(failures ? "FAILED\n" : "ok\n");
    return failures ? 1 : 0;
}
