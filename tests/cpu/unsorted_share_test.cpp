// Host restatement of opaque_share() (mako_amd/csrc/worker_sort.h), the record that stands for a share of a sorted
// list that was never sorted: inside one binade of the running fp32 sum the addends that are no exact ties are
// constant increments and commute, so their SUM is their composition; the exact ties are kept apart, ordered by
// weight, and each is composed in between the sums of the increments of the weights on either side of it.
//
// Checked against what the reference does (src/gen/sampler.cpp:80-82, :67-71): the weights sorted descending, added to
// (subtracted from) a running float one by one with real fp32 operations.  Whenever the record passes the tests under
// which tail_kernel applies it (seqfp::group_add_ok / group_sub_ok with the share's largest weight), the state it gives
// must be the sequential loop's, bit for bit, and the walk must not have stopped inside the share; shares with up to a
// dozen exact ties, duplicated weights, increments of zero and weights from higher binades (no map) are among the cases.
//
//   g++ -O2 -std=c++17 -ffp-contract=off -I ../../mako_amd/csrc unsorted_share_test.cpp -o unsorted_share_test
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <random>
#include <vector>

#include "seqfp.h"

using namespace seqfp;

// The map of an unsorted share for the epoch with exponent e, as opaque_share() builds it: one pass for the ties and
// the plain sum (here: the segment sums directly), the ties by weight, the composition.  kSat where the device gives up.
static Step32 share_map(const std::vector<float>& q, int e, uint32_t max_ties, uint32_t& n_ties)
{
    std::vector<uint32_t> ties; // bits(q) of the exact ties
    for (float x : q) {
        const Step32 s = step32_flat(x, e);
        if (s.d0 != s.d1)
            ties.push_back(f2u(x));
    }
    n_ties = (uint32_t)ties.size();
    uint32_t kmax = 0;
    for (float x : q)
        kmax = std::max(kmax, f2u(x));
    Step32 v{kSat, kSat, 0};
    if (ties.size() <= max_ties) {
        std::sort(ties.begin(), ties.end(), std::greater<uint32_t>());
        std::vector<unsigned long long> seg(ties.size() + 1, 0);
        for (float x : q) {
            const Step32 s = step32_flat(x, e);
            if (s.d0 != s.d1)
                continue;
            size_t k = 0; // the number of ties heavier than the weight
            while (k < ties.size() && ties[k] > f2u(x))
                ++k;
            seg[k] += std::min(s.d0, 1u << 24);
        }
        v = identity32();
        for (size_t s = 0; s <= ties.size(); ++s) {
            const uint32_t add = seg[s] < (1ull << 24) ? (uint32_t)seg[s] : kSat;
            v = compose32(v, Step32{add, add, 0});
            if (s < ties.size())
                v = compose32(v, step32_flat(u2f(ties[s]), e));
        }
    }
    v.cmax = step32_flat(u2f(kmax), e).cmax;
    return v;
}

int main()
{
    std::mt19937_64 rng(20261125);
    long cases = 0, applied_add = 0, applied_sub = 0, with_ties = 0, applied_ties = 0, failures = 0;
    for (int rep = 0; rep < 60000; ++rep) {
        // the running value: a float in a random binade, and a share of weights some binades below it
        const int e = 40 + (int)(rng() % 150);
        const uint32_t M = (1u << 23) | (uint32_t)(rng() & 0x7fffffu);
        const int shift_lo = (int)(rng() % 14), shift_hi = shift_lo + 1 + (int)(rng() % 6);
        const size_t n = 1 + rng() % (rep % 7 == 0 ? 3000 : 200);
        // (few mantissa bits: exact ties and duplicates become common)
        const int keep_bits = rep % 3 == 0 ? 24 : 1 + (int)(rng() % 12);
        std::vector<float> q(n);
        for (auto& x : q) {
            const int ex = e - shift_lo - (int)(rng() % (uint32_t)(shift_hi - shift_lo + 1));
            uint32_t m = (uint32_t)(rng() & 0x7fffffu);
            m &= ~((1u << (24 - keep_bits)) - 1u) & 0x7fffffu;
            x = u2f(((uint32_t)std::max(ex, 1) << 23) | m);
        }
        if (rep % 50 == 0)
            q[rng() % n] = u2f(((uint32_t)(e + 1) << 23) | 5u); // a weight from a higher binade: no map
        std::vector<float> sorted = q;
        std::sort(sorted.begin(), sorted.end(), std::greater<float>());
        std::shuffle(q.begin(), q.end(), rng);
        const float q_first = sorted[0];
        ++cases;

        // the running sum
        uint32_t n_ties = 0;
        const Step32 ma = share_map(q, e, 16, n_ties);
        with_ties += n_ties != 0;
        if (group_add_ok((long long)M, ma)) {
            float S = join(M, e);
            for (float x : sorted)
                S += x;
            const uint32_t after = M + ((M & 1u) ? ma.d1 : ma.d0);
            if (f2u(S) != f2u(join(after, e))) {
                ++failures;
                printf("FAIL add: rep %d n %zu e %d M %u ties %u: %a vs %a\n", rep, n, e, M, n_ties, S, join(after, e));
            }
            ++applied_add;
            applied_ties += n_ties != 0;
        }
        // the walk
        const Step32 mw = share_map(q, e, 16, n_ties);
        if (group_sub_ok((long long)M, e, mw, q_first)) {
            float r = join(M, e);
            bool stopped = false;
            for (float x : sorted) {
                if (r < x) {
                    stopped = true;
                    break;
                }
                r -= x;
            }
            const uint32_t after = M - ((M & 1u) ? mw.d1 : mw.d0);
            if (stopped || f2u(r) != f2u(join(after, e))) {
                ++failures;
                printf("FAIL sub: rep %d n %zu e %d M %u ties %u stopped %d: %a vs %a\n", rep, n, e, M, n_ties, (int)stopped, r,
                       join(after, e));
            }
            ++applied_sub;
        }
    }
    printf("%ld shares (%ld with exact ties): record applied to %ld running sums (%ld of them with ties) and %ld walks: %ld failures\n",
           cases, with_ties, applied_add, applied_ties, applied_sub, failures);
    // (the test is worth nothing if the records hardly ever pass the tests)
    if (applied_add < cases / 4 || applied_sub < cases / 8 || applied_ties < cases / 50) {
        printf("too few applications for the test to mean anything\n");
        return 1;
    }
    return failures ? 1 : 0;
}
