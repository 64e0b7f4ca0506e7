// Host unit test of mako_amd/csrc/seqfp.h: a scan over two-state integer maps must
// reproduce a sequential fp32 running sum and the sequential fp32 walk bit for bit.
// The driver below mirrors the kernels' windowed block algorithm with NT
// virtual threads.  Build: g++ -O2 -std=c++17 -ffp-contract=off.
#include "../../mako_amd/csrc/seqfp.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

using namespace seqfp;

static float seq_sum(const std::vector<float>& q)
{
    float s = 0;
    for (float v : q)
        s += v;
    return s;
}

static size_t seq_walk(const std::vector<float>& q, float r)
{
    for (size_t i = 0; i < q.size(); ++i) {
        if (r < q[i])
            return i;
        r -= q[i];
    }
    return q.size() - 1;
}

static float emu_sum(const std::vector<float>& q, int NT, int LMAX, long* rounds)
{
    const size_t n = q.size();
    float S = q[0];
    size_t i0 = 1;
    int L = 1;
    while (i0 < n) {
        ++*rounds;
        uint32_t M;
        int e;
        split(S, M, e);
        const long long m = M;
        const size_t W = std::min(n - i0, size_t(NT) * L);
        std::vector<Step> f(NT, identity());
        for (int t = 0; t < NT; ++t)
            for (size_t j = i0 + size_t(t) * L; j < std::min(i0 + size_t(t + 1) * L, i0 + W); ++j)
                f[t] = compose(f[t], add_step(q[j], e));
        Step pre = identity();
        size_t first = SIZE_MAX;
        long long mm_first = 0, m_end = m;
        for (int t = 0; t < NT; ++t) {
            long long mm = m + ((m & 1) ? pre.d1 : pre.d0);
            size_t j = i0 + size_t(t) * L;
            const size_t jend = std::min(i0 + size_t(t + 1) * L, i0 + W);
            for (; j < jend; ++j) {
                if (add_event(mm, q[j], e))
                    break;
                mm = add_apply(mm, q[j], e);
            }
            if (j < jend && j < first) {
                first = j;
                mm_first = mm;
            }
            if (jend > i0 + size_t(t) * L || t == 0)
                m_end = mm;
            pre = compose(pre, f[t]);
        }
        if (first == SIZE_MAX) {
            // state after the window: m + total map
            m_end = m + ((m & 1) ? pre.d1 : pre.d0);
            S = join(uint32_t(m_end), e);
            i0 += W;
            L = std::min(L * 2, LMAX);
        } else {
            S = join(uint32_t(mm_first), e) + q[first];
            i0 = first + 1;
        }
    }
    return S;
}

static size_t emu_walk(const std::vector<float>& q, float r, int NT, int LMAX)
{
    const size_t n = q.size();
    if (!(r == r) || std::isinf(r))
        return r < 0 ? 0 : n - 1;
    if (r < 0)
        return 0;
    size_t i0 = 0;
    int L = 1;
    for (;;) {
        if (i0 >= n)
            return n - 1;
        uint32_t M;
        int e;
        split(r, M, e);
        const long long m = M;
        const size_t W = std::min(n - i0, size_t(NT) * L);
        std::vector<Step> f(NT, identity());
        for (int t = 0; t < NT; ++t)
            for (size_t j = i0 + size_t(t) * L; j < std::min(i0 + size_t(t + 1) * L, i0 + W); ++j)
                f[t] = compose(f[t], sub_step(q[j], e));
        Step pre = identity();
        size_t first = SIZE_MAX;
        long long mm_first = 0;
        bool stop_first = false;
        for (int t = 0; t < NT; ++t) {
            long long mm = m - ((m & 1) ? pre.d1 : pre.d0);
            size_t j = i0 + size_t(t) * L;
            const size_t jend = std::min(i0 + size_t(t + 1) * L, i0 + W);
            bool stop = false;
            for (; j < jend; ++j) {
                if (walk_stop(mm, q[j], e)) {
                    stop = true;
                    break;
                }
                if (sub_event(mm, q[j], e))
                    break;
                mm = sub_apply(mm, q[j], e);
            }
            if (j < jend && j < first) {
                first = j;
                mm_first = mm;
                stop_first = stop;
            }
            pre = compose(pre, f[t]);
        }
        if (first == SIZE_MAX) {
            const long long m_end = m - ((m & 1) ? pre.d1 : pre.d0);
            r = join(uint32_t(m_end), e);
            i0 += W;
            L = std::min(L * 2, LMAX);
        } else if (stop_first) {
            return first;
        } else {
            r = join(uint32_t(mm_first), e) - q[first];
            i0 = first + 1;
        }
    }
}

// The grouped scheme of the kernels on a sorted list: group maps under epochs guessed from fp64 prefix
// sums, a serial chain that accepts a map only when group_add_ok / group_sub_ok hold and otherwise replays the
// group with real fp32 arithmetic.
static int exponent_of(float x)
{
    uint32_t M;
    int e;
    split(x, M, e);
    return e;
}

static float grouped_sum(const std::vector<float>& q, size_t GS, long* accepted, long* groups)
{
    const size_t n = q.size(), G = (n + GS - 1) / GS;
    std::vector<double> pg(G + 1, 0.0);
    for (size_t g = 0; g < G; ++g) {
        double s = 0;
        for (size_t i = g * GS; i < std::min(n, (g + 1) * GS); ++i)
            s += q[i];
        pg[g + 1] = pg[g] + s;
    }
    float S = 0.0f;
    for (size_t g = 0; g < G; ++g) {
        ++*groups;
        const int eg = pg[g] > 0 ? exponent_of(float(pg[g])) : 0;
        Step32 st = identity32();
        for (size_t i = g * GS; i < std::min(n, (g + 1) * GS); ++i)
            st = compose32(st, step32(q[i], eg));
        uint32_t M;
        int e;
        split(S, M, e);
        if (e == eg && group_add_ok(M, st)) {
            ++*accepted;
            S = join(uint32_t(M + ((M & 1) ? st.d1 : st.d0)), e);
        } else {
            for (size_t i = g * GS; i < std::min(n, (g + 1) * GS); ++i)
                S += q[i];
        }
    }
    return S;
}

static size_t grouped_walk(const std::vector<float>& q, float r, size_t GS, long* accepted, long* groups)
{
    const size_t n = q.size(), G = (n + GS - 1) / GS;
    if (r < 0)
        return 0;
    std::vector<double> pg(G + 1, 0.0);
    for (size_t g = 0; g < G; ++g) {
        double s = 0;
        for (size_t i = g * GS; i < std::min(n, (g + 1) * GS); ++i)
            s += q[i];
        pg[g + 1] = pg[g] + s;
    }
    const double r0 = r;
    for (size_t g = 0; g < G; ++g) {
        ++*groups;
        const double guess = r0 - pg[g];
        const int eg = guess > 0 ? exponent_of(float(guess)) : 0;
        Step32 st = identity32();
        for (size_t i = g * GS; i < std::min(n, (g + 1) * GS); ++i)
            st = compose32(st, step32(q[i], eg));
        uint32_t M;
        int e;
        split(r, M, e);
        if (e == eg && group_sub_ok(M, e, st, q[g * GS])) {
            ++*accepted;
            r = join(uint32_t(M - ((M & 1) ? st.d1 : st.d0)), e);
        } else {
            for (size_t i = g * GS; i < std::min(n, (g + 1) * GS); ++i) {
                if (r < q[i])
                    return i;
                r -= q[i];
            }
        }
    }
    return n - 1;
}

int main()
{
    std::mt19937_64 rng(12345);
    std::uniform_real_distribution<float> U(0.0f, 1.0f);
    std::normal_distribution<float> N(0.0f, 1.0f);
    long fails = 0, cases = 0, rounds = 0;
    // step32_flat() against step32(): every exponent pair, weights with ties, halves just missed, zero and subnormals
    for (int it = 0; it < 2000000; ++it) {
        uint32_t bits = uint32_t(rng()) & 0x7fffffffu;
        if (it % 4 == 1)
            bits &= ~((1u << (rng() % 24)) - 1u); // trailing zeros: exact ties at some shift
        if (it % 4 == 2)
            bits = (bits & 0x7f800000u) | ((1u << (rng() % 23)) + (rng() % 3) - 1u); // around a half
        if (it % 97 == 0)
            bits = uint32_t(rng() % 16); // zero and the smallest subnormals
        if (bits >= 0x7f800000u)
            continue;
        const float q = seqfp::u2f(bits);
        const int e = 1 + int(rng() % 254);
        const seqfp::Step32 x = seqfp::step32(q, e), y = seqfp::step32_flat(q, e);
        ++cases;
        if (x.d0 != y.d0 || x.d1 != y.d1 || x.cmax != y.cmax) {
            if (++fails < 10)
                printf("step32_flat differs: q bits %08x e %d: %u %u %u vs %u %u %u\n", bits, e, x.d0, x.d1, x.cmax, y.d0, y.d1, y.cmax);
        }
    }
    // step32_fp() (the map taken from real additions) against step32_flat(): equal wherever the weight is below 2^23
    // units of the epoch, the "unusable" mark from there on; weights around every tie and around the limits
    long fp_cases = 0, fp_marked = 0;
    for (int it = 0; it < 6000000; ++it) {
        const int e = 1 + int(rng() % 254);
        uint32_t bits;
        switch (it % 6) {
        case 0: bits = uint32_t(rng()) & 0x7fffffffu; break;
        case 1: { // an exponent close to the epoch's, any significand
            const int ex = std::max(0, std::min(254, e - 27 + int(rng() % 30)));
            bits = (uint32_t(ex) << 23) | (uint32_t(rng()) & 0x7fffffu);
            break;
        }
        case 2: { // exact ties and their neighbours at a shift the epoch makes relevant
            const int ex = std::max(0, std::min(254, e - int(rng() % 26)));
            const uint32_t low = 1u << (rng() % 23);
            bits = (uint32_t(ex) << 23) | (((uint32_t(rng()) & 0x7fffffu) & ~(2u * low - 1u)) + low + uint32_t(rng() % 3) - 1u);
            break;
        }
        case 3: bits = uint32_t(rng() % 64); break;                                                  // zero and subnormals
        case 4: bits = (uint32_t(e) << 23) + uint32_t(rng() % 5) - 2u; break;                         // around 2^23 units
        default: bits = (uint32_t(std::max(0, e - 24 - int(rng() % 3))) << 23) | (rng() % 2 ? 0u : uint32_t(rng()) & 0x7fffffu); // around half a unit
        }
        if (bits >= 0x7f800000u)
            continue;
        const float q = seqfp::u2f(bits);
        const seqfp::Step32 x = seqfp::step32_flat(q, e), y = seqfp::step32_fp(q, e);
        ++fp_cases;
        const bool big = !(q < seqfp::u2f(uint32_t(e) << 23)) || e > 253; // (and the last binade, where R + q may overflow)
        fp_marked += big;
        const bool same = big ? (y.d0 == seqfp::kSat && y.d1 == seqfp::kSat) : (x.d0 == y.d0 && x.d1 == y.d1 && x.cmax == y.cmax);
        if (!same && ++fails < 10)
            printf("step32_fp differs: q bits %08x e %d: %u %u %u vs %u %u %u\n", bits, e, x.d0, x.d1, x.cmax, y.d0, y.d1, y.cmax);
    }
    printf("step32_fp: %ld cases (%ld of them at or above 2^23 units)\n", fp_cases, fp_marked);
    for (int it = 0; it < 4000; ++it) {
        const int kind = it % 8;
        size_t n = 1 + rng() % (it % 50 == 0 ? 200000 : 3000);
        std::vector<float> q(n);
        for (auto& v : q) {
            switch (kind) {
            case 0: v = std::exp(3.0f * N(rng)); break;                       // wide
            case 1: v = std::exp(0.1f * N(rng)); break;                       // near flat
            case 2: v = seqfp::u2f(uint32_t(rng() % 0x3f800000u) + 1); break; // any exponent incl. subnormal
            case 3: v = seqfp::u2f(0x3f000000u + uint32_t(rng() % 4) * 0x400000u); break; // many ties
            case 4: v = U(rng); break;
            case 5: v = seqfp::u2f(1 + uint32_t(rng() % 64)); break;          // subnormals
            case 6: v = std::exp(10.0f * N(rng) - 20.0f); break;
            default: v = float(1 + rng() % 8) * 0.125f; break;
            }
            if (!(v > 0))
                v = 1.0f;
        }
        const float mx = *std::max_element(q.begin(), q.end());
        if (kind != 2 && kind != 5)
            for (auto& v : q)
                v = std::min(v / mx, 1.0f);
        const bool sorted = (it / 8) % 2 == 0;
        if (sorted)
            std::sort(q.begin(), q.end(), std::greater<float>());
        const int NT = (it % 3 == 0) ? 7 : ((it % 3 == 1) ? 64 : 1024);
        const int LMAX = (it % 5 == 0) ? 1 : 32;
        const float total = seq_sum(q);
        const float got = emu_sum(q, NT, LMAX, &rounds);
        ++cases;
        if (f2u(total) != f2u(got)) {
            ++fails;
            std::printf("SUM mismatch it=%d n=%zu kind=%d sorted=%d want=%a got=%a\n", it, n, kind, sorted, total, got);
        }
        for (int d = 0; d < 6; ++d) {
            float u = U(rng);
            if (d == 4) u = 0.0f;
            if (d == 5) u = std::nextafter(1.0f, 0.0f);
            const float r = u * total;
            const size_t a = seq_walk(q, r), b = emu_walk(q, r, NT, LMAX);
            ++cases;
            if (a != b) {
                ++fails;
                std::printf("WALK mismatch it=%d n=%zu kind=%d sorted=%d u=%a want=%zu got=%zu\n", it, n, kind, sorted, u, a, b);
            }
        }
    }
    // grouped scheme on sorted lists
    long acc = 0, grp = 0;
    for (int it = 0; it < 1500; ++it) {
        const int kind = it % 5;
        size_t n = 1 + rng() % (it % 25 == 0 ? 300000 : 20000);
        std::vector<float> q(n);
        for (auto& v : q) {
            switch (kind) {
            case 0: v = std::exp(2.5f * N(rng)); break;
            case 1: v = std::exp(0.1f * N(rng)); break;
            case 2: v = std::exp(6.0f * N(rng) - 6.0f); break;
            case 3: v = float(1 + rng() % 16) * 0.0625f; break;
            default: v = U(rng); break;
            }
            if (!(v > 0))
                v = 1.0f;
        }
        const float mx = *std::max_element(q.begin(), q.end());
        for (auto& v : q)
            v = std::min(v / mx, 1.0f);
        std::sort(q.begin(), q.end(), std::greater<float>());
        const size_t GS = (it % 2) ? 256 : 64;
        const float total = seq_sum(q);
        const float got = grouped_sum(q, GS, &acc, &grp);
        ++cases;
        if (f2u(total) != f2u(got)) {
            ++fails;
            std::printf("GROUP SUM mismatch it=%d n=%zu kind=%d want=%a got=%a\n", it, n, kind, total, got);
        }
        for (int dd = 0; dd < 5; ++dd) {
            float u = U(rng);
            if (dd == 3) u = 0.0f;
            if (dd == 4) u = std::nextafter(1.0f, 0.0f);
            const float r = u * total;
            const size_t a = seq_walk(q, r), b = grouped_walk(q, r, GS, &acc, &grp);
            ++cases;
            if (a != b) {
                ++fails;
                std::printf("GROUP WALK mismatch it=%d n=%zu kind=%d u=%a want=%zu got=%zu\n", it, n, kind, u, a, b);
            }
        }
    }
    std::printf("grouped: %ld of %ld groups took the fast map\n", acc, grp);
    std::printf("%ld cases, %ld failures, %ld sum rounds\n", cases, fails, rounds);
    return fails ? 1 : 0;
}
