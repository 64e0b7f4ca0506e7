// Exact parallel emulation of a sequential fp32 running sum and of the
// sequential fp32 inverse-CDF walk.
//
// The reference adds the candidate weights one by one in fp32
// (src/gen/sampler.cpp:80-82) and then subtracts them one by one from
// r = u * total until r < q (src/gen/sampler.cpp:67-71).  Both results depend
// on the order of the roundings, so a tree reduction is not token-exact.
//
// While the accumulator stays inside one binade its value is m * U with an
// integer m < 2^24 and U the binade's ulp.  Adding q = (a + f) * U, 0 <= f < 1,
// rounds to nearest-even: m += a, plus one if f > 1/2, plus (m + a) & 1 if
// f == 1/2.  So inside a binade every element is a map m -> m + c[m & 1]: two
// integers.  Such maps compose associatively, which lets a block scan replay
// thousands of dependent additions at once.  An element that could carry the
// accumulator out of the binade (an "event") is applied with a real fp32
// operation and starts a new epoch.  The same holds for r -= q going down.
//
// This header is plain C++ so that the host unit test and the HIP kernels
// share one implementation.
#pragma once

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define SEQFP_HD __host__ __device__ __forceinline__
#else
#define SEQFP_HD inline
#endif

namespace seqfp {

SEQFP_HD uint32_t f2u(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
SEQFP_HD float u2f(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

// A non-negative finite float is M * 2^(e - 150) with e the biased exponent
// (1 for subnormals) and M < 2^24.
SEQFP_HD void split(float x, uint32_t& M, int& e)
{
    const uint32_t b = f2u(x);
    const uint32_t ex = (b >> 23) & 0xffu;
    M = b & 0x7fffffu;
    if (ex) {
        M |= 0x800000u;
        e = int(ex);
    } else {
        e = 1;
    }
}

// Value m * 2^(e - 150) as a float; m < 2^24, and m >= 2^23 unless e == 1.
SEQFP_HD float join(uint32_t m, int e)
{
    if (m < 0x800000u)
        return u2f(m); // subnormal (e == 1)
    return u2f((uint32_t(e) << 23) | (m & 0x7fffffu));
}

// m -> m + d[m & 1] (sum) or m -> m - d[m & 1] (walk).
struct Step {
    long long d0, d1;
};

SEQFP_HD Step identity()
{
    return Step{0, 0};
}

// `first` then `second`; the same rule serves additions and subtractions
// because only the parity of the intermediate state matters.
SEQFP_HD Step compose(const Step& first, const Step& second)
{
    Step r;
    r.d0 = first.d0 + ((first.d0 & 1) ? second.d1 : second.d0);
    r.d1 = first.d1 + (((first.d1 + 1) & 1) ? second.d1 : second.d0);
    return r;
}

// Integer part, and the two parity-dependent increments, of q in units of the
// epoch's ulp.  Requires eq <= e.  The formulas hold for both directions:
// round-to-nearest-even of m + a + f and of m - a - f pick the same extra unit.
SEQFP_HD void unit_step(uint32_t Mq, int eq, int e, uint32_t& a, uint32_t& c_even, uint32_t& c_odd)
{
    const int d = e - eq;
    if (d > 25) {
        a = c_even = c_odd = 0;
        return;
    }
    if (d == 0) {
        a = c_even = c_odd = Mq;
        return;
    }
    a = Mq >> d;
    const uint32_t rem = Mq & ((1u << d) - 1u);
    const uint32_t half = 1u << (d - 1);
    if (rem == half) {
        c_even = a + (a & 1u);
        c_odd = a + ((a & 1u) ^ 1u);
    } else {
        c_even = c_odd = a + (rem > half ? 1u : 0u);
    }
}

// ---- running sum -----------------------------------------------------------

// Map of one addend inside the epoch with exponent e.  An addend from a higher
// binade cannot be expressed; it is reported as a huge increment so that the
// event test below fires on it.
SEQFP_HD Step add_step(float q, int e)
{
    uint32_t Mq, a, ce, co;
    int eq;
    split(q, Mq, eq);
    if (eq > e)
        return Step{1ll << 40, 1ll << 40};
    unit_step(Mq, eq, e, a, ce, co);
    return Step{(long long)ce, (long long)co};
}

// True when adding q to m * ulp(e) may leave the binade, or q is not
// expressible in it: the caller then performs a real fp32 addition.
// Conservative (may fire early), never late.
SEQFP_HD bool add_event(long long m, float q, int e)
{
    uint32_t Mq, a, ce, co;
    int eq;
    split(q, Mq, eq);
    if (eq > e)
        return true;
    unit_step(Mq, eq, e, a, ce, co);
    return m + (long long)a + 1 >= (1ll << 24);
}

SEQFP_HD long long add_apply(long long m, float q, int e)
{
    const Step s = add_step(q, e);
    return m + ((m & 1) ? s.d1 : s.d0);
}

// ---- walk ------------------------------------------------------------------

SEQFP_HD Step sub_step(float q, int e)
{
    uint32_t Mq, a, ce, co;
    int eq;
    split(q, Mq, eq);
    if (eq > e)
        return Step{1ll << 40, 1ll << 40};
    unit_step(Mq, eq, e, a, ce, co);
    return Step{(long long)ce, (long long)co};
}

// r < q for r = m * ulp(e).
SEQFP_HD bool walk_stop(long long m, float q, int e)
{
    uint32_t Mq;
    int eq;
    split(q, Mq, eq);
    if (m <= 0)
        return Mq != 0 || m < 0;
    const int d = e - eq;
    if (d < 0)
        return true;
    if (d > 25)
        return false;
    return (m << d) < (long long)Mq;
}

// True when r - q may fall below the binade of r (its ulp would shrink).
// The lowest binade (e == 1, subnormals included) has no lower neighbour.
SEQFP_HD bool sub_event(long long m, float q, int e)
{
    if (e <= 1)
        return false;
    uint32_t Mq, a, ce, co;
    int eq;
    split(q, Mq, eq);
    if (eq > e)
        return true;
    unit_step(Mq, eq, e, a, ce, co);
    return m - (long long)a - 1 < (1ll << 23);
}

SEQFP_HD long long sub_apply(long long m, float q, int e)
{
    const Step s = sub_step(q, e);
    return m - ((m & 1) ? s.d1 : s.d0);
}

} // namespace seqfp
