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

#include <math.h>
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

// ---- groups ----------------------------------------------------------------
//
// A long sorted list is cut into groups.  The map of a whole group under a GUESSED epoch (taken from an
// approximate fp64 prefix sum) can be built by any number of threads in parallel; a serial chain then walks
// the groups with the exact state and uses a group's map only if the guess was right and nothing inside the
// group can leave the binade (or, for the walk, stop).  A group that fails the test is replayed element by
// element.  Results never depend on the guess, only the speed does.

constexpr uint32_t kSat = 1u << 28; // "left the binade": larger than any state, small enough to add twice

// 32-bit form of Step with saturation; once saturated the parities are meaningless and the user must
// reject the map (d >= 2^24 can never pass the tests below).
struct Step32 {
    uint32_t d0, d1, cmax; // cmax: largest single increment seen
};

SEQFP_HD Step32 identity32()
{
    return Step32{0, 0, 0};
}

SEQFP_HD uint32_t sat_add(uint32_t a, uint32_t b)
{
    const uint32_t s = a + b;
    return s > kSat ? kSat : s;
}

SEQFP_HD Step32 compose32(const Step32& first, const Step32& second)
{
    Step32 r;
    r.d0 = sat_add(first.d0, (first.d0 & 1u) ? second.d1 : second.d0);
    r.d1 = sat_add(first.d1, ((first.d1 + 1u) & 1u) ? second.d1 : second.d0);
    r.cmax = first.cmax > second.cmax ? first.cmax : second.cmax;
    return r;
}

// Map of one element (for additions and subtractions alike) in the epoch with exponent e.
SEQFP_HD Step32 step32(float q, int e)
{
    uint32_t Mq, a, ce, co;
    int eq;
    split(q, Mq, eq);
    if (eq > e)
        return Step32{kSat, kSat, kSat};
    unit_step(Mq, eq, e, a, ce, co);
    return Step32{ce, co, ce > co ? ce : co};
}

// step32() in straight-line form (the same map for every weight q >= 0 and every exponent e >= 1): no branches for a
// GPU compiler to keep or to execute both sides of.  The host test compares the two.
SEQFP_HD Step32 step32_flat(float q, int e)
{
    const uint32_t b = f2u(q);
    const uint32_t ex = b >> 23; // (q is a weight: no sign bit)
    const uint32_t Mq = (b & 0x7fffffu) | (ex ? 0x800000u : 0u);
    const int d = e - int(ex ? ex : 1u);
    const uint32_t sh = uint32_t(d < 0 ? 0 : (d > 31 ? 31 : d));
    const uint32_t a = Mq >> sh;
    const uint32_t rem = Mq - (a << sh);
    const uint32_t half = (1u << sh) >> 1; // (0 when d == 0: nothing is rounded away, and rem is 0 too)
    const uint32_t up = rem > half ? 1u : 0u;
    const uint32_t tie = (rem == half && sh != 0u) ? 1u : 0u;
    uint32_t ce = a + (up | (tie & a)), co = a + (up | (tie & ~a));
    if (d > 25) // (the weight is below half a unit of the epoch's last place)
        ce = co = 0u;
    if (d < 0) // (a weight from a higher binade cannot be expressed)
        ce = co = kSat;
    return Step32{ce, co, ce > co ? ce : co};
}

// The same map taken from the adder itself: in the epoch with exponent e the states 2^23 (even) and 2^23 + 1 (odd) are
// the floats R0 and R1, and for a weight below 2^23 units R + q stays inside the binade, so (R + q) - R is, exactly, the
// increment that round-to-nearest-even gives a state of R's parity: two additions, two subtractions and two exact
// scalings instead of the integer arithmetic above.  A weight of 2^23 units or more gets the "unusable" mark (its
// map could never be applied to a state of a binade of 2^23 states; in the subnormal binade, whose states start at
// zero, that gives up maps step32_flat() would allow, which costs a replay and nothing else).  Compiled without
// contraction or reassociation, like every fp32 operation that stands for one of the reference's.
SEQFP_HD Step32 step32_fp(float q, int e)
{
    const float R0 = u2f(uint32_t(e) << 23), R1 = u2f((uint32_t(e) << 23) | 1u);
    const float t0 = (R0 + q) - R0, t1 = (R1 + q) - R1;
#if defined(__HIP_DEVICE_COMPILE__)
    uint32_t ce = (uint32_t)__builtin_ldexpf(t0, 150 - e), co = (uint32_t)__builtin_ldexpf(t1, 150 - e);
#else
    uint32_t ce = (uint32_t)ldexpf(t0, 150 - e), co = (uint32_t)ldexpf(t1, 150 - e);
#endif
    if (!(q < R0) || e > 253) // (in the last binade R + q may overflow: no maps there, running sums of weights never get near it)
        ce = co = kSat;
    return Step32{ce, co, ce > co ? ce : co};
}

// May a group's map g (built for exponent e) be applied to the running sum m * ulp(e)?  Sufficient: the state
// after the group, plus one more of its largest increments, still lies inside the binade.
SEQFP_HD bool group_add_ok(long long m, const Step32& g)
{
    const uint32_t d = (m & 1) ? g.d1 : g.d0;
    return d < (1u << 24) && m + (long long)d + (long long)g.cmax + 1 < (1ll << 24);
}

// Same for the walk state r = m * ulp(e), for a group of a DESCENDING list whose first (largest) weight is
// q_first: the state after the group must stay in the binade with room for one more decrement, and must
// still be at least q_first, so no element of the group can have stopped the walk.
SEQFP_HD bool group_sub_ok(long long m, int e, const Step32& g, float q_first)
{
    const uint32_t d = (m & 1) ? g.d1 : g.d0;
    if (d >= (1u << 24))
        return false;
    const long long m_end = m - (long long)d;
    if (e > 1 && m_end - (long long)g.cmax - 1 < (1ll << 23))
        return false;
    if (m_end <= 0)
        return false;
    return !walk_stop(m_end, q_first, e);
}

} // namespace seqfp
