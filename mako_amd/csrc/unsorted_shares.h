// Shares of a wide nucleus that need no sorting: who decides, and on what.
#pragma once

#include "sampler_common.h"
#include "seqfp.h"

namespace mako {

// Inside one binade of the running sum an addend that is not an exact tie is a constant increment (seqfp.h), and
// constant increments commute: the running fp32 sum after a whole share is the same in whatever order its weights are
// added, as long as the sum stays inside the binade, and so is the walk's r.  Deep in a list that is the rule: the
// sum (and r, until the walk is about to end) changes binade a dozen times in all, and a weight far below the running
// value is an exact tie with probability 2^-(difference of the exponents).  A share that the plan's estimates place
// (a) behind the head of the list that the tail keeps in LDS, (b) inside one binade of the running sum, (c) above the
// top-p cut and (d) where r stays inside one binade and cannot stop (or where the walk never gets) is not sorted: it
// is left as ONE record, its fp64 sum, the sum of its increments as the map of the running sum, the same for the walk
// (opaque_share()).  The few exact ties are kept apart: between two neighbouring ties (in value) the increments are
// summed, and the tie's own two-valued step is composed in at its place.  The estimates only decide who tries:
// tail_kernel applies such a record under the same exact tests as a group's map, and gives the row to the whole-row
// path if one fails (the share's order would be needed then and does not exist).
//
// Only batches with many top_k == 0 rows do this (the host decides and launches the kernels' instances for it): there
// sort_kernel is bound by the number of its workgroups, one per CU at a time, and a share that needs no sorting is summed
// by one wave of a collector workgroup that takes sixteen of them; on a small batch every worker has a CU to itself and the batch waits for the slowest anyway.

// A record that stands for a whole unsorted share (in GroupTable::pack): its maps are all there is.  Never among the
// first kHeadGroups groups of a list, and the list's entries at its positions are not written.
constexpr uint32_t kOpaque = 1u << 30;
constexpr int kOpaqueShift = 11;     // the share's largest weight lies at least this many binades below the sum and r
constexpr uint32_t kOpaqueTies = 16; // exact ties a share may hold (expected: entries * 2^-kOpaqueShift <= 3)
constexpr uint32_t kCollectors = 2;  // workgroups of sort_kernel that take a row's unsorted shares, one share per wave (work items kWorkers + c)
static_assert(kCollectors * (uint32_t)kWaves + 1u >= kWorkers, "a wave for every share but the last, which is never left unsorted");
constexpr double kOpaqueMu = 0.01;   // what the estimates of the mass above a share are trusted to ...
constexpr double kOpaqueMuCut = 0.03; // ... and of the mass below it

__device__ __forceinline__ int binade_of(double x) // exponent of x as a float (seqfp::split)
{
    uint32_t M;
    int e;
    seqfp::split((float)x, M, e);
    return e;
}

struct OpaqueGuess {
    bool cand;  // the share is left unsorted
    int e_tot;  // exponent of the running sum's binade at the share
    int e_walk; // of r's; 0: the walk is not expected to reach the share
};

// The binades for a share's maps.  `before` / `after`: the mass above the share and above the next one; r0: where the
// walk starts (0: none), all in the same units.  same_tot / same_walk: the margins leave no doubt about them.
__device__ __forceinline__ OpaqueGuess opaque_epochs(double before, double after, double r0, bool& same_tot, bool& same_walk)
{
    OpaqueGuess g{false, 0, 0};
    const int e_lo = binade_of(before * (1.0 - kOpaqueMu)), e_hi = binade_of(after * (1.0 + kOpaqueMu));
    same_tot = before > 0.0 && after > before && e_lo == e_hi;
    g.e_tot = binade_of(before);
    same_walk = true;
    if (r0 > 0.0) {
        const double rb_hi = r0 * (1.0 + kOpaqueMu) - before * (1.0 - kOpaqueMu), ra_lo = r0 * (1.0 - kOpaqueMu) - after * (1.0 + kOpaqueMu);
        if (ra_lo > 0.0) { // the walk passes the whole share
            g.e_walk = binade_of(r0 - after);
            same_walk = binade_of(rb_hi) == binade_of(ra_lo);
        } else if (!(rb_hi < 0.0)) {
            same_walk = false; // it may end in here
        }
    } else if (!(r0 <= 0.0)) {
        same_walk = false;
    }
    return g;
}

// The decision, from the plan's estimates alone (every number in the plan's units): cnt entries expected from position
// off of the list; mass_all: the whole row; key_hi: just above the largest bits(q) the share can hold; first_free: the
// first position an unsorted share may have.
// `rash` (always 0 in the library; a test build passes 1 << (row & 3), see MAKO_RASH_PLANS): which of the four rules is
// NOT applied (bit 0: the position, 1: the binades of sum and r and the ties, 2: the cut, 3: everything about the
// walk), so that shares are left unsorted that should not be and the tail has to give rows up.
__device__ __forceinline__ bool opaque_guess(bool allowed, uint32_t cnt, uint32_t off, uint32_t first_free, double before,
                                             double after, double mass_all, float top_p, double r0, uint32_t key_hi,
                                             uint32_t rash = 0u)
{
    bool same_tot, same_walk;
    const OpaqueGuess g = opaque_epochs(before, after, r0, same_tot, same_walk);
    const int e_q = binade_of((double)__uint_as_float(key_hi - 1u));
    bool ok = allowed && cnt > 0u && cnt <= 2u * kSegCap && after < mass_all;
    ok = ok && ((rash & 1u) || off >= first_free);
    ok = ok && ((rash & 2u) || (same_tot && g.e_tot >= e_q + kOpaqueShift));
    ok = ok && ((rash & 8u) || (same_walk && (g.e_walk == 0 || g.e_walk >= e_q + kOpaqueShift)));
    // the cut lies below the share: what the row holds below it is more than top-p leaves out
    ok = ok && ((rash & 4u) || (mass_all - after) * (1.0 - kOpaqueMuCut) > mass_all - (double)top_p * mass_all);
    return ok;
}

} // namespace mako
