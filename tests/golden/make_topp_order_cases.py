"""Finds top-p rows on which the ORDER of the fp64 additions decides the nucleus, and writes them to
tests/golden/topp_order_cases.json.

The reference adds the candidates' weights one after the other in fp64 (src/gen/sampler.cpp:46-48: the total, in
index order; :55-56: the sorted prefix).  A tree-shaped or exact sum of the same weights differs from that by a few
units in the last place, and for a few of the 2^23 float32 values of top_p in [0.5, 1) the product top_p * total then
falls on the other side of one of the sorted prefix sums: the nucleus has one entry more or fewer.  The rows are
built so that the difference is large (make_row()).  For each seeded row this script takes the weights q from the CPU oracle (a top_p = 1 call returns every candidate's q, the glibc
expf restated), forms the reference's sequential total and the correctly rounded exact total, and scans every float32
top_p for which the two give different cuts.  Only the seeds and the top_p bit patterns are kept: the test rebuilds
the rows.  The CPU oracle itself adds sequentially, like the reference (pinned against the compiled reference).

  python tests/golden/make_topp_order_cases.py        (about a minute on one core)
"""
import json
import math
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import pyoracle  # noqa: E402

V = 129280
N_MEDIUM = 20000


def make_row(seed, tiny_level):
    """One dominant logit, a plateau of N_MEDIUM medium ones holding a third of the mass (the nucleus ends inside it,
    in steps of 2.5e-5 of the total), and 109 279 tiny ones whose weights are `tiny_level` (+- a little) units in the
    last place of the running fp64 total, which stands near 1.5 when the reference's index-order loop reaches them:
    every one of those additions rounds the same way (up for 0.75, down to nothing for 0.3), so the sequential total
    drifts tens of thousands of units in the last place away from the exact sum."""
    rng = np.random.default_rng(seed)
    logits = np.empty(V, np.float32)
    logits[0] = 0.0
    logits[1:1 + N_MEDIUM] = np.log(0.5 / N_MEDIUM) + rng.normal(0.0, 0.05, N_MEDIUM)
    lo, hi = np.log((tiny_level - 0.1) * 2.0**-52), np.log((tiny_level + 0.1) * 2.0**-52)
    logits[1 + N_MEDIUM:] = rng.uniform(lo, hi, V - 1 - N_MEDIUM)
    return logits, np.float32(1.0)


def weights(orc, logits, temperature):
    p = pyoracle.make_params(temperature=float(temperature), top_k=0, top_p=1.0)
    _, tr = orc.sample(logits, p, 0.5, cap=V)
    n = tr["n_cand"]
    return tr["cand_idx"][:n].copy(), tr["cand_q"][:n].copy()


def main():
    orc = pyoracle.oracle()
    cases = []
    for seed, tiny_level in [(s, 0.75 if s % 2 else 0.3) for s in range(11, 27)]:
        logits, t = make_row(seed, tiny_level)
        idx, q = weights(orc, logits, t)
        q64 = q.astype(np.float64)
        total_seq = float(np.cumsum(q64)[-1])          # one addition after the other, index order
        total_exact = math.fsum(q64.tolist())          # correctly rounded exact sum
        order = np.lexsort((idx, -q64))                # (q desc, idx asc)
        cum = np.cumsum(q64[order])                    # the reference's running sum over the sorted prefix
        bits = np.arange(0x3F000000, 0x3F800000, dtype=np.uint32)  # every float32 in [0.5, 1)
        top_p = bits.view(np.float32).astype(np.float64)
        n_seq = np.searchsorted(cum, top_p * total_seq, side="left") + 1    # first n with cum[n-1] >= want
        n_exact = np.searchsorted(cum, top_p * total_exact, side="left") + 1
        differ = np.nonzero(n_seq != n_exact)[0]
        print("seed %d tiny level %.2f: %d candidates, sequential - exact = %+d ulp, %d of %d top_p values cut differently"
              % (seed, tiny_level, len(q), round((total_seq - total_exact) / math.ulp(total_exact)), len(differ),
                 len(bits)), flush=True)
        # a few per row, spread over the range
        for j in differ[:: max(1, len(differ) // 4)][:4]:
            cases.append(dict(seed=seed, tiny_level=tiny_level, top_p_bits=int(bits[j]),
                              n_reference=int(min(n_seq[j], len(q))), n_exact_total=int(min(n_exact[j], len(q)))))
    with open(os.path.join(HERE, "topp_order_cases.json"), "w") as f:
        json.dump(dict(vocab=V, logits="make_row(seed, tiny_level) of tests/golden/make_topp_order_cases.py", cases=cases), f,
                  indent=1)
        f.write("\n")
    print(len(cases), "cases written")


if __name__ == "__main__":
    main()
