"""Generates tests/golden/reference_vectors.json from the compiled reference sampler.

Run in the build container (needs /root/reference and `make -C oracle`):
    python tests/golden/make_golden.py
For every case the UNMODIFIED reference (oracle/_ref/libmako_ref.so: src/gen/sampler.cpp built with
g++ -O2 -ffp-contract=off against libstdc++ 11.4 / glibc 2.35) is given a seed; recorded are the token it
returns, the size of its final candidate list, a digest of that list (ids and weight bits, reference
order) and the fp32 total re-added in list order.  Inputs are regenerated from seeds by
mako_amd.workloads; `input_digest` guards against generator drift.  The vectors pin the oracle
(tests/test_oracle_cpu.py) and, through it, the HIP path.
"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from mako_amd import workloads  # noqa: E402
from oracle import pyoracle  # noqa: E402


def cases():
    """(name, workload, rows) -- small row subsets of every benchmark configuration plus tiny-vocab cases."""
    yield "config1", workloads.config1(rows=6), range(6)
    yield "config2a", workloads.config2(rows=3, greedy=True), range(3)
    yield "config2b", workloads.config2(rows=4, greedy=False), range(4)
    yield "config3", workloads.config3(rows=64), range(64)
    yield "config4", workloads.config4(rows=8), range(8)
    yield "config5_0.01", workloads.config5(rows=8, density=0.01), range(8)
    yield "config5_0.5", workloads.config5(rows=8, density=0.5), range(8)
    # top-k without top-p: the candidate order is the one libstdc++'s nth_element leaves
    w = workloads.config1(rows=4, seed=111)
    w["params"]["top_p"] = 1.0
    w["name"] = "topk_only"
    yield "topk_only", w, range(4)
    # tiny vocabulary with many ties
    rng = np.random.default_rng(4242)
    lg = (np.round(rng.standard_normal((16, 48)) * 2) / 2).astype(np.float32)
    p = workloads.make_params(16)
    p["temperature"] = rng.choice(np.array([0.5, 1.0, 1.5], np.float32), 16)
    p["top_k"] = rng.choice(np.array([0, 3, 10], np.uint32), 16)
    p["top_p"] = rng.choice(np.array([0.6, 0.9, 0.99], np.float32), 16)
    p["min_p"] = rng.choice(np.array([0.0, 0.1], np.float32), 16)
    yield "tiny_ties", dict(name="tiny_ties", logits=lg, params=p, u=np.zeros(16, np.float32),
                            seeds=rng.integers(0, 2**63, 16, dtype=np.uint64)), range(16)


def list_digest(idx, q):
    h = hashlib.sha256()
    h.update(np.ascontiguousarray(idx, np.int32).tobytes())
    h.update(np.ascontiguousarray(q, np.float32).tobytes())
    return h.hexdigest()[:16]


def main():
    ref = pyoracle.reference()
    if ref is None:
        raise SystemExit("oracle/_ref/libmako_ref.so missing: run `make -C oracle` with /root/reference mounted")
    out = dict(note="expected outputs of the unmodified reference sampler; see make_golden.py", cases=[])
    for name, w, rows in cases():
        v = w["logits"].shape[1]
        rec = dict(name=name, input_digest=workloads.input_digest(w), rows=[])
        for r in rows:
            p = pyoracle.params_from_record(w["params"][r])
            hist = w["hist"][r, : w["hist_len"][r]] if "hist" in w else None
            mask = w["mask"][r] if "mask" in w else None
            seed = int(w["seeds"][r])
            t, tr = ref.sample(w["logits"][r], p, seed, hist, mask, cap=v)
            total = np.float32(0)
            for q in tr["cand_q"]:
                total = np.float32(total + q)
            rec["rows"].append(dict(row=int(r), seed=seed, token=int(t), n_cand=int(tr["n_cand"]),
                                    list_digest=list_digest(tr["cand_idx"], tr["cand_q"]),
                                    total_bits=int(np.float32(total).view(np.uint32))))
        out["cases"].append(rec)
    # worst-case inputs of std::nth_element (they drive libstdc++'s introselect into its heap-select
    # branch), with a digest of the arrangement std::nth_element leaves
    out["nth_killers"] = []
    for n, nth in ((3000, 1500), (5000, 4000)):
        q, _ = ref.make_nth_killer(n, nth)
        rq, ri = ref.nth_element(q, np.arange(n, dtype=np.int32), nth)
        out["nth_killers"].append(dict(n=n, nth=nth, q=[int(v) for v in q], result_digest=list_digest(ri, rq)))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path, sum(len(c["rows"]) for c in out["cases"]), "rows")


if __name__ == "__main__":
    main()
