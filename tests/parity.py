"""Runs a workload through the HIP path (C ABI) and through the CPU oracle and compares them bit for bit."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np

from mako_amd import api, workloads
from oracle import pyoracle


def oracle_rows(w, rows=None, cap=0, order_mode=0, draft=None, u2=None):
    o = pyoracle.oracle()
    b = w["logits"].shape[0]
    rows = range(b) if rows is None else rows

    def one(r):
        p = pyoracle.params_from_record(w["params"][r])
        hist = w["hist"][r, : w["hist_len"][r]] if "hist" in w else None
        mask = w["mask"][r] if "mask" in w else None
        if draft is not None:
            t, acc = o.verify(w["logits"][r], p, int(draft[r]), float(w["u"][r]), float(u2[r]), hist, mask, order_mode)
            return t, dict(accepted=acc)
        return o.sample(w["logits"][r], p, float(w["u"][r]), hist, mask, order_mode, cap)

    with ThreadPoolExecutor(8) as ex:
        return list(ex.map(one, rows))


def gpu_rows(ctx, w, cap=0, draft=None, u2=None, hist_counts=None, hinted=False):
    """(hinted: the call also gets the host copy of the parameters, from which the library learns the rows' kinds)"""
    return api.sample(ctx, w["logits"], w["params"], w["u"], mask=w.get("mask"), hist=w.get("hist"),
                      hist_len=w.get("hist_len"), hist_counts=hist_counts, draft=draft, u2=u2, cand_cap=cap,
                      params_host=hinted)


def assert_parity(ctx, w, cap=256, rel_tol=1e-5, hinted=False):
    """Token ids, candidate counts, candidate id lists and weights must match the oracle exactly;
    probabilities q/total within rel_tol (they are in fact bit-identical)."""
    g = gpu_rows(ctx, w, cap=cap, hinted=hinted)
    ref = oracle_rows(w, cap=cap)
    bad = []
    for r, (t, tr) in enumerate(ref):
        greedy = w["params"][r]["temperature"] <= 0
        if g["tokens"][r] != t:
            bad.append((r, "token", int(g["tokens"][r]), t))
            continue
        if greedy:
            continue
        if g["n_cand"][r] != tr["n_cand"]:
            bad.append((r, "n_cand", int(g["n_cand"][r]), tr["n_cand"]))
            continue
        n = min(cap, tr["n_cand"])
        if n and not np.array_equal(g["cand_idx"][r, :n], tr["cand_idx"][:n]):
            bad.append((r, "cand_idx"))
            continue
        if n and not np.array_equal(g["cand_q"][r, :n].view(np.uint32), tr["cand_q"][:n].view(np.uint32)):
            bad.append((r, "cand_q"))
            continue
        if np.float32(g["total"][r]).view(np.uint32) != np.float32(tr["total"]).view(np.uint32):
            bad.append((r, "total", float(g["total"][r]), float(tr["total"])))
            continue
        pg, po = g["q"][r] / g["total"][r], tr["q_chosen"] / tr["total"]
        if not abs(pg - po) <= rel_tol * abs(po):
            bad.append((r, "prob", float(pg), float(po)))
    assert not bad, "%s: %d rows differ from the oracle: %s" % (w.get("name", "?"), len(bad), bad[:8])
    return g


def nucleus_batch(rows, vocab, seed, sigmas, temps, top_ps, us=None, name="unsorted"):
    """top_k = 0 rows: row r is N(0, sigma^2) logits with sigma, temperature and top_p taken in turn from the lists."""
    rng = np.random.Generator(np.random.PCG64([seed, 77]))
    logits = np.empty((rows, vocab), np.float32)
    p = workloads.make_params(rows, 1.0, 0, 0.9)
    for r in range(rows):
        logits[r] = (rng.standard_normal(vocab) * sigmas[r % len(sigmas)]).astype(np.float32)
        p["temperature"][r] = temps[(r // len(sigmas)) % len(temps)]
        p["top_p"][r] = top_ps[(r // (len(sigmas) * len(temps))) % len(top_ps)]
    u = workloads._uniforms(rng, rows) if us is None else np.asarray([us[r % len(us)] for r in range(rows)], np.float32)
    return dict(name=name, logits=logits, params=p, u=u)


def random_large_batch(seed):
    """A batch of 65-256 rows of every kind a top_k = 0 row comes in (wide and narrow, on grids of few distinct values,
    offset by hundreds, spiked, partly at -inf), a few top-k rows among them, with or without penalties, histories and
    masks; the number of candidates the caller wants written out varies too.  Returns (workload, cand_cap)."""
    rng = np.random.default_rng(seed)
    v = int(rng.choice([4099, 20000, 40000, 65537, 129280, 151552]))
    b = int(rng.choice([65, 100, 130, 200, 256])) if v < 100000 else int(rng.choice([65, 72, 96]))
    logits = np.empty((b, v), np.float32)
    kinds = rng.integers(0, 7, b)
    for r in range(b):
        kind = kinds[r]
        row = (rng.standard_normal(v) * [3.0, 3.0, 0.1, 0.02, 1.0, 6.0, 0.3][kind]).astype(np.float32)
        if kind == 1:
            row = (np.round(row * 4) / 4).astype(np.float32)
        if kind == 4:
            row += np.float32(rng.choice([0.0, 50.0, -50.0, 1000.0]))
        if kind == 5:
            row[rng.integers(0, v, rng.integers(1, 40))] += np.float32(rng.uniform(3, 15))
        logits[r] = row
    if rng.integers(0, 4) == 0:
        logits[:, rng.integers(0, v, max(1, v // 50))] = -np.inf
    p = workloads.make_params(b)
    p["temperature"] = rng.choice(np.array([0.3, 0.5, 0.8, 1.0, 1.3, 2.0, 5.0], np.float32), b)
    p["top_k"] = rng.choice(np.array([0, 0, 0, 0, 0, 0, 40], np.uint32), b)
    p["top_p"] = rng.choice(np.array([0.5, 0.8, 0.9, 0.95, 0.99, 0.999, 0.99999, 0.3], np.float32), b)
    p["min_p"] = rng.choice(np.array([0.0, 0.0, 0.0, 0.0, 1e-4, 0.02], np.float32), b)
    if rng.integers(0, 2):
        p["repetition_penalty"] = np.float32(1.1)
        p["frequency_penalty"] = np.float32(0.2)
        p["presence_penalty"] = np.float32(0.3)
    u = rng.random(b).astype(np.float32)
    u[rng.integers(0, b, 4)] = np.array([0.0, 1.0 - 2.0**-24, 0.5, 0.999999], np.float32)
    w = dict(name="random large batch %d" % seed, logits=logits, params=p, u=u)
    if rng.integers(0, 2):
        hl = int(rng.choice([5, 300, 2048]))
        w["hist"] = rng.integers(0, v, (b, hl)).astype(np.int32)
        w["hist_len"] = rng.integers(0, hl + 1, b).astype(np.uint32)
    if rng.integers(0, 4) == 0:
        w["mask"] = rng.integers(0, 2**32, (b, (v + 31) // 32), dtype=np.uint64).astype(np.uint32)
    return w, int(rng.choice([1, 64, 128, 3000, 12000]))
