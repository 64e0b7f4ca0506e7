"""Synthetic sampler workloads: the five benchmark configurations, regenerated from seeds.

Each generator returns a dict of host arrays:
  logits [B,V] f32, params PARAMS_DTYPE[B], u f32[B], and optionally
  hist int32[B,H] + hist_len u32[B], mask u32[B,ceil(V/32)], seeds u64[B].
`seeds` are per-row sampler seeds; `u` is what a std::mt19937_64 seeded with
seeds[r] yields through generate_canonical<float,24> only when the caller
fills it that way -- by default u is drawn from the workload's own stream.
"""
import hashlib

import numpy as np

from .api import PARAMS_DTYPE, make_params

V_DEEPSEEK = 129280
V_LARGE = 151552


def _rng(seed, *stream):
    return np.random.Generator(np.random.PCG64([seed, *stream]))


def _uniforms(rng, n):
    # top 24 bits of a 64-bit draw, scaled into [0, 1)
    return ((rng.integers(0, 2**64, n, dtype=np.uint64) >> np.uint64(40)).astype(np.float32) * np.float32(2.0**-24))


def _zipf_cdf(v, s=1.1):
    w = np.arange(1, v + 1, dtype=np.float64) ** (-s)
    c = np.cumsum(w)
    return c / c[-1]


def zipf_history(rng, cdf, rows, length):
    """Token histories drawn Zipf(s) over the vocabulary (rank k -> token k-1)."""
    r = rng.random((rows, length))
    return np.minimum(np.searchsorted(cdf, r), len(cdf) - 1).astype(np.int32)


def input_digest(w):
    h = hashlib.sha256()
    for k in sorted(w):
        if isinstance(w[k], np.ndarray):
            h.update(k.encode())
            h.update(np.ascontiguousarray(w[k]).tobytes())
    return h.hexdigest()[:16]


def config1(seed=101, rows=1, vocab=V_DEEPSEEK):
    """B=1: N(0,3^2) logits with 20 spikes of +10; T 0.7, top-k 40, top-p 0.95, no penalties."""
    rng = _rng(seed, 1)
    logits = (rng.standard_normal((rows, vocab)) * 3.0).astype(np.float32)
    for r in range(rows):
        logits[r, rng.choice(vocab, 20, replace=False)] += np.float32(10.0)
    return dict(name="config1", logits=logits, params=make_params(rows, 0.7, 40, 0.95), u=_uniforms(rng, rows),
                seeds=rng.integers(0, 2**63, rows, dtype=np.uint64))


def config2(seed=202, rows=1, vocab=V_LARGE, greedy=False, hist_len=512):
    """B=1: penalties 1.1 / 0.2 / 0.3 over a 512-token Zipf history; greedy, or T 1.0 + top-p 0.9."""
    rng = _rng(seed, 2)
    logits = (rng.standard_normal((rows, vocab)) * 3.0).astype(np.float32)
    hist = zipf_history(rng, _zipf_cdf(vocab), rows, hist_len)
    p = make_params(rows, 0.0 if greedy else 1.0, 0, 1.0 if greedy else 0.9, 0.0, 0.3, 0.2, 1.1)
    return dict(name="config2a" if greedy else "config2b", logits=logits, params=p, u=_uniforms(rng, rows), hist=hist,
                hist_len=np.full(rows, hist_len, np.uint32), seeds=rng.integers(0, 2**63, rows, dtype=np.uint64))


def config3(seed=303, rows=64, vocab=V_DEEPSEEK, hist_len=2048):
    """Decode batch: per-row T, top-k in {0,20,50,100}, top-p < 1, penalties over 2048-token Zipf histories."""
    rng = _rng(seed, 3)
    logits = (rng.standard_normal((rows, vocab)) * 3.0).astype(np.float32)
    for r in range(rows):
        k = int(rng.integers(1, 51))
        logits[r, rng.choice(vocab, k, replace=False)] += np.float32(10.0)
    p = make_params(rows)
    p["temperature"] = rng.uniform(0.3, 1.2, rows).astype(np.float32)
    p["top_k"] = rng.choice(np.array([0, 20, 50, 100], np.uint32), rows)
    p["top_p"] = np.minimum(rng.uniform(0.8, 1.0, rows).astype(np.float32), np.float32(1.0 - 2.0**-24))
    p["repetition_penalty"] = 1.1
    p["frequency_penalty"] = 0.2
    p["presence_penalty"] = 0.3
    hist = zipf_history(rng, _zipf_cdf(vocab), rows, hist_len)
    return dict(name="config3", logits=logits, params=p, u=_uniforms(rng, rows), hist=hist,
                hist_len=np.full(rows, hist_len, np.uint32), seeds=rng.integers(0, 2**63, rows, dtype=np.uint64))


def config4(seed=404, rows=256, vocab=V_LARGE):
    """Top-p 0.9 only: half the rows heavy-tailed Student-t(3)*4, half near-flat N(0, 0.1^2)."""
    rng = _rng(seed, 4)
    logits = np.empty((rows, vocab), np.float32)
    half = rows // 2
    logits[:half] = (rng.standard_t(3, (half, vocab)) * 4.0).astype(np.float32)
    logits[half:] = (rng.standard_normal((rows - half, vocab)) * 0.1).astype(np.float32)
    return dict(name="config4", logits=logits, params=make_params(rows, 1.0, 0, 0.9), u=_uniforms(rng, rows),
                seeds=rng.integers(0, 2**63, rows, dtype=np.uint64))


def config5(seed=505, rows=256, vocab=V_DEEPSEEK, density=0.01):
    """Verify-shaped batch (32 x 8 rows): per-row allowed-token bitmask, T 0.8, top-k 50, top-p 0.95."""
    rng = _rng(seed, 5, int(density * 1000))
    logits = (rng.standard_normal((rows, vocab)) * 3.0).astype(np.float32)
    words = (vocab + 31) // 32
    bits = rng.random((rows, words * 32)) < density
    bits[:, vocab:] = False
    for r in range(rows):
        if not bits[r].any():
            bits[r, int(rng.integers(0, vocab))] = True
    mask = np.packbits(bits.reshape(rows, words, 32), axis=2, bitorder="little").view(np.uint32).reshape(rows, words)
    return dict(name="config5_%g" % density, logits=logits, params=make_params(rows, 0.8, 50, 0.95),
                u=_uniforms(rng, rows), mask=np.ascontiguousarray(mask),
                seeds=rng.integers(0, 2**63, rows, dtype=np.uint64))


def bytes_per_row(w):
    """Algorithmic HBM bytes of one row: logits once, history tokens, mask words, params, u, token id."""
    v = w["logits"].shape[1]
    b = 4 * v + 28 + 4 + 4
    if "hist" in w:
        b += 4 * w["hist"].shape[1]
    if "mask" in w:
        b += 4 * ((v + 31) // 32)
    return b
