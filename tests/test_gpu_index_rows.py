"""GPU parity of rows that are cut neither to a top-k nor to a nucleus (temperature only: top_k = 0, top_p = 1), whose
candidates the reference adds up and walks in token order (src/gen/sampler.cpp:79-83, :64-72).  With the caller's host
copy of the parameters such rows take kernels of their own (mako_amd/csrc/index_rows.h: weights in place, group records,
exact fp32 total and walk by group maps over the unsorted list); tokens, candidate counts, candidate lists and fp32
totals must be the oracle's bit for bit, with gaps in the list (masks, min_p, underflow), at both ends of u, beside rows
of every other kind, and the results must equal those of the call without the host copy (the whole-row path)."""
import numpy as np
import pytest

from mako_amd import api, workloads
from parity import assert_parity, gpu_rows, oracle_rows

pytestmark = pytest.mark.gpu

PATH_INDEXED, PATH_GENERAL = api.PATH_INDEXED, api.PATH_GENERAL


def _say(msg):
    print(msg, flush=True)


def _plain_batch(rows, vocab, seed, sigmas=(3.0,), temps=(0.7,), us=None, spikes=True):
    rng = np.random.Generator(np.random.PCG64([seed, 91]))
    logits = np.empty((rows, vocab), np.float32)
    p = workloads.make_params(rows, 1.0, 0, 1.0)
    for r in range(rows):
        row = (rng.standard_normal(vocab) * sigmas[r % len(sigmas)]).astype(np.float32)
        if spikes:
            row[rng.integers(0, vocab, 20)] += np.float32(10.0)
        logits[r] = row
        p["temperature"][r] = temps[(r // len(sigmas)) % len(temps)]
    u = workloads._uniforms(rng, rows) if us is None else np.asarray([us[r % len(us)] for r in range(rows)], np.float32)
    return dict(name="temperature only %d" % seed, logits=logits, params=p, u=u)


def _paths(g):
    return np.bincount(g["path"], minlength=10).tolist()


def test_temperature_only_rows(gpu_ctx):
    w = _plain_batch(64, 129280, 1, sigmas=(3.0, 1.0, 0.1, 6.0), temps=(0.7, 1.0, 1.5))
    g = assert_parity(gpu_ctx, w, cap=300, hinted=True)
    _say("temperature only paths: %s" % _paths(g))
    assert (g["path"] == PATH_INDEXED).all()


def test_walk_ends_everywhere(gpu_ctx):
    us = [0.0, 2.0**-24, 1e-6, 1e-3, 0.1, 0.25, 0.4999999, 0.5, 0.5000001, 0.75, 0.9, 0.99, 0.999, 0.99999,
          1.0 - 2.0**-23, 1.0 - 2.0**-24]
    w = _plain_batch(64, 151552, 2, sigmas=(3.0, 0.05), temps=(1.0, 0.8), us=us)
    g = assert_parity(gpu_ctx, w, cap=64, hinted=True)
    _say("walk ends paths: %s" % _paths(g))
    assert (g["path"] == PATH_INDEXED).all()


def test_gaps_in_the_list(gpu_ctx):
    """Masks, a min_p floor and a cold temperature (weights that underflow to zero) leave logits that are no
    candidates: with no candidate list asked for the rows stay on the new path, with one they take the whole-row
    path; either way the oracle's results."""
    rng = np.random.Generator(np.random.PCG64([3, 92]))
    rows, vocab = 48, 129280
    w = _plain_batch(rows, vocab, 3, sigmas=(3.0, 8.0), temps=(0.3, 1.0, 0.1))
    w["params"]["min_p"][::3] = np.float32(1e-3)
    words = (vocab + 31) // 32
    bits = rng.random((rows, words * 32)) < 0.6
    bits[:, vocab:] = False
    bits[1::4] = True
    bits[:, vocab:] = False
    w["mask"] = np.ascontiguousarray(np.packbits(bits.reshape(rows, words, 32), axis=2, bitorder="little").view(np.uint32).reshape(rows, words))
    g0 = assert_parity(gpu_ctx, w, cap=0, hinted=True)
    _say("gaps, no candidate lists, paths: %s" % _paths(g0))
    assert (g0["path"] == PATH_INDEXED).sum() >= rows - 2
    g1 = assert_parity(gpu_ctx, w, cap=500, hinted=True)
    _say("gaps, candidate lists, paths: %s" % _paths(g1))
    assert np.array_equal(g0["tokens"], g1["tokens"])


def test_penalties_and_histories(gpu_ctx):
    rng = np.random.Generator(np.random.PCG64([4, 93]))
    rows, vocab, hl = 40, 129280, 2048
    w = _plain_batch(rows, vocab, 4, sigmas=(3.0,), temps=(0.9, 1.2))
    w["params"]["repetition_penalty"] = 1.1
    w["params"]["frequency_penalty"] = 0.2
    w["params"]["presence_penalty"] = 0.3
    w["hist"] = workloads.zipf_history(rng, workloads._zipf_cdf(vocab), rows, hl)
    w["hist_len"] = rng.integers(0, hl + 1, rows).astype(np.uint32)
    g = assert_parity(gpu_ctx, w, cap=128, hinted=True)
    _say("penalties paths: %s" % _paths(g))
    assert (g["path"] == PATH_INDEXED).all()


def test_beside_rows_of_every_kind(gpu_ctx):
    """config 3's batch with every fourth row made a temperature-only row."""
    w = workloads.config3()
    w["params"]["top_p"][::4] = np.float32(1.0)
    w["params"]["top_k"][::4] = 0
    g = assert_parity(gpu_ctx, w, cap=256, hinted=True)
    _say("mixed batch paths: %s" % _paths(g))
    # (cold rows have weights that underflow: with candidate lists asked for they take the whole-row path)
    assert np.isin(g["path"][::4], [PATH_INDEXED, PATH_GENERAL]).all() and (g["path"][::4] == PATH_INDEXED).sum() >= 4
    assert not (np.delete(g["path"], np.s_[::4]) == PATH_INDEXED).any()
    h = gpu_rows(gpu_ctx, w, cap=256)
    assert (h["path"][::4] == PATH_GENERAL).all()
    assert np.array_equal(h["tokens"], g["tokens"]) and np.array_equal(h["total"].view(np.uint32), g["total"].view(np.uint32))
    assert np.array_equal(h["n_cand"], g["n_cand"])


@pytest.mark.parametrize("vocab", [4, 252, 260, 4096, 4100, 20000, 65536])
def test_small_and_odd_vocabularies(vocab):
    ctx = api.SamplerContext(max_rows=24, max_vocab=vocab, max_hist=0)
    try:
        w = _plain_batch(24, vocab, 100 + vocab, sigmas=(2.0, 0.2), temps=(0.6, 1.0), spikes=False)
        g = assert_parity(ctx, w, cap=64, hinted=True)
    finally:
        ctx.close()
    _say("V = %d paths: %s" % (vocab, _paths(g)))
    assert (g["path"] == PATH_INDEXED).all()


@pytest.mark.parametrize("vocab", [4099, 50257])
def test_vocabularies_that_are_no_multiple_of_four(vocab):
    """The logits are then loaded one at a time (rows cannot be 16-byte aligned): the same kernels, the same results."""
    ctx = api.SamplerContext(max_rows=12, max_vocab=vocab, max_hist=0)
    try:
        w = _plain_batch(12, vocab, 7 + vocab, sigmas=(2.0, 0.5), temps=(0.7, 1.0))
        w["params"]["min_p"][::4] = np.float32(1e-3)
        g = assert_parity(ctx, w, cap=0, hinted=True)
        assert (g["path"] == PATH_INDEXED).all()
        assert_parity(ctx, w, cap=64, hinted=True)
    finally:
        ctx.close()


def test_rows_the_kernels_do_not_serve():
    """More logits than a row's group records cover (262 144): the rows take the whole-row path as before."""
    vocab = 262148
    ctx = api.SamplerContext(max_rows=2, max_vocab=vocab, max_hist=0)
    try:
        w = _plain_batch(2, vocab, 7, spikes=False)
        g = assert_parity(ctx, w, cap=16, hinted=True)
    finally:
        ctx.close()
    assert (g["path"] == PATH_GENERAL).all()


def test_no_candidate_survives(gpu_ctx):
    """Every logit masked out but for NaNs' sake nothing survives: the fallback token (sampler.cpp:37-38)."""
    w = _plain_batch(8, 129280, 8)
    w["logits"][0:4] = -np.inf
    w["logits"][4:6] = np.nan
    g = assert_parity(gpu_ctx, w, cap=16, hinted=True)
    _say("empty rows paths: %s" % _paths(g))


def test_other_rows_of_the_whole_row_path_get_their_weights_there_too(gpu_ctx):
    """Rows cut to a top-k without a top-p (the order nth_element leaves) and to a top-k beyond the candidate lists:
    with the host copy of the parameters their weights come from the same kernel as the rows' in token order, a
    workgroup per 16 384 logits, and the whole-row path goes on from there."""
    rng = np.random.Generator(np.random.PCG64([9, 94]))
    rows, vocab, hl = 36, 129280, 512
    w = _plain_batch(rows, vocab, 9, sigmas=(3.0, 1.0), temps=(0.7, 1.1))
    p = w["params"]
    p["top_k"][0::3], p["top_p"][0::3] = 40, 1.0
    p["top_k"][1::3], p["top_p"][1::3] = 700, 0.9
    p["top_k"][4], p["top_p"][4] = 5000, 1.0
    p["min_p"][::5] = np.float32(1e-4)
    p["repetition_penalty"] = 1.1
    p["frequency_penalty"] = 0.2
    p["presence_penalty"] = 0.3
    w["hist"] = workloads.zipf_history(rng, workloads._zipf_cdf(vocab), rows, hl)
    w["hist_len"] = rng.integers(0, hl + 1, rows).astype(np.uint32)
    words = (vocab + 31) // 32
    bits = rng.random((rows, words * 32)) < 0.8
    bits[::2] = True
    bits[:, vocab:] = False
    w["mask"] = np.ascontiguousarray(np.packbits(bits.reshape(rows, words, 32), axis=2, bitorder="little").view(np.uint32).reshape(rows, words))
    g = assert_parity(gpu_ctx, w, cap=128, hinted=True)
    _say("whole-row rows with the host copy, paths: %s" % _paths(g))
    assert (g["path"][0::3] == PATH_GENERAL).all() and (g["path"][1::3] == PATH_GENERAL).all()
    h = gpu_rows(gpu_ctx, w, cap=128)
    assert np.array_equal(h["tokens"], g["tokens"]) and np.array_equal(h["total"].view(np.uint32), g["total"].view(np.uint32))
    assert np.array_equal(h["cand_idx"], g["cand_idx"])


@pytest.mark.parametrize("vocab", [4099, 40000, 129280])
def test_wide_top_k_before_a_top_p_with_many_equal_weights(gpu_ctx, vocab):
    """A top-k beyond the candidate lists followed by a top-p: the library partitions the candidates as nth_element
    does and sorts the survivors only.  With logits on a coarse grid many candidates share a weight, at the top-k's edge
    and among the survivors: which of them survive, and their order (equal weights by token id), must be the
    reference's, on rows with and without gaps in the list, with and without the host copy of the parameters, also
    where the rows' length is no multiple of four (the weights kernel then leaves no list of its own)."""
    rng = np.random.Generator(np.random.PCG64([vocab, 97]))
    rows = 24
    logits = (np.round(rng.standard_normal((rows, vocab)) * 3.0 * 2.0) / 2.0).astype(np.float32)
    logits[1::4] = (np.round(rng.standard_normal((rows // 4, vocab)) * 0.5 * 8.0) / 8.0).astype(np.float32)
    logits[2::4, ::7] = -np.inf
    p = workloads.make_params(rows, 1.0, 0, 1.0)
    p["temperature"] = rng.choice(np.array([0.5, 1.0, 2.5], np.float32), rows)
    p["top_k"] = rng.choice(np.array([129, 200, 1000, 5000, 20000], np.uint32), rows)
    p["top_p"] = rng.choice(np.array([0.5, 0.9, 0.95, 0.999], np.float32), rows)
    p["top_p"][5::8] = 1.0  # (and a few rows whose survivors keep the partitions' order)
    p["min_p"][::6] = np.float32(0.01)
    u = workloads._uniforms(rng, rows)
    w = dict(name="wide top-k, equal weights, V=%d" % vocab, logits=logits, params=p, u=u)
    for hinted in (False, True):
        _say("wide top-k before a top-p, V=%d hinted=%s" % (vocab, hinted))
        g = assert_parity(gpu_ctx, w, cap=512, hinted=hinted)
        assert (g["path"] == PATH_GENERAL).all()


def test_verification_of_rows_in_token_order(gpu_ctx):
    """Sampler::verify (src/gen/sampler.cpp:86-107) on temperature-only rows: the draft's weight read off the list,
    the total by the chain of group maps, and for a rejected draft the walk over the list without it.  Drafts that
    are likely and unlikely tokens, no candidates (masked), the row's last candidate, and beyond the vocabulary's
    candidates; both uniforms from 0 to 1 - 2^-24."""
    rng = np.random.Generator(np.random.PCG64([10, 95]))
    rows, vocab = 64, 129280
    w = _plain_batch(rows, vocab, 10, sigmas=(3.0, 0.3), temps=(0.7, 1.0, 0.4))
    words = (vocab + 31) // 32
    bits = np.ones((rows, words * 32), bool)
    bits[::4] = rng.random((rows // 4, words * 32)) < 0.7
    bits[:, vocab:] = False
    bits[5, vocab - 3000:] = False  # (the row's last candidates masked out: the list ends early)
    w["mask"] = np.ascontiguousarray(np.packbits(bits.reshape(rows, words, 32), axis=2, bitorder="little").view(np.uint32).reshape(rows, words))
    masked = np.where(bits[:, :vocab], w["logits"], -np.inf)
    draft = rng.integers(0, vocab, rows).astype(np.int32)
    draft[0::3] = masked[0::3].argmax(axis=1)           # the most likely token: mostly accepted
    draft[7] = vocab - 1                                 # the row's last candidate
    draft[5] = vocab - 10                                # masked out: no candidate
    draft[9] = np.nonzero(bits[9, :vocab])[0][-1]        # the last candidate of a masked row
    u2 = workloads._uniforms(rng, rows)
    w["u"][11], u2[11] = np.float32(1.0 - 2.0**-24), np.float32(1.0 - 2.0**-24)  # rejected, and the redraw runs to the end
    w["u"][7], u2[7] = np.float32(1.0 - 2.0**-24), np.float32(1.0 - 2.0**-24)
    w["u"][9], u2[9] = np.float32(1.0 - 2.0**-24), np.float32(1.0 - 2.0**-24)
    w["u"][13], u2[13] = np.float32(0.0), np.float32(0.0)
    for cap in (0, 64):
        g = gpu_rows(gpu_ctx, w, cap=cap, draft=draft, u2=u2, hinted=True)
        ref = oracle_rows(w, draft=draft, u2=u2)
        bad = [(r, int(g["tokens"][r]), t, bool(g["accepted"][r]), bool(tr["accepted"])) for r, (t, tr) in enumerate(ref)
               if g["tokens"][r] != t or bool(g["accepted"][r]) != bool(tr["accepted"])]
        assert not bad, bad[:8]
        _say("verification (cap %d): %d accepted, paths %s" % (cap, int(g["accepted"].sum()), _paths(g)))
        assert (g["path"] == PATH_INDEXED).sum() >= rows // 2
        h = gpu_rows(gpu_ctx, w, cap=cap, draft=draft, u2=u2)
        assert np.array_equal(h["tokens"], g["tokens"]) and np.array_equal(h["accepted"], g["accepted"])
        assert np.array_equal(h["total"].view(np.uint32), g["total"].view(np.uint32))


def test_forced_and_close_tokens_beside_rows_in_token_order(gpu_ctx):
    """The decode loop's hooks (force_token, close_token) on a batch of temperature-only rows: a forced row is left to
    the launch that writes forced tokens, the others take the kernels of their own; the results are those of the call
    without the host copy of the parameters."""
    rng = np.random.Generator(np.random.PCG64([11, 96]))
    rows, vocab = 48, 129280
    w = _plain_batch(rows, vocab, 11, sigmas=(3.0, 1.0), temps=(0.8, 1.1))
    force = np.full(rows, -1, np.int32)
    force[::5] = rng.integers(0, vocab, len(force[::5]))
    close = np.full(rows, -1, np.int32)
    order = np.argsort(-w["logits"], axis=1, kind="stable")
    close[1::3] = order[1::3, 1]   # the second most likely token: taken (fewer than three logits above it)
    close[2::6] = order[2::6, 40]  # an unlikely one: not taken
    kw = dict(force_token=force, close_token=close, close_max_above=3, cand_cap=32)
    g = api.sample(gpu_ctx, w["logits"], w["params"], w["u"], params_host=True, **kw)
    h = api.sample(gpu_ctx, w["logits"], w["params"], w["u"], **kw)
    _say("forced beside rows in token order, paths: %s" % _paths(g))
    for key in ("tokens", "forced", "above", "n_cand"):
        assert np.array_equal(g[key], h[key]), key
    assert np.array_equal(g["total"].view(np.uint32), h["total"].view(np.uint32))
    forced = g["forced"] != api.FORCED_NONE
    assert forced.sum() >= 10 and (g["path"][forced] == api.PATH_FORCED).all() and (g["path"][~forced] == PATH_INDEXED).all()
    assert (g["tokens"][::5] == force[::5]).all()
    ref = oracle_rows(w)
    assert all(g["tokens"][r] == ref[r][0] for r in range(rows) if not forced[r])


def test_beside_a_large_batch_of_nucleus_rows():
    """config 4's 256 rows (the large batches' instances of the kernels, unsorted shares included) with every eighth
    row made a temperature-only row."""
    w = workloads.config4()
    rows, vocab = w["logits"].shape
    w["params"]["top_p"][::8] = np.float32(1.0)
    ctx = api.SamplerContext(max_rows=rows, max_vocab=vocab, max_hist=0)
    try:
        g = assert_parity(ctx, w, cap=0, hinted=True)
    finally:
        ctx.close()
    _say("large mixed batch paths: %s" % _paths(g))
    assert (g["path"][::8] == PATH_INDEXED).all() and (g["path"] == api.PATH_SUMMED).sum() >= 80


@pytest.mark.parametrize("hist_len", [5000, 10000])
def test_long_histories(hist_len):
    """Histories beyond two (eight) entries per thread take the weights kernel's other instances."""
    rng = np.random.Generator(np.random.PCG64([12, hist_len]))
    rows, vocab = 12, 65536
    w = _plain_batch(rows, vocab, 12, sigmas=(2.0,), temps=(0.8, 1.1))
    w["params"]["repetition_penalty"] = 1.2
    w["params"]["frequency_penalty"] = 0.1
    w["params"]["presence_penalty"] = 0.4
    w["hist"] = rng.integers(0, vocab, (rows, hist_len)).astype(np.int32)
    w["hist_len"] = rng.integers(hist_len // 2, hist_len + 1, rows).astype(np.uint32)
    ctx = api.SamplerContext(max_rows=rows, max_vocab=vocab, max_hist=hist_len)
    try:
        g = assert_parity(ctx, w, cap=32, hinted=True)
    finally:
        ctx.close()
    assert (g["path"] == PATH_INDEXED).all()


def test_more_rows_than_a_workgroup_has_threads():
    ctx = api.SamplerContext(max_rows=1100, max_vocab=320, max_hist=0)
    try:
        w = _plain_batch(1100, 320, 13, sigmas=(2.0, 0.3), temps=(0.7, 1.3), spikes=False)
        w["params"]["top_p"][::3] = np.float32(0.9)
        w["params"]["top_k"][1::5] = 7
        g = assert_parity(ctx, w, cap=8, hinted=True)
    finally:
        ctx.close()
    assert (g["path"] == PATH_INDEXED).sum() >= 400
