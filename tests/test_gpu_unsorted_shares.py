"""GPU parity of large batches of top_k = 0 rows, where the shares of a row's sorted list whose order cannot matter
to the fp32 total and walk are summed instead of sorted (mako_amd/csrc/unsorted_shares.h): tokens, nucleus sizes,
candidate lists and the fp32 totals against the CPU oracle, bit for bit, on rows chosen so that the walk ends before,
inside and behind such shares, that exact ties occur, that the plan's guesses fail, and that the staged head and the
candidates written out reach into what would otherwise be left unsorted."""
import numpy as np
import pytest

from mako_amd import api, workloads
from parity import assert_parity, gpu_rows, nucleus_batch as _batch, oracle_rows, random_large_batch

pytestmark = pytest.mark.gpu

PATH_SUMMED = api.PATH_SUMMED


def _say(msg):
    print(msg, flush=True)


def _paths(g):
    return np.bincount(g["path"], minlength=9).tolist()


def test_config4_summed_rows(gpu_ctx):
    """The benchmark batch: its near-flat rows are finished with most of their shares unsorted, none by the whole-row
    path."""
    g = assert_parity(gpu_ctx, workloads.config4(), cap=512)
    _say("config4 paths: %s" % _paths(g))
    assert not (g["path"] == api.PATH_GENERAL).any() and (g["path"] == PATH_SUMMED).sum() >= 100


def test_many_shapes(gpu_ctx):
    """Flat to peaked rows, cool to hot, narrow to nearly whole nuclei, one draw each."""
    w = _batch(192, 151552, 1, sigmas=[0.05, 0.1, 0.3, 1.0, 2.0, 3.0], temps=[0.5, 1.0, 1.5, 0.8],
               top_ps=[0.5, 0.8, 0.9, 0.99, 0.999, 0.95, 0.7, 0.9999])
    g = assert_parity(gpu_ctx, w, cap=128)
    _say("many shapes paths: %s" % _paths(g))
    assert (g["path"] == PATH_SUMMED).sum() >= 32


@pytest.mark.parametrize("sigma", [0.1, 1.0])
def test_walk_depths(gpu_ctx, sigma):
    """The same kind of row drawn at u from 0 to 1 - 2^-24: the walk ends in the sorted head, inside the region of
    unsorted shares (which the plan must then have left sorted around the end) and at the very cut."""
    us = [0.0, 2.0**-24, 1e-4, 0.01, 0.1, 0.25, 0.4999999, 0.5, 0.5000001, 0.6, 0.7, 0.8, 0.9, 0.95, 0.99, 0.999,
          0.9999, 0.99999, 1.0 - 2.0**-23, 1.0 - 2.0**-24, 0.3333333, 0.6666667, 0.125, 0.875]
    w = _batch(144, 129280, 2, sigmas=[sigma], temps=[1.0], top_ps=[0.9, 0.97, 0.6], us=us, name="walk depths")
    g = assert_parity(gpu_ctx, w, cap=64)
    _say("walk depths (sigma %g) paths: %s" % (sigma, _paths(g)))
    assert (g["path"] == PATH_SUMMED).sum() >= 32


def test_with_penalties_and_masks(gpu_ctx):
    rng = np.random.Generator(np.random.PCG64([3, 77]))
    rows, vocab, hl = 160, 129280, 512
    w = _batch(rows, vocab, 3, sigmas=[0.2, 1.5], temps=[0.9, 1.2], top_ps=[0.9, 0.98])
    w["params"]["repetition_penalty"] = 1.1
    w["params"]["frequency_penalty"] = 0.2
    w["params"]["presence_penalty"] = 0.3
    w["hist"] = workloads.zipf_history(rng, workloads._zipf_cdf(vocab), rows, hl)
    w["hist_len"] = np.full(rows, hl, np.uint32)
    words = (vocab + 31) // 32
    bits = rng.random((rows, words * 32)) < 0.7
    bits[:, vocab:] = False
    w["mask"] = np.ascontiguousarray(np.packbits(bits.reshape(rows, words, 32), axis=2, bitorder="little").view(np.uint32).reshape(rows, words))
    g = assert_parity(gpu_ctx, w, cap=64)
    _say("penalties and masks paths: %s" % _paths(g))
    assert (g["path"] == PATH_SUMMED).any()


def test_long_candidate_lists_written_out(gpu_ctx):
    """The caller asks for 20 000 candidates per row: what is written out must come from sorted shares."""
    w = _batch(136, 129280, 4, sigmas=[0.1, 0.5], temps=[1.0], top_ps=[0.9, 0.99])
    g = assert_parity(gpu_ctx, w, cap=20000)
    _say("long candidate lists paths: %s" % _paths(g))


def test_few_distinct_weights(gpu_ctx):
    """Logits on a coarse grid: thousands of equal weights per value, exact ties by the hundred.  Whatever route such
    rows take (shares with more ties than are kept apart are given up to the whole-row path), the results are the
    oracle's."""
    w = _batch(136, 65536, 5, sigmas=[0.3, 1.0, 2.0], temps=[1.0, 0.5], top_ps=[0.9, 0.99])
    w["logits"] = (np.round(w["logits"] * 16.0) / 16.0).astype(np.float32)
    g = assert_parity(gpu_ctx, w, cap=64)
    _say("few distinct weights paths: %s" % _paths(g))
    w["logits"] = (np.round(w["logits"] * 2.0) / 2.0).astype(np.float32)
    g = assert_parity(gpu_ctx, w, cap=64)
    _say("very few distinct weights paths: %s" % _paths(g))


def test_verification_rows_keep_their_sorted_lists(gpu_ctx):
    """Verification reads the list itself: a large batch of verification rows leaves nothing unsorted."""
    w = _batch(136, 129280, 6, sigmas=[0.1, 1.0], temps=[1.0], top_ps=[0.9])
    rng = np.random.Generator(np.random.PCG64([6, 78]))
    draft = rng.integers(0, 129280, 136).astype(np.int32)
    u2 = workloads._uniforms(rng, 136)
    g = gpu_rows(gpu_ctx, w, draft=draft, u2=u2)
    ref = oracle_rows(w, draft=draft, u2=u2)
    for r, (t, tr) in enumerate(ref):
        assert g["tokens"][r] == t and bool(g["accepted"][r]) == bool(tr["accepted"]), (r, g["tokens"][r], t)
    assert not (g["path"] == PATH_SUMMED).any()


def test_hinted_and_unhinted_calls_agree(gpu_ctx):
    """With the caller's host copy of the parameters the library counts the top_k = 0 rows itself (96 of 128 here:
    shares are left unsorted); the results are those of the plain call and the oracle's."""
    w = _batch(128, 129280, 7, sigmas=[0.1, 0.5, 2.0], temps=[1.0, 0.7], top_ps=[0.9, 0.95])
    w["params"]["top_k"][::4] = 40
    g = assert_parity(gpu_ctx, w, cap=64)
    b = api.Batch(w["logits"], w["params"], w["u"], diagnostics=True, params_host=True)
    gpu_ctx.sample_batch(b.desc, params_host=b.params_host)
    h = b.results()
    _say("hinted paths: %s, plain: %s" % (_paths(h), _paths(g)))
    assert np.array_equal(h["tokens"], g["tokens"]) and np.array_equal(h["n_cand"], g["n_cand"])
    assert np.array_equal(h["total"].view(np.uint32), g["total"].view(np.uint32))
    assert (h["path"] == PATH_SUMMED).any()


def test_random_large_batches():
    """Sixteen batches of random shape and content (random_large_batch), each with a context of its own size."""
    total = np.zeros(9, np.int64)
    for seed in range(9000, 9016):
        w, cap = random_large_batch(seed)
        b, v = w["logits"].shape
        ctx = api.SamplerContext(max_rows=b, max_vocab=v, max_hist=2048)
        try:
            g = assert_parity(ctx, w, cap=cap)
        finally:
            ctx.close()
        total += np.bincount(g["path"], minlength=9)[:9]
    _say("random large batches, rows by path: %s" % total.tolist())
    assert total[PATH_SUMMED] > 200
