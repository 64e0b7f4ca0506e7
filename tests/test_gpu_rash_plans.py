"""Large batches of top_k = 0 rows through libmako_sampler_rash.so: the checked library whose plans leave shares of the
sorted lists unsorted that they should NOT (each row drops one of the four rules of opaque_guess(),
mako_amd/csrc/unsorted_shares.h, in turn: the position behind the staged head, the binades of sum and r, the top-p cut,
the walk).  The plan's guesses only decide who tries: tail_kernel tests every record it applies and gives a row up to
the whole-row path when one does not hold, so the results must still be the oracle's, bit for bit, and no index check
may fail."""
import numpy as np
import pytest

from mako_amd import api, hip, workloads
from parity import assert_parity, nucleus_batch, random_large_batch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rash_ctx():
    if hip.device_count() < 1:
        pytest.fail("no HIP device: GPU tests need an MI355X")
    hip.set_device(0)
    ctx = api.SamplerContext(max_rows=256, max_vocab=151552, max_hist=1024, lib_path=api.RASH_LIB_PATH)
    yield ctx
    ctx.close()


def _run(ctx, w, cap):
    ctx.failed_checks()  # (clears what an earlier batch left)
    g = assert_parity(ctx, w, cap=cap)
    bits = ctx.failed_checks()
    assert bits == 1 << 31, "index checks failed: bit set 0x%x" % bits
    paths = np.bincount(g["path"], minlength=9).tolist()
    print("%s paths: %s" % (w["name"], paths), flush=True)
    return g


def test_rash_plans_config4(rash_ctx):
    g = _run(rash_ctx, workloads.config4(), 256)
    # (rows were given up, and rows got through on records that held)
    assert (g["path"] == api.PATH_GENERAL).any() and (g["path"] == api.PATH_SUMMED).any()


def test_rash_plans_many_shapes(rash_ctx):
    w = nucleus_batch(160, 129280, 11, sigmas=[0.05, 0.1, 0.3, 1.0, 2.0, 3.0, 0.2], temps=[0.5, 1.0, 1.5],
                      top_ps=[0.5, 0.9, 0.99, 0.999, 0.8], name="rash, many shapes")
    g = _run(rash_ctx, w, 128)
    assert (g["path"] == api.PATH_GENERAL).any()


def test_rash_plans_walk_depths(rash_ctx):
    us = [0.0, 1e-4, 0.01, 0.1, 0.25, 0.5, 0.6, 0.7, 0.8, 0.9, 0.95, 0.99, 0.999, 0.9999, 1.0 - 2.0**-24, 0.3333333, 0.6666667]
    w = nucleus_batch(136, 129280, 12, sigmas=[0.1, 1.0], temps=[1.0], top_ps=[0.9, 0.97], us=us, name="rash, walk depths")
    _run(rash_ctx, w, 64)


def test_rash_plans_random_large_batches():
    total = np.zeros(9, np.int64)
    for seed in range(9100, 9110):
        w, cap = random_large_batch(seed)
        b, v = w["logits"].shape
        ctx = api.SamplerContext(max_rows=b, max_vocab=v, max_hist=2048, lib_path=api.RASH_LIB_PATH)
        try:
            g = _run(ctx, w, cap)
        finally:
            ctx.close()
        total += np.bincount(g["path"], minlength=9)[:9]
    assert total[api.PATH_GENERAL] > 50
