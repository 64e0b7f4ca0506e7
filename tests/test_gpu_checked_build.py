"""The BASELINE workloads and the rarer paths through libmako_sampler_checked.so: the same kernels with every index
into the context's scratch arrays compared with the array's bound (-DMAKO_CHECKED).  No check may fail, and the tokens
must be the shipped library's."""
import numpy as np
import pytest

from mako_amd import api, hip, workloads
from parity import gpu_rows

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def checked_ctx():
    if hip.device_count() < 1:
        pytest.fail("no HIP device: GPU tests need an MI355X")
    hip.set_device(0)
    ctx = api.SamplerContext(max_rows=64, max_vocab=151552, max_hist=4096, lib_path=api.CHECKED_LIB_PATH)
    yield ctx
    ctx.close()


def _mixed_paths(rows, vocab, seed):
    """Decode rows plus rows for the whole-row path (top_k alone, top_k beyond the candidate lists) and a greedy row."""
    w = workloads.config3(seed=seed, rows=rows, vocab=vocab, hist_len=2048)
    p = w["params"]
    p["top_k"][0], p["top_p"][0] = 0, 0.999       # a very wide nucleus
    p["top_k"][1], p["top_p"][1] = 40, 1.0        # top_k alone: the partial-selection order
    p["top_k"][2], p["top_p"][2] = 700, 0.9       # more than the candidate lists certify
    p["temperature"][3] = 0.0                     # greedy
    return w


def test_no_index_check_fails_on_rows_in_token_order(gpu_ctx, checked_ctx):
    """Temperature-only rows beside the others, with the host copy of the parameters: the kernels of index_rows.h."""
    w = _mixed_paths(24, workloads.V_DEEPSEEK, 9108)
    w["params"]["top_k"][4::3] = 0
    w["params"]["top_p"][4::3] = 1.0
    checked_ctx.failed_checks()
    got = gpu_rows(checked_ctx, w, cap=0, hinted=True)
    bits = checked_ctx.failed_checks()
    assert bits == 1 << 31, "index checks failed: bit set 0x%x" % bits
    ref = gpu_rows(gpu_ctx, w, cap=0, hinted=True)
    assert np.array_equal(got["tokens"], ref["tokens"]) and np.array_equal(got["n_cand"], ref["n_cand"])
    assert (got["path"][4::3] == api.PATH_INDEXED).all()


@pytest.mark.parametrize("name", ["config3", "config4", "config5", "mixed"])
def test_no_index_check_fails(gpu_ctx, checked_ctx, name):
    if name == "config3":
        w = workloads.config3()
    elif name == "config4":
        w = workloads.config4(rows=32)
    elif name == "config5":
        w = workloads.config5(rows=32, density=0.5)
    else:
        w = _mixed_paths(24, workloads.V_DEEPSEEK, 9107)
    checked_ctx.failed_checks()  # (clears what an earlier batch left)
    got = gpu_rows(checked_ctx, w, cap=64)
    bits = checked_ctx.failed_checks()
    # bit 31: the checks are compiled in and their word is read; every other bit is a failed check
    assert bits == 1 << 31, "index checks failed: bit set 0x%x" % bits
    ref = gpu_rows(gpu_ctx, w, cap=64)
    assert np.array_equal(got["tokens"], ref["tokens"])
    assert np.array_equal(got["n_cand"], ref["n_cand"])
    assert gpu_ctx.failed_checks() == 0  # (the shipped library has no checks: always 0)


def test_no_index_check_fails_on_a_large_batch(gpu_ctx):
    """config 4 whole (256 rows: the second pass's looped pieces, sort_kernel's collectors of unsorted shares and the
    instance of tail_kernel that applies their records only occur on large batches)."""
    ctx = api.SamplerContext(max_rows=256, max_vocab=151552, max_hist=0, lib_path=api.CHECKED_LIB_PATH)
    try:
        w = workloads.config4()
        ctx.failed_checks()
        got = gpu_rows(ctx, w, cap=64)
        bits = ctx.failed_checks()
        assert bits == 1 << 31, "index checks failed: bit set 0x%x" % bits
        ref = gpu_rows(gpu_ctx, w, cap=64)
        assert np.array_equal(got["tokens"], ref["tokens"]) and np.array_equal(got["n_cand"], ref["n_cand"])
        assert (got["path"] == api.PATH_SUMMED).any()
    finally:
        ctx.close()
