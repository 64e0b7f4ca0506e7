"""mako_sampler_sample_batch_static (scratch memory inside the library's image, nothing allocated) against
mako_sampler_sample_batch on the same batches, through the C ABI: every output bit for bit, two calls in a row, the
second one smaller."""
import numpy as np
import pytest

from mako_amd import api, hip, workloads
from parity import oracle_rows

pytestmark = pytest.mark.gpu

KEYS = ("tokens", "n_cand", "total", "q", "path", "cand_idx", "cand_q")


def _both(ctx, w, cap=64):
    """The batch through the context's scratch memory and through the static one."""
    out = []
    for static in (False, True):
        b = api.Batch(w["logits"], w["params"], w["u"], hist=w.get("hist"), hist_len=w.get("hist_len"), cand_cap=cap)
        if static:
            ctx.sample_batch_static(b.desc)
        else:
            ctx.sample_batch(b.desc)
        out.append(b.results())
    return out


def _mixed(rows, vocab, hist_len, seed):
    """Decode-shaped rows (wide and narrow nuclei, top-k, penalties over a history) plus rows for the whole-row path
    (top_k alone, top_k beyond the candidate lists) and a greedy row."""
    w = workloads.config3(seed=seed, rows=rows, vocab=vocab, hist_len=hist_len)
    p = w["params"]
    p["top_k"][0], p["top_p"][0] = 0, 0.97          # a wide nucleus
    p["top_k"][1], p["top_p"][1] = 40, 1.0          # top_k alone: the partial-selection order
    p["top_k"][2], p["top_p"][2] = 700, 0.9         # more than the candidate lists certify
    p["temperature"][3] = 0.0                       # greedy
    return w


def _same(ref, got, what):
    for k in KEYS:
        a, b = np.ascontiguousarray(ref[k]), np.ascontiguousarray(got[k])
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), "%s: %s differs" % (what, k)


def test_static_scratch_matches_context_scratch(gpu_ctx, oracle):
    big = _mixed(api.STATIC_MAX_ROWS, workloads.V_DEEPSEEK, 2048, seed=7101)
    ref, got = _both(gpu_ctx, big)
    _same(ref, got, "16 x 129280")
    # and against the CPU restatement of the reference, so that both being wrong the same way would show
    for r, (t, _) in enumerate(oracle_rows(big)):
        assert got["tokens"][r] == t, (r, int(got["tokens"][r]), t)
    # the second call, smaller in both dimensions, on what the first one left in the array
    small = _mixed(5, 32000, 300, seed=7102)
    ref, got = _both(gpu_ctx, small)
    _same(ref, got, "5 x 32000")
    for r, (t, _) in enumerate(oracle_rows(small)):
        assert got["tokens"][r] == t, (r, int(got["tokens"][r]), t)
    # and the first again: what the small call left behind does not leak into a larger one
    ref, got = _both(gpu_ctx, big)
    _same(ref, got, "16 x 129280 again")


def test_static_call_allocates_no_device_memory(gpu_ctx):
    """What the entry point is for: the device's free memory is the same before the first and after the last of a
    run of static calls, of different sizes and with the per-kernel events of set_profile() recorded around them
    (inputs and outputs are allocated before the first reading)."""
    big = _mixed(api.STATIC_MAX_ROWS, workloads.V_DEEPSEEK, 2048, seed=7103)
    small = _mixed(5, 32000, 300, seed=7104)
    batches = [api.Batch(w["logits"], w["params"], w["u"], hist=w.get("hist"), hist_len=w.get("hist_len"), cand_cap=64)
               for w in (big, small, big)]
    gpu_ctx.set_profile(True)  # (the events are created here, not inside a call)
    try:
        gpu_ctx.sample_batch_static(batches[1].desc)  # (first use of every kernel: code objects are loaded by now)
        hip.synchronize()
        free_before, _ = hip.mem_get_info()
        for b in batches:
            gpu_ctx.sample_batch_static(b.desc)
            hip.synchronize()
            assert len(gpu_ctx.kernel_times_ms()) == api.SAMPLER_KERNELS
        free_after, _ = hip.mem_get_info()
    finally:
        gpu_ctx.set_profile(False)
    assert free_after == free_before, (free_before, free_after)
    for b, w in zip(batches, (big, small, big)):
        for r, (t, _) in enumerate(oracle_rows(w)):
            assert b.results()["tokens"][r] == t


def test_static_scratch_rejects_what_does_not_fit(gpu_ctx):
    w = workloads.config1(rows=api.STATIC_MAX_ROWS + 1, vocab=4096)
    b = api.Batch(w["logits"], w["params"], w["u"])
    with pytest.raises(api.MakoError, match="scratch memory holds batches of up to 16 rows"):
        gpu_ctx.sample_batch_static(b.desc)
    w = workloads.config1(rows=1, vocab=api.STATIC_MAX_VOCAB + 4)
    b = api.Batch(w["logits"], w["params"], w["u"])
    with pytest.raises(api.MakoError, match="131072 logits"):
        gpu_ctx.sample_batch_static(b.desc)
    gpu_ctx.sample_batch(b.desc)  # the context's own scratch memory takes it
    assert 0 <= int(b.results()["tokens"][0]) < api.STATIC_MAX_VOCAB + 4
