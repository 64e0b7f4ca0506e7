"""GPU parity tests: the HIP sampler, called through the C ABI, against the CPU oracle."""
import os
import sys

import numpy as np
import pytest

from mako_amd import api, hip, workloads
from oracle import pyoracle
from parity import assert_parity, gpu_rows, oracle_rows

pytestmark = pytest.mark.gpu

SAMPLER_TEST_LOGITS = np.array([[2.0, 1.5, 0.3, -0.5, 1.9, -2.0, 0.0, 1.0]], np.float32)  # tests/sampler_test.cpp:56


def _say(msg):
    print(msg, flush=True)


def test_device_expf_matches_oracle(gpu_ctx, oracle):
    """expf on the device equals the glibc restatement on 4M inputs incl. the underflow edge and specials."""
    rng = np.random.default_rng(7)
    x = np.concatenate([
        -np.abs(rng.standard_normal(1 << 21) * 30).astype(np.float32),
        rng.integers(0, 2**32, 1 << 21, dtype=np.uint64).astype(np.uint32).view(np.float32),
        np.linspace(-104.5, -102.5, 1 << 16).astype(np.float32),
        np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 88.0, 88.8, -87.9, -88.0, -103.9, -103.97, -103.98, -104.0, -1e-30, 1e-30,
                  -150.0], np.float32)])
    dx = hip.DeviceArray.from_host(x)
    dy = hip.DeviceArray(x.shape, np.float32)
    assert gpu_ctx.lib.mako_sampler_debug_expf(dx.ptr, dy.ptr, x.size, None) == 0
    hip.synchronize()
    y = dy.download()
    want = oracle.expf_array(x)  # every one of them
    same = (y.view(np.uint32) == want.view(np.uint32)) | (np.isnan(y) & np.isnan(want))
    assert same.all(), (x[~same][:5], y[~same][:5], want[~same][:5])


def test_device_division_is_ieee(gpu_ctx):
    rng = np.random.default_rng(8)
    a = rng.integers(0, 2**32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
    b = rng.integers(0, 2**32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
    a[:1000] = (rng.standard_normal(1000) * 5).astype(np.float32)
    b[:1000] = np.float32(1.1)
    da, db = hip.DeviceArray.from_host(a), hip.DeviceArray.from_host(b)
    dy = hip.DeviceArray(a.shape, np.float32)
    assert gpu_ctx.lib.mako_sampler_debug_div(da.ptr, db.ptr, dy.ptr, a.size, None) == 0
    hip.synchronize()
    y = dy.download()
    with np.errstate(all="ignore"):
        want = a / b
    same = (y.view(np.uint32) == want.view(np.uint32)) | (np.isnan(y) & np.isnan(want))
    assert same.all(), (a[~same][:5], b[~same][:5], y[~same][:5], want[~same][:5])


def test_reference_known_answers(gpu_ctx):
    """The exact checks of tests/sampler_test.cpp:61-67,135-144 and its truncation sets (:91-117)."""
    lg = SAMPLER_TEST_LOGITS
    u = np.array([0.3], np.float32)
    r = api.sample(gpu_ctx, lg, api.make_params(1, 0.0), u)
    assert r["tokens"][0] == 0
    r = api.sample(gpu_ctx, lg, api.make_params(1, 0.0), u, draft=np.array([4]), u2=u)
    assert r["tokens"][0] == 0 and r["accepted"][0] == 0
    r = api.sample(gpu_ctx, lg, api.make_params(1, 0.0), u, draft=np.array([0]), u2=u)
    assert r["tokens"][0] == 0 and r["accepted"][0] == 1
    r = api.sample(gpu_ctx, lg, api.make_params(1, 1e-40), u)
    assert r["tokens"][0] == 0 and r["path"][0] == api.PATH_FALLBACK
    r = api.sample(gpu_ctx, lg, api.make_params(1, 1.0, top_k=3), u, cand_cap=8)
    assert sorted(r["cand_idx"][0, :3].tolist()) == [0, 1, 4] and r["n_cand"][0] == 3
    r = api.sample(gpu_ctx, lg, api.make_params(1, 1.0, top_p=0.7), u, cand_cap=8)
    assert r["cand_idx"][0, :3].tolist() == [0, 4, 1] and r["n_cand"][0] == 3
    r = api.sample(gpu_ctx, lg, api.make_params(1, 1.0, min_p=0.3), u, cand_cap=8)
    assert sorted(r["cand_idx"][0, :4].tolist()) == [0, 1, 4, 7] and r["n_cand"][0] == 4
    # presence 0.5 + frequency 0.25, token 0 accepted twice: logit[0] -= 1.0 (:118-126)
    r = api.sample(gpu_ctx, lg, api.make_params(1, 1.0, presence_penalty=0.5, frequency_penalty=0.25), u,
                   hist=np.array([[0, 0]], np.int32), cand_cap=8)
    want = np.exp(np.float32(1.0) - np.float32(1.9))  # token 4 is now the max
    assert abs(r["cand_q"][0, 0] - want) < 1e-6 and r["cand_idx"][0, 0] == 0
    # repetition 2.0 with tokens 0 and 5: l0 / 2, l5 * 2 (:127-133)
    r = api.sample(gpu_ctx, lg, api.make_params(1, 1.0, repetition_penalty=2.0), u, hist=np.array([[0, 5]], np.int32),
                   cand_cap=8)
    q = dict(zip(r["cand_idx"][0].tolist(), r["cand_q"][0].tolist()))
    assert abs(q[0] - np.exp(1.0 - 1.9)) < 1e-6 and abs(q[5] - np.exp(-4.0 - 1.9)) < 1e-7
    r = api.sample(gpu_ctx, lg, api.make_params(1, 1.0, repetition_penalty=0.0), u, hist=np.array([[0, 4]], np.int32))
    assert 0 <= r["tokens"][0] < 8


def _random_case(rng, v, b):
    logits = (rng.standard_normal((b, v)) * 3).astype(np.float32)
    kind = rng.integers(0, 4)
    if kind == 1:
        logits = np.round(logits * 2) / 2  # many exact ties
    if kind == 2:
        logits = (logits * 0.03).astype(np.float32)  # near-flat: big nuclei
    p = api.make_params(b)
    p["temperature"] = rng.choice(np.array([0.0, 0.3, 0.7, 1.0, 1.2, 2.5], np.float32), b)
    p["top_k"] = rng.choice(np.array([0, 0, 1, 3, 20, 50, 100, 129, 5000, v, v + 7], np.uint32), b)
    p["top_p"] = rng.choice(np.array([1.0, 0.999, 0.95, 0.9, 0.5, 0.0, 1.5, -1.0], np.float32), b)
    p["min_p"] = rng.choice(np.array([0.0, 0.0, 0.0, 0.05, 0.5, 1.0, 2.0], np.float32), b)
    p["presence_penalty"] = rng.choice(np.array([0.0, 0.3, -0.5], np.float32), b)
    p["frequency_penalty"] = rng.choice(np.array([0.0, 0.2], np.float32), b)
    p["repetition_penalty"] = rng.choice(np.array([1.0, 1.1, 2.0, 0.5, 0.0], np.float32), b)
    w = dict(name="random_v%d" % v, logits=logits, params=p, u=rng.random(b).astype(np.float32))
    hl = int(rng.choice([0, 1, 17, 600]))
    if hl:
        w["hist"] = rng.integers(0, v, (b, hl)).astype(np.int32)
        w["hist"][:, : hl // 2] = w["hist"][:, :1]  # repeats
        w["hist_len"] = rng.integers(0, hl + 1, b).astype(np.uint32)
    if rng.integers(0, 3) == 0:
        w["mask"] = rng.integers(0, 2**32, (b, (v + 31) // 32), dtype=np.uint64).astype(np.uint32)
    return w


@pytest.mark.parametrize("v", [1, 2, 8, 63, 64, 65, 1000, 4096, 16384, 16385, 40000, 129280])
def test_random_parameters(gpu_ctx, v):
    """Random parameter mixes (ties, near-flat rows, masks, histories, extreme values) at many vocabulary sizes."""
    rng = np.random.default_rng(1000 + v)
    for it in range(3):
        w = _random_case(rng, v, 24 if v < 100000 else 8)
        _say("random case v=%d it=%d" % (v, it))
        assert_parity(gpu_ctx, w, cap=min(v, 512))


@pytest.mark.parametrize("v", [65, 4096, 40000, 129280])
def test_random_parameters_with_zipf_histories(gpu_ctx, v):
    """The same random mixes with Zipf(1.1) histories (most of a history in the first slice, few distinct tokens
    many times over) and, now and then, a NaN logit at a penalised position."""
    rng = np.random.default_rng(3000 + v)
    done = 0
    while done < 4:
        w = _random_case(rng, v, 24 if v < 100000 else 8)
        if "hist" not in w:
            continue
        b, hl = w["hist"].shape
        w["hist"] = np.minimum(v - 1, rng.zipf(1.1, (b, hl)) - 1).astype(np.int32)
        if done % 2:
            w["logits"][0, int(w["hist"][0, 0])] = np.nan
        _say("zipf history case v=%d it=%d" % (v, done))
        assert_parity(gpu_ctx, w, cap=min(v, 512))
        done += 1


def _topk_only_case(rng, v, b, ks):
    w = _random_case(rng, v, b)
    p = w["params"]
    p["temperature"] = rng.choice(np.array([0.3, 0.7, 1.0, 2.5], np.float32), b)
    p["top_k"] = rng.choice(np.array(ks, np.uint32), b)
    p["top_p"] = rng.choice(np.array([1.0, 1.5], np.float32), b)
    return w


@pytest.mark.parametrize("v", [4, 5, 8, 65, 1000, 16385, 40000, 129280, 151552])
def test_topk_alone_keeps_nth_element_order(gpu_ctx, v):
    """top_k without top-p: the survivors are summed and walked in the order libstdc++'s nth_element leaves
    (src/gen/sampler.cpp:39-43, 79-83); candidate lists, fp32 totals and tokens equal the oracle's, whose
    introselect is pinned against std::nth_element itself on the CPU."""
    rng = np.random.default_rng(4100 + v)
    ks = [1, 2, 3, 7, 40, 100, 129, 1000, 5000, v // 2, v - 1, v]
    for it in range(3):
        w = _topk_only_case(rng, v, 24 if v < 100000 else 6, [k for k in ks if 0 < k])
        _say("top-k alone v=%d it=%d" % (v, it))
        assert_parity(gpu_ctx, w, cap=min(v, 512))


def test_topk_alone_verify(gpu_ctx):
    """Sampler::verify over the nth_element order: the draft's weight, and the redraw over the list without it."""
    rng = np.random.default_rng(4200)
    v, b = 20000, 32
    w = _topk_only_case(rng, v, b, [3, 40, 100, 1000])
    first = oracle_rows(w)
    draft = np.array([t for t, _ in first], np.int32)
    draft[::3] = rng.integers(0, v, len(draft[::3]))
    u2 = rng.random(b).astype(np.float32)
    g = gpu_rows(gpu_ctx, w, draft=draft, u2=u2)
    ref = oracle_rows(w, draft=draft, u2=u2)
    for r, (t, tr) in enumerate(ref):
        assert g["tokens"][r] == t and bool(g["accepted"][r]) == tr["accepted"], (r, g["tokens"][r], t)


def test_topk_alone_depth_limit(gpu_ctx, oracle):
    """Worst-case orders recorded from libstdc++ (tests/golden: nth_killers) drive introselect to its depth limit:
    the heap select must leave the library's arrangement too.  The logits keep the recorded weights' order."""
    import json
    import os
    golden = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
    for k in golden["nth_killers"]:
        q = np.array(k["q"], np.float32)
        ranks = np.unique(-q, return_inverse=True)[1]  # 0 = heaviest; equal weights keep equal logits
        logits = (-(ranks.astype(np.float32)) * np.float32(0.002)).reshape(1, -1)
        p = api.make_params(1, 1.0, top_k=int(k["nth"]))
        w = dict(name="nth_killer_%d" % k["n"], logits=logits, params=p, u=np.array([0.61], np.float32))
        before = oracle.heap_selects()
        _say("depth limit case n=%d nth=%d" % (k["n"], k["nth"]))
        assert_parity(gpu_ctx, w, cap=int(k["n"]))
        assert oracle.heap_selects() > before, "the case no longer reaches the depth limit"


@pytest.mark.parametrize("nth", [3000, 20000, 100000])
def test_topk_alone_depth_limit_whole_row(gpu_ctx, oracle, reference, nth):
    """The same at full size: an adversary (McIlroy's, run against std::nth_element itself by the reference build's
    shim) orders a 129 280-entry row so that introselect spends its depth limit while the range is still the whole row
    in device memory, and the heap select that follows has to pop nearly every entry.  The heap holds nth + 1 entries:
    inside LDS (3000) or only its upper levels there (20000, 100000).  The call must stay short (the sweep goes 64 entries
    per ballot, the heap is built level by level) and leave the library's arrangement."""
    import time
    n = workloads.V_DEEPSEEK
    q, _ = reference.make_nth_killer(n, nth)
    ranks = np.unique(-q, return_inverse=True)[1]  # 0 = heaviest; equal weights keep equal logits
    logits = (-(ranks.astype(np.float32)) * np.float32(0.0007)).reshape(1, -1)  # (every weight stays above zero)
    p = api.make_params(1, 1.0, top_k=nth)
    w = dict(name="nth_killer_%d_%d" % (n, nth), logits=logits, params=p, u=np.array([0.61], np.float32))
    before = oracle.heap_selects()
    _say("depth limit case n=%d nth=%d" % (n, nth))
    cap = min(nth, 4096)
    t0 = time.perf_counter()
    g = gpu_rows(gpu_ctx, w, cap=cap)
    dt = time.perf_counter() - t0
    _say("  the call took %.1f ms" % (dt * 1e3))
    assert_parity(gpu_ctx, w, cap=cap)
    assert g["n_cand"][0] == nth
    assert oracle.heap_selects() > before, "the case no longer reaches the depth limit"
    assert dt < 2.0, "the depth limit's heap select took %.2f s" % dt


def test_special_values(gpu_ctx):
    """NaN/inf logits, all-masked rows, NaN parameters: the fallbacks of src/gen/sampler.cpp:37-38."""
    v = 5000
    rng = np.random.default_rng(5)
    base = (rng.standard_normal((12, v)) * 3).astype(np.float32)
    base[0, 0] = np.nan
    base[1, 17] = np.nan
    base[2, :] = -np.inf
    base[3, 100] = np.inf
    base[4, 100] = np.inf
    base[4, 200] = np.inf
    base[5, :] = 1.25
    base[6, :] = 0.0
    base[6, 7] = -0.0
    base[7, 1:] = np.nan
    p = api.make_params(12, 0.8, 0, 0.9)
    p["temperature"][8] = np.nan
    p["top_p"][9] = np.nan
    p["min_p"][10] = np.nan
    p["temperature"][11] = 1e-40
    w = dict(name="special", logits=base, params=p, u=rng.random(12).astype(np.float32))
    assert_parity(gpu_ctx, w)
    w["params"] = api.make_params(12, 0.0)
    assert_parity(gpu_ctx, w)
    mask = np.zeros((12, (v + 31) // 32), np.uint32)
    mask[1, 3] = 1 << 5
    w["mask"] = mask
    w["params"] = p
    assert_parity(gpu_ctx, w)


@pytest.mark.parametrize("hist_len", [1500, 3000, 9000])
def test_history_lengths(gpu_ctx, hist_len):
    """Histories of up to 2 and up to 8 entries per thread stay in registers, longer ones take the generic route:
    all three against the oracle, with heavy repetition (Zipf) and tokens that hit the row maximum."""
    w = workloads.config3(rows=12, vocab=50000, hist_len=hist_len, seed=600 + hist_len)
    top = w["logits"].argmax(axis=1)
    w["hist"][:, 0] = top          # the most likely token is penalised
    w["hist"][:6, 1] = 0           # and token 0
    w["logits"][3, 0] = np.nan     # NaN at index 0 of a penalised token
    assert_parity(gpu_ctx, w, cap=512)


def test_history_forms_agree(gpu_ctx):
    """Raw accept() token lists and pre-aggregated (id, count) pairs give identical results."""
    w = workloads.config3(rows=8, vocab=30000, hist_len=300)
    g1 = gpu_rows(gpu_ctx, w)
    hist = np.zeros_like(w["hist"])
    cnts = np.zeros(w["hist"].shape, np.uint32)
    lens = np.zeros(8, np.uint32)
    for r in range(8):
        ids, c = np.unique(w["hist"][r], return_counts=True)
        hist[r, : len(ids)], cnts[r, : len(ids)], lens[r] = ids, c, len(ids)
    w2 = dict(w, hist=hist, hist_len=lens)
    g2 = gpu_rows(gpu_ctx, w2, hist_counts=cnts)
    assert np.array_equal(g1["tokens"], g2["tokens"]) and np.array_equal(g1["total"], g2["total"])


def test_verify_matches_oracle(gpu_ctx):
    """Sampler::verify (src/gen/sampler.cpp:86-107): accept/reject and the redraw, against the oracle."""
    rng = np.random.default_rng(77)
    v, b = 20000, 48
    w = _random_case(rng, v, b)
    w["params"]["temperature"][: b // 2] = 0.9
    w["params"]["top_k"][: b // 2] = 40
    w["params"]["top_p"][: b // 2] = 0.95
    first = oracle_rows(w)
    draft = np.array([t for t, _ in first], np.int32)
    draft[::3] = rng.integers(0, v, len(draft[::3]))
    u2 = rng.random(b).astype(np.float32)
    g = gpu_rows(gpu_ctx, w, draft=draft, u2=u2)
    ref = oracle_rows(w, draft=draft, u2=u2)
    for r, (t, tr) in enumerate(ref):
        assert g["tokens"][r] == t and bool(g["accepted"][r]) == tr["accepted"], (r, g["tokens"][r], t)


def _choose(o, w, r, force, close, max_above):
    """Session::run's `choose` (src/gen/session.cpp:441-443) with ReasoningBudget::forced's last-stretch test as the
    callback (src/server/openai.cpp:589-604): (token, forced kind, logits above the close token)."""
    above = 0xFFFFFFFF
    kind, tok = api.FORCED_NONE, -1
    mask = w["mask"][r] if "mask" in w else None
    if close is not None and close[r] >= 0:
        t, above = o.close_forced(w["logits"][r], int(close[r]), max_above, mask)
        if t >= 0:
            kind, tok = api.FORCED_CLOSE, t
    if force is not None and force[r] >= 0:
        kind, tok = api.FORCED_TOKEN, int(force[r])
    if kind == api.FORCED_NONE:
        p = pyoracle.params_from_record(w["params"][r])
        hist = w["hist"][r, : w["hist_len"][r]] if "hist" in w else None
        tok = o.sample(w["logits"][r], p, float(w["u"][r]), hist, mask)[0]
    return tok, kind, above


@pytest.mark.parametrize("v", [1000, 40000, 129280])
def test_forced_and_close_tokens(gpu_ctx, v):
    """The decode loop's `forced` hook: known tokens, and the close token taken iff fewer than three logits lie
    strictly above its own (src/server/openai.cpp:596-603), counted in the sampler's own pass over the logits."""
    rng = np.random.default_rng(4000 + v)
    o = pyoracle.oracle()
    b = 32
    for it in range(3):
        w = _random_case(rng, v, b)
        close = rng.integers(0, v, b).astype(np.int32)
        order = np.argsort(-w["logits"], axis=1, kind="stable")
        for r in range(b):  # put the close token near the top in most rows: ranks 0..5, ties included
            if r % 4 != 3:
                close[r] = order[r, int(rng.integers(0, min(6, v)))]
        close[::7] = -1
        close[5] = v + 3  # out of range: ignored (:594)
        force = np.full(b, -1, np.int32)
        force[::5] = rng.integers(0, v, len(force[::5]))
        max_above = int(rng.choice([3, 3, 1, 0, 5]))
        _say("forced/close case v=%d it=%d max_above=%d" % (v, it, max_above))
        g = api.sample(gpu_ctx, w["logits"], w["params"], w["u"], mask=w.get("mask"), hist=w.get("hist"),
                       hist_len=w.get("hist_len"), force_token=force, close_token=close, close_max_above=max_above)
        for r in range(b):
            tok, kind, above = _choose(o, w, r, force, close, max_above)
            assert (g["tokens"][r], g["forced"][r], g["above"][r]) == (tok, kind, above), \
                (r, g["tokens"][r], g["forced"][r], g["above"][r], tok, kind, above)
            if kind != api.FORCED_NONE:
                assert g["path"][r] == api.PATH_FORCED


def test_forced_token_meets_draft(gpu_ctx):
    """With a draft, a forced token is returned and the draft is kept only if it equals it
    (src/gen/session.cpp:483-485, 524-525)."""
    rng = np.random.default_rng(91)
    v, b = 5000, 16
    w = _random_case(rng, v, b)
    force = np.full(b, -1, np.int32)
    force[::2] = rng.integers(0, v, b // 2)
    draft = rng.integers(0, v, b).astype(np.int32)
    draft[::4] = force[::4]
    u2 = rng.random(b).astype(np.float32)
    g = api.sample(gpu_ctx, w["logits"], w["params"], w["u"], mask=w.get("mask"), hist=w.get("hist"),
                   hist_len=w.get("hist_len"), draft=draft, u2=u2, force_token=force)
    ref = oracle_rows(w, draft=draft, u2=u2)
    for r in range(b):
        if force[r] >= 0:
            assert g["tokens"][r] == force[r] and bool(g["accepted"][r]) == (force[r] == draft[r]) and g["forced"][r] == 1
        else:
            assert g["tokens"][r] == ref[r][0] and bool(g["accepted"][r]) == ref[r][1]["accepted"] and g["forced"][r] == 0


def test_append_history_decode_loop(gpu_ctx):
    """Sampler::accept on the device (src/gen/session.cpp:419-421): six decode steps whose histories never leave the
    GPU give the tokens of a host loop that keeps the histories itself, forced tokens included; a full history
    buffer is left as it is."""
    rng = np.random.default_rng(12)
    o = pyoracle.oracle()
    v, b, stride, steps = 3000, 12, 16, 6
    p = api.make_params(b, 0.8, 0, 0.95, presence_penalty=0.4, frequency_penalty=0.3, repetition_penalty=1.3)
    p["top_k"][::3] = 20
    p["temperature"][1] = 0.0
    hist = rng.integers(0, v, (b, stride)).astype(np.int32)
    hist_len = rng.integers(0, 12, b).astype(np.uint32)
    hist_len[2] = stride - 2  # fills up on the way
    host_hist = [list(hist[r, : hist_len[r]]) for r in range(b)]
    logits0 = (rng.standard_normal((b, v)) * 2).astype(np.float32)
    batch = api.Batch(logits0, p, np.zeros(b, np.float32), hist=hist, hist_len=hist_len, force_token=np.full(b, -1, np.int32),
                      append_history=True)
    for step in range(steps):
        logits = (rng.standard_normal((b, v)) * 2).astype(np.float32)
        logits[np.arange(b), [h[-1] if h else 0 for h in host_hist]] += 3.0  # the penalties matter
        u = rng.random(b).astype(np.float32)
        force = np.full(b, -1, np.int32)
        force[step % b] = int(rng.integers(0, v))
        batch.d_logits.upload(logits)
        batch.d_u.upload(u)
        batch.d_force.upload(force)
        _say("append step %d" % step)
        gpu_ctx.sample_batch(batch.desc)
        g = batch.results()
        for r in range(b):
            if force[r] >= 0:
                tok = int(force[r])
            else:
                tok = o.sample(logits[r], pyoracle.params_from_record(p[r]), float(u[r]), np.array(host_hist[r], np.int32))[0]
            assert g["tokens"][r] == tok, (step, r, g["tokens"][r], tok)
            if len(host_hist[r]) < stride:
                host_hist[r].append(tok)
    ht, hl = batch.history()
    for r in range(b):
        assert hl[r] == len(host_hist[r]) and list(ht[r, : hl[r]]) == host_hist[r], r


def test_config1(gpu_ctx):
    assert_parity(gpu_ctx, workloads.config1(rows=4))


def test_config2(gpu_ctx):
    assert_parity(gpu_ctx, workloads.config2(rows=2, greedy=True))
    assert_parity(gpu_ctx, workloads.config2(rows=4, greedy=False), cap=1024)


def test_config3_full_batch(gpu_ctx):
    g = assert_parity(gpu_ctx, workloads.config3())
    _say("config3 paths: %s" % np.bincount(g["path"], minlength=8).tolist())
    # (no row of the benchmark batch may need the whole-row path: a plan that keeps too little would still give the
    # right tokens, a hundred times slower)
    assert not (g["path"] == api.PATH_GENERAL).any() and (g["path"] == api.PATH_SORTED).any()


def test_config4_reduced(gpu_ctx):
    """16 of the 256 rows (8 heavy-tailed, 8 near-flat with ~133K-token nuclei)."""
    w = workloads.config4(rows=16)
    g = assert_parity(gpu_ctx, w, cap=2048)
    _say("config4 nuclei: %s" % g["n_cand"].tolist())


def test_config5_masks(gpu_ctx):
    for density in (0.01, 0.5):
        assert_parity(gpu_ctx, workloads.config5(rows=32, density=density))


def test_config4_all_256_rows(gpu_ctx):
    """The whole benchmark batch (128 heavy-tailed rows, 128 near-flat ones with ~133K-token nuclei) against the
    oracle: the second pass's looped piece search, whole-slice pieces and sort_kernel's rounds of workgroups only
    occur beyond 64 rows."""
    g = assert_parity(gpu_ctx, workloads.config4(), cap=512)
    _say("config4 (256 rows) paths: %s" % np.bincount(g["path"], minlength=8).tolist())
    assert not (g["path"] == api.PATH_GENERAL).any() and ((g["path"] == api.PATH_SORTED) | (g["path"] == api.PATH_SUMMED)).sum() >= 128


@pytest.mark.parametrize("density", [0.01, 0.5])
def test_config5_all_256_rows(gpu_ctx, density):
    """The whole verify-shaped batch (32 x 8 rows under per-row bitmasks) against the oracle."""
    g = assert_parity(gpu_ctx, workloads.config5(density=density), cap=64)
    _say("config5 (256 rows, density %g) paths: %s" % (density, np.bincount(g["path"], minlength=6).tolist()))


def test_wide_nucleus_walk_depths(gpu_ctx):
    """top_k = 0 rows whose nuclei hold tens of thousands of tokens, drawn at u from 0 to 1 - 2^-24: the walk
    ends anywhere between the first candidate and the last, crossing many binades of r on the way."""
    rng = np.random.default_rng(4242)
    us = np.array([0.0, 1e-7, 0.03, 0.5, 0.9, 0.999, 0.99999, 1.0 - 2.0**-24], np.float32)
    b = 2 * len(us)
    logits = (rng.standard_normal((b, 129280)) * 3).astype(np.float32)
    p = api.make_params(b, 1.0, 0, 0.95)
    p["temperature"] = np.repeat(np.array([1.0, 1.2], np.float32), len(us))
    p["top_p"] = rng.choice(np.array([0.9, 0.99, 0.9999], np.float32), b)
    w = dict(name="walk_depths", logits=logits, params=p, u=np.tile(us, 2))
    g = assert_parity(gpu_ctx, w, cap=1024)
    _say("walk depths: nuclei %s" % g["n_cand"].tolist())
    assert g["n_cand"].min() > 5000


@pytest.mark.parametrize("u", [0.9, 0.999, 1.0 - 2.0**-24])
def test_config3_deep_walks(gpu_ctx, u):
    """The decode batch drawn at one large u on every row: on its peaked wide rows (a few spikes, then tens of
    thousands of small weights) the walk runs through several blocks of 64 groups, whose maps are rebuilt from the
    exact r at each block's start, and r falls through many binades."""
    w = workloads.config3()
    w["u"] = np.full(64, u, np.float32)
    assert_parity(gpu_ctx, w, cap=64)


def test_tied_wide_nucleus(gpu_ctx):
    """Logits on a grid of 1/8: every weight is shared by hundreds of tokens, so candidates tie in q and the order
    inside a tie is by token id.  The workers' counting sort gives such rows to the stable radix sort."""
    rng = np.random.default_rng(4343)
    b = 6
    logits = (np.round(rng.standard_normal((b, 129280)) * 3 * 8) / 8).astype(np.float32)
    p = api.make_params(b, 1.0, 0, 0.95)
    p["top_p"] = np.array([0.5, 0.9, 0.95, 0.99, 0.999, 0.95], np.float32)
    p["temperature"][5] = 0.4
    w = dict(name="tied_wide", logits=logits, params=p, u=rng.random(b).astype(np.float32))
    assert_parity(gpu_ctx, w, cap=2048)


def test_narrow_nucleus_inside_one_slice(gpu_ctx):
    """A nucleus of ~200 tokens that all live in one 16K-token slice, 14 to each wavefront of the scan: the slice
    keeps only those at or above the smallest of the wavefronts' 8th largest, the certificate of the candidate
    list fails, and the row is finished from the weights the second pass kept for it."""
    rng = np.random.default_rng(4444)
    b, v = 4, 129280
    slice_len = 16160  # ceil(129280 / 8)
    logits = (rng.standard_normal((b, v)) * 0.5).astype(np.float32)
    for r in range(b):
        for wave in range(16):
            lanes = rng.choice(64, 14, replace=False)
            hot = slice_len + 4 * (64 * wave + lanes)  # element 0 of 14 threads of this wave, slice 1
            logits[r, hot] += np.float32(12.0) + rng.random(14).astype(np.float32)
    p = api.make_params(b, 1.0, 0, 0.9)
    p["top_p"] = np.array([0.5, 0.9, 0.97, 0.99], np.float32)
    w = dict(name="one_slice", logits=logits, params=p, u=rng.random(b).astype(np.float32))
    g = assert_parity(gpu_ctx, w, cap=512)
    _say("one-slice nuclei: %s paths %s" % (g["n_cand"].tolist(), g["path"].tolist()))
    assert (g["path"] == api.PATH_SORTED).any() and (g["path"] == api.PATH_NUCLEUS).any()


def test_plan_with_logits_of_extreme_magnitude(gpu_ctx):
    """The second pass plans a top_k == 0 row from counts of its logits by weight octave.  Logits so large that the
    octave arithmetic saturates (everything lands in one bin, or far outside the bins), tiny ones (a near-flat row
    inside a single bin), infinities and temperatures at the ends of the server's range still give the reference's
    tokens: the plan only sizes the work, the weights decide."""
    rng = np.random.default_rng(90210)
    b, v = 12, 40000
    base = rng.standard_normal((b, v)).astype(np.float32)
    scales = np.array([1e9, 1e7, 1e5, 3e3, 1e-3, 1e-6, 1e-30, 3.0, 3.0, 3.0, 1e4, 1e-2], np.float32)
    logits = (base * scales[:, None]).astype(np.float32)
    logits[7, ::3] = -np.inf
    logits[8, 5] = np.inf
    logits[9] += np.float32(3e38)  # (+inf wherever the sum overflows)
    p = api.make_params(b, 1.0, 0, 0.9)
    p["temperature"] = np.array([1.0, 100.0, 1.0, 1.0, 1.0, 1e-3, 1.0, 0.5, 0.7, 1.0, 1e-3, 100.0], np.float32)
    p["top_p"] = np.array([0.9, 0.5, 0.99, 0.9, 0.9, 0.9, 0.95, 0.9, 0.9, 0.9, 0.9, 0.999], np.float32)
    w = dict(name="extreme_magnitudes", logits=logits, params=p, u=rng.random(b).astype(np.float32))
    g = assert_parity(gpu_ctx, w, cap=256)
    _say("extreme magnitudes: nuclei %s paths %s" % (g["n_cand"].tolist(), g["path"].tolist()))


def test_plans_hold_for_top_p_close_to_one(gpu_ctx):
    """The second pass's plan keeps what its coarse counts say the nucleus needs, with a margin on the mass that may be
    left out.  For top_p up to 0.9999 and temperatures from 0.3 to 3 on Gaussian, spiked and near-flat rows the kept
    list must reach the nucleus' end: every row is finished from the sorted list or the candidate lists, none by the
    whole-row path."""
    rng = np.random.default_rng(2718)
    b, v = 24, 129280
    logits = (rng.standard_normal((b, v)) * 3).astype(np.float32)
    logits[8:16] = (logits[8:16] * 0.03).astype(np.float32)  # near-flat
    for r in range(16, 24):  # spikes
        logits[r, rng.integers(0, v, 1 + r)] += np.float32(8.0)
    p = api.make_params(b, 1.0, 0, 0.9)
    p["temperature"] = np.tile(np.array([0.3, 0.7, 1.0, 1.3, 2.0, 3.0, 1.0, 0.5], np.float32), 3)
    p["top_p"] = np.tile(np.array([0.9999, 0.999, 0.99, 0.9999, 0.95, 0.9999, 0.999, 0.9], np.float32), 3)
    w = dict(name="top_p_near_one", logits=logits, params=p, u=rng.random(b).astype(np.float32))
    g = assert_parity(gpu_ctx, w, cap=256)
    _say("top_p near one: nuclei %s paths %s" % (g["n_cand"].tolist(), g["path"].tolist()))
    assert not (g["path"] == api.PATH_GENERAL).any()


@pytest.mark.parametrize("v", [257, 4099, 20000])
def test_shares_hold_what_their_bins_promise(v):
    """The workers' shares get room for the logits their bins count (plus 1/64 and 64 entries).  Quantised logits
    (thousands of equal weights per bin), near-flat rows of small vocabularies (where the slack is most of the row)
    and logits far from zero (coarse float spacing) must not outgrow it: every top_k == 0 row takes the sorted list or
    the candidate lists, none the whole-row path."""
    rng = np.random.default_rng(4000 + v)
    b = 70
    logits = (rng.standard_normal((b, v)) * 3).astype(np.float32)
    logits[:24] = (np.round(logits[:24] * 4) / 4).astype(np.float32)       # quantised: many equal weights
    logits[24:40] = (logits[24:40] * 0.007).astype(np.float32)             # near-flat
    logits[40:48] += np.float32(1000.0)                                    # coarse float spacing
    logits[48:56] -= np.float32(50.0)
    p = api.make_params(b, 1.0, 0, 0.9)
    p["temperature"] = np.tile(np.array([2.0, 0.5, 1.0, 2.0, 0.3, 2.0, 1.3], np.float32), 10)
    p["top_p"] = np.tile(np.array([0.999, 0.99, 0.9, 0.5, 0.95], np.float32), 14)
    w = dict(name="shares_v%d" % v, logits=logits, params=p, u=rng.random(b).astype(np.float32))
    w["hist"] = rng.integers(0, v, (b, 300)).astype(np.int32)
    w["hist_len"] = rng.integers(0, 301, b).astype(np.uint32)
    ctx = api.SamplerContext(max_rows=b, max_vocab=v, max_hist=300)
    try:
        g = assert_parity(ctx, w, cap=128)
        _say("shares v=%d paths %s" % (v, np.bincount(g["path"], minlength=8).tolist()))
        assert not (g["path"] == api.PATH_GENERAL).any()
    finally:
        ctx.close()


def test_big_batches_with_few_top_p_rows(gpu_ctx):
    """Batches of more than 64 rows share the second pass's workgroups by the number of top_k == 0 rows: one round of
    single pieces while they fit, else a few workgroups per row that take their pieces in turn."""
    v = 40000
    for b, n_nucleus in ((100, 5), (100, 60), (200, 200), (70, 1)):
        rng = np.random.default_rng(7000 + b + n_nucleus)
        w = _random_case(rng, v, b)
        w["params"]["temperature"] = np.float32(0.9)
        w["params"]["top_p"] = np.float32(0.97)
        w["params"]["top_k"] = np.uint32(30)
        w["params"]["top_k"][rng.permutation(b)[:n_nucleus]] = 0
        _say("big batch b=%d nucleus rows=%d" % (b, n_nucleus))
        ctx = api.SamplerContext(max_rows=b, max_vocab=v, max_hist=1024)
        try:
            assert_parity(ctx, w, cap=256)
        finally:
            ctx.close()


@pytest.mark.parametrize("v", [40000, 129280])
def test_second_pass_piece_sizes(gpu_ctx, v):
    """The second pass over top_k == 0 rows is cut into pieces of one to four 4096-logit blocks depending on how many
    such rows the batch has: every cut gives the same tokens, totals and candidate lists."""
    rng = np.random.default_rng(600 + v)
    b = 64
    for n_nucleus in (1, 5, 8, 16, 21, 33, 64):
        w = _random_case(rng, v, b)
        w["params"]["temperature"] = np.float32(0.9)
        w["params"]["top_p"] = np.float32(0.93)
        w["params"]["top_k"] = np.uint32(40)
        w["params"]["top_k"][rng.permutation(b)[:n_nucleus]] = 0
        _say("piece sizes v=%d nucleus rows=%d" % (v, n_nucleus))
        assert_parity(gpu_ctx, w, cap=256)


def test_nucleus_sizes_around_path_boundaries(gpu_ctx):
    """Nuclei just below and above the sizes at which the sorted tail changes its route (one wave up to 256 entries,
    total and walk from LDS up to 1024; a walk that ends within the 8192 entries staged in LDS goes entry by entry,
    group maps beyond), each drawn at the first entry, deep inside and at the very end."""
    v = 129280
    rng = np.random.default_rng(2024)
    targets = [200, 256, 257, 300, 1000, 1024, 1025, 1100, 2040, 2048, 2049, 2100, 4096, 5000, 8100, 8192, 8193, 8300,
               9000, 16500, 20000]
    us = [0.0, 1e-7, 0.3, 0.9, 0.97, 0.99999994]
    base = -np.arange(v, dtype=np.float64) * 2e-4  # distinct, slowly falling weights
    q = np.exp(base)
    csum = np.cumsum(q)
    rows = [(t, u) for t in targets for u in us]
    b = len(rows)
    logits = np.empty((b, v), np.float32)
    p = api.make_params(b, 1.0, 0, 0.5)
    uu = np.empty(b, np.float32)
    for r, (t, u) in enumerate(rows):
        logits[r] = base.astype(np.float32)[rng.permutation(v)]
        p["top_p"][r] = np.float32((csum[t - 1] - 0.25 * q[t - 1]) / csum[-1])  # the nucleus ends at entry t or next to it
        uu[r] = u
    w = dict(name="path_boundaries", logits=logits, params=p, u=uu)
    g = assert_parity(gpu_ctx, w, cap=64)
    sizes = sorted(set(int(x) for x in g["n_cand"]))
    _say("nucleus sizes: %s" % sizes)
    assert min(sizes) <= 256 and any(256 < x <= 1024 for x in sizes) and any(1024 < x <= 8192 for x in sizes) \
        and any(x > 8192 for x in sizes)


def test_host_parameter_copy_only_skips_work(gpu_ctx):
    """With the host copy of the parameters the call leaves out kernels no row needs: the results are those of the
    full pipeline and of the oracle, for batches without top_k == 0 rows (where a tied or overflowing top-k row
    then takes the whole-row path inside plan_kernel), without any sampled row, with whole-row rows only, and mixed."""
    rng = np.random.default_rng(77001)
    v, b = 20000, 32
    for case in range(8):
        w = _random_case(rng, v, b)
        p = w["params"]
        if case < 3:  # top-k rows only (plus greedy ones), ties and overflows included by the generator
            p["top_k"] = rng.choice(np.array([1, 3, 20, 50, 100, 128], np.uint32), b)
            p["top_p"] = rng.choice(np.array([0.999, 0.95, 0.5], np.float32), b)
            if case == 2:
                w["logits"] = np.round(w["logits"]).astype(np.float32)  # heavy ties: uncertifiable candidate lists
        elif case == 3:
            p["temperature"] = np.float32(0.0)  # greedy only
        elif case == 4:  # whole-row rows only: top_k beyond the fast path
            p["top_k"] = np.uint32(5000)
            p["top_p"] = np.float32(0.97)
            p["temperature"] = np.float32(0.9)
        elif case == 5:  # top-k alone: whole-row rows in nth_element's order
            p["top_k"] = rng.choice(np.array([3, 40, 1000], np.uint32), b)
            p["top_p"] = np.float32(1.0)
            p["temperature"] = np.float32(0.9)
        _say("host parameter copy case %d" % case)
        kw = dict(mask=w.get("mask"), hist=w.get("hist"), hist_len=w.get("hist_len"), cand_cap=64)
        full = api.sample(gpu_ctx, w["logits"], p, w["u"], **kw)
        lean = api.sample(gpu_ctx, w["logits"], p, w["u"], params_host=True, **kw)
        for key in ("tokens", "n_cand", "cand_idx"):
            assert np.array_equal(full[key], lean[key]), (case, key)
        # (rows in token order: the whole-row path without the host copy, kernels of their own with it)
        lean_path = np.where(lean["path"] == api.PATH_INDEXED, api.PATH_GENERAL, lean["path"])
        assert np.array_equal(full["path"], lean_path), (case, "path")
        assert np.array_equal(full["total"].view(np.uint32), lean["total"].view(np.uint32)), case
        ref = oracle_rows(w)
        assert [t for t, _ in ref] == [int(t) for t in lean["tokens"]], case


def test_more_rows_than_threads():
    """1100 rows in one batch: the per-workgroup search for its piece of work loops over the rows."""
    ctx = api.SamplerContext(max_rows=1100, max_vocab=320, max_hist=0)
    try:
        rng = np.random.default_rng(4545)
        w = _random_case(rng, 320, 1100)
        w.pop("hist", None)
        w.pop("hist_len", None)
        assert_parity(ctx, w, cap=64)
    finally:
        ctx.close()


def test_full_size_properties(gpu_ctx):
    """Size-independent properties at the full benchmark sizes (B=256, V=151552), no oracle:
    ids inside the allowed set, greedy rows equal numpy's first argmax, u=0 returns the most likely candidate,
    and the same batch twice gives the same ids."""
    w = workloads.config4()
    g1 = gpu_rows(gpu_ctx, w)
    g2 = gpu_rows(gpu_ctx, w)
    assert np.array_equal(g1["tokens"], g2["tokens"])
    assert ((g1["tokens"] >= 0) & (g1["tokens"] < w["logits"].shape[1])).all()
    w0 = dict(w, u=np.zeros(256, np.float32))
    g0 = gpu_rows(gpu_ctx, w0)
    assert np.array_equal(g0["tokens"], w["logits"].argmax(axis=1))
    wg = dict(w, params=api.make_params(256, 0.0))
    gg = gpu_rows(gpu_ctx, wg)
    assert np.array_equal(gg["tokens"], w["logits"].argmax(axis=1))
    w5 = workloads.config5(density=0.01)
    g5 = gpu_rows(gpu_ctx, w5)
    t = g5["tokens"]
    allowed = (w5["mask"][np.arange(256), t >> 5] >> (t & 31).astype(np.uint32)) & 1
    assert allowed.all()


def test_argument_errors(gpu_ctx):
    """n_vocab == 0 is the reference's std::invalid_argument (src/gen/sampler.cpp:11-12); other bad arguments too."""
    b = api.Batch(SAMPLER_TEST_LOGITS, api.make_params(1), np.zeros(1, np.float32))
    d = b.desc
    d.n_vocab = 0
    with pytest.raises(api.MakoError, match="empty vocabulary"):
        gpu_ctx.sample_batch(d)
    d.n_vocab = 8
    d.out_tokens = None
    with pytest.raises(api.MakoError):
        gpu_ctx.sample_batch(d)
    d.out_tokens = b.o_tokens.ptr
    d.n_rows = 100000
    with pytest.raises(api.MakoError, match="exceeds"):
        gpu_ctx.sample_batch(d)


def test_host_call_argument_errors(gpu_ctx):
    """The host-pointer call refuses strides that do not cover a row and history lengths beyond the stride (the
    staging rows' further columns hold older calls' ids) instead of sampling from them."""
    v, rows = 4096, 2
    w = workloads.config1(rows=rows, vocab=v)
    lg = np.ascontiguousarray(w["logits"], np.float32)
    pr = np.ascontiguousarray(w["params"])
    uu = np.ascontiguousarray(w["u"], np.float32)
    hist = np.zeros((rows, 8), np.int32)
    mask = np.full((rows, v // 32), 0xffffffff, np.uint32)
    tok = np.zeros(rows, np.int32)

    def call(logits_stride=v, mask_stride=v // 32, hlen=(8, 8)):
        hl = np.array(hlen, np.uint32)
        return gpu_ctx.lib.mako_sampler_sample_host(
            gpu_ctx.ptr, lg.ctypes.data, logits_stride, rows, v, pr.ctypes.data, uu.ctypes.data, mask.ctypes.data,
            mask_stride, hist.ctypes.data, None, 8, hl.ctypes.data, None, None, None, tok.ctypes.data)

    assert call() == api.MAKO_OK
    good = tok.copy()
    assert call(logits_stride=v - 1) == api.MAKO_ERR_INVALID_ARG and "logits_stride" in gpu_ctx.last_error()
    assert call(mask_stride=v // 32 - 1) == api.MAKO_ERR_INVALID_ARG and "mask_stride" in gpu_ctx.last_error()
    assert call(hlen=(8, 9)) == api.MAKO_ERR_INVALID_ARG and "hist_len" in gpu_ctx.last_error()
    assert call() == api.MAKO_OK and np.array_equal(tok, good)


def _topp_order_rows():
    """The rows of tests/golden/topp_order_cases.json: on each the ORDER of the reference's fp64 additions decides the
    nucleus (its sequential total and the exact total put top_p * total on different sides of a sorted prefix sum)."""
    import json
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    import make_topp_order_cases as gen
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "topp_order_cases.json")) as f:
        cases = json.load(f)["cases"]
    logits = np.stack([gen.make_row(c["seed"], c["tiny_level"])[0] for c in cases])
    p = api.make_params(len(cases), 1.0, 0, 0.9)
    p["top_p"] = np.array([c["top_p_bits"] for c in cases], np.uint32).view(np.float32)
    u = np.random.default_rng(77).random(len(cases)).astype(np.float32)
    return dict(name="topp_order", logits=logits, params=p, u=u), cases


def test_top_p_cut_follows_the_reference_addition_order(gpu_ctx):
    """Twenty rows found by CPU brute force (tests/golden/make_topp_order_cases.py) whose nucleus has one entry more
    or fewer depending on whether the fp64 total is added up one weight after the other in index order, as the
    reference does (src/gen/sampler.cpp:46-48), or exactly: the device path must land on the reference's side."""
    w, cases = _topp_order_rows()
    g = assert_parity(gpu_ctx, w, cap=64)
    assert [int(n) for n in g["n_cand"]] == [c["n_reference"] for c in cases]
    assert all(c["n_reference"] != c["n_exact_total"] for c in cases)
    # and as top-k + top-p rows over the same weights (top_k beyond the fast path: the whole-row path, where the
    # reference's total runs over the top_k survivors in the order nth_element leaves them)
    w["params"]["top_k"] = 60000
    assert_parity(gpu_ctx, w, cap=64)


def test_nucleus_longer_than_the_group_records():
    """A top-p row whose nucleus has more entries than the workers' group records hold (256 x 992): it takes the
    whole-row path, in the last launch."""
    v = 300000
    rng = np.random.default_rng(4242)
    logits = (rng.standard_normal((2, v)) * 0.05).astype(np.float32)
    p = api.make_params(2, 1.0, 0, 0.99)
    w = dict(name="long_nucleus", logits=logits, params=p, u=np.array([0.3, 0.97], np.float32))
    ctx = api.SamplerContext(max_rows=2, max_vocab=v, max_hist=0)
    try:
        g = assert_parity(ctx, w, cap=256)
        assert (g["n_cand"] > 256 * 992).all()
        assert (g["path"] == api.PATH_GENERAL).all()
    finally:
        ctx.close()
