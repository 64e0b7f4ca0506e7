#!/usr/bin/env python3
"""Headline benchmark: sampled rows/s of the HIP sampler on the decode batch B=64 x V=129280 fp32
(penalties over 2048-token histories, per-row temperature / top-k / top-p), one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload config3|config4|config5|config1|config2b|config1_topk_alone|topk_alone_64|temperature_only_1|temperature_only_64|temperature_only_256]

A step is one batch through the whole sampling pipeline with every input already resident in HBM.
The logits are rotated through a pool of copies larger than the 256 MB Infinity Cache so each step
reads them from HBM.  Prints one JSON line; `roofline` prices the batch's algorithmic bytes against the
HBM peak using HIP-event time on the launch stream, `cpu_baseline` is the reference CPU sampler timed
on this host on the same rows.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per batch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by what the same counters read
# for a device-to-device copy of known size: records written by mako_amd/traffic_record.py, each tied to the kernel
# sources it was measured on (null is reported once they have changed)
TRAFFIC_RECORDS = {"config3": os.path.join(ROOT, "profiles", "config3_hbm_traffic.json")}


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return None


def make_workload(name):
    from mako_amd import workloads
    if name == "config1":
        return workloads.config1()
    if name == "config1_topk_alone":  # config 1 without top-p: the survivors stay in nth_element's order
        w = workloads.config1()
        w["params"]["top_p"] = np.float32(1.0)
        w["name"] = name
        return w
    if name == "topk_alone_64":  # 64 such rows
        w = workloads.config1(rows=64)
        w["params"]["top_p"] = np.float32(1.0)
        w["name"] = name
        return w
    if name in ("temperature_only_1", "temperature_only_64", "temperature_only_256"):  # rows with neither top-k nor top-p: the whole vocabulary in token order
        w = workloads.config1(rows=int(name.rsplit("_", 1)[1]))
        w["params"]["top_p"] = np.float32(1.0)
        w["params"]["top_k"] = np.uint32(0)
        w["name"] = name
        return w
    if name == "config2b":
        return workloads.config2()
    if name == "config3":
        return workloads.config3()
    if name == "config4":
        return workloads.config4()
    if name == "config5":
        return workloads.config5(density=0.5)
    raise SystemExit("unknown workload " + name)


def cpu_baseline(w, budget_s):
    """The reference CPU sampler (or, if it was not built, the oracle port) on this host's cores."""
    from oracle import pyoracle
    ref = pyoracle.reference()
    rows = w["logits"].shape[0]
    cores = os.cpu_count() or 1
    if ref is not None:
        kw = dict(hist=w.get("hist"), hist_len=w.get("hist_len"), mask=w.get("mask"))
        t1, tok = ref.sample_batch_timed(w["logits"], w["params"], w["seeds"], n_threads=1, **kw)
        reps, spent, wall = 0, 0.0, 0.0
        while spent < budget_s and reps < 50:
            t0 = time.perf_counter()
            ref.sample_batch_timed(w["logits"], w["params"], w["seeds"], n_threads=cores, **kw)
            wall += time.perf_counter() - t0
            spent += wall / (reps + 1)
            reps += 1
        return dict(value=rows * reps / wall, unit="rows/s", cores=cores, cpu_model=cpu_model(), kind="reference",
                    value_1thread=rows / t1,
                    sample="%d x the %d-row %s batch, one fresh Sampler per row, sample() only (history replay and "
                           "thread start included in the %d-thread wall time)" % (reps, rows, w["name"], cores)), tok
    o = pyoracle.oracle()
    t0 = time.perf_counter()
    tok = []
    n = min(rows, 16)
    for r in range(n):
        p = pyoracle.params_from_record(w["params"][r])
        hist = w["hist"][r, : w["hist_len"][r]] if "hist" in w else None
        tok.append(o.sample(w["logits"][r], p, float(w["u"][r]), hist, w["mask"][r] if "mask" in w else None)[0])
    dt = time.perf_counter() - t0
    return dict(value=n / dt, unit="rows/s", cores=1, cpu_model=cpu_model(), kind="port",
                sample="first %d rows of the %s batch through the plain-C oracle" % (n, w["name"])), None


def time_other(w, steps, warmup, pool_mb, orc, stream):
    """One more workload through the same timed loop: ms per batch, rows/s, roofline fraction, parity with the reference."""
    from mako_amd import api, hip, workloads
    from oracle import pyoracle
    rows, vocab = w["logits"].shape
    w["u"] = np.array([orc.uniforms(int(s), 1)[0] for s in w["seeds"]], np.float32)
    ctx = api.SamplerContext(max_rows=rows, max_vocab=vocab, max_hist=w["hist"].shape[1] if "hist" in w else 0)
    batch = api.Batch(w["logits"], w["params"], w["u"], mask=w.get("mask"), hist=w.get("hist"),
                      hist_len=w.get("hist_len"), diagnostics=False, params_host=True)
    n_copies = max(2, -(-pool_mb * (1 << 20) // (rows * vocab * 4)))
    pool = [batch.d_logits] + [hip.DeviceArray.from_host(w["logits"]) for _ in range(n_copies - 1)]

    def step(i):
        batch.desc.logits = pool[i % n_copies].ptr
        ctx.sample_batch(batch.desc, stream, params_host=batch.params_host)

    for i in range(warmup):
        step(i)
    stream.synchronize()
    e0, e1 = hip.Event(), hip.Event()
    e0.record(stream)
    for i in range(steps):
        step(warmup + i)
    e1.record(stream)
    e1.synchronize()
    ms = e0.elapsed_ms(e1) / steps
    tokens = batch.o_tokens.download()
    ctx.set_profile(True)
    split = np.zeros(api.SAMPLER_KERNELS)
    for i in range(min(steps, 10)):
        step(warmup + steps + i)
        split += np.array(ctx.kernel_times_ms())
    split /= min(steps, 10)
    ctx.close()
    mism = None
    ref = pyoracle.reference()
    if ref is not None:
        kw = dict(hist=w.get("hist"), hist_len=w.get("hist_len"), mask=w.get("mask"))
        _, tok = ref.sample_batch_timed(w["logits"], w["params"], w["seeds"], n_threads=os.cpu_count() or 1, **kw)
        mism = int((np.asarray(tok) != tokens).sum())
    nbytes = rows * workloads.bytes_per_row(w)
    gbs = nbytes / (ms * 1e-3) / 1e9
    return dict(workload="%s: B=%d x V=%d" % (w["name"], rows, vocab), steps=steps, ms_per_batch=ms,
                rows_per_s=rows / (ms * 1e-3), bytes_per_batch=nbytes, achieved_gbs=gbs, roofline_frac=gbs / HBM_PEAK_GBS,
                kernel_ms=dict(zip(["scan_kernel", "finish_or_plan_kernel", "sort_kernel", "tail_kernel"],
                                   [float(x) for x in split])),
                parity_mismatches=mism)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--workload", default="config3")
    ap.add_argument("--pool-mb", type=int, default=640, help="rotate the logits through this many MB of copies")
    ap.add_argument("--cpu-seconds", type=float, default=10.0, help="budget of the CPU baseline leg (0 = skip)")
    ap.add_argument("--host-pointer-calls", type=int, default=5,
                    help="also time this many calls of the host-pointer entry point (PCIe-inclusive rate; 0 = skip)")
    ap.add_argument("--overlap-steps", type=int, default=400,
                    help="batches of the several-contexts-on-their-own-streams measurement (0 = skip)")
    ap.add_argument("--other-steps", type=int, default=20,
                    help="with the default workload: also time configs 4 and 5 for this many batches each and report "
                         "them under other_configs (0 = skip)")
    ap.add_argument("--calibrate-copy-mb", type=int, default=0,
                    help="also run one device-to-device copy of this many MB (a kernel of known traffic, to scale "
                         "rocprofv3's FETCH_SIZE / WRITE_SIZE counters by)")
    a = ap.parse_args()
    if a.gpus != 1:
        raise SystemExit("bench.py measures one GPU: rows are independent, so a multi-GPU run is a plain split of "
                         "the batch by rows with nothing exchanged; run with --gpus 1")

    from mako_amd import api, hip, workloads
    from oracle import pyoracle
    if hip.device_count() < 1:
        raise SystemExit("bench.py needs an MI355X")
    hip.set_device(0)

    w = make_workload(a.workload)
    rows, vocab = w["logits"].shape
    # the uniforms a reference Sampler seeded with seeds[r] would draw, so both sides consume the same u
    orc = pyoracle.oracle()
    w["u"] = np.array([orc.uniforms(int(s), 1)[0] for s in w["seeds"]], np.float32)

    ctx = api.SamplerContext(max_rows=rows, max_vocab=vocab, max_hist=w["hist"].shape[1] if "hist" in w else 0)
    # (the host copy of the parameters goes along, as a serving loop that built them on the host would pass it)
    batch = api.Batch(w["logits"], w["params"], w["u"], mask=w.get("mask"), hist=w.get("hist"),
                      hist_len=w.get("hist_len"), diagnostics=False, params_host=True)
    row_bytes = workloads.bytes_per_row(w)
    batch_bytes = rows * row_bytes
    n_copies = max(2, -(-a.pool_mb * (1 << 20) // (rows * vocab * 4)))
    pool = [batch.d_logits] + [hip.DeviceArray.from_host(w["logits"]) for _ in range(n_copies - 1)]
    stream = hip.Stream()

    def step(i):
        batch.desc.logits = pool[i % n_copies].ptr
        ctx.sample_batch(batch.desc, stream, params_host=batch.params_host)

    if a.calibrate_copy_mb:
        n = a.calibrate_copy_mb << 20
        src, dst = hip.DeviceArray((n,), np.uint8), hip.DeviceArray((n,), np.uint8)
        hip.check(hip.lib().hipMemcpy(dst.ptr, src.ptr, n, hip.hipMemcpyDeviceToDevice), "hipMemcpy D2D")
        hip.synchronize()
    for i in range(a.warmup):
        step(i)
    stream.synchronize()
    hip.synchronize()
    e0, e1 = hip.Event(), hip.Event()
    t0 = time.perf_counter()
    e0.record(stream)
    for i in range(a.steps):
        step(a.warmup + i)
    e1.record(stream)
    e1.synchronize()
    hip.synchronize()
    wall = time.perf_counter() - t0
    ms = e0.elapsed_ms(e1)
    ms_per_step = ms / a.steps
    tokens = batch.o_tokens.download()

    # per-kernel split of a batch: HIP events recorded by the library on the launch stream, a few extra steps
    ctx.set_profile(True)
    split = np.zeros(api.SAMPLER_KERNELS)
    n_split = min(a.steps, 50)
    for i in range(n_split):
        step(a.warmup + a.steps + i)
        split += np.array(ctx.kernel_times_ms())
    split /= n_split
    ctx.set_profile(False)

    # several contexts, each with its own stream and scratch, taking turns (independent decode batches in flight, as
    # a server with several model replicas' or micro-batches' logits would have): the stages of one batch are latency-
    # bound and leave most CUs idle, so batches overlap.  Reported beside the headline value, never as it.
    overlapped = None
    if a.overlap_steps > 0:
        overlapped = {}
        lanes = [(ctx, batch, stream)]
        for n_ctx in (2, 4):
            while len(lanes) < n_ctx:
                lanes.append((api.SamplerContext(max_rows=rows, max_vocab=vocab,
                                                 max_hist=w["hist"].shape[1] if "hist" in w else 0),
                              api.Batch(w["logits"], w["params"], w["u"], mask=w.get("mask"), hist=w.get("hist"),
                                        hist_len=w.get("hist_len"), diagnostics=False, params_host=True),
                              hip.Stream()))

            def step_n(i):
                c, b, st = lanes[i % n_ctx]
                b.desc.logits = pool[i % n_copies].ptr
                c.sample_batch(b.desc, st, params_host=b.params_host)

            for i in range(n_ctx * a.warmup):
                step_n(i)
            for _, _, st in lanes:
                st.synchronize()
            t0 = time.perf_counter()
            for i in range(a.overlap_steps):
                step_n(i)
            for _, _, st in lanes:
                st.synchronize()
            overlapped["%d_contexts_rows_per_s" % n_ctx] = rows * a.overlap_steps / (time.perf_counter() - t0)
            for _, b, _ in lanes:
                if not np.array_equal(b.o_tokens.download(), tokens):
                    raise SystemExit("overlapped batches disagree with the serial ones")
        for c, _, _ in lanes[1:]:
            c.close()

    # the host-pointer entry point on the same batch (logits staged over PCIe inside the call): reported beside the
    # headline value, never as it
    host_rate = None
    if a.host_pointer_calls > 0:
        tok_h = np.zeros(rows, np.int32)
        hist = np.ascontiguousarray(w["hist"], np.int32) if "hist" in w else None
        hlen = np.ascontiguousarray(w["hist_len"], np.uint32) if "hist" in w else None
        mask = np.ascontiguousarray(w["mask"], np.uint32) if "mask" in w else None
        lg = np.ascontiguousarray(w["logits"], np.float32)
        pr = np.ascontiguousarray(w["params"])
        uu = np.ascontiguousarray(w["u"], np.float32)

        def host_call():
            rc = ctx.lib.mako_sampler_sample_host(
                ctx.ptr, lg.ctypes.data, vocab, rows, vocab, pr.ctypes.data, uu.ctypes.data,
                mask.ctypes.data if mask is not None else None, mask.shape[1] if mask is not None else 0,
                hist.ctypes.data if hist is not None else None, None, hist.shape[1] if hist is not None else 0,
                hlen.ctypes.data if hlen is not None else None, None, None, None, tok_h.ctypes.data)
            if rc != 0:
                raise SystemExit("mako_sampler_sample_host failed: %s" % ctx.last_error())

        host_call()
        t0 = time.perf_counter()
        for _ in range(a.host_pointer_calls):
            host_call()
        host_rate = rows * a.host_pointer_calls / (time.perf_counter() - t0)
        if not np.array_equal(tok_h, tokens):
            raise SystemExit("host-pointer call disagrees with the device-pointer call")

    base, ref_tok = (None, None)
    if a.cpu_seconds > 0:
        base, ref_tok = cpu_baseline(w, a.cpu_seconds)
    parity = None
    if ref_tok is not None:
        parity = dict(rows=rows, mismatches=int((np.asarray(ref_tok) != tokens).sum()), against="reference sampler")

    # BASELINE's two 256-row configurations, event-timed on the same stream with the logits rotated the same way and
    # their tokens checked against the reference CPU sampler (untimed): beside the headline value, never part of it.
    # (And a batch of rows with a temperature only, what an API request without top_k / top_p asks for, and one of rows
    # cut to a top-k without a top-p, whose survivors keep nth_element's order: no BASELINE configurations, but the
    # kinds of row that take kernels of their own and the whole-row path.)
    others = None
    if a.workload == "config3" and a.other_steps > 0:
        others = {}
        ctx.close()
        for key, name in (("config4", "config4"), ("config5_0.5", "config5"), ("temperature_only_64", "temperature_only_64"),
                          ("topk_alone_64", "topk_alone_64")):
            others[key] = time_other(make_workload(name), a.other_steps, max(2, a.other_steps // 4), a.pool_mb, orc, stream)

    achieved = batch_bytes / (ms_per_step * 1e-3) / 1e9
    from mako_amd import traffic_record
    traffic = traffic_record.load_record(TRAFFIC_RECORDS[a.workload], a.workload) if a.workload in TRAFFIC_RECORDS else None
    out = {
        "metric": "sampled rows/sec at B=64xV=129280 fp32; achieved HBM GB/s vs peak",
        "value": rows * a.steps / (ms * 1e-3),
        "unit": "rows/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "%s: B=%d x V=%d fp32, full penalty + top-k + top-p pipeline" % (w["name"], rows, vocab),
                   "rows": rows, "vocab": vocab, "logit_copies_rotated": n_copies,
                   "host_wall_ms_per_step": wall * 1e3 / a.steps},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "bytes_per_launch": batch_bytes,
                     "kernel": "scan + finish + sort + tail kernels (the four launches of one batch)",
                     "launch_ms": ms_per_step,
                     "kernel_ms": dict(zip(["scan_kernel", "finish_kernel", "sort_kernel", "tail_kernel"],
                                           [float(x) for x in split])),
                     "scan_kernel_gbs": batch_bytes / (split[0] * 1e-3) / 1e9},
        "host_pointer_rows_per_s": host_rate,
        "overlapped_batches": overlapped,
        "other_configs": others,
        "cpu_baseline": base,
        "parity": parity,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
