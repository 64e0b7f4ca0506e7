"""ctypes bindings for the CPU oracle and the compiled reference -- TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the bench's CPU-baseline leg may import this
module.  `oracle` wraps oracle/liboracle.so (the plain-C restatement);
`reference()` wraps oracle/_ref/libmako_ref.so (the unmodified reference sampler
compiled by oracle/Makefile) and returns None where that file was not built.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


class Params(C.Structure):
    # SamplingParams, src/gen/sampler.hpp:11-20
    _fields_ = [
        ("temperature", C.c_float),
        ("top_k", C.c_uint32),
        ("top_p", C.c_float),
        ("min_p", C.c_float),
        ("presence_penalty", C.c_float),
        ("frequency_penalty", C.c_float),
        ("repetition_penalty", C.c_float),
    ]


PARAMS_DTYPE = np.dtype(
    [
        ("temperature", "<f4"),
        ("top_k", "<u4"),
        ("top_p", "<f4"),
        ("min_p", "<f4"),
        ("presence_penalty", "<f4"),
        ("frequency_penalty", "<f4"),
        ("repetition_penalty", "<f4"),
    ]
)


def make_params(temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, presence_penalty=0.0, frequency_penalty=0.0,
                repetition_penalty=1.0):
    return Params(temperature, top_k, top_p, min_p, presence_penalty, frequency_penalty, repetition_penalty)


def params_from_record(rec):
    return Params(*(rec[n].item() for n in PARAMS_DTYPE.names))


class Trace(C.Structure):
    _fields_ = [
        ("n_cand", C.c_uint32),
        ("total", C.c_float),
        ("q_chosen", C.c_float),
        ("max_logit", C.c_float),
        ("cap", C.c_uint32),
        ("cand_idx", C.POINTER(C.c_int32)),
        ("cand_q", C.POINTER(C.c_float)),
    ]


def build(force=False):
    """Compile the oracle (and the reference where /root/reference is mounted)."""
    if force or not os.path.exists(os.path.join(_HERE, "liboracle.so")):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True)


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _ip(a):
    return a.ctypes.data_as(C.POINTER(C.c_int32))


def _up(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint32))


class _Oracle:
    def __init__(self):
        build()
        self.lib = lib = C.CDLL(os.path.join(_HERE, "liboracle.so"))
        lib.or_expf.restype = C.c_float
        lib.or_expf.argtypes = [C.c_float]
        lib.or_expf_array.restype = None
        lib.or_expf_array.argtypes = [C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_size_t]
        lib.or_uniforms.argtypes = [C.c_uint64, C.c_uint32, C.POINTER(C.c_float)]
        lib.or_sample.restype = C.c_int32
        lib.or_sample.argtypes = [C.POINTER(C.c_float), C.c_uint32, C.POINTER(Params), C.POINTER(C.c_int32),
                                  C.c_uint32, C.POINTER(C.c_uint32), C.c_float, C.c_int, C.POINTER(Trace)]
        lib.or_verify.restype = C.c_int32
        lib.or_verify.argtypes = [C.POINTER(C.c_float), C.c_uint32, C.POINTER(Params), C.POINTER(C.c_int32),
                                  C.c_uint32, C.POINTER(C.c_uint32), C.c_int32, C.c_float, C.c_float, C.c_int,
                                  C.POINTER(C.c_int), C.POINTER(Trace)]
        lib.or_nth_element.argtypes = [C.POINTER(C.c_float), C.POINTER(C.c_int32), C.c_uint32, C.c_uint32]
        lib.or_debug_heap_selects.restype = C.c_long
        lib.or_close_forced.restype = C.c_int32
        lib.or_close_forced.argtypes = [C.POINTER(C.c_float), C.c_uint32, C.POINTER(C.c_uint32), C.c_int32, C.c_uint32,
                                        C.POINTER(C.c_uint32)]

    def close_forced(self, logits, think_end, max_above=3, mask=None):
        """(token or -1, logits strictly above logits[think_end]) -- ReasoningBudget::forced's last-stretch test."""
        logits = np.ascontiguousarray(logits, np.float32)
        m = np.ascontiguousarray(mask, np.uint32) if mask is not None else None
        above = C.c_uint32()
        t = self.lib.or_close_forced(_fp(logits), logits.shape[0], _up(m) if m is not None else None, int(think_end),
                                     int(max_above), C.byref(above))
        return int(t), int(above.value)

    def heap_selects(self):
        return self.lib.or_debug_heap_selects()

    def expf(self, x):
        return self.lib.or_expf(float(x))

    def expf_array(self, x):
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty_like(x)
        self.lib.or_expf_array(_fp(x), _fp(y), x.size)
        return y

    def uniforms(self, seed, n):
        out = np.empty(n, np.float32)
        self.lib.or_uniforms(seed, n, _fp(out))
        return out

    def _args(self, logits, hist, mask):
        logits = np.ascontiguousarray(logits, np.float32)
        hist = np.ascontiguousarray(hist if hist is not None else [], np.int32)
        maskp = None
        if mask is not None:
            mask = np.ascontiguousarray(mask, np.uint32)
            maskp = _up(mask)
        return logits, hist, mask, maskp

    def sample(self, logits, params, u, hist=None, mask=None, order_mode=0, cap=0):
        """Returns (token, dict trace)."""
        logits, hist, mask, maskp = self._args(logits, hist, mask)
        tr = Trace()
        ci = np.zeros(max(cap, 1), np.int32)
        cq = np.zeros(max(cap, 1), np.float32)
        tr.cap, tr.cand_idx, tr.cand_q = cap, _ip(ci), _fp(cq)
        t = self.lib.or_sample(_fp(logits), logits.size, C.byref(params), _ip(hist), hist.size, maskp,
                               C.c_float(u), order_mode, C.byref(tr))
        n = min(cap, tr.n_cand)
        return t, dict(n_cand=tr.n_cand, total=np.float32(tr.total), q_chosen=np.float32(tr.q_chosen),
                       max_logit=np.float32(tr.max_logit), cand_idx=ci[:n].copy(), cand_q=cq[:n].copy())

    def verify(self, logits, params, draft, u1, u2, hist=None, mask=None, order_mode=0):
        logits, hist, mask, maskp = self._args(logits, hist, mask)
        acc = C.c_int(0)
        t = self.lib.or_verify(_fp(logits), logits.size, C.byref(params), _ip(hist), hist.size, maskp, draft,
                               C.c_float(u1), C.c_float(u2), order_mode, C.byref(acc), None)
        return t, bool(acc.value)

    def nth_element(self, q, idx, nth):
        q = np.array(q, np.float32)
        idx = np.array(idx, np.int32)
        self.lib.or_nth_element(_fp(q), _ip(idx), q.size, nth)
        return q, idx


class _Reference:
    def __init__(self, path):
        self.lib = lib = C.CDLL(path)
        lib.ref_uniforms.argtypes = [C.c_uint64, C.c_uint32, C.POINTER(C.c_float)]
        lib.ref_sample.restype = C.c_int32
        lib.ref_sample.argtypes = [C.POINTER(C.c_float), C.c_uint32, C.POINTER(Params), C.POINTER(C.c_int32),
                                   C.c_uint32, C.POINTER(C.c_uint32), C.c_uint64, C.POINTER(C.c_uint32),
                                   C.POINTER(C.c_int32), C.POINTER(C.c_float), C.c_uint32]
        lib.ref_verify.restype = C.c_int32
        lib.ref_verify.argtypes = [C.POINTER(C.c_float), C.c_uint32, C.POINTER(Params), C.POINTER(C.c_int32),
                                   C.c_uint32, C.POINTER(C.c_uint32), C.c_uint64, C.c_int32, C.POINTER(C.c_int)]
        lib.ref_nth_element.argtypes = [C.POINTER(C.c_float), C.POINTER(C.c_int32), C.c_uint32, C.c_uint32]
        lib.ref_make_nth_killer.restype = C.c_long
        lib.ref_make_nth_killer.argtypes = [C.c_uint32, C.c_uint32, C.POINTER(C.c_float)]
        lib.ref_libm_expf.restype = C.c_float
        lib.ref_libm_expf.argtypes = [C.c_float]
        lib.ref_sample_batch_timed.restype = C.c_double
        lib.ref_sample_batch_timed.argtypes = [C.POINTER(C.c_float), C.c_int64, C.c_uint32, C.c_uint32, C.c_void_p,
                                               C.POINTER(C.c_int32), C.c_int64, C.POINTER(C.c_uint32),
                                               C.POINTER(C.c_uint32), C.c_int64, C.POINTER(C.c_uint64), C.c_uint32,
                                               C.POINTER(C.c_int32)]

    def uniforms(self, seed, n):
        out = np.empty(n, np.float32)
        self.lib.ref_uniforms(seed, n, _fp(out))
        return out

    def sample(self, logits, params, seed, hist=None, mask=None, cap=0):
        logits = np.ascontiguousarray(logits, np.float32)
        hist = np.ascontiguousarray(hist if hist is not None else [], np.int32)
        maskp = None
        if mask is not None:
            mask = np.ascontiguousarray(mask, np.uint32)
            maskp = _up(mask)
        n = C.c_uint32(0)
        ci = np.zeros(max(cap, 1), np.int32)
        cq = np.zeros(max(cap, 1), np.float32)
        t = self.lib.ref_sample(_fp(logits), logits.size, C.byref(params), _ip(hist), hist.size, maskp, seed,
                                C.byref(n), _ip(ci), _fp(cq), cap)
        k = min(cap, n.value)
        return t, dict(n_cand=n.value, cand_idx=ci[:k].copy(), cand_q=cq[:k].copy())

    def verify(self, logits, params, seed, draft, hist=None, mask=None):
        logits = np.ascontiguousarray(logits, np.float32)
        hist = np.ascontiguousarray(hist if hist is not None else [], np.int32)
        maskp = None
        if mask is not None:
            mask = np.ascontiguousarray(mask, np.uint32)
            maskp = _up(mask)
        acc = C.c_int(0)
        t = self.lib.ref_verify(_fp(logits), logits.size, C.byref(params), _ip(hist), hist.size, maskp, seed, draft,
                                C.byref(acc))
        return t, bool(acc.value)

    def nth_element(self, q, idx, nth):
        q = np.array(q, np.float32)
        idx = np.array(idx, np.int32)
        self.lib.ref_nth_element(_fp(q), _ip(idx), q.size, nth)
        return q, idx

    def make_nth_killer(self, n, nth):
        q = np.zeros(n, np.float32)
        ncmp = self.lib.ref_make_nth_killer(n, nth, _fp(q))
        return q, ncmp

    def libm_expf(self, x):
        return self.lib.ref_libm_expf(float(x))

    def sample_batch_timed(self, logits, params, seeds, hist=None, hist_len=None, mask=None, n_threads=1):
        """logits [B,V] f32, params PARAMS_DTYPE[B], seeds u64[B]; returns (seconds, tokens)."""
        logits = np.ascontiguousarray(logits, np.float32)
        b, v = logits.shape
        params = np.ascontiguousarray(params, PARAMS_DTYPE)
        seeds = np.ascontiguousarray(seeds, np.uint64)
        out = np.zeros(b, np.int32)
        hp = hl = mp = None
        hs = ms = 0
        if hist is not None:
            hist = np.ascontiguousarray(hist, np.int32)
            hist_len = np.ascontiguousarray(hist_len, np.uint32)
            hp, hl, hs = _ip(hist), _up(hist_len), hist.shape[1]
        if mask is not None:
            mask = np.ascontiguousarray(mask, np.uint32)
            mp, ms = _up(mask), mask.shape[1]
        secs = self.lib.ref_sample_batch_timed(_fp(logits), v, b, v, params.ctypes.data, hp, hs, hl, mp, ms,
                                               seeds.ctypes.data_as(C.POINTER(C.c_uint64)), n_threads, _ip(out))
        return secs, out


_oracle = None
_reference = False


def oracle():
    global _oracle
    if _oracle is None:
        _oracle = _Oracle()
    return _oracle


def reference():
    global _reference
    if _reference is False:
        path = os.path.join(_HERE, "_ref", "libmako_ref.so")
        _reference = _Reference(path) if os.path.exists(path) else None
    return _reference
