"""ctypes binding of include/mako_sampler.h plus a small batched front end.

The sampler itself is the HIP library; this module only moves pointers.  It
raises if libmako_sampler.so is missing -- there is no CPU fallback.
"""
import ctypes as C
import os

import numpy as np

from . import hip

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmako_sampler.so")

MAKO_OK = 0
MAKO_ERR_INVALID_ARG = -1
MAKO_ERR_HIP = -2
SAMPLER_KERNELS = 4  # MAKO_SAMPLER_KERNELS
PATH_GREEDY, PATH_FALLBACK, PATH_TOPK, PATH_NUCLEUS, PATH_GENERAL, PATH_FORCED, PATH_SORTED, PATH_SUMMED, PATH_INDEXED = 1, 2, 3, 4, 5, 6, 7, 8, 9
FORCED_NONE, FORCED_TOKEN, FORCED_CLOSE = 0, 1, 2

# mako_sampling_params / SamplingParams (src/gen/sampler.hpp:11-20)
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


def make_params(n, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, presence_penalty=0.0, frequency_penalty=0.0,
                repetition_penalty=1.0):
    """n rows of SamplingParams with the reference's defaults; arguments broadcast."""
    p = np.zeros(n, PARAMS_DTYPE)
    p["temperature"] = temperature
    p["top_k"] = top_k
    p["top_p"] = top_p
    p["min_p"] = min_p
    p["presence_penalty"] = presence_penalty
    p["frequency_penalty"] = frequency_penalty
    p["repetition_penalty"] = repetition_penalty
    return p


class Desc(C.Structure):
    _fields_ = [
        ("logits", C.c_void_p),
        ("logits_stride", C.c_int64),
        ("n_rows", C.c_uint32),
        ("n_vocab", C.c_uint32),
        ("params", C.c_void_p),
        ("u", C.c_void_p),
        ("mask", C.c_void_p),
        ("mask_stride", C.c_int64),
        ("hist_tokens", C.c_void_p),
        ("hist_counts", C.c_void_p),
        ("hist_stride", C.c_int64),
        ("hist_len", C.c_void_p),
        ("draft", C.c_void_p),
        ("u2", C.c_void_p),
        ("out_accepted", C.c_void_p),
        ("out_tokens", C.c_void_p),
        ("out_n_cand", C.c_void_p),
        ("out_total", C.c_void_p),
        ("out_q", C.c_void_p),
        ("out_path", C.c_void_p),
        ("out_cand_idx", C.c_void_p),
        ("out_cand_q", C.c_void_p),
        ("cand_cap", C.c_uint32),
        ("force_token", C.c_void_p),
        ("close_token", C.c_void_p),
        ("close_max_above", C.c_uint32),
        ("out_forced", C.c_void_p),
        ("out_above", C.c_void_p),
        ("append_history", C.c_uint32),
    ]


STATIC_MAX_ROWS, STATIC_MAX_VOCAB = 16, 131072  # MAKO_STATIC_MAX_ROWS, MAKO_STATIC_MAX_VOCAB

EXPORTS = [
    "mako_sampler_create",
    "mako_sampler_destroy",
    "mako_sampler_sample_batch",
    "mako_sampler_sample_batch_hinted",
    "mako_sampler_sample_batch_static",
    "mako_sampler_sample_host",
    "mako_sampler_last_error",
    "mako_sampler_slices",
    "mako_sampler_set_profile",
    "mako_sampler_kernel_times",
    "mako_sampler_debug_expf",
    "mako_sampler_debug_div",
    "mako_sampler_debug_checks",
]

_libs = {}
# the library with the kernels' index checks compiled in (mako_amd/build.py, checked=True): tests only
CHECKED_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmako_sampler_checked.so")
# the checked library whose plans for large batches leave shares unsorted that they should not (rash=True): tests only
RASH_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libmako_sampler_rash.so")


def load(path=None):
    """The C-ABI library (LIB_PATH unless another build of it is named), loaded once per path."""
    path = path or LIB_PATH
    if path not in _libs:
        if not os.path.exists(path):
            raise RuntimeError("%s is not built: run `python -m mako_amd.build` (needs hipcc)" % os.path.basename(path))
        lib = C.CDLL(path)
        lib.mako_sampler_create.argtypes = [C.POINTER(C.c_void_p), C.c_int, C.c_uint32, C.c_uint32, C.c_uint32]
        lib.mako_sampler_destroy.argtypes = [C.c_void_p]
        lib.mako_sampler_sample_batch.argtypes = [C.c_void_p, C.POINTER(Desc), C.c_void_p]
        lib.mako_sampler_sample_batch_hinted.argtypes = [C.c_void_p, C.POINTER(Desc), C.c_void_p, C.c_void_p]
        lib.mako_sampler_sample_batch_static.argtypes = [C.c_void_p, C.POINTER(Desc), C.c_void_p]
        lib.mako_sampler_last_error.restype = C.c_char_p
        lib.mako_sampler_last_error.argtypes = [C.c_void_p]
        lib.mako_sampler_set_profile.argtypes = [C.c_void_p, C.c_int]
        lib.mako_sampler_kernel_times.argtypes = [C.c_void_p, C.POINTER(C.c_float)]
        lib.mako_sampler_slices.restype = C.c_uint32
        lib.mako_sampler_slices.argtypes = [C.c_uint32]
        lib.mako_sampler_debug_expf.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p]
        lib.mako_sampler_debug_div.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p]
        lib.mako_sampler_sample_host.argtypes = [
            C.c_void_p, C.c_void_p, C.c_int64, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
            C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        lib.mako_sampler_debug_checks.argtypes = [C.c_void_p, C.POINTER(C.c_uint32)]
        _libs[path] = lib
    return _libs[path]


class MakoError(RuntimeError):
    pass


class SamplerContext:
    """Owner of a mako_sampler_ctx."""

    def __init__(self, max_rows, max_vocab, max_hist=0, device=0, lib_path=None):
        self.lib = load(lib_path)
        p = C.c_void_p()
        rc = self.lib.mako_sampler_create(C.byref(p), device, max_rows, max_vocab, max_hist)
        self.ptr = p.value
        if rc != MAKO_OK:
            msg = self.lib.mako_sampler_last_error(self.ptr).decode() if self.ptr else "invalid argument"
            self.close()
            raise MakoError("mako_sampler_create: %d %s" % (rc, msg))
        self.max_rows, self.max_vocab, self.max_hist = max_rows, max_vocab, max_hist

    def close(self):
        if getattr(self, "ptr", None):
            self.lib.mako_sampler_destroy(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def last_error(self):
        return self.lib.mako_sampler_last_error(self.ptr).decode()

    def failed_checks(self):
        """Bit set of the index checks that failed since the last call (always 0 unless the library is the checked build)."""
        bits = C.c_uint32(0)
        rc = self.lib.mako_sampler_debug_checks(self.ptr, C.byref(bits))
        if rc != MAKO_OK:
            raise MakoError("mako_sampler_debug_checks: %d %s" % (rc, self.last_error()))
        return int(bits.value)

    def set_profile(self, enabled):
        rc = self.lib.mako_sampler_set_profile(self.ptr, 1 if enabled else 0)
        if rc != MAKO_OK:
            raise MakoError("mako_sampler_set_profile: %d %s" % (rc, self.last_error()))

    def kernel_times_ms(self):
        """(scan, finish, sort, tail) kernel milliseconds of the last batch sampled while profiling was on."""
        out = (C.c_float * SAMPLER_KERNELS)()
        rc = self.lib.mako_sampler_kernel_times(self.ptr, out)
        if rc != MAKO_OK:
            raise MakoError("mako_sampler_kernel_times: %d %s" % (rc, self.last_error()))
        return [float(x) for x in out]

    def sample_batch(self, desc, stream=None, params_host=None):
        """Enqueues one batch.  params_host: address of a host copy of the rows' parameters (Batch.params_host),
        with which the library leaves out the kernels no row needs."""
        if params_host:
            rc = self.lib.mako_sampler_sample_batch_hinted(self.ptr, C.byref(desc), params_host,
                                                           stream.ptr if stream else None)
        else:
            rc = self.lib.mako_sampler_sample_batch(self.ptr, C.byref(desc), stream.ptr if stream else None)
        if rc != MAKO_OK:
            raise MakoError("mako_sampler_sample_batch: %d %s" % (rc, self.last_error()))

    def sample_batch_static(self, desc, stream=None):
        """mako_sampler_sample_batch_static: the same batch on the library's own scratch memory (STATIC_MAX_ROWS x
        STATIC_MAX_VOCAB at most); allocates nothing."""
        rc = self.lib.mako_sampler_sample_batch_static(self.ptr, C.byref(desc), stream.ptr if stream else None)
        if rc != MAKO_OK:
            raise MakoError("mako_sampler_sample_batch_static: %d %s" % (rc, self.last_error()))


class Batch:
    """Device-resident inputs and outputs of one batch, built from host arrays."""

    def __init__(self, logits, params, u, mask=None, hist=None, hist_len=None, hist_counts=None, draft=None, u2=None,
                 cand_cap=0, diagnostics=True, force_token=None, close_token=None, close_max_above=3,
                 append_history=False, params_host=False):
        logits = np.ascontiguousarray(logits, np.float32)
        self.n_rows, self.n_vocab = logits.shape
        b = self.n_rows
        self.keep = []
        d = Desc()
        self.d_logits = self._up(logits)
        d.logits, d.logits_stride = self.d_logits.ptr, self.n_vocab
        d.n_rows, d.n_vocab = b, self.n_vocab
        self.h_params = np.ascontiguousarray(params, PARAMS_DTYPE)
        d.params = self._up(self.h_params).ptr
        # the host copy's address, for the library to leave out kernels that have no work (None: not offered)
        self.params_host = self.h_params.ctypes.data if params_host else None
        self.d_u = self._up(np.ascontiguousarray(u, np.float32))
        d.u = self.d_u.ptr
        if mask is not None:
            mask = np.ascontiguousarray(mask, np.uint32)
            d.mask, d.mask_stride = self._up(mask).ptr, mask.shape[1]
        if hist is not None:
            hist = np.ascontiguousarray(hist, np.int32)
            if hist_len is None:
                hist_len = np.full(b, hist.shape[1], np.uint32)
            self.d_hist = self._up(hist)
            self.d_hist_len = self._up(np.ascontiguousarray(hist_len, np.uint32))
            d.hist_tokens, d.hist_stride = self.d_hist.ptr, hist.shape[1]
            d.hist_len = self.d_hist_len.ptr
            if hist_counts is not None:
                d.hist_counts = self._up(np.ascontiguousarray(hist_counts, np.uint32)).ptr
        if draft is not None:
            d.draft = self._up(np.ascontiguousarray(draft, np.int32)).ptr
            d.u2 = self._up(np.ascontiguousarray(u2, np.float32)).ptr
            self.o_acc = self._new((b,), np.uint8)
            d.out_accepted = self.o_acc.ptr
        self.o_tokens = self._new((b,), np.int32)
        d.out_tokens = self.o_tokens.ptr
        self.diagnostics = diagnostics
        if diagnostics:
            self.o_n = self._new((b,), np.uint32)
            self.o_total = self._new((b,), np.float32)
            self.o_q = self._new((b,), np.float32)
            self.o_path = self._new((b,), np.uint8)
            d.out_n_cand, d.out_total, d.out_q, d.out_path = self.o_n.ptr, self.o_total.ptr, self.o_q.ptr, self.o_path.ptr
        self.hooks = force_token is not None or close_token is not None
        if force_token is not None:
            self.d_force = self._up(np.ascontiguousarray(force_token, np.int32))
            d.force_token = self.d_force.ptr
        if close_token is not None:
            d.close_token = self._up(np.ascontiguousarray(close_token, np.int32)).ptr
            d.close_max_above = close_max_above
            self.o_above = self._new((b,), np.uint32)
            d.out_above = self.o_above.ptr
        if self.hooks:
            self.o_forced = self._new((b,), np.uint8)
            d.out_forced = self.o_forced.ptr
        d.append_history = 1 if append_history else 0
        self.cand_cap = cand_cap
        if cand_cap:
            self.o_ci = self._new((b, cand_cap), np.int32)
            self.o_cq = self._new((b, cand_cap), np.float32)
            d.out_cand_idx, d.out_cand_q, d.cand_cap = self.o_ci.ptr, self.o_cq.ptr, cand_cap
        self.desc = d

    def _up(self, a):
        x = hip.DeviceArray.from_host(a)
        self.keep.append(x)
        return x

    def _new(self, shape, dtype):
        x = hip.DeviceArray(shape, dtype)
        x.zero()
        self.keep.append(x)
        return x

    def results(self):
        hip.synchronize()
        r = dict(tokens=self.o_tokens.download())
        if self.diagnostics:
            r.update(n_cand=self.o_n.download(), total=self.o_total.download(), q=self.o_q.download(),
                     path=self.o_path.download())
        if self.cand_cap:
            r.update(cand_idx=self.o_ci.download(), cand_q=self.o_cq.download())
        if hasattr(self, "o_acc"):
            r["accepted"] = self.o_acc.download()
        if self.hooks:
            r["forced"] = self.o_forced.download()
        if hasattr(self, "o_above"):
            r["above"] = self.o_above.download()
        return r

    def history(self):
        """(tokens, lengths) of the device-resident histories, as append_history leaves them."""
        hip.synchronize()
        return self.d_hist.download(), self.d_hist_len.download()


def sample(ctx, logits, params, u, **kw):
    """One batch through the device path from host arrays; returns a dict of host arrays."""
    b = Batch(logits, params, u, **kw)
    ctx.sample_batch(b.desc, params_host=b.params_host)
    return b.results()
