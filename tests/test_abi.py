"""The C-ABI library loads and exports every function include/mako_sampler.h declares (no GPU needed)."""
import ctypes
import os
import re

from mako_amd import api

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "mako_sampler.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mako_sampler_\w+)\s*\(", text)))


def test_exports_match_header():
    lib = api.load()
    names = declared_functions()
    assert set(names) == set(api.EXPORTS), names
    for n in names:
        assert hasattr(lib, n), n


def test_host_only_entry_points():
    lib = api.load()
    assert lib.mako_sampler_slices(129280) == 8 and lib.mako_sampler_slices(151552) == 10
    assert lib.mako_sampler_slices(1) == 1
    assert lib.mako_sampler_last_error(None) == b"null context"
    assert lib.mako_sampler_create(None, 0, 1, 1, 0) == api.MAKO_ERR_INVALID_ARG
    p = ctypes.c_void_p()
    assert lib.mako_sampler_create(ctypes.byref(p), 0, 0, 8, 0) == api.MAKO_ERR_INVALID_ARG
    # more rows than the kernels' grids can index (two workgroups per row in a y dimension of at most 65535), and a
    # vocabulary of more than 64 slices: refused before anything is allocated
    assert lib.mako_sampler_create(ctypes.byref(p), 0, 32768, 8, 0) == api.MAKO_ERR_INVALID_ARG
    assert lib.mako_sampler_create(ctypes.byref(p), 0, 1, 64 * 16384 + 1, 0) == api.MAKO_ERR_INVALID_ARG


def test_params_layout():
    assert api.PARAMS_DTYPE.itemsize == 28  # mako_sampling_params, src/gen/sampler.hpp:11-20
