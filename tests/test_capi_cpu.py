"""The shared library loads without a GPU, exports every function include/elmo_xmc.h declares, and rejects bad
arguments with the documented status codes before touching the device (no kernel is launched here)."""
import ctypes
import os
import re

import pytest

from elmo_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "elmo_xmc.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xmc_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    lib = _lib.load()
    names = declared_functions()
    assert {"xmc_version", "xmc_error_string", "xmc_workspace_bytes", "xmc_fp8_step", "xmc_fp8_forward",
            "xmc_step_error_word", "xmc_profile_events", "xmc_copy_probe", "xmc_select_step_kernel", "xmc_tiled_step", "xmc_tiled_workspace_bytes", "xmc_fp8_forward_topk", "xmc_topk_scratch_bytes"} <= set(names)
    for n in names:
        assert hasattr(lib, n), n


def test_library_was_built_from_the_sources_in_the_tree():
    """The GPU runs load the library that is in the tree: one that predates an edit of the sources would test and
    measure the old kernels.  The library carries a digest of the sources it was compiled from."""
    from elmo_amd import build
    built_from = _lib.load().xmc_source_hash().decode()
    assert built_from == build.source_hash(), "the sources changed after the library was built: rebuild it"


def test_version_and_error_strings():
    lib = _lib.load()
    assert lib.xmc_version() >= 1
    assert lib.xmc_error_string(0) == b"ok"
    for code in range(-8, 0):
        assert len(lib.xmc_error_string(code)) > 3
    assert lib.xmc_error_string(-99) == b"unknown status"


def test_workspace_bytes():
    lib = _lib.load()
    a = lib.xmc_workspace_bytes(11, 60928)
    b = lib.xmc_workspace_bytes(2, 64)
    assert a > b > 50 * 2 ** 20 and a % 256 == 0       # grad_X partials dominate: about 50 MiB
    assert a < 80 * 2 ** 20
    assert lib.xmc_workspace_bytes(0, 64) == 0 and lib.xmc_workspace_bytes(65, 64) == 0 and lib.xmc_workspace_bytes(2, 0) == 0


def _call_step(lib, chunk_ptrs, nc, rows, x, batch, feat, labels, nnz, seeds, mode, sw, sx, gout, ws, wsb):
    arr = (ctypes.c_void_p * max(nc, 1))(*chunk_ptrs) if chunk_ptrs is not None else None
    sarr = (ctypes.c_uint32 * max(nc, 1))(*seeds) if seeds is not None else None
    return lib.xmc_fp8_step(arr, nc, rows, x, batch, feat, labels, nnz, 0.05, sarr, mode, sw, sx, gout, None, ws, wsb, None)


def test_argument_validation_without_a_device():
    lib = _lib.load()
    P = 0x10000        # a plausible, aligned, never dereferenced address
    big = 1 << 30
    ok_args = dict(chunk_ptrs=[P, P], nc=2, rows=64, x=P, batch=16, feat=768, labels=P, nnz=4, seeds=[1, 2], mode=0,
                   sw=1.0, sx=1.0, gout=P, ws=P, wsb=big)

    def status(**kw):
        a = dict(ok_args); a.update(kw)
        return _call_step(lib, **a)

    assert status(chunk_ptrs=None) == -1
    assert status(x=None) == -1 and status(ws=None) == -1 and status(gout=None) == -1
    assert status(chunk_ptrs=[P, 0]) == -1
    assert status(feat=512) == -2 and status(batch=17) == -2 and status(batch=144) == -2 and status(batch=0) == -2
    assert status(rows=65) == -2 and status(rows=0) == -2
    assert status(nc=65, chunk_ptrs=[P] * 65, seeds=[0] * 65) == -4
    assert status(chunk_ptrs=[P, P + 4]) == -3 and status(x=P + 2) == -3 and status(ws=P + 16) == -3
    assert status(wsb=1024) == -5
    assert status(nnz=1 << 20) == -4 and status(nnz=-1) == -4
    assert status(mode=3) == -6 and status(mode=-1) == -6
    assert status(mode=2, seeds=None) == -1
    assert status(sw=0.0) == -2 and status(sx=-1.0) == -2
    assert status(labels=None, nnz=3) == -1
    assert status(labels=P + 4) == -3          # the (row, label) pairs are read whole: 8-byte alignment


def test_python_wrapper_raises_on_error_status():
    with pytest.raises(_lib.XmcError):
        _lib.check(-2, "xmc_fp8_step")
    _lib.check(0, "xmc_fp8_step")
