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
            "xmc_step_error_word", "xmc_debug_spin_limit", "xmc_profile_events", "xmc_copy_probe", "xmc_step_error_offset", "xmc_step_sticky_error_offset", "xmc_fp8_step_ex", "xmc_fp8_kahan_step", "xmc_tiled_step_ex", "xmc_step_workgroups", "xmc_step_xcc_ids", "xmc_quad_placement_check", "xmc_fp8_forward_static", "xmc_tiled_step", "xmc_tiled_workspace_bytes", "xmc_tiled_workspace_bytes_ex", "xmc_fp8_forward_topk", "xmc_topk_scratch_bytes", "xmc_fp8_forward_topk_fused", "xmc_topk_fused_scratch_bytes", "xmc_dropout_quantize"} <= set(names)
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
    assert a > b > 34 * 2 ** 20 and a % 256 == 0       # grad_X partials (24 MiB) and the G exchange ring (10 MiB) dominate
    assert a < 40 * 2 ** 20
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


def test_quad_placement_comparison():
    """The comparison the device makes at the end of every fused step (the four workgroups of a quad must have recorded
    one XCC id), on the host: the placement the kernel assumes passes, any member elsewhere is counted."""
    lib = _lib.load()
    n = 256
    ids = (ctypes.c_int32 * n)(*[g % 8 for g in range(n)])             # workgroup g on XCD g % 8
    assert lib.xmc_quad_placement_check(ids, n) == 0
    ids[8 * 5 + 3] = 4                                                 # workgroup 43 = member 1 of quad 8*1+3 ran on XCD 4
    assert lib.xmc_quad_placement_check(ids, n) == 1
    ids2 = (ctypes.c_int32 * n)(*[(g // 4) % 8 for g in range(n)])     # four consecutive workgroups per XCD: every quad is split
    assert lib.xmc_quad_placement_check(ids2, n) == n // 4
    ids3 = (ctypes.c_int32 * n)(*[(g + 3) % 8 for g in range(n)])      # a rotated but consistent placement is fine
    assert lib.xmc_quad_placement_check(ids3, n) == 0
    assert lib.xmc_quad_placement_check(None, n) == -1
    assert lib.xmc_quad_placement_check(ids, 40) == -4
    assert lib.xmc_step_error_offset() % 4 == 0


def test_static_forward_rejects_bad_arguments_before_touching_the_device():
    lib = _lib.load()
    P = 0x7F0000001000
    arr = (ctypes.c_void_p * 1)(P)
    call = lambda **k: lib.xmc_fp8_forward_static(k.get("arr", arr), k.get("nc", 1), k.get("rows", 64), k.get("x", P), k.get("batch", 16),
                                                  k.get("feat", 768), 1.0, 1.0, P, 64, 64, None)
    assert call(arr=None) == -1 and call(x=None) == -1
    assert call(batch=144) == -2 and call(batch=8) == -2 and call(feat=1024) == -2 and call(rows=40) == -2
    assert call(nc=65) == -4
    assert call(x=P + 2) == -3


def test_two_pass_topk_rejects_bad_arguments_before_touching_the_device():
    lib = _lib.load()
    need = lib.xmc_topk_fused_scratch_bytes()
    assert 0 < need < 1000000                       # group maxima, bounds, counts, 1,024 candidates per row
    P = 0x7F0000001000
    arr = (ctypes.c_void_p * 1)(P)
    wsb = lib.xmc_workspace_bytes(1, 1 << 20)

    def call(**k):
        return lib.xmc_fp8_forward_topk_fused(k.get("arr", arr), 1, k.get("rows", 1 << 20), P, 16, k.get("feat", 768), 1.0, 1.0,
                                              k.get("labels", 1 << 20), k.get("k", 100), P, k.get("idx", P), k.get("i64", 0), P, k.get("wsb", wsb),
                                              k.get("scratch", P), k.get("sb", need), k.get("status", P), None)
    assert call(arr=None) == -1 and call(scratch=None) == -1 and call(status=None) == -1
    assert call(feat=1024) == -2 and call(k=0) == -2 and call(k=129) == -2 and call(labels=(1 << 20) + 1) == -2
    assert call(scratch=P + 16) == -3 and call(status=P + 2) == -3
    assert call(idx=P + 4, i64=1) == -3 and call(idx=P + 4, i64=0) != -3 and call(idx=P + 2) == -3
    assert call(sb=need - 1) == -5 and call(wsb=wsb - 1) == -5
    # too few labels for a bound from sampled tiles: fewer than 4 k tiles of 32 labels
    assert call(labels=12000, k=100) == -4 and call(labels=600, k=5) == -4


def test_dropout_quantize_rejects_bad_arguments_before_touching_the_device():
    lib = _lib.load()
    P = 0x7F0000001000
    call = lambda **k: lib.xmc_dropout_quantize(k.get("x", P), k.get("t", 0), k.get("rows", 16), k.get("cols", 768), k.get("p", 0.1), 40,
                                                k.get("out", P), None)
    assert call(x=None) == -1 and call(out=None) == -1
    assert call(t=2) == -6
    assert call(cols=770) == -2 and call(rows=0) == -2 and call(p=1.0) == -2 and call(p=-0.1) == -2
    assert call(rows=1 << 22, cols=1024) == -4
    assert call(x=P + 4) == -3 and call(x=P + 4, t=1) != -3 and call(out=P + 2) == -3


def test_three_kernel_path_accepts_label_spaces_of_2_24_and_more():
    """The sort key keeps 24 bits for the label; the three-kernel path takes larger label spaces in segments of whole
    chunks, so 64 chunks of 262,272 rows (16,785,408 labels) pass the range check and fail only on the workspace size
    given here (no device is touched).  A single chunk of 2^24 rows, and the fused path at this size, are refused."""
    lib = _lib.load()
    P = 0x10000
    nc, rows = 64, 262272
    assert nc * rows >= 1 << 24
    arr = (ctypes.c_void_p * nc)(*([P] * nc))

    def tiled(nc_, rows_, wsb):
        return lib.xmc_tiled_step(arr, nc_, rows_, rows_, 0, P, 32, 768, P, 4, 0.05, None, 0, 1, 1, None, 0, 0, P, None, None,
                                  P, wsb, None)

    assert tiled(nc, rows, 1024) == -5            # XMC_ERR_WORKSPACE: the label count itself is accepted
    assert tiled(1, 1 << 24, 1 << 40) == -4       # one chunk must stay below 2^24 rows
    sarr = (ctypes.c_uint32 * nc)(*([0] * nc))
    assert lib.xmc_fp8_step(arr, nc, rows, P, 32, 768, P, 4, 0.05, sarr, 0, 1.0, 1.0, P, None, P, 1 << 40, None) == -4
