"""ctypes binding of libelmo_xmc.so (declarations: include/elmo_xmc.h).  There is no fallback: if the
library has not been built, or a call fails, an exception is raised."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libelmo_xmc.so")

ROUND_MODES = {"rtn": 0, "sr_philox": 1, "sr_fast": 2}

_lib = None


class XmcError(RuntimeError):
    pass


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise XmcError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(hipcc --offload-arch=gfx950); there is no CPU fallback for the classifier step")
    # A library that predates an edit of the sources would run the old kernels.  build() leaves the digest of the sources
    # beside the library; it is compared BEFORE the library is loaded, because a loaded library cannot be replaced within
    # the process (loading the same path again returns the mapping that is already there).  On a mismatch the library
    # is rebuilt under a temporary name and moved into place, then loaded.
    from . import build as _build
    if LIB_PATH == _build.OUT and _build.built_hash() != _build.source_hash():
        try:
            _build.build()
        except Exception as e:
            raise XmcError(f"{LIB_PATH} was built from other sources than those in the tree and could not be rebuilt: {e}")
    lib = ctypes.CDLL(LIB_PATH)
    lib.xmc_source_hash.restype = ctypes.c_char_p
    if LIB_PATH == _build.OUT and lib.xmc_source_hash().decode() != _build.source_hash():
        raise XmcError(f"{LIB_PATH} reports other sources than those in the tree: rebuild it "
                       "(python -c 'import __graft_entry__ as g; g.build()') and start the process again")
    vp, i32, f32, sz, ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t, ctypes.c_longlong
    lib.xmc_version.restype = i32
    lib.xmc_source_hash.restype = ctypes.c_char_p
    lib.xmc_error_string.restype = ctypes.c_char_p
    lib.xmc_error_string.argtypes = [i32]
    lib.xmc_workspace_bytes.restype = sz
    lib.xmc_workspace_bytes.argtypes = [i32, i32]
    lib.xmc_fp8_step.restype = i32
    lib.xmc_fp8_step.argtypes = [ctypes.POINTER(vp), i32, i32, vp, i32, i32, vp, i32, f32,
                                 ctypes.POINTER(ctypes.c_uint32), i32, f32, f32, vp, vp, vp, sz, vp]
    lib.xmc_fp8_step_ex.restype = i32
    lib.xmc_fp8_step_ex.argtypes = [ctypes.POINTER(vp), i32, i32, vp, i32, i32, vp, i32, f32,
                                    ctypes.POINTER(ctypes.c_uint32), i32, f32, f32, f32, f32, ctypes.c_ulonglong, vp, vp, vp, sz, vp]
    lib.xmc_fp8_kahan_step.restype = i32
    lib.xmc_fp8_kahan_step.argtypes = [ctypes.POINTER(vp), i32, i32, vp, i32, i32, vp, i32, f32,
                                       ctypes.POINTER(ctypes.c_uint32), i32, vp, i32, i32, vp, vp, vp, sz, vp]
    lib.xmc_fp8_forward.restype = i32
    lib.xmc_fp8_forward.argtypes = [ctypes.POINTER(vp), i32, i32, vp, i32, i32, f32, f32, vp, ll, ll, vp, sz, vp]
    lib.xmc_fp8_forward_static.restype = i32
    lib.xmc_fp8_forward_static.argtypes = [ctypes.POINTER(vp), i32, i32, vp, i32, i32, f32, f32, vp, ll, ll, vp]
    lib.xmc_step_error_word.restype = i32
    lib.xmc_step_error_word.argtypes = [vp, i32, i32, vp]
    lib.xmc_tiled_workspace_bytes.restype = sz
    lib.xmc_tiled_workspace_bytes.argtypes = [i32, i32, i32]
    lib.xmc_debug_spin_limit.restype = i32
    lib.xmc_debug_spin_limit.argtypes = [i32]
    lib.xmc_tiled_workspace_bytes_ex.restype = sz
    lib.xmc_tiled_workspace_bytes_ex.argtypes = [i32, i32, i32, i32]
    lib.xmc_tiled_step.restype = i32
    lib.xmc_tiled_step.argtypes = [ctypes.POINTER(vp), i32, i32, i32, i32, vp, i32, i32, vp, i32, f32,
                                   ctypes.POINTER(ctypes.c_uint32), i32, i32, i32, vp, i32, i32, vp, vp, vp, vp, sz, vp]
    lib.xmc_tiled_step_ex.restype = i32
    lib.xmc_tiled_step_ex.argtypes = [ctypes.POINTER(vp), i32, i32, i32, i32, vp, i32, i32, vp, i32, f32,
                                      ctypes.POINTER(ctypes.c_uint32), i32, i32, i32, vp, i32, i32, f32, f32, ctypes.c_ulonglong,
                                      vp, vp, vp, vp, sz, vp]
    lib.xmc_topk_scratch_bytes.restype = sz
    lib.xmc_topk_scratch_bytes.argtypes = [i32]
    lib.xmc_fp8_forward_topk.restype = i32
    lib.xmc_fp8_forward_topk.argtypes = [ctypes.POINTER(vp), i32, i32, vp, i32, i32, f32, f32, ctypes.c_longlong, i32, vp, vp,
                                         vp, sz, vp, sz, vp]
    lib.xmc_topk_fused_scratch_bytes.restype = sz
    lib.xmc_topk_fused_scratch_bytes.argtypes = []
    lib.xmc_fp8_forward_topk_fused.restype = i32
    lib.xmc_fp8_forward_topk_fused.argtypes = [ctypes.POINTER(vp), i32, i32, vp, i32, i32, f32, f32, ctypes.c_longlong, i32, vp,
                                               vp, i32, vp, sz, vp, sz, vp, vp]
    lib.xmc_dropout_quantize.restype = i32
    lib.xmc_dropout_quantize.argtypes = [vp, i32, i32, i32, f32, ctypes.c_ulonglong, vp, vp]
    lib.xmc_step_error_offset.restype = sz
    lib.xmc_step_sticky_error_offset.restype = sz
    lib.xmc_step_workgroups.restype = i32
    lib.xmc_step_xcc_ids.restype = i32
    lib.xmc_step_xcc_ids.argtypes = [vp, ctypes.POINTER(ctypes.c_int32), i32, vp]
    lib.xmc_quad_placement_check.restype = i32
    lib.xmc_quad_placement_check.argtypes = [ctypes.POINTER(ctypes.c_int32), i32]
    lib.xmc_copy_probe.restype = i32
    lib.xmc_copy_probe.argtypes = [vp, vp, sz, vp]
    lib.xmc_profile_events.restype = i32
    lib.xmc_profile_events.argtypes = [vp, vp]
    _lib = lib
    return lib


XMC_ERR_RANGE = -4


def check(status, what):
    if status != 0:
        msg = load().xmc_error_string(status).decode()
        raise XmcError(f"{what} failed: {msg} (status {status})")
