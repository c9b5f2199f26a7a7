"""ctypes binding of libncn_hip.so (C ABI declared in include/ncn_hip.h).

There is no CPU or PyTorch fallback.  A library that is missing, or was made from other sources than those beside it
(compared by content, see _build.py), is built on the spot with hipcc; if that cannot be done, loading raises.
"""
import ctypes
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libncn_hip.so")

NCN_F32, NCN_BF16, NCN_BF16X2 = 0, 1, 2
ACT_TANH, ACT_RELU, ACT_SIGMOID, ACT_LEAKY_RELU, ACT_LINEAR = 0, 1, 2, 3, -1

EXPORTS = ("ncn_forward", "ncn_backward", "ncn_inverse", "ncn_forward_indexed", "ncn_backward_indexed",
           "ncn_inverse_indexed", "ncn_inverse_ws", "ncn_forward_radix", "ncn_backward_radix", "ncn_inverse_radix", "ncn_plan_radix", "ncn_workspace_bytes", "ncn_workspace_bytes_stages",
           "ncn_plan_passes", "ncn_kernel_path",
           "ncn_check_shape", "ncn_error_string", "ncn_version", "ncn_backward_static", "ncn_static_scratch_bytes", "ncn_kernel_path_scalars",
           "ncn_build_id", "ncn_probe_issue", "ncn_probe_issue_info")


class NcnShape(ctypes.Structure):
    _fields_ = [("batch", ctypes.c_int64), ("N", ctypes.c_int64), ("E", ctypes.c_int64),
                ("n_head", ctypes.c_int32), ("n_cache", ctypes.c_int32)]


_lib = None


def _stale_reason():
    """Why the shared library has to be built before it can be loaded, or None.  Decided by content: the library carries
    a hash of the sources it was made from (ncn_build_id), compared here with the hash of the sources beside it.  File
    times play no part, so a copy or checkout that disturbs them changes nothing."""
    from . import _build
    if not os.path.exists(LIB_PATH):
        return "libncn_hip.so is missing"
    if not _build.have_sources():
        return None                       # an installed copy without sources: take the library as it is
    have, want = _build.library_build_id(LIB_PATH), _build.source_build_id()
    if have != want:
        return f"libncn_hip.so was built from other sources (build id {have}, sources {want})"
    return None


def load():
    """Load the shared library once and declare the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    reason = _stale_reason()
    if reason:
        import sys
        from . import _build
        if os.path.exists(LIB_PATH) and not _build.have_hipcc():
            print(f"ncn_cuda_amd: warning: {reason}, and there is no hipcc here to rebuild it: loading it as it is",
                  file=sys.stderr)
        else:
            print(f"ncn_cuda_amd: {reason}: building what changed with hipcc (up to a minute)", file=sys.stderr)
            try:
                _build.build(force=False)   # under a file lock; checks again whether another process has built it
            except Exception as exc:
                raise RuntimeError(
                    f"{LIB_PATH}: {reason}, and building it failed ({exc}); build it with `python -m ncn_cuda_amd._build` "
                    "(or __graft_entry__.build()): there is no CPU or PyTorch fallback for the NCN kernels") from exc
    lib = ctypes.CDLL(LIB_PATH)
    vp, f32p, shp = ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(NcnShape)
    i, fl = ctypes.c_int, ctypes.c_float
    lib.ncn_forward.restype = i
    lib.ncn_forward.argtypes = [vp, vp, i, vp, vp, i, f32p, f32p, f32p, vp, ctypes.c_size_t, shp, i, i, fl, fl, i, vp]
    lib.ncn_backward.restype = i
    lib.ncn_backward.argtypes = [vp, vp, i, vp, vp, i, vp, vp, i, f32p, f32p, f32p, f32p, vp, ctypes.c_size_t,
                                 shp, i, i, fl, fl, i, vp]
    lib.ncn_backward_static.restype = i
    lib.ncn_backward_static.argtypes = [vp, vp, i, vp, vp, i, vp, vp, i, f32p, f32p, f32p, f32p, shp, i, i, fl, fl, i, vp]
    lib.ncn_static_scratch_bytes.restype = ctypes.c_size_t
    lib.ncn_static_scratch_bytes.argtypes = []
    lib.ncn_inverse.restype = i
    lib.ncn_inverse.argtypes = [vp, vp, i, vp, vp, i, f32p, shp, i, i, fl, fl, i, vp]
    lib.ncn_forward_indexed.restype = i
    lib.ncn_forward_indexed.argtypes = [vp, vp, i, vp, vp, i, f32p, f32p, f32p, vp, vp, shp, i, i, fl, fl, i, vp]
    lib.ncn_backward_indexed.restype = i
    lib.ncn_backward_indexed.argtypes = [vp, vp, i, vp, vp, i, vp, vp, i, f32p, f32p, f32p, f32p, vp, ctypes.c_size_t,
                                         vp, vp, shp, i, i, fl, fl, i, vp]
    lib.ncn_inverse_ws.restype = i
    lib.ncn_inverse_ws.argtypes = [vp, vp, i, vp, vp, i, f32p, vp, ctypes.c_size_t, shp, i, i, fl, fl, i, vp]
    lib.ncn_inverse_indexed.restype = i
    lib.ncn_inverse_indexed.argtypes = [vp, vp, i, vp, vp, i, f32p, vp, vp, shp, i, i, fl, fl, i, vp]
    lib.ncn_forward_radix.restype = i
    lib.ncn_forward_radix.argtypes = [vp, vp, i, vp, vp, i, f32p, f32p, f32p, shp, i, i, fl, fl, i, vp]
    lib.ncn_backward_radix.restype = i
    lib.ncn_backward_radix.argtypes = [vp, vp, i, vp, vp, i, vp, vp, i, f32p, f32p, f32p, f32p, vp, ctypes.c_size_t,
                                       shp, i, i, fl, fl, i, vp]
    lib.ncn_inverse_radix.restype = i
    lib.ncn_inverse_radix.argtypes = [vp, vp, i, vp, vp, i, f32p, shp, i, i, fl, fl, i, vp]
    lib.ncn_plan_radix.restype = i
    lib.ncn_plan_radix.argtypes = [shp, i, i, i, i, ctypes.POINTER(ctypes.c_int32), i]
    lib.ncn_workspace_bytes.restype = ctypes.c_size_t
    lib.ncn_workspace_bytes.argtypes = [shp]
    lib.ncn_workspace_bytes_stages.restype = ctypes.c_size_t
    lib.ncn_workspace_bytes_stages.argtypes = [shp, i, i, i, i]
    lib.ncn_plan_passes.restype = i
    lib.ncn_plan_passes.argtypes = [shp, i, i, i, i, ctypes.POINTER(ctypes.c_int32), i]
    lib.ncn_kernel_path.restype = i
    lib.ncn_kernel_path.argtypes = [shp]
    lib.ncn_kernel_path_scalars.restype = i
    lib.ncn_kernel_path_scalars.argtypes = [shp, fl, fl]
    lib.ncn_check_shape.restype = i
    lib.ncn_check_shape.argtypes = [shp, i, i, i]
    lib.ncn_error_string.restype = ctypes.c_char_p
    lib.ncn_error_string.argtypes = [i]
    lib.ncn_version.restype = ctypes.c_char_p
    lib.ncn_version.argtypes = []
    lib.ncn_build_id.restype = ctypes.c_char_p
    lib.ncn_build_id.argtypes = []
    lib.ncn_probe_issue.restype = i
    lib.ncn_probe_issue.argtypes = [i, i, i, i, vp, vp]
    lib.ncn_probe_issue_info.restype = i
    lib.ncn_probe_issue_info.argtypes = [i, ctypes.POINTER(i), ctypes.POINTER(i)]
    _lib = lib
    return lib


def error_string(code):
    return load().ncn_error_string(int(code)).decode()


def check(code, what):
    if code != 0:
        raise RuntimeError(f"{what} failed: {error_string(code)} (code {code})")
