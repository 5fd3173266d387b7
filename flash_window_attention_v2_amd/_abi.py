"""ctypes binding of libfwa2.so (C ABI declared in include/fwa2.h).

The structure layouts below mirror include/fwa2.h field by field; the library
checks `struct_bytes` and `abi_version` on every call, so a mismatch is
reported instead of being mis-read.  There is no fallback: if the shared
library is missing every operator call raises.
"""
import ctypes
import os
import threading

ABI_VERSION = 4

OK, ERR_INVALID_ARGUMENT, ERR_UNSUPPORTED, ERR_HIP, ERR_NO_DEVICE = range(5)
F16, BF16, F32 = 0, 1, 2
SCALE_DEFAULT, SCALE_TENSOR = 0, 1
STATIC_SCRATCH_BYTES = 128 << 20    # FWA2_STATIC_SCRATCH_BYTES of include/fwa2.h
MASK_REGION_BYTES = 272             # FWA2_MASK_REGION_BYTES of include/fwa2.h

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libfwa2.so")

EXPORTS = (
    "fwa2_abi_version",
    "fwa2_last_error",
    "fwa2_validate",
    "fwa2_mask_scan",
    "fwa2_mask_scan_regions",
    "fwa2_backward_workspace_bytes",
    "fwa2_forward",
    "fwa2_backward",
    "fwa2_backward_static",
    "fwa2_cpb_bias_forward",
    "fwa2_cpb_bias_backward",
)


class Tensor4(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_bw", ctypes.c_int64), ("stride_h", ctypes.c_int64),
                ("stride_n", ctypes.c_int64)]


class Tensor3(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_a", ctypes.c_int64), ("stride_n", ctypes.c_int64)]


class Problem(ctypes.Structure):
    _fields_ = [
        ("struct_bytes", ctypes.c_uint32), ("abi_version", ctypes.c_uint32),
        ("dtype", ctypes.c_int32), ("mask_dtype", ctypes.c_int32), ("scale_kind", ctypes.c_int32),
        ("bw", ctypes.c_int32), ("heads", ctypes.c_int32), ("n", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("n_windows", ctypes.c_int32),
        ("q", Tensor4), ("k", Tensor4), ("v", Tensor4), ("o", Tensor4),
        ("logit_scale", ctypes.c_void_p),
        ("bias", Tensor3), ("mask", Tensor3),
        ("mask_live", ctypes.c_void_p),
        ("lse", ctypes.c_void_p), ("lse_stride_bw", ctypes.c_int64), ("lse_stride_h", ctypes.c_int64),
        ("d_o", Tensor4), ("dq", Tensor4), ("dk", Tensor4), ("dv", Tensor4),
        ("dbias", ctypes.c_void_p), ("dscale", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
        ("stream", ctypes.c_void_p),
        ("grid_h", ctypes.c_int32), ("grid_w", ctypes.c_int32),
        ("win_h", ctypes.c_int32), ("win_w", ctypes.c_int32),
        ("shift_h", ctypes.c_int32), ("shift_w", ctypes.c_int32),
        ("n_keys", ctypes.c_int32), ("scale_head_dim", ctypes.c_int32),
        ("mask_regions", ctypes.c_void_p),
        ("ev_start", ctypes.c_void_p), ("ev_stop", ctypes.c_void_p),
    ]


class Fwa2Error(RuntimeError):
    """A HIP failure or an unsupported configuration reported by libfwa2."""


_lib = None
_lock = threading.Lock()


def lib_path():
    return _LIB_PATH


def load():
    """Load libfwa2.so once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(_LIB_PATH):
            raise Fwa2Error(
                f"{_LIB_PATH} is missing: build it with `make -C {os.path.dirname(_LIB_PATH)}/../csrc` "
                "(or `python -c 'import __graft_entry__ as g; g.build()'`). There is no fallback path.")
        lib = ctypes.CDLL(_LIB_PATH)
        lib.fwa2_abi_version.restype = ctypes.c_int
        lib.fwa2_last_error.restype = ctypes.c_char_p
        lib.fwa2_validate.argtypes = [ctypes.POINTER(Problem), ctypes.c_int]
        lib.fwa2_validate.restype = ctypes.c_int
        lib.fwa2_mask_scan.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
                                       ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
        lib.fwa2_mask_scan.restype = ctypes.c_int
        lib.fwa2_mask_scan_regions.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int64,
                                               ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        lib.fwa2_mask_scan_regions.restype = ctypes.c_int
        lib.fwa2_backward_workspace_bytes.argtypes = [ctypes.POINTER(Problem)]
        lib.fwa2_backward_workspace_bytes.restype = ctypes.c_size_t
        lib.fwa2_forward.argtypes = [ctypes.POINTER(Problem)]
        lib.fwa2_forward.restype = ctypes.c_int
        lib.fwa2_backward.argtypes = [ctypes.POINTER(Problem)]
        lib.fwa2_backward.restype = ctypes.c_int
        lib.fwa2_backward_static.argtypes = [ctypes.POINTER(Problem)]
        lib.fwa2_backward_static.restype = ctypes.c_int
        lib.fwa2_cpb_bias_forward.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                              ctypes.c_void_p, ctypes.c_void_p]
        lib.fwa2_cpb_bias_forward.restype = ctypes.c_int
        lib.fwa2_cpb_bias_backward.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                               ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        lib.fwa2_cpb_bias_backward.restype = ctypes.c_int
        if lib.fwa2_abi_version() != ABI_VERSION:
            raise Fwa2Error(f"libfwa2 ABI {lib.fwa2_abi_version()} != binding ABI {ABI_VERSION}")
        _lib = lib
    return _lib


def new_problem():
    p = Problem()
    p.struct_bytes = ctypes.sizeof(Problem)
    p.abi_version = ABI_VERSION
    return p


def check(status, what):
    """Map a libfwa2 status to the exception the reference would raise."""
    if status == OK:
        return
    msg = load().fwa2_last_error().decode("utf-8", "replace")
    if status == ERR_INVALID_ARGUMENT:
        raise AssertionError(f"{what}: {msg}")
    if status == ERR_UNSUPPORTED:
        raise NotImplementedError(f"{what}: {msg}")
    raise Fwa2Error(f"{what}: {msg} (status {status})")
