"""ctypes binding of libflute_hip.so (the C ABI declared in include/flute_hip.h).

The library is built in-tree by csrc/Makefile into ../lib/.  There is no other
implementation behind this module: if the shared object is missing, importing
fails with an ImportError that says how to build it.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libflute_hip.so")

FLUTE_OK = 0
FLUTE_ERR_INVALID = 1
FLUTE_ERR_UNSUPPORTED = 2
FLUTE_ERR_HIP = 3
FLUTE_ERR_NOMEM = 4

F16, BF16, F32, U8 = 0, 1, 2, 3


class FluteLinear(ctypes.Structure):
    """struct flute_linear."""
    _fields_ = [
        ("q1", ctypes.c_void_p),
        ("lut1", ctypes.c_void_p),
        ("q2", ctypes.c_void_p),
        ("lut2", ctypes.c_void_p),
        ("resB", ctypes.c_void_p),
        ("resA", ctypes.c_void_p),
        ("bias", ctypes.c_void_p),
        ("signs", ctypes.c_void_p),
        ("awq", ctypes.c_void_p),
        ("q1_bytes", ctypes.c_int64),
        ("q2_bytes", ctypes.c_int64),
        ("lut_rows", ctypes.c_int32),
        ("N", ctypes.c_int32),
        ("K", ctypes.c_int32),
        ("R", ctypes.c_int32),
        ("b1", ctypes.c_int32),
        ("b2", ctypes.c_int32),
        ("group_size", ctypes.c_int32),
        ("lut_dtype", ctypes.c_int32),
        ("rot_block", ctypes.c_int32),
        ("k_group", ctypes.c_int32),
    ]


class FluteTensor(ctypes.Structure):
    """struct flute_tensor: what a binding knows about one tensor."""
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("dtype_name", ctypes.c_char_p),
        ("numel", ctypes.c_int64),
        ("size", ctypes.c_int64 * 4),
        ("ndim", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("contiguous", ctypes.c_int32),
        ("device", ctypes.c_int32),
        ("present", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


class FluteOperands(ctypes.Structure):
    """struct flute_operands: the operands of one weight as an entry point received them."""
    _fields_ = [(n, FluteTensor) for n in
                ("A", "indices", "lut", "indices2", "lut2", "resB", "resA", "bias", "signs", "awq")] + [
        ("K", ctypes.c_int64),
        ("b1", ctypes.c_int32),
        ("b2", ctypes.c_int32),
        ("group_size", ctypes.c_int32),
        ("rot_block", ctypes.c_int32),
        ("max_rank", ctypes.c_int32),
        ("gs_allowed", ctypes.c_uint32),
    ]


# every symbol include/flute_hip.h declares: (restype, argtypes)
_P = ctypes.c_void_p
_LP = ctypes.POINTER(FluteLinear)
_I = ctypes.c_int
SYMBOLS = {
    "flute_abi_version": (_I, []),
    "flute_last_error": (ctypes.c_char_p, []),
    "flute_target_arch": (ctypes.c_char_p, []),
    "flute_check_input": (_I, [ctypes.c_char_p, ctypes.POINTER(FluteTensor), _I]),
    "flute_describe_linear": (_I, [ctypes.c_char_p, ctypes.POINTER(FluteOperands), _LP,
                                   ctypes.POINTER(ctypes.c_int64)]),
    "flute_gemv": (_I, [_LP, _P, _P, _I, _I, _P]),
    "flute_gemv_noalloc": (_I, [_LP, _P, _P, _I, _I, _P]),
    "flute_gemv_mlp": (_I, [_LP, _LP, _P, _P, _I, _I, _P]),
    "flute_gemv_multi": (_I, [_LP, _I, _P, ctypes.POINTER(_P), _I, _I, _P]),
    "flute_mlp_block": (_I, [_LP, _LP, _LP, _P, _P, _P, _I, _P]),
    "flute_gemm": (_I, [_LP, _P, _P, _I, ctypes.c_int64, ctypes.c_int64, _I, _P]),
    "flute_gemm_debug_simple": (_I, [_P, ctypes.c_int64, _I, _P, _I, _I, _I, _I, _I, _I, _P, _P, _I,
                                     ctypes.c_int64, ctypes.c_int64, _I, _P]),
    "flute_dequant": (_I, [_LP, _I, _P, _P]),
    "flute_fht": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "flute_embedding": (_I, [_LP, _P, ctypes.c_int64, _P, _P]),
    "flute_pick_split": (_I, [_I, _I]),
    "flute_gemv_lds_bytes": (ctypes.c_int64, [_LP, _I]),
    "flute_validate": (_I, [_LP, _I]),
    "flute_release_workspaces": (None, []),
    "flute_reload_tuning": (None, []),
    "flute_workspace_decision": (_I, [ctypes.c_int64] * 4 + [_I]),
    "flute_join_address_halves": (ctypes.c_uint64, [ctypes.c_int32, ctypes.c_int32]),
    "flute_build_id": (ctypes.c_char_p, []),
    "flute_read_probe": (_I, [_P, ctypes.c_int64, _I, _I, _P, _P]),
}

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"flute_extended: {LIB_PATH} is missing. Build it with "
        f"`make -C {os.path.join(os.path.dirname(_HERE), 'csrc')}` (hipcc, gfx950). "
        "There is no fallback implementation.")

lib = ctypes.CDLL(LIB_PATH)
for _name, (_res, _args) in SYMBOLS.items():
    _fn = getattr(lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args


def build_id() -> str:
    """What the loaded library says it was built from (flute_build_id)."""
    return lib.flute_build_id().decode("ascii")


def tree_build_id() -> str:
    """The same hash over the sources as they are in the tree now (csrc/Makefile's BUILD_ID:
    the .hip sources in the Makefile's order, the csrc headers sorted by name, the C header).
    Differs from build_id() when the library on disk is older than the sources."""
    import glob
    import hashlib
    import re
    csrc = os.path.join(os.path.dirname(_HERE), "csrc")
    with open(os.path.join(csrc, "Makefile")) as f:
        srcs = re.search(r"^SRCS := (.*)$", f.read(), re.M).group(1).split()
    files = [os.path.join(csrc, n) for n in srcs] + sorted(glob.glob(os.path.join(csrc, "*.h")))
    files.append(os.path.join(os.path.dirname(os.path.dirname(_HERE)), "include", "flute_hip.h"))
    h = hashlib.sha256()
    for name in files:
        with open(name, "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def last_error() -> str:
    return lib.flute_last_error().decode("utf-8", "replace")


def check(status: int) -> None:
    """Turn a flute_status into the exception upstream's TORCH_CHECK would raise."""
    if status != FLUTE_OK:
        raise RuntimeError(last_error() or f"libflute_hip: status {status}")
