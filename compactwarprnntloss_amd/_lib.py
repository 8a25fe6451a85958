"""ctypes binding of libcwarp_rnnt_hip.so (declared in include/cwarp_rnnt_hip.h).

The library is built in-tree by compactwarprnntloss_amd.build; loading fails loudly when it is
missing -- there is no fallback implementation.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# CWARP_RNNT_LIB points at a library built elsewhere (same ABI); the default is the in-tree build
LIB_PATH = os.environ.get("CWARP_RNNT_LIB") or os.path.join(HERE, "libcwarp_rnnt_hip.so")

# enum cwr_dtype / cwr_mode / cwr_flag
F32, F16, BF16, F64 = 0, 1, 2, 3
MODE_LOGPROB, MODE_FUSED = 0, 1
NOALLOC_SCRATCH_BYTES = 128 << 20  # CWR_NOALLOC_SCRATCH_BYTES
FLAG_ROWS_MISMATCH, FLAG_BAD_LENGTH, FLAG_BAD_LABEL, FLAG_FB_MISMATCH, FLAG_U_TOO_LARGE, FLAG_INTERNAL = \
    1, 2, 4, 8, 16, 32
FLAG_NAMES = {
    FLAG_ROWS_MISMATCH: "sum(lx*(ly+1)) differs from the number of rows of x",
    FLAG_BAD_LENGTH: "a frame length <= 0 or a label length < 0",
    FLAG_BAD_LABEL: "a label outside [0, V)",
    FLAG_FB_MISMATCH: "forward/backward likelihood mismatch above 0.1 %",
    FLAG_U_TOO_LARGE: "a label length above the max_u given",
    FLAG_INTERNAL: "a bounded wait inside a kernel ran out",
}

_p, _i64, _i32, _sz = C.c_void_p, C.c_int64, C.c_int32, C.c_size_t

SIGNATURES = {
    "cwr_version": (C.c_int, []),
    "cwr_strerror": (C.c_char_p, [C.c_int]),
    "cwr_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "cwr_workspace_section": (C.c_int, [_i64, _i64, _i64, C.c_int, C.POINTER(_sz), C.POINTER(_sz)]),
    "cwr_lattice_slot": (_i64, [_i64, _i64, _i64, _i64]),
    "cwr_cost_rule": (C.c_int, [C.c_double, C.c_double, C.POINTER(C.c_float)]),
    "cwr_debug_wait_limit": (None, [C.c_int]),
    "cwr_offsets": (C.c_int, [_p, _p, _i64, _i64, _p, _p, _p, _p]),
    "cwr_forward": (C.c_int, [_p, C.c_int, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, C.c_int, _i64,
                              _p, _sz, _p, _p, _p, _p, _p, _p, _p, _p]),
    "cwr_debug_forward_stage_times": (C.c_int, [_p, C.c_int, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, C.c_int,
                                                _i64, _p, _sz, _p, _p, _p, _p, _p, _p, _p, _p,
                                                C.POINTER(C.c_float)]),
    "cwr_forward_noalloc": (C.c_int, [_p, C.c_int, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, C.c_int, _i64,
                                      _p, _p, _p, _p, _p, _p, _p, _p]),
    "cwr_loss": (C.c_int, [_p, C.c_int, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, C.c_int, _i64,
                           _p, _sz, _p, _p, _p, _p, _p]),
    "cwr_forward_reduced": (C.c_int, [_p, C.c_int, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, C.c_int, _i64,
                                      _p, _sz, _p, _p, _p, _p, _p, _p, _p, _p, _p]),
    "cwr_loss_reduced": (C.c_int, [_p, C.c_int, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, C.c_int, _i64,
                                   _p, _sz, _p, _p, _p, _p, _p, _p]),
    "cwr_backward": (C.c_int, [_p, C.c_int, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, C.c_int,
                               _p, _p, _p, _p, _p, _p, _i64, C.c_float, _p, _p]),
    "cwr_rowinfo": (C.c_int, [_p, _p, _p, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _p]),
    "cwr_export_lattice": (C.c_int, [_p, _p, _i64, _i64, _i64, _p, _sz, _i64, _i64, _p, _p, _p]),
    "cwr_pack": (C.c_int, [_p, C.c_int, _i64, _i64, _i64, _i64, _p, _p, _p, _i64, _p, _p, _p]),
    "cwr_unpack": (C.c_int, [_p, C.c_int, _i64, _i64, _i64, _i64, _p, _p, _p, _i64, _p, _p]),
    "cwr_joint_forward": (C.c_int, [_p, _p, _p, C.c_int, _i64, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i32, _i64,
                                    _p, _sz, _p, _p, _p, _p, _p, _p, _p, _p]),
    "cwr_joint_forward_fg": (C.c_int, [_p, _p, C.c_int, _i64, _i64, _p, _p, _p, C.c_int, _i64, _i64, _i64, _p, _p, _p,
                                       _i64, _i64, _i64, _i32, _i64, _p, _sz, _p, _p, _p, _p, _p, _p, _p, _p]),
    "cwr_joint_backward": (C.c_int, [_p, _p, _p, C.c_int, _i64, _i64, _i64, _i64, _i32, _p, _p, _p, _p, _i64, C.c_float,
                                     _p, _p]),
    "cwr_join": (C.c_int, [_p, _p, C.c_int, C.c_int, _i64, _i64, _i64, _i64, _p, _p, _p, _i64, _p, _p, _p]),
    "cwr_join_backward": (C.c_int, [_p, _p, C.c_int, C.c_int, _i64, _i64, _i64, _i64, _p, _p, _p, _i64, _p, _p, _p]),
}

_lib = None


def load() -> C.CDLL:
    """Load the shared library once and attach the argument types."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m compactwarprnntloss_amd.build` "
            "(needs hipcc); there is no CPU or PyTorch fallback for this path")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def strerror(code: int) -> str:
    return load().cwr_strerror(code).decode()


def check(code: int, what: str) -> None:
    if code != 0:
        raise RuntimeError(f"{what}: {strerror(code)} (cwr_status {code})")


def describe_flags(flags: int) -> str:
    return "; ".join(txt for bit, txt in FLAG_NAMES.items() if flags & bit) or "none"
