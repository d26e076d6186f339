"""ctypes binding of ``libtrifast_hip.so`` (the C ABI in ``include/trifast_hip.h``).

The library is the only implementation of the operator: if it is missing or does
not load, importing it raises -- there is no fallback path.
"""

from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_int, c_int64, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libtrifast_hip.so"

ABI_VERSION = 3

F32, BF16, F16 = 0, 1, 2
KERNEL_FWD, KERNEL_BWD_Q, KERNEL_BWD_KV, KERNEL_BWD_B = 0, 1, 2, 3
KERNEL_NAMES = {KERNEL_FWD: "_fwd", KERNEL_BWD_Q: "_bwd_q", KERNEL_BWD_KV: "_bwd_kv", KERNEL_BWD_B: "_bwd_b"}

_I64P = POINTER(c_int64)
_INTP = POINTER(c_int)

# name -> (restype, argtypes); one entry per declaration in include/trifast_hip.h
SIGNATURES = {
    "trifast_abi_version": (c_int, []),
    "trifast_last_error": (c_char_p, []),
    "trifast_device_clock_mhz": (c_int, [c_int]),
    "trifast_num_tiles": (c_int, [c_int]),
    "trifast_tile_info": (c_int, [c_int, c_int, _INTP, _INTP, _INTP]),
    "trifast_supports": (c_int, [c_int, c_int, c_int64, c_int64, c_int64, c_int]),
    "trifast_default_tile": (c_int, [c_int, c_int64, c_int64, c_int64, c_int]),
    "trifast_bwd_kv_tile_writes_dq": (c_int, [c_int]),
    "trifast_fwd_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64, c_int64, c_int]),
    "trifast_bwd_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64, c_int64, c_int]),
    "trifast_fwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int64, c_int64, c_int,
         _I64P, _I64P, _I64P, _I64P, _I64P,
         c_int, c_void_p, c_int64, c_void_p],
    ),
    "trifast_fwd_static": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int64, c_int64, c_int,
         _I64P, _I64P, _I64P, _I64P, _I64P,
         c_int, c_void_p],
    ),
    "trifast_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int64, c_int64, c_int,
         _I64P, _I64P, _I64P, _I64P, _I64P, _I64P,
         _I64P, _I64P, _I64P, _I64P,
         _INTP, c_void_p, c_int64, c_void_p],
    ),
    "trifast_bwd_one": (
        c_int,
        [c_int, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int64, c_int64, c_int64, c_int,
         _I64P, _I64P, _I64P, _I64P, _I64P, _I64P,
         _I64P, _I64P, _I64P, _I64P,
         c_int, c_void_p, c_int64, c_void_p],
    ),
    "trifast_linear_dw_workspace_bytes": (c_int64, [c_int64, c_int64, c_int64]),
    "trifast_linear_fwd": (c_int, [c_void_p, c_int64, c_int64, c_int, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64), POINTER(c_int64), c_int, c_void_p]),
    "trifast_linear_dx": (c_int, [c_void_p, c_int64, c_int64, c_int, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64), POINTER(c_int64), c_int, c_void_p]),
    "trifast_linear_dw": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p, c_int64, c_void_p]),
    "trifast_gate_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]),
    "trifast_gate_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once; raise if it is absent or has the wrong ABI."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m trifast_amd.build` "
            "(needs hipcc; there is no fallback implementation)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    got = lib.trifast_abi_version()
    if got != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI version {got}, expected {ABI_VERSION}: rebuild it")
    _lib = lib
    return lib


def last_error() -> str:
    msg = load().trifast_last_error()
    return msg.decode() if msg else ""


def check(rc: int, what: str) -> None:
    """Turn a return code of the C ABI into a Python exception."""
    if rc == 0:
        return
    msg = f"{what} failed ({rc}): {last_error()}"
    if rc < 0:
        raise ValueError(msg)
    raise RuntimeError(msg)


def i64_array(values) -> ctypes.Array:
    return (c_int64 * len(values))(*values)


def tile_info(kernel: int, tile: int) -> dict:
    bj, bk, nw = c_int(), c_int(), c_int()
    check(load().trifast_tile_info(kernel, tile, bj, bk, nw), "trifast_tile_info")
    return {"BLOCK_J": bj.value, "BLOCK_K": bk.value, "num_waves": nw.value}
