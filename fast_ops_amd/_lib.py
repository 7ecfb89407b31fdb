"""ctypes binding of libfastops_hip.so (the C ABI declared in include/fastops.h).

There is no fallback: if the library is missing or does not load, importing a kernel wrapper raises. The reference
behaves the same way - its extensions are compiled at import and a failed build is an import error
(fast_ops/lion/lion_optimizer.py:15-26, fast_ops/flash_attention/flash_attention.py:13-25).
"""
from __future__ import annotations

import ctypes
import os
import threading

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libfastops_hip.so")

FO_LION_CHUNK = 8192
FO_ATTN_BWD_STATIC_ROWS = 1 << 20
ABI_MAJOR = 2            # fo_version() // 1000 the signatures below belong to
FO_DTYPE_F16, FO_DTYPE_BF16, FO_DTYPE_F32 = 0, 1, 2
FO_ATTN_KERNEL_ROWS128, FO_ATTN_KERNEL_ROWS128_EXACT, FO_ATTN_KERNEL_ROWS128_PIPE, FO_ATTN_KERNEL_ROWS256_W8, FO_ATTN_KERNEL_ROWS256_W4 = 0, 1, 8, 16, 32


class FoLionConsts(ctypes.Structure):
    _fields_ = [(n, ctypes.c_float) for n in ("c_wd", "c_b1", "c_1b1", "c_nlr", "c_b2", "c_1b2")]


class FoLionChunk(ctypes.Structure):
    _fields_ = [("p", ctypes.c_void_p), ("g", ctypes.c_void_p), ("m", ctypes.c_void_p), ("n", ctypes.c_int32), ("reserved", ctypes.c_int32)]


# every symbol include/fastops.h declares: name -> (restype, argtypes)
_I64P = ctypes.POINTER(ctypes.c_int64)
SIGNATURES = {
    "fo_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "fo_version": (ctypes.c_int, []),
    "fo_tune_set": (ctypes.c_int, [ctypes.c_char_p, ctypes.c_int]),
    "fo_tune_get": (ctypes.c_int, [ctypes.c_char_p]),
    "fo_attn_fwd": (ctypes.c_int, [ctypes.c_void_p] * 5 + [ctypes.c_int] * 5 + [_I64P] * 4 + [ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "fo_attn_fwd_kernel": (ctypes.c_int, [ctypes.c_int] * 5 + [_I64P] * 2 + [ctypes.c_int] * 3),
    "fo_attn_bwd": (ctypes.c_int, [ctypes.c_void_p] * 10 + [ctypes.c_int] * 5 + [ctypes.POINTER(_I64P), ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "fo_attn_bwd_static_ws": (ctypes.c_int, [ctypes.c_void_p] * 9 + [ctypes.c_int] * 5 + [ctypes.POINTER(_I64P), ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "fo_attn_fwd_dropout": (ctypes.c_int, [ctypes.c_void_p] * 5 + [ctypes.c_int] * 5 + [_I64P] * 4 + [ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p]),
    "fo_dropout_mask": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p]),
    "fo_attn_fwd_ex": (ctypes.c_int, [ctypes.c_void_p] * 5 + [ctypes.c_int] * 5 + [_I64P] * 4 + [ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "fo_attn_bwd_ex": (ctypes.c_int, [ctypes.c_void_p] * 10 + [ctypes.c_int] * 5 + [ctypes.POINTER(_I64P), ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "fo_attn_bwd_dropout": (ctypes.c_int, [ctypes.c_void_p] * 10 + [ctypes.c_int] * 5 + [ctypes.POINTER(_I64P), ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p]),
    "fo_lion_make_consts": (ctypes.c_int, [ctypes.c_double] * 4 + [ctypes.POINTER(FoLionConsts)]),
    "fo_lion_update": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_int64, ctypes.POINTER(FoLionConsts), ctypes.c_void_p]),
    "fo_lion_step": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.POINTER(FoLionConsts), ctypes.c_void_p]),
    "fo_lion_fill_chunks": (ctypes.c_int64, [ctypes.c_void_p] * 3 + [ctypes.c_int64, ctypes.c_void_p]),
    "fo_lion_make_consts_typed": (ctypes.c_int, [ctypes.c_double] * 4 + [ctypes.c_int, ctypes.c_int, ctypes.POINTER(FoLionConsts)]),
    "fo_lion_fill_chunks_typed": (ctypes.c_int64, [ctypes.c_void_p] * 3 + [ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]),
    "fo_lion_step_typed": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.POINTER(FoLionConsts), ctypes.c_void_p]),
    "fo_lion_update_typed": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.POINTER(FoLionConsts), ctypes.c_void_p]),
}

_lock = threading.Lock()
_lib = None


class FastOpsLibraryError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Loads the library once; raises FastOpsLibraryError (a RuntimeError) when it is absent or broken."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise FastOpsLibraryError(
                f"{LIB_PATH} is missing: build it with `python -m fast_ops_amd.build` (needs hipcc). "
                "There is no CPU or PyTorch fallback for these kernels."
            )
        try:
            lib = ctypes.CDLL(LIB_PATH)
        except OSError as e:
            raise FastOpsLibraryError(f"could not load {LIB_PATH}: {e}") from e
        for name, (restype, argtypes) in SIGNATURES.items():
            try:
                fn = getattr(lib, name)
            except AttributeError as e:
                raise FastOpsLibraryError(f"{LIB_PATH} does not export {name}; rebuild it") from e
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.fo_version() // 1000 != ABI_MAJOR:
            raise FastOpsLibraryError(f"{LIB_PATH} has ABI version {lib.fo_version()}, this package needs {ABI_MAJOR}xxx; rebuild it")
        _lib = lib
    return _lib


def strerror(status: int) -> str:
    return load().fo_strerror(status).decode()


def check(status: int, what: str) -> None:
    """Maps a negative fo_status to RuntimeError, the exception type the reference's extensions surface
    (std::runtime_error / TORCH_CHECK, fast_ops/lion/lion_update.cu:109-112,132-135)."""
    if status != 0:
        raise RuntimeError(f"{what}: {strerror(status)} (fo_status {status})")


def tune_set(key: str, value: int) -> None:
    check(load().fo_tune_set(key.encode(), int(value)), f"fo_tune_set({key!r}, {value})")
