"""ctypes binding of librglru_hip.so (the C ABI declared in include/rglru_hip.h)."""

from __future__ import annotations

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "librglru_hip.so")

RGLRU_F32 = 0
RGLRU_BF16 = 1
FLAG_RESET = 1
FLAG_INACTIVE = 2
CHUNK = 32
ABI_VERSION = 19
PATH_PORTABLE, PATH_FAST_TILED, PATH_FAST_CHAIN, PATH_WIDE, PATH_PRE = range(5)
PATH_NAMES = ("portable", "fast_tiled", "fast_chain", "wide", "pre")

_lock = threading.Lock()
_lib = None
_load_error: str | None = None

_P = ctypes.c_void_p
_I = ctypes.c_int64
_SIGNATURES = {
    "rglru_hip_abi_version": (ctypes.c_int, []),
    "rglru_hip_last_error": (ctypes.c_char_p, []),
    "rglru_hip_max_block_width": (ctypes.c_int, []),
    "rglru_hip_scan_workspace_bytes": (ctypes.c_size_t, [_I, _I, _I]),
    "rglru_hip_scan_fwd": (ctypes.c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _P]),
    "rglru_hip_scan_bwd": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, ctypes.c_int, _I, _I, _I, _P]),
    "rglru_hip_prep_bytes": (ctypes.c_size_t, [_I, _I, ctypes.c_int]),
    "rglru_hip_prepare": (ctypes.c_int, [_P, _P, _P, _P, _P, ctypes.c_float, _I, _I, ctypes.c_int, ctypes.c_int, _P, _P]),
    "rglru_hip_workspace_bytes": (ctypes.c_size_t, [_I, _I, _I, _I]),
    "rglru_hip_bwd_scratch_bytes": (ctypes.c_size_t, [_I, _I, _I, _I, ctypes.c_int]),
    "rglru_hip_fwd": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_static_workspace_bytes": (ctypes.c_size_t, []),
    "rglru_hip_fwd_static": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_prepare_fwd": (ctypes.c_int, [_P, _P, _P, _P, _P, ctypes.c_float, ctypes.c_int, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_bwd": (ctypes.c_int, [_P] * 17 + [_I, _I, _I, _I, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_fast_path": (ctypes.c_int, [_I, _I, ctypes.c_int]),
    "rglru_hip_wide_path": (ctypes.c_int, [_I, _I, ctypes.c_int]),
    "rglru_hip_bwd_full": (ctypes.c_int, [_P] * 16 + [_I, _I, _I, _I, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_bwd_wide": (ctypes.c_int, [_P] * 15 + [_I, _I, _I, _I, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_pre_path": (ctypes.c_int, [_I, _I, ctypes.c_int]),
    "rglru_hip_backward_path": (ctypes.c_int, [_I, _I, _I, _I, ctypes.c_int, ctypes.c_int]),
    "rglru_hip_fwd_pre": (ctypes.c_int, [_P] * 8 + [_I, _I, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_bwd_pre": (ctypes.c_int, [_P] * 17 + [_I, _I, _I, _I, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_step": (ctypes.c_int, [_P, _P, _P, _P, _P, _I, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_steps": (ctypes.c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_conv_max_kernel_size": (ctypes.c_int, []),
    "rglru_hip_conv_fwd": (ctypes.c_int, [_P] * 7 + [_I, _I, _I, _I, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_conv_scratch_bytes": (ctypes.c_size_t, [_I, _I, _I, _I]),
    "rglru_hip_conv_bwd": (ctypes.c_int, [_P] * 7 + [_I] + [_P] * 3 + [_I, _I, _I, _I, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_conv_padded_scratch_bytes": (ctypes.c_size_t, [_I, _I]),
    "rglru_hip_conv_padded_fwd": (ctypes.c_int, [_P] * 9 + [_I, _I, _I, _I, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_conv_padded_bwd": (ctypes.c_int, [_P] * 12 + [_I, _I, _I, _I, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_colsum_scratch_bytes": (ctypes.c_size_t, [_I, _I]),
    "rglru_hip_colsum": (ctypes.c_int, [_P, _P, _P, _I, _I, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_sum_sets": (ctypes.c_int, [_P, _P, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_gelu_gate_fwd": (ctypes.c_int, [_P, _P, _P, _I, ctypes.c_int, _P]),
    "rglru_hip_gelu_gate_bwd": (ctypes.c_int, [_P, _P, _P, _P, _P, _I, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_rmsnorm_max_width": (ctypes.c_int, [ctypes.c_int, ctypes.c_int]),
    "rglru_hip_rmsnorm_fwd": (ctypes.c_int, [_P, _P, _P, _P, _I, _I, ctypes.c_float, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_rmsnorm_scratch_bytes": (ctypes.c_size_t, [_I, _I]),
    "rglru_hip_rmsnorm_bwd": (ctypes.c_int, [_P] * 7 + [_I, _I, ctypes.c_int, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_decode_prepare": (ctypes.c_int, [_P, _I] + [_P] * 10 + [_I, _I, _I, ctypes.c_int, ctypes.c_int, _P]),
    "rglru_hip_block_fwd_path": (ctypes.c_int, [_I, _I, _I, ctypes.c_int]),
    "rglru_hip_block_flags": (ctypes.c_int, [_P, _P, _I, _P]),
    "rglru_hip_block_fwd": (ctypes.c_int, [_P, _I, _P, _I, _P, _P, _P, _I, ctypes.c_int] + [_P] * 9
                            + [_I, _I, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_prepare_block_fwd": (ctypes.c_int, [_P] * 5 + [ctypes.c_float, ctypes.c_int, _P]
                                    + [_P, _I, _P, _I, _P, _P, _P, _I] + [_P] * 8
                                    + [_I, _I, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_step_gated": (ctypes.c_int, [_P] * 6 + [_I, _P] + [_I, _I, _I, ctypes.c_int, _P]),
    "rglru_hip_set_spin_limit": (ctypes.c_int64, [_I]),
    "rglru_hip_set_reproducible": (ctypes.c_int, [ctypes.c_int]),
    "rglru_hip_set_chain_forward": (ctypes.c_int, [ctypes.c_int]),
    "rglru_hip_set_timing": (ctypes.c_int, [ctypes.c_int]),
    "rglru_hip_kernel_ms": (ctypes.c_float, [ctypes.c_int]),
    "rglru_hip_workspace_status": (ctypes.c_int, [_P, _I, _I, _I, _I, ctypes.c_int, _P, ctypes.POINTER(ctypes.c_int)]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def library_path() -> str:
    return LIB_PATH


def load():
    """Return the loaded library; raises RuntimeError when it is missing or does not load."""
    global _lib, _load_error
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            _load_error = (
                f"{LIB_PATH} is not built; run `python -m griffin_amd.build` (needs hipcc) first"
            )
            raise RuntimeError("RG-LRU HIP library unavailable: " + _load_error)
        try:
            lib = ctypes.CDLL(LIB_PATH)
            for name, (restype, argtypes) in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            if lib.rglru_hip_abi_version() != ABI_VERSION:
                raise OSError(f"ABI version {lib.rglru_hip_abi_version()} != expected {ABI_VERSION}")
        except (OSError, AttributeError) as error:
            _load_error = str(error)
            raise RuntimeError("RG-LRU HIP library unavailable: " + _load_error) from error
        _lib = lib
        return _lib


def available() -> bool:
    """True when the shared library exists and loads (says nothing about a GPU being present)."""
    try:
        load()
    except RuntimeError:
        return False
    return True


def check(code: int, what: str) -> None:
    """Raise the Python exception that matches a non-zero return code of the C ABI."""
    if code == 0:
        return
    message = load().rglru_hip_last_error().decode("utf-8", "replace")
    text = f"{what} failed: {message}"
    if code in (1, 2):
        raise ValueError(text)
    raise RuntimeError(text)
