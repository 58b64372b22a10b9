"""ctypes binding of libmamba_hip.so (the C ABI declared in include/mamba_hip.h).

There is no fallback: if the shared library is missing or fails to load, every
op raises.  Build it with `python -m mamba_rs_amd.build`.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_char_p, c_float, c_int, c_int64, c_size_t, c_uint, c_uint64, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libmamba_hip.so"


class MambaHipError(RuntimeError):
    """An mrs_* entry point returned a non-zero code."""

    def __init__(self, fn: str, code: int, message: str):
        super().__init__(f"{fn} failed ({code}): {message}")
        self.fn, self.code, self.message = fn, code, message


_P = c_void_p
_SIGNATURES = {
    "mrs_version": (c_int, []),
    "mrs_last_error": (c_char_p, []),
    "mrs_scan_use_parallel": (c_int, [c_int, c_int64, c_int64]),
    "mrs_exp_negate": (c_int, [_P, _P, _P, c_int64]),
    "mrs_a_neg_is_s4d_real": (c_int, [_P, _P, _P, c_int, c_int]),
    "mrs_ssm_scan_fwd": (c_int, [_P, c_int, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int]),
    "mrs_ssm_scan_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "mrs_ssm_scan_flag_bytes": (c_size_t, [c_int, c_int]),
    "mrs_ssm_scan_fwd_ex": (c_int, [_P, c_int, _P, _P, _P, _P, _P, _P, c_int64, _P, _P, _P, c_int64, c_uint, _P, c_size_t,
                                    c_int, c_int, c_int, c_int]),
    "mrs_ssm_scan_fwd_static": (c_int, [_P, c_int, _P, _P, _P, _P, _P, _P, c_int64, _P, _P, _P, c_int64, c_uint,
                                        c_int, c_int, c_int, c_int]),
    "mrs_ssm_step": (c_int, [_P, c_int, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int]),
    "mrs_ssm_step_gather_gate": (c_int, [_P, c_int, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int,
                                         c_int, c_int, c_int]),
    "mrs_conv1d_step": (c_int, [_P, c_int, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int]),
    "mrs_conv1d_seq_silu": (c_int, [_P, c_int, _P, _P, _P, c_int64, _P, _P, c_int, c_int, c_int, c_int]),
    "mrs_gemm_skinny": (c_int, [_P, c_int, _P, c_int, c_int64, _P, c_int64, _P, c_int, c_int, c_int]),
    "mrs_tiled_weight_bytes": (c_size_t, [c_int, c_int, c_int]),
    "mrs_tile_weight": (c_int, [_P, c_int, _P, _P, c_int, c_int]),
    "mrs_gemm_tiled": (c_int, [_P, c_int, _P, c_int, c_int64, _P, c_int64, _P, c_int, c_int, c_int]),
    "mrs_transpose": (c_int, [_P, c_int, _P, _P, c_int, c_int]),
    "mrs_xoshiro_seed": (None, [c_uint64, POINTER(c_uint64)]),
    "mrs_sample_tokens": (c_int, [_P, _P, _P, _P, c_int64, c_int, c_int, _P, _P, _P, _P]),
    "mrs_m3_step": (c_int, [_P, c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int]),
    "mrs_m3_seq_fwd": (c_int, [_P, c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int]),
    "mrs_m3_compute_abg": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int64]),
    "mrs_m3_ssd_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "mrs_m3_ssd_fwd": (c_int, [_P, c_int, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_size_t, c_uint,
                               c_int, c_int, c_int, c_int, c_int, c_int]),
}

_lib = None


def load() -> ctypes.CDLL:
    """dlopen the library once; raise (never fall back) if it is not there."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise MambaHipError("dlopen", -100, f"{LIB_PATH} not built; run `python -m mamba_rs_amd.build`")
        lib = ctypes.CDLL(str(LIB_PATH))
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def exported_names() -> list[str]:
    return sorted(_SIGNATURES)


def call(name: str, *args):
    """Call an int-returning entry point and raise MambaHipError on failure."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise MambaHipError(name, rc, lib.mrs_last_error().decode())
    return rc
