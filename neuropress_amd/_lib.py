"""ctypes binding of ``libnpamd.so`` (the C ABI declared in ``include/npamd.h``).

The library is loaded lazily on first use.  There is no CPU fallback behind
these calls: if the shared object is missing or a call fails, a
``RuntimeError`` is raised with the library's own message.
"""

from __future__ import annotations

import ctypes
import os
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libnpamd.so"

F16, BF16, F32 = 0, 1, 2
GEMV_MAX_M = 32
ABI_VERSION = 3

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int

# name -> argtypes, exactly the order of include/npamd.h
_VQ_LINEAR = [_vp, _i64, _vp, _i64, _int, _vp, _int, _int, _int, _vp, _vp, _i64,
              _int, _int, _int, _int, _vp]  # fmt: skip
_WS = [_vp, _i64]  # workspace pointer and size, before the stream, in the *_gemm_tile entry points
_RVQ_LINEAR = [_vp, _i64, _vp, _i64, _int, _vp, _i64, _int, _vp, _int, _vp, _int, _vp, _vp, _int,
               _vp, _vp, _i64, _int, _int, _int, _int, _vp]  # fmt: skip
_Q_LINEAR = [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _int, _int, _int, _int, _int, _int, _vp]
SIGNATURES: dict[str, list] = {
    "npamd_vq_dequant": [_vp, _i64, _int, _vp, _int, _int, _i64, _vp, _int, _vp],
    "npamd_vq_gemv": _VQ_LINEAR,
    "npamd_vq_gemv_perm": _VQ_LINEAR[:2] + [_vp] + _VQ_LINEAR[2:],
    "npamd_vq_gemv_perm_supported": [_int] * 6,
    "npamd_vq_gemm_tile": _VQ_LINEAR[:-1] + _WS + [_vp],
    "npamd_gemm_tile_workspace_bytes": [_int, _int, _int],
    "npamd_vq_widen_u16": [_vp, _i64, _int, _i64, _vp, _vp],
    "npamd_vq_lut_gather": [_vp, _vp, _i64, _int, _vp, _int, _int, _int, _int, _vp],
    "npamd_vq_sliced_build": [_vp, _i64, _int, _int, _int, _int, _int, _int, _vp, _i64,
                              ctypes.POINTER(_i64)],  # fmt: skip
    "npamd_vq_sliced_check": [_vp, _i64],
    "npamd_vq_fused_supported": [_int, _int, _int],
    "npamd_gemv_stages_activations": [_int, _int, _int, _int],
    "npamd_q_fused_supported": [_int, _int, _int],
    "npamd_vq_gemv_coded": [_vp, _i64, _int, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _int, _int, _vp, _vp,
                            _i64, _int, _int, _int, _int, _vp],  # fmt: skip
    "npamd_vq_sliced_workspace_bytes": [_vp, _int],
    "npamd_vq_gemv_sliced": [_vp, _i64, _vp, _vp, _vp, _vp, _int, _vp, _vp, _i64, _int, _int, _vp, _i64, _vp],
    "npamd_vq_gemv_sliced_static": [_vp, _i64, _vp, _vp, _vp, _vp, _int, _vp, _vp, _i64, _int, _int, _vp],
    "npamd_rvq_dequant": [_vp, _i64, _int, _vp, _i64, _int, _vp, _int, _vp, _int, _vp, _vp, _int,
                          _int, _int, _vp, _int, _vp],  # fmt: skip
    "npamd_rvq_gemv": _RVQ_LINEAR,
    "npamd_rvq_gemm_tile": _RVQ_LINEAR[:-1] + _WS + [_vp],
    "npamd_q_dequant": [_vp, _vp, _vp, _int, _int, _int, _int, _vp, _int, _vp],
    "npamd_q_gemv": _Q_LINEAR,
    "npamd_rms_norm": [_vp, _i64, _vp, _vp, _i64, _int, _int, ctypes.c_float, _int, _vp],
    "npamd_vq_embedding": [_vp, _i64, _vp, _i64, _int, _vp, _int, _int, _vp, ctypes.c_float, _vp, _int, _vp],
    "npamd_q_embedding": [_vp, _i64, _vp, _vp, _vp, _int, _int, _i64, _int, _i64, ctypes.c_float, _vp, _int, _vp],
    "npamd_q_gemm_tile": _Q_LINEAR[:-1] + _WS + [_vp],
    "npamd_diag_reload_tuning": [],
    "npamd_diag_last_gemv_staged": [],
    "npamd_diag_stream_read": [_vp, _i64, _vp, _vp],
    "npamd_diag_gather": [_vp, _i64, _vp, _int, _int, _vp, _vp],
    "npamd_diag_mfma": [_vp, _int, _int, _int, _vp, _vp],
}

_RESTYPES = {"npamd_vq_sliced_workspace_bytes": _i64, "npamd_gemm_tile_workspace_bytes": _i64,
             "npamd_diag_reload_tuning": None}
SLICED_HEADER_BYTES = 128
SLICED_STATIC_WORKSPACE_BYTES = 4 * 1024 * 1024

_lib: ctypes.CDLL | None = None
_load_error: str | None = None


def load() -> ctypes.CDLL:
    """Load the shared library (once) and declare every entry point."""
    global _lib, _load_error
    if _lib is not None:
        return _lib
    if _load_error is not None:
        raise RuntimeError(_load_error)
    try:
        if not LIB_PATH.exists():
            raise OSError(f"{LIB_PATH} does not exist; build it with `python -m neuropress_amd.build`")
        lib = ctypes.CDLL(os.fspath(LIB_PATH))
        lib.npamd_version.restype = _int
        lib.npamd_last_error.restype = ctypes.c_char_p
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, _int)
        if lib.npamd_version() != ABI_VERSION:
            raise OSError(f"libnpamd ABI version {lib.npamd_version()} != expected {ABI_VERSION}")
    except (OSError, AttributeError) as exc:
        _load_error = f"neuropress_amd: cannot load the HIP kernel library: {exc}"
        raise RuntimeError(_load_error) from exc
    _lib = lib
    return lib


def is_available() -> bool:
    """True when the shared library loads (says nothing about a GPU being present)."""
    try:
        load()
        return True
    except RuntimeError:
        return False


def call(name: str, *args) -> None:
    """Call entry point *name*; raise ``RuntimeError`` with the library's message on failure."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.npamd_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{name} failed (code {rc}): {msg}")
