"""ctypes binding of ``np_oracle.c`` on numpy arrays (test infrastructure only).

16-bit float tensors cross this boundary as ``uint16`` bit patterns so that
bit-exactness is checked on the bits themselves, never through a float
comparison.  Helpers ``f16_bits`` / ``bf16_bits`` turn torch tensors into those
patterns and ``from_bits`` turns results back into torch tensors.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path

import numpy as np

DT_F16, DT_BF16, DT_F32 = 0, 1, 2

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / "libnp_oracle.so"
_lib: ctypes.CDLL | None = None

_u8p = ctypes.POINTER(ctypes.c_uint8)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_i64p = ctypes.POINTER(ctypes.c_int64)
_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int


def build(force: bool = False) -> Path:
    """Compile ``np_oracle.c`` with gcc (a second or two) and return the .so path."""
    src = _HERE / "np_oracle.c"
    if force or not _LIB_PATH.exists() or _LIB_PATH.stat().st_mtime < src.stat().st_mtime:
        subprocess.run(
            ["make", "-C", str(_HERE), "-B" if force else "-s", "libnp_oracle.so"],
            check=True,
            stdout=subprocess.DEVNULL,
        )
    return _LIB_PATH


def _load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not _LIB_PATH.exists():
        build()
    lib = ctypes.CDLL(os.fspath(_LIB_PATH))
    lib.np_oracle_bits_for.argtypes = [_i64]
    lib.np_oracle_bits_for.restype = _int
    lib.np_oracle_unpack_indices.argtypes = [_u8p, _i64, _int, _i64, _i64p]
    lib.np_oracle_pack_indices.argtypes = [_i64p, _i64, _int, _u8p]
    for name in ("np_oracle_tiered_unpack", "np_oracle_ntier_unpack", "np_oracle_zesc_unpack"):
        getattr(lib, name).argtypes = [_u8p, _i64, _i64, _i64p]
        getattr(lib, name).restype = _i64
    lib.np_oracle_vq_decode.argtypes = [_u8p, _i64, _int, _u16p, _i64, _int, _i64, _int, _vp]
    lib.np_oracle_rvq_decode.argtypes = [
        _u8p, _i64, _int, _u8p, _i64, _int, _u16p, _i64, _u16p, _i64,
        _u16p, _u16p, _int, _i64, _i64, _int, _vp,
    ]  # fmt: skip
    lib.np_oracle_q_decode.argtypes = [_u8p, _u16p, _u16p, _i64, _i64, _int, _int, _int, _vp]
    lib.np_oracle_linear.argtypes = [_vp, _int, _vp, _int, _vp, _int, _i64, _i64, _i64, _f64p]
    _i32p = ctypes.POINTER(ctypes.c_int32)
    lib.np_oracle_rms_norm.argtypes = [_vp, _vp, _int, _i64, _i64, ctypes.c_double, _f64p]
    lib.np_oracle_vq_embedding.argtypes = [_i64p, _i64, _u16p, _i64, _i64, _u16p, _i64, _i64, _i32p,
                                           ctypes.c_float, _int, _vp]  # fmt: skip
    lib.np_oracle_q_embedding.argtypes = [_i64p, _i64, _u8p, _u16p, _u16p, _int, _i64, _i64, _i64, _i64,
                                          ctypes.c_float, _int, _vp]  # fmt: skip
    lib.np_oracle_f32_to_f16.argtypes = [ctypes.c_float]
    lib.np_oracle_f32_to_f16.restype = ctypes.c_uint16
    lib.np_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
    lib.np_oracle_f32_to_bf16.restype = ctypes.c_uint16
    lib.np_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
    lib.np_oracle_f16_to_f32.restype = ctypes.c_float
    _lib = lib
    return lib


def _c(a: np.ndarray, dtype) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _ptr(a: np.ndarray | None, ctype):
    if a is None:
        return None
    return a.ctypes.data_as(ctype)


def _out_array(n: int, dtype_code: int) -> np.ndarray:
    return np.empty(n, dtype=np.float32 if dtype_code == DT_F32 else np.uint16)


def _check(rc: int, what: str) -> None:
    if rc == -2:
        raise IndexError(f"{what}: index out of range for the codebook")
    if rc != 0:
        raise ValueError(f"{what}: invalid arguments (rc={rc})")


def bits_for(num_centroids: int) -> int:
    b = _load().np_oracle_bits_for(int(num_centroids))
    if b < 0:
        raise ValueError(f"num_centroids={num_centroids} outside [2, 2**20]")
    return b


def unpack_indices(packed: np.ndarray, bits: int, n: int) -> np.ndarray:
    packed = _c(packed, np.uint8)
    out = np.empty(n, dtype=np.int64)
    rc = _load().np_oracle_unpack_indices(_ptr(packed, _u8p), packed.size, bits, n, _ptr(out, _i64p))
    _check(rc, "unpack_indices")
    return out


def pack_indices(idx: np.ndarray, bits: int) -> np.ndarray:
    idx = _c(np.asarray(idx).reshape(-1), np.int64)
    out = np.empty((idx.size * bits + 7) // 8, dtype=np.uint8)
    rc = _load().np_oracle_pack_indices(_ptr(idx, _i64p), idx.size, bits, _ptr(out, _u8p))
    _check(rc, "pack_indices")
    return out


def entropy_unpack(kind: str, packed: np.ndarray) -> np.ndarray:
    """Indices of a prefix-coded buffer; kind in {"tiered", "ntier", "zero_escape"}."""
    fn = {"tiered": "np_oracle_tiered_unpack", "ntier": "np_oracle_ntier_unpack",
          "zero_escape": "np_oracle_zesc_unpack"}[kind]  # fmt: skip
    packed = _c(packed, np.uint8)
    out = np.empty(packed.size * 8, dtype=np.int64)  # an index costs at least one stream bit
    n = getattr(_load(), fn)(_ptr(packed, _u8p), packed.size, out.size, _ptr(out, _i64p))
    if n < 0:
        raise ValueError(f"{fn}: malformed buffer (code {n})")
    return out[:n].copy()


def vq_decode(
    packed: np.ndarray,
    bits: int,
    centroids_bits: np.ndarray,
    n_rows: int,
    k_cols: int,
    out_dtype: int,
) -> np.ndarray:
    """Decoded ``[N, K]`` weight: uint16 bit patterns (f16/bf16) or float32."""
    packed = _c(packed, np.uint8)
    cb = _c(centroids_bits, np.uint16)
    nc, vl = cb.shape
    n_vec = n_rows * k_cols // vl
    out = _out_array(n_rows * k_cols, out_dtype)
    rc = _load().np_oracle_vq_decode(
        _ptr(packed, _u8p), packed.size, bits, _ptr(cb, _u16p), nc, vl, n_vec, out_dtype,
        out.ctypes.data_as(_vp),
    )  # fmt: skip
    _check(rc, "vq_decode")
    return out.reshape(n_rows, k_cols)


def rvq_decode(
    packed_main: np.ndarray,
    bits_main: int,
    packed_res: np.ndarray,
    bits_res: int,
    cb_main_bits: np.ndarray,
    cb_res_bits: np.ndarray,
    scale_bits: np.ndarray | None,
    wbias_bits: np.ndarray | None,
    n_rows: int,
    k_cols: int,
    out_dtype: int,
) -> np.ndarray:
    pm = _c(packed_main, np.uint8)
    pr = _c(packed_res, np.uint8)
    cm = _c(cb_main_bits, np.uint16)
    cr = _c(cb_res_bits, np.uint16)
    sc = None if scale_bits is None else _c(scale_bits, np.uint16)
    wb = None if wbias_bits is None else _c(wbias_bits, np.uint16)
    vl = cm.shape[1]
    out = _out_array(n_rows * k_cols, out_dtype)
    rc = _load().np_oracle_rvq_decode(
        _ptr(pm, _u8p), pm.size, bits_main, _ptr(pr, _u8p), pr.size, bits_res,
        _ptr(cm, _u16p), cm.shape[0], _ptr(cr, _u16p), cr.shape[0],
        _ptr(sc, _u16p), _ptr(wb, _u16p), vl, n_rows, k_cols, out_dtype,
        out.ctypes.data_as(_vp),
    )  # fmt: skip
    _check(rc, "rvq_decode")
    return out.reshape(n_rows, k_cols)


def q_decode(
    blob: np.ndarray,
    scale_bits: np.ndarray,
    zero_point_bits: np.ndarray | None,
    nbits: int,
    group_size: int,
    out_dtype: int,
) -> np.ndarray:
    blob = _c(blob, np.uint8)
    n_rows, kb = blob.shape
    k_cols = kb * (8 // nbits)
    sc = _c(scale_bits, np.uint16).reshape(-1)
    zp = None if zero_point_bits is None else _c(zero_point_bits, np.uint16).reshape(-1)
    out = _out_array(n_rows * k_cols, out_dtype)
    rc = _load().np_oracle_q_decode(
        _ptr(blob, _u8p), _ptr(sc, _u16p), _ptr(zp, _u16p), n_rows, k_cols, nbits, group_size,
        out_dtype, out.ctypes.data_as(_vp),
    )  # fmt: skip
    _check(rc, "q_decode")
    return out.reshape(n_rows, k_cols)


def rms_norm_f64(x_bits: np.ndarray, w_bits: np.ndarray, dtype_code: int, eps: float) -> np.ndarray:
    """RMSNorm of ``x`` ([M, H], given as dtype bits / float32 values) in double precision."""
    x = _as_typed(x_bits, dtype_code)
    w = _as_typed(w_bits, dtype_code)
    m, h = x.shape
    out = np.empty((m, h), dtype=np.float64)
    rc = _load().np_oracle_rms_norm(x.ctypes.data_as(_vp), w.ctypes.data_as(_vp), dtype_code, m, h, float(eps),
                                    _ptr(out, _f64p))  # fmt: skip
    _check(rc, "rms_norm")
    return out


def vq_embedding(ids: np.ndarray, indices_u16: np.ndarray, cb_bits: np.ndarray, scale: float,
                 inv_perm: np.ndarray | None, out_dtype_code: int) -> np.ndarray:  # fmt: skip
    """Rows of a VQ embedding table as output-dtype bits (float32 values for code 2): ``[n_ids, groups * VL]``."""
    ids = _c(np.asarray(ids).reshape(-1), np.int64)
    idx = _c(indices_u16, np.uint16)
    cb = _c(cb_bits, np.uint16)
    perm = None if inv_perm is None else _c(np.asarray(inv_perm).reshape(-1), np.int32)
    vocab, groups = idx.shape
    nc, vl = cb.shape
    out = _out_array(ids.size * groups * vl, out_dtype_code)
    i32p = ctypes.POINTER(ctypes.c_int32)
    rc = _load().np_oracle_vq_embedding(_ptr(ids, _i64p), ids.size, _ptr(idx, _u16p), vocab, groups, _ptr(cb, _u16p),
                                        nc, vl, None if perm is None else perm.ctypes.data_as(i32p), float(scale),
                                        out_dtype_code, out.ctypes.data_as(_vp))  # fmt: skip
    _check(rc, "vq_embedding")
    return out.reshape(ids.size, groups * vl)


def q_embedding(ids: np.ndarray, blob: np.ndarray, scale_bits: np.ndarray, zp_bits: np.ndarray | None, nbits: int,
                group_size: int, padding_idx: int | None, embed_scale: float, out_dtype_code: int) -> np.ndarray:  # fmt: skip
    """Rows of a group-affine n-bit embedding table as output-dtype bits: ``[n_ids, dim]``."""
    ids = _c(np.asarray(ids).reshape(-1), np.int64)
    blob = _c(blob, np.uint8)
    sc = _c(np.asarray(scale_bits).reshape(-1), np.uint16)
    zp = None if zp_bits is None else _c(np.asarray(zp_bits).reshape(-1), np.uint16)
    vocab = blob.shape[0]
    dim = blob.shape[1] * (8 // nbits)
    out = _out_array(ids.size * dim, out_dtype_code)
    rc = _load().np_oracle_q_embedding(_ptr(ids, _i64p), ids.size, _ptr(blob, _u8p), _ptr(sc, _u16p),
                                       _ptr(zp, _u16p), nbits, group_size, vocab, dim,
                                       -1 if padding_idx is None else padding_idx, float(embed_scale),
                                       out_dtype_code, out.ctypes.data_as(_vp))  # fmt: skip
    _check(rc, "q_embedding")
    return out.reshape(ids.size, dim)


def _as_typed(a: np.ndarray, dtype_code: int) -> np.ndarray:
    return _c(a, np.float32 if dtype_code == DT_F32 else np.uint16)


def linear_f64(
    x: np.ndarray,
    x_dtype: int,
    w: np.ndarray,
    w_dtype: int,
    bias: np.ndarray | None = None,
    bias_dtype: int = DT_F32,
) -> np.ndarray:
    """``x @ W.T (+ bias)`` accumulated in double; inputs as bit patterns / float32."""
    x = _as_typed(x, x_dtype)
    w = _as_typed(w, w_dtype)
    m_rows, k_cols = x.shape
    n_rows = w.shape[0]
    b = None if bias is None else _as_typed(bias, bias_dtype)
    y = np.empty((m_rows, n_rows), dtype=np.float64)
    rc = _load().np_oracle_linear(
        x.ctypes.data_as(_vp), x_dtype, w.ctypes.data_as(_vp), w_dtype,
        None if b is None else b.ctypes.data_as(_vp), bias_dtype,
        m_rows, n_rows, k_cols, _ptr(y, _f64p),
    )  # fmt: skip
    _check(rc, "linear")
    return y


# ---------------------------------------------------------------------------
# torch <-> bit-pattern helpers
# ---------------------------------------------------------------------------


def torch_dtype_code(dtype) -> int:
    import torch

    return {torch.float16: DT_F16, torch.bfloat16: DT_BF16, torch.float32: DT_F32}[dtype]


def to_bits(t) -> np.ndarray:
    """torch f16/bf16 tensor -> uint16 bit patterns; f32 -> float32 array."""
    import torch

    t = t.detach().cpu().contiguous()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.to(torch.float32).numpy()


def from_bits(a: np.ndarray, dtype):
    """Inverse of :func:`to_bits` for the given torch dtype."""
    import torch

    if dtype in (torch.float16, torch.bfloat16):
        return torch.from_numpy(np.ascontiguousarray(a).view(np.int16).copy()).view(dtype)
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32).copy())
