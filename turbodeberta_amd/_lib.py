"""ctypes binding of libtdb_attn.so (declared in include/tdb_attn.h).

The library is loaded from the package directory only.  If it has not been built, loading raises:
there is no fallback path -- every operator in this package runs the HIP kernels or fails."""
from __future__ import annotations

import ctypes as C
import os
import threading

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG, "libtdb_attn.so")

TDB_F32, TDB_BF16, TDB_F16 = 0, 1, 2
TDB_FLAG_FORCE_GENERIC = 1
ABI_VERSION = 2

ERROR_NAMES = {
    -1: "TDB_ERR_NULL", -2: "TDB_ERR_DTYPE", -3: "TDB_ERR_SHAPE", -4: "TDB_ERR_STRIDE", -5: "TDB_ERR_ALIGN",
    -6: "TDB_ERR_CAUSAL", -7: "TDB_ERR_CU_SEQLENS", -8: "TDB_ERR_POSITION", -9: "TDB_ERR_BUCKET_MARGIN",
    -10: "TDB_ERR_LAUNCH",
}
# argument errors surface as ValueError, launch failures as RuntimeError
_VALUE_ERRORS = {-1, -2, -3, -4, -5, -6, -7, -8, -9}

EXPORTS = ("tdb_version", "tdb_last_error", "tdb_attn_fwd_fixed", "tdb_attn_fwd_varlen", "tdb_bucket_table",
           "tdb_delta_table", "tdb_check_cu_seqlens", "tdb_set_workgroup_limit")


class PosArgs(C.Structure):
    _fields_ = [
        ("span", C.c_int32), ("lut_half", C.c_int32), ("delta_lut", C.c_void_p),
        ("pos_key", C.c_void_p), ("pos_query", C.c_void_p),
        ("pos_key_stride_h", C.c_int64), ("pos_key_stride_r", C.c_int64),
        ("pos_query_stride_h", C.c_int64), ("pos_query_stride_r", C.c_int64),
        ("c2p_strip", C.c_void_p), ("p2c_strip", C.c_void_p),
        ("c2p_stride_b", C.c_int64), ("c2p_stride_h", C.c_int64), ("c2p_stride_l", C.c_int64),
        ("p2c_stride_b", C.c_int64), ("p2c_stride_h", C.c_int64), ("p2c_stride_l", C.c_int64),
    ]


class FixedArgs(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32), ("batch", C.c_int32), ("heads", C.c_int32), ("head_dim", C.c_int32),
        ("seqlen", C.c_int32), ("causal", C.c_int32), ("flags", C.c_int32), ("sm_scale", C.c_float),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
        ("q_stride_b", C.c_int64), ("q_stride_h", C.c_int64), ("q_stride_l", C.c_int64),
        ("k_stride_b", C.c_int64), ("k_stride_h", C.c_int64), ("k_stride_l", C.c_int64),
        ("v_stride_b", C.c_int64), ("v_stride_h", C.c_int64), ("v_stride_l", C.c_int64),
        ("o_stride_b", C.c_int64), ("o_stride_h", C.c_int64), ("o_stride_l", C.c_int64),
        ("seqlens_k", C.c_void_p),
        ("pos", PosArgs),
    ]


class VarlenArgs(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32), ("batch", C.c_int32), ("heads", C.c_int32), ("head_dim", C.c_int32),
        ("total_tokens", C.c_int32), ("max_seqlen", C.c_int32), ("causal", C.c_int32), ("flags", C.c_int32),
        ("sm_scale", C.c_float),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
        ("q_stride_t", C.c_int64), ("q_stride_h", C.c_int64),
        ("k_stride_t", C.c_int64), ("k_stride_h", C.c_int64),
        ("v_stride_t", C.c_int64), ("v_stride_h", C.c_int64),
        ("o_stride_t", C.c_int64), ("o_stride_h", C.c_int64),
        ("cu_seqlens", C.c_void_p),
        ("pos", PosArgs),
    ]


_lock = threading.Lock()
_lib = None


def load() -> C.CDLL:
    """The loaded library; raises RuntimeError if it is missing or its ABI version differs."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m turbodeberta_amd._build` "
                "(hipcc, gfx950).  There is no fallback implementation.")
        lib = C.CDLL(LIB_PATH)
        lib.tdb_version.restype = C.c_int
        lib.tdb_last_error.restype = C.c_char_p
        lib.tdb_attn_fwd_fixed.argtypes = [C.POINTER(FixedArgs), C.c_void_p]
        lib.tdb_attn_fwd_fixed.restype = C.c_int
        lib.tdb_attn_fwd_varlen.argtypes = [C.POINTER(VarlenArgs), C.c_void_p]
        lib.tdb_attn_fwd_varlen.restype = C.c_int
        for name in ("tdb_bucket_table", "tdb_delta_table"):
            fn = getattr(lib, name)
            fn.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int32]
            fn.restype = C.c_int
        lib.tdb_check_cu_seqlens.argtypes = [C.c_void_p, C.c_int32, C.c_int32, C.c_int32]
        lib.tdb_check_cu_seqlens.restype = C.c_int
        lib.tdb_set_workgroup_limit.argtypes = [C.c_int]
        lib.tdb_set_workgroup_limit.restype = C.c_int
        if lib.tdb_version() != ABI_VERSION:
            raise RuntimeError(f"libtdb_attn.so has ABI {lib.tdb_version()}, this package expects {ABI_VERSION}")
        _lib = lib
    return _lib


def check(rc: int) -> None:
    """Map a status code to the Python exception the operators raise."""
    if rc >= 0:
        return
    msg = f"{ERROR_NAMES.get(rc, rc)}: {load().tdb_last_error().decode()}"
    raise (ValueError if rc in _VALUE_ERRORS else RuntimeError)(msg)


def bucket_table(max_len: int, position_buckets: int, max_position: int) -> np.ndarray:
    out = np.empty(2 * max_len - 1, dtype=np.int32)
    check(load().tdb_bucket_table(out.ctypes.data, max_len, position_buckets, max_position))
    return out


def delta_table(max_len: int, position_buckets: int, max_position: int) -> np.ndarray:
    out = np.empty(2 * max_len - 1, dtype=np.int32)
    check(load().tdb_delta_table(out.ctypes.data, max_len, position_buckets, max_position))
    return out


def check_cu_seqlens(cu_host: np.ndarray, total_tokens: int, max_seqlen: int) -> None:
    cu = np.ascontiguousarray(cu_host, dtype=np.int32)
    check(load().tdb_check_cu_seqlens(cu.ctypes.data, len(cu) - 1, total_tokens, max_seqlen))


def set_workgroup_limit(workgroups: int) -> int:
    """Cap the persistent workgroups (one per compute unit) of the matrix-core launches of this process;
    0 lifts the cap.  Returns the cap in force (a multiple of 8)."""
    return int(load().tdb_set_workgroup_limit(int(workgroups)))
