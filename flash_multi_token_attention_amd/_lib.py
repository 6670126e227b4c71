"""ctypes binding of libconvattn_hip.so (the C ABI declared in include/convattn.h)."""
from __future__ import annotations

import ctypes as C
import os
import threading

_PKG = os.path.dirname(os.path.abspath(__file__))
# CONVATTN_LIB points at another build of the same C ABI (e.g. an instrumented one).
LIB_PATH = os.environ.get("CONVATTN_LIB") or os.path.join(_PKG, "libconvattn_hip.so")

BF16, F32 = 0, 1
OP_FWD, OP_BWD, OP_DECODE = 0, 1, 2
FLAG_EXACT = 1
FLAG_LOW_MEMORY = 2
ERR_QROWS = -8


class Desc(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("H", C.c_int32), ("Nq", C.c_int32), ("Nk", C.c_int32), ("d", C.c_int32),
        ("c_q", C.c_int32), ("c_k", C.c_int32),
        ("scale", C.c_float),
        ("causal", C.c_int32),
        ("in_dtype", C.c_int32), ("out_dtype", C.c_int32),
        ("n_splits", C.c_int32),
        ("flags", C.c_uint32),
    ]


class KvLayout(C.Structure):
    """struct convattn_kv_layout of include/convattn.h."""
    _fields_ = [
        ("H_kv", C.c_int32), ("page_size", C.c_int32),
        ("batch_stride", C.c_int64), ("head_stride", C.c_int64), ("page_stride", C.c_int64),
        ("block_table", C.c_void_p),
        ("table_stride", C.c_int32), ("reserved", C.c_int32),
        ("seq_lens", C.c_void_p),
    ]


class HeadmixDesc(C.Structure):
    """struct convattn_headmix_desc of include/convattn.h."""
    _fields_ = [
        ("B", C.c_int32), ("H", C.c_int32), ("N", C.c_int32), ("d", C.c_int32),
        ("scale", C.c_float), ("causal", C.c_int32),
        ("in_dtype", C.c_int32), ("out_dtype", C.c_int32),
    ]


_P = C.c_void_p
_D = C.POINTER(Desc)
_HD = C.POINTER(HeadmixDesc)
_SIGNATURES = {
    "convattn_version": (C.c_int, []),
    "convattn_strerror": (C.c_char_p, [C.c_int]),
    "convattn_validate": (C.c_int, [_D, C.c_int]),
    "convattn_kernel_path": (C.c_int, [_D, C.c_int]),
    "convattn_fwd": (C.c_int, [_D] + [_P] * 8),
    "convattn_bwd_preprocess": (C.c_int, [_D] + [_P] * 7),
    "convattn_dw_partial_bytes": (C.c_size_t, [_D]),
    "convattn_bwd_dq_dw": (C.c_int, [_D] + [_P] * 10),
    "convattn_dw_reduce": (C.c_int, [_D] + [_P] * 3),
    "convattn_bwd_dkdv": (C.c_int, [_D] + [_P] * 10),
    "convattn_bwd_fused_workspace_bytes": (C.c_size_t, [_D]),
    "convattn_bwd_fused": (C.c_int, [_D] + [_P] * 13),
    "convattn_bwd_fused_dkdv": (C.c_int, [_D] + [_P] * 11),
    "convattn_bwd_fused_dq": (C.c_int, [_D] + [_P] * 10),
    "convattn_bwd_fused_dw": (C.c_int, [_D] + [_P] * 3),
    "convattn_decode_partial_bytes": (C.c_size_t, [_D]),
    "convattn_decode": (C.c_int, [_D] + [_P] * 8),
    "convattn_decode_strided": (C.c_int, [_D] + [_P] * 4 + [C.c_longlong] * 2 + [_P] * 4),
    "convattn_decode_kv": (C.c_int, [_D] + [_P] * 3 + [C.POINTER(KvLayout)] + [_P] * 5),
    "convattn_decode_combine": (C.c_int, [_D] + [_P] * 7),
    "convattn_decode_noalloc_bytes": (C.c_size_t, [_D]),
    "convattn_decode_noalloc": (C.c_int, [_D] + [_P] * 4 + [C.c_longlong] * 2 + [_P] * 4),
    "convattn_headmix_validate": (C.c_int, [_HD]),
    "convattn_headmix_fwd": (C.c_int, [_HD] + [_P] * 8),
    "convattn_headmix_bwd_workspace_bytes": (C.c_size_t, [_HD]),
    "convattn_headmix_bwd_dq_dw": (C.c_int, [_HD] + [_P] * 12),
    "convattn_headmix_bwd_dkdv": (C.c_int, [_HD] + [_P] * 12),
}
EXPORTS = tuple(_SIGNATURES)

_lib = None
_lock = threading.Lock()


def load() -> C.CDLL:
    """The loaded library; raises if it has not been built (there is no fallback)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build it with "
                    "`python -m flash_multi_token_attention_amd.build` (needs hipcc); "
                    "this package has no non-HIP code path")
            lib = C.CDLL(LIB_PATH)
            for name, (res, args) in _SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype, fn.argtypes = res, args
            _lib = lib
    return _lib


def strerror(code: int) -> str:
    return load().convattn_strerror(int(code)).decode()


def check(code: int, what: str) -> None:
    if code == 0:
        return
    msg = f"{what}: {strerror(code)}"
    if code > 0:
        msg += f" (hipError_t {code})"
    raise RuntimeError(msg)
