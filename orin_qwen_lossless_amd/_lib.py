"""ctypes binding of libbf16n_hip.so (C ABI declared in include/bf16n_c.h).  The library must have been built
(python -m orin_qwen_lossless_amd.build); there is no fallback path: loading fails loudly when it is missing."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libbf16n_hip.so")

OK, EINVAL, ERUNTIME = 0, 1, 2


class Weight(C.Structure):
    _fields_ = [("plane", C.c_void_p), ("aux", C.c_void_p), ("format", C.c_int32), ("R", C.c_int32), ("K", C.c_int64),
                ("rows", C.c_int64), ("flags", C.c_uint32), ("pad_", C.c_uint32), ("off_a", C.c_uint64),
                ("off_b", C.c_uint64), ("off_c", C.c_uint64), ("off_d", C.c_uint64)]


class MmvArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("y", C.c_void_p), ("ids", C.c_void_p), ("x_tok", C.c_int64), ("y_tok", C.c_int64),
                ("ids_s0", C.c_int64), ("ids_s1", C.c_int64), ("x_slot", C.c_int64), ("y_slot", C.c_int64),
                ("rows_per_matrix", C.c_int64), ("row0", C.c_int64), ("nrows", C.c_int64), ("ncols", C.c_int32),
                ("n_used", C.c_int32), ("x_per_slot", C.c_int32), ("x_bf16", C.c_uint8), ("y_bf16", C.c_uint8),
                ("pad_", C.c_uint8 * 2)]


# name -> (restype, argtypes); every symbol declared in include/bf16n_c.h
_i, _i64, _u32, _vp, _cp = C.c_int, C.c_int64, C.c_uint32, C.c_void_p, C.c_char_p
_WP, _AP = C.POINTER(Weight), C.POINTER(MmvArgs)
SYMBOLS = {
    "bf16n_last_error": (_cp, []),
    "bf16n_last_kernel": (_cp, []),
    "bf16n_encode": (_i, [_vp, _i64, _i64, _i, _i, _u32, C.POINTER(_vp)]),
    "bf16n_encoded_plane": (_vp, [_vp, C.POINTER(C.c_uint64)]),
    "bf16n_encoded_aux": (_vp, [_vp, C.POINTER(C.c_uint64)]),
    "bf16n_encoded_format": (_i, [_vp]),
    "bf16n_encoded_R": (_i, [_vp]),
    "bf16n_encoded_free": (None, [_vp]),
    "bf16n_set_encode_threads": (None, [_i]),
    "bf16n_choose": (_i, [_i64, _i64, _i64, _i, _i, _i64, _i, _i, C.POINTER(_i)]),
    "bf16n_init": (_i, []),
    "bf16n_cu_count": (_i, [C.POINTER(_i)]),
    "bf16n_mmv": (_i, [_WP, _AP, _vp, _i]),
    "bf16n_gemv_max_tokens": (_i, [_WP, C.POINTER(_i)]),
    "bf16n_linear_dense_sizes": (_i, [_WP, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "bf16n_linear_dense": (_i, [_WP, _vp, _i64, _i, _vp, _i64, _vp, C.c_uint64, _vp, C.c_uint64, _vp]),
    "bf16n_mmv_glu": (_i, [_WP, _AP, _vp]),
    "bf16n_mmv_glu2": (_i, [_WP, _WP, _AP, _vp]),
    "bf16n_mmv_glu2_topk": (_i, [_WP, _WP, _AP, _vp, _i64, _i, _i, _i, _vp, _i64, _vp]),
    "bf16n_dequant": (_i, [_WP, _i64, _i64, _vp, _vp]),
    "bf16n_get_rows": (_i, [_WP, _vp, _i64, _i64, _vp, _i, _i64, _vp, _i64]),
    "bf16n_mm_ids_supported": (_i, [_WP, _WP]),
    "bf16n_mm_ids_route": (_i, [_vp, _i, _i64, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "bf16n_mm_ids": (_i, [_WP, _WP, _vp, _i64, _vp, _vp, _vp, _vp, _i, _i64, _i, _i, _i, _vp]),
    "bf16n_mm_ids_scratch_bytes": (_i, [_WP, _WP, _i, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "bf16n_mm_ids_scratch": (_i, [_WP, _WP, _vp, _i64, _vp, _vp, _vp, _vp, _i, _i64, _i, _vp, C.c_uint64, _vp]),
    "bf16n_moe_mm_ids_static": (_i, [_WP, _WP, _vp, _i64, _vp, _i, _i64, _i, _vp, _i, _i64, _i, _i, _i, _vp]),
    "bf16n_moe_combine": (_i, [_vp, _vp, _i, _vp, _i, _i, _i, _i64, _vp]),
    "bf16n_add_rmsnorm": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _i, _i64, C.c_float, _vp]),
    "bf16n_swiglu": (_i, [_vp, _vp, _vp, _i64, _vp]),
    "bf16n_router_topk": (_i, [_vp, _i64, _i, _i, _i, _i, _vp, _vp, _vp]),
    "bf16n_router_topk_strided": (_i, [_vp, _i64, _i, _i, _i, _i, _vp, _vp, _i64, _vp]),
    "bf16n_router_topk_route_fits": (_i, [_i, _i, _i]),
    "bf16n_router_topk_route": (_i, [_vp, _i64, _i, _i, _i, _i, _vp, _vp, _i64, _i, _i, _vp, _vp, _vp, _i, _i, _vp]),
    "bf16n_adapter_choose": (_i, [_i64, _i64, _i64, _cp, _i64, _i, _i]),
    "bf16n_adapter_convert": (_i, [_vp, _vp, _i64, _i64, _i64, _i, _i, _i, _vp, _cp, _i, C.POINTER(_i)]),
    "bf16n_verify_roundtrip": (_i, [_WP, _vp, C.POINTER(_i)]),
    "bf16n_adapter_register": (_i, [_WP, _vp]),
    "bf16n_adapter_lookup": (_i, [_vp, _WP, C.POINTER(_i64), C.POINTER(_i)]),
    "bf16n_adapter_release": (_i, [_vp, C.POINTER(_i)]),
    "bf16n_adapter_count": (_i, []),
}

_lib = None


def lib():
    """The loaded library. Raises OSError with the build command when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError(f"{LIB_PATH} is missing: build it with `python -m orin_qwen_lossless_amd.build` "
                          "(there is no CPU or eager fallback for the BF16N kernels)")
        _lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(_lib, name)
            fn.restype = res
            fn.argtypes = args
    return _lib


def check(status: int) -> None:
    """Map a C ABI status to the exceptions of the reference's torch binding (ValueError for std::invalid_argument,
    core/torch/torch_bindings.cpp:102-107; RuntimeError otherwise)."""
    if status == OK:
        return
    msg = lib().bf16n_last_error().decode()
    if status == EINVAL:
        raise ValueError(msg)
    raise RuntimeError(msg)
