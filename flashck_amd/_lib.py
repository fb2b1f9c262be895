"""ctypes binding of libflashck_fmha.so (the C ABI declared in include/flashck/fmha/fmha_c_api.h).

The library is the only compute path: when it is missing the import of any operator fails with an error that
says how to build it; nothing falls back to another implementation.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# the one library the operators use: the in-tree build next to this file (no environment override)
LIB_PATH = os.path.join(_HERE, "libflashck_fmha.so")

_vp, _i64, _i32, _u32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_uint32, ctypes.c_float

class Attrs(ctypes.Structure):
    """fck_fmha_attrs of the header."""
    _fields_ = [("size", ctypes.c_uint32), ("bias_type", ctypes.c_int32), ("bias", ctypes.c_void_p),
                ("bias_batch_stride", ctypes.c_int64), ("bias_head_stride", ctypes.c_int64), ("bias_row_stride", ctypes.c_int64),
                ("logits_soft_cap", ctypes.c_float), ("kv_dtype", ctypes.c_int32), ("k_descale", ctypes.c_float),
                ("v_descale", ctypes.c_float), ("decode_variant", ctypes.c_int32), ("prefill_variant", ctypes.c_int32),
                ("bias_cols", ctypes.c_int64), ("max_seqlen_k", ctypes.c_int64), ("o_scale", ctypes.c_float)]


_ap = ctypes.POINTER(Attrs)

# name -> (restype, argtypes); order and types follow the header
SIGNATURES = {
    "fck_last_error": (ctypes.c_char_p, []),
    "fck_fmha_version": (ctypes.c_char_p, []),
    "fck_fmha_last_kernel": (ctypes.c_char_p, []),
    "fck_fmha_fwd": (ctypes.c_int, [_vp] * 8 + [_i64] * 8 + [_f32, _i64, _i64, _u32, _i32, _vp]),
    "fck_fmha_fwd_attrs": (ctypes.c_int, [_vp] * 8 + [_i64] * 8 + [_f32, _i64, _i64, _u32, _i32, _ap, _vp]),
    "fck_fmha_fwd_splitkv_attrs": (ctypes.c_int, [_vp] * 11 + [_i64] * 11 + [_f32, _i64, _i64, _u32, _i32, _ap, _vp]),
    "fck_fmha_batch_prefill_attrs": (ctypes.c_int, [_vp] * 8 + [_i64] * 8 + [_f32, _i64, _i64, _u32, _i32, _ap, _vp]),
    "fck_fmha_fwd_pagedkv_attrs": (ctypes.c_int, [_vp] * 7 + [_i64] * 9 + [_f32, _i64, _i64, _u32, _i32, _ap, _vp]),
    "fck_fmha_fwd_splitkv": (ctypes.c_int, [_vp] * 11 + [_i64] * 11 + [_f32, _i64, _i64, _u32, _i32, _vp]),
    "fck_fmha_fwd_splitkv_fused": (ctypes.c_int, [_vp] * 10 + [_i64] * 11 + [_f32, _i64, _i64, _u32, _i32, _vp]),
    "fck_fmha_fused_reset": (ctypes.c_int, [_vp]),
    "fck_fmha_validate_paged": (ctypes.c_int, [_vp] * 6 + [_i64] * 3 + [_vp, _vp]),
    "fck_fmha_fwd_splitkv_combine": (ctypes.c_int, [_vp] * 4 + [_i64] * 6 + [_i32, _vp]),
    "fck_fmha_fwd_appendkv": (ctypes.c_int, [_vp] * 7 + [_i64, _vp, _vp, _i64, _i32, _i32, _vp, _i64, _i64, _vp]
                              + [_i64] * 6 + [_i32, _vp]),
    "fck_fmha_fwd_appendkv_attrs": (ctypes.c_int, [_vp] * 7 + [_i64, _vp, _vp, _i64, _i32, _i32, _vp, _i64, _i64, _vp]
                                    + [_i64] * 6 + [_i32, _ap, _vp]),
    "fck_fmha_batch_prefill": (ctypes.c_int, [_vp] * 8 + [_i64] * 8 + [_f32, _i64, _i64, _u32, _i32, _vp]),
    "fck_fmha_fwd_pagedkv": (ctypes.c_int, [_vp] * 7 + [_i64] * 9 + [_f32, _i64, _i64, _u32, _i32, _vp]),
    "fck_fmha_num_splits_heuristic": (ctypes.c_int, [_i64] * 7),
    "fck_fmha_splitkv_workspace_bytes": (ctypes.c_size_t, [_i64] * 5),
}

_lib = None


class FlashCKLibraryError(RuntimeError):
    pass


def load():
    """Load the library once; raises FlashCKLibraryError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FlashCKLibraryError(
                f"{LIB_PATH} is missing: build it with `python -m flashck_amd.build` (needs hipcc); "
                "there is no fallback implementation")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def last_error():
    return load().fck_last_error().decode()
