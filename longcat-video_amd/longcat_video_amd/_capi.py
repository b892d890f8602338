"""ctypes binding of libbsa_mi355x.so (declared in include/bsa_mi355x.h).

The library is loaded from the package's ``lib`` directory; a missing library is
an error, never a reason to fall back to another implementation.
"""
from __future__ import annotations

import ctypes as C
import os

BSA_OK = 0
BSA_ERR_BAD_ARG = -1
BSA_ERR_UNSUPPORTED = -2
BSA_ERR_SHAPE = -3
BSA_ERR_WORKSPACE = -4
BSA_ERR_HIP = -5
BSA_ERR_BUSY = -6

BSA_BF16, BSA_F16, BSA_F32 = 0, 1, 2
BSA_STATIC_SCRATCH_BYTES = 64 << 20

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libbsa_mi355x.so")


class Bsa3dParams(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "B", "Hn", "D", "dtype", "Tq", "Hq", "Wq", "Tk", "Hk", "Wk",
        "tq", "hq", "wq", "tk", "hk", "wk", "k_sel")] + [("sm_scale", C.c_float), ("cdf_threshold", C.c_float)]


class BsaQkNorm(C.Structure):
    _fields_ = [("q_weight", C.c_void_p), ("k_weight", C.c_void_p), ("rope_table", C.c_void_p), ("table_T", C.c_int),
                ("t_offset_q", C.c_int), ("t_offset_k", C.c_int), ("eps", C.c_float)]


_i, _i64, _p, _f = C.c_int, C.c_int64, C.c_void_p, C.c_float
_strides = C.POINTER(C.c_int64)

# name -> (restype, argtypes); the order follows include/bsa_mi355x.h
SIGNATURES = {
    "bsa_version": (_i, []),
    "bsa_last_error": (C.c_char_p, []),
    "bsa_num_selected": (_i, [C.c_double, _i]),
    "bsa_padded_tokens": (_i64, [_i] * 6),
    "bsa_permute_thw_to_blocks": (_i, [_p, _strides, _p, _p, _p] + [_i] * 10 + [_p]),
    "bsa_unpermute_blocks_to_thw": (_i, [_p, _p, _strides] + [_i] * 10 + [_p]),
    "bsa_mean_pool": (_i, [_p, _p, _i, _i, _i64, _i, _i, _i, _p]),
    "bsa_score_topk": (_i, [_p, _p, _p, _p, _p, _p] + [_i] * 7 + [_p]),
    "bsa_topk_from_score": (_i, [_p, _p, _p, _p] + [_i] * 6 + [_p]),
    "bsa_visit_order": (_i, [_p, _p, _p, _i64, _i, _i, _p]),
    "bsa_score_cdf": (_i, [_p, _p, _p, _p, _p, _p] + [_i] * 5 + [_f, _f, _i, _i, _i, _p]),
    "bsa_cdf_from_score": (_i, [_p, _p, _p, _p] + [_i] * 4 + [_f, _f, _i, _i, _i, _p]),
    "bsa_fwd": (_i, [_p] * 8 + [_i, _i, _i64, _i64, _i, _i, _i, _i, _f, _i, _p]),
    "bsa_fwd_fragment_workspace_bytes": (C.c_size_t, [_i, _i, _i64, _i64, _i, _i]),
    "bsa_fwd_fragment": (_i, [_p] * 8 + [_i, _i, _i64, _i64, _i, _i, _i, _i, _f, _i, _p, C.c_size_t, _p]),
    "bsa_bwd_workspace_bytes": (C.c_size_t, [_i, _i, _i64, _i64, _i, _i, _i, _i, _i]),
    "bsa_bwd": (_i, [_p] * 12 + [_i, _i, _i64, _i64, _i, _i, _i, _i, _f, _i, _p, C.c_size_t, _p]),
    "bsa_bwd_3d_workspace_bytes": (C.c_size_t, [C.POINTER(Bsa3dParams), _i]),
    "bsa_bwd_3d": (_i, [C.POINTER(Bsa3dParams)] + [_p, _strides] * 5 + [_p, _p, _p, _i] + [_p, _strides] * 3 + [_p, C.c_size_t, _p]),
    "bsa_workspace_bytes": (C.c_size_t, [C.POINTER(Bsa3dParams)]),
    "bsa_fwd_3d": (_i, [C.POINTER(Bsa3dParams), _p, _strides, _p, _strides, _p, _strides, _p, _strides,
                        _p, C.c_size_t, _p, _p, _p, _p]),
    "bsa_fwd_3d_lse": (_i, [C.POINTER(Bsa3dParams), _p, _strides, _p, _strides, _p, _strides, _p, _strides,
                            _p, _p, _p, _p, C.c_size_t, _p]),
    "bsa_fwd_3d_qknorm": (_i, [C.POINTER(Bsa3dParams), C.POINTER(BsaQkNorm), _p, _strides, _p, _strides, _p, _strides, _p, _strides,
                               _p, _strides, _p, C.c_size_t, _p, _p, _p, _p]),
    "bsa_fwd_3d_static": (_i, [C.POINTER(Bsa3dParams), _p, _strides, _p, _strides, _p, _strides, _p, _strides,
                               _p, _p, _p, _p]),
    "bsa_thw_prepare": (_i, [C.POINTER(Bsa3dParams), _p, _strides, _p, _strides, _p, C.c_size_t, _p]),
    "bsa_fwd_thw": (_i, [C.POINTER(Bsa3dParams), _p, _strides, _p, _strides, _p, _strides, _p, _strides,
                         _p, _p, _i, _p, _p, C.c_size_t, _p]),
    "bsa_rmsnorm": (_i, [_p, _p, _p, _i64, _i, _f, _i, _p]),
    "bsa_layernorm_modulate": (_i, [_p, _p, _p, _p, _i64, _i, _i, _f, _i, _p]),
    "bsa_gated_residual": (_i, [_p, _p, _p, _p, _i64, _i, _i, _i, _p]),
    "bsa_norm_rope": (_i, [_p, _strides, _p, _strides, _p, _p] + [_i] * 8 + [_f, _i, _p]),
    "bsa_qk_norm_rope": (_i, [_p, _strides, _p, _strides, _p, _p, _p] + [_i] * 6 + [_f, _i, _p]),
    "bsa_linear_bf16": (_i, [_p, _p, _p, _p, _p, _i64, _i, _i, _p, C.c_size_t, _p]),
    "bsa_linear_bf16_ld": (_i, [_p, _i64, _p, _i64, _p, _p, _p, _i64, _i64, _i, _i, _p, C.c_size_t, _p]),
    "bsa_linear_bf16_tune": (_i, [_p, _i64, _p, _i64, _p, _p, _p, _i64, _i64, _i, _i, _p, C.c_size_t, _p, _p, _p]),
    "bsa_lora_add": (_i, [_p, _p, _p, _p, _i, _p, _i64, _i, _p]),
    "bsa_gemm_bf16": (_i, [_p, _i64, _p, _i64, _p, _p, _i64, _p, _i64, _i64, _i, _i, _p]),
    "bsa_qkv_projection": (_i, [_p, _i64, _p, _i64, _p, _p, _p, _p, _p, _p, _p, _strides] + [_i] * 9 + [_f, _p]),
}

_lib = None


def load() -> C.CDLL:
    """Loads the engine (once) and types every entry point the header declares."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libbsa_mi355x.so is not built (%s); run `python longcat-video_amd/build.py`" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)      # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def last_error() -> str:
    return load().bsa_last_error().decode("utf-8", "replace")


def strides3(values) -> C.Array:
    return (C.c_int64 * 3)(*[int(v) for v in values])


def check(status: int, what: str = "") -> None:
    """Maps a bsa_status to the exception the reference raises in that case:
    shape violations are AssertionError (bsa_interface.py:627-640, 543-544)."""
    if status == BSA_OK:
        return
    msg = "%s%s" % (what + ": " if what else "", last_error())
    if status == BSA_ERR_SHAPE:
        raise AssertionError(msg)
    if status == BSA_ERR_BAD_ARG:
        raise ValueError(msg)
    if status == BSA_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)          # workspace, HIP and busy errors
