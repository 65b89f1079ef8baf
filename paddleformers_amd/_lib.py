"""ctypes binding of libpf8.so (the C ABI declared in include/pf8.h).

The library is the only compute path: if it is missing, or a call is made without a GPU tensor,
this module raises -- there is no CPU or framework fallback.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpf8.so")

_lib = None

_i64, _i32, _vp = C.c_int64, C.c_int, C.c_void_p

# name -> argtypes; mirrors include/pf8.h (and the self-test hooks of include/pf8_selftest.h) one for one
SIGNATURES = {
    "pf8_version": [],
    "pf8_set_num_cus": [_i32],
    "pf8_get_num_cus": [],
    "pf8_effective_num_cus": [],
    "pf8_quant_1x128": [_vp, _i64, _i64, _i64, _vp, _vp, _i32, _i32, _vp],
    "pf8_quant_128x128": [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _i32, _vp],
    "pf8_quant_transpose": [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _i32, _i32, _vp],
    "pf8_stack_transpose_quant": [_vp, _i32, _i64, _i64, _i32, _vp, _vp, _i32, _vp],
    "pf8_stack_quant_both": [_vp, _i32, _i64, _i64, _vp, _vp, _vp, _vp, _i32, _vp],
    "pf8_stack_quant_both_fm": [_vp, _i32, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp],
    "pf8_swiglu_weighted_quant": [_vp, _vp, _i64, _i64, _vp, _vp, _vp, _i32, _i32, _vp],
    "pf8_transpose_split_quant": [_vp, _vp, _i32, _i32, _vp, _i32, _i64, _vp, _vp, _i32, _vp],
    "pf8_transpose_split_quant_gather": [_vp, _vp, _i32, _i32, _i64, _vp, _vp, _i32, _i64, _vp, _vp, _i32, _vp],
    "pf8_quant_and_transpose_split": [_vp, _vp, _i32, _i64, _vp, _vp, _i32, _vp, _vp, _i32, _vp],
    "pf8_act_dequant": [_vp, _vp, _i32, _i64, _i64, _vp, _vp],
    "pf8_weight_dequant": [_vp, _vp, _i64, _i64, _vp, _vp],
    "pf8_block_dequant": [_vp, _vp, _i32, _i64, _i64, _i64, _i64, _i64, _vp, _i32, _vp],
    "pf8_moe_permute": [_vp, _i32, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _vp, _i32, _vp, _vp, _vp, _vp, _vp, _vp],
    "pf8_moe_permute_map": [_vp, _vp, _i64, _i32, _i32, _vp, _i32, _vp, _vp, _vp, _vp, _vp],
    "pf8_moe_unpermute": [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _vp, _vp, _vp],
    "pf8_rms_norm_fwd": [_vp, _vp, C.c_float, _i64, _i64, _vp, _vp, _vp],
    "pf8_rms_norm_bwd": [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _i64, _vp],
    "pf8_swiglu_weighted_bwd": [_vp, _vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp],
    "pf8_swiglu_weighted_bwd_quant": [_vp, _vp, _vp, _vp, _i32, _i64, _vp, _vp, _i32, _i32, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp],
    "pf8_gemm_nt": [_vp, _vp, _i32, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp],
    "pf8_gemm_nt_1d1d_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i32, _vp],
    "pf8_gemm_nt_1d1d_f32_pow2": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i32, _vp],
    "pf8_grouped_gemm_nt_contiguous": [_vp, _vp, _i32, _vp, _vp, _i32, _i64, _i64, _i64, _vp, _vp, _vp],
    "pf8_weight_to_fragment_major": [_vp, _i32, _i64, _i64, _vp, _vp],
    "pf8_gemm_fm_supported": [_i64, _i64, _i64],
    "pf8_gemm_nt_fm": [_vp, _vp, _i32, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp],
    "pf8_grouped_gemm_nt_contiguous_fm": [_vp, _vp, _i32, _vp, _vp, _i32, _i64, _i64, _i64, _vp, _vp, _vp],
    "pf8_grouped_gemm_nt_contiguous_fm_gather": [_vp, _i64, _vp, _vp, _i32, _vp, _vp, _i32, _i64, _i64, _i64, _vp, _vp, _vp],
    "pf8_gather_row_scales": [_vp, _i64, _i64, _vp, _i64, _vp, _i32, _vp],
    "pf8_grouped_gemm_swiglu_quant_nt_contiguous": [_vp, _vp, _i32, _vp, _vp, _i32, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i32, _vp],
    "pf8_gemm_nt_ue8m0": [_vp, _vp, _i64, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp],
    "pf8_grouped_gemm_nt_contiguous_ue8m0": [_vp, _vp, _i64, _vp, _vp, _i32, _i64, _i64, _i64, _vp, _vp, _vp, _vp],
    "pf8_grouped_gemm_nt_contiguous_ue8m0_noalloc": [_vp, _vp, _i64, _vp, _vp, _i32, _i64, _i64, _i64, _vp, _vp, _vp],
    "pf8_scales_to_ue8m0": [_vp, _i64, _vp, _vp, _vp],
    "pf8_grouped_items_build": [_vp, _i64, _vp, _vp],
    "pf8_grouped_gemm_nt_masked": [_vp, _vp, _vp, _vp, _i32, _i64, _i64, _i64, _vp, _i32, _vp, _vp],
    "pf8_grouped_wgrad": [_vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp, _i32, _vp],
    "pf8_grouped_wgrad_pow2": [_vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp, _i32, _vp],
    "pf8_debug_grouped_gemm_fm_cycles": [_vp, _vp, _vp, _vp, _i32, _i64, _i64, _i64, _vp, _vp, _vp, _i64, _i32, _vp],
    "pf8_debug_copy": [_vp, _vp, _i64, _vp],
    "pf8_debug_encode": [_vp, _i64, _vp, _vp],
    "pf8_debug_div_encode": [_vp, _vp, _i64, _vp, _vp],
    "pf8_debug_silu": [_vp, _i64, _vp, _vp],
    "pf8_debug_silu_sigmoid": [_vp, _i64, _vp, _vp, _vp],
    "pf8_debug_set_wgrad_tile256_min_blocks": [_i32],
}


class Pf8Error(RuntimeError):
    """A libpf8 entry point returned a negative status."""


def lib():
    """Load libpf8.so once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m paddleformers_amd.build` (needs hipcc). "
                "There is no fallback path."
            )
        handle = C.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = C.c_int
        handle.pf8_last_error.argtypes = []
        handle.pf8_last_error.restype = C.c_char_p
        _lib = handle
    return _lib


def last_error() -> str:
    return lib().pf8_last_error().decode("utf-8", "replace")


def call(name: str, *args) -> None:
    """Call an entry point and turn a negative status into the exception the reference would raise
    (ValueError for bad arguments, RuntimeError otherwise)."""
    rc = getattr(lib(), name)(*args)
    if rc != 0:
        msg = f"{name} failed ({rc}): {last_error()}"
        if rc == -1:
            raise ValueError(msg)
        raise Pf8Error(msg)
