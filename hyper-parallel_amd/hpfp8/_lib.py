"""ctypes binding of libhpfp8.so (the C ABI declared in include/hpfp8.h).

There is no fallback: if the library is missing, or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# HPFP8_LIBRARY points at another build of the same C ABI (e.g. an instrumented one)
LIB_PATH = os.environ.get("HPFP8_LIBRARY") or os.path.join(_HERE, "libhpfp8.so")

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float

# name -> argtypes; every function returns int (status) unless noted below
SIGNATURES = {
    "hpfp8_version": [],
    "hpfp8_check_device": [],
    "hpfp8_amax_bf16": [_vp, _i64, _vp, _vp],
    "hpfp8_cast_per_tensor_bf16": [_vp, _i64, _vp, _vp, _vp, _vp, _vp],
    "hpfp8_quantize_per_tensor_bf16": [_vp, _i64, _vp, _vp, _vp, _vp, _vp],
    "hpfp8_quantize_per_tensor_sync_bf16": [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp],
    "hpfp8_quantize_per_tensor_noalloc_bf16": [_vp, _i64, _vp, _vp, _vp, _vp],
    "hpfp8_quantize_1x128_bf16": [_vp, _i64, _i64, _vp, _vp, _vp, _vp],
    "hpfp8_quantize_1x128_kmajor_bf16": [_vp, _i64, _i64, _vp, _vp, _vp, _vp],
    "hpfp8_quantize_128x1_t_kmajor_bf16": [_vp, _i64, _i64, _vp, _i64, _vp, _vp, _vp],
    "hpfp8_swiglu_quantize_1x128_bf16": [_vp, _i64, _i64, _i64, ctypes.c_int, _vp, _vp, _vp, _vp, _vp],
    "hpfp8_swiglu_quantize_1x128_pow2_bf16": [_vp, _i64, _i64, _i64, ctypes.c_int, _vp, _vp, _vp, _vp, _vp],
    "hpfp8_swiglu_quantize_1x128_and_128x1_t_bf16": [_vp, _i64, _i64, _i64, ctypes.c_int, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp],
    "hpfp8_swiglu_backward_quantize_1x128_and_128x1_t_bf16": [_vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp],
    "hpfp8_swiglu_backward_bf16": [_vp, _i64, _i64, _i64, _vp, _vp, _i64, _vp],
    "hpfp8_swiglu_quantize_1x128_fast_bf16": [_vp, _i64, _i64, _i64, ctypes.c_int, ctypes.c_int, _vp, _vp, _vp, _vp, _vp],
    "hpfp8_dequantize_1x128_accumulate_f32": [_vp, _vp, _i64, _i64, _vp, ctypes.c_float, _vp],
    "hpfp8_transpose_codes": [_vp, _i64, _i64, _i64, _vp, _i64, _vp],
    "hpfp8_bucket_pack_quantize_bf16": [_vp, _vp, _vp, ctypes.c_int, ctypes.c_int, _i64, _vp, _vp, _vp, _vp],
    "hpfp8_bucket_unpack_dequantize_bf16": [_vp, _vp, _vp, ctypes.c_int, _i64, _vp, _vp, ctypes.c_float, _vp],
    "hpfp8_quantize_1x128_and_128x1_t_bf16": [_vp, _i64, _i64, ctypes.c_int, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp],
    "hpfp8_quantize_128x128_bf16": [_vp, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _vp],
    "hpfp8_quantize_128x1_t_colsum_bf16": [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _vp, ctypes.c_int, _vp, _vp],
    "hpfp8_column_sum_finish": [_vp, _i64, _i64, _vp, _vp, _vp],
    "hpfp8_debug_transpose_traffic_model": [_vp, _i64, _i64, _vp, _i64, _vp, _vp],
    "hpfp8_column_sum_bf16": [_vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp],
    "hpfp8_quantize_1x128_kmajor_pow2_bf16": [_vp, _i64, _i64, _vp, _vp, _vp, _vp],
    "hpfp8_quantize_128x128_pow2_bf16": [_vp, _i64, _i64, _vp, _vp, _i64, _vp, _vp, _vp],
    "hpfp8_quantize_128x1_t_kmajor_pow2_bf16": [_vp, _i64, _i64, _vp, _i64, _vp, _vp, _vp],
    "hpfp8_quantize_1x128_and_128x1_t_pow2_bf16": [_vp, _i64, _i64, ctypes.c_int, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _vp],
    "hpfp8_quantize_128x1_t_bf16": [_vp, _i64, _i64, _vp, _i64, _vp, _vp, _vp],
    "hpfp8_dequantize_1x128_bf16": [_vp, _vp, _i64, _i64, _vp, _f32, _vp],
    "hpfp8_dequantize_128x128_bf16": [_vp, _vp, _i64, _i64, _vp, _vp],
    "hpfp8_dequantize_per_tensor": [_vp, _i64, _vp, _vp, _int, _vp],
    "hpfp8_gemm_blockwise": [_vp, _i64, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _int, _i64, _i64, _i64, _vp,
                             _vp, _i64, _int, _int, _vp],
    "hpfp8_gemm_blockwise_pow2": [_vp, _i64, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _int, _i64, _i64, _i64, _vp,
                                  _vp, _i64, _int, _int, _vp],
    "hpfp8_gemm_blockwise_swiglu_quantize": [_vp, _i64, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _i64,
                                             _int, _int, _int, _vp, _i64, _vp, _vp, _vp],
    "hpfp8_gemm_per_tensor": [_vp, _i64, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _int, _vp],
    "hpfp8_gemm_grouped_blockwise": [_vp, _i64, _vp, _i64, _i64, _vp, _vp, _vp, _int, _i64, _i64, _i64, _vp, _i64,
                                     _int, _vp],
    "hpfp8_gemm_grouped_blockwise_pow2": [_vp, _i64, _vp, _i64, _i64, _vp, _vp, _vp, _int, _i64, _i64, _i64, _vp, _i64,
                                          _int, _vp],
    "hpfp8_gemm_grouped_blockwise_strided": [_vp, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _int,
                                             _i64, _i64, _i64, _vp, _i64, _int, _int, _vp],
    "hpfp8_grouped_layout": [_vp, _int, _i64, _vp, _vp],
    "hpfp8_quantize_128x1_t_grouped_bf16": [_vp, _i64, _i64, _vp, _int, _vp, _i64, _vp, _vp, _vp, _vp],
    "hpfp8_gemm_grouped_wgrad": [_vp, _i64, _vp, _vp, _i64, _vp, _vp, _int, _i64, _i64, _i64, _vp, _int, _vp],
    "hpfp8_grouped_zero_unrouted_rows_bf16": [_vp, _i64, _vp, _int, _i64, _i64, _vp],
}
# functions that return a size, not a status
SIZE_FUNCTIONS = {
    "hpfp8_grouped_padded_rows": [_int, _i64],
    "hpfp8_grouped_layout_words": [_int, _i64],
}

OUT_BF16, OUT_F32 = 0, 1

_lib = None


class Hpfp8Error(RuntimeError):
    """A C-ABI call returned a negative status."""


def load():
    """Load libhpfp8.so once; raise ImportError with the build command if it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP extension has not been built. Run "
            f"`python {os.path.join(os.path.dirname(_HERE), 'build.py')}` (needs hipcc, gfx950). "
            "There is no CPU or PyTorch fallback for this path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _int
    for name, argtypes in SIZE_FUNCTIONS.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _i64
    lib.hpfp8_debug_set_spin_limit.argtypes = [ctypes.c_uint32]
    lib.hpfp8_debug_set_spin_limit.restype = None
    lib.hpfp8_debug_set_small_gemm.argtypes = [_int]
    lib.hpfp8_debug_set_small_gemm.restype = None
    lib.hpfp8_last_error.argtypes = []
    lib.hpfp8_last_error.restype = ctypes.c_char_p
    _lib = lib
    return lib


def call(name: str, *args) -> None:
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.hpfp8_last_error().decode("utf-8", "replace")
        raise Hpfp8Error(f"{name} failed ({rc}): {msg}")
