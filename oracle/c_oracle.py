"""ctypes binding of the C restatement of the oracle (fp8_oracle.c).  TEST INFRASTRUCTURE ONLY.

Arrays are numpy: bf16 tensors as uint16 bit patterns, codes as uint8, scales as float32.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libfp8_oracle.so")
_lib = None

_u16p = ctypes.POINTER(ctypes.c_uint16)
_u8p = ctypes.POINTER(ctypes.c_uint8)
_f32p = ctypes.POINTER(ctypes.c_float)
_i64 = ctypes.c_int64


def build(force: bool = False) -> str:
    """Compile fp8_oracle.c with gcc (seconds)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        l = ctypes.CDLL(_LIB_PATH)
        l.hpo_e4m3_decode.argtypes = [ctypes.c_uint8]
        l.hpo_e4m3_decode.restype = ctypes.c_float
        l.hpo_e4m3_encode.argtypes = [ctypes.c_float]
        l.hpo_e4m3_encode.restype = ctypes.c_uint8
        l.hpo_amax_bf16.argtypes = [_u16p, _i64]
        l.hpo_amax_bf16.restype = ctypes.c_float
        l.hpo_quantize_per_tensor.argtypes = [_u16p, _i64, _u8p, _f32p, _f32p]
        l.hpo_quantize_1x128.argtypes = [_u16p, _i64, _i64, _u8p, _f32p, _f32p]
        l.hpo_quantize_128x128.argtypes = [_u16p, _i64, _i64, _u8p, _f32p, _f32p]
        l.hpo_quantize_128x1_t.argtypes = [_u16p, _i64, _i64, _u8p, _f32p, _f32p]
        l.hpo_dequantize_1x128.argtypes = [_u8p, _f32p, _i64, _i64, _u16p]
        l.hpo_gemm_blockwise.argtypes = [_u8p, _f32p, _u8p, _f32p, _i64, _i64, _i64, ctypes.c_int,
                                         _f32p, _f32p, _u16p]
        l.hpo_num_threads.restype = ctypes.c_int
        l.hpo_scales_pow2.argtypes = [ctypes.c_float, _f32p, _f32p]
        l.hpo_scales_pow2.restype = None
        l.hpo_exp_spec.argtypes = [ctypes.c_float]
        l.hpo_exp_spec.restype = ctypes.c_float
        l.hpo_swiglu.argtypes = [_u16p, _i64, _i64, _u16p]
        l.hpo_swiglu.restype = None
        for name in ("hpo_quantize_per_tensor", "hpo_quantize_1x128", "hpo_quantize_128x128",
                     "hpo_quantize_128x1_t", "hpo_dequantize_1x128", "hpo_gemm_blockwise"):
            getattr(l, name).restype = None
        _lib = l
    return _lib


def _p(a, t):
    return a.ctypes.data_as(t)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def num_threads() -> int:
    return int(lib().hpo_num_threads())


def e4m3_encode(x: np.ndarray) -> np.ndarray:
    l = lib()
    flat = _c(x, np.float32).reshape(-1)
    return np.fromiter((l.hpo_e4m3_encode(float(v)) for v in flat), dtype=np.uint8,
                       count=flat.size).reshape(np.shape(x))


def e4m3_decode(codes: np.ndarray) -> np.ndarray:
    l = lib()
    flat = _c(codes, np.uint8).reshape(-1)
    return np.array([l.hpo_e4m3_decode(int(v)) for v in flat], dtype=np.float32).reshape(np.shape(codes))


def quantize_per_tensor(x_bits):
    x = _c(x_bits, np.uint16)
    q = np.empty(x.shape, np.uint8)
    s = np.empty(1, np.float32)
    si = np.empty(1, np.float32)
    lib().hpo_quantize_per_tensor(_p(x, _u16p), x.size, _p(q, _u8p), _p(s, _f32p), _p(si, _f32p))
    return q, s[0], si[0]


def _blocked(fn, x_bits, sshape, qshape=None):
    x = _c(x_bits, np.uint16)
    q = np.empty(qshape or x.shape, np.uint8)
    s = np.empty(sshape, np.float32)
    si = np.empty(sshape, np.float32)
    fn(_p(x, _u16p), x.shape[0], x.shape[1], _p(q, _u8p), _p(s, _f32p), _p(si, _f32p))
    return q, s, si


def quantize_1x128(x_bits):
    r, c = x_bits.shape
    return _blocked(lib().hpo_quantize_1x128, x_bits, (r, c // 128))


def quantize_128x128(w_bits):
    r, c = w_bits.shape
    return _blocked(lib().hpo_quantize_128x128, w_bits, (r // 128, c // 128))


def quantize_128x1_t(x_bits):
    m, k = x_bits.shape
    return _blocked(lib().hpo_quantize_128x1_t, x_bits, (k, m // 128), qshape=(k, m))


def dequantize_1x128(codes, scale_inv):
    q = _c(codes, np.uint8)
    si = _c(scale_inv, np.float32)
    out = np.empty(q.shape, np.uint16)
    lib().hpo_dequantize_1x128(_p(q, _u8p), _p(si, _f32p), q.shape[0], q.shape[1], _p(out, _u16p))
    return out


def gemm_blockwise(a, sa_inv, b, sb_inv, sb_per_row=False, bias_f32=None):
    a = _c(a, np.uint8)
    b = _c(b, np.uint8)
    sa = _c(sa_inv, np.float32)
    sb = _c(sb_inv, np.float32)
    m, k = a.shape
    n = b.shape[0]
    out = np.empty((m, n), np.float32)
    out_b = np.empty((m, n), np.uint16)
    bias = None if bias_f32 is None else _c(bias_f32, np.float32)
    lib().hpo_gemm_blockwise(_p(a, _u8p), _p(sa, _f32p), _p(b, _u8p), _p(sb, _f32p), m, n, k,
                             int(bool(sb_per_row)), None if bias is None else _p(bias, _f32p),
                             _p(out, _f32p), _p(out_b, _u16p))
    return out, out_b


def scales_pow2(amax: np.ndarray):
    """(scale, scale_inv) of the power-of-two recipe for every amax of an array."""
    l = lib()
    flat = _c(amax, np.float32).reshape(-1)
    s = np.empty(flat.size, np.float32)
    si = np.empty(flat.size, np.float32)
    a, b = ctypes.c_float(), ctypes.c_float()
    for i, v in enumerate(flat):
        l.hpo_scales_pow2(float(v), ctypes.byref(a), ctypes.byref(b))
        s[i], si[i] = a.value, b.value
    return s.reshape(np.shape(amax)), si.reshape(np.shape(amax))


def exp_spec(t: np.ndarray) -> np.ndarray:
    l = lib()
    flat = _c(t, np.float32).reshape(-1)
    return np.array([l.hpo_exp_spec(float(v)) for v in flat], dtype=np.float32).reshape(np.shape(t))


def swiglu(h_bits: np.ndarray) -> np.ndarray:
    h = _c(h_bits, np.uint16)
    rows, w2 = h.shape
    act = np.empty((rows, w2 // 2), np.uint16)
    lib().hpo_swiglu(_p(h, _u16p), rows, w2 // 2, _p(act, _u16p))
    return act
