"""The C-ABI library loads and exports every symbol include/hpfp8.h declares; argument checks that
return before any kernel launch work without a GPU."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hpfp8.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hpfp8_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ("hpfp8_amax_bf16", "hpfp8_quantize_per_tensor_bf16", "hpfp8_quantize_1x128_bf16",
                 "hpfp8_quantize_128x128_bf16", "hpfp8_quantize_128x1_t_bf16", "hpfp8_dequantize_1x128_bf16",
                 "hpfp8_gemm_blockwise", "hpfp8_gemm_per_tensor", "hpfp8_gemm_grouped_blockwise"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from hpfp8 import _lib
    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/hpfp8.h but not exported"
    bound = set(_lib.SIGNATURES) | set(_lib.SIZE_FUNCTIONS) | {"hpfp8_last_error", "hpfp8_debug_set_spin_limit", "hpfp8_debug_set_small_gemm"}
    assert bound == set(declared_functions()), "python binding and header disagree"
    assert lib.hpfp8_version() >= 100


def test_argument_errors_are_reported_without_launching():
    from hpfp8 import _lib
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.cast(buf, ctypes.c_void_p).value
    p = (p + 15) & ~15
    # last dim not a multiple of 128
    rc = lib.hpfp8_quantize_1x128_bf16(p, 4, 100, p, None, p, None)
    assert rc == -2 and b"multiple of 128" in lib.hpfp8_last_error()
    # misaligned pointer
    rc = lib.hpfp8_quantize_1x128_bf16(p + 2, 1, 128, p, None, p, None)
    assert rc == -3
    # null buffer
    rc = lib.hpfp8_quantize_128x128_bf16(None, 128, 128, p, None, 0, None, p, None)
    assert rc == -1
    # bad scale granularity, bad K
    rc = lib.hpfp8_gemm_blockwise(p, 128, p, 1, 1, p, 128, p, 1, 1, 7, 128, 128, 128, None, p, 128, 0, 0, None)
    assert rc == -1
    rc = lib.hpfp8_gemm_blockwise(p, 128, p, 1, 1, p, 128, p, 1, 1, 128, 128, 128, 100, None, p, 128, 0, 0, None)
    assert rc == -2
    # accumulate needs fp32 output
    rc = lib.hpfp8_gemm_blockwise(p, 128, p, 1, 1, p, 128, p, 1, 1, 128, 128, 128, 128, None, p, 128, 0, 1, None)
    assert rc == -1
    # rows of c are written in 16-byte pieces: ldc a multiple of 8 for bf16, of 4 for fp32
    rc = lib.hpfp8_gemm_blockwise(p, 128, p, 1, 1, p, 128, p, 1, 1, 128, 128, 128, 128, None, p, 132, 0, 0, None)
    assert rc == -3 and b"ldc" in lib.hpfp8_last_error()
    # negative scale stride
    rc = lib.hpfp8_gemm_blockwise(p, 128, p, -1, 1, p, 128, p, 1, 1, 128, 128, 128, 128, None, p, 128, 0, 0, None)
    assert rc == -2 and b"stride" in lib.hpfp8_last_error()
    # a scale array spanning 2 GiB or more
    rc = lib.hpfp8_gemm_blockwise(p, 128, p, 1 << 30, 1, p, 128, p, 1, 1, 128, 128, 128, 128, None, p, 128, 0, 0, None)
    assert rc == -2 and b"2 GiB" in lib.hpfp8_last_error()
    # empty problems succeed without touching the device
    assert lib.hpfp8_quantize_1x128_bf16(None, 0, 128, None, None, None, None) == 0
    assert lib.hpfp8_gemm_per_tensor(None, 128, None, None, 128, None, 0, 128, 128, None, None, 128, 0, None) == 0


def test_argument_errors_of_the_fused_and_one_launch_entry_points():
    """The gate/up GEMM with the SwiGLU + quantizer epilogue, the fused SwiGLU-backward quantizer and the one-launch
    per-tensor quantizer check their arguments before anything is launched."""
    from hpfp8 import _lib
    lib = _lib.load()
    buf = (ctypes.c_char * 8192)()
    p = (ctypes.cast(buf, ctypes.c_void_p).value + 255) & ~255
    ep = lib.hpfp8_gemm_blockwise_swiglu_quantize
    # flags other than 0 / 1; a width that is not a multiple of 128; ldq below the width; null scale_inv
    assert ep(p, 128, p, 1, 1, p, 128, p, 1, 1, 128, 128, 128, 2, 0, 0, p, 128, None, p, None) == -1
    assert ep(p, 128, p, 1, 1, p, 128, p, 1, 1, 128, 100, 128, 0, 0, 0, p, 128, None, p, None) == -2
    assert b"multiple of 128" in lib.hpfp8_last_error()
    assert ep(p, 128, p, 1, 1, p, 128, p, 1, 1, 128, 256, 128, 0, 0, 0, p, 128, None, p, None) == -2
    assert ep(p, 128, p, 1, 1, p, 128, p, 1, 1, 128, 128, 128, 0, 0, 0, p, 128, None, None, None) == -1
    # a weight whose codes span 2 GiB or more cannot be addressed from one tile's buffer resource
    assert ep(p, 1 << 14, p, 1, 1, p, 1 << 14, p, 1, 1, 128, 1 << 16, 1 << 14, 0, 0, 0, p, 1 << 16, None, p, None) == -2
    assert b"2 GiB" in lib.hpfp8_last_error()
    # empty problems succeed
    assert ep(None, 128, None, 1, 1, None, 128, None, 1, 1, 0, 128, 128, 0, 0, 0, None, 128, None, None, None) == 0
    bw = lib.hpfp8_swiglu_backward_quantize_1x128_and_128x1_t_bf16
    assert bw(p, 100, 128, 256, p, p, None, p, p, 128, None, p, None) == -2          # rows not a multiple of 128
    assert bw(p, 128, 128, 200, p, p, None, p, p, 128, None, p, None) == -2          # ld_h below twice the width
    assert bw(p, 128, 128, 256, None, p, None, p, p, 128, None, p, None) == -1       # no dact
    assert bw(p, 128, 128, 256, p, p, None, p, p, 64, None, p, None) == -2           # ld_t below the row count
    sy = lib.hpfp8_quantize_per_tensor_sync_bf16
    assert sy(p, (1 << 22) + 8, p, None, None, p, p, None) == -2 and b"one-pass" in lib.hpfp8_last_error()
    assert sy(p, 1024, p, None, None, p, None, None) == -1
    assert sy(p, 1024, p, None, None, p, p + 16, None) == -3
    assert sy(p + 2, 1024, p, None, None, p, p, None) == -3


def test_python_wrappers_reject_cpu_tensors_and_bad_shapes():
    import torch
    import hpfp8
    x = torch.zeros(4, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="no CPU fallback"):
        hpfp8.quantize_1x128(x)
    with pytest.raises(TypeError):
        hpfp8.fp8_linear(torch.zeros(4, 128), torch.zeros(128, 128, dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        hpfp8.fp8_linear(x, torch.zeros(128, 256, dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        hpfp8.fp8_linear(x, torch.zeros(128, 128, dtype=torch.bfloat16), recipe="nope")
    with pytest.raises(ValueError):
        hpfp8.Fp8Linear(100, 128)
    with pytest.raises(ValueError):
        hpfp8.quantize_bucket(torch.zeros(100, dtype=torch.bfloat16))
