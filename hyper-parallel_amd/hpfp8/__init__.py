"""hpfp8: MI355X-native FP8 mixed-precision linear path (quantizers, scaled GEMMs, fp8_linear).

Importing the package loads libhpfp8.so; it raises ImportError if the HIP extension is not built.
"""
from . import _lib

_lib.load()

from .ops import (amax, quantize_per_tensor, quantize_1x128, quantize_128x128, quantize_128x1_t,  # noqa: E402
                  quantize_1x128_and_128x1_t, transpose_codes, swiglu_quantize_1x128,
                  dequantize_1x128, dequantize_1x128_accumulate, dequantize_128x128, dequantize_per_tensor, gemm_blockwise, gemm_blockwise_swiglu_quantize, gemm_per_tensor,
                  gemm_grouped_blockwise)
from .linear import (fp8_linear, Fp8Linear, fp8_grouped_linear, fp8_swiglu_mlp, Fp8SwiGLUMLP, Fp8Weight,  # noqa: E402
                     quantize_weight, quantize_grouped_weight, invalidate_fp8_caches, attach_optimizer)
from . import fsdp, checkpoint  # noqa: E402
from .bucket import quantize_bucket, dequantize_bucket, Fp8GradBucket  # noqa: E402
from .policy import Fp8MixedPrecisionPolicy, Fp8Tensor, cast_fp_tensor, tensor_type_cast  # noqa: E402

__all__ = [
    "Fp8MixedPrecisionPolicy", "Fp8Tensor", "cast_fp_tensor", "tensor_type_cast",
    "amax", "quantize_per_tensor", "quantize_1x128", "quantize_128x128", "quantize_128x1_t",
    "quantize_1x128_and_128x1_t", "transpose_codes", "swiglu_quantize_1x128", "Fp8Weight", "quantize_weight", "fsdp", "checkpoint",
    "invalidate_fp8_caches", "attach_optimizer", "quantize_grouped_weight",
    "dequantize_1x128", "dequantize_1x128_accumulate", "dequantize_128x128", "dequantize_per_tensor", "gemm_blockwise", "gemm_blockwise_swiglu_quantize", "gemm_per_tensor",
    "gemm_grouped_blockwise", "fp8_linear", "Fp8Linear", "fp8_grouped_linear", "fp8_swiglu_mlp", "Fp8SwiGLUMLP",
    "quantize_bucket", "dequantize_bucket", "Fp8GradBucket",
]
