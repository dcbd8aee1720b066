"""MI355X-native block-scaled FP8 kernels of DeepSeek-V3's inference path."""
from .kernel import act_quant, fp8_gemm, fp8_gemm_f32, fp8_gemm_pow2, weight_dequant  # noqa: F401
from .quantize import weight_quant  # noqa: F401

__all__ = ["act_quant", "weight_dequant", "fp8_gemm", "fp8_gemm_f32", "fp8_gemm_pow2", "weight_quant"]
