"""MI355X-native row-wise FP8 GEMM backend for the tritonbench `fp8_gemm_rowwise` operator."""

__all__ = ["ops", "build"]
