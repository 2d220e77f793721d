from .block_quant import fa_block_quant_preprocess
from .fp8_attention import fp8_attention_forward
from .mxfp8 import mx_quantize, mxfp8_matmul, mxfp8_gemm_swiglu

__all__ = ["fa_block_quant_preprocess", "fp8_attention_forward", "mx_quantize", "mxfp8_matmul", "mxfp8_gemm_swiglu"]
