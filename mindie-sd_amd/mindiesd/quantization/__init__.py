from .layer import FP8RotateQuantFA, W8A8MXFP8QuantLinear
from .quantize import QuantAlgorithm, add_fa_quant, get_cfg_and_weights, quantize

__all__ = ["FP8RotateQuantFA", "W8A8MXFP8QuantLinear", "QuantAlgorithm", "add_fa_quant", "get_cfg_and_weights",
           "quantize"]
