from .layer import FP8RotateQuantFA, W8A8MXFP8QuantLinear

__all__ = ["FP8RotateQuantFA", "W8A8MXFP8QuantLinear"]
