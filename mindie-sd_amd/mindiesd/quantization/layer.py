"""Quantised layers of the attention path (mindiesd/quantization/layer.py)."""
import torch
from torch import nn

from ..layers.quant.fp8_attention import fp8_attention_forward
from ..layers.quant.mxfp8 import mx_quantize, mxfp8_matmul
from ..utils.exception import ParametersInvalid


def _get_weight(weights, name):
    """``weights`` is a safetensors handle (``keys()`` / ``get_tensor``; mindiesd/quantization/quantize.py:229-238) or a
    plain mapping name -> tensor; a missing entry raises ParametersInvalid (quantization/utils.py:70-87)."""
    if weights is None or name not in weights.keys():
        raise ParametersInvalid(f"Critical parameter missing: {name}.")
    return weights.get_tensor(name) if hasattr(weights, "get_tensor") else weights[name]


class FP8RotateQuantFA(nn.Module):
    """Rotate q and k with fixed [D, D] matrices, quantise q, k, v to FP8 and run FP8 attention
    (mindiesd/quantization/layer.py:274-324).  ``forward(query, key, value, layout='BNSD'|'BSND')``
    returns the attention output in the layout and dtype of ``query``.

    The reference quantises K and V per 256-token block for its vendor kernel; this build's kernel
    takes K per 128-token block and V per channel (the Wan2.1-14B 480p FP8 workload's recipe)."""

    def __init__(self, prefix=None, weights=None):
        super().__init__()
        self.register_buffer("q_rot", _get_weight(weights, f"{prefix}.q_rot"), persistent=False)
        self.register_buffer("k_rot", _get_weight(weights, f"{prefix}.k_rot"), persistent=False)

    def forward(self, query, key, value, **kwargs):
        layout = kwargs.get("layout", "BNSD")
        if layout not in ("BNSD", "BSND"):
            raise ValueError(f"Unsupported layout: {layout}, expected 'BNSD' or 'BSND'.")
        # the two rotations (torch.matmul in the reference, layer.py:284-285) run inside the quantisation pass
        return fp8_attention_forward(query, key, value, scale=query.shape[-1] ** -0.5, layout=layout,
                                     q_rot=self.q_rot, k_rot=self.k_rot)


class W8A8MXFP8QuantLinear(nn.Module):
    """Linear layer with MXFP8 weights and dynamically MX-quantised activations
    (mindiesd/quantization/layer.py:327-372 and its base :77-116).

    ``weights`` provides ``{prefix}.weight`` (E4M3 [out, in]), ``{prefix}.weight_scale`` (E8M0, one
    per 32 input features; stored by the reference as [out, in/64, 2]) and, with ``bias=True``,
    ``{prefix}.bias``.  kwargs: ``dtype`` (output dtype, default bf16), ``mul_scale`` (per-feature
    multiplier applied to the activations before quantisation), ``swiglu`` (not in the reference:
    treat the weight as [gate | up] and return silu(gate) * up, half as many output features)."""

    def __init__(self, in_features, out_features, bias=True, weights=None, prefix=None, **kwargs):
        super().__init__()
        self.dtype = kwargs.get("dtype", torch.bfloat16)
        self.input_feature = in_features
        self.output_feature = out_features
        self.is_dynamic = True
        self.swiglu = bool(kwargs.get("swiglu", False))
        if bias:
            self.register_buffer("bias", _get_weight(weights, f"{prefix}.bias").to(torch.float32), persistent=False)
        else:
            self.bias = None
        mul_scale = kwargs.get("mul_scale", None)
        if mul_scale is not None:
            self.register_buffer("mul_scale", mul_scale.to(self.dtype), persistent=False)
        else:
            self.mul_scale = None
        weight_scale = _get_weight(weights, f"{prefix}.weight_scale")
        self.register_buffer("weight_scale", weight_scale.reshape(weight_scale.shape[0], -1, 2), persistent=False)
        self.register_buffer("weight", _get_weight(weights, f"{prefix}.weight"), persistent=False)

    def quant_matmul(self, x):
        if x.dtype != self.dtype:
            x = x.to(self.dtype)
        if self.mul_scale is not None:
            x = x * self.mul_scale
        x1, input_scale = mx_quantize(x)
        return mxfp8_matmul(x1, input_scale, self.weight, self.weight_scale, self.bias, self.dtype, self.swiglu)

    def forward(self, x):
        if x.ndim >= 3:  # the reference flattens to 2-D as well (layer.py:104-116)
            out = self.quant_matmul(x.reshape(x.shape[:-1].numel(), -1))
            return out.view(*x.shape[:-1], out.shape[1])
        return self.quant_matmul(x)
