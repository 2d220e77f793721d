"""Activation layers by name (mindiesd/layers/activation.py:19-61).  Only ``silu`` is on the attention / FFN hot
path of this build (the SwiGLU of the MXFP8 FFN, which the fused GEMM applies on its accumulators); the table is
the reference's, so that model code that asks for another entry keeps working."""
import torch
import torch.nn as nn
import torch.nn.functional as F

from ..utils.exception import ParametersInvalid


class GELU(nn.Module):
    """``approximate``: 'none', 'tanh' (torch's two forms) or 'fast' = x * sigmoid(1.702 x), the closed form of
    the vendor's fast-GELU op (activation.py:27-28)."""

    def __init__(self, approximate="none"):
        super().__init__()
        self.approximate = approximate

    def forward(self, hidden_states):
        if self.approximate in ("none", "tanh"):
            return F.gelu(hidden_states, approximate=self.approximate)
        if self.approximate == "fast":
            return hidden_states * torch.sigmoid(1.702 * hidden_states)
        raise ParametersInvalid(f"The approximate only support 'none', 'tanh' and 'fast', but got {self.approximate}")


ACTIVATION_FUNCTIONS = {
    "swish": nn.SiLU(),
    "silu": nn.SiLU(),
    "mish": nn.Mish(),
    "gelu": GELU(),
    "relu": nn.ReLU(),
    "gelu-tanh": GELU(approximate="tanh"),
    "gelu-fast": GELU(approximate="fast"),
}


def get_activation_layer(act_type: str) -> nn.Module:
    """Activation module for ``act_type`` ('swish', 'silu', 'mish', 'gelu', 'relu', 'gelu-tanh', 'gelu-fast';
    case insensitive); anything else raises ParametersInvalid."""
    act_type = act_type.lower()
    if act_type in ACTIVATION_FUNCTIONS:
        return ACTIVATION_FUNCTIONS[act_type]
    raise ParametersInvalid(f"Unsupported activation function: {act_type}")
