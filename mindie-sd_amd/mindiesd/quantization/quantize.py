"""``quantize(model, quant_des_path)``: swap the quantised layers of the attention path into a model from a weight
descriptor (mindiesd/quantization/quantize.py:158-161, 190-241, 280-335).

Descriptor: a JSON object ``{"model_quant_type": ALGO, "<key>": ALGO | "FLOAT", ...}`` next to a safetensors
file ``quant_model_weight_<algo in lower case>[_<rank>].safetensors`` (``_<rank>`` when the descriptor's own name
ends in ``_<digits>``: one file pair per rank).  A module named ``name`` is looked up under the keys
``name.linear.weight``, ``name.weight``, ``name``, ``name.fa_q.scale``, ``name.quant_type`` (:33-41); "FLOAT"
leaves it alone.  Of the reference's algorithms this build carries the two on its hot path:

* ``W8A8_MXFP8``  - an ``nn.Linear`` (or a class given in ``map``) is replaced by ``W8A8MXFP8QuantLinear``;
* ``FP8_DYNAMIC`` - the module gets an attribute ``fa_quant = FP8RotateQuantFA(name, weights)`` that its attention
  processor calls instead of ``attention_forward``.

Any other algorithm raises ParametersInvalid: the INT8 / INT4 / time-step layers are not part of this build."""
import enum
import json
import os
from collections import OrderedDict
from inspect import Parameter, signature

import torch
from torch import nn

from ..utils.exception import ConfigError, ParametersInvalid
from ..utils.logs import logger
from .layer import FP8RotateQuantFA, W8A8MXFP8QuantLinear


class QuantAlgorithm(str, enum.Enum):
    """The algorithm names a descriptor may carry (mindiesd/quantization/mode.py:24-47)."""
    W8A8 = "W8A8"
    W8A8_TIMESTEP = "W8A8_TIMESTEP"
    W8A8_DYNAMIC = "W8A8_DYNAMIC"
    W4A4_DYNAMIC = "W4A4_DYNAMIC"
    W8A8_MXFP8 = "W8A8_MXFP8"
    W4A4_MXFP4_DYNAMIC = "W4A4_MXFP4"
    W8A16 = "W8A16"
    W4A16 = "W4A16"
    FP8_DYNAMIC = "FP8_DYNAMIC"
    NO_QUANT = "NO_QUANT"
    W4A4_MXFP4_SVD = "W4A4_MXFP4_SVD"
    W4A4_MXFP4_DUALSCALE = "W4A4_MXFP4_DUALSCALE"


SUPPORTED = (QuantAlgorithm.W8A8_MXFP8, QuantAlgorithm.FP8_DYNAMIC)
_ALGO_VALUES = {a.value for a in QuantAlgorithm}


def get_key_patterns(layer_name):
    return [f"{layer_name}.linear.weight", f"{layer_name}.weight", f"{layer_name}", f"{layer_name}.fa_q.scale",
            f"{layer_name}.quant_type"]


class QuantDescriptor:
    """Parsed descriptor: model-wide algorithm, per-key algorithms, keys that stay in floating point."""

    def __init__(self, quant_algo, quantized_layers, exclude_layers):
        self.quant_algo = quant_algo
        self.quantized_layers = quantized_layers      # key -> QuantAlgorithm
        self.exclude_layers = tuple(exclude_layers)

    def algo_of(self, name):
        for pattern in get_key_patterns(name):
            if pattern in self.quantized_layers:
                return self.quantized_layers[pattern]
        return None

    def excluded(self, name):
        return any(pattern in self.exclude_layers for pattern in get_key_patterns(name))


def replace_rank_suffix(file_path):
    """``foo_3.json`` names a per-rank descriptor: the file of THIS rank is used (mindiesd/quantization/utils.py:41-67).
    Returns (path, rank); rank -1 for a descriptor without a numeric suffix."""
    dir_path, filename = os.path.split(file_path)
    basename, ext = os.path.splitext(filename)
    parts = basename.rsplit("_", 1)
    if len(parts) > 1 and parts[-1].isdigit():
        import torch.distributed as dist
        if not dist.is_initialized():
            raise ConfigError(f"must init distributed env if use distributed config {filename}")
        rank = dist.get_rank()
        return os.path.join(dir_path, f"{parts[0]}_{rank}{ext}"), rank
    return file_path, -1


def get_cfg_and_weights(quant_des_path):
    """-> (QuantDescriptor, safetensors handle with ``keys()`` / ``get_tensor(name)``)."""
    import safetensors
    quant_des_path, rank = replace_rank_suffix(quant_des_path)
    if not os.path.isfile(quant_des_path):
        raise ConfigError(f"quant descriptor not found: {quant_des_path}")
    with open(quant_des_path, "r", encoding="utf-8") as reader:
        des = json.loads(reader.read(), strict=False)
    if not des or not isinstance(des, dict):
        raise ParametersInvalid("quant_des_dict is none!")
    quant_algo = des.get("model_quant_type", None)
    if quant_algo is None or str(quant_algo).upper() not in _ALGO_VALUES:
        raise ParametersInvalid("quant_algo must be the type of QuantAlgorithm.")
    exclude = [k for k, v in des.items() if v == "FLOAT"]
    layers = {k: QuantAlgorithm(v.upper()) for k, v in des.items()
              if k != "model_quant_type" and isinstance(v, str) and v.upper() in _ALGO_VALUES}
    cfg = QuantDescriptor(QuantAlgorithm(str(quant_algo).upper()), layers, exclude)
    suffix = f"_{rank}" if rank != -1 else ""
    weight_path = os.path.join(os.path.dirname(quant_des_path),
                               f"quant_model_weight_{str(quant_algo).lower()}{suffix}.safetensors")
    if not os.path.isfile(weight_path):
        raise ConfigError(f"quant weight file not found: {weight_path}")
    weights = safetensors.safe_open(weight_path, framework="pytorch")
    logger.info(f"Quant Weight Path:{weight_path}")
    return cfg, weights


def extract_constructor_args(instance, quant_cls):
    """Constructor arguments of ``instance`` (by attribute of the same name) that ``quant_cls`` also takes."""
    own = [k for k, v in signature(instance.__class__.__init__).parameters.items()
           if v.kind == Parameter.POSITIONAL_OR_KEYWORD and k != "self"]
    wanted = {k for k in signature(quant_cls.__init__).parameters if k != "self"}
    return {k: getattr(instance, k) for k in own if k in wanted and hasattr(instance, k)}


def mxfp8_quantize(name, layer, quant_weights, **kwargs):
    """nn.Linear (or a class of ``map``) -> W8A8MXFP8QuantLinear; returns (layer, replaced?)."""
    quant_map = OrderedDict([(nn.Linear, W8A8MXFP8QuantLinear)])
    user_map = kwargs.get("map", None)
    if user_map:
        for key, value in user_map.items():
            quant_map[key] = value
        for key in user_map.keys():
            quant_map.move_to_end(key, last=False)
    quant_cls = next((quant_map[cls] for cls in quant_map if isinstance(layer, cls)), None)
    if quant_cls is None:
        return layer, False
    init_params = extract_constructor_args(layer, quant_cls)
    init_params["bias"] = isinstance(init_params.get("bias", None), nn.Parameter)
    init_params["is_dynamic"] = True
    init_params["weights"] = quant_weights
    init_params["prefix"] = name
    if f"{name}.div.mul_scale" in quant_weights.keys():   # outlier suppression: activations are scaled first
        init_params["mul_scale"] = quant_weights.get_tensor(f"{name}.div.mul_scale")
        init_params["prefix"] = f"{name}.linear"
    extra = {k: v for k, v in kwargs.items() if k != "map"}
    return quant_cls(**init_params, **extra), True


def add_fa_quant(layer, cfg, prefix, quant_weights):
    """Attach the FP8 attention module to ``layer`` when ``cfg`` (a QuantAlgorithm or an object with ``quant_algo``)
    asks for it (quantize.py:158-161)."""
    algo = getattr(cfg, "quant_algo", cfg)
    if algo == QuantAlgorithm.FP8_DYNAMIC:
        layer.fa_quant = FP8RotateQuantFA(prefix, quant_weights)


def quantize(model, quant_des_path, **kwargs):
    """Quantise ``model`` in place from the descriptor at ``quant_des_path`` and return it.
    kwargs: ``dtype`` (torch.float16 / torch.bfloat16, output type of the quantised linears), ``map`` (extra
    {float class: quantised class} rules, tried first)."""
    if not isinstance(model, nn.Module):
        raise ParametersInvalid(f"The model must be the type of nn.Module, but currently got {type(model)}.")
    if not isinstance(quant_des_path, str) or not quant_des_path.strip():
        raise ConfigError("Invalid string path for quant_des_path.")
    dtype = kwargs.get("dtype", torch.bfloat16)
    if not isinstance(dtype, torch.dtype) or dtype not in (torch.float16, torch.bfloat16):
        raise ParametersInvalid(f"Dtype must be torch.float16 or torch.bfloat16, but currently got {dtype}.")
    module_map = kwargs.get("map", None)
    if module_map is not None and (not isinstance(module_map, dict)
                                   or not all(isinstance(k, type) and isinstance(v, type) for k, v in module_map.items())):
        raise ParametersInvalid("The data type of map must be dictionary of module classes.")
    cfg, quant_weights = get_cfg_and_weights(os.path.abspath(quant_des_path))
    if not cfg.quantized_layers:
        logger.debug("Quantization content is none, Without enabling quantization.")
        return model
    replaced = []
    for name, layer in model.named_modules():
        if cfg.excluded(name):
            continue
        algo = cfg.algo_of(name)
        if algo is None or algo == QuantAlgorithm.NO_QUANT:
            continue
        if algo not in SUPPORTED:
            raise ParametersInvalid(f"Quant algorithm {algo.value} of layer {name} is not part of this build "
                                    f"(supported: {[a.value for a in SUPPORTED]}).")
        if algo == QuantAlgorithm.W8A8_MXFP8:
            quant_layer, is_modified = mxfp8_quantize(name, layer, quant_weights, **kwargs)
            if is_modified:
                replaced.append((name, quant_layer))
        else:
            add_fa_quant(layer, algo, name, quant_weights)
    for name, layer in replaced:   # after the walk: named_modules must not see the graph change under it
        parent, _, attr = name.rpartition(".")
        setattr(model.get_submodule(parent), attr, layer)
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return model
