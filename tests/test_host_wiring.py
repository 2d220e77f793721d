"""Host-side pieces around the kernels that need no GPU: get_activation_layer, the step-level attention cache and
the quantize() wiring that swaps the quantised layers into a model from a descriptor + safetensors file."""
import json
import os

import pytest
import torch
from torch import nn

import mindiesd
from mindiesd import CacheAgent, CacheConfig, ConfigError, ParametersInvalid, get_activation_layer, quantize
from mindiesd.quantization import FP8RotateQuantFA, QuantAlgorithm, W8A8MXFP8QuantLinear, add_fa_quant, get_cfg_and_weights


# ---- get_activation_layer (mindiesd/layers/activation.py:34-61) ---------------------------------------------------
def test_activation_table():
    x = torch.linspace(-4, 4, 101)
    assert isinstance(get_activation_layer("silu"), nn.SiLU) and isinstance(get_activation_layer("SWISH"), nn.SiLU)
    assert torch.equal(get_activation_layer("silu")(x), torch.nn.functional.silu(x))
    assert torch.equal(get_activation_layer("gelu-tanh")(x), torch.nn.functional.gelu(x, approximate="tanh"))
    assert torch.equal(get_activation_layer("gelu")(x), torch.nn.functional.gelu(x))
    assert torch.allclose(get_activation_layer("gelu-fast")(x), x / (1 + torch.exp(-1.702 * x)), atol=1e-6)
    assert isinstance(get_activation_layer("relu"), nn.ReLU) and isinstance(get_activation_layer("mish"), nn.Mish)
    with pytest.raises(ParametersInvalid, match="Unsupported activation function"):
        get_activation_layer("softplus")
    assert "get_activation_layer" in mindiesd.__all__ and "quantize" in mindiesd.__all__


# ---- CacheAgent / AttentionCache -----------------------------------------------------------------------------------
# Known answers of the reference's own test (tests/cache/test_attention_cache.py:24-50, :52-82): 7 steps x 5 blocks,
# window step_start=1 .. step_end=5, interval 3; the function returns its argument(s).
KAT_ONE = [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 5, 6, 7, 8, 9, 5, 6, 7, 8, 9, 20, 21, 22, 23, 24, 20, 21, 22, 23, 24,
           30, 31, 32, 33, 34]
KAT_TWO_STEPS = [0, 1, 1, 1, 4, 4, 6]


def _agent():
    return CacheAgent(CacheConfig(method="attention_cache", blocks_count=5, steps_count=7, step_start=1, step_end=5,
                                  step_interval=3))


def test_attention_cache_known_answers():
    agent = _agent()
    for _ in range(5):       # the counters wrap around after steps_count steps
        got = [agent.apply(lambda i: i, step * 5 + block) for step in range(7) for block in range(5)]
        assert got == KAT_ONE
    agent = _agent()
    for _ in range(3):
        got = [agent.apply(lambda i, j: (i, j), step, block) for step in range(7) for block in range(5)]
        assert got == [(KAT_TWO_STEPS[step], block) for step in range(7) for block in range(5)]


def test_cache_agent_pass_through_and_checks():
    calls = []
    f = lambda x: calls.append(x) or x
    # interval 1, a window that never opens, a block range that is empty: every call goes through
    for kw in (dict(step_interval=1), dict(step_start=9), dict(step_start=2, step_end=2), dict(block_start=5),
               dict(block_start=1, block_end=1)):
        agent = CacheAgent(CacheConfig(method="attention_cache", blocks_count=2, steps_count=4, **kw))
        calls.clear()
        assert [agent.apply(f, i) for i in range(8)] == list(range(8)) and calls == list(range(8))
    with pytest.raises(ParametersInvalid):
        _agent().apply(3)
    for bad in (dict(method="dit_block_cache"), dict(blocks_count=0), dict(steps_count=0), dict(step_start=-1),
                dict(step_interval=0), dict(step_start=3, step_end=2), dict(block_start=3, block_end=2)):
        kw = dict(method="attention_cache", blocks_count=2, steps_count=4)
        kw.update(bad)
        with pytest.raises(ConfigError):
            CacheAgent(CacheConfig(**kw))


def test_attention_cache_reuses_tensors_not_copies():
    agent = CacheAgent(CacheConfig(method="attention_cache", blocks_count=1, steps_count=4, step_start=0, step_end=3,
                                   step_interval=2))
    outs = [agent.apply(lambda: torch.randn(3)) for _ in range(4)]
    assert outs[1] is outs[0] and outs[2] is not outs[0] and outs[3] is outs[2]


# ---- quantize() ------------------------------------------------------------------------------------------------------
class _Attn(nn.Module):
    def __init__(self):
        super().__init__()
        self.to_q = nn.Linear(64, 64)


class _Block(nn.Module):
    def __init__(self):
        super().__init__()
        self.attn = _Attn()
        self.ffn_up = nn.Linear(64, 128, bias=False)
        self.ffn_down = nn.Linear(128, 64)
        self.act = nn.SiLU()


class _Toy(nn.Module):
    def __init__(self):
        super().__init__()
        self.blocks = nn.ModuleList([_Block(), _Block()])
        self.head = nn.Linear(64, 10)


def _mx_weights(prefix, out_f, in_f, bias):
    w = {f"{prefix}.weight": torch.randn(out_f, in_f).to(torch.float8_e4m3fn),
         f"{prefix}.weight_scale": torch.full((out_f, in_f // 32), 127, dtype=torch.uint8)}
    if bias:
        w[f"{prefix}.bias"] = torch.randn(out_f)
    return w


def _write(tmp_path, des, weights, algo):
    from safetensors.torch import save_file
    path = os.path.join(tmp_path, "quant_model_description.json")
    with open(path, "w") as f:
        json.dump(des, f)
    save_file(weights, os.path.join(tmp_path, f"quant_model_weight_{algo.lower()}.safetensors"))
    return path


def test_quantize_swaps_linears_and_attaches_fa_quant(tmp_path):
    torch.manual_seed(0)
    des = {"model_quant_type": "W8A8_MXFP8", "head.weight": "FLOAT"}
    weights = {}
    for b in range(2):
        des[f"blocks.{b}.ffn_up.weight"] = "W8A8_MXFP8"
        des[f"blocks.{b}.ffn_down.weight"] = "W8A8_MXFP8"
        des[f"blocks.{b}.attn.to_q.weight"] = "FLOAT" if b else "W8A8_MXFP8"
        des[f"blocks.{b}.attn.fa_q.scale"] = "FP8_DYNAMIC"
        weights.update(_mx_weights(f"blocks.{b}.ffn_up", 128, 64, False))
        weights.update(_mx_weights(f"blocks.{b}.ffn_down", 64, 128, True))
        weights[f"blocks.{b}.attn.q_rot"] = torch.eye(128, dtype=torch.bfloat16)
        weights[f"blocks.{b}.attn.k_rot"] = torch.eye(128, dtype=torch.bfloat16)
    # outlier suppression on one layer: the activations are scaled first and the weights live under "<name>.linear"
    weights.update(_mx_weights("blocks.0.attn.to_q.linear", 64, 64, True))
    weights["blocks.0.attn.to_q.div.mul_scale"] = torch.rand(64) + 0.5
    model = quantize(_Toy(), _write(str(tmp_path), des, weights, "W8A8_MXFP8"), dtype=torch.float16)
    for b in range(2):
        blk = model.blocks[b]
        assert isinstance(blk.ffn_up, W8A8MXFP8QuantLinear) and blk.ffn_up.bias is None
        assert isinstance(blk.ffn_down, W8A8MXFP8QuantLinear) and blk.ffn_down.bias.dtype == torch.float32
        assert blk.ffn_up.dtype == torch.float16 and blk.ffn_up.weight.dtype == torch.float8_e4m3fn
        assert tuple(blk.ffn_up.weight_scale.shape) == (128, 1, 2)           # the reference's [out, in/64, 2] view
        assert isinstance(blk.attn.fa_quant, FP8RotateQuantFA) and blk.attn.fa_quant.q_rot.shape == (128, 128)
        assert isinstance(blk.act, nn.SiLU)
    q0 = model.blocks[0].attn.to_q
    assert isinstance(q0, W8A8MXFP8QuantLinear) and q0.mul_scale is not None and q0.mul_scale.dtype == torch.float16
    assert torch.equal(q0.weight.view(torch.uint8), weights["blocks.0.attn.to_q.linear.weight"].view(torch.uint8))
    assert isinstance(model.blocks[1].attn.to_q, nn.Linear) and isinstance(model.head, nn.Linear)
    assert not hasattr(model.blocks[0], "fa_quant")


def test_quantize_parameter_and_descriptor_errors(tmp_path):
    with pytest.raises(ParametersInvalid):
        quantize("not a module", "x.json")
    with pytest.raises(ConfigError):
        quantize(_Toy(), "   ")
    with pytest.raises(ConfigError):
        quantize(_Toy(), os.path.join(str(tmp_path), "missing.json"))
    with pytest.raises(ParametersInvalid):
        quantize(_Toy(), "x.json", dtype=torch.float32)
    with pytest.raises(ParametersInvalid):
        quantize(_Toy(), "x.json", map={"a": 1})
    # an algorithm outside this build
    path = _write(str(tmp_path), {"model_quant_type": "W8A8", "head.weight": "W8A8"}, {"x": torch.zeros(1)}, "W8A8")
    with pytest.raises(ParametersInvalid, match="not part of this build"):
        quantize(_Toy(), path)
    # no model_quant_type / weight file missing / a critical tensor missing
    bad = os.path.join(str(tmp_path), "bad.json")
    with open(bad, "w") as f:
        json.dump({"head.weight": "W8A8_MXFP8"}, f)
    with pytest.raises(ParametersInvalid):
        get_cfg_and_weights(bad)
    sub = os.path.join(str(tmp_path), "sub")
    os.makedirs(sub)
    lone = os.path.join(sub, "d.json")
    with open(lone, "w") as f:
        json.dump({"model_quant_type": "FP8_DYNAMIC"}, f)
    with pytest.raises(ConfigError, match="weight file"):
        get_cfg_and_weights(lone)
    path = _write(sub, {"model_quant_type": "W8A8_MXFP8", "head.weight": "W8A8_MXFP8"}, {"x": torch.zeros(1)}, "W8A8_MXFP8")
    with pytest.raises(ParametersInvalid, match="Critical parameter missing: head.bias"):
        quantize(_Toy(), path)
    # a per-rank descriptor needs an initialised process group
    ranked = os.path.join(sub, "d_0.json")
    with open(ranked, "w") as f:
        json.dump({"model_quant_type": "FP8_DYNAMIC"}, f)
    with pytest.raises(ConfigError, match="distributed"):
        get_cfg_and_weights(ranked)


def test_add_fa_quant_only_for_fp8_dynamic():
    """tests/quantization/test_quantize.py:355-372 of the reference: FP8_DYNAMIC attaches the module, anything else
    leaves the layer alone."""
    weights = {"test_layer.q_rot": torch.randn(128, 128, dtype=torch.float16),
               "test_layer.k_rot": torch.randn(128, 128, dtype=torch.float16)}
    layer = nn.Module()
    add_fa_quant(layer, QuantAlgorithm.FP8_DYNAMIC, "test_layer", weights)
    assert isinstance(layer.fa_quant, FP8RotateQuantFA)
    other = nn.Linear(10, 10)
    add_fa_quant(other, QuantAlgorithm.NO_QUANT, "test_layer", weights)
    assert not hasattr(other, "fa_quant")
