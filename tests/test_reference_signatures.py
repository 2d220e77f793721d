"""The drop-in boundary in Python: every public function of the attention path takes the reference's arguments
under the reference's names, in its order, with its defaults.  The expected declarations are data in
tests/golden/reference_signatures.json (written by tests/golden/make_reference_signatures.py, which parses the
reference's files as text; each entry carries the file:line of the ``def``).  Arguments this build adds must come
after the reference's and carry defaults, so that every reference call site still binds the same way."""
import ast
import importlib
import inspect
import json
import os

import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_signatures.json")) as f:
    TABLE = json.load(f)

# where this build keeps a name that the reference declares elsewhere
MOVED = {
    "mindiesd.cache_agent.attention_cache:AttentionCache.apply_imp": "mindiesd.cache_agent.cache_agent:AttentionCache.apply_imp",
    # the reference's MXFP8 linear inherits forward() from its base class
    "mindiesd.quantization.layer:W8A8QuantBaseLinear.forward": "mindiesd.quantization.layer:W8A8MXFP8QuantLinear.forward",
}
# defaults the reference spells with its vendor module
NON_LITERAL = {"torch_npu.float8_e4m3fn": torch.float8_e4m3fn}

# the rows of the hot-path contract the table has to cover (function -> at least one entry)
REQUIRED = [
    "attention_forward:attention_forward", "attention_forward:check_input_params", "common:AttentionParam.__init__",
    "attention_func:attention_math", "sparse_flash_attn:sparse_attention",
    "sparse_flash_attn_rf_v2:rearrange_with_remaining", "sparse_flash_attn_rf_v2:inv_rearrange_with_remaining",
    "sparse_flash_attn_rf_v3:_bsa_inv_rearrange", "sparse_flash_attn_rf_v3:do_tensor_rearrange_only",
    "sparse_flash_attn_rf_v2:do_tensor_inv_rearrange", "sparse_flash_attn_rf_v2:avgpool",
    "sparse_flash_attn_rf_v2:do_tensor_rearrange_pooling", "sparse_flash_attn_rf_v2:get_blockwise_mask",
    "sparse_flash_attn_rf_v2:get_mask_index", "sparse_flash_attn_rf_v2:rain_fusion_attention",
    "_custom_ops:rain_fusion_attention", "sparse_flash_attn_rf_v3:rain_fusion_attention_v3",
    "sparse_flash_attn_rf_v3:bsa_sparse_attention_v3", "_custom_ops:block_sparse_attention",
    "block_quant:fa_block_quant_preprocess", "layer:FP8RotateQuantFA.forward", "layer:W8A8MXFP8QuantLinear.__init__",
    "activation:get_activation_layer", "_custom_ops:sparse_block_estimate", "_custom_ops:ada_block_sparse_attention",
    "sparse_flash_attn_ada_bsa:get_estimate_mask", "attention_forward_varlen:attention_forward_varlen",
    "quantize:quantize", "attention_cache:AttentionCache.apply_imp",
]


def test_table_covers_the_path():
    keys = list(TABLE)
    for want in REQUIRED:
        assert any(k.endswith("." + want) or k.endswith(want) for k in keys), want
    for entry in TABLE.values():
        path, line = entry["at"].rsplit(":", 1)
        assert path.startswith("mindiesd/") and int(line) > 0


def _resolve(key):
    module, name = MOVED.get(key, key).split(":")
    obj = importlib.import_module(module)
    for part in name.split("."):
        obj = getattr(obj, part)
    return obj


def _expected_default(text):
    if text in NON_LITERAL:
        return NON_LITERAL[text]
    return ast.literal_eval(text)


@pytest.mark.parametrize("key", sorted(TABLE))
def test_signature_matches_the_reference(key):
    want = TABLE[key]
    obj = _resolve(key)
    owner_is_class = key.endswith(".__init__")
    if owner_is_class:
        # constructors: whatever way the class builds them (dataclass, NamedTuple, plain __init__)
        module, name = MOVED.get(key, key).split(":")
        cls = getattr(importlib.import_module(module), name.split(".")[0])
        params = [inspect.Parameter("self", inspect.Parameter.POSITIONAL_OR_KEYWORD)] + \
            list(inspect.signature(cls).parameters.values())
    else:
        params = list(inspect.signature(obj).parameters.values())
    positional = [p for p in params if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD)]
    names = [p.name for p in positional]
    where = f"{key} (reference {want['at']})"
    assert names[:len(want["args"])] == want["args"], f"{where}: {names} vs {want['args']}"
    by_name = {p.name: p for p in params}
    for name in want["args"]:
        p = by_name[name]
        if name in want["defaults"]:
            exp = _expected_default(want["defaults"][name])
            assert p.default is not inspect.Parameter.empty, f"{where}: {name} lost its default"
            assert type(p.default) is type(exp) and p.default == exp, f"{where}: {name}={p.default!r} vs {exp!r}"
        else:
            assert p.default is inspect.Parameter.empty, f"{where}: {name} gained a default"
    # what this build adds must not disturb a reference call
    for p in positional[len(want["args"]):]:
        assert p.default is not inspect.Parameter.empty, f"{where}: extra argument {p.name} without a default"
    for name in want["kwonly"]:
        assert name in by_name and by_name[name].kind == inspect.Parameter.KEYWORD_ONLY, f"{where}: {name}"
    if want["kwarg"]:
        assert any(p.kind == p.VAR_KEYWORD for p in params), f"{where}: **{want['kwarg']} missing"
    if want["vararg"]:
        assert any(p.kind == p.VAR_POSITIONAL for p in params), f"{where}: *{want['vararg']} missing"
