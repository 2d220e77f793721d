"""Writes tests/golden/reference_signatures.json: for every public function / method of the attention path
the argument names, their order and their default values as the reference declares them, each with the
file:line of the ``def``.  The reference's files are parsed as text (``ast``), never imported or run; the
table holds declarations (data), no source text.

    python tests/golden/make_reference_signatures.py [/root/reference]

tests/test_reference_signatures.py compares this build's functions of the same names against the table.
"""
import ast
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))

# reference file -> names to record ("Class.method" for methods); "*" = every public top-level function
WANTED = {
    "mindiesd/layers/flash_attn/attention_forward.py": ["attention_forward", "check_input_params"],
    "mindiesd/layers/flash_attn/attention_forward_varlen.py": ["attention_forward_varlen"],
    "mindiesd/layers/flash_attn/attention_func.py": ["attention_math"],
    "mindiesd/layers/flash_attn/common.py": ["AttentionParam.__init__", "lru_cache_by_attn_param"],
    "mindiesd/layers/flash_attn/sparse_flash_attn.py": ["sparse_attention"],
    "mindiesd/layers/flash_attn/sparse_flash_attn_rf_v2.py": "*",
    "mindiesd/layers/flash_attn/sparse_flash_attn_rf_v3.py": "*",
    "mindiesd/layers/flash_attn/sparse_flash_attn_ada_bsa.py": "*",
    "mindiesd/layers/_custom_ops.py": ["rain_fusion_attention", "block_sparse_attention", "sparse_block_estimate",
                                       "ada_block_sparse_attention", "rain_fusion_attention_fake",
                                       "block_sparse_attention_fake", "sparse_block_estimate_fake",
                                       "ada_block_sparse_attention_fake"],
    "mindiesd/layers/quant/block_quant.py": ["fa_block_quant_preprocess"],
    "mindiesd/layers/activation.py": ["get_activation_layer"],
    "mindiesd/quantization/layer.py": ["FP8RotateQuantFA.__init__", "FP8RotateQuantFA.forward",
                                       "W8A8MXFP8QuantLinear.__init__", "W8A8MXFP8QuantLinear.quant_matmul",
                                       # forward is inherited from the base class
                                       "W8A8QuantBaseLinear.forward"],
    "mindiesd/quantization/quantize.py": ["quantize"],
    "mindiesd/cache_agent/attention_cache.py": ["AttentionCache.apply_imp"],
}


def describe(fn, path):
    a = fn.args
    pos = [x.arg for x in a.posonlyargs + a.args]
    defaults = {}
    for name, d in zip(pos[len(pos) - len(a.defaults):], a.defaults):
        defaults[name] = ast.unparse(d)
    for x, d in zip(a.kwonlyargs, a.kw_defaults):
        if d is not None:
            defaults[x.arg] = ast.unparse(d)
    return {"at": f"{path}:{fn.lineno}", "args": pos, "kwonly": [x.arg for x in a.kwonlyargs],
            "vararg": a.vararg.arg if a.vararg else None, "kwarg": a.kwarg.arg if a.kwarg else None,
            "defaults": defaults}


def main(ref_root):
    table = {}
    for path, names in WANTED.items():
        with open(os.path.join(ref_root, path)) as f:
            tree = ast.parse(f.read())
        found = {}
        for node in tree.body:
            if isinstance(node, ast.FunctionDef):
                found[node.name] = node
            elif isinstance(node, ast.ClassDef):
                for sub in node.body:
                    if isinstance(sub, ast.FunctionDef):
                        found[f"{node.name}.{sub.name}"] = sub
                fields = [sub for sub in node.body if isinstance(sub, ast.AnnAssign)]
                if f"{node.name}.__init__" not in found and fields:
                    # a dataclass: its constructor takes self + the annotated fields in order
                    found[f"{node.name}.__init__"] = ast.FunctionDef(
                        name="__init__", lineno=node.lineno, args=ast.arguments(
                            posonlyargs=[], args=[ast.arg("self")] + [ast.arg(f.target.id) for f in fields],
                            vararg=None, kwonlyargs=[], kw_defaults=[], kwarg=None,
                            defaults=[f.value for f in fields if f.value is not None]))
        if names == "*":
            names = [n for n in found if "." not in n and not n.startswith("__")]
        module = path[:-3].replace("/", ".")
        for n in names:
            table[f"{module}:{n}"] = describe(found[n], path)
    out = os.path.join(HERE, "reference_signatures.json")
    with open(out, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
    print(out, len(table), "signatures")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
