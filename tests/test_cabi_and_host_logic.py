"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares, the
ctypes table matches the header, and the host logic of the front doors (argument checks, dispatch
key, LRU cache, registry, op schemas and fake implementations) behaves like the reference's."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mindiesd_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mindiesd_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    import mindiesd
    from mindiesd import _native
    path = _native.lib_path()
    if not os.path.isfile(path):
        import __graft_entry__
        __graft_entry__.build()
    handle = ctypes.CDLL(path)
    names = _declared_symbols()
    assert len(names) >= 13
    for name in names:
        assert hasattr(handle, name), f"{name} declared in the header but not exported"
    assert sorted(_native.SIGNATURES) == names, "ctypes table and header disagree"
    assert _native.lib() is _native.lib()


def test_argument_checks_without_gpu_calls():
    """Entry points validate before touching the device: null pointers / bad sizes give error 1."""
    from mindiesd import _native
    lib = _native.lib()
    z = [0] * 12
    assert lib.mindiesd_flash_attention_fwd(None, None, None, None, None, 0, 1, 1, 1, 1, 1, 128, *z, 1.0, None) == 1
    assert lib.mindiesd_mask_to_index(None, 1, 1, 1, None, None, 1, None) == 1
    assert lib.mindiesd_mx_quant(None, None, None, 0, 1, 32, 32, None) == 1
    assert lib.mindiesd_fp8_v_quant_workspace_size(2, 3) == 2 * 3 * 128 * 4
    with pytest.raises(RuntimeError):
        _native.check(2, "x")


def test_attention_forward_argument_checks():
    import mindiesd
    from mindiesd import ParametersInvalid
    q = torch.randn(1, 16, 2, 128, dtype=torch.bfloat16)
    for bad in (dict(query=1), dict(key="k"), dict(value=None)):
        args = dict(query=q, key=q, value=q)
        args.update(bad)
        with pytest.raises(ParametersInvalid):
            mindiesd.attention_forward(**args)
    with pytest.raises(ParametersInvalid):
        mindiesd.attention_forward(q[0], q, q)
    with pytest.raises(ParametersInvalid):
        mindiesd.attention_forward(q, q, q, fused=1)
    with pytest.raises(ParametersInvalid):
        mindiesd.attention_forward(q, q, q, scale=1)
    with pytest.raises(ParametersInvalid):
        mindiesd.attention_forward(q, q, q, attn_mask=[[1]])
    with pytest.raises(ParametersInvalid) as e:
        mindiesd.attention_forward(q, q, q, opt_mode="auto")
    assert "[MIE06E000001] Parameters invalid." in str(e.value)
    # fused call on CPU tensors must fail loudly, never fall back to torch math
    with pytest.raises(ParametersInvalid):
        mindiesd.attention_forward(q, q, q)
    out = mindiesd.attention_forward(q, q, q, fused=False)
    assert out.shape == q.shape and out.dtype == q.dtype


def test_unfused_path_is_the_reference_math():
    import mindiesd
    from oracle.attention import attention_math
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(2, 40, 3, 128, generator=g).to(torch.bfloat16) for _ in range(3))
    mask = torch.rand(40, 40, generator=g) > 0.3
    mask[:, 0] = True
    for head_first in (False, True):
        a = (q, k, v) if not head_first else tuple(t.transpose(1, 2) for t in (q, k, v))
        got = mindiesd.attention_forward(*a, attn_mask=mask, scale=0.1, fused=False, head_first=head_first)
        assert torch.equal(got, attention_math(*a, mask, 0.1, head_first=head_first))
    with pytest.raises(mindiesd.ParametersInvalid):
        mindiesd.attention_forward(q, k, v, attn_mask=torch.ones(3, 40, 40, dtype=torch.bool), fused=False)


def test_dispatch_key_lru_and_registry():
    from mindiesd.layers.flash_attn import common
    from mindiesd.layers.flash_attn.attention_func import get_attention_function, get_attention_function_runtime
    from mindiesd.layers.flash_attn.attention_operate import AttnOpRegistry, device_mi355x_op
    from mindiesd import ParametersInvalid
    p1 = common.AttentionParam(1, 12, 128, 4096, 4096, torch.bfloat16, True)
    p2 = common.AttentionParam(1, 12, 128, 4096, 4096, torch.bfloat16, False)
    assert p1.to_hash() != p2.to_hash() and "head_dim:128" in p1.to_str()
    common.attn_cache.clear()
    f1 = get_attention_function_runtime(p1)
    assert get_attention_function_runtime(p1) is f1 and len(common.attn_cache) == 1
    calls = []

    @common.lru_cache_by_attn_param(maxsize=2)
    def probe(param):
        calls.append(param.q_seqlen)
        return param.q_seqlen

    common.attn_cache.clear()
    ps = [common.AttentionParam(1, 1, 128, s, s, torch.float16, True) for s in (1, 2, 3)]
    for p in ps:
        probe(p)
    probe(ps[0])                      # evicted by the third insert -> computed again
    assert calls == [1, 2, 3, 1]
    common.attn_cache.clear()
    for name in ("hip_flash_attn", "prompt_flash_attn", "fused_attn_score", "ascend_laser_attention"):
        assert name in device_mi355x_op.get_all()
    with pytest.raises(ParametersInvalid):
        get_attention_function(p1, "nope", "BNSD")
    with pytest.raises(ParametersInvalid):
        get_attention_function(p1, "hip_flash_attn", "SBH")
    with pytest.raises(ParametersInvalid):
        get_attention_function(common.AttentionParam(1, 1, 128, 8, 8, torch.float32, True), "hip_flash_attn", "BNSD")
    with pytest.raises(ParametersInvalid):
        get_attention_function(common.AttentionParam(1, 1, 68, 8, 8, torch.float16, True), "hip_flash_attn", "BNSD")
    with pytest.raises(ParametersInvalid):
        get_attention_function(common.AttentionParam(1, 1, 264, 8, 8, torch.float16, True), "hip_flash_attn", "BNSD")
    get_attention_function(common.AttentionParam(1, 1, 64, 8, 8, torch.float16, True), "hip_flash_attn", "BNSD")
    reg = AttnOpRegistry()
    with pytest.raises(ParametersInvalid):
        reg.register(3, print)
    with pytest.raises(ParametersInvalid):
        reg.get("missing")


def test_op_schemas_and_fake_impls():
    import mindiesd  # noqa: F401
    q = torch.empty(2, 4, 300, 128, device="meta", dtype=torch.bfloat16)
    m = torch.empty(2, 4, 3, 3, device="meta", dtype=torch.int8)
    out, lse = torch.ops.mindiesd.block_sparse_attention(q, q, q, m)
    assert out.shape == q.shape and lse.shape == (2, 4, 300, 1) and lse.dtype == torch.float32
    t = torch.empty(600, 4, 128, device="meta", dtype=torch.float16)
    out, lse = torch.ops.mindiesd.block_sparse_attention(t, t, t, m, q_input_layout="TND", kv_input_layout="TND",
                                                         actual_seq_lengths=[300, 300], actual_seq_lengths_kv=[300, 300])
    assert out.shape == t.shape and lse.shape == (600, 4, 1)
    idx = torch.empty(3, 4, 3, device="meta", dtype=torch.int64)
    out, lse = torch.ops.mindiesd.rainfusionattention(q, q, q, idx, idx[..., 0], [128, 128], q_input_layout="BNSD",
                                                      kv_input_layout="BNSD", head_num=4)
    assert out.shape == q.shape and lse.shape == (2, 4, 300) and lse.dtype == q.dtype
    out, lse = torch.ops.mindiesd.flash_attention_fwd(q, q, q)
    assert out.shape == q.shape and lse.shape == (2, 4, 300)
    schema = str(torch.ops.mindiesd.block_sparse_attention.default._schema)
    block_shape = [a for a in torch.ops.mindiesd.block_sparse_attention.default._schema.arguments
                   if a.name == "block_shape"][0]
    assert block_shape.default_value == [128, 128] and str(block_shape.type) == "List[int]"
    for piece in ("Tensor? block_sparse_mask=None", "int[] block_shape=", "str q_input_layout=\"BNSD\"",
                  "int num_key_value_heads=1", "float scale_value=1.", "int softmax_lse_flag=0"):
        assert piece in schema, (piece, schema)


def test_new_ops_have_schemas_and_fake_impls():
    """The FP8 / MXFP8 / RainFusion-mask ops of this build on meta tensors (what torch.compile sees)."""
    import mindiesd  # noqa: F401
    x = torch.empty(2, 300, 4, 128, device="meta", dtype=torch.bfloat16)
    codes, scale = torch.ops.mindiesd.fa_block_quant(x, block_size=256, input_layout="BSND")
    assert codes.shape == (2, 4, 300, 128) and codes.dtype == torch.float8_e4m3fn
    assert scale.shape == (2, 4, 2, 1) and scale.dtype == torch.float32
    rot = torch.empty(128, 128, device="meta", dtype=torch.bfloat16)
    out = torch.ops.mindiesd.fp8_attention_fwd(x, x, x, scale_value=0.1, input_layout="BSND", q_rot=rot, k_rot=rot)
    assert out.shape == x.shape and out.dtype == x.dtype
    a = torch.empty(3, 50, 256, device="meta", dtype=torch.float16)
    w = torch.empty(512, 256, device="meta", dtype=torch.float8_e4m3fn)
    ws = torch.empty(512, 8, device="meta", dtype=torch.uint8)
    assert torch.ops.mindiesd.mxfp8_gemm_swiglu(a, w, ws).shape == (3, 50, 256)
    assert torch.ops.mindiesd.mxfp8_gemm_swiglu(a, w, ws, swiglu=False).shape == (3, 50, 512)
    pool = torch.empty(3, 4, 9, 128, device="meta", dtype=torch.bfloat16)
    mask = torch.ops.mindiesd.rf_block_mask(pool, 0, 0.5, 0.09, [2, 24, 24])
    assert mask.shape == (1, 4, 9, 9) and mask.dtype == torch.int8
    for name in ("fa_block_quant", "fp8_attention_fwd", "mxfp8_gemm_swiglu", "rf_block_mask"):
        assert hasattr(torch.ops.mindiesd, name)


def test_sparse_front_door_checks():
    import mindiesd
    q = torch.randn(1, 2, 256, 128, dtype=torch.bfloat16)
    with pytest.raises(mindiesd.ParametersInvalid):
        mindiesd.sparse_attention(q, q, q, input_layout="BSH")
    with pytest.raises(mindiesd.ParametersInvalid):
        mindiesd.sparse_attention(q, q, q, sparse_type="rf_v9")
    with pytest.raises(mindiesd.ParametersInvalid):
        mindiesd.sparse_attention(q, q, q, sparse_type="rf_v3")             # latent_shape_q missing
    with pytest.raises(mindiesd.ParametersInvalid):
        mindiesd.sparse_attention(q, q, q, sparse_type="rf_v3", latent_shape_q=(1, 16, 16))  # CPU tensors
    from mindiesd.layers.flash_attn.rainfusion import keep_len_of
    assert keep_len_of(591, 0.75) == 148
