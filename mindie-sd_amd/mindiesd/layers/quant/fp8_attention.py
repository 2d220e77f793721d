"""FP8 attention on the MI355X fp8 matrix cores.

Stands where the reference calls ``torch_npu.npu_fused_infer_attention_score_v2`` with per-block
dequantisation scales (mindiesd/quantization/layer.py:297-316).  Recipe: Q and K E4M3 with one fp32
scale per (head, 128-token block), V E4M3 with one scale per (head, channel), probabilities
re-quantised to E4M3 per tile, fp32 accumulation, output in the input dtype."""
import torch

from ... import _native
from ...utils.exception import ParametersInvalid
from ..flash_attn.hip_flash_attn import HEAD_DIM, _strides_bns
from .block_quant import _block_quant, _rot_block_quant


def quantize_v_per_channel(value, layout="BNSD"):
    """value [B,N,S,128] / [B,S,N,128] -> (V8T uint8 [B, N, 128, S128] in the kernel's transposed,
    key-permuted layout, fp32 per-channel scale [B, N, 128])."""
    if value.dtype not in _native.DTYPE_CODE or not value.is_cuda:
        raise ParametersInvalid(f"fp8 attention needs bf16/fp16 GPU tensors, but got {value.dtype} on {value.device}.")
    ok = value.stride(-1) == 1 and value.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in value.stride()[:-1])
    v = value if ok else value.contiguous()
    b, n, s = (v.shape[0], v.shape[1], v.shape[2]) if layout == "BNSD" else (v.shape[0], v.shape[2], v.shape[1])
    s128 = (s + 127) // 128 * 128
    v8t = torch.empty((b, n, HEAD_DIM, s128), dtype=torch.uint8, device=v.device)
    vscale = torch.empty((b, n, HEAD_DIM), dtype=torch.float32, device=v.device)
    lib = _native.lib()
    ws = torch.empty(lib.mindiesd_fp8_v_quant_workspace_size(b, n), dtype=torch.uint8, device=v.device)
    with _native.on_device(v.device):
        rc = lib.mindiesd_fp8_v_quant(v.data_ptr(), v8t.data_ptr(), vscale.data_ptr(), _native.DTYPE_CODE[v.dtype],
                                      b, n, s, HEAD_DIM, *_strides_bns(v, layout), ws.data_ptr(), ws.numel(),
                                      _native.stream_ptr(v.device))
    _native.check(rc, "mindiesd_fp8_v_quant")
    return v8t, vscale


LOG2E = 1.4426950408889634
# flag bits of mindiesd_fp8_attention_fwd (include/mindiesd_hip.h)
FLAG_LOG2_DOMAIN, FLAG_P_EXP2, FLAG_K_BLOCK_256 = 1, 2, 4
P_RULES = ("linear", "exp2")


def fp8_attention_quantized(q8, q_scale, k8, k_scale, v8t, v_scale, scale, out_dtype=torch.bfloat16, layout="BNSD",
                            log2_domain=False, p_rule="linear", k_block=128):
    """Attention on already quantised operands (see ``quantize_v_per_channel`` and ``_block_quant``
    with block 128).  Output [B,N,S,128] ('BNSD') or [B,S,N,128] ('BSND') in ``out_dtype``.
    ``log2_domain``: the query was quantised with ``prescale = scale * log2(e)`` and both q and k with
    power-of-two scales; ``scale`` is then not used.
    ``p_rule``: how a tile's probabilities become E4M3 - see ``fp8_attention_forward``.
    ``k_block``: 128 or 256 keys per entry of ``k_scale``."""
    if p_rule not in P_RULES:
        raise ParametersInvalid(f"p_rule must be one of {P_RULES}, but got {p_rule}.")
    if k_block not in (128, 256):
        raise ParametersInvalid(f"k_block must be 128 or 256, but got {k_block}.")
    flags = ((FLAG_LOG2_DOMAIN if log2_domain else 0) | (FLAG_P_EXP2 if p_rule == "exp2" else 0)
             | (FLAG_K_BLOCK_256 if k_block == 256 else 0))
    b, n, sq, d = q8.shape
    skv = k8.shape[2]
    shape = (b, n, sq, d) if layout == "BNSD" else (b, sq, n, d)
    out = torch.empty(shape, dtype=out_dtype, device=q8.device)
    with _native.on_device(q8.device):
        rc = _native.lib().mindiesd_fp8_attention_fwd(
            q8.data_ptr(), k8.data_ptr(), v8t.data_ptr(), q_scale.data_ptr(), k_scale.data_ptr(), v_scale.data_ptr(),
            out.data_ptr(), _native.DTYPE_CODE[out_dtype], b, n, sq, skv, d, *_strides_bns(out, layout),
            float(scale), flags, _native.stream_ptr(q8.device))
    _native.check(rc, "mindiesd_fp8_attention_fwd")
    return out


def fp8_attention_forward(query, key, value, scale=None, layout="BNSD", q_rot=None, k_rot=None, recipe="amax",
                          p_rule="linear", k_block=128):
    """Quantise q, k, v (bf16/fp16, 'BNSD' or 'BSND') and run FP8 attention; output like ``query``.
    ``q_rot`` / ``k_rot`` ([128, 128]): query @ q_rot and key @ k_rot are formed inside the quantisation
    pass (the rotated tensors are never written).
    ``recipe``: 'amax' (default, the reference's dynamic block quantisation) - Q and K block scales amax/448, the
    scores are rescaled in the softmax; 'pow2' - block scales rounded up to powers of two and the softmax scale
    folded into the query before quantisation, so the matrix instruction applies the scales through its exponent
    operands and the softmax needs no multiply (about 4 % faster).  On inputs without outliers both give the same
    accuracy; with amax/448 the largest element of every block is encoded exactly (code 448), which 'pow2' gives
    up, and on inputs whose softmax is decided by a few outliers that costs accuracy (cosine 0.979 against 0.987
    at 32760 tokens with 1 % of the elements scaled by 8).
    ``p_rule``: 'linear' (default) - the E4M3 code of a probability is computed directly as
    round(8 * (score - reference) + const): the exponential with its mantissa interpolated linearly between powers of
    two (at most 6 % above 2^x, 3 % rms after the common factor cancels against the denominator, which is summed
    from the same codes) - one multiply-add and one conversion per score; 'exp2' - 2^(score - reference) by the
    exponential instruction, rounded to E4M3 (slower: two quarter-rate instructions per score).  Both stay inside
    the FP8 workload's tolerance (cosine >= 0.999 against the quantise -> dequantise path).
    ``k_block``: tokens per K scale, 128 (default, the FP8 workload's recipe) or 256 (the K recipe of the reference's
    FP8RotateQuantFA, mindiesd/quantization/layer.py:297-302; not together with ``k_rot``, whose fused pass quantises
    per 128 tokens)."""
    for name, t in (("query", query), ("key", key), ("value", value)):
        if not isinstance(t, torch.Tensor) or t.dim() != 4:
            raise ParametersInvalid(f"The input {name} must be a 4-D torch.Tensor.")
    if layout not in ("BNSD", "BSND"):
        raise ParametersInvalid(f"Unsupported layout: {layout}, expected 'BNSD' or 'BSND'.")
    if key.shape != value.shape or query.shape[-1] != HEAD_DIM or key.shape[-1] != HEAD_DIM:
        raise ParametersInvalid("fp8 attention needs head_dim 128 and equal key/value shapes.")
    nq = query.shape[1] if layout == "BNSD" else query.shape[2]
    nk = key.shape[1] if layout == "BNSD" else key.shape[2]
    if nq != nk or query.shape[0] != key.shape[0]:
        raise ParametersInvalid("fp8 attention needs the same batch and head count for query and key/value.")
    if scale is None:
        scale = query.shape[-1] ** -0.5
    if recipe not in ("pow2", "amax"):
        raise ParametersInvalid(f"recipe must be 'pow2' or 'amax', but got {recipe}.")
    if k_block not in (128, 256) or (k_block == 256 and k_rot is not None):
        raise ParametersInvalid(f"k_block must be 128, or 256 without k_rot, but got {k_block}.")
    p2 = recipe == "pow2"
    pre = float(scale) * LOG2E if p2 else 1.0
    q8, qs = (_block_quant(query, 128, layout, pre, p2) if q_rot is None
              else _rot_block_quant(query, q_rot, layout, pre, p2))
    k8, ks = (_block_quant(key, k_block, layout, 1.0, p2) if k_rot is None
              else _rot_block_quant(key, k_rot, layout, 1.0, p2))
    v8t, vs = quantize_v_per_channel(value, layout)
    return fp8_attention_quantized(q8, qs, k8, ks, v8t, vs, scale, query.dtype, layout, log2_domain=p2, p_rule=p_rule,
                                   k_block=k_block)
