"""``torch.ops.mindiesd.*`` operators of the attention path and their keyword wrappers.

Schemas of ``rainfusionattention`` and ``block_sparse_attention`` are the reference's
(csrc/plugin/register_ops.cpp:41-45, :62-67), likewise ``ada_block_sparse_attention`` and
``sparse_block_estimate`` (:46-59); the wrappers mirror mindiesd/layers/_custom_ops.py
(:124-189, :204-305, :330-390).  New ops of this build (no counterpart in the reference, which reaches the
vendor kernels through torch_npu): ``flash_attention_fwd`` (dense kernel), ``fa_block_quant``, ``fp8_attention_fwd``,
``mxfp8_gemm_swiglu`` and ``rf_block_mask``; each has a fake implementation, so that ``torch.compile`` traces
through the FP8 / MXFP8 / RainFusion path the way the reference's ops do (mindiesd/layers/register_ops.py:90-128)."""
from typing import List, Optional, Tuple

import torch

from . import register_ops
from ..utils.exception import ParametersInvalid

register_ops.define_op(
    "rainfusionattention",
    "(Tensor query, Tensor key, Tensor value, Tensor select_idx, Tensor select_num_idx, int[] blockshape, "
    "Tensor? attn_mask=None, int[]? actual_seq_qlen=None, int[]? actual_seq_kvlen=None, Tensor? block_table=None, "
    "str q_input_layout='TND', str kv_input_layout='TND', int head_num=1, int mask_type=0, float scale=1.0, "
    "int inner_precise=1, int block_size=0) -> (Tensor, Tensor)")
register_ops.define_op(
    "block_sparse_attention",
    "(Tensor query, Tensor key, Tensor value, Tensor? block_sparse_mask=None, int[] block_shape=[128,128], "
    "str q_input_layout='BNSD', str kv_input_layout='BNSD', int num_key_value_heads=1, float scale_value=1.0, "
    "int inner_precise=0, int[]? actual_seq_lengths=None, int[]? actual_seq_lengths_kv=None, "
    "int softmax_lse_flag=0) -> (Tensor, Tensor)")
register_ops.define_op(
    "ada_block_sparse_attention",
    "(Tensor query, Tensor key, Tensor value, Tensor sparse_mask, Tensor sparse_count_table, "
    "str input_layout='BNSD', int sparse_size=128, int num_heads=1, int num_key_value_heads=1, float scale_value=1, "
    "bool causal=True, int inner_precise=1, int pre_tokens=214748647, int next_tokens=0, "
    "int[]? actual_seq_lengths=None, int[]? actual_seq_lengths_kv=None) -> Tensor")
register_ops.define_op(
    "sparse_block_estimate",
    "(Tensor query, Tensor key, int[]? actual_seq_lengths=None, int[]? actual_seq_lengths_kv=None, "
    "str input_layout='BNSD', int stride=8, int sparse_size=128, int num_heads=1, int num_key_value_heads=1, "
    "float scale_value=1, float threshold=1, bool causal=True, bool keep_sink=True, bool keep_recent=True, "
    "float row_sparse=1) -> (Tensor, Tensor)")
register_ops.define_op(
    "flash_attention_fwd",
    "(Tensor query, Tensor key, Tensor value, float scale_value=1.0, str input_layout='BNSD') -> (Tensor, Tensor)")
register_ops.define_op(
    "fa_block_quant",
    "(Tensor x, int block_size=128, str input_layout='BNSD') -> (Tensor, Tensor)")
register_ops.define_op(
    "fp8_attention_fwd",
    "(Tensor query, Tensor key, Tensor value, float scale_value=1.0, str input_layout='BNSD', Tensor? q_rot=None, "
    "Tensor? k_rot=None, str recipe='amax', str p_rule='linear') -> Tensor")
register_ops.define_op(
    "mxfp8_gemm_swiglu",
    "(Tensor x, Tensor weight, Tensor weight_scale, Tensor? bias=None, bool swiglu=True) -> Tensor")
register_ops.define_op(
    "rf_block_mask",
    "(Tensor qkv_pool, int txt_len, float sparsity, float scale, int[] latent_shape, str input_layout='BNSD', "
    "bool protect_first_frame=True, bool keep_diagonal=False) -> Tensor")


def _tnd_as_bsnd(t, seq_lens, what):
    """View a packed [T, N, D] tensor whose sequences all have one length as [B, S, N, D]."""
    if t.dim() != 3:
        raise RuntimeError(f"{what}: TND layout expects a 3-D tensor, got {t.dim()}-D")
    if not seq_lens:
        return t.unsqueeze(0)
    if len(set(seq_lens)) != 1 or seq_lens[0] * len(seq_lens) != t.shape[0]:
        raise RuntimeError(f"{what}: TND layout supports equal sequence lengths that sum to T only")
    return t.reshape(len(seq_lens), seq_lens[0], t.shape[1], t.shape[2])


def _varlen(what, *args, **kwargs):
    """rf.block_sparse_attention_varlen with argument errors as RuntimeError (what TORCH_CHECK gives in the
    reference's plugin)."""
    from .flash_attn import rainfusion as rf
    try:
        return rf.block_sparse_attention_varlen(*args, **kwargs)
    except ParametersInvalid as e:
        raise RuntimeError(f"{what}: {e}") from e


def _check_lengths(actual, s, what):
    if actual is not None and any(int(a) != s for a in actual):
        raise RuntimeError(f"{what}: per-batch sequence lengths shorter than the tensor are not supported")


@register_ops.register_device_impl("flash_attention_fwd")
def _flash_attention_fwd_impl(query, key, value, scale_value=1.0, input_layout="BNSD"):
    from .flash_attn.hip_flash_attn import flash_attention
    if input_layout not in ("BNSD", "BSND"):
        raise RuntimeError(f"flash_attention_fwd: input_layout only supports 'BNSD' and 'BSND', got {input_layout}")
    return flash_attention(query, key, value, scale_value, input_layout, return_lse=True)


@register_ops.register_mindie_fake_op("flash_attention_fwd")
def _flash_attention_fwd_fake(query, key, value, scale_value=1.0, input_layout="BNSD"):
    b, n, s = (query.shape[0], query.shape[1], query.shape[2]) if input_layout == "BNSD" else \
        (query.shape[0], query.shape[2], query.shape[1])
    return torch.empty_like(query), torch.empty((b, n, s), device=query.device, dtype=torch.float32)


@register_ops.register_device_impl("block_sparse_attention")
def _block_sparse_attention_impl(query, key, value, block_sparse_mask=None, block_shape=(128, 128),
                                 q_input_layout="BNSD", kv_input_layout="BNSD", num_key_value_heads=1,
                                 scale_value=1.0, inner_precise=0, actual_seq_lengths=None,
                                 actual_seq_lengths_kv=None, softmax_lse_flag=0):
    """csrc/plugin/block_sparse_attention.cpp:31-121: same argument checks (RuntimeError), callee
    allocates ``(attention_out like query, softmax_lse fp32 [B,N,S,1] or [T,N,1])``; the lse is only
    written when ``softmax_lse_flag != 0``."""
    from .flash_attn import rainfusion as rf
    if q_input_layout not in ("TND", "BNSD"):
        raise RuntimeError(f"block_sparse_attention: q_input_layout only supports 'TND' and 'BNSD', got {q_input_layout}")
    if kv_input_layout not in ("TND", "BNSD"):
        raise RuntimeError(f"block_sparse_attention: kv_input_layout only supports 'TND' and 'BNSD', got {kv_input_layout}")
    if q_input_layout != kv_input_layout:
        raise RuntimeError("block_sparse_attention: q_input_layout and kv_input_layout must be consistent.")
    if q_input_layout == "TND" and (actual_seq_lengths is None or actual_seq_lengths_kv is None):
        raise RuntimeError("block_sparse_attention: actual_seq_lengths and actual_seq_lengths_kv are required "
                           "for TND layout.")
    if list(block_shape) != [128, 128]:
        raise RuntimeError(f"block_sparse_attention: block_shape only supports [128, 128], got {list(block_shape)}")
    if block_sparse_mask is None:
        raise RuntimeError("block_sparse_attention: block_sparse_mask is required")
    want_lse = softmax_lse_flag != 0
    lens_q = [int(x) for x in actual_seq_lengths] if actual_seq_lengths is not None else None
    lens_kv = [int(x) for x in actual_seq_lengths_kv] if actual_seq_lengths_kv is not None else None
    if q_input_layout == "TND":
        equal = len(set(lens_q)) == 1 and len(set(lens_kv)) == 1 and len(lens_q) == len(lens_kv)
        if not equal:  # sequences of different lengths packed one after the other
            res = _varlen("block_sparse_attention", query, key, value, block_sparse_mask, scale_value, lens_q, lens_kv,
                          "TND", return_lse=want_lse)
            out, lse = res if want_lse else (res, None)
            lse_out = lse.unsqueeze(-1) if want_lse else torch.empty(
                (query.shape[0], query.shape[1], 1), dtype=torch.float32, device=query.device)
            return out, lse_out
        q4 = _tnd_as_bsnd(query, lens_q, "block_sparse_attention")
        k4 = _tnd_as_bsnd(key, lens_kv, "block_sparse_attention")
        v4 = _tnd_as_bsnd(value, lens_kv, "block_sparse_attention")
        layout = "BSND"
    else:
        q4, k4, v4, layout = query, key, value, "BNSD"
        full_q = lens_q is None or all(x == query.shape[2] for x in lens_q)
        full_kv = lens_kv is None or all(x == key.shape[2] for x in lens_kv)
        if not (full_q and full_kv):  # batch entries shorter than the tensor
            res = _varlen("block_sparse_attention", query, key, value, block_sparse_mask, scale_value,
                          lens_q if lens_q is not None else [query.shape[2]] * query.shape[0],
                          lens_kv if lens_kv is not None else [key.shape[2]] * key.shape[0], "BNSD", return_lse=want_lse)
            out, lse = res if want_lse else (res, None)
            lse_out = lse.unsqueeze(-1) if want_lse else torch.empty(
                (query.shape[0], query.shape[1], query.shape[2], 1), dtype=torch.float32, device=query.device)
            return out, lse_out
    res = rf.block_sparse_attention_mask(q4, k4, v4, block_sparse_mask, scale_value, layout, return_lse=want_lse)
    out, lse = res if want_lse else (res, None)
    if q_input_layout == "TND":
        out = out.reshape(query.shape)
        lse_out = torch.empty((query.shape[0], query.shape[1], 1), dtype=torch.float32, device=query.device)
        if want_lse:  # [B, N, S] -> [T, N, 1]
            lse_out.copy_(lse.permute(0, 2, 1).reshape(query.shape[0], query.shape[1], 1))
    else:
        lse_out = lse.unsqueeze(-1) if want_lse else torch.empty(
            (query.shape[0], query.shape[1], query.shape[2], 1), dtype=torch.float32, device=query.device)
    return out, lse_out


@register_ops.register_mindie_fake_op("block_sparse_attention")
def block_sparse_attention_fake(query, key, value, block_sparse_mask=None, block_shape=None, q_input_layout="BNSD",
                                kv_input_layout="BNSD", num_key_value_heads=1, scale_value=1.0, inner_precise=0,
                                actual_seq_lengths=None, actual_seq_lengths_kv=None, softmax_lse_flag=0):
    if q_input_layout == "TND":
        lse_shape = [query.shape[0], query.shape[1], 1]
    else:
        lse_shape = [query.shape[0], query.shape[1], query.shape[2], 1]
    return torch.empty_like(query), torch.empty(lse_shape, device=query.device, dtype=torch.float32)


@register_ops.register_device_impl("rainfusionattention")
def _rainfusionattention_impl(query, key, value, select_idx, select_num_idx, blockshape, attn_mask=None,
                              actual_seq_qlen=None, actual_seq_kvlen=None, block_table=None, q_input_layout="TND",
                              kv_input_layout="TND", head_num=1, mask_type=0, scale=1.0, inner_precise=1,
                              block_size=0):
    """csrc/plugin/rainfusionattention.cpp:27-64.  ``select_idx`` [qb, N, kb] (-1 padded),
    ``select_num_idx`` [qb, N]: one selection shared by every batch entry (the reference builds it
    from batch 0, sparse_flash_attn_rf_v2.py:131-134).  Returns ``(out, softmax_lse)`` with the
    reference's lse shape ``query.shape[:3]`` in the query dtype."""
    from .flash_attn import rainfusion as rf
    if q_input_layout not in ("TND", "BNSD"):
        raise RuntimeError("q_input_layout only supports 'TND' and 'BNSD' now.")
    if kv_input_layout not in ("TND", "BNSD"):
        raise RuntimeError("kv_input_layout only supports 'TND' and 'BNSD' now.")
    if q_input_layout != kv_input_layout:
        raise RuntimeError("q_input_layout and kv_input_layout must be consistent.")
    if list(blockshape) != [128, 128]:
        raise RuntimeError(f"blockshape only supports [128, 128], got {list(blockshape)}")
    if attn_mask is not None or block_table is not None or mask_type != 0 or block_size != 0:
        raise RuntimeError("attn_mask / block_table / mask_type / block_size are not supported.")
    lens_q = [int(x) for x in actual_seq_qlen] if actual_seq_qlen else None
    lens_kv = [int(x) for x in actual_seq_kvlen] if actual_seq_kvlen else None
    unequal = q_input_layout == "TND" and lens_q and lens_kv and (len(set(lens_q)) > 1 or len(set(lens_kv)) > 1)
    if unequal:
        q4 = k4 = v4 = None
        layout, b, n = "TND", len(lens_q), query.shape[1]
    elif q_input_layout == "TND":
        q4 = _tnd_as_bsnd(query, lens_q, "rainfusionattention")
        k4 = _tnd_as_bsnd(key, lens_kv, "rainfusionattention")
        v4 = _tnd_as_bsnd(value, lens_kv, "rainfusionattention")
        layout = "BSND"
        b, n = q4.shape[0], q4.shape[2]
    else:
        q4, k4, v4, layout = query, key, value, "BNSD"
        b, n = query.shape[0], query.shape[1]
    if select_idx.dim() != 3 or select_idx.shape[1] != n or tuple(select_num_idx.shape) != tuple(select_idx.shape[:2]):
        raise RuntimeError("select_idx must be [q_blocks, N, kv_blocks] and select_num_idx [q_blocks, N]")
    # The selection as an int8 mask: entry j of a row counts if j < select_num_idx and the id names a key block
    # (ids outside [0, kv_blocks) and entries past the count are dropped, so a malformed list cannot make the
    # kernel read outside its tables).  The mask form runs the kernel over paired query blocks.
    skv = max(lens_kv) if unequal else (k4.shape[2] if layout == "BNSD" else k4.shape[1])
    kb = (skv + 127) // 128
    sel = select_idx.permute(1, 0, 2).to(torch.int64)                               # [N, qb, width]
    num = select_num_idx.permute(1, 0).to(torch.int64).unsqueeze(-1)                # [N, qb, 1]
    pos = torch.arange(sel.shape[-1], device=sel.device).view(1, 1, -1)
    valid = (pos < num) & (sel >= 0) & (sel < kb)
    mask = torch.zeros((n, sel.shape[1], kb + 1), dtype=torch.int8, device=sel.device)
    mask.scatter_(2, torch.where(valid, sel + 1, torch.zeros_like(sel)), 1)         # column 0 takes the dropped ones
    mask = mask[:, :, 1:].unsqueeze(0).expand(b, -1, -1, -1).contiguous()
    if unequal:  # packed sequences of different lengths, the same selection for each
        out, lse = _varlen("rainfusionattention", query, key, value, mask, scale, lens_q, lens_kv, "TND", return_lse=True)
        lse_out = torch.zeros(query.shape, dtype=query.dtype, device=query.device)
        lse_out[:, :, 0] = lse.to(query.dtype)
        return out, lse_out
    out, lse = rf.block_sparse_attention_mask(q4, k4, v4, mask, scale, layout, return_lse=True)
    if q_input_layout == "TND":
        out = out.reshape(query.shape)
        lse_out = torch.zeros(query.shape, dtype=query.dtype, device=query.device)
        lse_out[:, :, 0] = lse.permute(0, 2, 1).reshape(query.shape[0], query.shape[1]).to(query.dtype)
    else:
        lse_out = lse.to(query.dtype)
    return out, lse_out


@register_ops.register_mindie_fake_op("rainfusionattention")
def rain_fusion_attention_fake(query, key, value, select_idx, select_num_idx, blockshape, attn_mask=None,
                               actual_seq_qlen=None, actual_seq_kvlen=None, block_table=None, q_input_layout="TND",
                               kv_input_layout="TND", head_num=1, mask_type=0, scale=1.0, inner_precise=1,
                               block_size=0):
    lse = torch.empty([query.shape[0], query.shape[1], query.shape[2]], device=query.device, dtype=query.dtype)
    return torch.empty_like(query), lse


def rain_fusion_attention(query, key, value, select_idx, select_num_idx, blockshape: List[int],
                          attn_mask: Optional[torch.Tensor] = None, actual_seq_qlen: Optional[List[int]] = None,
                          actual_seq_kvlen: Optional[List[int]] = None, block_table: Optional[torch.Tensor] = None,
                          q_input_layout: str = "TND", kv_input_layout: str = "TND", head_num: int = 1,
                          mask_type: int = 0, scale: float = 1.0, inner_precise: int = 1,
                          block_size: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    return torch.ops.mindiesd.rainfusionattention(
        query=query, key=key, value=value, select_idx=select_idx, select_num_idx=select_num_idx,
        blockshape=blockshape, attn_mask=attn_mask, actual_seq_qlen=actual_seq_qlen,
        actual_seq_kvlen=actual_seq_kvlen, block_table=block_table, q_input_layout=q_input_layout,
        kv_input_layout=kv_input_layout, head_num=head_num, mask_type=mask_type, scale=scale,
        inner_precise=inner_precise, block_size=block_size)


def block_sparse_attention(query, key, value, block_sparse_mask: Optional[torch.Tensor] = None,
                           block_shape: List[int] = None, q_input_layout: str = "BNSD", kv_input_layout: str = "BNSD",
                           num_key_value_heads: int = 1, scale_value: float = 1.0, inner_precise: int = 0,
                           actual_seq_lengths: Optional[List[int]] = None,
                           actual_seq_lengths_kv: Optional[List[int]] = None,
                           softmax_lse_flag: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
    kwargs = dict(query=query, key=key, value=value, block_sparse_mask=block_sparse_mask,
                  block_shape=block_shape if block_shape is not None else [128, 128],
                  q_input_layout=q_input_layout, kv_input_layout=kv_input_layout,
                  num_key_value_heads=num_key_value_heads, scale_value=scale_value, inner_precise=inner_precise,
                  softmax_lse_flag=softmax_lse_flag)
    if actual_seq_lengths is not None:
        kwargs["actual_seq_lengths"] = actual_seq_lengths
    if actual_seq_lengths_kv is not None:
        kwargs["actual_seq_lengths_kv"] = actual_seq_lengths_kv
    return torch.ops.mindiesd.block_sparse_attention(**kwargs)


# ---- adaptive block-sparse attention (mindiesd/layers/_custom_ops.py:204-305) -----------------------------------
@register_ops.register_device_impl("sparse_block_estimate")
def _sparse_block_estimate_impl(query, key, actual_seq_lengths=None, actual_seq_lengths_kv=None, input_layout="BNSD",
                                stride=8, sparse_size=128, num_heads=1, num_key_value_heads=1, scale_value=1.0,
                                threshold=1.0, causal=True, keep_sink=True, keep_recent=True, row_sparse=1.0):
    from .flash_attn.ada_bsa import sparse_block_estimate as run
    s = query.shape[2] if input_layout == "BNSD" else query.shape[1]
    _check_lengths(actual_seq_lengths, s, "sparse_block_estimate")
    _check_lengths(actual_seq_lengths_kv, s, "sparse_block_estimate")
    return run(query, key, input_layout, stride, sparse_size, scale_value, threshold, causal, keep_sink, keep_recent,
               row_sparse)


@register_ops.register_mindie_fake_op("sparse_block_estimate")
def sparse_block_estimate_fake(query, key, actual_seq_lengths=None, actual_seq_lengths_kv=None, input_layout="BNSD",
                               stride=8, sparse_size=128, num_heads=1, num_key_value_heads=1, scale_value=1.0,
                               threshold=1.0, causal=False, keep_sink=True, keep_recent=True, row_sparse=1.0):
    b, nq, s = (query.shape[0], query.shape[1], query.shape[2]) if input_layout == "BNSD" else \
        (query.shape[0], query.shape[2], query.shape[1])
    nb = (s + sparse_size - 1) // sparse_size
    return (torch.empty((b, nq, nb, (nb + 31) // 32 * 32), device=query.device, dtype=torch.int8),
            torch.empty((b, nq, nb), device=query.device, dtype=torch.int32))


def sparse_block_estimate(query, key, actual_seq_lengths: Optional[List[int]] = None,
                          actual_seq_lengths_kv: Optional[List[int]] = None, input_layout: str = "BNSD",
                          stride: int = 8, sparse_size: int = 128, num_heads: int = 1, num_key_value_heads: int = 1,
                          scale_value: float = 1.0, threshold: float = 1.0, causal: bool = False,
                          keep_sink: bool = True, keep_recent: bool = True,
                          row_sparse: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    return torch.ops.mindiesd.sparse_block_estimate(
        query=query, key=key, actual_seq_lengths=actual_seq_lengths, actual_seq_lengths_kv=actual_seq_lengths_kv,
        input_layout=input_layout, stride=stride, sparse_size=sparse_size,
        num_heads=1 if num_heads is None else num_heads,
        num_key_value_heads=1 if num_key_value_heads is None else num_key_value_heads, scale_value=scale_value,
        threshold=threshold, causal=causal, keep_sink=keep_sink, keep_recent=keep_recent, row_sparse=row_sparse)


@register_ops.register_device_impl("ada_block_sparse_attention")
def _ada_block_sparse_attention_impl(query, key, value, sparse_mask, sparse_count_table, input_layout="BNSD",
                                     sparse_size=128, num_heads=1, num_key_value_heads=1, scale_value=1.0, causal=True,
                                     inner_precise=1, pre_tokens=214748647, next_tokens=0, actual_seq_lengths=None,
                                     actual_seq_lengths_kv=None):
    from .flash_attn.ada_bsa import ada_block_sparse_attention as run
    s = query.shape[2] if input_layout == "BNSD" else query.shape[1]
    _check_lengths(actual_seq_lengths, s, "ada_block_sparse_attention")
    _check_lengths(actual_seq_lengths_kv, s, "ada_block_sparse_attention")
    return run(query, key, value, sparse_mask, sparse_count_table, input_layout, sparse_size, scale_value, causal)


@register_ops.register_mindie_fake_op("ada_block_sparse_attention")
def ada_block_sparse_attention_fake(query, key, value, sparse_mask, sparse_count_table, input_layout="BNSD",
                                    sparse_size=128, num_heads=1, num_key_value_heads=1, scale_value=1.0, causal=False,
                                    inner_precise=1, pre_tokens=214748647, next_tokens=214748647, actual_seq_lengths=None,
                                    actual_seq_lengths_kv=None):
    return torch.empty_like(query)


def ada_block_sparse_attention(query, key, value, sparse_mask, sparse_count_table, input_layout: str = "BNSD",
                               sparse_size: int = 128, num_heads: int = 1, num_key_value_heads: int = 1,
                               scale_value: float = 1.0, causal: bool = False, inner_precise: int = 1,
                               pre_tokens: int = 214748647, next_tokens: int = 214748647,
                               actual_seq_lengths: Optional[List[int]] = None,
                               actual_seq_lengths_kv: Optional[List[int]] = None) -> torch.Tensor:
    return torch.ops.mindiesd.ada_block_sparse_attention(
        query=query, key=key, value=value, sparse_mask=sparse_mask, sparse_count_table=sparse_count_table,
        input_layout=input_layout, sparse_size=sparse_size, num_heads=1 if num_heads is None else num_heads,
        num_key_value_heads=1 if num_key_value_heads is None else num_key_value_heads, scale_value=scale_value,
        causal=causal, inner_precise=inner_precise, pre_tokens=pre_tokens, next_tokens=next_tokens,
        actual_seq_lengths=actual_seq_lengths, actual_seq_lengths_kv=actual_seq_lengths_kv)


# ---- FP8 / MXFP8 / RainFusion mask as ops --------------------------------------------------------------------------
@register_ops.register_device_impl("fa_block_quant")
def _fa_block_quant_impl(x, block_size=128, input_layout="BNSD"):
    """-> (float8_e4m3fn [B, N, S, D], fp32 scale [B, N, ceil(S / block_size), 1]); see fa_block_quant_preprocess."""
    from .quant.block_quant import fa_block_quant_preprocess
    return fa_block_quant_preprocess(x, block_size=block_size, layout=input_layout)


@register_ops.register_mindie_fake_op("fa_block_quant")
def _fa_block_quant_fake(x, block_size=128, input_layout="BNSD"):
    b, n, s = (x.shape[0], x.shape[1], x.shape[2]) if input_layout == "BNSD" else (x.shape[0], x.shape[2], x.shape[1])
    return (torch.empty((b, n, s, x.shape[3]), device=x.device, dtype=torch.float8_e4m3fn),
            torch.empty((b, n, (s + block_size - 1) // block_size, 1), device=x.device, dtype=torch.float32))


@register_ops.register_device_impl("fp8_attention_fwd")
def _fp8_attention_fwd_impl(query, key, value, scale_value=1.0, input_layout="BNSD", q_rot=None, k_rot=None,
                            recipe="amax", p_rule="linear"):
    from .quant.fp8_attention import fp8_attention_forward
    return fp8_attention_forward(query, key, value, scale_value, input_layout, q_rot, k_rot, recipe, p_rule)


@register_ops.register_mindie_fake_op("fp8_attention_fwd")
def _fp8_attention_fwd_fake(query, key, value, scale_value=1.0, input_layout="BNSD", q_rot=None, k_rot=None,
                            recipe="amax", p_rule="linear"):
    return torch.empty_like(query)


@register_ops.register_device_impl("mxfp8_gemm_swiglu")
def _mxfp8_gemm_swiglu_impl(x, weight, weight_scale, bias=None, swiglu=True):
    """x [.., K] bf16/fp16 (quantised here, per 32 values along K), weight E4M3 [Nw, K] with E8M0 scales
    [Nw, K/32]; ``swiglu``: weight rows are [gate | up] and the result is silu(gate) * up [.., Nw/2]."""
    from .quant.mxfp8 import mx_quantize, mxfp8_matmul
    x2 = x.reshape(-1, x.shape[-1])
    xq, xs = mx_quantize(x2)
    out = mxfp8_matmul(xq, xs, weight, weight_scale, bias, x.dtype, swiglu)
    return out.view(*x.shape[:-1], out.shape[-1])


@register_ops.register_mindie_fake_op("mxfp8_gemm_swiglu")
def _mxfp8_gemm_swiglu_fake(x, weight, weight_scale, bias=None, swiglu=True):
    nout = weight.shape[0] // 2 if swiglu else weight.shape[0]
    return torch.empty((*x.shape[:-1], nout), device=x.device, dtype=x.dtype)


@register_ops.register_device_impl("rf_block_mask")
def _rf_block_mask_impl(qkv_pool, txt_len, sparsity, scale, latent_shape, input_layout="BNSD",
                        protect_first_frame=True, keep_diagonal=False):
    from .flash_attn.rainfusion import get_blockwise_mask
    return get_blockwise_mask(qkv_pool, txt_len, sparsity, scale, 128, list(latent_shape), list(latent_shape),
                              input_layout, return_binary=True, protect_first_frame=protect_first_frame,
                              keep_diagonal=keep_diagonal)


@register_ops.register_mindie_fake_op("rf_block_mask")
def _rf_block_mask_fake(qkv_pool, txt_len, sparsity, scale, latent_shape, input_layout="BNSD",
                        protect_first_frame=True, keep_diagonal=False):
    b = qkv_pool.shape[0] // 3
    n, nb = (qkv_pool.shape[1], qkv_pool.shape[2]) if input_layout == "BNSD" else (qkv_pool.shape[2], qkv_pool.shape[1])
    return torch.empty((b, n, nb, nb), device=qkv_pool.device, dtype=torch.int8)
