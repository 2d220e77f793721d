"""``sparse_attention``: the sparse attention front door (mindiesd/layers/flash_attn/sparse_flash_attn.py:36-183)."""
from typing import Optional

import torch

from . import rainfusion as rf
from .hip_flash_attn import flash_attention
from .sparse_flash_attn_ada_bsa import ada_block_sparse_attention, get_estimate_mask
from ...utils.exception import ParametersInvalid


def check_params(input_layout, sparse_type):
    if input_layout not in ["BSND", "BNSD"]:
        raise ParametersInvalid(f"The input_layout must in ['BSND', 'BNSD'], but got {input_layout}.")
    if sparse_type not in [None, "rf_v2", "rf_v3", "ada_bsa"]:
        raise ParametersInvalid(f"sparse_type must be None, 'rf_v2', 'rf_v3' or 'ada_bsa', but got {sparse_type}.")


def sparse_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, attn_mask: Optional[torch.Tensor] = None,
                     scale: Optional[float] = None, is_causal: Optional[bool] = False, head_num: int = 1,
                     input_layout: str = "BNSD", inner_precise: int = 0, sparse_type: Optional[str] = None,
                     txt_len: int = 0, block_size: int = 128, latent_shape_q: Optional[list] = None,
                     latent_shape_k: Optional[list] = None, keep_sink: Optional[bool] = True,
                     keep_recent: Optional[bool] = True, cdf_threshold: float = 1.0, sparsity: float = 0.0, **kwargs):
    """Sparse attention over q/k/v in 'BNSD' ([B, N, S, D]) or 'BSND' ([B, S, N, D]).

    ``sparse_type``: None = dense flash attention; 'rf_v2' / 'rf_v3' = RainFusion2.0 block sparsity
    (index-list and int8-mask variants; both need ``latent_shape_q`` = (t, h, w) with
    t*h*w + txt_len == S, ``block_size`` 128 and ``sparsity`` in [0, 1)); 'ada_bsa' = adaptive block
    sparsity (mask estimated from strided anti-diagonal scores, ``cdf_threshold``, ``sparsity`` as the cap,
    ``keep_sink`` / ``keep_recent``, ``is_causal``).
    The output has the layout, dtype and token order of ``q``."""
    check_params(input_layout, sparse_type)
    head_dim = q.shape[-1]
    scale = head_dim ** -0.5 if scale is None else scale
    if sparse_type in ("rf_v2", "rf_v3") and latent_shape_q is None:
        raise ParametersInvalid("latent_shape_q is required for RainFusion sparse attention.")

    if sparse_type == "rf_v2":
        q_rf, k_rf, v_rf, qkv_pool = rf.do_tensor_rearrange_pooling(q, k, v, txt_len, block_size, latent_shape_q,
                                                                  latent_shape_k, input_layout)
        select_idx, select_num_idx = rf.get_blockwise_mask(qkv_pool, txt_len, sparsity, scale, block_size,
                                                           latent_shape_q, latent_shape_k, input_layout)
        batch = q.shape[0]
        if input_layout == "BSND":
            q_seq, kv_seq = q_rf.shape[1], k_rf.shape[1]
            n = q_rf.shape[2]
            layout = "TND"
            q_rf, k_rf, v_rf = (t.reshape(-1, n, head_dim) for t in (q_rf, k_rf, v_rf))
        else:
            q_seq, kv_seq = q_rf.shape[2], k_rf.shape[2]
            n = q_rf.shape[1]
            layout = input_layout
        out = rf.rain_fusion_attention(q_rf, k_rf, v_rf, scale=scale, head_num=n, input_layout=layout,
                                       select_idx=select_idx, select_num_idx=select_num_idx,
                                       blockshape=[block_size, block_size], actual_seq_lengths=[q_seq] * batch,
                                       actual_seq_lengths_kv=[kv_seq] * batch, inner_precise=inner_precise)
        if layout == "TND":
            out = out.reshape(batch, q_seq, n, head_dim)
        return rf.do_tensor_inv_rearrange(out, txt_len, latent_shape_q, latent_shape_k, input_layout)
    if sparse_type == "rf_v3":
        out, _ = rf.bsa_sparse_attention_v3(q, k, v, latent_shape_q=latent_shape_q, latent_shape_k=latent_shape_k,
                                            txt_len=txt_len, pool_size=block_size, sparsity=sparsity,
                                            input_layout=input_layout, head_num=head_num, scale=scale,
                                            inner_precise=inner_precise)
        return out
    if sparse_type == "ada_bsa":
        # sparse_flash_attn.py:151-173 of the reference
        smask, sct = get_estimate_mask(q, k, v, scale=scale, head_num=head_num, is_causal=is_causal,
                                       input_layout=input_layout, keep_sink=keep_sink, keep_recent=keep_recent,
                                       sparsity=sparsity, cdf_threshold=cdf_threshold, sparse_size=block_size)
        return ada_block_sparse_attention(q, k, v, smask, sct, scale=scale, head_num=head_num, is_causal=is_causal,
                                          input_layout=input_layout, sparse_size=block_size)
    return flash_attention(q, k, v, scale, input_layout)
