"""Oracle: RainFusion2.0 host pipeline on the CPU (test infrastructure only).

Restates mindiesd/layers/flash_attn/sparse_flash_attn_rf_v2.py (window permutation :137-289,
block mean pooling :24-73, block mask :94-134, index lists :76-91, pipeline glue :292-337)
and the rf_v3 glue of sparse_flash_attn_rf_v3.py (:193-295).

Rounding model.  The reference evaluates the mask in the *input dtype* with torch CPU ops:
block mean = cast_fp32 -> sum -> div -> cast (torch's ``mean`` for 16-bit types), ``einsum``
rounded to the dtype, ``* scale`` rounded to the dtype, ``softmax`` computed in fp32 and
rounded to the dtype, then ``topk`` / ``>=``.  The fp32 sums inside those ops depend on the
summation order of the BLAS / vectorised loops of the machine they run on, so the reference's
own result is only defined up to last-bit ties.  The oracle keeps every rounding point of the
reference but evaluates each sum EXACTLY (fp64 accumulation of 16-bit inputs is exact) before
rounding, which makes it independent of summation order; the HIP kernels do the same, so GPU
and oracle masks can be compared bit for bit.  ``get_blockwise_mask_torch`` is the literal
torch-op composite of the reference and is used by the tests to pin this oracle.
"""
import math

import numpy as np
import torch

from .attention import block_sparse_attention


# --------------------------------------------------------------------------------------------
# token permutation (rf_v2.py:137-196) expressed as a gather index list
# --------------------------------------------------------------------------------------------
def window_order(t, h, w):
    """src[i] = original (t,h,w)-flattened token index stored at position i after the rearrange.

    Grid aligned to 8 in both h and w: every frame is cut into 8x8 windows,
    ``(f hn hb wn wb) -> (f hn wn hb wb)`` (rf_v2.py:169-170).  Otherwise the first frame stays
    in place and each later frame becomes [8x8-windowed aligned part | bottom rows h >= h-h%8
    (all columns) | right columns w >= w-w%8 of the aligned rows] (rf_v2.py:148-167).
    """
    ids = np.arange(t * h * w, dtype=np.int64)
    if h % 8 == 0 and w % 8 == 0:
        return ids.reshape(t, h // 8, 8, w // 8, 8).transpose(0, 1, 3, 2, 4).reshape(-1)
    h8, w8 = h - h % 8, w - w % 8
    first = ids[: h * w]
    if t == 1:  # a single frame: nothing follows the frame that stays in place
        return first
    grid = ids[h * w:].reshape(t - 1, h, w)
    parts = [grid[:, :h8, :w8].reshape(t - 1, h8 // 8, 8, w8 // 8, 8).transpose(0, 1, 3, 2, 4).reshape(t - 1, -1)]
    if h % 8:
        parts.append(grid[:, h8:, :].reshape(t - 1, -1))
    if w % 8:
        parts.append(grid[:, :h8, w8:].reshape(t - 1, -1))
    return np.concatenate([first, np.concatenate(parts, axis=1).reshape(-1)])


def _seq_dim(layout):
    return 1 if layout == "BSND" else 2


def rearrange_with_remaining(tensor, latent_shape_q, latent_shape_k=None, input_layout="BNSD"):
    src = torch.from_numpy(window_order(*latent_shape_q))
    return tensor.index_select(_seq_dim(input_layout), src)


def inv_rearrange_with_remaining(tensor, latent_shape_q, latent_shape_k=None, input_layout="BNSD"):
    """Inverse of the rearrange (rf_v2.py:199-289; rf_v3.py:22-97 is a second implementation)."""
    src = window_order(*latent_shape_q)
    inv = np.empty_like(src)
    inv[src] = np.arange(src.size)
    return tensor.index_select(_seq_dim(input_layout), torch.from_numpy(inv))


# --------------------------------------------------------------------------------------------
# block mean pooling (rf_v2.py:24-73)
# --------------------------------------------------------------------------------------------
def avgpool(x, pool_size=128, input_layout="BNSD"):
    """Mean over consecutive ``pool_size``-token blocks; a shorter tail block is averaged over its
    own length (rf_v2.py:37-40, :60-63).  Exact sum -> fp32 -> fp32 divide -> input dtype."""
    dim = _seq_dim(input_layout)
    s = x.shape[dim]
    xs = x.double().movedim(dim, 0)
    outs = []
    for b0 in range(0, s, pool_size):
        blk = xs[b0:b0 + pool_size]
        tot = blk.sum(dim=0).to(torch.float32)
        outs.append((tot / np.float32(blk.shape[0])).to(x.dtype))
    return torch.stack(outs, dim=0).movedim(0, dim)


def do_tensor_rearrange_pooling(query, key, value, text_len, pool_size, latent_shape_q, latent_shape_k,
                                input_layout):
    """rf_v2.py:292-317: cat(q,k,v) on dim 0, text tokens (the first ``text_len``) moved behind the
    permuted image tokens, image and text pooled separately."""
    tensor = torch.cat((query, key, value), dim=0)
    dim = _seq_dim(input_layout)
    if text_len != 0:
        t_t = tensor.narrow(dim, 0, text_len)
        t_i = tensor.narrow(dim, text_len, tensor.shape[dim] - text_len)
        t_i2 = rearrange_with_remaining(t_i, latent_shape_q, latent_shape_k, input_layout)
        pool = torch.cat((avgpool(t_i2, pool_size, input_layout), avgpool(t_t, pool_size, input_layout)), dim=dim)
        tensor = torch.cat((t_i2, t_t), dim=dim)
    else:
        tensor = rearrange_with_remaining(tensor, latent_shape_q, latent_shape_k, input_layout)
        pool = avgpool(tensor, pool_size, input_layout)
    q_, k_, v_ = torch.chunk(tensor, 3, dim=0)
    return q_, k_, v_, pool


def do_tensor_inv_rearrange(tensor, text_len, latent_shape_q, latent_shape_k, input_layout):
    """rf_v2.py:321-337: undo the permutation and move the text tokens back to the front."""
    dim = _seq_dim(input_layout)
    if text_len != 0:
        s = tensor.shape[dim]
        t_t = tensor.narrow(dim, s - text_len, text_len)
        t_i = inv_rearrange_with_remaining(tensor.narrow(dim, 0, s - text_len), latent_shape_q, latent_shape_k,
                                           input_layout)
        return torch.cat((t_t, t_i), dim=dim)
    return inv_rearrange_with_remaining(tensor, latent_shape_q, latent_shape_k, input_layout)


# --------------------------------------------------------------------------------------------
# block mask (rf_v2.py:94-134) and index lists (rf_v2.py:76-91)
# --------------------------------------------------------------------------------------------
def keep_len_of(cols, sparsity):
    """rf_v2.py:112, evaluated in Python floats exactly like the reference."""
    return math.ceil(cols * (1 - sparsity))


def block_scores(qkv_pool, scale, input_layout="BNSD"):
    """softmax(q_pool . k_pool * scale) rounded like the reference (rf_v2.py:102-108), exact sums."""
    dtype = qkv_pool.dtype
    qp, kp, _ = torch.chunk(qkv_pool, 3, dim=0)
    if input_layout == "BSND":
        qp, kp = qp.transpose(1, 2), kp.transpose(1, 2)
    s = torch.einsum("bnld,bnsd->bnls", qp.double(), kp.double()).to(torch.float32).to(dtype)
    s = (s.to(torch.float32) * np.float32(scale)).to(dtype)
    x = s.double()
    e = torch.exp(x - x.max(dim=-1, keepdim=True).values)
    return (e / e.sum(dim=-1, keepdim=True)).to(torch.float32).to(dtype)


def apply_forced_blocks(mask, txt_len, pool_size, latent_shape_q, protect_first_frame=True):
    """rf_v2.py:116-126: text rows/cols (at the end) and first-frame rows/cols are always kept."""
    text_block_num = (txt_len + pool_size - 1) // pool_size
    if text_block_num > 0:
        mask[:, :, -text_block_num:, :] = True
        mask[:, :, :, -text_block_num:] = True
    if protect_first_frame:
        ff = (latent_shape_q[1] * latent_shape_q[2] + pool_size - 1) // pool_size
        if ff > 0:
            mask[:, :, :ff, :] = True
            mask[:, :, :, :ff] = True
    return mask


def get_mask_index(mask):
    """Per row: ascending indices of the True entries, padded with -1 (rf_v2.py:76-91)."""
    m = np.asarray(mask, dtype=bool)
    cols = m.shape[-1]
    idx = np.where(m, np.arange(cols), cols + 1)
    idx = np.sort(idx, axis=-1)
    cnt = m.sum(axis=-1, keepdims=True)
    return torch.from_numpy(np.where(np.arange(cols) < cnt, idx, -1).astype(np.int64))


def get_blockwise_mask(qkv_pool, txt_len, sparsity, scale, pool_size, latent_shape_q, latent_shape_k,
                       input_layout, return_binary=False, protect_first_frame=True, keep_diagonal=False):
    """rf_v2.py:94-134.  ``mask = score >= k-th largest score`` (ties keep extra blocks, :113-115).

    ``keep_diagonal`` ORs in the diagonal blocks; the reference has no such switch in rf_v2/rf_v3
    (its ada_bsa path has the analogous ``keep_recent``, csrc/ops/sparse_block_estimate/op_kernel/
    sparse_block_estimate.h:1051-1053); the Wan2.1-14B 720p workload of this build asks for it.
    """
    p = block_scores(qkv_pool, scale, input_layout)
    cols = p.shape[-1]
    keep_len = keep_len_of(cols, sparsity)
    kth = torch.topk(p.to(torch.float32), k=keep_len, dim=-1).values[..., -1:]
    mask = p.to(torch.float32) >= kth
    mask = apply_forced_blocks(mask, txt_len, pool_size, latent_shape_q, protect_first_frame)
    if keep_diagonal:
        d = torch.arange(min(mask.shape[-2], cols))
        mask[:, :, d, d] = True
    if return_binary:
        return mask.to(torch.int8)
    select_idx = get_mask_index(mask)[0].transpose(0, 1)
    select_num_idx = mask[0].transpose(0, 1).sum(dim=-1)
    return select_idx, select_num_idx


def get_blockwise_mask_torch(qkv_pool, txt_len, sparsity, scale, pool_size, latent_shape_q, latent_shape_k,
                             input_layout, protect_first_frame=True):
    """The reference's literal op sequence (rf_v2.py:102-126) with torch CPU kernels in the input
    dtype; returns the boolean mask.  Only used to pin ``get_blockwise_mask``."""
    qp, kp, _ = torch.chunk(qkv_pool, 3, dim=0)
    if input_layout == "BSND":
        scores = torch.einsum("blnd,bsnd->bnls", qp, kp) * scale
    else:
        scores = torch.einsum("bnld,bnsd->bnls", qp, kp) * scale
    sm = torch.nn.functional.softmax(scores, dim=-1)
    keep_len = keep_len_of(sm.shape[-1], sparsity)
    kth = torch.topk(sm, k=keep_len, dim=-1).values[..., -1:]
    return apply_forced_blocks(sm >= kth, txt_len, pool_size, latent_shape_q, protect_first_frame)


# --------------------------------------------------------------------------------------------
# end-to-end rf_v3 (rf_v3.py:193-295) on the CPU
# --------------------------------------------------------------------------------------------
def bsa_sparse_attention_v3(q, k, v, latent_shape_q, latent_shape_k=None, txt_len=0, pool_size=128, sparsity=0.5,
                            input_layout="BSND", scale=None, cached_mask=None, protect_first_frame=True,
                            keep_diagonal=False):
    """rearrange -> (pool -> mask | cached mask) -> block-sparse attention -> inverse rearrange.
    Returns (out fp32 in the input layout and token order, int8 mask)."""
    if latent_shape_k is None:
        latent_shape_k = latent_shape_q
    if scale is None:
        scale = float(q.shape[-1]) ** -0.5
    q_, k_, v_, pool = do_tensor_rearrange_pooling(q, k, v, txt_len, pool_size, latent_shape_q, latent_shape_k,
                                                   input_layout)
    if cached_mask is None:
        mask = get_blockwise_mask(pool, txt_len, sparsity, scale, pool_size, latent_shape_q, latent_shape_k,
                                  input_layout, return_binary=True, protect_first_frame=protect_first_frame,
                                  keep_diagonal=keep_diagonal)
    else:
        mask = cached_mask
    if input_layout == "BSND":
        q_, k_, v_ = (t.transpose(1, 2) for t in (q_, k_, v_))
    out = block_sparse_attention(q_, k_, v_, mask, scale=scale, block=pool_size)
    if input_layout == "BSND":
        out = out.transpose(1, 2)
    out = do_tensor_inv_rearrange(out, txt_len, latent_shape_q, latent_shape_k, input_layout)
    return out, mask
