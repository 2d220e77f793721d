"""RainFusion2.0 block-sparse attention on the MI355X.

GPU counterparts of the reference's host pipeline
(mindiesd/layers/flash_attn/sparse_flash_attn_rf_v2.py and sparse_flash_attn_rf_v3.py):
window permutation and block mean pooling run as one HBM pass, the block mask (pooled scores,
softmax, top-k threshold, forced text / first-frame blocks) as one kernel that also emits the
compacted block lists the attention kernel walks, then the block-sparse flash-attention kernel and
the inverse permutation.  Every function keeps the reference's signature and layouts.
"""
import math

import threading

import torch

from .hip_flash_attn import HEAD_DIM, _strides_bns
from ... import _native
from ...utils.exception import ParametersInvalid

BLOCK = 128


def _check_gpu16(t, what):
    if not isinstance(t, torch.Tensor) or t.dim() != 4:
        raise ParametersInvalid(f"{what} must be a 4-D torch.Tensor.")
    if not t.is_cuda:
        raise ParametersInvalid(f"{what} must live on the GPU, but is on {t.device}.")
    if t.dtype not in _native.DTYPE_CODE:
        raise ParametersInvalid(f"{what} must be bf16 or fp16, but got {t.dtype}.")
    if t.shape[-1] != HEAD_DIM:
        raise ParametersInvalid(f"{what} must have head_dim == {HEAD_DIM}, but got {t.shape[-1]}.")


def _check_layout(input_layout):
    if input_layout not in ("BSND", "BNSD"):
        raise ParametersInvalid(f"The input_layout must in ['BSND', 'BNSD'], but got {input_layout}.")


def _dims(t, layout):
    """(B, N, S) of a 4-D tensor in ``layout``."""
    return (t.shape[0], t.shape[1], t.shape[2]) if layout == "BNSD" else (t.shape[0], t.shape[2], t.shape[1])


def _aligned(t):
    ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:-1])
    return t if ok else t.contiguous()


def _pool_strides(pool, layout):
    """(batch, head, block) strides of a pooled tensor [X, N, NB, D] / [X, NB, N, D]."""
    return _strides_bns(pool, layout)


def _run_rearrange(srcs, dsts, pool, layout, grid, txt_len, inverse):
    """Launch the permute(+pool) kernel on 1..3 same-shaped tensors.  ``grid`` = (t, h, w) or
    (0, 0, 0) for the identity order.  ``pool`` is [len(srcs) * B, ...] in ``layout`` or None."""
    x = srcs[0]
    b, n, s = _dims(x, layout)
    ptr = lambda lst, i: lst[i].data_ptr() if i < len(lst) and lst[i] is not None else None
    d0 = next((d for d in (dsts or []) if d is not None), x)  # all destinations share one set of strides
    if pool is not None:
        psb, psn, psblk = _pool_strides(pool, layout)
        pst = b * pool.stride(0)
    else:
        pst = psb = psn = psblk = 0
    with _native.on_device(x.device):
        rc = _native.lib().mindiesd_rf_rearrange_pool(
            ptr(srcs, 0), ptr(srcs, 1), ptr(srcs, 2), ptr(dsts, 0), ptr(dsts, 1), ptr(dsts, 2),
            pool.data_ptr() if pool is not None else None, _native.DTYPE_CODE[x.dtype], b, n, s, x.shape[-1],
            *_strides_bns(x, layout), *_strides_bns(d0, layout), pst, psb, psn, psblk,
            int(grid[0]), int(grid[1]), int(grid[2]), int(txt_len), int(inverse), len(srcs),
            _native.stream_ptr(x.device))
    _native.check(rc, "mindiesd_rf_rearrange_pool")


def _same_strides(ts):
    return all(t.stride() == ts[0].stride() and t.shape == ts[0].shape for t in ts)


def _check_grid(latent_shape, s_img):
    t, h, w = (int(v) for v in latent_shape)
    if t <= 0 or h < 8 or w < 8:
        raise ParametersInvalid(f"latent_shape_q must be (t, h, w) with h >= 8 and w >= 8, but got {latent_shape}.")
    if t * h * w != s_img:
        raise ParametersInvalid(f"latent_shape_q {latent_shape} does not match the image sequence length {s_img}.")
    return t, h, w


# ------------------------------------------------------------------------------------------------
# rf_v2.py:24-73
# ------------------------------------------------------------------------------------------------
def avgpool(input_tensor, pool_size=128, input_layout="BNSD"):
    """Mean over consecutive 128-token blocks (a shorter tail block averages its own length)."""
    _check_layout(input_layout)
    _check_gpu16(input_tensor, "input_tensor")
    if pool_size != BLOCK:
        raise ParametersInvalid(f"pool_size only supports {BLOCK}, but got {pool_size}.")
    x = _aligned(input_tensor)
    b, n, s = _dims(x, input_layout)
    nb = (s + BLOCK - 1) // BLOCK
    shape = (b, n, nb, x.shape[-1]) if input_layout == "BNSD" else (b, nb, n, x.shape[-1])
    pool = torch.empty(shape, dtype=x.dtype, device=x.device)
    _run_rearrange([x], [None], pool, input_layout, (0, 0, 0), 0, 0)
    return pool


# ------------------------------------------------------------------------------------------------
# rf_v2.py:137-289
# ------------------------------------------------------------------------------------------------
def rearrange_with_remaining(tensor, latent_shape_q, latent_shape_k, input_layout):
    """8x8-window token order (all frames if h and w are multiples of 8, else frames 1.. with the
    remainder rows/columns appended per frame).  Only ``latent_shape_q`` is used, as in the reference."""
    _check_layout(input_layout)
    _check_gpu16(tensor, "tensor")
    x = _aligned(tensor)
    grid = _check_grid(latent_shape_q, _dims(x, input_layout)[2])
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _run_rearrange([x], [out], None, input_layout, grid, 0, 0)
    return out


def inv_rearrange_with_remaining(tensor, latent_shape_q, latent_shape_k, input_layout):
    """Back from the 8x8-window order to T-H-W order (rf_v2.py:199-289)."""
    _check_layout(input_layout)
    _check_gpu16(tensor, "tensor")
    x = _aligned(tensor)
    grid = _check_grid(latent_shape_q, _dims(x, input_layout)[2])
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _run_rearrange([x], [out], None, input_layout, grid, 0, 1)
    return out


# ------------------------------------------------------------------------------------------------
# rf_v2.py:292-337 and rf_v3.py:100-118
# ------------------------------------------------------------------------------------------------
def _rearrange_qkv(query, key, value, text_len, latent_shape_q, input_layout, want_pool):
    _check_layout(input_layout)
    for name, t in (("query", query), ("key", key), ("value", value)):
        _check_gpu16(t, name)
    if not (query.shape == key.shape == value.shape and query.dtype == key.dtype == value.dtype):
        raise ParametersInvalid("RainFusion needs query, key and value of one shape and dtype "
                                "(self-attention over the latent grid).")
    q, k, v = _aligned(query), _aligned(key), _aligned(value)
    if not _same_strides((q, k, v)):
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    b, n, s = _dims(q, input_layout)
    grid = _check_grid(latent_shape_q, s - text_len)
    outs = [torch.empty(q.shape, dtype=q.dtype, device=q.device) for _ in range(3)]
    pool = None
    if want_pool:
        nb = (s - text_len + BLOCK - 1) // BLOCK + (text_len + BLOCK - 1) // BLOCK
        shape = (3 * b, n, nb, q.shape[-1]) if input_layout == "BNSD" else (3 * b, nb, n, q.shape[-1])
        pool = torch.empty(shape, dtype=q.dtype, device=q.device)
    _run_rearrange([q, k, v], outs, pool, input_layout, grid, text_len, 0)
    return outs[0], outs[1], outs[2], pool


def do_tensor_rearrange_pooling(query, key, value, text_len, pool_size, latent_shape_q, latent_shape_k,
                                input_layout):
    """Returns the permuted q, k, v ([image in window order | text]) and the pooled tensor
    [3B, ...] (image blocks, then text blocks), all in ``input_layout``."""
    if pool_size != BLOCK:
        raise ParametersInvalid(f"pool_size only supports {BLOCK}, but got {pool_size}.")
    return _rearrange_qkv(query, key, value, text_len, latent_shape_q, input_layout, True)


def do_tensor_rearrange_only(q, k, v, txt_len, latent_shape_q, latent_shape_k, input_layout):
    """Permutation without pooling, used when the block mask is cached (rf_v3.py:100-118)."""
    return _rearrange_qkv(q, k, v, txt_len, latent_shape_q, input_layout, False)[:3]


def do_tensor_inv_rearrange(tensor, text_len, latent_shape_q, latent_shape_k, input_layout):
    """Undo the permutation and move the text tokens back to the front."""
    _check_layout(input_layout)
    _check_gpu16(tensor, "tensor")
    x = _aligned(tensor)
    grid = _check_grid(latent_shape_q, _dims(x, input_layout)[2] - text_len)
    out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    _run_rearrange([x], [out], None, input_layout, grid, text_len, 1)
    return out


def _bsa_inv_rearrange(out, tq, hq, wq, input_layout="BSND"):
    """The rf_v3 spelling of the inverse permutation without text tokens (rf_v3.py:22-97): the same token map as
    ``inv_rearrange_with_remaining`` on the grid (tq, hq, wq)."""
    return inv_rearrange_with_remaining(out, (tq, hq, wq), None, input_layout)


def do_tensor_pooling(tensor, text_len):
    """rf_v2.py:340-348 as written there: the tensor is cut at ``text_len`` along dim 1, both parts are pooled by
    ``avgpool`` with its default layout (blocks of 128 along dim 2) and joined along dim 1, first part first."""
    parts = [t for t in (tensor[:, :text_len], tensor[:, text_len:]) if t.shape[1] > 0]
    pooled = [avgpool(t, pool_size=BLOCK) for t in parts]
    return pooled[0] if len(pooled) == 1 else torch.concat(pooled, dim=1)


# ------------------------------------------------------------------------------------------------
# rf_v2.py:76-134
# ------------------------------------------------------------------------------------------------
def get_mask_index(mask):
    """Per row: ascending indices of the True entries, padded with -1; int64 [B, N, S, S]."""
    if mask.dim() != 4 or not mask.is_cuda:
        raise ParametersInvalid("mask must be a 4-D GPU tensor [B, N, S, S].")
    b, n, qb, kb = mask.shape
    m8 = mask.to(torch.int8).contiguous()
    idx = torch.empty((b, n, qb, kb), dtype=torch.int32, device=mask.device)
    cnt = torch.empty((b, n, qb), dtype=torch.int32, device=mask.device)
    with _native.on_device(mask.device):
        rc = _native.lib().mindiesd_mask_to_index(m8.data_ptr(), b * n, qb, kb, idx.data_ptr(), cnt.data_ptr(), kb,
                                                  _native.stream_ptr(mask.device))
    _native.check(rc, "mindiesd_mask_to_index")
    return idx.to(torch.int64)


def keep_len_of(cols, sparsity):
    """Number of key blocks kept per row before forced blocks (rf_v2.py:112, same float expression)."""
    return math.ceil(cols * (1 - sparsity))


def _block_mask(qkv_pool, txt_len, sparsity, scale, pool_size, latent_shape_q, input_layout, protect_first_frame,
                keep_diagonal, want_mask, want_lists, want_ref_lists):
    _check_layout(input_layout)
    _check_gpu16(qkv_pool, "qkv_pool")
    if qkv_pool.shape[0] % 3 != 0:
        raise ParametersInvalid("qkv_pool must stack the pooled query, key and value along dim 0.")
    pool = _aligned(qkv_pool)
    b = pool.shape[0] // 3
    _, n, nb = _dims(pool, input_layout)
    keep_len = keep_len_of(nb, sparsity)
    if not 1 <= keep_len <= nb:
        raise ParametersInvalid(f"sparsity must be in [0, 1), but got {sparsity}.")
    txt_blocks = (txt_len + pool_size - 1) // pool_size
    ff_blocks = 0
    if protect_first_frame:
        ff_blocks = min(nb, (int(latent_shape_q[1]) * int(latent_shape_q[2]) + pool_size - 1) // pool_size)
    dev = pool.device
    mask = torch.empty((b, n, nb, nb), dtype=torch.int8, device=dev) if want_mask else None
    idx = torch.empty((b, n, nb, nb), dtype=torch.int32, device=dev) if want_lists else None
    cnt = torch.empty((b, n, nb), dtype=torch.int32, device=dev) if want_lists else None
    sel = torch.empty((nb, n, nb), dtype=torch.int64, device=dev) if want_ref_lists else None
    sel_num = torch.empty((nb, n), dtype=torch.int64, device=dev) if want_ref_lists else None
    qp, kp = pool[:b], pool[b:2 * b]
    p = lambda t: t.data_ptr() if t is not None else None
    with _native.on_device(dev):
        rc = _native.lib().mindiesd_rf_block_mask(
            qp.data_ptr(), kp.data_ptr(), _native.DTYPE_CODE[pool.dtype], b, n, nb, pool.shape[-1],
            *_pool_strides(qp, input_layout), float(scale), keep_len, txt_blocks, ff_blocks, int(bool(keep_diagonal)),
            p(mask), p(idx), p(cnt), nb, p(sel), p(sel_num), _native.stream_ptr(dev))
    _native.check(rc, "mindiesd_rf_block_mask")
    return mask, idx, cnt, sel, sel_num


def get_blockwise_mask(qkv_pool, txt_len, sparsity, scale, pool_size, latent_shape_q, latent_shape_k, input_layout,
                       return_binary=False, protect_first_frame=True, keep_diagonal=False):
    """Block mask from pooled q/k: ``softmax(q_pool . k_pool * scale) >= k-th largest`` per row with
    ``k = ceil(cols * (1 - sparsity))`` (ties keep extra blocks), text and first-frame rows/columns
    forced.  Returns int8 [B, N, qb, kb] if ``return_binary`` else the reference's
    ``(select_idx [qb, N, kb] int64 padded with -1, select_num_idx [qb, N])`` of batch 0.
    ``keep_diagonal`` (not in the reference) also forces the diagonal blocks."""
    if pool_size != BLOCK:
        raise ParametersInvalid(f"pool_size only supports {BLOCK}, but got {pool_size}.")
    mask, _, _, sel, sel_num = _block_mask(qkv_pool, txt_len, sparsity, scale, pool_size, latent_shape_q, input_layout,
                                           protect_first_frame, keep_diagonal, return_binary, False, not return_binary)
    if return_binary:
        return mask
    return sel, sel_num


# ------------------------------------------------------------------------------------------------
# block-sparse attention kernels (rf_v2.py:351-381, rf_v3.py:122-190)
# ------------------------------------------------------------------------------------------------
_token_order_cache = {}            # key -> (table, event or None once the fill is known to have finished)
_token_order_lock = threading.Lock()


def _build_token_order(t, h, w, txt_len, dev):
    s = t * h * w + txt_len
    tok = torch.empty((s,), dtype=torch.int32, device=dev)
    with _native.on_device(dev):
        rc = _native.lib().mindiesd_rf_token_order(tok.data_ptr(), s, t, h, w, txt_len, _native.stream_ptr(dev))
    _native.check(rc, "mindiesd_rf_token_order")
    return tok


def token_order(latent_shape, txt_len, device):
    """int32 [t*h*w + txt_len]: row of the original [text | image] sequence that holds the token at position i
    of RainFusion's [image in 8x8-window order | text] sequence (the index map of rearrange_with_remaining,
    rf_v2.py:137-196, 297-312).  Built once per (grid, text length, device) by a small kernel on the current
    stream and kept; the host never waits for it.  A later call on another stream is ordered after the fill by an
    event.  Under HIP graph capture a table whose fill is not yet known to be over is not reused: the call builds
    its own inside the graph (a kernel node like any other), so a first call for a grid can be captured."""
    t, h, w = (int(v) for v in latent_shape)
    txt_len = int(txt_len)
    if t <= 0 or h < 8 or w < 8:
        raise ParametersInvalid(f"latent_shape_q must be (t, h, w) with h >= 8 and w >= 8, but got {latent_shape}.")
    dev = torch.device(device)
    key = (t, h, w, txt_len, dev.type, dev.index if dev.index is not None else torch.cuda.current_device())
    capturing = torch.cuda.is_current_stream_capturing()
    with _token_order_lock:
        entry = _token_order_cache.get(key)
    if entry is not None:
        tok, done = entry
        if done is None:
            return tok
        if not capturing:
            if done.query():
                with _token_order_lock:
                    _token_order_cache[key] = (tok, None)
            else:
                torch.cuda.current_stream(dev).wait_event(done)
            return tok
    tok = _build_token_order(t, h, w, txt_len, dev)
    if not capturing:
        done = torch.cuda.Event()
        done.record(torch.cuda.current_stream(dev))
        with _token_order_lock:
            if len(_token_order_cache) >= 16:
                _token_order_cache.clear()
            _token_order_cache[key] = (tok, done)
    return tok


def block_sparse_attention_lists(query, key, value, blk_idx, blk_cnt, scale, layout="BNSD", return_lse=False,
                                 order=None):
    """Attention of every 128-row query block over the key blocks listed for it.
    ``blk_idx`` int32 [B, N, qb, stride] ascending block ids, ``blk_cnt`` int32 [B, N, qb].
    A query block with an empty list yields zeros.
    ``order`` (int32 [S], from :func:`token_order`): query position i - the position the lists and the rows of
    key and value refer to - is row ``order[i]`` of query and of the output (self-attention only): with key and
    value permuted and query left as it is, this is attention on the permuted query and the inverse permutation
    of the result in one pass."""
    for name, t in (("query", query), ("key", key), ("value", value)):
        _check_gpu16(t, name)
    q, k, v = _aligned(query), _aligned(key), _aligned(value)
    b, n, sq = _dims(q, layout)
    _, nkv, skv = _dims(k, layout)
    if k.shape != v.shape or k.shape[0] != b or n % nkv != 0 or k.dtype != q.dtype or v.dtype != q.dtype:
        raise ParametersInvalid("Inconsistent query/key/value shapes or dtypes.")
    qb, kb = (sq + BLOCK - 1) // BLOCK, (skv + BLOCK - 1) // BLOCK
    if (blk_idx.dtype != torch.int32 or blk_cnt.dtype != torch.int32 or tuple(blk_cnt.shape) != (b, n, qb)
            or tuple(blk_idx.shape[:3]) != (b, n, qb) or not blk_idx.is_contiguous() or not blk_cnt.is_contiguous()):
        raise ParametersInvalid(f"block lists must be contiguous int32 [B,N,{qb},stride] / [B,N,{qb}].")
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    lse = torch.empty((b, n, sq), dtype=torch.float32, device=q.device) if return_lse else None
    if order is not None:
        if (order.dtype != torch.int32 or order.dim() != 1 or order.shape[0] != sq or skv != sq or not order.is_contiguous()
                or order.device != q.device):
            raise ParametersInvalid(f"order must be a contiguous int32 [{sq}] tensor on the inputs' device "
                                    "(self-attention only).")
        with _native.on_device(q.device):
            rc = _native.lib().mindiesd_block_sparse_attention_gather_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr() if return_lse else None,
                _native.DTYPE_CODE[q.dtype], b, n, nkv, sq, q.shape[-1],
                *_strides_bns(q, layout), *_strides_bns(k, layout), *_strides_bns(v, layout), *_strides_bns(out, layout),
                float(scale), blk_idx.data_ptr(), blk_cnt.data_ptr(), blk_idx.shape[3], order.data_ptr(),
                _native.stream_ptr(q.device))
        _native.check(rc, "mindiesd_block_sparse_attention_gather_fwd")
        return (out, lse) if return_lse else out
    with _native.on_device(q.device):
        rc = _native.lib().mindiesd_block_sparse_attention_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr() if return_lse else None,
            _native.DTYPE_CODE[q.dtype], b, n, nkv, sq, skv, q.shape[-1],
            *_strides_bns(q, layout), *_strides_bns(k, layout), *_strides_bns(v, layout), *_strides_bns(out, layout),
            float(scale), blk_idx.data_ptr(), blk_cnt.data_ptr(), blk_idx.shape[3], None,
            _native.stream_ptr(q.device))
    _native.check(rc, "mindiesd_block_sparse_attention_fwd")
    return (out, lse) if return_lse else out


def block_sparse_attention_mask(query, key, value, block_sparse_mask, scale, layout="BNSD", return_lse=False,
                                order=None):
    """Attention of every 128-row query block over the key blocks its mask row selects
    (``block_sparse_mask`` int8/bool [B, N, qb, kb], non-zero = attend; an all-zero row yields zeros).
    Runs the kernel over paired query blocks (query blocks with similar mask rows share their K/V
    tiles); masks too large for the pairing kernels go through the block lists.  ``order`` as in
    :func:`block_sparse_attention_lists`."""
    for name, t in (("query", query), ("key", key), ("value", value)):
        _check_gpu16(t, name)
    q, k, v = _aligned(query), _aligned(key), _aligned(value)
    b, n, sq = _dims(q, layout)
    _, nkv, skv = _dims(k, layout)
    if k.shape != v.shape or k.shape[0] != b or n % nkv != 0 or k.dtype != q.dtype or v.dtype != q.dtype:
        raise ParametersInvalid("Inconsistent query/key/value shapes or dtypes.")
    qb, kb = (sq + BLOCK - 1) // BLOCK, (skv + BLOCK - 1) // BLOCK
    if block_sparse_mask.dim() != 4 or tuple(block_sparse_mask.shape) != (b, n, qb, kb) or not block_sparse_mask.is_cuda:
        raise ParametersInvalid(f"block_sparse_mask must be a GPU tensor [B, N, {qb}, {kb}], but got "
                                f"{tuple(block_sparse_mask.shape)}.")
    if order is not None and (order.dtype != torch.int32 or order.dim() != 1 or order.shape[0] != sq or skv != sq
                              or not order.is_contiguous() or order.device != q.device):
        raise ParametersInvalid(f"order must be a contiguous int32 [{sq}] tensor on the inputs' device "
                                "(self-attention only).")
    m8 = block_sparse_mask if block_sparse_mask.dtype == torch.int8 else block_sparse_mask.to(torch.int8)
    m8 = m8.contiguous()
    lib = _native.lib()
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    lse = torch.empty((b, n, sq), dtype=torch.float32, device=q.device) if return_lse else None
    ws_bytes = lib.mindiesd_block_sparse_attention_paired_workspace_size(b, n, sq, skv)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    with _native.on_device(q.device):
        rc = lib.mindiesd_block_sparse_attention_paired_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr() if return_lse else None,
            _native.DTYPE_CODE[q.dtype], b, n, nkv, sq, skv, q.shape[-1],
            *_strides_bns(q, layout), *_strides_bns(k, layout), *_strides_bns(v, layout), *_strides_bns(out, layout),
            float(scale), m8.data_ptr(), order.data_ptr() if order is not None else None, ws.data_ptr(), ws_bytes,
            _native.stream_ptr(q.device))
    if rc == 2 and q.shape[-1] == HEAD_DIM:  # mask too large for the pairing kernels
        idx, cnt = mask_to_lists(m8)
        return block_sparse_attention_lists(q, k, v, idx, cnt, scale, layout, return_lse, order)
    _native.check(rc, "mindiesd_block_sparse_attention_paired_fwd")
    return (out, lse) if return_lse else out


def block_sparse_attention_varlen(query, key, value, block_sparse_mask, scale, seq_lens_q, seq_lens_kv, layout,
                                  return_lse=False):
    """Block-sparse attention with one length per batch entry (``actual_seq_lengths`` / ``actual_seq_lengths_kv`` of
    the reference op, csrc/plugin/block_sparse_attention.cpp:42-66).
    ``layout`` 'BNSD': query [B, N, S, D], sequence b uses its first ``seq_lens_q[b]`` query and ``seq_lens_kv[b]``
    key tokens; the other output rows are zero.  'TND': packed [T, N, D] tensors, sequence b follows sequence b - 1.
    ``block_sparse_mask`` [B, N, ceil(max q len / 128), ceil(max kv len / 128)].  Returns the output like ``query``
    (and the log-sum-exp [B, N, S] / [T, N] with ``return_lse``)."""
    for name, t in (("query", query), ("key", key), ("value", value)):
        if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype not in _native.DTYPE_CODE or t.shape[-1] != HEAD_DIM:
            raise ParametersInvalid(f"{name} must be a bf16/fp16 GPU tensor with head_dim {HEAD_DIM}.")
    q, k, v = _aligned(query), _aligned(key), _aligned(value)
    lq, lk = [int(x) for x in seq_lens_q], [int(x) for x in seq_lens_kv]
    b = len(lq)
    if b == 0 or len(lk) != b or min(lq) <= 0 or min(lk) <= 0:
        raise ParametersInvalid("sequence lengths must be positive, one per batch entry for queries and for keys.")
    if layout == "TND":
        if q.dim() != 3 or k.dim() != 3 or sum(lq) != q.shape[0] or sum(lk) != k.shape[0] or k.shape != v.shape:
            raise ParametersInvalid("TND layout: [T, N, D] tensors whose token counts equal the sums of the lengths.")
        n, nkv = q.shape[1], k.shape[1]
        q_str, k_str, v_str = (0, q.stride(1), q.stride(0)), (0, k.stride(1), k.stride(0)), (0, v.stride(1), v.stride(0))
        starts_q = [sum(lq[:i]) for i in range(b)]
        starts_k = [sum(lk[:i]) for i in range(b)]
        out = torch.empty_like(q)
        lse = torch.empty((q.shape[0], n), dtype=torch.float32, device=q.device) if return_lse else None
    elif layout == "BNSD":
        if q.dim() != 4 or k.dim() != 4 or q.shape[0] != b or k.shape[0] != b or k.shape != v.shape:
            raise ParametersInvalid("BNSD layout: 4-D tensors with one length per batch entry.")
        if max(lq) > q.shape[2] or max(lk) > k.shape[2]:
            raise ParametersInvalid("a sequence length exceeds the tensor.")
        n, nkv = q.shape[1], k.shape[1]
        q_str, k_str, v_str = _strides_bns(q, layout), _strides_bns(k, layout), _strides_bns(v, layout)
        starts_q = starts_k = [0] * b
        out = torch.zeros_like(q)
        lse = torch.zeros((b, n, q.shape[2]), dtype=torch.float32, device=q.device) if return_lse else None
    else:
        raise ParametersInvalid(f"layout must be 'BNSD' or 'TND', but got {layout}.")
    if n % nkv != 0 or k.dtype != q.dtype or v.dtype != q.dtype:
        raise ParametersInvalid("Inconsistent query/key/value head counts or dtypes.")
    sq, skv = max(lq), max(lk)
    qb, kb = (sq + BLOCK - 1) // BLOCK, (skv + BLOCK - 1) // BLOCK
    # a mask sized for the padded tensors (more block rows / columns than the longest sequence needs) is cut down
    if (block_sparse_mask.dim() != 4 or tuple(block_sparse_mask.shape[:2]) != (b, n) or block_sparse_mask.shape[2] < qb
            or block_sparse_mask.shape[3] < kb):
        raise ParametersInvalid(f"block_sparse_mask must be [B, N, >= {qb}, >= {kb}] = [{b}, {n}, ...], "
                                f"but got {tuple(block_sparse_mask.shape)}.")
    idx, cnt = mask_to_lists(block_sparse_mask[:, :, :qb, :kb])
    meta = torch.tensor([[starts_q[i], lq[i], starts_k[i], lk[i]] for i in range(b)], dtype=torch.int32).to(q.device)
    o_str = (0, out.stride(1), out.stride(0)) if layout == "TND" else _strides_bns(out, layout)
    with _native.on_device(q.device):
        rc = _native.lib().mindiesd_block_sparse_attention_general_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr() if return_lse else None,
            _native.DTYPE_CODE[q.dtype], b, n, nkv, sq, skv, q.shape[-1], *q_str, *k_str, *v_str, *o_str, float(scale),
            idx.data_ptr(), cnt.data_ptr(), idx.shape[3], meta.data_ptr(), int(layout == "TND"), 0,
            _native.stream_ptr(q.device))
    _native.check(rc, "mindiesd_block_sparse_attention_general_fwd")
    return (out, lse) if return_lse else out


def mask_to_lists(block_sparse_mask):
    """int8/bool [B, N, qb, kb] (non-zero = attend) -> (blk_idx int32 [B,N,qb,kb], blk_cnt int32 [B,N,qb])."""
    if block_sparse_mask.dim() != 4 or not block_sparse_mask.is_cuda:
        raise ParametersInvalid("block_sparse_mask must be a 4-D GPU tensor [B, N, q_blocks, kv_blocks].")
    m8 = block_sparse_mask.to(torch.int8).contiguous()
    b, n, qb, kb = m8.shape
    idx = torch.empty((b, n, qb, kb), dtype=torch.int32, device=m8.device)
    cnt = torch.empty((b, n, qb), dtype=torch.int32, device=m8.device)
    with _native.on_device(m8.device):
        rc = _native.lib().mindiesd_mask_to_index(m8.data_ptr(), b * n, qb, kb, idx.data_ptr(), cnt.data_ptr(), kb,
                                                  _native.stream_ptr(m8.device))
    _native.check(rc, "mindiesd_mask_to_index")
    return idx, cnt


def rain_fusion_attention(query, key, value, scale=None, head_num=None, input_layout="TND", select_idx=None,
                          select_num_idx=None, blockshape=None, actual_seq_lengths=None, actual_seq_lengths_kv=None,
                          inner_precise=0):
    """Index-list driven sparse attention (rf_v2.py:351-381).  ``select_idx`` [qb, N, kb] int64 (-1
    padded), ``select_num_idx`` [qb, N]; layouts 'TND' (one sequence) or 'BNSD'."""
    from .. import _custom_ops as ops
    out, _ = ops.rain_fusion_attention(
        query, key, value, select_idx, select_num_idx, blockshape if blockshape is not None else [BLOCK, BLOCK],
        attn_mask=None, actual_seq_qlen=actual_seq_lengths, actual_seq_kvlen=actual_seq_lengths_kv, block_table=None,
        q_input_layout=input_layout, kv_input_layout=input_layout, head_num=head_num if head_num is not None else 1,
        mask_type=0, scale=scale if scale is not None else query.shape[-1] ** -0.5, inner_precise=inner_precise,
        block_size=0)
    return out


def rain_fusion_attention_v3(query, key, value, block_sparse_mask, scale=None, head_num=None, num_key_value_heads=None,
                             input_layout="BNSD", actual_seq_lengths=None, actual_seq_lengths_kv=None, sparse_size=128,
                             inner_precise=4):
    """Mask driven sparse attention (rf_v3.py:122-190): int8 mask [B, N, qb, kb], 1 = attend.  BSND
    inputs run in place (the reference copies them to BNSD first)."""
    if scale is None:
        scale = query.shape[-1] ** -0.5
    _check_layout(input_layout)
    if sparse_size != BLOCK:
        raise ParametersInvalid(f"sparse_size only supports {BLOCK}, but got {sparse_size}.")
    return block_sparse_attention_mask(query, key, value, block_sparse_mask, scale, input_layout)


def bsa_sparse_attention_v3(q, k, v, latent_shape_q, latent_shape_k=None, txt_len=0, pool_size=128, sparsity=0.5,
                            input_layout="BSND", head_num=None, num_key_value_heads=None, scale=None, inner_precise=4,
                            cached_mask=None, protect_first_frame=True, keep_diagonal=False):
    """End-to-end rf_v3 sparse attention (rf_v3.py:193-295): permute(+pool) -> mask -> block-sparse
    attention -> inverse permute.  Returns ``(out, mask)``; pass the mask back as ``cached_mask`` on
    later diffusion steps to skip pooling and mask generation."""
    if latent_shape_k is None:
        latent_shape_k = latent_shape_q
    if scale is None:
        scale = float(q.shape[-1]) ** -0.5
    if pool_size != BLOCK:
        raise ParametersInvalid(f"pool_size only supports {BLOCK}, but got {pool_size}.")
    # Only key and value are copied into the window order (their tiles must be contiguous for the kernel's
    # LDS-DMA); the query is pooled through the order and read by the attention kernel through the same table,
    # which also stores the output rows straight to their original places.
    _check_layout(input_layout)
    for name, t in (("query", q), ("key", k), ("value", v)):
        _check_gpu16(t, name)
    if not (q.shape == k.shape == v.shape and q.dtype == k.dtype == v.dtype):
        raise ParametersInvalid("RainFusion needs query, key and value of one shape and dtype "
                                "(self-attention over the latent grid).")
    q, k, v = _aligned(q), _aligned(k), _aligned(v)
    if not _same_strides((q, k, v)):
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    b, n, s = _dims(q, input_layout)
    grid = _check_grid(latent_shape_q, s - txt_len)
    k_ = torch.empty(k.shape, dtype=k.dtype, device=k.device)
    v_ = torch.empty(v.shape, dtype=v.dtype, device=v.device)
    if cached_mask is None:
        nb = (s - txt_len + BLOCK - 1) // BLOCK + (txt_len + BLOCK - 1) // BLOCK
        shape = (3 * b, n, nb, q.shape[-1]) if input_layout == "BNSD" else (3 * b, nb, n, q.shape[-1])
        pool = torch.empty(shape, dtype=q.dtype, device=q.device)
        _run_rearrange([q, k, v], [None, k_, v_], pool, input_layout, grid, txt_len, 0)
        new_mask, _, _, _, _ = _block_mask(pool, txt_len, sparsity, scale, pool_size, latent_shape_q, input_layout,
                                           protect_first_frame, keep_diagonal, True, False, False)
    else:
        _run_rearrange([k, v], [k_, v_], None, input_layout, grid, txt_len, 0)
        new_mask = cached_mask
    out = block_sparse_attention_mask(q, k_, v_, new_mask, scale, input_layout,
                                      order=token_order(grid, txt_len, q.device))
    return out, new_mask
