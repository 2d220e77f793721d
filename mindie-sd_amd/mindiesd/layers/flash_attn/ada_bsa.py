"""Host side of adaptive block-sparse attention: the mask estimate (sparse_block_estimate) and the
attention over the estimated mask (ada_block_sparse_attention).

Stands where the reference's torch ops call its in-tree AscendC kernels
(csrc/plugin/sparse_block_estimate.cpp:27-85, csrc/plugin/ada_block_sparse_attention.cpp:27-57).
The estimate is two launches of this library: the block scores (anti-diagonal strided products, their row
softmax and the sums over 16 x 16 blocks in one kernel that reads q and k in place) and the per-row selection
of key blocks.
"""
import torch

from ... import _native
from ...utils.exception import ParametersInvalid
from .hip_flash_attn import HEAD_DIM, _strides_bns
from .rainfusion import BLOCK, _aligned, _check_gpu16, _dims, block_sparse_attention_mask, mask_to_lists

STRIDE = 8
# Scratch of the score kernel is allocated up to this size; with more heads than fit, the library goes
# through them in groups.
_WORKSPACE_BYTES = 1 << 30


def sparse_block_estimate(query, key, input_layout="BNSD", stride=8, sparse_size=128, scale_value=1.0, threshold=1.0,
                          causal=False, keep_sink=True, keep_recent=True, row_sparse=1.0, return_scores=False):
    """-> (sparse_mask int8 [B, N, nb, align32(nb)], sparse_count_table int32 [B, N, nb]), nb = ceil(S / 128).
    ``scale_value`` multiplies the strided products (the caller passes softmax_scale / stride)."""
    for name, t in (("query", query), ("key", key)):
        _check_gpu16(t, name)
    if input_layout not in ("BNSD", "BSND"):
        raise RuntimeError(f"input_layout only supports 'BNSD' and 'BSND', got {input_layout}")
    if stride != STRIDE or sparse_size != BLOCK:
        raise RuntimeError(f"sparse_block_estimate supports stride {STRIDE} and sparse_size {BLOCK} only, "
                           f"got {stride} and {sparse_size}")
    q, k = _aligned(query), _aligned(key)
    b, n, s = _dims(q, input_layout)
    kb, nkv, ks = _dims(k, input_layout)
    if kb != b or ks != s or nkv == 0 or n % nkv != 0 or k.dtype != q.dtype:
        raise RuntimeError("sparse_block_estimate: query and key must have the same batch, length, head_dim and dtype")
    nb = (s + BLOCK - 1) // BLOCK
    pitch = (nb + 31) // 32 * 32
    lib = _native.lib()
    scores = torch.empty((b * n, nb, nb), dtype=torch.float32, device=q.device)
    one_head = lib.mindiesd_sbe_scores_workspace_size(1, s)
    ws_bytes = min(one_head * b * n, max(one_head, _WORKSPACE_BYTES // one_head * one_head))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
    mask = torch.empty((b, n, nb, pitch), dtype=torch.int8, device=q.device)
    count = torch.empty((b, n, nb), dtype=torch.int32, device=q.device)
    with _native.on_device(q.device):
        stream = _native.stream_ptr(q.device)
        rc = lib.mindiesd_sbe_scores(q.data_ptr(), k.data_ptr(), scores.data_ptr(), _native.DTYPE_CODE[q.dtype], b, n,
                                     nkv, s, HEAD_DIM, *_strides_bns(q, input_layout), *_strides_bns(k, input_layout),
                                     float(scale_value), int(bool(causal)), ws.data_ptr(), ws_bytes, stream)
        _native.check(rc, "mindiesd_sbe_scores")
        rc = lib.mindiesd_sbe_select(scores.data_ptr(), mask.data_ptr(), count.data_ptr(), b * n, nb, pitch,
                                     float(threshold), float(row_sparse), int(bool(keep_sink)), int(bool(keep_recent)),
                                     int(bool(causal)), stream)
        _native.check(rc, "mindiesd_sbe_select")
    if return_scores:
        return mask, count, scores.view(b, n, nb, nb)
    return mask, count


def ada_block_sparse_attention(query, key, value, sparse_mask, sparse_count_table=None, input_layout="BNSD",
                               sparse_size=128, scale_value=1.0, causal=False):
    """Attention of every 128-row query block over the key blocks its mask row selects; with ``causal`` keys
    after the query are masked inside the blocks as well.  The count table is implied by the mask and only
    checked for its shape."""
    if input_layout not in ("BNSD", "BSND"):
        raise RuntimeError(f"input_layout only supports 'BNSD' and 'BSND', got {input_layout}")
    if sparse_size != BLOCK:
        raise RuntimeError(f"ada_block_sparse_attention supports sparse_size {BLOCK} only, got {sparse_size}")
    for name, t in (("query", query), ("key", key), ("value", value)):
        _check_gpu16(t, name)
    q, k, v = _aligned(query), _aligned(key), _aligned(value)
    b, n, s = _dims(q, input_layout)
    _, nkv, skv = _dims(k, input_layout)
    if k.shape != v.shape or skv != s or n % nkv != 0 or k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError("ada_block_sparse_attention: query, key and value must share batch, length and dtype")
    nb = (s + BLOCK - 1) // BLOCK
    if sparse_mask.dim() != 4 or tuple(sparse_mask.shape[:3]) != (b, n, nb) or sparse_mask.shape[3] < nb:
        raise RuntimeError(f"sparse_mask must be [B, N, {nb}, >= {nb}], got {tuple(sparse_mask.shape)}")
    if sparse_count_table is not None and tuple(sparse_count_table.shape) != (b, n, nb):
        raise RuntimeError(f"sparse_count_table must be [B, N, {nb}], got {tuple(sparse_count_table.shape)}")
    if not causal and q.shape[-1] == HEAD_DIM:
        # without the in-block causal test this is plain block-sparse attention: the kernel over paired
        # query blocks, driven by the mask itself
        return block_sparse_attention_mask(q, k, v, sparse_mask[..., :nb], scale_value, input_layout)
    idx, cnt = mask_to_lists(sparse_mask)
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    with _native.on_device(q.device):
        rc = _native.lib().mindiesd_ada_block_sparse_attention_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), _native.DTYPE_CODE[q.dtype], b, n, nkv, s,
            q.shape[-1], *_strides_bns(q, input_layout), *_strides_bns(k, input_layout), *_strides_bns(v, input_layout),
            *_strides_bns(out, input_layout), float(scale_value), idx.data_ptr(), cnt.data_ptr(), idx.shape[3],
            int(bool(causal)), _native.stream_ptr(q.device))
    _native.check(rc, "mindiesd_ada_block_sparse_attention_fwd")
    return out
