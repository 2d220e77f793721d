"""Host side of adaptive block-sparse attention: the mask estimate (sparse_block_estimate) and the
attention over the estimated mask (ada_block_sparse_attention).

Stands where the reference's torch ops call its in-tree AscendC kernels
(csrc/plugin/sparse_block_estimate.cpp:27-85, csrc/plugin/ada_block_sparse_attention.cpp:27-57).
The estimate is three steps: the anti-diagonal strided score matrix P' (a plain GEMM, handed to the GEMM
library through torch.bmm), its row softmax summed over 16 x 16 blocks, and the per-row selection of key
blocks; the last two are HIP kernels of this library.
"""
import torch

from ... import _native
from ...utils.exception import ParametersInvalid
from .hip_flash_attn import HEAD_DIM, _strides_bns
from .rainfusion import BLOCK, _aligned, _check_gpu16, _dims, mask_to_lists

STRIDE = 8
# Heads are processed in groups whose P' matrices together stay below 2^30 elements (2 GiB in 16 bits).
_PMAT_ELEMS = 1 << 30
# Longest sequence the estimate accepts.  Runs at 32760 and 75600 tokens ended in a GPU memory fault whose
# cause has not been established (the kernels' index arithmetic checks out on paper; sequences up to 3000
# tokens pass their parity tests), so longer sequences are refused until it is.
MAX_ESTIMATE_TOKENS = 3072


def _to_bnsd(t, layout):
    if layout == "BNSD":
        return t
    if layout == "BSND":
        return t.transpose(1, 2)
    raise RuntimeError(f"input_layout only supports 'BNSD' and 'BSND', got {layout}")


def sparse_block_estimate(query, key, input_layout="BNSD", stride=8, sparse_size=128, scale_value=1.0, threshold=1.0,
                          causal=False, keep_sink=True, keep_recent=True, row_sparse=1.0, return_scores=False):
    """-> (sparse_mask int8 [B, N, nb, align32(nb)], sparse_count_table int32 [B, N, nb]), nb = ceil(S / 128).
    ``scale_value`` multiplies the strided products (the caller passes softmax_scale / stride)."""
    for name, t in (("query", query), ("key", key)):
        _check_gpu16(t, name)
    if query.dim() != 4 or key.dim() != 4:
        raise RuntimeError("sparse_block_estimate expects 4-D query and key")
    if stride != STRIDE or sparse_size != BLOCK:
        raise RuntimeError(f"sparse_block_estimate supports stride {STRIDE} and sparse_size {BLOCK} only, "
                           f"got {stride} and {sparse_size}")
    s_tokens = query.shape[2] if input_layout == "BNSD" else query.shape[1]
    if s_tokens > MAX_ESTIMATE_TOKENS:
        raise RuntimeError(f"sparse_block_estimate: sequences longer than {MAX_ESTIMATE_TOKENS} tokens are switched off in "
                           f"this build (got {s_tokens})")
    q, k = _to_bnsd(query, input_layout), _to_bnsd(key, input_layout)
    b, n, s, d = q.shape
    if k.shape[0] != b or k.shape[2] != s or k.shape[3] != d or n % k.shape[1] != 0 or k.dtype != q.dtype:
        raise RuntimeError("sparse_block_estimate: query and key must have the same batch, length, head_dim and dtype")
    if k.shape[1] != n:
        k = k.repeat_interleave(n // k.shape[1], dim=1)
    sp = (s + STRIDE - 1) // STRIDE * STRIDE
    sr = sp // STRIDE
    ldp = (sr + 7) // 8 * 8
    nb = (s + BLOCK - 1) // BLOCK
    pitch = (nb + 31) // 32 * 32
    # Q': the 8 tokens of a group in reverse order, side by side; K': in order; tokens past S are zeros
    qp = torch.zeros((b, n, sp, d), dtype=q.dtype, device=q.device)
    qp[:, :, :s] = q
    qp = qp.view(b * n, sr, STRIDE, d).flip(2).reshape(b * n, sr, STRIDE * d)
    kp = torch.zeros((b * n, ldp, STRIDE * d), dtype=q.dtype, device=q.device)
    kp[:, :sr].view(b * n, sr * STRIDE, d)[:, :s] = k.reshape(b * n, s, d)
    scores = torch.empty((b * n, nb, nb), dtype=torch.float32, device=q.device)
    if sr * ldp > _PMAT_ELEMS:
        raise RuntimeError(f"sparse_block_estimate: sequence length {s} is beyond what this build estimates")
    group = max(1, min(b * n, _PMAT_ELEMS // (sr * ldp)))
    lib = _native.lib()
    with torch.cuda.device(q.device):
        for g0 in range(0, b * n, group):
            g1 = min(b * n, g0 + group)
            pmat = torch.bmm(qp[g0:g1], kp[g0:g1].transpose(1, 2))  # [g, sr, ldp] raw strided products
            rc = lib.mindiesd_sbe_block_scores(pmat.data_ptr(), scores[g0:g1].data_ptr(), _native.DTYPE_CODE[q.dtype],
                                               g1 - g0, sr, ldp, float(scale_value), int(bool(causal)),
                                               max(1, s // STRIDE), _native.stream_ptr(q.device))
            _native.check(rc, "mindiesd_sbe_block_scores")
            del pmat
        mask = torch.empty((b, n, nb, pitch), dtype=torch.int8, device=q.device)
        count = torch.empty((b, n, nb), dtype=torch.int32, device=q.device)
        rc = lib.mindiesd_sbe_select(scores.data_ptr(), mask.data_ptr(), count.data_ptr(), b * n, nb, pitch,
                                     float(threshold), float(row_sparse), int(bool(keep_sink)), int(bool(keep_recent)),
                                     int(bool(causal)), _native.stream_ptr(q.device))
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
    idx, cnt = mask_to_lists(sparse_mask)
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    with torch.cuda.device(q.device):
        rc = _native.lib().mindiesd_ada_block_sparse_attention_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), _native.DTYPE_CODE[q.dtype], b, n, nkv, s,
            q.shape[-1], *_strides_bns(q, input_layout), *_strides_bns(k, input_layout), *_strides_bns(v, input_layout),
            *_strides_bns(out, input_layout), float(scale_value), idx.data_ptr(), cnt.data_ptr(), idx.shape[3],
            int(bool(causal)), _native.stream_ptr(q.device))
    _native.check(rc, "mindiesd_ada_block_sparse_attention_fwd")
    return out
