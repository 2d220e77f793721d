"""The MI355X attention kernel behind ``attention_forward``.

Takes the place of the reference's vendor-op wrappers (prompt_flash_attn.py:22-130,
fused_attn_score.py:22-131, ascend_laser_attention.py:38-119).  Those normalise the layout with
transposes / reshapes before calling a layout-specific NPU kernel; the HIP kernel takes explicit
batch / head / token strides, so BNSD, BSND and BSH inputs all run in place without a copy.
"""
import torch

from .attention_operate import AttentionOperateBase, register_op_mi355x
from .common import AttentionParam
from ... import _native
from ...utils.exception import ParametersInvalid

HEAD_DIM = 128        # the head_dim of the tuned kernels (sparse, FP8 and the DiT shapes)
MAX_HEAD_DIM = 256    # dense attention takes every multiple of 8 up to this


def _strides_bns(t, layout):
    """(batch, head, token) element strides of a 4-D tensor in ``layout`` with a contiguous last dim."""
    s0, s1, s2, s3 = t.stride()
    if s3 != 1:
        raise ParametersInvalid("The last dimension of query/key/value must be contiguous.")
    return (s0, s1, s2) if layout == "BNSD" else (s0, s2, s1)


def _check_qkv(query, key, value):
    for name, t in (("query", query), ("key", key), ("value", value)):
        if not t.is_cuda:
            raise ParametersInvalid(f"The fused attention kernel needs GPU tensors, but {name} is on {t.device}.")
    if query.dtype not in _native.DTYPE_CODE or key.dtype != query.dtype or value.dtype != query.dtype:
        raise ParametersInvalid(f"The fused attention kernel supports bf16/fp16 with equal q/k/v dtypes, "
                                f"but got {query.dtype}, {key.dtype}, {value.dtype}.")
    d = query.shape[-1]
    if d % 8 != 0 or not 0 < d <= MAX_HEAD_DIM or key.shape[-1] != d or value.shape[-1] != d:
        raise ParametersInvalid(f"The fused attention kernel supports equal q/k/v head_dim, a multiple of 8 up to "
                                f"{MAX_HEAD_DIM}, but got {d}, {key.shape[-1]}, {value.shape[-1]}.")


def _aligned(t):
    st = t.stride()
    if st[-1] != 1 or t.data_ptr() % 16:
        return t.contiguous()
    for s in st[:-1]:
        if s % 8:
            return t.contiguous()
    return t


def flash_attention(query, key, value, scale, layout="BNSD", return_lse=False, attn_mask=None, causal=False):
    """softmax(scale * Q K^T) V on the GPU.  ``layout`` is 'BNSD' or 'BSND'; the output has the
    input's layout and dtype.  Grouped-query attention is supported (N % N_kv == 0).

    ``attn_mask``: [Sq|1, Skv] or [B|1, N|1, Sq|1, Skv] (query dimension 1: one row for all queries),
    non-zero / True = attend (the reference's fused
    wrappers hand the vendor kernel ``~mask.to(torch.bool)``, prompt_flash_attn.py:46-47); ``causal``
    keeps key j for query i iff j <= i + (Skv - Sq).  Rows without any visible key give zeros."""
    _check_qkv(query, key, value)
    if layout == "BNSD":
        b, n, sq, d = query.shape
        nkv, skv = key.shape[1], key.shape[2]
    else:
        b, sq, n, d = query.shape
        skv, nkv = key.shape[1], key.shape[2]
    if key.shape != value.shape or key.shape[0] != b or n % nkv != 0:
        raise ParametersInvalid("Inconsistent query/key/value shapes.")
    query, key, value = _aligned(query), _aligned(key), _aligned(value)
    out = torch.empty(query.shape, dtype=query.dtype, device=query.device)
    lse = torch.empty((b, n, sq), dtype=torch.float32, device=query.device) if return_lse else None
    strides = (*_strides_bns(query, layout), *_strides_bns(key, layout), *_strides_bns(value, layout),
               *_strides_bns(out, layout))
    with _native.on_device(query.device):
        if attn_mask is None and not causal:
            rc = _native.lib().mindiesd_flash_attention_fwd(
                query.data_ptr(), key.data_ptr(), value.data_ptr(), out.data_ptr(),
                lse.data_ptr() if lse is not None else None, _native.DTYPE_CODE[query.dtype],
                b, n, nkv, sq, skv, d, *strides, float(scale), _native.stream_ptr(query.device))
            _native.check(rc, "mindiesd_flash_attention_fwd")
        else:
            mask, m_sb, m_sn, m_sq = None, 0, 0, 0
            if attn_mask is not None:
                mask = attn_mask
                if mask.dim() == 2:
                    mask = mask[None, None]
                if (mask.dim() != 4 or mask.shape[-1] != skv or mask.shape[-2] not in (1, sq)
                        or mask.shape[0] not in (1, b) or mask.shape[1] not in (1, n)):
                    raise ParametersInvalid(f"attn_mask must be [Sq|1, Skv] or [B|1, N|1, Sq|1, Skv] = "
                                            f"[{b}|1, {n}|1, {sq}|1, {skv}], but got {tuple(attn_mask.shape)}.")
                mask = mask.to(device=query.device, dtype=torch.bool)
                if mask.stride(-1) != 1:
                    mask = mask.contiguous()
                m_sb = mask.stride(0) if mask.shape[0] > 1 else 0
                m_sn = mask.stride(1) if mask.shape[1] > 1 else 0
                # 0 for a mask row shared by all queries (a key-padding mask, given as such or expanded over the queries)
                m_sq = 0 if mask.shape[2] == 1 and sq > 1 else (mask.stride(2) if sq > 1 else skv)
            rc = _native.lib().mindiesd_flash_attention_general_fwd(
                query.data_ptr(), key.data_ptr(), value.data_ptr(), out.data_ptr(),
                lse.data_ptr() if lse is not None else None, _native.DTYPE_CODE[query.dtype],
                b, n, nkv, sq, skv, d, *strides, float(scale), None, int(bool(causal)),
                mask.data_ptr() if mask is not None else None, m_sb, m_sn, m_sq, _native.stream_ptr(query.device))
            _native.check(rc, "mindiesd_flash_attention_general_fwd")
    return (out, lse) if return_lse else out


def _varlen_meta(cu_q, cu_k, total_q, total_k, device, max_q=None, max_k=None):
    """Cumulative lengths -> (int32 [B, 4] device table {first query token, query count, first key token, key
    count}, longest query count, longest key count, B).  Host lists / CPU tensors are validated and give exact
    bounds; device tensors are turned into the table on the device without a host synchronisation - the bounds
    are then the token totals (workgroups past a sequence's end return at once) unless the caller names the longest
    sequences (``max_q`` / ``max_k``), and the entries are clamped to the tensors instead of validated: a malformed
    device table cannot be rejected without reading it back, so it yields clamped sequences, never an access outside
    the tensors."""
    on_device = isinstance(cu_q, torch.Tensor) and cu_q.is_cuda and isinstance(cu_k, torch.Tensor) and cu_k.is_cuda
    if on_device:
        if cu_q.dim() != 1 or cu_k.dim() != 1 or cu_q.shape[0] != cu_k.shape[0] or cu_q.shape[0] < 2:
            raise ParametersInvalid("cu_seqlens_q and cu_seqlens_k must be 1-D with batch_size + 1 entries each.")
        cq = cu_q.to(device=device, dtype=torch.int32).contiguous()   # no copies when they already are int32
        ck = cu_k.to(device=device, dtype=torch.int32).contiguous()
        bound_q = total_q if max_q is None else max(min(int(max_q), total_q), 1)
        bound_k = total_k if max_k is None else max(min(int(max_k), total_k), 0)
        meta = torch.empty((cq.shape[0] - 1, 4), dtype=torch.int32, device=device)
        with _native.on_device(device):
            rc = _native.lib().mindiesd_varlen_meta(cq.data_ptr(), ck.data_ptr(), cq.shape[0] - 1, total_q, total_k,
                                                    bound_q, bound_k, meta.data_ptr(), _native.stream_ptr(device))
        _native.check(rc, "mindiesd_varlen_meta")
        return meta, bound_q, max(bound_k, 1), cq.shape[0] - 1
    def lengths(cu, name):
        vals = [int(x) for x in (cu.detach().cpu().tolist() if isinstance(cu, torch.Tensor) else cu)]
        if len(vals) < 2 or vals[0] != 0 or any(b < a for a, b in zip(vals, vals[1:])):
            raise ParametersInvalid(f"{name} must start at 0, be non-decreasing and hold batch_size + 1 entries, "
                                    f"but got {vals}.")
        return [b - a for a, b in zip(vals, vals[1:])]
    seqlens_q, seqlens_k = lengths(cu_q, "cu_seqlens_q"), lengths(cu_k, "cu_seqlens_k")
    if len(seqlens_q) != len(seqlens_k) or len(seqlens_q) == 0:
        raise ParametersInvalid("cu_seqlens_q and cu_seqlens_k must describe the same, non-zero number of sequences.")
    if sum(seqlens_q) != total_q or sum(seqlens_k) != total_k:
        raise ParametersInvalid("The cumulative sequence lengths do not match the token dimensions of q / k.")
    meta, oq, ok = [], 0, 0
    for lq, lk in zip(seqlens_q, seqlens_k):
        meta += [oq, lq, ok, lk]
        oq += lq
        ok += lk
    meta_t = torch.tensor(meta, dtype=torch.int32).view(-1, 4).to(device, non_blocking=True)
    return meta_t, max(seqlens_q), max(max(seqlens_k), 1), len(seqlens_q)


def flash_attention_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, scale, causal=False, max_seqlen_q=None,
                           max_seqlen_k=None):
    """Packed sequences: q [Tq, N, D], k / v [Tk, Nkv, D]; ``cu_seqlens_q`` / ``cu_seqlens_k``: cumulative sequence
    lengths (batch + 1 entries; lists, CPU tensors or device tensors - the latter are used without a host
    synchronisation).  Returns [Tq, N, D].  Host tables are validated (ParametersInvalid).  Device tables are
    clamped to the tensors instead; query rows that no sequence of such a table covers come back as zeros, and
    ``max_seqlen_q`` / ``max_seqlen_k`` (optional, device tables only) bound the launch to the longest sequence
    instead of the token totals."""
    _check_qkv(q, k, v)
    if q.dim() != 3 or k.shape != v.shape or k.dim() != 3 or q.shape[1] % k.shape[1] != 0:
        raise ParametersInvalid("Inconsistent query/key/value shapes.")
    q, k, v = _aligned(q), _aligned(k), _aligned(v)
    unchecked = isinstance(cu_seqlens_q, torch.Tensor) and cu_seqlens_q.is_cuda
    out = (torch.zeros if unchecked else torch.empty)(q.shape, dtype=q.dtype, device=q.device)
    if q.shape[0] == 0:
        return out
    meta_t, max_q, max_k, nseq = _varlen_meta(cu_seqlens_q, cu_seqlens_k, q.shape[0], k.shape[0], q.device,
                                              max_seqlen_q, max_seqlen_k)
    if max_q == 0:
        return out
    tn = lambda t: (0, t.stride(1), t.stride(0))  # (batch, head, token) strides of a [T, N, D] tensor
    if unchecked and max_seqlen_q is None and max_seqlen_k is None:
        # lengths known to the device only: the grid comes from the token totals, the workgroups find their sequence
        with _native.on_device(q.device):
            rc = _native.lib().mindiesd_flash_attention_packed_fwd(
                q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), _native.DTYPE_CODE[q.dtype],
                nseq, q.shape[1], k.shape[1], q.shape[0], k.shape[0], q.shape[2],
                *tn(q)[1:], *tn(k)[1:], *tn(v)[1:], *tn(out)[1:], float(scale), meta_t.data_ptr(), int(bool(causal)),
                _native.stream_ptr(q.device))
        _native.check(rc, "mindiesd_flash_attention_packed_fwd")
        return out
    with _native.on_device(q.device):
        rc = _native.lib().mindiesd_flash_attention_general_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), None, _native.DTYPE_CODE[q.dtype],
            nseq, q.shape[1], k.shape[1], max_q, max_k, q.shape[2],
            *tn(q), *tn(k), *tn(v), *tn(out), float(scale), meta_t.data_ptr(), int(bool(causal)), None, 0, 0, 0,
            _native.stream_ptr(q.device))
    _native.check(rc, "mindiesd_flash_attention_general_fwd")
    return out


@register_op_mi355x("hip_flash_attn", "prompt_flash_attn", "fused_attn_score", "ascend_laser_attention")
class HipFlashAttention(AttentionOperateBase):
    """Registered under its own name and under the reference's three op names, so call sites that
    pass ``op_type='fused_attn_score'`` etc. (attention_forward.py:72-80) keep working."""
    supported_layout = ["BNSD", "BSND", "BSH"]
    supported_dtype = [torch.bfloat16, torch.float16]

    @classmethod
    def is_supported_shape(cls, attn_param: AttentionParam) -> bool:
        return attn_param.head_dim % 8 == 0 and 0 < attn_param.head_dim <= MAX_HEAD_DIM

    @classmethod
    def _run(cls, attn_param, query, key, value, mask, scale):
        if scale is None:
            scale = attn_param.head_dim ** -0.5
        return flash_attention(query, key, value, scale, "BNSD" if attn_param.head_first else "BSND", attn_mask=mask)

    # The kernel is stride-generic, so the three "layouts" of the reference differ only in how the
    # caller's tensors are viewed: nothing is transposed or copied for any of them.
    @classmethod
    def forward_attn_bnsd(cls, attn_param, query, key, value, mask=None, scale=None):
        return cls._run(attn_param, query, key, value, mask, scale)

    @classmethod
    def forward_attn_bsnd(cls, attn_param, query, key, value, mask=None, scale=None):
        return cls._run(attn_param, query, key, value, mask, scale)

    @classmethod
    def forward_attn_bsh(cls, attn_param, query, key, value, mask=None, scale=None):
        return cls._run(attn_param, query, key, value, mask, scale)
