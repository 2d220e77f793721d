"""Oracle: dense and block-sparse attention on the CPU (test infrastructure only).

Follows the reference's unfused fallback ``attention_math``
(mindiesd/layers/flash_attn/attention_func.py:32-55) operation for operation, including
its rounding points, and the numpy reference of the block-sparse kernel
(tests/plugin/test_block_sparse_attention.py:32-65).
"""
import math

import numpy as np
import torch


def attention_math(query, key, value, attn_mask=None, scale=None, head_first=False):
    """softmax(scale * Q K^T + bias) V with the reference's rounding points.

    attention_func.py:32-55: BSND inputs are viewed as BNSD (:33-36); ``q * scale`` is
    rounded to the input dtype (:40); ``q @ k^T`` is produced in the input dtype (:41) and
    only then widened to fp32 (:42); a boolean mask (True = keep) becomes a -inf bias
    (:43-49); softmax runs in fp32 (:50); the probabilities are rounded to the input dtype
    (:51) before ``@ v`` (:52); the layout is restored (:53-54).
    """
    if scale is None:
        scale = query.shape[-1] ** -0.5
    if not head_first:
        query, key, value = (t.transpose(1, 2) for t in (query, key, value))
    dtype = query.dtype
    sq, skv = query.size(-2), key.size(-2)
    q = query * scale
    attn = (q @ key.transpose(-2, -1)).to(torch.float32)
    if attn_mask is not None:
        if attn_mask.dim() not in (2, 4) or attn_mask.size(-2) != sq or attn_mask.size(-1) != skv:
            raise ValueError("attn_mask must be [Sq,Skv] or [B,N,Sq,Skv]")
        bias = torch.zeros(attn_mask.shape, dtype=dtype)
        bias.masked_fill_(attn_mask.logical_not(), float("-inf"))
        attn = attn + bias
    attn = torch.softmax(attn, dim=-1).to(dtype)
    out = attn @ value
    if not head_first:
        out = out.transpose(1, 2)
    return out


def attention_math_rows(query, key, value, scale=None, row_chunk=4096, q_rows=None):
    """``attention_math`` for one BNSD problem evaluated ``row_chunk`` query rows at a time.

    Every query row is independent in attention_func.py:40-52, so chunking the rows changes
    nothing but the size of the S x S temporaries.  ``q_rows`` (slice) restricts the
    evaluation to a sample of rows (used for head/row-subset checks at sizes where a whole
    S x S matrix per head does not fit in host memory).
    """
    b, n, sq, d = query.shape
    rows = range(sq)[q_rows] if q_rows is not None else range(sq)
    start, stop, step = rows.start, rows.stop, rows.step
    assert step == 1
    outs = []
    for r0 in range(start, stop, row_chunk):
        r1 = min(r0 + row_chunk, stop)
        outs.append(attention_math(query[:, :, r0:r1], key, value, None, scale, head_first=True))
    return torch.cat(outs, dim=2)


def causal_keep_mask(sq, skv):
    """Boolean [sq, skv] mask of the vendor kernel's ``sparse_mode=3`` ("rightDownCausal", the mode
    attention_forward_varlen.py:134-136 selects): the lower triangle aligned to the bottom-right
    corner, i.e. key j is visible to query i iff j <= i + (skv - sq)."""
    i = torch.arange(sq)[:, None]
    j = torch.arange(skv)[None, :]
    return j <= i + (skv - sq)


def attention_varlen(q, k, v, cu_seqlens_q, cu_seqlens_k, scale=None, causal=False):
    """Packed [T, N, D] sequences (attention_forward_varlen.py:59-149): every sequence is an independent
    ``attention_math`` problem over its own slice of q and k / v (grouped-query heads repeated), with the
    bottom-right aligned causal mask when ``causal``.  Rows without a visible key (possible when a
    sequence has fewer keys than queries) are defined as zeros here."""
    t, n, d = q.shape
    nkv = k.shape[1]
    out = torch.zeros(q.shape, dtype=q.dtype)
    for i in range(len(cu_seqlens_q) - 1):
        q0, q1, k0, k1 = int(cu_seqlens_q[i]), int(cu_seqlens_q[i + 1]), int(cu_seqlens_k[i]), int(cu_seqlens_k[i + 1])
        if q1 == q0 or k1 == k0:
            continue
        qs = q[q0:q1].transpose(0, 1)[None]
        ks = k[k0:k1].transpose(0, 1).repeat_interleave(n // nkv, dim=0)[None]
        vs = v[k0:k1].transpose(0, 1).repeat_interleave(n // nkv, dim=0)[None]
        mask = causal_keep_mask(q1 - q0, k1 - k0) if causal else None
        o = attention_math(qs, ks, vs, mask, scale, head_first=True)
        if mask is not None:
            o = torch.where(mask.any(dim=-1)[None, None, :, None], o, torch.zeros((), dtype=o.dtype))
        out[q0:q1] = o[0].transpose(0, 1)
    return out


def attention_fp64(query, key, value, scale, keep=None):
    """Brute-force fp64 softmax(scale QK^T)V for one [S,D] problem; pins attention_math."""
    q = query.double().numpy()
    k = key.double().numpy()
    v = value.double().numpy()
    s = (q @ k.T) * scale
    if keep is not None:
        s = np.where(keep, s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    return torch.from_numpy(p @ v)


def block_sparse_attention(query, key, value, block_mask, scale=None, block=128):
    """Block-sparse attention, BNSD, fp32 arithmetic on the CPU.

    Semantics of the reference's numpy model (tests/plugin/test_block_sparse_attention.py:32-65):
    for query block ``i`` the softmax runs only over the keys of the key blocks ``j`` with
    ``block_mask[b, n, i, j] != 0``; a query block that selects nothing yields zeros (:54-55);
    grouped-query heads map ``n -> n // (Nq // Nkv)`` (:36, :52).  The reference divides by
    ``sqrt(D)``; ``scale`` generalises that (the op takes ``scale_value``,
    csrc/plugin/register_ops.cpp:62-67).
    """
    b, nq, sq, d = query.shape
    nkv, skv = key.shape[1], key.shape[2]
    gqa = nq // nkv
    if scale is None:
        scale = 1.0 / math.sqrt(d)
    qb = math.ceil(sq / block)
    kb = math.ceil(skv / block)
    qf, kf, vf = query.float().numpy(), key.float().numpy(), value.float().numpy()
    m = np.asarray(block_mask)
    out = np.zeros((b, nq, sq, d), dtype=np.float32)
    for bi in range(b):
        for ni in range(nq):
            for i in range(qb):
                keep = np.repeat(m[bi, ni, i, :kb] != 0, block)[:skv]
                r0, r1 = i * block, min((i + 1) * block, sq)
                if not keep.any():
                    continue
                kk, vv = kf[bi, ni // gqa][keep], vf[bi, ni // gqa][keep]
                p = (qf[bi, ni, r0:r1] @ kk.T) * np.float32(scale)
                p = p - p.max(axis=-1, keepdims=True)
                e = np.exp(p)
                out[bi, ni, r0:r1] = (e / (e.sum(axis=-1, keepdims=True) + 1e-12)) @ vv
    return torch.from_numpy(out)


def ref_compare(golden, actual, err):
    """Tolerance rule of the reference's kernel tests (tests/plugin/test_block_sparse_attention.py:68-74):
    |diff| <= err * max(1, |golden|) everywhere and mean relative error <= err / 2."""
    golden = golden.to(torch.float32)
    nmax = torch.clamp(golden.abs(), min=1)
    abs_error = (actual.to(torch.float32) - golden).abs()
    eb = torch.mean(abs_error / nmax)
    ok = bool((abs_error <= err * nmax).all()) and bool(eb <= err / 2)
    return eb.item(), ok, abs_error.max().item()


def data_compare(actual, golden, rel=1e-3, pass_frac=0.999, max_rel=0.1):
    """Tolerance rule of the reference's fused-vs-fallback tests
    (tests/utils/utils/precision_compare.py:89-158): element-wise relative difference
    (absolute for |golden| < 1) within ``rel`` for at least ``pass_frac`` of the elements and
    never above ``max_rel``."""
    a, g = actual.float().flatten(), golden.float().flatten()
    diff = (a - g).abs() / torch.clamp(g.abs(), min=1.0)
    return bool((diff <= rel).float().mean() >= pass_frac) and bool(diff.max() < max_rel)


def cosine(a, b):
    a, b = a.double().flatten(), b.double().flatten()
    return float((a @ b) / (a.norm() * b.norm() + 1e-300))
