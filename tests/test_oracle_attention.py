"""Pins the dense / block-sparse attention oracle against independent computations
(fp64 brute force, torch's own SDPA, special cases), not against its own formula."""
import math

import numpy as np
import pytest
import torch

from oracle.attention import (attention_fp64, attention_math, attention_math_rows, block_sparse_attention, cosine,
                              data_compare, ref_compare)


def _qkv(shape, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(shape, generator=g).to(dtype) for _ in range(3))


def test_fp32_matches_fp64_brute_force():
    q, k, v = _qkv((2, 3, 37, 16), 0)
    out = attention_math(q, k, v, None, 0.25, head_first=True)
    for b in range(2):
        for n in range(3):
            ref = attention_fp64(q[b, n], k[b, n], v[b, n], 0.25)
            assert (out[b, n].double() - ref).abs().max() < 1e-5


def test_matches_torch_sdpa_fp32():
    q, k, v = _qkv((1, 4, 65, 32), 1)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, scale=0.3)
    assert (attention_math(q, k, v, None, 0.3, head_first=True) - ref).abs().max() < 1e-5


def test_layouts_agree_and_default_scale():
    q, k, v = _qkv((2, 50, 3, 8), 2)
    a = attention_math(q, k, v, None, None, head_first=False)
    b = attention_math(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, 8 ** -0.5, head_first=True)
    assert a.shape == q.shape and torch.allclose(a, b.transpose(1, 2), atol=1e-6)


def test_mask_true_means_keep_2d_and_4d():
    q, k, v = _qkv((1, 2, 9, 8), 3)
    mask = torch.rand(9, 9) > 0.4
    mask[:, 0] = True
    out = attention_math(q, k, v, mask, 0.5, head_first=True)
    out4 = attention_math(q, k, v, mask.expand(1, 2, 9, 9), 0.5, head_first=True)
    for n in range(2):
        ref = attention_fp64(q[0, n], k[0, n], v[0, n], 0.5, keep=mask.numpy())
        assert (out[0, n].double() - ref).abs().max() < 1e-5
    assert torch.allclose(out, out4)
    with pytest.raises(ValueError):
        attention_math(q, k, v, torch.ones(1, 9, 9, dtype=torch.bool), 0.5, head_first=True)


def test_uniform_keys_give_mean_of_values():
    """Closed form: equal scores -> softmax is uniform -> output is the mean of V."""
    q, _, v = _qkv((1, 1, 5, 8), 4)
    k = torch.zeros(1, 1, 7, 8)
    v = torch.randn(1, 1, 7, 8)
    out = attention_math(q, k, v, None, 1.0, head_first=True)
    assert torch.allclose(out, v.mean(dim=2, keepdim=True).expand_as(out), atol=1e-6)


def test_bf16_rounding_points_are_the_references():
    """q*scale, QK^T and P are rounded to bf16 (attention_func.py:40-41, :51): a step-by-step
    evaluation with explicit roundings must agree bit for bit; an all-fp32 evaluation must not."""
    q, k, v = _qkv((1, 1, 33, 16), 5, torch.bfloat16)
    out = attention_math(q, k, v, None, 0.25, head_first=True)
    qs = (q.float() * 0.25).to(torch.bfloat16)
    s = (qs.float() @ k.float().transpose(-1, -2)).to(torch.bfloat16).float()
    p = torch.softmax(s, dim=-1).to(torch.bfloat16)
    manual = (p.float() @ v.float()).to(torch.bfloat16)
    assert (out.float() - manual.float()).abs().max() <= 2 ** -7  # at most one bf16 ulp (accumulation order)
    assert cosine(out, attention_fp64(q[0, 0], k[0, 0], v[0, 0], 0.25)) > 0.9999


def test_row_chunking_changes_nothing():
    q, k, v = _qkv((1, 2, 300, 16), 6, torch.bfloat16)
    full = attention_math(q, k, v, None, 0.25, head_first=True)
    assert torch.equal(attention_math_rows(q, k, v, 0.25, row_chunk=64), full)
    assert torch.equal(attention_math_rows(q, k, v, 0.25, row_chunk=64, q_rows=slice(100, 250)), full[:, :, 100:250])


# ---- block-sparse reference -------------------------------------------------------------------
def test_block_sparse_all_ones_is_dense():
    q, k, v = _qkv((1, 2, 300, 16), 7)
    nb = math.ceil(300 / 128)
    out = block_sparse_attention(q, k, v, torch.ones(1, 2, nb, nb, dtype=torch.int8), scale=0.25)
    assert (out - attention_math(q, k, v, None, 0.25, head_first=True)).abs().max() < 1e-5


def test_block_sparse_empty_row_is_zero_and_default_scale():
    q, k, v = _qkv((1, 1, 256, 16), 8)
    m = torch.tensor([[[[1, 0], [0, 0]]]], dtype=torch.int8)
    out = block_sparse_attention(q, k, v, m)
    assert (out[0, 0, 128:] == 0).all()
    ref = attention_fp64(q[0, 0, :128], k[0, 0, :128], v[0, 0, :128], 1 / math.sqrt(16))
    assert (out[0, 0, :128].double() - ref).abs().max() < 1e-5


def test_block_sparse_gathers_selected_key_blocks_brute_force():
    q, k, v = _qkv((1, 2, 300, 8), 9)   # 3 blocks, the last one holds 44 tokens
    m = torch.tensor([[[1, 0, 1], [0, 1, 0], [1, 1, 1]], [[0, 0, 1], [1, 1, 0], [0, 1, 1]]], dtype=torch.int8)[None]
    out = block_sparse_attention(q, k, v, m, scale=0.4)
    for n in range(2):
        for i in range(3):
            keys = np.concatenate([np.arange(j * 128, min((j + 1) * 128, 300)) for j in range(3) if m[0, n, i, j]])
            rows = slice(i * 128, min((i + 1) * 128, 300))
            ref = attention_fp64(q[0, n, rows], k[0, n, keys], v[0, n, keys], 0.4)
            assert (out[0, n, rows].double() - ref).abs().max() < 1e-5


def test_block_sparse_gqa_head_mapping():
    q, _, _ = _qkv((1, 4, 130, 8), 10)
    _, k, v = _qkv((1, 2, 130, 8), 11)
    m = torch.ones(1, 4, 2, 2, dtype=torch.int8)
    out = block_sparse_attention(q, k, v, m, scale=0.3)
    ref = attention_math(q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1), None, 0.3, head_first=True)
    assert (out - ref).abs().max() < 1e-5


def test_tolerance_rules():
    g = torch.tensor([0.5, 2.0, -4.0])
    assert ref_compare(g, g + torch.tensor([0.005, 0.02, 0.02]), 2 ** -6)[1]
    assert not ref_compare(g, g + torch.tensor([0.02, 0.0, 0.0]), 2 ** -6)[1]
    assert data_compare(g + 1e-4, g) and not data_compare(g + 0.2, g)


# ---- causal mask (bottom-right aligned) and packed variable-length sequences ---------------------------------
def test_causal_keep_mask_closed_forms():
    from oracle.attention import causal_keep_mask
    # square: the ordinary lower triangle
    assert torch.equal(causal_keep_mask(5, 5), torch.ones(5, 5).tril().bool())
    # more keys than queries: the last query sees everything, the first sees skv - sq + 1 keys
    m = causal_keep_mask(3, 7)
    assert torch.equal(m, torch.ones(3, 7).tril(diagonal=4).bool()) and m[-1].all() and int(m[0].sum()) == 5
    # fewer keys than queries: the first sq - skv queries see nothing, the last sees all keys
    m = causal_keep_mask(6, 2)
    assert not m[:4].any() and m[-1].all() and torch.equal(m, torch.ones(6, 2).tril(diagonal=-4).bool())


def test_attention_varlen_matches_sdpa_per_sequence():
    from oracle.attention import attention_varlen, causal_keep_mask
    g = torch.Generator().manual_seed(3)
    lens_q, lens_k = [5, 0, 17, 9], [5, 4, 30, 3]
    cu_q = [0] + list(torch.tensor(lens_q).cumsum(0))
    cu_k = [0] + list(torch.tensor(lens_k).cumsum(0))
    q = torch.randn(sum(lens_q), 4, 16, generator=g)
    k = torch.randn(sum(lens_k), 2, 16, generator=g)
    v = torch.randn(sum(lens_k), 2, 16, generator=g)
    for causal in (False, True):
        got = attention_varlen(q, k, v, cu_q, cu_k, causal=causal)
        for i, (lq, lk) in enumerate(zip(lens_q, lens_k)):
            if lq == 0:
                continue
            qs = q[cu_q[i]:cu_q[i + 1]].transpose(0, 1)
            ks = k[cu_k[i]:cu_k[i + 1]].transpose(0, 1).repeat_interleave(2, dim=0)
            vs = v[cu_k[i]:cu_k[i + 1]].transpose(0, 1).repeat_interleave(2, dim=0)
            keep = causal_keep_mask(lq, lk) if causal else torch.ones(lq, lk, dtype=torch.bool)
            want = torch.nn.functional.scaled_dot_product_attention(qs, ks, vs, attn_mask=keep)
            want = torch.where(keep.any(-1)[None, :, None], want, torch.zeros(()))  # SDPA gives NaN for empty rows
            assert torch.allclose(got[cu_q[i]:cu_q[i + 1]].transpose(0, 1), want, atol=2e-6, rtol=1e-5)
    # square causal == torch's own is_causal
    qs = torch.randn(1, 2, 9, 16, generator=g)
    want = torch.nn.functional.scaled_dot_product_attention(qs, qs, qs, is_causal=True)
    got = attention_varlen(qs[0].transpose(0, 1), qs[0].transpose(0, 1), qs[0].transpose(0, 1), [0, 9], [0, 9], causal=True)
    assert torch.allclose(got.transpose(0, 1), want[0], atol=2e-6, rtol=1e-5)
