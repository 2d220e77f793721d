"""Pins of the adaptive block-sparse oracle (oracle/ada_bsa.py): the chunked running-softmax statement of
the block scores against a direct global softmax, the selection rule on hand-worked rows, and the sparse
attention against dense / causal attention in the cases where they coincide."""
import numpy as np
import pytest
import torch

from oracle import ada_bsa as oab
from oracle.attention import attention_math


def _global_block_scores(q, k, stride=8, reduce=16):
    d = q.shape[1]
    sq = -(-q.shape[0] // stride) * stride
    qp = np.zeros((sq, d), np.float64)
    qp[:q.shape[0]] = q
    kp = np.zeros((sq, d), np.float64)
    kp[:k.shape[0]] = k
    sr = sq // stride
    p = np.zeros((sr, sr))
    for i in range(sr):
        for s in range(stride):
            p[i] += qp[stride * i + stride - 1 - s] @ kp[s::stride].T
    p /= np.sqrt(d) * stride
    prob = np.exp(p - p.max(-1, keepdims=True))
    prob /= prob.sum(-1, keepdims=True)
    nb = -(-sr // reduce)
    pad = np.zeros((nb * reduce, nb * reduce))
    pad[:sr, :sr] = prob
    return pad.reshape(nb, reduce, nb, reduce).sum((1, 3))


@pytest.mark.parametrize("s", [128, 1000, 1027, 9000])
def test_block_scores_equal_global_softmax(s):
    rng = np.random.RandomState(s)
    q = rng.standard_normal((s, 8)).astype(np.float32) * 2
    k = rng.standard_normal((s, 8)).astype(np.float32) * 2
    got = oab.block_scores(q, k)
    want = _global_block_scores(q, k)
    assert got.shape == want.shape == (-(-s // 128), -(-s // 128))
    assert np.abs(got - want).max() < 2e-5
    # every strided row carries probability mass 1
    assert abs(got.sum() - (-(-s // 8))) < 1e-2


def test_select_blocks_hand_worked_rows():
    row = [0.5, 0.2, 0.1, 0.15, 0.05]
    # ranking without the last block: 0.5 0.2 0.15 0.1 0; total 0.95; 0.6 * 0.95 = 0.57 is passed by the second
    assert oab.select_blocks(row, 0.6, 1.0).tolist() == [True, True, False, False, True]
    # without the forced blocks the guard alone decides (0.2): the sink passes it anyway, the last block does not
    assert oab.select_blocks(row, 0.6, 1.0, keep_sink=False, keep_recent=False).tolist() == [True, True, False, False, False]
    # threshold 1: everything that carries mass (and, through the zeroed last entry, the rest)
    assert oab.select_blocks(row, 1.0, 1.0).all()
    # cap: at most int(0.4 * 5) = 2 ranked blocks although 0.99 asks for 4
    assert oab.select_blocks(row, 0.99, 0.4).tolist() == [True, True, False, False, True]
    # a sink that would not make it on its own is forced
    assert oab.select_blocks([0.01, 0.6, 0.3, 0.09], 0.5, 1.0).tolist() == [True, True, False, True]
    # ties: stable order, both tied blocks pass the guard
    assert oab.select_blocks([0.3, 0.3, 0.3, 0.1], 0.4, 1.0).tolist() == [True, True, True, True]


def test_select_blocks_kernel_hand_worked_rows():
    """The kernel's own selection rules (sparse_block_estimate.h:947-1078) on rows worked out by hand."""
    row = [0.5, 0.2, 0.1, 0.15, 0.05]
    # sink and last block left out: ranked 0.2 0.15 0.1 0 0, total 0.45, 0.6 * 0.45 = 0.27 reached by the second
    # (0.15), which is the guard; the guard itself passes (it is lowered by 1e-5), 0.1 does not
    assert oab.select_blocks_kernel(row, 0.6, 1.0).tolist() == [True, True, False, True, True]
    # both switches off, not causal: the last block is still left out and forced, the first is ranked:
    # 0.5 0.2 0.15 0.1 0, total 0.95, 0.57 reached by the second (0.2)
    assert oab.select_blocks_kernel(row, 0.6, 1.0, False, False).tolist() == [True, True, False, False, True]
    # threshold 1: every column, also those without mass
    assert oab.select_blocks_kernel([0.5, 0.0, 0.0, 0.5], 1.0, 1.0).all()
    # the first block is kept even when nothing forces or ranks it
    assert oab.select_blocks_kernel([0.0, 0.6, 0.3, 0.1], 0.5, 1.0, keep_sink=False).tolist() == [True, True, False, True]
    # the cap applies from 10 columns on: 12 columns, 0.99 asks for nearly all, 0.25 * 12 = 3 ranked ones stay
    row12 = [0.0, 0.3, 0.25, 0.2, 0.1, 0.05, 0.04, 0.03, 0.02, 0.005, 0.005, 0.0]
    assert oab.select_blocks_kernel(row12, 0.99, 0.25).tolist() == [True, True, True, True] + [False] * 7 + [True]
    assert oab.select_blocks_kernel(row12[:9], 0.99, 0.25).sum() > 5            # 9 columns: no cap
    # causal: rows of at most two columns keep them all; the diagonal is ranked unless keep_recent leaves it out
    assert oab.select_blocks_kernel([0.1, 0.9], 0.1, 0.1, causal=True).all()
    diag_heavy = [0.05, 0.1, 0.05, 0.8]
    assert oab.select_blocks_kernel(diag_heavy, 0.5, 1.0, keep_recent=False, causal=True).tolist() == [True, False, False, True]
    assert oab.select_blocks_kernel(diag_heavy, 0.5, 1.0, keep_recent=True, causal=True).tolist() == [True, True, False, True]


def test_kernel_rules_equal_the_numpy_statement_when_the_sink_carries_no_mass():
    """With a first block of score 0 (nothing to leave out of the total), no cap and the default switches the two
    statements of the selection are the same rule; rows whose guard has a near tie below it are left out, because
    the kernel's lowered guard lets such a tie pass."""
    rng = np.random.RandomState(0)
    compared = 0
    for _ in range(200):
        n = int(rng.randint(3, 40))
        row = rng.rand(n).astype(np.float32) ** 3
        row[0] = 0
        thr = float(rng.uniform(0.2, 0.95))
        a, b = oab.select_blocks(row, thr, 1.0), oab.select_blocks_kernel(row, thr, 1.0)
        if (a != b).any():
            ranked = np.sort(row[:-1])
            assert np.diff(ranked).min() < 2e-5, (row, thr)
            continue
        compared += 1
    assert compared > 190


def test_sparse_estimate_invariants():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 2, 1100, 32, generator=g)
    k = torch.randn(1, 1, 1100, 32, generator=g)
    m = oab.sparse_estimate(q, k, threshold=0.7, force_sparse=0.5)
    assert m.shape == (1, 2, 9, 9) and m[..., 0].all() and m[..., -1].all()
    assert (m.sum(-1) <= int(0.5 * 9) + 2).all()
    assert oab.sparse_estimate(q, k, threshold=1.0, force_sparse=1.0).all()
    # monotone in the threshold
    lo, hi = oab.sparse_estimate(q, k, threshold=0.3), oab.sparse_estimate(q, k, threshold=0.9)
    assert (hi | ~lo).all()


def test_ada_attention_reduces_to_dense_and_causal():
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(1, 2, 300, 16, generator=g) for _ in range(3))
    full = np.ones((1, 2, 3, 3), dtype=bool)
    dense = attention_math(q, k, v, None, 16 ** -0.5, head_first=True)
    assert torch.allclose(oab.ada_block_sparse_attention(q, k, v, full, blocksize=128), dense, atol=1e-5)
    tril = np.tril(np.ones((3, 3), dtype=bool))[None, None].repeat(2, axis=1)
    causal = attention_math(q, k, v, torch.ones(300, 300).tril().bool(), 16 ** -0.5, head_first=True)
    assert torch.allclose(oab.ada_block_sparse_attention(q, k, v, tril, causal=True, blocksize=128), causal, atol=1e-5)
    # an empty row gives zeros; grouped-query heads share keys
    m = full.copy()
    m[0, 1, 2] = False
    out = oab.ada_block_sparse_attention(q, k[:, :1], v[:, :1], m, blocksize=128)
    assert not out[0, 1, 256:].any() and out[0, 0].abs().sum() > 0


# ---- causal estimate (restated from the branches of the reference's numpy statement that its test does not run) ----
def _qk(s, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(1, 1, s, 128, generator=g), torch.randn(1, 1, s, 128, generator=g)


def test_causal_estimate_stays_in_the_lower_triangle_and_keeps_first_rows():
    q, k = _qk(2100, 1)
    m = oab.sparse_estimate(q, k, threshold=0.6, force_sparse=0.5, causal=True)[0, 0]
    assert not np.triu(m, 1).any()
    assert m[0, 0] and m[1, :2].all()
    assert m[:, 0].all() and np.diag(m).all()          # sink and diagonal forced
    m2 = oab.sparse_estimate(q, k, threshold=0.6, force_sparse=0.5, causal=True, keep_recent=False)[0, 0]
    assert not np.diag(m2)[2:].any()                   # the diagonal block is ranked as zero and not forced


def test_causal_estimate_with_threshold_one_is_the_lower_triangle():
    q, k = _qk(1500, 2)
    m = oab.sparse_estimate(q, k, threshold=1.0, force_sparse=1.0, causal=True)[0, 0]
    assert np.array_equal(m, np.tril(np.ones_like(m)))


def test_causal_scores_ignore_keys_after_the_query_step():
    """A step of 1024 query tokens sees the keys up to its own end: later keys change nothing in its rows."""
    q, k = _qk(2048 + 512, 3)
    a = oab.block_scores(q[0, 0].numpy(), k[0, 0].numpy(), causal=True)
    k2 = k.clone()
    k2[0, 0, 1024:] += 3.0
    b = oab.block_scores(q[0, 0].numpy(), k2[0, 0].numpy(), causal=True)
    assert np.array_equal(a[:8], b[:8]) and not np.allclose(a[8:16], b[8:16])
    assert not a[:8, 8:].any() and not a[8:16, 16:].any()
    np.testing.assert_allclose(a[:8].sum(1), 16.0, rtol=1e-4)      # 16 strided rows of unit mass per block row


def test_causal_scores_of_a_single_step_equal_the_plain_ones():
    q, k = _qk(1024, 4)
    a = oab.block_scores(q[0, 0].numpy(), k[0, 0].numpy(), causal=True)
    b = oab.block_scores(q[0, 0].numpy(), k[0, 0].numpy(), causal=False)
    assert np.array_equal(a, b)


def test_causal_estimate_kernel_rules_invariants():
    q, k = _qk(2100, 5)
    m = oab.sparse_estimate(q, k, threshold=0.6, force_sparse=0.5, causal=True, rules="kernel")[0, 0]
    assert not np.triu(m, 1).any() and m[:, 0].all() and np.diag(m).all()
    full = oab.sparse_estimate(q, k, threshold=1.0, force_sparse=1.0, causal=True, rules="kernel")[0, 0]
    assert np.array_equal(full, np.tril(np.ones_like(full)))
    n = oab.sparse_estimate(q, k, threshold=0.7, force_sparse=1.0, rules="kernel")[0, 0]
    assert n[:, 0].all() and n[:, -1].all()


def test_ada_attention_causal_rules_agree_when_rows_end_with_their_diagonal_block():
    """The reference's numpy statement (triangle on the last selected block) and its kernel (triangle only when that
    block is the diagonal one) are the same function on masks whose rows end with the diagonal block, and differ
    where a row ends below it."""
    import numpy as np
    import torch
    from oracle import ada_bsa as oab
    g = torch.Generator().manual_seed(0)
    s, nb = 300, 3
    q, k, v = (torch.randn((1, 1, s, 128), generator=g).to(torch.bfloat16) for _ in range(3))
    m = np.tril(np.ones((nb, nb), dtype=bool))[None, None]
    a = oab.ada_block_sparse_attention(q, k, v, m, causal=True, rules="numpy")
    b = oab.ada_block_sparse_attention(q, k, v, m, causal=True, rules="kernel")
    assert torch.equal(a, b)
    m2 = m.copy()
    m2[0, 0, 2, 2] = False          # the last row ends with block 1, below its diagonal block
    a = oab.ada_block_sparse_attention(q, k, v, m2, causal=True, rules="numpy")
    b = oab.ada_block_sparse_attention(q, k, v, m2, causal=True, rules="kernel")
    assert torch.equal(a[:, :, :256], b[:, :, :256]) and not torch.equal(a[:, :, 256:], b[:, :, 256:])
    # kernel rule, row without its diagonal block: plain attention over the selected blocks
    sel = torch.cat([k[0, 0, :256]]), torch.cat([v[0, 0, :256]])
    p = torch.softmax(q[0, 0, 256:].float() @ sel[0].float().T / 128 ** 0.5, dim=-1) @ sel[1].float()
    assert torch.allclose(b[0, 0, 256:], p, atol=1e-5)
