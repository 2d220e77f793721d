"""GPU parity of the block-sparse attention over paired query blocks (mindiesd_block_sparse_attention_paired_fwd)
against the CPU oracle (the reference's numpy model of its block-sparse kernel,
tests/plugin/test_block_sparse_attention.py:32-65) within the reference's kernel rule |err| <= 2^-6 * max(1, |golden|),
and against the one-pass list kernel on the same mask."""
import numpy as np
import pytest
import torch

from oracle import attention as oa

pytestmark = pytest.mark.gpu


def _rand(shape, seed, dtype=torch.bfloat16, mul=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * mul).to(dtype)


def _banded_mask(b, n, qb, kb, seed, period=5, keep=0.3):
    """Mask rows that repeat with a period (query blocks `period` apart select nearly the same key blocks, as the
    same spatial region of neighbouring video frames does) plus per-row noise, a full row, an empty row."""
    g = torch.Generator().manual_seed(seed)
    base = torch.rand(b, n, period, kb, generator=g) < keep
    m = base[:, :, torch.arange(qb) % period]
    flip = torch.rand(b, n, qb, kb, generator=g) < 0.08
    m = m ^ flip
    m[:, :, 0] = True
    if qb > 3:
        m[:, :, 3] = False
    return m


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("s,n,nkv", [(1100, 2, 2), (2048, 4, 2), (1500, 1, 1), (130, 2, 1)])
def test_paired_vs_oracle_and_lists(cuda, s, n, nkv, dtype):
    from mindiesd.layers.flash_attn import rainfusion as rf
    q = _rand((2, n, s, 128), 1, dtype)
    k, v = _rand((2, nkv, s, 128), 2, dtype), _rand((2, nkv, s, 128), 3, dtype)
    nb = (s + 127) // 128
    m = _banded_mask(2, n, nb, nb, seed=s)
    want = oa.block_sparse_attention(q, k, v, m.numpy())
    qd, kd, vd, md = q.to(cuda), k.to(cuda), v.to(cuda), m.to(torch.int8).to(cuda)
    out, lse = rf.block_sparse_attention_mask(qd, kd, vd, md, 128 ** -0.5, "BNSD", return_lse=True)
    eb, ok, mx = oa.ref_compare(want, out.cpu(), 2.0 ** -6)
    assert ok, (eb, mx)
    if nb > 3:
        assert not out[:, :, 3 * 128:4 * 128].any()                       # the empty mask row gives zeros
    idx, cnt = rf.mask_to_lists(md)
    out1, lse1 = rf.block_sparse_attention_lists(qd, kd, vd, idx, cnt, 128 ** -0.5, "BNSD", return_lse=True)
    assert (out.float() - out1.float()).abs().max().item() <= (2e-2 if dtype == torch.bfloat16 else 3e-3)
    rows = torch.isfinite(lse1)
    assert torch.equal(rows, torch.isfinite(lse))
    assert (lse[rows] - lse1[rows]).abs().max().item() < 5e-3


def test_paired_scores_far_below_zero(cuda):
    """Every score hundreds of units below zero (q = +8, k near -8): the first key block of a row moves the running
    maximum far down in both passes.  (Constant queries: the kernel's rounding of q * scale * log2(e) to bf16 is then a
    common factor of all scores, which at |s| ~ 700 would otherwise exceed the tolerance.)"""
    from mindiesd.layers.flash_attn import rainfusion as rf
    s, n = 1100, 2
    g = torch.Generator().manual_seed(11)
    q = torch.full((1, n, s, 128), 8.0, dtype=torch.bfloat16)
    k = (-8.0 + 0.5 * torch.randn((1, n, s, 128), generator=g)).to(torch.bfloat16)
    v = torch.randn((1, n, s, 128), generator=g).to(torch.bfloat16)
    nb = (s + 127) // 128
    m = _banded_mask(1, n, nb, nb, seed=12)
    want = oa.block_sparse_attention(q, k, v, m.numpy())
    out = rf.block_sparse_attention_mask(q.to(cuda), k.to(cuda), v.to(cuda), m.to(torch.int8).to(cuda), 128 ** -0.5, "BNSD")
    assert not torch.isnan(out.float()).any()
    eb, ok, mx = oa.ref_compare(want, out.cpu(), 2.0 ** -6)
    assert ok, (eb, mx)
    idx, cnt = rf.mask_to_lists(m.to(torch.int8).to(cuda))
    out1 = rf.block_sparse_attention_lists(q.to(cuda), k.to(cuda), v.to(cuda), idx, cnt, 128 ** -0.5, "BNSD")
    assert oa.ref_compare(want, out1.cpu(), 2.0 ** -6)[1]


def test_paired_bsnd_cross_lengths_and_full_mask(cuda):
    """BSND tensors in place, more keys than queries, and the all-ones mask (= dense attention)."""
    from mindiesd.layers.flash_attn import rainfusion as rf
    sq, skv, n = 700, 1300, 3
    q, k, v = _rand((1, sq, n, 128), 4), _rand((1, skv, n, 128), 5), _rand((1, skv, n, 128), 6)
    qb, kb = (sq + 127) // 128, (skv + 127) // 128
    m = _banded_mask(1, n, qb, kb, seed=7, period=2, keep=0.5)
    want = oa.block_sparse_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), m.numpy())
    out = rf.block_sparse_attention_mask(q.to(cuda), k.to(cuda), v.to(cuda), m.to(torch.int8).to(cuda), 128 ** -0.5, "BSND")
    assert out.shape == q.shape
    assert oa.ref_compare(want, out.cpu().transpose(1, 2), 2.0 ** -6)[1]
    full = torch.ones(1, n, qb, kb, dtype=torch.int8)
    dense = oa.attention_math(q, k, v, None, 128 ** -0.5, head_first=False)
    out = rf.block_sparse_attention_mask(q.to(cuda), k.to(cuda), v.to(cuda), full.to(cuda), 128 ** -0.5, "BSND")
    assert (out.cpu().float() - dense.float()).abs().max().item() <= 2e-2


def test_paired_with_token_order_matches_explicit_permutation(cuda):
    """Query and output addressed through a token table = attention on the permuted query + inverse permutation."""
    from mindiesd.layers.flash_attn import rainfusion as rf
    s, n = 1000, 2
    q, k, v = _rand((1, n, s, 128), 8), _rand((1, n, s, 128), 9), _rand((1, n, s, 128), 10)
    nb = (s + 127) // 128
    m = _banded_mask(1, n, nb, nb, seed=11, period=3).to(torch.int8).to(cuda)
    perm = torch.randperm(s, generator=torch.Generator().manual_seed(12)).to(torch.int32).to(cuda)
    qd, kd, vd = q.to(cuda), k.to(cuda), v.to(cuda)
    a = rf.block_sparse_attention_mask(qd, kd, vd, m, 128 ** -0.5, "BNSD", order=perm)
    b = rf.block_sparse_attention_mask(qd[:, :, perm.long()].contiguous(), kd, vd, m, 128 ** -0.5, "BNSD")
    inv = torch.empty_like(b)
    inv[:, :, perm.long()] = b
    assert torch.equal(a, inv)


def test_pairs_cover_every_block_once_and_lists_partition_the_mask(cuda):
    """The pair tables straight from the workspace: every query block in exactly one pair, shared + exclusive lists
    of a block = its mask row, partners found for rows that repeat with a period."""
    from mindiesd import _native
    lib = _native.lib()
    s, n = 128 * 37, 2
    nb = 37
    m = _banded_mask(1, n, nb, nb, seed=13, period=7)
    q = _rand((1, n, s, 128), 14).to(cuda)
    md = m.to(torch.int8).to(cuda)
    out = torch.empty_like(q)
    wsb = lib.mindiesd_block_sparse_attention_paired_workspace_size(1, n, s, s)
    ws = torch.zeros(wsb // 4, dtype=torch.int32, device=cuda)
    rc = lib.mindiesd_block_sparse_attention_paired_fwd(
        q.data_ptr(), q.data_ptr(), q.data_ptr(), out.data_ptr(), None, 0, 1, n, n, s, s, 128,
        *q.stride()[:3], *q.stride()[:3], *q.stride()[:3], *out.stride()[:3], 128 ** -0.5, md.data_ptr(), None,
        ws.data_ptr(), wsb, _native.stream_ptr(cuda))
    assert rc == 0
    w = ws.cpu().numpy()
    np_ = (nb + 1) // 2
    off = n * s                      # the state array comes first
    off += n * nb * ((nb + 31) // 32) + n * nb   # bit rows and their counts
    off += n * nb * 4                # candidates
    pairs = w[off:off + n * np_ * 2].reshape(n, np_, 2); off += n * np_ * 2
    sh_idx = w[off:off + n * np_ * nb].reshape(n, np_, nb); off += n * np_ * nb
    sh_cnt = w[off:off + n * np_].reshape(n, np_); off += n * np_
    ex_idx = w[off:off + n * nb * nb].reshape(n, nb, nb); off += n * nb * nb
    ex_cnt = w[off:off + n * nb].reshape(n, nb); off += n * nb
    init_cnt = w[off:off + n * nb].reshape(n, nb)
    mm = m[0].numpy()
    far = 0
    for h in range(n):
        members = pairs[h].reshape(-1)
        members = members[members >= 0]
        assert sorted(members.tolist()) == list(range(nb))
        for p in range(np_):
            a, b = pairs[h, p]
            shared = set(sh_idx[h, p, :sh_cnt[h, p]].tolist())
            for blk in (a, b):
                if blk < 0:
                    continue
                excl = ex_idx[h, blk, :ex_cnt[h, blk]].tolist()
                assert excl == sorted(excl) and not (set(excl) & shared)
                assert sorted(shared | set(excl)) == np.nonzero(mm[h, blk])[0].tolist()
                assert init_cnt[h, blk] == sh_cnt[h, p]
            if b >= 0:
                assert shared == set(np.nonzero(mm[h, a] & mm[h, b])[0].tolist())
                far += (b - a) % 7 == 0
    assert far >= n * np_ // 2      # most pairs are rows one period apart


def test_rainfusionattention_lists_with_malformed_entries(cuda):
    """The index-list op (csrc/plugin/rainfusionattention.cpp:27-64) on lists with ids outside the key blocks, -1
    padding inside the counted part and a count beyond the row width: such entries are dropped, the rest attends
    as the same selection given as a mask."""
    import mindiesd  # noqa: F401
    s, n, nb = 600, 2, 5
    q, k, v = (_rand((1, n, s, 128), 20 + i).to(cuda) for i in range(3))
    sel = torch.full((nb, n, nb), -1, dtype=torch.int64)
    num = torch.zeros((nb, n), dtype=torch.int64)
    keep = torch.zeros(1, n, nb, nb, dtype=torch.int8)
    rows = {0: [0, 2, 4], 1: [1], 2: [0, 1, 2, 3, 4], 3: [3, 99, 0], 4: [4, -1, 2]}
    for i, ids in rows.items():
        for h in range(n):
            sel[i, h, :len(ids)] = torch.tensor(ids)
            num[i, h] = len(ids) if i != 2 else 9          # a count beyond the width of the row
            for j in ids:
                if 0 <= j < nb:
                    keep[0, h, i, j] = 1
    out, lse = torch.ops.mindiesd.rainfusionattention(q, k, v, sel.to(cuda), num.to(cuda), [128, 128], q_input_layout="BNSD",
                                                      kv_input_layout="BNSD", head_num=n, scale=128 ** -0.5)
    want, _ = torch.ops.mindiesd.block_sparse_attention(q, k, v, keep.to(cuda), scale_value=128 ** -0.5)
    assert torch.equal(out, want)
    assert oa.ref_compare(oa.block_sparse_attention(q.cpu(), k.cpu(), v.cpu(), keep.numpy()), out.cpu(), 2.0 ** -6)[1]


def test_block_sparse_op_with_per_batch_lengths(cuda):
    """actual_seq_lengths / actual_seq_lengths_kv of the block_sparse_attention op
    (csrc/plugin/block_sparse_attention.cpp:42-66): batch entries shorter than the BNSD tensor, and TND tensors packing
    sequences of different lengths; each sequence against the oracle on its own slice."""
    import mindiesd  # noqa: F401
    n, s = 2, 900
    lens_q, lens_kv = [900, 333], [700, 900]
    q, k, v = _rand((2, n, s, 128), 31), _rand((2, n, s, 128), 32), _rand((2, n, s, 128), 33)
    nb = (s + 127) // 128
    m = _banded_mask(2, n, nb, nb, seed=34, period=3, keep=0.5)
    m[:, :, 3] = m[:, :, 2]
    out, lse = torch.ops.mindiesd.block_sparse_attention(
        q.to(cuda), k.to(cuda), v.to(cuda), m.to(torch.int8).to(cuda), scale_value=128 ** -0.5,
        actual_seq_lengths=lens_q, actual_seq_lengths_kv=lens_kv, softmax_lse_flag=1)
    assert out.shape == q.shape and lse.shape == (2, n, s, 1)
    for b in range(2):
        lq, lk = lens_q[b], lens_kv[b]
        qb, kb = (lq + 127) // 128, (lk + 127) // 128
        want = oa.block_sparse_attention(q[b:b + 1, :, :lq], k[b:b + 1, :, :lk], v[b:b + 1, :, :lk], m[b:b + 1, :, :qb, :kb].numpy())
        assert oa.ref_compare(want, out[b:b + 1, :, :lq].cpu(), 2.0 ** -6)[1]
        assert not out[b, :, lq:].any()
    # the same two sequences packed as TND
    qt = torch.cat([q[b, :, :lens_q[b]].transpose(0, 1) for b in range(2)]).contiguous()
    kt = torch.cat([k[b, :, :lens_kv[b]].transpose(0, 1) for b in range(2)]).contiguous()
    vt = torch.cat([v[b, :, :lens_kv[b]].transpose(0, 1) for b in range(2)]).contiguous()
    out_t, lse_t = torch.ops.mindiesd.block_sparse_attention(
        qt.to(cuda), kt.to(cuda), vt.to(cuda), m.to(torch.int8).to(cuda), q_input_layout="TND", kv_input_layout="TND",
        scale_value=128 ** -0.5, actual_seq_lengths=lens_q, actual_seq_lengths_kv=lens_kv, softmax_lse_flag=1)
    assert out_t.shape == qt.shape and lse_t.shape == (sum(lens_q), n, 1)
    t0 = 0
    for b in range(2):
        lq = lens_q[b]
        assert torch.equal(out_t[t0:t0 + lq].transpose(0, 1), out[b, :, :lq])
        assert torch.equal(lse_t[t0:t0 + lq, :, 0].transpose(0, 1), lse[b, :, :lq, 0])
        t0 += lq
    with pytest.raises(RuntimeError):
        torch.ops.mindiesd.block_sparse_attention(q.to(cuda), k.to(cuda), v.to(cuda), m.to(torch.int8).to(cuda),
                                                  actual_seq_lengths=[901, 5], actual_seq_lengths_kv=lens_kv)
    # every sequence shorter than the tensors: a mask sized for the tensors is accepted, its leading blocks are used
    lens_q, lens_kv = [300, 129], [257, 640]
    out2, _ = torch.ops.mindiesd.block_sparse_attention(
        q.to(cuda), k.to(cuda), v.to(cuda), m.to(torch.int8).to(cuda), scale_value=128 ** -0.5,
        actual_seq_lengths=lens_q, actual_seq_lengths_kv=lens_kv, softmax_lse_flag=1)
    for b in range(2):
        lq, lk = lens_q[b], lens_kv[b]
        qb, kb = (lq + 127) // 128, (lk + 127) // 128
        want = oa.block_sparse_attention(q[b:b + 1, :, :lq], k[b:b + 1, :, :lk], v[b:b + 1, :, :lk], m[b:b + 1, :, :qb, :kb].numpy())
        assert oa.ref_compare(want, out2[b:b + 1, :, :lq].cpu(), 2.0 ** -6)[1]
        assert not out2[b, :, lq:].any()
