"""Pins the RainFusion oracle: permutation against the reference's einops pattern strings,
pooling against known answers and torch.mean, the exact-sum block mask against the literal torch-op
composite of the reference, index lists against the reference's known answers."""
import math

import numpy as np
import pytest
import torch
from einops import rearrange

from oracle import rainfusion as orf

# grids of the reference's own tests (tests/layers/flash_attn/test_sparse_flash_attn_rf_v2.py:32-38)
GRIDS = [(3, 40, 80), (3, 30, 52), (2, 21, 32), (2, 24, 45)]


def _einops_window_order(t, h, w):
    """Token ids pushed through the reference's pattern strings (rf_v2.py:148-170) with einops."""
    ids = torch.arange(t * h * w).reshape(1, 1, t * h * w, 1)
    if h % 8 == 0 and w % 8 == 0:
        return rearrange(ids, "b n (f hn hb wn wb) d -> b n (f hn wn hb wb) d", f=t, hb=8, wb=8, hn=h // 8,
                         wn=w // 8).flatten()
    first, rest = ids[:, :, :h * w], ids[:, :, h * w:]
    x = rearrange(rest, "b n (f h w) d -> b n f h w d", f=t - 1, h=h, w=w)
    h_r = w_r = None
    if h % 8:
        x, h_r = torch.split(x, h - h % 8, dim=3)
        h_r = h_r.reshape(1, 1, t - 1, -1, 1)
    if w % 8:
        x, w_r = torch.split(x, w - w % 8, dim=4)
        w_r = w_r.reshape(1, 1, t - 1, -1, 1)
    x = rearrange(x, "b n f (hn hb) (wn wb) d -> b n f (hn wn hb wb) d", f=t - 1, hb=8, wb=8, hn=h // 8, wn=w // 8)
    if h_r is not None:
        x = torch.cat((x, h_r), dim=3)
    if w_r is not None:
        x = torch.cat((x, w_r), dim=3)
    return torch.cat([first, x.reshape(1, 1, -1, 1)], dim=2).flatten()


@pytest.mark.parametrize("grid", GRIDS + [(1, 8, 8), (2, 9, 8), (2, 8, 9), (4, 15, 17)])
def test_window_order_matches_einops_patterns(grid):
    src = orf.window_order(*grid)
    assert np.array_equal(src, _einops_window_order(*grid).numpy())
    assert np.array_equal(np.sort(src), np.arange(src.size)), "must be a permutation"


def test_window_order_tiny_brute_force():
    """2 frames of 8x16: frame f, window column wn, inside the window row-major."""
    src = orf.window_order(2, 8, 16)
    expect = [f * 128 + hb * 16 + wn * 8 + wb for f in range(2) for wn in range(2) for hb in range(8) for wb in range(8)]
    assert src.tolist() == expect


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("grid", GRIDS)
def test_round_trip(grid, layout):
    s = grid[0] * grid[1] * grid[2]
    x = torch.randn((1, 2, s, 4) if layout == "BNSD" else (1, s, 2, 4))
    y = orf.rearrange_with_remaining(x, grid, grid, layout)
    assert y.shape == x.shape and not torch.equal(y, x)
    assert torch.equal(orf.inv_rearrange_with_remaining(y, grid, grid, layout), x)


@pytest.mark.parametrize("grid", GRIDS)
def test_inverse_matches_reshape_permute_inverse(grid):
    """Second, independent inverse: the reshape/permute construction of rf_v3.py:22-97 (BNSD)."""
    t, h, w = grid
    x = torch.randn(1, 1, t * h * w, 2)
    y = orf.rearrange_with_remaining(x, grid, grid, "BNSD")
    hn, wn = h // 8, w // 8
    if h % 8 == 0 and w % 8 == 0:
        inv = y.reshape(1, 1, t, hn, wn, 8, 8, 2).permute(0, 1, 2, 3, 5, 4, 6, 7).reshape(1, 1, -1, 2)
    else:
        first, rest = y[:, :, :h * w], y[:, :, h * w:].reshape(1, 1, t - 1, h * w, 2)
        nblk, hrem = hn * wn * 64, (h % 8) * w
        blk = rest[:, :, :, :nblk].reshape(1, 1, t - 1, hn, wn, 8, 8, 2).permute(0, 1, 2, 3, 5, 4, 6, 7)
        blk = blk.reshape(1, 1, t - 1, hn * 8, wn * 8, 2)
        if w % 8:
            blk = torch.cat([blk, rest[:, :, :, nblk + hrem:].reshape(1, 1, t - 1, hn * 8, w % 8, 2)], dim=4)
        if h % 8:
            blk = torch.cat([blk, rest[:, :, :, nblk:nblk + hrem].reshape(1, 1, t - 1, h % 8, w, 2)], dim=3)
        inv = torch.cat([first, blk.reshape(1, 1, -1, 2)], dim=2)
    assert torch.equal(inv, x)


# ---- pooling -------------------------------------------------------------------------------------
@pytest.mark.parametrize("layout,shape", [("BSND", (1, 256, 1, 1)), ("BNSD", (1, 1, 256, 1))])
def test_avgpool_reference_known_answers(layout, shape):
    """test_sparse_flash_attn_rf_v2.py:104-119: arange(256) -> 63.5 and 191.5."""
    out = orf.avgpool(torch.arange(256, dtype=torch.float32).reshape(shape), 128, layout).flatten()
    assert out.tolist() == [63.5, 191.5]


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
@pytest.mark.parametrize("s", [64, 768, 800])
def test_avgpool_shapes_and_tail(layout, s):
    x = torch.randn((1, 2, s, 64) if layout == "BNSD" else (1, s, 2, 64))
    out = orf.avgpool(x, 128, layout)
    nb = math.ceil(s / 128)
    assert out.shape == ((1, 2, nb, 64) if layout == "BNSD" else (1, nb, 2, 64))
    dim = 2 if layout == "BNSD" else 1
    tail = x.narrow(dim, (nb - 1) * 128, s - (nb - 1) * 128).double().mean(dim=dim)
    assert torch.allclose(out.select(dim, nb - 1).double(), tail, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_avgpool_agrees_with_torch_mean_16bit(dtype):
    """torch's mean (cast_fp32 -> sum -> div -> cast) differs from the exact-sum oracle only where
    its fp32 summation order rounds differently: a vanishing fraction, never more than one ulp."""
    x = torch.randn(2, 3, 1000, 128).to(dtype)
    got = orf.avgpool(x, 128, "BNSD")
    want = torch.cat([x[:, :, :896].view(2, 3, 7, 128, 128).mean(dim=3), x[:, :, 896:].mean(dim=2, keepdim=True)], 2)
    diff = (got.float() - want.float()).abs()
    assert (diff > 0).float().mean() < 1e-3
    ulp = torch.finfo(dtype).eps
    assert (diff <= ulp * want.float().abs().clamp(min=2.0 ** -6)).all()


# ---- index lists -----------------------------------------------------------------------------------
def test_get_mask_index_reference_known_answers():
    """test_sparse_flash_attn_rf_v2.py:191-216."""
    pos = orf.get_mask_index(torch.ones(1, 2, 8, 8, dtype=torch.bool))
    assert pos.shape == (1, 2, 8, 8) and pos.dtype == torch.int64
    assert all(pos[0, 0, r].tolist() == list(range(8)) for r in range(8))
    m = torch.zeros(1, 1, 4, 4, dtype=torch.bool)
    m[0, 0, 0, 0] = m[0, 0, 0, 2] = True
    pos = orf.get_mask_index(m)
    assert pos[0, 0, 0].tolist() == [0, 2, -1, -1]


# ---- block mask ------------------------------------------------------------------------------------
def _pool(n, nb, seed, dtype, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(3, n, nb, 128, generator=g) * spread).to(dtype)


def test_keep_len_expression():
    assert orf.keep_len_of(591, 0.75) == 148 and orf.keep_len_of(256, 0.8) == math.ceil(256 * (1 - 0.8))
    assert orf.keep_len_of(10, 0.0) == 10


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("sparsity", [0.0, 0.5, 0.75, 0.9])
def test_block_mask_matches_torch_op_composite(dtype, sparsity):
    """The oracle (exact sums, same rounding points) against the reference's literal torch ops.
    They may differ only on entries whose score ties with the threshold after a last-bit change of
    an fp32 sum; on these seeds the masks are identical."""
    grid = (3, 30, 52)
    pool = _pool(4, 37, 3, dtype, spread=0.8)
    want = orf.get_blockwise_mask_torch(pool, 0, sparsity, 128 ** -0.5, 128, grid, grid, "BNSD")
    got = orf.get_blockwise_mask(pool, 0, sparsity, 128 ** -0.5, 128, grid, grid, "BNSD", return_binary=True)
    mismatch = (got.bool() != want).float().mean().item()
    assert mismatch <= 2e-3, mismatch
    if dtype != torch.float32 or sparsity == 0.0:
        assert mismatch == 0.0


@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
def test_block_mask_layouts_and_forms_agree(layout):
    grid = (3, 40, 80)
    pool = _pool(2, 75, 5, torch.bfloat16)
    p = pool if layout == "BNSD" else pool.transpose(1, 2).contiguous()
    binary = orf.get_blockwise_mask(p, 0, 0.5, 0.09, 128, grid, grid, layout, return_binary=True)
    ref = orf.get_blockwise_mask(pool, 0, 0.5, 0.09, 128, grid, grid, "BNSD", return_binary=True)
    assert binary.dtype == torch.int8 and torch.equal(binary, ref)
    sel, num = orf.get_blockwise_mask(p, 0, 0.5, 0.09, 128, grid, grid, layout)
    assert sel.shape == (75, 2, 75) and num.shape == (75, 2)       # rf_v2.py:131-134: [qb, N, kb], [qb, N]
    assert torch.equal(num, binary[0].transpose(0, 1).sum(-1))
    for r in (0, 30, 74):
        for n in range(2):
            c = int(num[r, n])
            assert sel[r, n, :c].tolist() == torch.nonzero(binary[0, n, r]).flatten().tolist()
            assert (sel[r, n, c:] == -1).all()


def test_block_mask_invariants():
    """First-frame and text protection (tests/plugin/test_rf_v3_attention.py:99-120), keep count,
    threshold semantics (score >= k-th largest keeps ties)."""
    grid = (3, 30, 52)            # first frame = 1560 tokens -> 13 blocks
    nb = math.ceil((3 * 30 * 52 + 200) / 128) + 0
    nb_img = math.ceil(3 * 30 * 52 / 128)
    pool = _pool(2, nb_img + 2, 7, torch.bfloat16)
    m = orf.get_blockwise_mask(pool, 200, 0.8, 0.09, 128, grid, grid, "BNSD", return_binary=True).bool()
    assert m[:, :, :13, :].all() and m[:, :, :, :13].all()
    assert m[:, :, -2:, :].all() and m[:, :, :, -2:].all()
    keep = orf.keep_len_of(m.shape[-1], 0.8)
    assert int(m.sum(-1).min()) >= keep
    free = orf.get_blockwise_mask(pool, 0, 0.8, 0.09, 128, grid, grid, "BNSD", return_binary=True,
                                  protect_first_frame=False).bool()
    p = orf.block_scores(pool, 0.09).float()
    kth = torch.sort(p, dim=-1, descending=True).values[..., keep - 1:keep]
    assert torch.equal(free, p >= kth)
    assert int(free.sum(-1).min()) >= keep and not free[:, :, :13, :].all()
    diag = orf.get_blockwise_mask(pool, 0, 0.8, 0.09, 128, grid, grid, "BNSD", return_binary=True,
                                  protect_first_frame=False, keep_diagonal=True).bool()
    assert torch.diagonal(diag, dim1=-2, dim2=-1).all() and (diag | free).equal(diag)


def test_block_scores_sum_to_one_and_follow_exact_scores():
    pool = _pool(1, 20, 9, torch.bfloat16)
    p = orf.block_scores(pool, 0.09)
    assert p.dtype == torch.bfloat16 and (p.float().sum(-1) - 1).abs().max() < 0.02
    exact = torch.softmax(torch.einsum("bnld,bnsd->bnls", pool[:1].double(), pool[1:2].double()) * 0.09, -1)
    assert (p.double() - exact).abs().max() < 0.01


# ---- pipeline glue ---------------------------------------------------------------------------------
@pytest.mark.parametrize("layout", ["BNSD", "BSND"])
def test_rearrange_pooling_text_goes_last_and_comes_back(layout):
    grid, txt = (2, 21, 32), 200
    s = 2 * 21 * 32 + txt
    shape = (1, 2, s, 8) if layout == "BNSD" else (1, s, 2, 8)
    q, k, v = (torch.randn(shape) for _ in range(3))
    q_, k_, v_, pool = orf.do_tensor_rearrange_pooling(q, k, v, txt, 128, grid, grid, layout)
    dim = 2 if layout == "BNSD" else 1
    assert torch.equal(q_.narrow(dim, s - txt, txt), q.narrow(dim, 0, txt))
    nb = math.ceil((s - txt) / 128) + math.ceil(txt / 128)
    assert pool.shape[0] == 3 and pool.shape[dim] == nb
    assert torch.equal(orf.do_tensor_inv_rearrange(k_, txt, grid, grid, layout), k)


def test_end_to_end_sparsity_zero_is_dense():
    from oracle.attention import attention_math
    grid = (2, 16, 16)
    q, k, v = (torch.randn(1, 2, 512, 16) for _ in range(3))
    out, mask = orf.bsa_sparse_attention_v3(q, k, v, grid, sparsity=0.0, input_layout="BNSD", scale=0.25)
    assert bool(mask.all())
    assert (out - attention_math(q, k, v, None, 0.25, head_first=True)).abs().max() < 1e-5
