"""Tensors larger than 4 GiB: batch, head and row offsets are 64-bit inside the kernels (only the offsets inside one
(batch, head) K/V panel are 32-bit, and the entry points refuse panels beyond 2 GiB).  A batch of six problems of the
Wan2.1-14B 720p shape (4.6 GB per tensor) must give, batch by batch, the very bits of the one-problem calls."""
import pytest
import torch

pytestmark = pytest.mark.gpu

B, N, S, D = 6, 40, 75600, 128


@pytest.fixture(scope="module")
def big_qkv(cuda):
    free, _ = torch.cuda.mem_get_info(cuda)
    if free < 48 * 2 ** 30:
        pytest.skip("needs 48 GiB of free device memory")
    g = torch.Generator(device=cuda).manual_seed(0)
    qkv = tuple(torch.randn((B, N, S, D), generator=g, device=cuda, dtype=torch.bfloat16) for _ in range(3))
    assert qkv[0].numel() * 2 > 2 ** 32
    yield qkv
    del qkv
    torch.cuda.empty_cache()


def test_dense_batches_beyond_4gib(cuda, big_qkv):
    import mindiesd
    q, k, v = big_qkv
    out = mindiesd.attention_forward(q, k, v, head_first=True)
    for b in (0, B - 1):
        one = mindiesd.attention_forward(q[b:b + 1], k[b:b + 1], v[b:b + 1], head_first=True)
        assert torch.equal(out[b:b + 1], one), f"batch {b}"
    # token-major layout: the head offset is small, the row stride N * D, the batch offset beyond 2^31 elements
    qs, ks, vs = (t[3:].transpose(1, 2).contiguous() for t in (q, k, v))
    got = mindiesd.attention_forward(qs, ks, vs)
    assert torch.equal(got[2:3].transpose(1, 2), out[5:6])


def test_block_sparse_batches_beyond_4gib(cuda, big_qkv):
    from mindiesd.layers.flash_attn import rainfusion as rf
    q, k, v = big_qkv
    nb = (S + 127) // 128
    g = torch.Generator(device=cuda).manual_seed(1)
    mask = (torch.rand((B, N, nb, nb), generator=g, device=cuda) < 0.1).to(torch.int8)
    out = rf.block_sparse_attention_mask(q, k, v, mask, D ** -0.5, "BNSD")
    assert not torch.isnan(out[B - 1].float()).any()
    for b in (0, B - 1):
        one = rf.block_sparse_attention_mask(q[b:b + 1], k[b:b + 1], v[b:b + 1], mask[b:b + 1].contiguous(),
                                             D ** -0.5, "BNSD")
        assert torch.equal(out[b:b + 1], one), f"batch {b}"
