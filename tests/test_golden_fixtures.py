"""The committed vectors of tests/golden/: the CPU oracle must reproduce them (guards the checker against
drift) and the HIP path must match them (bit-exact for integer/byte/index outputs, the stated tolerances
for floating point).  tests/golden/make_fixtures.py documents where every vector comes from."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import attention as oa
from oracle import quant as oq
from oracle import rainfusion as orf

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def _rand16(shape, seed, dtype=torch.bfloat16, scale=1.0):
    x = np.random.RandomState(seed).standard_normal(size=shape).astype(np.float32) * np.float32(scale)
    return torch.from_numpy(x).to(dtype)


def _bits(t):
    return t.contiguous().view(torch.int16).numpy()


def _from_bits(a, dtype=torch.bfloat16):
    return torch.from_numpy(np.ascontiguousarray(a)).view(dtype)


def _attention_inputs(fx):
    q = _rand16((1, 2, 200, 128), int(fx["seeds"][0]), scale=0.5)
    k = _rand16((1, 1, 200, 128), int(fx["seeds"][1]), scale=0.5)
    v = _rand16((1, 1, 200, 128), int(fx["seeds"][2]), scale=0.5)
    assert int(_bits(q).astype(np.int64).sum()) == int(fx["q_checksum"]), "seeded inputs changed"
    return q, k, v


def _rainfusion_inputs(fx):
    grid = tuple(int(g) for g in fx["grid"])
    s = grid[0] * grid[1] * grid[2]
    q, k, v = (_rand16((1, 2, s, 128), int(sd)) for sd in fx["seeds"])
    assert int(_bits(q).astype(np.int64).sum()) == int(fx["q_checksum"]), "seeded inputs changed"
    return grid, q, k, v


def _fp8_input(fx):
    x = _rand16((1, 2, 300, 128), int(fx["seed"])) * torch.logspace(-1, 1, 300)[None, None, :, None].to(torch.bfloat16)
    assert int(_bits(x).astype(np.int64).sum()) == int(fx["x_checksum"]), "seeded inputs changed"
    return x


# ---- CPU: reference known answers and the oracle against the fixtures --------------------------------------
def test_reference_known_answers():
    kats = json.load(open(os.path.join(GOLDEN, "reference_kats.json")))
    x = torch.arange(256, dtype=torch.float32).reshape(1, 1, 256, 1)
    pooled = orf.avgpool(x, 128, "BNSD")
    assert [pooled[0, 0, 0, 0].item(), pooled[0, 0, 1, 0].item()] == kats["avgpool"]["means"]
    pos = orf.get_mask_index(torch.ones(1, 1, 4, 4, dtype=torch.bool))
    assert all(pos[0, 0, r].tolist() == kats["get_mask_index"]["all_true_4x4_rows"] for r in range(4))
    m = torch.zeros(1, 1, 4, 4, dtype=torch.bool)
    for c in kats["get_mask_index"]["partial"]["true_at_row0_cols"]:
        m[0, 0, 0, c] = True
    assert orf.get_mask_index(m)[0, 0, 0, :3].tolist() == kats["get_mask_index"]["partial"]["row0_first_three"]
    for t, h, w in kats["grids"]["t_h_w"]:
        order = np.asarray(orf.window_order(t, h, w))
        assert sorted(order.tolist()) == list(range(t * h * w))
    g = torch.tensor([0.5, -4.0])
    err = kats["kernel_tolerance"]["err"]
    assert oa.ref_compare(g, g + torch.tensor([err, 4 * err]) * 0.49, err)[1]
    assert not oa.ref_compare(g, g + torch.tensor([1.01 * err, 0.0]), err)[1]


def test_oracle_reproduces_attention_fixture():
    fx = _load("attention_small.npz")
    q, k, v = _attention_inputs(fx)
    dense = oa.attention_math(q, k.expand(1, 2, 200, 128), v.expand(1, 2, 200, 128), head_first=True)
    want = _from_bits(fx["dense_out"]).float()
    assert (dense.float() - want).abs().max() <= 2.0 ** -8 * want.abs().max()  # one bf16 ulp of the largest value
    sparse = oa.block_sparse_attention(q, k, v, torch.from_numpy(fx["block_mask"]))
    wants = _from_bits(fx["sparse_out"]).float()
    assert (sparse.float() - wants).abs().max() <= 2.0 ** -8 * max(1.0, wants.abs().max().item())
    assert not wants[0, 1, 128:].any()  # the query block with an empty list gives zeros


def test_oracle_reproduces_rainfusion_fixture():
    fx = _load("rainfusion_small.npz")
    grid, q, k, v = _rainfusion_inputs(fx)
    assert np.array_equal(np.asarray(orf.window_order(*grid)), fx["order"])
    q_, k_, v_, pool = orf.do_tensor_rearrange_pooling(q, k, v, 0, 128, grid, grid, "BNSD")
    assert np.array_equal(_bits(q_[0, 0, :, 0]), fx["q_perm_row0"])
    assert np.array_equal(_bits(pool), fx["pool"])
    for key, diag in (("mask", False), ("mask_keep_diagonal", True)):
        mask = orf.get_blockwise_mask(pool, 0, 0.5, 128 ** -0.5, 128, grid, grid, "BNSD", return_binary=True,
                                      keep_diagonal=diag)
        assert np.array_equal(mask.numpy(), fx[key])


def test_oracle_reproduces_quant_fixtures():
    fx = _load("fp8_small.npz")
    assert np.array_equal(oq.e4m3_decode(np.arange(256, dtype=np.uint8)), fx["e4m3_table"], equal_nan=True)
    x = _fp8_input(fx)
    codes, scale = oq.dynamic_block_quant(x[0, 0], 128, 128)
    assert np.array_equal(codes.numpy(), fx["block_codes_head0"]) and np.array_equal(scale.numpy(), fx["block_scale_head0"])
    vc, vs = oq.per_channel_quant(x[0, 0])
    assert np.array_equal(vc.numpy(), fx["v_codes_head0"]) and np.array_equal(vs.numpy(), fx["v_scale_head0"])
    mx = _load("mxfp8_small.npz")
    xm, wm = _from_bits(mx["x"]), _from_bits(mx["w"])
    c, e = oq.mx_quant(xm)
    assert np.array_equal(c.numpy(), mx["x_codes"]) and np.array_equal(e.numpy(), mx["x_e8m0"])
    assert np.allclose(oq.mxfp8_gemm_swiglu(xm, wm, torch.float32).numpy(), mx["swiglu_out"], rtol=1e-6, atol=1e-7)


# ---- GPU: the HIP path against the fixtures ---------------------------------------------------------------------
@pytest.mark.gpu
def test_gpu_attention_fixture(cuda):
    from mindiesd import attention_forward
    fx = _load("attention_small.npz")
    q, k, v = _attention_inputs(fx)
    out = attention_forward(q.to(cuda), k.expand(1, 2, 200, 128).contiguous().to(cuda),
                            v.expand(1, 2, 200, 128).contiguous().to(cuda), head_first=True).cpu()
    want = _from_bits(fx["dense_out"]).float()
    assert (out.float() - want).abs().max() <= 2e-2 and oa.cosine(out, want) >= 0.9999
    qb, kb = 2, 2
    mask = torch.from_numpy(fx["block_mask"]).to(cuda)
    sp, _ = torch.ops.mindiesd.block_sparse_attention(q.to(cuda), k.to(cuda), v.to(cuda), mask, scale_value=128 ** -0.5,
                                                      num_key_value_heads=1)
    wants = _from_bits(fx["sparse_out"]).float()
    assert oa.ref_compare(wants, sp.cpu(), 2.0 ** -6)[1]
    assert not sp.cpu()[0, 1, 128:].any()


@pytest.mark.gpu
def test_gpu_rainfusion_fixture(cuda):
    from mindiesd.layers.flash_attn import rainfusion as rf
    fx = _load("rainfusion_small.npz")
    grid, q, k, v = _rainfusion_inputs(fx)
    q_, k_, v_, pool = rf.do_tensor_rearrange_pooling(q.to(cuda), k.to(cuda), v.to(cuda), 0, 128, grid, grid, "BNSD")
    assert np.array_equal(_bits(q_.cpu()[0, 0, :, 0]), fx["q_perm_row0"])
    assert np.array_equal(_bits(pool.cpu()), fx["pool"])
    for key, diag in (("mask", False), ("mask_keep_diagonal", True)):
        mask = rf.get_blockwise_mask(pool, 0, 0.5, 128 ** -0.5, 128, grid, grid, "BNSD", return_binary=True,
                                     keep_diagonal=diag)
        assert np.array_equal(mask.cpu().numpy(), fx[key])


@pytest.mark.gpu
def test_gpu_quant_fixtures(cuda):
    from mindiesd.layers.quant import fa_block_quant_preprocess, mx_quantize, mxfp8_gemm_swiglu
    from mindiesd.layers.quant.fp8_attention import quantize_v_per_channel
    fx = _load("fp8_small.npz")
    x = _fp8_input(fx)
    codes, scale = fa_block_quant_preprocess(x.to(cuda), block_size=128, layout="BNSD")
    assert np.array_equal(codes.view(torch.uint8).cpu().numpy()[0, 0], fx["block_codes_head0"])
    assert np.array_equal(scale.cpu().numpy().reshape(2, -1)[0], fx["block_scale_head0"].reshape(-1))
    mx = _load("mxfp8_small.npz")
    xm, wm = _from_bits(mx["x"]), _from_bits(mx["w"])
    c, e = mx_quantize(xm.to(cuda))
    got, want = c.view(torch.uint8).cpu().numpy(), mx["x_codes"]
    assert np.array_equal(got & 0x7f, want & 0x7f) and np.array_equal(e.view(torch.uint8).cpu().numpy(), mx["x_e8m0"])
    nz = (want & 0x7f) != 0
    assert np.array_equal((got >> 7)[nz], (want >> 7)[nz])
    wq, ws = mx_quantize(wm.to(cuda))
    out = mxfp8_gemm_swiglu(xm.to(cuda), wq, ws).cpu()
    w = torch.from_numpy(mx["swiglu_out"])
    assert oa.cosine(out, w) >= 0.999 and ((out.float() - w).abs() <= 2.0 ** -7 * w.abs() + 1e-3).all()
