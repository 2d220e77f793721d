"""Writes the fixtures of tests/golden/ (run from the repository root: python tests/golden/make_fixtures.py).

Two kinds of data:
  * reference_kats.json - known answers copied (as data) from the reference's own tests of this path,
    each with the file:line it comes from;
  * *.npz - seeded inputs and the outputs of the CPU oracle for them, written after the oracle
    had been pinned (tests/test_oracle_*.py).  The reference's vendor kernels cannot run here, and its
    Python was read, not run, so no vector in this folder was produced by executing reference code.
The tests in tests/test_golden_fixtures.py check the oracle (CPU) and the HIP path (GPU) against them.
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import attention as oa  # noqa: E402
from oracle import quant as oq  # noqa: E402
from oracle import rainfusion as orf  # noqa: E402


def bits16(t):
    return t.contiguous().view(torch.int16).numpy()


def rand16(shape, seed, dtype=torch.bfloat16, scale=1.0):
    """Seeded inputs from numpy's frozen legacy generator (its stream is guaranteed not to change), so the
    large inputs need not be stored: tests regenerate them with the same call."""
    x = np.random.RandomState(seed).standard_normal(size=shape).astype(np.float32) * np.float32(scale)
    return torch.from_numpy(x).to(dtype)


def main():
    kats = {
        "avgpool": {
            "source": "tests/layers/flash_attn/test_sparse_flash_attn_rf_v2.py:104-119",
            "input": "arange(256) along the sequence, pool 128", "means": [63.5, 191.5]},
        "get_mask_index": {
            "source": "tests/layers/flash_attn/test_sparse_flash_attn_rf_v2.py:198-216",
            "all_true_4x4_rows": [0, 1, 2, 3],
            "partial": {"true_at_row0_cols": [0, 2], "row0_first_three": [0, 2, -1]}},
        "grids": {
            "source": "tests/layers/flash_attn/test_sparse_flash_attn_rf_v2.py:32-38",
            "t_h_w": [[3, 40, 80], [3, 30, 52], [2, 21, 32], [2, 24, 45]]},
        "kernel_tolerance": {
            "source": "tests/plugin/test_adablocksparseattention.py:26-32,173",
            "rule": "|actual-golden| <= err * max(1, |golden|) everywhere and mean(|actual-golden| / max(1, |golden|)) <= err / 2",
            "err": 2.0 ** -6},
        "data_compare": {
            "source": "tests/utils/utils/precision_compare.py:89 (diff_thd=0.001, pct_thd=0.999, max_diff_hd=0.1)",
            "rule": ">= 99.9 % of elements within rel 1e-3 (abs where |golden| < 1), none beyond 0.1"},
    }
    with open(os.path.join(HERE, "reference_kats.json"), "w") as f:
        json.dump(kats, f, indent=1)

    # dense + block-sparse attention, one batch, two heads (one KV head), 200 tokens (a 72-token tail block)
    q = rand16((1, 2, 200, 128), 11, scale=0.5)
    k = rand16((1, 1, 200, 128), 12, scale=0.5)
    v = rand16((1, 1, 200, 128), 13, scale=0.5)
    kk, vv = k.expand(1, 2, 200, 128), v.expand(1, 2, 200, 128)
    dense = oa.attention_math(q, kk, vv, head_first=True)
    bmask = torch.tensor([[[[1, 0], [1, 1]], [[0, 1], [0, 0]]]], dtype=torch.int8)
    sparse = oa.block_sparse_attention(q, k, v, bmask)
    np.savez_compressed(os.path.join(HERE, "attention_small.npz"), seeds=np.array([11, 12, 13]),
                        q_checksum=np.array(bits16(q).astype(np.int64).sum()),
                        dense_out=bits16(dense.to(torch.bfloat16)), block_mask=bmask.numpy(),
                        sparse_out=bits16(sparse.to(torch.bfloat16)))

    # RainFusion: grid (3, 16, 24) = 1152 tokens = 9 blocks, 2 heads, bf16, sparsity 0.5
    grid = (3, 16, 24)
    s = grid[0] * grid[1] * grid[2]
    rq, rk, rv = (rand16((1, 2, s, 128), 20 + i) for i in range(3))
    q_, k_, v_, pool = orf.do_tensor_rearrange_pooling(rq, rk, rv, 0, 128, grid, grid, "BNSD")
    mask = orf.get_blockwise_mask(pool, 0, 0.5, 128 ** -0.5, 128, grid, grid, "BNSD", return_binary=True)
    mask_d = orf.get_blockwise_mask(pool, 0, 0.5, 128 ** -0.5, 128, grid, grid, "BNSD", return_binary=True,
                                    keep_diagonal=True)
    np.savez_compressed(os.path.join(HERE, "rainfusion_small.npz"), grid=np.array(grid), seeds=np.array([20, 21, 22]),
                        q_checksum=np.array(bits16(rq).astype(np.int64).sum()), order=np.asarray(orf.window_order(*grid)).astype(np.int32),
                        q_perm_row0=bits16(q_[0, 0, :, 0]), pool=bits16(pool), mask=mask.numpy(),
                        mask_keep_diagonal=mask_d.numpy())

    # FP8 E4M3: the decode table, block quantisation, per-channel quantisation
    x = rand16((1, 2, 300, 128), 31) * torch.logspace(-1, 1, 300)[None, None, :, None].to(torch.bfloat16)
    codes, scale = oq.dynamic_block_quant(x[0, 0], 128, 128)
    vcodes, vscale = oq.per_channel_quant(x[0, 0])
    np.savez_compressed(os.path.join(HERE, "fp8_small.npz"), seed=np.array(31),
                        x_checksum=np.array(bits16(x).astype(np.int64).sum()),
                        e4m3_table=oq.e4m3_decode(np.arange(256, dtype=np.uint8)),
                        block_codes_head0=codes.numpy(), block_scale_head0=scale.numpy(),
                        v_codes_head0=vcodes.numpy(), v_scale_head0=vscale.numpy())

    # MXFP8: quantisation and GEMM + SwiGLU
    xm = rand16((40, 256), 41) * torch.logspace(-2, 2, 40)[:, None].to(torch.bfloat16)
    wm = rand16((2 * 24, 256), 42, scale=0.05)
    mc, me = oq.mx_quant(xm)
    np.savez_compressed(os.path.join(HERE, "mxfp8_small.npz"), x=bits16(xm), w=bits16(wm), x_codes=mc.numpy(),
                        x_e8m0=me.numpy(), swiglu_out=oq.mxfp8_gemm_swiglu(xm, wm, torch.float32).numpy(),
                        gemm_out=oq.mxfp8_gemm(xm, wm).float().numpy())
    for name in sorted(os.listdir(HERE)):
        print(name, os.path.getsize(os.path.join(HERE, name)))


if __name__ == "__main__":
    main()
