#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu]

Prints ONE JSON line.  A step is one dense bf16 flash-attention forward at the Wan2.1-14B 720p
shape (B=1, N=40, S=75600 = 21x45x80 latent grid, D=128, non-causal, scale 1/sqrt(128)) on synthetic
N(0,1)*0.5 inputs already resident in HBM; ``value`` is the achieved TFLOP/s (4*N*S^2*D flops per
step), which for a dense kernel equals the dense-equivalent figure.  ``roofline`` prices the same
kernel against the bf16 dense MFMA peak, from HIP-event timings of the launches on the stream they
run on.  ``extras`` carries the other workloads of the path (dense at the Wan2.1-1.3B shape,
RainFusion block-sparse attention with and without mask generation, and - when built - FP8
attention and the MXFP8 GEMM+SwiGLU).  ``cpu_baseline`` times the CPU oracle (a restatement of the
reference's unfused torch path) on a bounded sample of the same workload on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "mindie-sd_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA
PEAK_HBM_GBS = 8000.0
DENSE_PROFILE = os.path.join(ROOT, "profiles", "fa_fwd_dense_bf16_wan14b_720p.md")


def dense_traffic_bytes():
    """HBM-side bytes of one dense 14B-720p launch (fetch + write) as the committed rocprofv3 summary states them
    (--pmc FETCH_SIZE / WRITE_SIZE scaled by a 1 GiB copy kernel); None when the summary is not there."""
    import re
    try:
        with open(DENSE_PROFILE) as f:
            text = f.read()
        head = text[text.index("### the headline launch"):]
        m = re.search(r"fetch ([0-9.]+) GB.*?write ([0-9.]+) GB", head)
        return (float(m.group(1)) + float(m.group(2))) * 1e9
    except (OSError, ValueError, AttributeError):
        return None

# workloads
CFG_14B_720P = dict(B=1, N=40, S=75600, D=128, grid=(21, 45, 80))
CFG_1P3B = dict(B=1, N=12, S=32760, D=128, grid=(21, 30, 52))
CFG_14B_480P = dict(B=1, N=40, S=32760, D=128, grid=(21, 30, 52))
CFG_PARITY = dict(B=1, N=12, S=4096, D=128)
CFG_FFN = dict(M=32760, K=5120, N=13824)


def attn_flops(cfg):
    return 4.0 * cfg["B"] * cfg["N"] * cfg["S"] * cfg["S"] * cfg["D"]


from workloads import dense_inputs, outlier_inputs, smooth_field_inputs  # noqa: E402  (seeded synthetic inputs)


# ---- timing -----------------------------------------------------------------------------------------
def time_steps(fn, steps, warmup):
    """Per-step durations in ms from HIP events on the current stream (the stream the kernels are
    launched on), plus the wall-clock total of the timed region."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    evs[0].record()
    for i in range(steps):
        fn()
        evs[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return [evs[i].elapsed_time(evs[i + 1]) for i in range(steps)], wall_ms


def median(xs):
    s = sorted(xs)
    return s[len(s) // 2] if len(s) % 2 else 0.5 * (s[len(s) // 2 - 1] + s[len(s) // 2])


# ---- CPU baseline -------------------------------------------------------------------------------------
def cpu_baseline_dense(cfg, target_s=12.0):
    """The oracle's attention_math (the reference's unfused torch path restated) on single heads of
    the benchmark shape: blocks of 4096 query rows against the full key/value sequence until about
    ``target_s`` seconds of CPU work have been timed; throughput in TFLOP/s over that sample."""
    import torch
    from oracle.attention import attention_math_rows
    g = torch.Generator().manual_seed(0)
    s, d = cfg["S"], cfg["D"]
    k = (torch.randn(1, 1, s, d, generator=g) * 0.5).to(torch.bfloat16)
    v = (torch.randn(1, 1, s, d, generator=g) * 0.5).to(torch.bfloat16)
    rows_blk = 4096
    q = (torch.randn(1, 1, rows_blk, d, generator=g) * 0.5).to(torch.bfloat16)
    attention_math_rows(q[:, :, :256], k, v, d ** -0.5, row_chunk=256)   # warm the thread pool
    rows, t0 = 0, time.perf_counter()
    while True:
        attention_math_rows(q, k, v, d ** -0.5, row_chunk=512)
        rows += rows_blk
        dt = time.perf_counter() - t0
        if dt >= target_s or rows >= 40 * s:
            break
    flops = 4.0 * rows * s * d
    return {
        "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"oracle attention_math, one head at a time, {rows} query rows x {s} keys of the benchmark shape "
                  f"({rows / s:.2f} heads of 40), {dt:.1f} s on {os.cpu_count()} visible CPUs "
                  f"(torch threads {torch.get_num_threads()})",
    }


def cpu_baseline_sparse(cfg, device, target_s=8.0):
    """The oracle's RainFusion pipeline on ONE head of the 14B 720p workload: window permutation + block means +
    mask for the whole head, then the block-sparse attention of the first query blocks until about ``target_s``
    seconds are spent; dense-equivalent TFLOP/s over the attended rows (permutation and mask time included
    pro rata)."""
    import torch
    from oracle import rainfusion as orf
    from oracle.attention import block_sparse_attention
    one = dict(cfg, N=1)
    q, k, v = (t.cpu() for t in smooth_field_inputs(one, device, seed=3))
    s, d, grid = cfg["S"], cfg["D"], cfg["grid"]
    t0 = time.perf_counter()
    q_, k_, v_, pool = orf.do_tensor_rearrange_pooling(q, k, v, 0, 128, grid, grid, "BNSD")
    mask = orf.get_blockwise_mask(pool, 0, 0.75, d ** -0.5, 128, grid, grid, "BNSD", return_binary=True,
                                  keep_diagonal=True)
    prep = time.perf_counter() - t0
    nb = mask.shape[-2]
    blocks, t1 = 0, time.perf_counter()
    while blocks < nb and time.perf_counter() - t1 < target_s:
        r = min(8, nb - blocks)
        block_sparse_attention(q_[:, :, blocks * 128:(blocks + r) * 128], k_, v_, mask[:, :, blocks:blocks + r],
                               scale=d ** -0.5)
        blocks += r
    att = time.perf_counter() - t1
    rows = min(blocks * 128, s)
    dt = att + prep * rows / s
    return {"value": 4.0 * rows * s * d / dt / 1e12, "unit": "TFLOP/s (dense-equivalent)",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle rf_v3 pipeline, one head of 40: permutation + block means + mask of the whole head "
                      f"({prep:.1f} s, charged pro rata) and block-sparse attention of the first {blocks} of {nb} "
                      f"query blocks ({att:.1f} s), mask density {float(mask.float().mean()):.3f}"}


def cpu_baseline_gemm(target_s=8.0):
    """The oracle's MXFP8 GEMM + SwiGLU (quantise, dequantise, fp64 product) on row and column slices of the FFN
    shape: 512 tokens x K=5120 x 2x1024 output columns per pass."""
    import torch
    from oracle.quant import mxfp8_gemm_swiglu
    g = torch.Generator().manual_seed(5)
    kdim, rows, cols = CFG_FFN["K"], 512, 1024
    w = (torch.randn((2 * cols, kdim), generator=g) * 0.02).to(torch.bfloat16)
    passes, t0 = 0, time.perf_counter()
    while True:
        x = torch.randn((rows, kdim), generator=g).to(torch.bfloat16)
        mxfp8_gemm_swiglu(x, w)
        passes += 1
        dt = time.perf_counter() - t0
        if dt >= target_s:
            break
    flops = 2.0 * rows * kdim * 2 * cols * passes
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle mxfp8_gemm_swiglu, {passes} passes of {rows} tokens x K={kdim} x 2x{cols} columns "
                      f"(weights re-quantised every pass, as the oracle does), {dt:.1f} s"}


# ---- extras ---------------------------------------------------------------------------------------------
def extra_dense_1p3b(device, steps, warmup):
    import mindiesd
    q, k, v = dense_inputs(CFG_1P3B, device, seed=2)
    ms, _ = time_steps(lambda: mindiesd.attention_forward(q, k, v, head_first=True), steps, warmup)
    m = median(ms)
    return {"workload": "dense bf16 B1 N12 S32760 D128", "ms": m, "tflops": attn_flops(CFG_1P3B) / m / 1e9,
            "frac_of_bf16_peak": attn_flops(CFG_1P3B) / m / 1e9 / PEAK_BF16_TFLOPS}


def extra_head_dims(device, steps, warmup):
    """Dense attention at head dims other than 128 at a 17776-token sequence: 64 (its own kernel), 72 and 96 (computed
    as head_dim 128 on the dense kernel) and 256 (its own kernel of the same design)."""
    import torch
    import mindiesd
    res = {"workload": "dense bf16 B1 S17776 (13x30x45 latent tokens + 226 text tokens), N48 D64 / N48 D72 / N32 D96 / N12 D256"}
    for n, d in ((48, 64), (48, 72), (32, 96), (12, 256)):
        g = torch.Generator(device=device).manual_seed(7)
        q, k, v = ((torch.randn((1, n, 17776, d), device=device, generator=g) * 0.5).to(torch.bfloat16) for _ in range(3))
        ms, _ = time_steps(lambda: mindiesd.attention_forward(q, k, v, head_first=True), steps, warmup)
        m = median(ms)
        res[f"d{d}_ms"] = m
        res[f"d{d}_tflops"] = 4.0 * n * 17776 * 17776 * d / m / 1e9
        res[f"d{d}_frac_of_bf16_peak"] = res[f"d{d}_tflops"] / PEAK_BF16_TFLOPS
    return res


def extra_mid_size_grids(device, steps, warmup):
    """Dense calls whose grid fills the 256 CUs badly as 256-row workgroups (few heads, a few thousand tokens): the
    entry point runs them as 128-row workgroups; both choices timed (MINDIESD_DENSE_TILE_ROWS forces either)."""
    import os
    import torch
    import mindiesd
    res = {"workload": "dense bf16 B1: N16 S2048 D128, N24 S3072 D128, N16 S4608 D128, N24 S4096 D64 "
                       "(128, 288, 288 and 384 workgroups of 256 rows)"}
    keep = os.environ.get("MINDIESD_DENSE_TILE_ROWS")
    try:
        for n, s, d in ((16, 2048, 128), (24, 3072, 128), (16, 4608, 128), (24, 4096, 64)):
            g = torch.Generator(device=device).manual_seed(13)
            q, k, v = ((torch.randn((1, n, s, d), device=device, generator=g) * 0.5).to(torch.bfloat16) for _ in range(3))
            for rows in ("auto", "256"):
                os.environ.pop("MINDIESD_DENSE_TILE_ROWS", None)
                if rows != "auto":
                    os.environ["MINDIESD_DENSE_TILE_ROWS"] = rows
                ms, _ = time_steps(lambda: mindiesd.attention_forward(q, k, v, head_first=True), max(steps, 10), max(warmup, 3))
                m = median(ms)
                key = f"n{n}_s{s}_d{d}" + ("" if rows == "auto" else "_256_rows_forced")
                res[key + "_us"] = 1e3 * m
                res[key + "_tflops"] = 4.0 * n * s * s * d / m / 1e9
    finally:
        os.environ.pop("MINDIESD_DENSE_TILE_ROWS", None)
        if keep is not None:
            os.environ["MINDIESD_DENSE_TILE_ROWS"] = keep
    return res


def extra_cross_attention(device, steps, warmup):
    """Dense attention of the 720p video tokens over a short text (few key tiles per query tile: the launch is
    mostly reading Q and writing O)."""
    import torch
    import mindiesd
    cfg = CFG_14B_720P
    n, s, d = cfg["N"], cfg["S"], cfg["D"]
    g = torch.Generator(device=device).manual_seed(11)
    q = (torch.randn((1, n, s, d), device=device, generator=g) * 0.5).to(torch.bfloat16)
    res = {"workload": f"dense bf16 B1 N{n} Sq{s} D{d} over 226 / 512 keys",
           "q_plus_out_gb": 2.0 * n * s * d * 2 / 1e9}
    for skv in (226, 512):
        k, v = ((torch.randn((1, n, skv, d), device=device, generator=g) * 0.5).to(torch.bfloat16) for _ in range(2))
        ms, _ = time_steps(lambda: mindiesd.attention_forward(q, k, v, head_first=True), steps, warmup)
        m = median(ms)
        res[f"skv{skv}_ms"] = m
        res[f"skv{skv}_tflops"] = 4.0 * n * s * skv * d / m / 1e9
        res[f"skv{skv}_frac_of_hbm_peak"] = res["q_plus_out_gb"] / m * 1e3 / PEAK_HBM_GBS
    return res


def extra_causal_varlen(device, steps, warmup):
    """General mode of the dense kernel at the 1.3B shape: bottom-right causal mask (about half of the
    score matrix is skipped) and the same tokens packed as 7 sequences of unequal length."""
    import torch
    import mindiesd
    from mindiesd.layers.flash_attn.hip_flash_attn import flash_attention
    cfg = CFG_1P3B
    q, k, v = dense_inputs(cfg, device, seed=2)
    s, n, d = cfg["S"], cfg["N"], cfg["D"]
    c_ms, _ = time_steps(lambda: flash_attention(q, k, v, d ** -0.5, "BNSD", causal=True), steps, warmup)
    lens = [8192, 4096, 300, 12000, 1, 5000, s - 29589]
    cu = torch.tensor([0] + lens).cumsum(0).tolist()
    qt, kt, vt = (t[0].transpose(0, 1).contiguous() for t in (q, k, v))
    v_ms, _ = time_steps(lambda: mindiesd.attention_forward_varlen(qt, kt, vt, cu, cu), steps, warmup)
    # many short sequences, cumulative lengths as host lists and as device tensors (no host read-back of the lengths)
    nseq, slen = 63, 512
    cu_s = [i * slen for i in range(nseq + 1)]
    cu_d = torch.tensor(cu_s, dtype=torch.int32, device=device)
    qp, kp, vp = (t[:nseq * slen] for t in (qt, kt, vt))
    h_ms, _ = time_steps(lambda: mindiesd.attention_forward_varlen(qp, kp, vp, cu_s, cu_s), steps, warmup)
    d_ms, _ = time_steps(lambda: mindiesd.attention_forward_varlen(qp, kp, vp, cu_d, cu_d), steps, warmup)
    # boolean masks, all true (timing of the mask path itself): one row shared by all queries, and a full [S, S] one
    pad = torch.ones(1, 1, 1, s, dtype=torch.bool, device=device).expand(1, 1, s, s)
    p_ms, _ = time_steps(lambda: flash_attention(q, k, v, d ** -0.5, "BNSD", attn_mask=pad), steps, warmup)
    full = torch.ones(s, s, dtype=torch.bool, device=device)
    f_ms, _ = time_steps(lambda: flash_attention(q, k, v, d ** -0.5, "BNSD", attn_mask=full), steps, warmup)
    del full
    cm, vm = median(c_ms), median(v_ms)
    causal_flops = 4.0 * n * d * (s * (s + 1) / 2)
    varlen_flops = 4.0 * n * d * sum(l * l for l in lens)
    return {"workload": "bf16 B1 N12 S32760 D128: causal; and packed as 7 sequences " + str(lens),
            "causal_ms": cm, "causal_tflops_unmasked_work": causal_flops / cm / 1e9,
            "varlen_ms": vm, "varlen_tflops": varlen_flops / vm / 1e9,
            "packed_63x512_host_lists_ms": median(h_ms), "packed_63x512_device_cu_seqlens_ms": median(d_ms),
            "key_padding_mask_ms": median(p_ms), "full_mask_ms": median(f_ms),
            "full_mask_tflops": attn_flops(cfg) / median(f_ms) / 1e9}


def extra_sparse(device, steps, warmup, dense_ms):
    """RainFusion block-sparse attention at the 14B 720p shape: top 25 % of key blocks per query
    block + first-frame blocks + diagonal.  Reported with the whole pipeline (permute + pool + mask +
    attention + inverse permute) and with a cached mask (permute + attention + inverse permute)."""
    import torch
    from mindiesd.layers.flash_attn import rainfusion as rf
    cfg = CFG_14B_720P
    q, k, v = smooth_field_inputs(cfg, device, seed=3)
    args = dict(latent_shape_q=cfg["grid"], sparsity=0.75, input_layout="BNSD", keep_diagonal=True)
    out, mask = rf.bsa_sparse_attention_v3(q, k, v, **args)
    density = float(mask.float().mean())
    full_ms, _ = time_steps(lambda: rf.bsa_sparse_attention_v3(q, k, v, **args), steps, warmup)
    cached_ms, _ = time_steps(lambda: rf.bsa_sparse_attention_v3(q, k, v, cached_mask=mask, **args), steps, warmup)
    # attention kernel alone on already permuted tensors and prebuilt lists
    q_, k_, v_, pool = rf.do_tensor_rearrange_pooling(q, k, v, 0, 128, cfg["grid"], cfg["grid"], "BNSD")
    kern_ms, _ = time_steps(lambda: rf.block_sparse_attention_mask(q_, k_, v_, mask, cfg["D"] ** -0.5, "BNSD"),
                            steps, warmup)
    idx, cnt = rf.mask_to_lists(mask)
    list_ms, _ = time_steps(lambda: rf.block_sparse_attention_lists(q_, k_, v_, idx, cnt, cfg["D"] ** -0.5, "BNSD"),
                            steps, warmup)
    mask_ms, _ = time_steps(lambda: rf.get_blockwise_mask(pool, 0, 0.75, cfg["D"] ** -0.5, 128, cfg["grid"],
                                                          cfg["grid"], "BNSD", return_binary=True,
                                                          keep_diagonal=True), steps, warmup)
    perm_ms, _ = time_steps(lambda: rf.do_tensor_rearrange_pooling(q, k, v, 0, 128, cfg["grid"], cfg["grid"], "BNSD"),
                            steps, warmup)
    # the same pipeline with the top 25 % of the key blocks alone (no forced first-frame / diagonal blocks)
    args25 = dict(latent_shape_q=cfg["grid"], sparsity=0.75, input_layout="BNSD", keep_diagonal=False,
                  protect_first_frame=False)
    out, mask25 = rf.bsa_sparse_attention_v3(q, k, v, **args25)
    density25 = float(mask25.float().mean())
    full25_ms, _ = time_steps(lambda: rf.bsa_sparse_attention_v3(q, k, v, **args25), steps, warmup)
    kern25_ms, _ = time_steps(lambda: rf.block_sparse_attention_mask(q_, k_, v_, mask25, cfg["D"] ** -0.5, "BNSD"),
                              steps, warmup)
    del out
    torch.cuda.empty_cache()
    f = attn_flops(cfg)
    fm, cm, km = median(full_ms), median(cached_ms), median(kern_ms)
    return {
        "workload": "RainFusion rf_v3 B1 N40 S75600 D128, sparsity 0.75 + first frame + diagonal, smooth-field inputs",
        "mask_density": density,
        "pipeline_ms": fm, "pipeline_dense_equiv_tflops": f / fm / 1e9, "speedup_vs_dense": dense_ms / fm,
        "cached_mask_ms": cm, "cached_mask_speedup_vs_dense": dense_ms / cm,
        "attention_kernel_ms": km, "attention_kernel_tflops_actual": f * density / km / 1e9,
        "attention_kernel_speedup_vs_dense": dense_ms / km,
        "one_pass_list_kernel_ms": median(list_ms),
        # HBM-bound pass: algorithmic bytes = q, k, v read once and written once in window order (+ the pooled blocks)
        "permute_pool_ms": median(perm_ms), "permute_pool_gbs": 6 * 774.144e6 / median(perm_ms) / 1e6,
        "permute_pool_algorithmic_gb": 6 * 0.774144,
        "permute_pool_frac_of_hbm_peak": 6 * 774.144e6 / median(perm_ms) / 1e6 / PEAK_HBM_GBS,
        "mask_ms": median(mask_ms),
        "topk_only_mask_density": density25,
        "topk_only_pipeline_ms": median(full25_ms), "topk_only_speedup_vs_dense": dense_ms / median(full25_ms),
        "topk_only_attention_kernel_ms": median(kern25_ms),
        "topk_only_attention_kernel_speedup_vs_dense": dense_ms / median(kern25_ms),
    }


def extra_ada_bsa(device, steps, warmup, dense_ms):
    """Adaptive block-sparse attention (ada_bsa) at the 14B 720p shape on the smooth-field inputs: mask estimate
    (strided scores + block selection) and attention over the estimated mask."""
    import torch
    from mindiesd.layers.flash_attn import ada_bsa
    cfg = CFG_14B_720P
    q, k, v = smooth_field_inputs(cfg, device, seed=3)
    scale = cfg["D"] ** -0.5
    est = lambda: ada_bsa.sparse_block_estimate(q, k, scale_value=scale / 8, threshold=0.9, row_sparse=0.25)
    smask, sct = est()
    nb = (cfg["S"] + 127) // 128
    density = float(smask[..., :nb].float().mean())
    est_ms, _ = time_steps(est, steps, warmup)
    att = lambda: ada_bsa.ada_block_sparse_attention(q, k, v, smask, sct, scale_value=scale)
    att_ms, _ = time_steps(att, steps, warmup)
    em, am = median(est_ms), median(att_ms)
    est_flops = 2.0 * cfg["N"] * (cfg["S"] / 8) ** 2 * 8 * cfg["D"]
    return {"workload": "ada_bsa B1 N40 S75600 D128, cdf threshold 0.9, at most 25 % of the key blocks per row, "
                        "smooth-field inputs",
            "mask_density": density, "estimate_ms": em, "estimate_tflops": est_flops / em / 1e9,
            "attention_ms": am, "total_ms": em + am, "speedup_vs_dense": dense_ms / (em + am),
            "attention_speedup_vs_dense": dense_ms / am}


def extra_fp8(device, steps, warmup):
    """FP8 attention at the Wan2.1-14B 480p shape vs the bf16 kernel on the same inputs."""
    import torch
    import mindiesd
    from mindiesd.layers.quant import fp8_attention as f8
    from mindiesd.layers.quant.block_quant import _block_quant
    cfg = CFG_14B_480P
    q, k, v = outlier_inputs(cfg, device, seed=4)
    scale = cfg["D"] ** -0.5
    bf16_ms, _ = time_steps(lambda: mindiesd.attention_forward(q, k, v, head_first=True), steps, warmup)
    # default recipe: block scales amax/448, as the reference's block quantisation leaves them
    e2e_ms, _ = time_steps(lambda: f8.fp8_attention_forward(q, k, v), steps, warmup)
    quant = lambda: (_block_quant(q, 128, "BNSD"), _block_quant(k, 128, "BNSD"), f8.quantize_v_per_channel(v))
    (q8, qs), (k8, ks), (v8t, vs) = quant()
    quant_ms, _ = time_steps(quant, steps, warmup)
    kern_ms, _ = time_steps(lambda: f8.fp8_attention_quantized(q8, qs, k8, ks, v8t, vs, scale), steps, warmup)
    out8 = f8.fp8_attention_quantized(q8, qs, k8, ks, v8t, vs, scale)
    out16 = mindiesd.attention_forward(q, k, v, head_first=True)
    cos = float(torch.nn.functional.cosine_similarity(out8.float().flatten(), out16.float().flatten(), dim=0))
    # the older rule for the probabilities (exponential instruction + E4M3 rounding) on the same operands
    xkern_ms, _ = time_steps(lambda: f8.fp8_attention_quantized(q8, qs, k8, ks, v8t, vs, scale, p_rule="exp2"),
                             steps, warmup)
    out8x = f8.fp8_attention_quantized(q8, qs, k8, ks, v8t, vs, scale, p_rule="exp2")
    cos_x = float(torch.nn.functional.cosine_similarity(out8x.float().flatten(), out16.float().flatten(), dim=0))
    cos_lx = float(torch.nn.functional.cosine_similarity(out8x.float().flatten(), out8.float().flatten(), dim=0))
    del q8, k8, out8, out8x
    # the optional recipe: power-of-two block scales, softmax scale folded into the query (log2-domain kernel)
    pre = scale * f8.LOG2E
    (a8, asq), (b8, bsk) = _block_quant(q, 128, "BNSD", pre, True), _block_quant(k, 128, "BNSD", 1.0, True)
    pkern_ms, _ = time_steps(lambda: f8.fp8_attention_quantized(a8, asq, b8, bsk, v8t, vs, scale, log2_domain=True),
                             steps, warmup)
    pe2e_ms, _ = time_steps(lambda: f8.fp8_attention_forward(q, k, v, recipe="pow2"), steps, warmup)
    outp = f8.fp8_attention_quantized(a8, asq, b8, bsk, v8t, vs, scale, log2_domain=True)
    cos_p = float(torch.nn.functional.cosine_similarity(outp.float().flatten(), out16.float().flatten(), dim=0))
    del a8, b8, outp
    # the FP8RotateQuantFA recipe: an orthogonal (Hadamard) rotation of q and k spreads the outliers over the
    # channels before quantisation; here it runs inside the quantisation pass
    from mindiesd.layers.quant.block_quant import _rot_block_quant
    had = torch.ones((1, 1), device=device)
    while had.shape[0] < cfg["D"]:
        had = torch.cat([torch.cat([had, had], 1), torch.cat([had, -had], 1)], 0)
    rot = (had / had.shape[0] ** 0.5).to(torch.bfloat16)
    rot_ms, _ = time_steps(lambda: f8.fp8_attention_forward(q, k, v, q_rot=rot, k_rot=rot), steps, warmup)
    rq_ms, _ = time_steps(lambda: (_rot_block_quant(q, rot, "BNSD"), _rot_block_quant(k, rot, "BNSD")), steps, warmup)
    mm_ms, _ = time_steps(lambda: (_block_quant(torch.matmul(q, rot), 128, "BNSD"),
                                   _block_quant(torch.matmul(k, rot), 128, "BNSD")), steps, warmup)
    out8r = f8.fp8_attention_forward(q, k, v, q_rot=rot, k_rot=rot)
    cos_rot = float(torch.nn.functional.cosine_similarity(out8r.float().flatten(), out16.float().flatten(), dim=0))
    # rotation + power-of-two scales: with the outliers spread, the faster recipe loses no accuracy
    rotp_ms, _ = time_steps(lambda: f8.fp8_attention_forward(q, k, v, q_rot=rot, k_rot=rot, recipe="pow2"), steps, warmup)
    out8r = f8.fp8_attention_forward(q, k, v, q_rot=rot, k_rot=rot, recipe="pow2")
    cos_rotp = float(torch.nn.functional.cosine_similarity(out8r.float().flatten(), out16.float().flatten(), dim=0))
    f = attn_flops(cfg)
    bm, km, qm, em = median(bf16_ms), median(kern_ms), median(quant_ms), median(e2e_ms)
    # quantisation pass: read q, k once and v twice (maximum, then quantise), write one byte per element
    quant_bytes = (4 * 2 + 3 * 1) * cfg["N"] * cfg["S"] * cfg["D"]
    alg_bytes = (3 * 2 + 3 * 1) * cfg["N"] * cfg["S"] * cfg["D"]
    return {"workload": "FP8 attention B1 N40 S32760 D128, N(0,1) with 1% x8 outliers; Q,K per-128-token scales "
                        "(amax/448), V per-channel, P e4m3 per tile (linear code rule)",
            "bf16_ms": bm, "bf16_tflops": f / bm / 1e9,
            "fp8_kernel_ms": km, "fp8_kernel_tflops": f / km / 1e9, "fp8_kernel_frac_of_fp8_peak": f / km / 1e9 / PEAK_FP8_TFLOPS,
            "fp8_kernel_speedup_vs_bf16": bm / km,
            # HBM-bound pass.  quant_pass_gbs counts what the kernels move (V is read twice: maximum, then codes);
            # the roofline fraction prices the algorithmic bytes: q, k, v read once, one byte per element written
            "quant_pass_ms": qm, "quant_pass_gbs": quant_bytes / qm / 1e6,
            "quant_pass_algorithmic_gb": alg_bytes / 1e9,
            "quant_pass_frac_of_hbm_peak": alg_bytes / qm / 1e6 / PEAK_HBM_GBS,
            "fp8_end_to_end_ms": em, "fp8_end_to_end_speedup_vs_bf16": bm / em,
            "cosine_fp8_vs_unquantised_bf16_kernel": cos,
            "exp2_rule_kernel_ms": median(xkern_ms), "exp2_rule_kernel_speedup_vs_bf16": bm / median(xkern_ms),
            "exp2_rule_cosine_vs_unquantised_bf16_kernel": cos_x, "cosine_linear_rule_vs_exp2_rule": cos_lx,
            "pow2_recipe_kernel_ms": median(pkern_ms), "pow2_recipe_kernel_speedup_vs_bf16": bm / median(pkern_ms),
            "pow2_recipe_end_to_end_ms": median(pe2e_ms), "pow2_recipe_end_to_end_speedup_vs_bf16": bm / median(pe2e_ms),
            "pow2_recipe_cosine_vs_unquantised_bf16_kernel": cos_p,
            "rotated_end_to_end_ms": median(rot_ms), "rotated_end_to_end_speedup_vs_bf16": bm / median(rot_ms),
            "rotate_quant_qk_fused_ms": median(rq_ms), "rotate_quant_qk_matmul_then_quant_ms": median(mm_ms),
            # q and k read once (2 B), one code byte written per element
            "rotate_quant_qk_frac_of_hbm_peak": 2 * 3 * cfg["N"] * cfg["S"] * cfg["D"] / median(rq_ms) / 1e6 / PEAK_HBM_GBS,
            "cosine_rotated_fp8_vs_unquantised_bf16_kernel": cos_rot,
            "rotated_pow2_end_to_end_ms": median(rotp_ms), "rotated_pow2_end_to_end_speedup_vs_bf16": bm / median(rotp_ms),
            "cosine_rotated_pow2_fp8_vs_unquantised_bf16_kernel": cos_rotp}


def extra_gemm(device, steps, warmup):
    """MXFP8 GEMM + SwiGLU of the DiT FFN up-projection."""
    import torch
    from mindiesd.layers.quant import mx_quantize, mxfp8_matmul
    m, k, f = CFG_FFN["M"], CFG_FFN["K"], CFG_FFN["N"]
    g = torch.Generator(device=device).manual_seed(5)
    x = torch.randn((m, k), generator=g, device=device).to(torch.bfloat16)
    w = (torch.randn((2 * f, k), generator=g, device=device) * 0.02).to(torch.bfloat16)
    wq, ws = mx_quantize(w)
    del w
    xq, xs = mx_quantize(x)
    gemm_ms, _ = time_steps(lambda: mxfp8_matmul(xq, xs, wq, ws, None, torch.bfloat16, swiglu=True), steps, warmup)
    quant_ms, _ = time_steps(lambda: mx_quantize(x), steps, warmup)
    flops = 2.0 * m * k * 2 * f
    gm, qm = median(gemm_ms), median(quant_ms)
    return {"workload": "MXFP8 GEMM + SwiGLU M32760 K5120 N2x13824, x N(0,1), w N(0,0.02)",
            "gemm_ms": gm, "gemm_tflops": flops / gm / 1e9, "gemm_frac_of_fp8_peak": flops / gm / 1e9 / PEAK_FP8_TFLOPS,
            "act_quant_ms": qm, "act_quant_gbs": (m * k * 3 + m * k / 32) / qm / 1e6,
            "act_quant_algorithmic_gb": (m * k * 3 + m * k / 32) / 1e9,
            "act_quant_frac_of_hbm_peak": (m * k * 3 + m * k / 32) / qm / 1e6 / PEAK_HBM_GBS,
            "with_act_quant_ms": gm + qm}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (reference kernel for scaling rocprof byte counters)")
    ap.add_argument("--extras-only", default="",
                    help="comma separated subset of extras to run (dense_wan1p3b,head_dims,cross_attention,causal_varlen,sparse_rf_v3,ada_bsa,fp8_attention,"
                         "mxfp8_gemm_swiglu)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs one GPU's share of the attention path on ONE MI355X; "
              "--gpus must be 1 (no collectives or sharding are part of it).", file=sys.stderr)
        sys.exit(2)

    import torch
    import mindiesd
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.calib_copy:
        src = torch.zeros(1 << 28, dtype=torch.float32, device=device)   # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    cfg = CFG_14B_720P
    q, k, v = dense_inputs(cfg, device, seed=1)
    step = lambda: mindiesd.attention_forward(q, k, v, head_first=True)
    ms, wall_ms = time_steps(step, args.steps, args.warmup)
    del q, k, v
    torch.cuda.empty_cache()
    ms_per_step = wall_ms / args.steps          # whole-job figure: wall clock of the timed region
    kernel_ms = sum(ms) / len(ms)               # average launch duration from HIP events
    flops = attn_flops(cfg)
    value = flops / ms_per_step / 1e9
    achieved = flops / kernel_ms / 1e9

    result = {
        "metric": "attn fwd TFLOPS (dense-equiv) + ms at Wan2.1-14B 720p shape; % of MFMA peak",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "dense bf16 flash-attention forward, B=1 N=40 S=75600 (21x45x80) D=128, non-causal, "
                               "BNSD, q/k/v = 0.5*N(0,1) seeded"},
        "pct_of_bf16_mfma_peak": 100.0 * value / PEAK_BF16_TFLOPS,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / PEAK_BF16_TFLOPS, "traffic": dense_traffic_bytes(),
                     "traffic_source": "read from profiles/fa_fwd_dense_bf16_wan14b_720p.md: rocprofv3 --pmc FETCH_SIZE / "
                                       "WRITE_SIZE of this launch, scaled by a 1 GiB copy; not re-measured per run",
                     "kernel": "fa_fwd16_kernel<bf16, 8 waves x 32 rows, 128-key tiles>",
                     "algorithmic_flops_per_launch": flops, "avg_launch_ms": kernel_ms},
    }
    if not args.no_extras:
        extras = {}
        for name, fn in (("dense_wan1p3b", lambda: extra_dense_1p3b(device, args.steps, args.warmup)),
                         ("head_dims", lambda: extra_head_dims(device, args.steps, args.warmup)),
                         ("mid_size_grids", lambda: extra_mid_size_grids(device, args.steps, args.warmup)),
                         ("cross_attention", lambda: extra_cross_attention(device, args.steps, args.warmup)),
                         ("causal_varlen", lambda: extra_causal_varlen(device, args.steps, args.warmup)),
                         ("sparse_rf_v3", lambda: extra_sparse(device, args.steps, args.warmup, kernel_ms)),
                         ("ada_bsa", lambda: extra_ada_bsa(device, args.steps, args.warmup, kernel_ms)),
                         ("fp8_attention", lambda: extra_fp8(device, args.steps, args.warmup)),
                         ("mxfp8_gemm_swiglu", lambda: extra_gemm(device, args.steps, args.warmup))):
            if args.extras_only and name not in args.extras_only.split(","):
                continue
            try:
                extras[name] = fn()
            except Exception as e:  # an extra must never cost the main line
                extras[name] = {"error": f"{type(e).__name__}: {e}"}
        result["extras"] = extras
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline_dense(cfg)
        # the same for the other workloads of the path, next to their GPU figures
        for name, fn in (("sparse_rf_v3", lambda: cpu_baseline_sparse(cfg, device)),
                         ("mxfp8_gemm_swiglu", cpu_baseline_gemm)):
            if name in result.get("extras", {}) and "error" not in result["extras"][name]:
                try:
                    result["extras"][name]["cpu_baseline"] = fn()
                except Exception as e:
                    result["extras"][name]["cpu_baseline"] = {"error": f"{type(e).__name__}: {e}"}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
