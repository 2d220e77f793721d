"""Seeded synthetic inputs of the benchmark workloads (shared by bench.py and the full-size GPU tests).

Every generator takes ``cfg`` = dict(B, N, S, D[, grid]) and a torch device and returns BNSD tensors."""
import math

def dense_inputs(cfg, device, seed=0, mul=0.5, dtype=None):
    """q, k, v = mul * N(0,1), BNSD."""
    import torch
    dtype = dtype or torch.bfloat16
    g = torch.Generator(device=device).manual_seed(seed)
    shape = (cfg["B"], cfg["N"], cfg["S"], cfg["D"])
    return tuple((torch.randn(shape, generator=g, device=device, dtype=torch.float32) * mul).to(dtype)
                 for _ in range(3))


def _gauss_kernel(sigma, device):
    import torch
    r = int(math.ceil(3 * sigma))
    x = torch.arange(-r, r + 1, device=device, dtype=torch.float32)
    k = torch.exp(-0.5 * (x / sigma) ** 2)
    return k / k.sum()


def smooth_field_inputs(cfg, device, seed=0, sigma=2.0, noise=0.3, heads=None, dtype=None):
    """q, k, v (BNSD, tokens flattened T-H-W): per (head, channel) an N(0,1) field on the latent grid,
    Gaussian filtered with sigma tokens along T, H and W (separable, zero padded), renormalised to
    unit variance per head, plus ``noise`` * N(0,1).  Block scores are therefore structured."""
    import torch
    import torch.nn.functional as F
    dtype = dtype or torch.bfloat16
    t, h, w = cfg["grid"]
    n, d = (cfg["N"] if heads is None else heads), cfg["D"]
    g = torch.Generator(device=device).manual_seed(seed)
    kern = _gauss_kernel(sigma, device)
    r = kern.numel() // 2
    outs = []
    for _ in range(3):
        heads_out = []
        for _n in range(n):
            f = torch.randn((d, 1, t, h, w), generator=g, device=device)
            f = F.conv3d(f, kern.view(1, 1, -1, 1, 1), padding=(r, 0, 0))
            f = F.conv3d(f, kern.view(1, 1, 1, -1, 1), padding=(0, r, 0))
            f = F.conv3d(f, kern.view(1, 1, 1, 1, -1), padding=(0, 0, r))
            f = f / f.std()
            f = f + noise * torch.randn(f.shape, generator=g, device=device)
            heads_out.append(f.reshape(d, t * h * w).t().to(dtype))
        outs.append(torch.stack(heads_out, 0).unsqueeze(0).contiguous())
    return tuple(outs)


def outlier_inputs(cfg, device, seed=0, dtype=None):
    """q, k, v = N(0,1) with 1 % of the elements (seeded Bernoulli) scaled by 8, BNSD."""
    import torch
    dtype = dtype or torch.bfloat16
    g = torch.Generator(device=device).manual_seed(seed)
    shape = (cfg["B"], cfg["N"], cfg["S"], cfg["D"])
    outs = []
    for _ in range(3):
        x = torch.randn(shape, generator=g, device=device)
        m = torch.rand(shape, generator=g, device=device) < 0.01
        outs.append(torch.where(m, x * 8, x).to(dtype))
    return tuple(outs)
