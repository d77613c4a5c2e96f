"""Seeded synthetic K/V tensors with the shapes and statistics of the benchmark configurations.

Generated in fp32 on the CPU and cast to fp16, so every run (CPU oracle, GPU kernels) sees the same bits.
Layout is the kernel path's [T, B, H, D] (models/cache/kvcomp_encode.py:83)."""
import numpy as np
import torch

SEED_K, SEED_V, SEED_Q, SEED_OUTLIER, SEED_MASK = 1234, 1235, 1236, 1237, 1238


def synth_k(T, B, H, D, seed=SEED_K):
    """N(0,1) times per-(head, channel) log-normal(0, 0.5) scales, 4 outlier channels per head x20."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(T, B, H, D, generator=g, dtype=torch.float32)
    c = torch.exp(0.5 * torch.randn(H, D, generator=g, dtype=torch.float32))
    go = torch.Generator(device="cpu").manual_seed(SEED_OUTLIER)
    for h in range(H):
        idx = torch.randperm(D, generator=go)[:4]
        c[h, idx] *= 20.0
    return (x * c.view(1, 1, H, D)).to(torch.float16)


def synth_v(T, B, H, D, seed=SEED_V):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(T, B, H, D, generator=g, dtype=torch.float32).to(torch.float16)


def synth_laplace(T, B, H, D, seed):
    """Laplace(0,1) with 2% of the entries multiplied by 50 (long-context stress configuration)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    u = torch.rand(T, B, H, D, generator=g, dtype=torch.float32) - 0.5
    x = -torch.sign(u) * torch.log1p(-2.0 * u.abs().clamp(max=0.4999999))
    gm = torch.Generator(device="cpu").manual_seed(SEED_MASK + seed)
    m = torch.rand(T, B, H, D, generator=gm) < 0.02
    return torch.where(m, x * 50.0, x).to(torch.float16)


def synth_q(B, Hq, D, seed=SEED_Q):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(B, Hq, D, generator=g, dtype=torch.float32).to(torch.float16)


def synth_p(B, Hq, T, seed=SEED_Q + 7):
    """softmax(2.5 * randn) attention weights (kvcomp_cuda_extension/scripts/test_py_ctx_v.py:41-48)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.softmax(2.5 * torch.randn(B, Hq, T, generator=g, dtype=torch.float32), dim=-1).to(torch.float16)


def blocked(x, block_size):
    """[T,B,H,D] -> [NB,BS,B,H,D] view (models/cache/kvcomp_encode.py:83)."""
    T, B, H, D = x.shape
    return x.reshape(T // block_size, block_size, B, H, D)


def np16(t):
    return t.contiguous().numpy()
