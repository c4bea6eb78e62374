"""Seeded synthetic inputs shared by the parity tests and the benchmark (CPU generator,
values drawn in fp32 and then cast, as the measurement plan prescribes)."""
import torch


def gen(seed):
    return torch.Generator().manual_seed(seed)


def normal(shape, seed, dtype=torch.bfloat16, std=1.0):
    return (torch.randn(shape, generator=gen(seed)) * std).to(dtype)


def uniform(shape, seed, dtype=torch.bfloat16):
    return torch.rand(shape, generator=gen(seed)).to(dtype)


def normal_with_outliers(shape, seed, dtype=torch.bfloat16, frac=1e-3, factor=100.0):
    g = gen(seed)
    x = torch.randn(shape, generator=g)
    n = x.numel()
    k = max(1, round(frac * n))
    idx = torch.randperm(n, generator=g)[:k]
    flat = x.view(-1)
    flat[idx] *= factor
    return x.to(dtype)


def rows_log_uniform_sigma(shape, seed, dtype=torch.float32):
    g = gen(seed)
    sig = 10 ** (torch.rand(shape[0], 1, generator=g) * 6 - 3)
    return (torch.randn(shape, generator=g) * sig).to(dtype)


def student_t(shape, seed, dtype=torch.bfloat16, df=3):
    g = gen(seed)
    n = torch.randn(shape, generator=g)
    chi = torch.zeros(shape)
    for _ in range(df):
        chi += torch.randn(shape, generator=g) ** 2
    return (n / torch.sqrt(chi / df)).to(dtype)


def codes(t):
    """fp8 / e8m0 tensor -> uint8 codes on the CPU"""
    return t.detach().view(torch.uint8).cpu()
