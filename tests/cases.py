"""Seeded synthetic inputs shared by the tests, the smoke check and the benchmark.

Everything is drawn on the CPU from torch.Generator().manual_seed(seed), so the CPU oracle
and the GPU path see identical bits after `.to(device)`."""

import math

import torch

OLMOE = dict(E=64, k=8, H=2048, I=1024)


def layer(N, E=64, k=8, H=2048, I=1024, seed=0, dtype=torch.float16, wstd=0.02):
    """The benchmark recipe: h ~ N(0,1); router, gate_up, down ~ N(0, wstd)."""
    g = torch.Generator().manual_seed(seed)
    router = (torch.randn(E, H, generator=g) * wstd).to(dtype)
    gate_up = (torch.randn(E, 2 * I, H, generator=g) * wstd).to(dtype)
    down = (torch.randn(E, H, I, generator=g) * wstd).to(dtype)
    h = torch.randn(N, H, generator=torch.Generator().manual_seed(seed + 1000 + N)).to(dtype)
    return h, router, gate_up, down


def unit_layer(N, E=64, k=8, H=256, I=128, seed=0, skew=0.0, dtype=torch.float16):
    """The reference's kernel-test recipe (tests/test_kernels_cuda.py:11-18): unit-variance
    projections, router * 0.2, `skew` added to the first E/8 routers' weights."""
    g = torch.Generator().manual_seed(seed)
    h = torch.randn(N, H, generator=g).to(dtype)
    router = torch.randn(E, H, generator=g) * 0.2
    router[: max(1, E // 8)] += skew
    gate_up = (torch.randn(E, 2 * I, H, generator=g) * H ** -0.5).to(dtype)
    down = (torch.randn(E, H, I, generator=g) * I ** -0.5).to(dtype)
    return h, router.to(dtype), gate_up, down


def zipf_bias(E=64, s=1.1, alpha=1.0, seed=1):
    """Per-expert logit bias alpha * (-s * ln(rank)), rank a fixed permutation of 1..E."""
    rank = torch.randperm(E, generator=torch.Generator().manual_seed(seed)) + 1
    return -alpha * s * torch.log(rank.float())


def adversarial_bias(E=64, k=8):
    """Every token picks exactly experts 0..k-1."""
    b = torch.zeros(E)
    b[:k] = 100.0
    return b


def expected_used(N, E=64, k=8):
    return E * (1.0 - (1.0 - k / E) ** N)


def weight_bytes(used, H=2048, I=1024):
    return used * 3 * H * I * 2


def layer_flops(M, H=2048, I=1024):
    return M * 6 * H * I


def golden_sort_vector():
    """The reference's own known-answer vector for sort_by_expert (tests/golden/README.md)."""
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "sort_by_expert_reference_vector.json")) as f:
        return json.load(f)
