"""Seeded synthetic inputs of the benchmark configurations (test infrastructure).

All tensors come from ``torch.Generator().manual_seed(seed)`` on the CPU so the GPU box and this
container build identical data.
"""

from __future__ import annotations

import torch

from .fp8 import quantize_weight_rows

GEMM_SHAPES = ((960, 2560), (720, 2048), (2048, 16384), (16384, 2048), (2048, 2048))  # (K, N)
GEMM_MS = (1, 16, 50, 64)


def shape_seed(m: int, k: int, n: int) -> int:
    return (m * 1_000_003 + k * 10_007 + n) % (2**31 - 1)


def gemm_case(m: int, k: int, n: int, seed: int | None = None):
    """bf16 ``x [M, K] ~ N(0,1)``, ``W [N, K] ~ N(0, 0.02)`` quantised per row -> ``(x, w8, scale)``."""
    g = torch.Generator().manual_seed(shape_seed(m, k, n) if seed is None else seed)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    w = torch.randn(n, k, generator=g) * 0.02
    w8, s = quantize_weight_rows(w)
    return x, w8, s


def ffn_case(m: int = 50, k: int = 720, i: int = 2048, seed: int = 0):
    """Config 1: ``x [50,720]`` bf16, gate/up ``[2048,720]``, down ``[720,2048]`` ~ N(0,0.02), fp8."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16)
    wg = torch.randn(i, k, generator=g) * 0.02
    wu = torch.randn(i, k, generator=g) * 0.02
    wd = torch.randn(k, i, generator=g) * 0.02
    return (x, *quantize_weight_rows(wg), *quantize_weight_rows(wu), *quantize_weight_rows(wd))


def attn_case(m: int = 50, p: int = 241, h: int = 15, g_heads: int = 5, d: int = 64, seed: int = 0, kv_dtype=torch.bfloat16):
    """Config 3: q ``[50,15,64]``, prefix K/V ``[241,5,64]``, suffix K/V ``[50,5,64]``, all ~N(0,1)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(m, h, d, generator=g).to(torch.bfloat16)
    k_pre = torch.randn(p, g_heads, d, generator=g).to(kv_dtype)
    v_pre = torch.randn(p, g_heads, d, generator=g).to(kv_dtype)
    k_suf = torch.randn(m, g_heads, d, generator=g).to(torch.bfloat16)
    v_suf = torch.randn(m, g_heads, d, generator=g).to(torch.bfloat16)
    return q, k_pre, v_pre, k_suf, v_suf
