"""Seeded synthetic inputs of the five benchmark configurations (CPU tensors).

Shared by the parity tests and bench.py so both see identical data.
"""
from __future__ import annotations

import numpy as np
import torch


def _gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(seed)


def gamma_like(g: torch.Generator, n: int) -> torch.Tensor:
    return (1.0 + 0.1 * torch.randn(n, generator=g)).to(torch.bfloat16)


def cfg1_rmsnorm_quant(M: int = 8192, n: int = 2048):
    """RMSNorm + 1x128 e4m3 quant forward: x ~ N(0,1), gamma ~ N(1, 0.1), eps 1e-6."""
    g = _gen(1001)
    x = torch.randn(M, n, generator=g).to(torch.bfloat16)
    return dict(x=x, gamma=gamma_like(g, n), eps=1e-6)


def cfg2_swiglu_fwd(M: int = 8192, n: int = 2048):
    """SwiGLU + quant forward: x ~ N(0,1) [M, 2n] with 0.1 % of the entries x50."""
    g = _gen(1002)
    x = torch.randn(M, 2 * n, generator=g)
    mask = torch.rand(M, 2 * n, generator=g) < 0.001
    x = torch.where(mask, x * 50.0, x).to(torch.bfloat16)
    return dict(x=x)


def zipf_counts(total: int, n_experts: int, seed: int, n_empty: int = 4, s: float = 1.1):
    """Rows per expert: multinomial(total, p) with p a Zipf(s) popularity assigned
    to experts in a seeded random order; the n_empty least popular get p = 0."""
    rng = np.random.default_rng(seed)
    p = np.arange(1, n_experts + 1, dtype=np.float64) ** (-s)
    if n_empty:
        p[-n_empty:] = 0.0
    p /= p.sum()
    perm = rng.permutation(n_experts)
    counts = np.zeros(n_experts, dtype=np.int64)
    counts[perm] = rng.multinomial(total, p)
    return [int(c) for c in counts]


def cfg3_batched_swiglu(tokens: int = 8192, topk: int = 8, n_experts: int = 256, n: int = 512):
    """Batched per-expert SwiGLU + quant: tokens*topk rows over n_experts experts."""
    M = tokens * topk
    counts = zipf_counts(M, n_experts, seed=1003)
    g = _gen(1003)
    x = torch.randn(M, 2 * n, generator=g).to(torch.bfloat16)
    w = torch.rand(M, 1, generator=g)
    dy = (1e-3 * torch.randn(M, n, generator=g)).to(torch.bfloat16)
    return dict(x=x, weight=w, counts=counts, dy=dy)


def cfg4_swiglu_bwd(M: int = 8192, n: int = 2048):
    """SwiGLU + quant backward: g ~ N(0, 1e-3) [M, n], x ~ N(0,1) [M, 2n]."""
    g = _gen(1004)
    dy = (1e-3 * torch.randn(M, n, generator=g)).to(torch.bfloat16)
    x = torch.randn(M, 2 * n, generator=g).to(torch.bfloat16)
    return dict(dy=dy, x=x)


OUTLIER_CHANNELS = (0, 1023, 2047, 3071, 4095, 5119, 6143, 7167)


def cfg5_rmsnorm_large(M: int = 16384, n: int = 7168):
    """RMSNorm backward + forward quant at large hidden: x Student-t(3) with 8
    fixed channels x100, gamma ~ N(1, 0.1), grad ~ N(0, 1e-3)."""
    g = _gen(1005)
    x = torch.empty(M, n, dtype=torch.bfloat16)
    rows = 2048
    for r0 in range(0, M, rows):  # in slabs, to bound host memory
        r1 = min(M, r0 + rows)
        z = torch.randn(r1 - r0, n, generator=g)
        chi = torch.randn(r1 - r0, n, 3, generator=g).pow_(2).sum(-1).div_(3.0).sqrt_()
        t = z / chi
        for c in OUTLIER_CHANNELS:
            if c < n:
                t[:, c] *= 100.0
        x[r0:r1] = t.to(torch.bfloat16)
    gamma = gamma_like(g, n)
    dy = (1e-3 * torch.randn(M, n, generator=g)).to(torch.bfloat16)
    return dict(x=x, gamma=gamma, dy=dy, eps=1e-6)


def next_permute_pad_quant(tokens: int = 16384, n: int = 2048, n_experts: int = 32, topk: int = 2):
    """Gather + pad-to-16 + quant (the step before the expert GEMM; shape of the
    reference's own test, tests/test_gather.py:597): tokens*topk routed rows over
    n_experts experts, Zipf counts with two empty experts, each expert's tokens a
    random subset of the source rows."""
    counts = zipf_counts(tokens * topk, n_experts, seed=1101, n_empty=2)
    g = _gen(1101)
    x = torch.randn(tokens, n, generator=g).to(torch.bfloat16)
    probs = torch.rand(tokens, n_experts, generator=g)
    parts, plain = [], []
    for c in counts:
        pc = (c + 15) // 16 * 16
        src = torch.randint(0, tokens, (c,), generator=g, dtype=torch.int32)
        plain.append(src)
        parts += [src, torch.zeros(pc - c, dtype=torch.int32)]
    return dict(x=x, probs=probs, counts=counts, indices=torch.cat(parts), indices_unpadded=torch.cat(plain))


# algorithmic HBM bytes per call as (bytes read, bytes written): each input read once, each
# output written once; scratch (dgamma / dw partial sums, the re-ordered router weight) is
# not counted
def rw_rmsnorm_quant(M, n, mode=2):
    x = 2 * M * n + 2 * n
    row = M * n + 4 * (n // 128) * M
    col = M * n + 4 * ((M + 127) // 128) * n
    if mode == 0:
        return x, row + 4 * M
    if mode == 1:
        return x + 4 * M, col
    return x, row + col + 4 * M


def rw_swiglu_fwd(M, n, mode=2):
    row = M * n + 4 * (n // 128) * M
    col = M * n + 4 * ((M + 127) // 128) * n
    return 2 * M * 2 * n, (row if mode != 1 else 0) + (col if mode != 0 else 0)


def rw_swiglu_bwd(M, n):
    N = 2 * n
    return 2 * M * n + 2 * M * N, 2 * M * N + 4 * (N // 128) * M + 4 * ((M + 127) // 128) * N


def rw_batched_swiglu_fwd(M, n, counts):
    blocks = sum((c + 127) // 128 for c in counts)
    return 2 * M * 2 * n + 4 * M, 2 * M * n + 4 * M * (n // 128) + 4 * blocks * n


def rw_batched_swiglu_bwd(M, n, counts):
    blocks = sum((c + 127) // 128 for c in counts)
    N = 2 * n
    return 2 * M * n + 2 * M * N + 4 * M, 2 * M * N + 4 * M * (N // 128) + 4 * blocks * N + 4 * M


def rw_rmsnorm_bwd(M, n):
    return 2 * (2 * M * n) + 2 * n, 2 * M * n + 4 * n


def rw_permute_pad_quant(n, counts):
    """each routed row read once (2 B/element) with its index and prob, both code layouts and scales written"""
    routed = sum(counts)
    padded = sum((c + 15) // 16 * 16 for c in counts)
    blocks = sum((c + 127) // 128 for c in counts)
    return (2 * routed * n + 4 * padded + 4 * routed,
            2 * padded * n + 4 * padded * (n // 128) + 4 * blocks * n + 4 * padded)


def rw_weighted_silu(M, n, backward):
    if backward:
        return 2 * M * 2 * n + 2 * M * n + 4 * M, 2 * M * 2 * n + 4 * M
    return 2 * M * 2 * n + 4 * M, 2 * M * n


def rw_block_quant(M, N):
    return 2 * M * N, M * N + 4 * (M // 128) * (N // 128)


def rw_router(M, N, K):
    return 2 * M * K + 2 * N * K + 2 * K, 2 * M * K + M * K + 4 * M * N + 4 * (K // 128) * M + 4 * M


def bytes_rmsnorm_quant(M, n, mode=2):
    return sum(rw_rmsnorm_quant(M, n, mode))


def bytes_swiglu_fwd(M, n):
    return sum(rw_swiglu_fwd(M, n))


def bytes_swiglu_bwd(M, n):
    return sum(rw_swiglu_bwd(M, n))


def bytes_batched_swiglu_fwd(M, n, counts):
    return sum(rw_batched_swiglu_fwd(M, n, counts))


def bytes_batched_swiglu_bwd(M, n, counts):
    return sum(rw_batched_swiglu_bwd(M, n, counts))


def bytes_rmsnorm_bwd(M, n):
    return sum(rw_rmsnorm_bwd(M, n))


def bytes_permute_pad_quant(n, counts):
    return sum(rw_permute_pad_quant(n, counts))
