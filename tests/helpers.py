"""Shared helpers of the parity tests: seeded inputs of the benchmark configs,
and the comparison of one kernel result with the CPU oracle."""
from __future__ import annotations

import sys

import numpy as np
import torch

from oracle import compare as C

E4M3 = torch.float8_e4m3fn
E5M2 = torch.float8_e5m2


def announce(*what):
    """Name the case before it touches the GPU (a faulting run returns only the
    tail of its output)."""
    print("[case]", *what, flush=True)
    sys.stdout.flush()


def gen(seed):
    return torch.Generator().manual_seed(seed)


def randn_bf16(g, *shape, scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def gamma_bf16(g, n):
    return (1.0 + 0.1 * torch.randn(n, generator=g)).to(torch.bfloat16)


def zipf_counts(total, n_experts, seed, n_empty=4, s=1.1):
    """Per-expert row counts: multinomial over a Zipf(s) popularity with the
    n_empty least popular experts forced to zero."""
    rng = np.random.default_rng(seed)
    p = np.arange(1, n_experts + 1, dtype=np.float64) ** (-s)
    if n_empty:
        p[-n_empty:] = 0.0
    p /= p.sum()
    perm = rng.permutation(n_experts)
    counts = np.zeros(n_experts, dtype=np.int64)
    counts[perm] = rng.multinomial(total, p)
    return [int(c) for c in counts]


def check_quant_pair(name, ref_codes, ref_scales, got_codes, got_scales, *, scale_max_ulp=1,
                     scale_min_within1=1.0, min_identical=0.9999, max_step=1, truth=None, bound=None):
    """truth / bound: fp64 scales and their fp32 error bounds (tests/truth.py), in the
    layout of got_scales; see oracle.compare.assert_scales."""
    got_codes = got_codes.detach().cpu()
    got_scales = got_scales.detach().cpu()
    srep = C.assert_scales(ref_scales.reshape(-1), got_scales.reshape(-1), name + ".scale",
                           max_ulp=scale_max_ulp, min_within_1ulp=scale_min_within1,
                           truth=truth, bound=bound)
    crep = C.assert_codes(ref_codes.reshape(-1), got_codes.reshape(-1), name + ".codes",
                          min_identical=min_identical, max_step=max_step)
    print(f"[parity] {name}: codes identical {crep.identical}/{crep.total} max_step {crep.max_step}; "
          f"scales exact {srep.exact}/{srep.total} <=1ulp {srep.within_1ulp} max {srep.max_ulp} ulp",
          flush=True)
    return crep, srep
