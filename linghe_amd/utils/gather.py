"""Gather + pad + blockwise-FP8 quant entry point (reference:
linghe/utils/gather.py:960-1113).  Name, argument order, defaults, output
tensors and layouts are the reference's; ``fp8_dtype`` is a keyword-only
extension (the reference always emits e4m3fn).
"""
from __future__ import annotations

import torch

from .. import _lib


def triton_batch_block_pad_permute_with_indices(
    xs, token_count_per_expert, indices, splits, probs=None, round_scale=False, *,
    fp8_dtype=torch.float8_e4m3fn, plan=None
):
    """
    select and quant, used in megatron 0.12 flex moe
    Args:
        xs: [bs, dim] bf16
        token_count_per_expert: device int tensor [n_experts]
        indices: int32 [sum of the counts each rounded up to 16]: expert e's region holds
            the source rows of its tokens followed by padding entries (ignored)
        splits: python int list of token_count_per_expert
        probs: route weights, [bs, n_experts]
        round_scale: whether round scale to power of 2
        plan: optional linghe_amd.utils.silu.ExpertPlan of the same counts built with pad=16

    Returns:
        x_q [M, dim], x_scale [M, dim/128] (per expert [dim/128, padded count]),
        xt_q [M, dim] (per expert [dim, padded count]), xt_scale [blocks, dim],
        prob_output [M] or None
    """
    assert xs.is_contiguous()
    m, N = xs.shape
    assert N % 128 == 0
    _lib.require_device_bf16(xs, "xs")
    n_experts = token_count_per_expert.size(0)
    M = indices.shape[0]
    device = xs.device
    x_q = torch.empty((M, N), device=device, dtype=fp8_dtype)
    x_scale = torch.empty((M, N // 128), device=device, dtype=torch.float32)
    blocks = sum((int(c) + 127) // 128 for c in splits)
    xt_q = torch.empty((M, N), device=device, dtype=fp8_dtype)
    xt_scale = torch.empty((blocks, N), device=device, dtype=torch.float32)
    prob_output = None
    if probs is not None:
        prob_output = torch.empty((M,), device=device, dtype=probs.dtype)
    if m == 0 or M == 0:
        return x_q, x_scale, xt_q, xt_scale, prob_output
    padded = sum((int(c) + 15) // 16 * 16 for c in splits)
    assert M == padded, f"indices holds {M} entries, the counts rounded up to 16 add up to {padded}"
    if indices.dtype != torch.int32:
        raise TypeError(f"indices must be int32, got {indices.dtype}")
    assert indices.is_contiguous() and token_count_per_expert.is_contiguous()
    counts = token_count_per_expert
    if counts.dtype == torch.int64:
        is64 = 1
    elif counts.dtype == torch.int32:
        is64 = 0
    else:
        raise TypeError(f"token_count_per_expert must be int32 or int64, got {counts.dtype}")
    pbf16 = 0
    if probs is not None:
        assert probs.is_contiguous() and probs.shape == (m, n_experts)
        if probs.dtype == torch.bfloat16:
            pbf16 = 1
        elif probs.dtype != torch.float32:
            raise TypeError(f"probs must be float32 or bfloat16, got {probs.dtype}")
    if plan is not None:
        if plan.blocks != blocks or plan.pad != 16 or plan.table.device != device:
            raise ValueError("plan does not belong to these splits / this layout (pad=16) / this device")
        with _lib.on_device(device):
            _lib.check(_lib.lib.fq_batched_pad_permute_quant_planned(
                _lib.ptr(xs), _lib.ptr(plan.table), plan.shape, n_experts, _lib.ptr(indices), _lib.ptr(probs), pbf16,
                _lib.ptr(prob_output), _lib.ptr(x_q), _lib.ptr(x_scale), _lib.ptr(xt_q), _lib.ptr(xt_scale), m, M, N,
                int(bool(round_scale)), _lib.fp8_kind(fp8_dtype), _lib.stream_of(xs)))
        return x_q, x_scale, xt_q, xt_scale, prob_output
    with _lib.on_device(device):
        _lib.check(_lib.lib.fq_batched_pad_permute_quant(
            _lib.ptr(xs), _lib.ptr(counts), is64, n_experts, blocks, _lib.ptr(indices),
            _lib.ptr(probs), pbf16, _lib.ptr(prob_output), _lib.ptr(x_q), _lib.ptr(x_scale), _lib.ptr(xt_q),
            _lib.ptr(xt_scale), m, M, N, int(bool(round_scale)), _lib.fp8_kind(fp8_dtype), _lib.stream_of(xs)))
    return x_q, x_scale, xt_q, xt_scale, prob_output
