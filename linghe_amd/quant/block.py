"""Plain 1x128 / 128x1 blockwise quantisers (reference: linghe/quant/block.py
:129-170 and :251-297)."""
from __future__ import annotations

import torch

from .. import _lib


def triton_block_quant(x, block_size=128, round_scale=False, *, fp8_dtype=torch.float8_e4m3fn):
    """
    blockwise quantize x, used for blockwise recipe for weight in megatron
    Args:
        x: input tensor, bf16 [M, N], M and N multiples of 128
        block_size: block wise (128)
        round_scale: whether round scale to power of 2

    Returns:
        - y: quantized tensor, float8_e4m3fn
        - s: quantization scale, float32 [M/128, N/128]
    """
    assert x.is_contiguous()
    assert block_size == 128, "only 128x128 blocks"
    M, N = x.size()
    assert M % 128 == 0 and N % 128 == 0
    _lib.require_device_bf16(x, "x")
    y = torch.empty((M, N), dtype=fp8_dtype, device=x.device)
    s = torch.empty(M // block_size, N // block_size, dtype=torch.float32, device=x.device)
    with _lib.on_device(x.device):
        _lib.check(_lib.lib.fq_block_quant(_lib.ptr(x), _lib.ptr(y), _lib.ptr(s), M, N, int(bool(round_scale)),
                                           _lib.fp8_kind(fp8_dtype), _lib.stream_of(x)))
    return y, s


def triton_blockwise_quant(x, round_scale=False, output_mode=2, *, fp8_dtype=torch.float8_e4m3fn):
    """
    blockwise quantization, used in blockwise recipe in megatron
    Args:
        x: input tensor, bf16 [M, N]
        round_scale: whether round scale to power of 2
        output_mode: one of {0, 1, 2}
            0: only output non-transposed quantized tensor
            1: only output transposed quantized tensor
            2: output both

    Returns:
        x_q [M, N], x_scale [N/128, M], xt_q [N, M], xt_scale [ceil(M/128), N]
    """
    M, N = x.shape
    assert M % 16 == 0 and x.is_contiguous()
    assert N % 128 == 0
    assert output_mode in (0, 1, 2)
    _lib.require_device_bf16(x, "x")
    device = x.device
    x_q = torch.empty((M, N), device=device, dtype=fp8_dtype)
    x_scale = torch.empty((N // 128, M), device=device, dtype=torch.float32)
    xt_q = torch.empty((N, M), device=device, dtype=fp8_dtype)
    xt_scale = torch.empty(((M + 127) // 128, N), device=device, dtype=torch.float32)
    if M > 0:
        with _lib.on_device(device):
            _lib.check(_lib.lib.fq_blockwise_quant(
                _lib.ptr(x), _lib.ptr(x_q), _lib.ptr(x_scale), _lib.ptr(xt_q), _lib.ptr(xt_scale), M, N,
                int(bool(round_scale)), output_mode, _lib.fp8_kind(fp8_dtype), _lib.stream_of(x)))
    return x_q, x_scale, xt_q, xt_scale


def triton_batch_blockwise_quant(xs, token_count_per_expert, splits, round_scale=False, *,
                                 fp8_dtype=torch.float8_e4m3fn, plan=None):
    """
    per-expert blockwise quantisation (megatron flex MoE)
    Args:
        xs: [bs, dim] bf16
        token_count_per_expert: device int tensor [n_experts]
        splits: python int list of token_count_per_expert
        round_scale: whether round scale to power of 2
        plan: optional linghe_amd.utils.silu.ExpertPlan built from the same counts

    Returns (flat, per-expert packed):
        x_q [bs, dim], x_scale (bs*dim/128,), xt_q (bs*dim,), xt_scale (blocks*dim,)
    """
    assert xs.is_contiguous()
    _lib.require_device_bf16(xs, "xs")
    M, N = xs.shape
    assert N % 128 == 0
    n_experts = token_count_per_expert.size(0)
    device = xs.device
    x_q = torch.empty((M, N), device=device, dtype=fp8_dtype)
    x_scale = torch.empty((M * N // 128,), device=device, dtype=torch.float32)
    xt_q = torch.empty((M * N,), device=device, dtype=fp8_dtype)
    blocks = sum((int(c) + 127) // 128 for c in splits)
    xt_scale = torch.empty((blocks * N,), device=device, dtype=torch.float32)
    if M == 0:
        return x_q, x_scale, xt_q, xt_scale
    if plan is not None:
        if plan.blocks != blocks or plan.pad != 1 or plan.table.device != device:
            raise ValueError("plan does not belong to these splits / this device")
        with _lib.on_device(device):
            _lib.check(_lib.lib.fq_batched_blockwise_quant_planned(
                _lib.ptr(xs), _lib.ptr(plan.table), plan.shape, _lib.ptr(x_q), _lib.ptr(x_scale), _lib.ptr(xt_q),
                _lib.ptr(xt_scale), M, N, int(bool(round_scale)), _lib.fp8_kind(fp8_dtype), _lib.stream_of(xs)))
        return x_q, x_scale, xt_q, xt_scale
    counts = token_count_per_expert
    if counts.dtype == torch.int64:
        is64 = 1
    elif counts.dtype == torch.int32:
        is64 = 0
    else:
        raise TypeError(f"token_count_per_expert must be int32 or int64, got {counts.dtype}")
    with _lib.on_device(device):
        _lib.check(_lib.lib.fq_batched_blockwise_quant(
            _lib.ptr(xs), _lib.ptr(counts), is64, n_experts, blocks, _lib.ptr(x_q), _lib.ptr(x_scale),
            _lib.ptr(xt_q), _lib.ptr(xt_scale), M, N, int(bool(round_scale)), _lib.fp8_kind(fp8_dtype),
            _lib.stream_of(xs)))
    return x_q, x_scale, xt_q, xt_scale
