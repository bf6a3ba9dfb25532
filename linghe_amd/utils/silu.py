"""SwiGLU + blockwise-FP8 quant entry points (reference: linghe/utils/silu.py
:279-335, :424-464, :797-950, :1293-1393).  Names, argument order, defaults,
output tensors and scale layouts are the reference's; ``fp8_dtype`` is a
keyword-only extension (the reference always emits e4m3fn).
"""
from __future__ import annotations

import torch

from .. import _lib


def _blocks_of(splits) -> int:
    return sum((int(c) + 127) // 128 for c in splits)


class ExpertPlan:
    """Device-side table of the 128-row blocks of one set of per-expert counts.

    The per-expert entry points find each workgroup's tile by a prefix scan over
    ``counts``; handing them a plan (keyword ``plan``) replaces that scan by one
    16-byte read and sizes the launch for exactly the workgroups that have a tile.
    Build it once per set of counts (``build_expert_plan``) and reuse it for every
    per-expert call of the layer: forward, backward, quantiser.  No counterpart in
    the reference, whose kernels are launched on a grid derived from the host-side
    ``splits`` instead.
    """

    __slots__ = ("table", "shape", "blocks", "pad")

    def __init__(self, table: torch.Tensor, shape):
        self.table = table
        self.shape = shape            # ctypes int64[5]: row blocks, whole / halved / quartered ones, pad
        self.blocks = int(shape[0])
        self.pad = int(shape[4])


def build_expert_plan(counts: torch.Tensor, splits, pad: int = 1) -> ExpertPlan:
    """counts: device int32/int64 [n_experts]; splits: the same numbers as a python list;
    pad: 1 for the layouts with the experts back to back (SwiGLU, blockwise quantiser), 16 for
    gather + pad + quant (every expert's region of the outputs rounded up to 16 rows)."""
    import ctypes

    n = len(splits)
    host = (ctypes.c_int64 * max(n, 1))(*[int(c) for c in splits])
    shape = (ctypes.c_int64 * 5)()
    _lib.check(_lib.lib.fq_expert_plan_shape(host, n, pad, shape))
    nbytes = int(_lib.lib.fq_expert_plan_bytes(shape))
    table = torch.empty((max(nbytes, 16),), device=counts.device, dtype=torch.uint8)
    if shape[0]:
        with _lib.on_device(counts.device):
            _lib.check(_lib.lib.fq_build_expert_plan(
                _lib.ptr(counts), _counts_flag(counts), counts.shape[0], shape, _lib.ptr(table),
                _lib.stream_of(counts)))
    return ExpertPlan(table, shape)


def _check_plan(plan: ExpertPlan, blocks: int, device) -> None:
    if plan.blocks != blocks:
        raise ValueError(f"plan was built for {plan.blocks} row blocks, splits give {blocks}")
    if plan.pad != 1:
        raise ValueError("plan was built for the padded layout of gather + pad + quant")
    if plan.table.device != device:
        raise ValueError("plan lives on another device")


def _counts_flag(counts: torch.Tensor) -> int:
    if counts.dtype == torch.int64:
        return 1
    if counts.dtype == torch.int32:
        return 0
    raise TypeError(f"counts must be int32 or int64, got {counts.dtype}")


def _weight_flag(weight: torch.Tensor) -> int:
    if weight.dtype == torch.float32:
        return 0
    if weight.dtype == torch.bfloat16:
        return 1
    raise TypeError(f"weight must be float32 or bfloat16, got {weight.dtype}")


def triton_weighted_silu_forward(x, weight=None, out=None, asm=False):
    """
    compute silu(x)*weight, used in bf16/fp16 training with MoE
    Args:
        x: input tensor, bf16 [M, 2n] (gate | up)
        weight: tokenwise weight [M, 1] or [M], fp32 or bf16
        asm: accepted for compatibility (the reference's alternative exp2 path); ignored
    Returns:
        out: output tensor, bf16 [M, n]
    """
    assert x.is_contiguous()
    _lib.require_device_bf16(x, "x")
    M, N = x.shape
    assert N % 256 == 0
    if out is None:
        out = torch.empty((M, N // 2), device=x.device, dtype=x.dtype)
    wflag = 0
    if weight is not None:
        assert weight.is_contiguous() and weight.numel() == M
        wflag = _weight_flag(weight)
    with _lib.on_device(x.device):
        _lib.check(_lib.lib.fq_swiglu_fwd(_lib.ptr(x), _lib.ptr(weight), wflag, _lib.ptr(out), M, N // 2,
                                          _lib.stream_of(x)))
    return out


def triton_weighted_silu_backward(g, x, weight=None):
    """
    backward of triton_weighted_silu_forward
    Args:
        g: gradient tensor, bf16 [M, n]
        x: input tensor, bf16 [M, 2n]
        weight: weight tensor [M, 1] or [M]

    Returns:
        - dx: gradient of x, bf16 [M, 2n]
        - dw: gradient of weight (weight's shape and dtype), None without weight
    """
    assert g.is_contiguous() and x.is_contiguous()
    _lib.require_device_bf16(x, "x")
    _lib.require_device_bf16(g, "g")
    M, N = x.shape
    assert N % 256 == 0
    assert g.shape == (M, N // 2)
    dw, wflag = None, 0
    if weight is not None:
        assert weight.is_contiguous() and weight.numel() == M
        wflag = _weight_flag(weight)
        dw = torch.empty(weight.shape, device=x.device, dtype=weight.dtype)
    dx = torch.empty((M, N), device=x.device, dtype=x.dtype)
    with _lib.on_device(x.device):
        _lib.check(_lib.lib.fq_swiglu_bwd(_lib.ptr(g), _lib.ptr(x), _lib.ptr(weight), wflag, _lib.ptr(dx),
                                          _lib.ptr(dw), M, N // 2, _lib.stream_of(x)))
    return dx, dw


def triton_silu_and_block_quant_forward(
    x, out=None, scale=None, round_scale=False, output_mode=2, *, fp8_dtype=torch.float8_e4m3fn
):
    """
    fused silu and blockwise quantization, used in shared expert
    Args:
        x: input tensor, bf16 [M, 2n] (gate | up)
        round_scale: whether round scale to power of 2
        output_mode: one of {0, 1, 2}
            0: only output non-transposed quantized tensor
            1: only output transposed quantized tensor
            2: output both

    Returns:
        - out: quantized tensor [M, n]
        - scale: quantization scale [n/128, M]
        - transpose_output: quantized tensor of transposed output [n, M]
        - transpose_scale: quantization scale of transposed output [ceil(M/128), n]
    """
    assert x.is_contiguous()
    _lib.require_device_bf16(x, "x")
    M, N = x.shape
    n = N // 2
    assert output_mode in (0, 1, 2)
    assert n % 128 == 0 and N == 2 * n
    device = x.device
    if out is None:
        out = torch.empty((M, n), device=device, dtype=fp8_dtype)
    if scale is None:
        scale = torch.empty((n // 128, M), device=device, dtype=torch.float32)
    transpose_output = torch.empty((n, M), device=device, dtype=fp8_dtype)
    transpose_scale = torch.empty(((M + 127) // 128, n), device=device, dtype=torch.float32)
    if M > 0:
        with _lib.on_device(device):
            _lib.check(_lib.lib.fq_swiglu_quant_fwd(
                _lib.ptr(x), _lib.ptr(out), _lib.ptr(scale), _lib.ptr(transpose_output),
                _lib.ptr(transpose_scale), M, n, int(bool(round_scale)), output_mode,
                _lib.fp8_kind(fp8_dtype), _lib.stream_of(x)))
    return out, scale, transpose_output, transpose_scale


def triton_silu_and_block_quant_backward(g, x, round_scale=False, *, fp8_dtype=torch.float8_e4m3fn):
    """
    backward of triton_silu_and_block_quant_forward
    Args:
        g: gradient, bf16 [M, n]
        x: input tensor, bf16 [M, 2n]
        round_scale: whether round to power of 2

    Returns:
        - dx: quantized non-transposed gradient [M, 2n]
        - dx_scale: scales of quantization non-transposed gradient [2n/128, M]
        - transpose_dx: quantized transposed gradient [2n, M]
        - transpose_dx_scale: scales of quantization transposed gradient [M/128, 2n]
    """
    assert g.is_contiguous()
    assert x.is_contiguous()
    M, N = x.shape
    n = N // 2
    assert M % 128 == 0 and N % 256 == 0
    assert g.shape == (M, n)
    _lib.require_device_bf16(x, "x")
    _lib.require_device_bf16(g, "g")
    device = x.device
    dx = torch.empty((M, N), device=device, dtype=fp8_dtype)
    dx_scale = torch.empty((N // 128, M), device=device, dtype=torch.float32)
    transpose_dx = torch.empty((N, M), device=device, dtype=fp8_dtype)
    transpose_dx_scale = torch.empty(((M + 127) // 128, N), device=device, dtype=torch.float32)
    if M > 0:
        with _lib.on_device(device):
            _lib.check(_lib.lib.fq_swiglu_quant_bwd(
                _lib.ptr(g), _lib.ptr(x), _lib.ptr(dx), _lib.ptr(dx_scale), _lib.ptr(transpose_dx),
                _lib.ptr(transpose_dx_scale), M, n, int(bool(round_scale)), _lib.fp8_kind(fp8_dtype),
                _lib.stream_of(x)))
    return dx, dx_scale, transpose_dx, transpose_dx_scale


def triton_batch_weighted_silu_and_block_quant_forward(
    x,
    weight,
    counts,
    splits=None,
    out=None,
    scale=None,
    round_scale=False,
    output_mode=2,
    *,
    fp8_dtype=torch.float8_e4m3fn,
    plan=None,
):
    """
    silu and blockwise quantize activation in routed experts
    Args:
        x: activation tensor in routed experts, bf16 [M, 2n]
        weight: router prob tensor [M, 1]
        counts: device tensor of token count per expert
        splits: python int list of token count per expert
        round_scale: whether round scale to power of 2
        output_mode: one of {0, 1, 2}
        plan: optional ExpertPlan built from the same counts (same results, no scan of the counts)

    Returns (per-expert packed layouts):
        - out: quantized tensor [M, n]
        - scale: per expert [n/128, count_e] blocks, allocated [M, n/128]
        - transpose_output: per expert [n, count_e] blocks, allocated [M, n]
        - transpose_scale: [sum ceil(count_e/128), n]
    """
    assert splits is not None, "batch mode need splits to launch kernels"
    assert x.is_contiguous() and weight.is_contiguous()
    _lib.require_device_bf16(x, "x")
    M, N = x.shape
    n = N // 2
    n_experts = counts.shape[0]
    assert N <= 8192
    assert n % 128 == 0 and N == 2 * n
    assert output_mode in (0, 1, 2)
    assert weight.numel() == M
    device = x.device
    if out is None:
        out = torch.empty((M, n), device=device, dtype=fp8_dtype)
    if scale is None:
        scale = torch.empty((M, n // 128), device=device, dtype=torch.float32)
    blocks = _blocks_of(splits)
    transpose_output = torch.empty((M, n), device=device, dtype=fp8_dtype)
    transpose_scale = torch.empty((blocks, n), device=device, dtype=torch.float32)
    if M == 0:
        return out, scale, transpose_output, transpose_scale
    if plan is not None:
        _check_plan(plan, blocks, device)
        with _lib.on_device(device):
            _lib.check(_lib.lib.fq_batched_swiglu_quant_fwd_planned(
                _lib.ptr(x), _lib.ptr(weight), _weight_flag(weight), _lib.ptr(plan.table), plan.shape,
                _lib.ptr(out), _lib.ptr(scale), _lib.ptr(transpose_output), _lib.ptr(transpose_scale), M, n,
                int(bool(round_scale)), output_mode, _lib.fp8_kind(fp8_dtype), _lib.stream_of(x)))
        return out, scale, transpose_output, transpose_scale
    with _lib.on_device(device):
        _lib.check(_lib.lib.fq_batched_swiglu_quant_fwd(
            _lib.ptr(x), _lib.ptr(weight), _weight_flag(weight), _lib.ptr(counts), _counts_flag(counts),
            n_experts, blocks, _lib.ptr(out), _lib.ptr(scale), _lib.ptr(transpose_output),
            _lib.ptr(transpose_scale), M, n, int(bool(round_scale)), output_mode,
            _lib.fp8_kind(fp8_dtype), _lib.stream_of(x)))
    return out, scale, transpose_output, transpose_scale


def triton_batch_weighted_silu_and_block_quant_backward(
    g, x, weight, counts, splits=None, round_scale=False, *, fp8_dtype=torch.float8_e4m3fn, plan=None
):
    """
    backward of triton_batch_weighted_silu_and_block_quant_forward
    (plan: optional ExpertPlan built from the same counts)
    Returns:
        - dx: quantized non-transposed gradient [M, 2n]
        - dx_scale: per-expert packed scales, allocated [M, 2n/128]
        - dw: gradient of weight, shape and dtype of weight
        - transpose_dx: per-expert packed transposed gradient, allocated [M, 2n]
        - transpose_dx_scale: [sum ceil(count_e/128), 2n]
    """
    M, N = x.shape
    n = N // 2
    n_expert = counts.shape[0]
    assert n % 128 == 0
    assert g.is_contiguous()
    assert x.is_contiguous() and weight.is_contiguous()
    assert splits is not None, "batch mode need splits to launch kernels"
    _lib.require_device_bf16(x, "x")
    _lib.require_device_bf16(g, "g")
    device = x.device
    dx = torch.empty((M, N), device=device, dtype=fp8_dtype)
    dx_scale = torch.empty((M, N // 128), device=device, dtype=torch.float32)
    s = _blocks_of(splits)
    transpose_dx = torch.empty((M, N), device=device, dtype=fp8_dtype)
    transpose_dx_scale = torch.empty((s, N), device=device, dtype=torch.float32)
    dw = torch.empty_like(weight)
    if s == 0:
        return dx, dx_scale, dw, transpose_dx, transpose_dx_scale
    dws = torch.empty((M, n // 128), device=device, dtype=torch.float32)
    if plan is not None:
        _check_plan(plan, s, device)
        with _lib.on_device(device):
            _lib.check(_lib.lib.fq_batched_swiglu_quant_bwd_planned(
                _lib.ptr(g), _lib.ptr(x), _lib.ptr(weight), _weight_flag(weight), _lib.ptr(plan.table), plan.shape,
                _lib.ptr(dx), _lib.ptr(dx_scale), _lib.ptr(dw), _lib.ptr(transpose_dx),
                _lib.ptr(transpose_dx_scale), _lib.ptr(dws), M, n, int(bool(round_scale)),
                _lib.fp8_kind(fp8_dtype), _lib.stream_of(x)))
        return dx, dx_scale, dw, transpose_dx, transpose_dx_scale
    with _lib.on_device(device):
        _lib.check(_lib.lib.fq_batched_swiglu_quant_bwd(
            _lib.ptr(g), _lib.ptr(x), _lib.ptr(weight), _weight_flag(weight), _lib.ptr(counts),
            _counts_flag(counts), n_expert, s, _lib.ptr(dx), _lib.ptr(dx_scale), _lib.ptr(dw),
            _lib.ptr(transpose_dx), _lib.ptr(transpose_dx_scale), _lib.ptr(dws), M, n,
            int(bool(round_scale)), _lib.fp8_kind(fp8_dtype), _lib.stream_of(x)))
    return dx, dx_scale, dw, transpose_dx, transpose_dx_scale
