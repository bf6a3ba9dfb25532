"""Autograd callers of the SwiGLU + quantisation path (contract:
linghe/facade/silu.py:11-170): the dense form on a [s, b, 2h] activation and the
per-expert weighted form on [tokens, 2h].  Forward and backward both return the
caller's quantised-tensor class; the backward's codes are in the FP8 format of the
gradient quantizer.
"""
import torch

from ..utils.silu import (
    build_expert_plan,
    triton_batch_weighted_silu_and_block_quant_backward,
    triton_batch_weighted_silu_and_block_quant_forward,
    triton_silu_and_block_quant_backward,
    triton_silu_and_block_quant_forward,
)
from ._qtensor import Codes, Folded, kernel_fp8_dtype, output_mode, wrap


class BlockSiluFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, quantizer, grad_quantizer, cls):
        assert input.dim() == 3
        act = Folded(input)
        half = act.shape[-1] // 2
        ctx.save_for_backward(input)
        ctx.sidecar = (grad_quantizer, cls, input.requires_grad)
        got = triton_silu_and_block_quant_forward(
            act.matrix(input), round_scale=quantizer.force_pow_2_scales,
            fp8_dtype=kernel_fp8_dtype(quantizer.dtype))
        return wrap(cls, act.unfold(Codes(*got), half), shape=(*act.lead, half), dtype=input.dtype,
                    quantizer=quantizer, fp8_tag=quantizer.dtype, requires_grad=input.requires_grad)

    @staticmethod
    def backward(ctx, grad_output):
        (input,) = ctx.saved_tensors
        grad_quantizer, cls, needs_grad = ctx.sidecar
        act = Folded(input)
        got = triton_silu_and_block_quant_backward(
            act.matrix(grad_output.contiguous()), act.matrix(input),
            round_scale=grad_quantizer.force_pow_2_scales, fp8_dtype=kernel_fp8_dtype(grad_quantizer.dtype))
        dx = wrap(cls, act.unfold(Codes(*got), act.shape[-1]), shape=act.shape, dtype=grad_output.dtype,
                  quantizer=grad_quantizer, fp8_tag=grad_quantizer.dtype, requires_grad=needs_grad)
        return dx, None, None, None


def block_silu_impl(input, quantizer, grad_quantizer, cls):
    return BlockSiluFunction.apply(input, quantizer, grad_quantizer, cls)


class BlockBatchWeightedSiluFunction(torch.autograd.Function):
    """Per-expert form: rows of `input` are grouped by expert (`counts` on the device,
    `splits` the same numbers on the host), `weights` is one router probability per
    row.  Outputs keep the kernels' per-expert packing, so nothing is re-viewed.
    The quantizer lists are passed through to the tensor class; their first member
    gives the scale rounding and the FP8 format of all experts.  `plan` (optional, an
    ExpertPlan of the same counts) is handed to the forward and kept for the backward; when
    a backward will follow and the caller brought none, the forward builds one (one small
    launch that both kernels gain more from than it costs)."""

    @staticmethod
    def forward(ctx, input, weights, counts, splits, quantizers, grad_quantizers, cls, is_recomputing, plan=None):
        lead = quantizers[0]
        ctx.save_for_backward(input, weights, counts)
        if plan is None and (input.requires_grad or weights.requires_grad) and input.shape[0] > 0:
            plan = build_expert_plan(counts, splits)
        ctx.sidecar = (splits, grad_quantizers, cls, input.requires_grad, plan)
        got = triton_batch_weighted_silu_and_block_quant_forward(
            input, weights, counts, splits=splits, round_scale=lead.force_pow_2_scales,
            output_mode=output_mode(is_recomputing), fp8_dtype=kernel_fp8_dtype(lead.dtype), plan=plan)
        codes = Codes(*got)
        return wrap(cls, codes, shape=codes.row.shape, dtype=input.dtype, quantizer=quantizers,
                    fp8_tag=lead.dtype, requires_grad=input.requires_grad)

    @staticmethod
    def backward(ctx, grad_output):
        input, weights, counts = ctx.saved_tensors
        splits, grad_quantizers, cls, needs_grad, plan = ctx.sidecar
        lead = grad_quantizers[0]
        dq, dq_scale, dweights, dqt, dqt_scale = triton_batch_weighted_silu_and_block_quant_backward(
            grad_output.contiguous(), input, weights, counts, splits=splits,
            round_scale=lead.force_pow_2_scales, fp8_dtype=kernel_fp8_dtype(lead.dtype), plan=plan)
        dx = wrap(cls, Codes(dq, dq_scale, dqt, dqt_scale), shape=input.shape, dtype=grad_output.dtype,
                  quantizer=grad_quantizers, fp8_tag=lead.dtype, requires_grad=needs_grad)
        # one gradient slot per forward argument: input, weights, then seven non-tensors
        return (dx, dweights) + (None,) * 7


def block_batch_weighted_silu_impl(input, weights, counts, splits, quantizers, grad_quantizers, cls,
                                   is_recomputing=None, *, plan=None):
    assert input.ndim == 2
    return BlockBatchWeightedSiluFunction.apply(input, weights, counts, splits, quantizers, grad_quantizers,
                                                cls, is_recomputing, plan)
