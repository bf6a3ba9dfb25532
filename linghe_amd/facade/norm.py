"""Autograd callers of the RMSNorm path (contract: linghe/facade/norm.py:15-112).

``rms_norm`` is the bf16 layer; ``block_rms_norm`` normalises and quantises in one
call and hands the codes to the caller's quantised-tensor class.  Both
differentiate through the same bf16 backward kernel.
"""
import torch

from ..utils.norm import (
    triton_rms_norm_and_block_quant_forward,
    triton_rms_norm_backward,
    triton_rms_norm_forward,
)
from ._qtensor import Codes, Folded, kernel_fp8_dtype, output_mode, wrap


def _input_grads(ctx, dy):
    """(dx, dgamma) of an RMSNorm whose forward saved (x, gamma) and eps on ctx."""
    x, gamma = ctx.saved_tensors
    act = Folded(x)
    dx, dgamma = triton_rms_norm_backward(act.matrix(dy.contiguous()), act.matrix(x), gamma, eps=ctx.eps)
    return dx.view(act.shape), dgamma


class RMSNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps=1e-6):
        ctx.eps = eps
        ctx.save_for_backward(x, weight)
        return triton_rms_norm_forward(x, weight, eps)[0]

    @staticmethod
    def backward(ctx, dy):
        return (*_input_grads(ctx, dy), None)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6):
    """bf16 RMSNorm of x (last dimension) with weight."""
    assert x.is_contiguous() and weight.is_contiguous()
    return RMSNormFunction.apply(x, weight, eps)


class BlockRMSNorm(torch.autograd.Function):
    """RMSNorm + 1x128 / 128x1 blockwise quantisation of a [s, b, h] activation.
    Returns (quantised tensor, 1/rms); `rms` is the saved statistic, required when
    `is_recomputing` is True (only the transposed copy is produced then)."""

    @staticmethod
    def forward(ctx, input, weight, rms, eps, quantizer, cls, is_recomputing):
        assert input.dim() == 3
        act = Folded(input)
        ctx.eps = eps
        ctx.save_for_backward(input, weight)
        q, q_scale, stat, qt, qt_scale = triton_rms_norm_and_block_quant_forward(
            act.matrix(input), weight, eps=eps, rms=rms, round_scale=quantizer.force_pow_2_scales,
            output_mode=output_mode(is_recomputing), fp8_dtype=kernel_fp8_dtype(quantizer.dtype))
        codes = act.unfold(Codes(q, q_scale, qt, qt_scale), act.shape[-1])
        out = wrap(cls, codes, shape=input.shape, dtype=input.dtype, quantizer=quantizer,
                   fp8_tag=quantizer.dtype, requires_grad=input.requires_grad)
        return out, stat

    @staticmethod
    def backward(ctx, grad_output, grad_rms):
        return (*_input_grads(ctx, grad_output), None, None, None, None, None)


def block_rms_norm(input, weight, rms, quantizer, cls, eps=1e-6, is_recomputing=None):
    out, stat = BlockRMSNorm.apply(input, weight, rms, eps, quantizer, cls, is_recomputing)
    return out, stat.detach()
