"""Autograd callers of the RMSNorm path (reference: linghe/facade/norm.py:15-112).

``cls`` is the caller's quantised-tensor class (TransformerEngine's
Float8BlockwiseQTensor in Megatron); it is constructed with the same keyword
arguments the reference passes.
"""
import torch

from ..utils.norm import (
    triton_rms_norm_and_block_quant_forward,
    triton_rms_norm_backward,
    triton_rms_norm_forward,
)


class RMSNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps=1e-6):
        output, _ = triton_rms_norm_forward(x, weight, eps)
        ctx.save_for_backward(x, weight)
        ctx.eps = eps
        return output

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        dx, dw = triton_rms_norm_backward(dy.contiguous(), x, weight, ctx.eps)
        return dx, dw, None


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6):
    """bf16 RMSNorm of x with weight."""
    assert x.is_contiguous()
    assert weight.is_contiguous()
    return RMSNormFunction.apply(x, weight, eps)


def _mode_of(is_recomputing):
    # None -> both layouts, True -> transposed only (recompute in backward),
    # False -> row-wise only
    if is_recomputing is None:
        return 2
    return 1 if is_recomputing else 0


class BlockRMSNorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, weight, rms, eps, quantizer, cls, is_recomputing):
        shape = input.shape
        assert len(shape) == 3
        rows = shape[0] * shape[1]
        x_q, x_scale, output_rms, xt_q, xt_scale = triton_rms_norm_and_block_quant_forward(
            input.view(rows, shape[2]),
            weight,
            rms=rms,
            eps=eps,
            round_scale=quantizer.force_pow_2_scales,
            output_mode=_mode_of(is_recomputing),
        )
        output = cls(
            shape=shape,
            dtype=input.dtype,
            fp8_dtype=quantizer.dtype,
            rowwise_data=x_q.view(shape) if x_q is not None else None,
            rowwise_scale_inv=x_scale,
            columnwise_data=xt_q.view(shape[2], shape[0], shape[1]) if xt_q is not None else None,
            columnwise_scale_inv=xt_scale,
            quantizer=quantizer,
            requires_grad=input.requires_grad,
            is_2D_scaled=False,
        )
        ctx.shape = shape
        ctx.eps = eps
        ctx.save_for_backward(input, weight)
        return output, output_rms

    @staticmethod
    def backward(ctx, grad_output, grad_rms):
        shape = ctx.shape
        rows = shape[0] * shape[1]
        input, weight = ctx.saved_tensors
        dx, dw = triton_rms_norm_backward(
            grad_output.contiguous().view(rows, shape[2]), input.view(rows, shape[2]), weight, eps=ctx.eps
        )
        return dx.view(*shape), dw, None, None, None, None, None


def block_rms_norm(input, weight, rms, quantizer, cls, eps=1e-6, is_recomputing=None):
    output, output_rms = BlockRMSNorm.apply(input, weight, rms, eps, quantizer, cls, is_recomputing)
    return output, output_rms.detach()
