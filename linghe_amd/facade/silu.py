"""Autograd callers of the SwiGLU+quant path (reference: linghe/facade/silu.py:11-170)."""
import torch

from ..utils.silu import (
    triton_batch_weighted_silu_and_block_quant_backward,
    triton_batch_weighted_silu_and_block_quant_forward,
    triton_silu_and_block_quant_backward,
    triton_silu_and_block_quant_forward,
)


def _mode_of(is_recomputing):
    if is_recomputing is None:
        return 2
    return 1 if is_recomputing else 0


class BlockSiluFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, quantizer, grad_quantizer, cls):
        shape = input.shape
        assert len(shape) == 3
        rows, half = shape[0] * shape[1], shape[2] // 2
        ctx.grad_quantizer = grad_quantizer
        ctx.input_requires_grad = input.requires_grad
        ctx.shape = shape
        ctx.cls = cls
        ctx.save_for_backward(input)
        x_q, x_scale, xt_q, xt_scale = triton_silu_and_block_quant_forward(
            input.view(rows, shape[2]), round_scale=quantizer.force_pow_2_scales
        )
        out_shape = (shape[0], shape[1], half)
        return cls(
            shape=out_shape,
            dtype=input.dtype,
            fp8_dtype=quantizer.dtype,
            rowwise_data=x_q.view(out_shape),
            rowwise_scale_inv=x_scale,
            columnwise_data=xt_q.view(half, shape[0], shape[1]),
            columnwise_scale_inv=xt_scale,
            quantizer=quantizer,
            requires_grad=input.requires_grad,
            is_2D_scaled=False,
        )

    @staticmethod
    def backward(ctx, grad_output):
        gshape = grad_output.shape
        rows = gshape[0] * gshape[1]
        (input,) = ctx.saved_tensors
        gq = ctx.grad_quantizer
        x_q, x_scale, xt_q, xt_scale = triton_silu_and_block_quant_backward(
            grad_output.contiguous().view(rows, gshape[2]),
            input.view(rows, gshape[2] * 2),
            round_scale=gq.force_pow_2_scales,
        )
        output = ctx.cls(
            shape=ctx.shape,
            dtype=grad_output.dtype,
            fp8_dtype=gq.dtype,
            rowwise_data=x_q.view(ctx.shape),
            rowwise_scale_inv=x_scale,
            columnwise_data=xt_q.view(ctx.shape[2], gshape[0], gshape[1]),
            columnwise_scale_inv=xt_scale,
            quantizer=gq,
            requires_grad=ctx.input_requires_grad,
            is_2D_scaled=False,
        )
        return output, None, None, None


def block_silu_impl(input, quantizer, grad_quantizer, cls):
    return BlockSiluFunction.apply(input, quantizer, grad_quantizer, cls)


class BlockBatchWeightedSiluFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, weights, counts, splits, quantizers, grad_quantizers, cls, is_recomputing):
        ctx.grad_quantizers = grad_quantizers
        ctx.input_requires_grad = input.requires_grad
        ctx.shape = input.shape
        ctx.splits = splits
        ctx.cls = cls
        ctx.save_for_backward(input, weights, counts)
        x_q, x_scale, xt_q, xt_scale = triton_batch_weighted_silu_and_block_quant_forward(
            input,
            weights,
            counts,
            splits=splits,
            round_scale=quantizers[0].force_pow_2_scales,
            output_mode=_mode_of(is_recomputing),
        )
        return cls(
            shape=x_q.shape,
            dtype=input.dtype,
            fp8_dtype=quantizers[0].dtype,
            rowwise_data=x_q,
            rowwise_scale_inv=x_scale,
            columnwise_data=xt_q,
            columnwise_scale_inv=xt_scale,
            quantizer=quantizers,
            requires_grad=input.requires_grad,
            is_2D_scaled=False,
        )

    @staticmethod
    def backward(ctx, grad_output):
        input, weights, counts = ctx.saved_tensors
        gqs = ctx.grad_quantizers
        x_q, x_scale, wgrad, xt_q, xt_scale = triton_batch_weighted_silu_and_block_quant_backward(
            grad_output.contiguous(),
            input,
            weights,
            counts,
            splits=ctx.splits,
            round_scale=gqs[0].force_pow_2_scales,
        )
        output = ctx.cls(
            shape=ctx.shape,
            dtype=grad_output.dtype,
            fp8_dtype=gqs[0].dtype,
            rowwise_data=x_q,
            rowwise_scale_inv=x_scale,
            columnwise_data=xt_q,
            columnwise_scale_inv=xt_scale,
            quantizer=gqs,
            requires_grad=ctx.input_requires_grad,
            is_2D_scaled=False,
        )
        return output, wgrad, None, None, None, None, None, None


def block_batch_weighted_silu_impl(
    input, weights, counts, splits, quantizers, grad_quantizers, cls, is_recomputing=None
):
    assert input.ndim == 2
    return BlockBatchWeightedSiluFunction.apply(
        input, weights, counts, splits, quantizers, grad_quantizers, cls, is_recomputing
    )
