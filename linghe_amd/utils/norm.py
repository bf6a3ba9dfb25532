"""RMSNorm entry points (reference: linghe/utils/norm.py:58-93, 144-179, 343-502).

Same names, argument order, defaults and return tuples as the reference's
Triton wrappers; the bodies enqueue HIP kernels on torch's current stream.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _lib

_MAX_HIDDEN = 8192  # the reference asserts next_power_of_2(n) <= 8192


def _rows_cols(x):
    shape = x.shape
    assert len(shape) in (2, 3)
    if len(shape) == 3:
        return shape[0] * shape[1], shape[2]
    return shape[0], shape[1]


def _check_hidden(n: int) -> None:
    assert n <= _MAX_HIDDEN, f"hidden size {n} > {_MAX_HIDDEN}"
    if n % 8 != 0:
        raise ValueError(f"hidden size {n} must be a multiple of 8 (128-bit bf16 loads)")


def triton_rms_norm_forward(x, weight, eps=1e-6, out=None, rms=None):
    """
    rms norm
    Args:
        x: input tensor, bf16 [M, n] or [s, b, n]
        weight: weight of rms norm, bf16 [n]
        eps: epsilon of rms norm
        rms: use x*rms to calculate output if rms is not None
    Returns:
        out: output tensor (dtype and shape of x)
        rms: 1/rms of input tensor, fp32 [M]
    """
    assert x.is_contiguous() and weight.is_contiguous()
    M, n = _rows_cols(x)
    _check_hidden(n)
    _lib.require_device_bf16(x, "x")
    _lib.require_device_bf16(weight, "weight")
    if out is None:
        out = torch.empty_like(x)
    reuse = rms is not None
    if not reuse:
        rms = torch.empty((M,), device=x.device, dtype=torch.float32)
    if M > 0:
        with _lib.on_device(x.device):
            _lib.check(_lib.lib.fq_rmsnorm_fwd(_lib.ptr(x), _lib.ptr(weight), _lib.ptr(out), _lib.ptr(rms),
                                               M, n, float(eps), int(reuse), _lib.stream_of(x)))
    return out, rms


def triton_rms_norm_backward(grad_output, x, w, eps=1e-6, rms=None):
    """
    backward of rms norm
    Returns:
        dx: gradient of x (dtype and shape of x)
        dw: gradient of the weight, fp32 [n]
    """
    assert grad_output.is_contiguous()
    M, n = _rows_cols(x)
    _check_hidden(n)
    _lib.require_device_bf16(x, "x")
    _lib.require_device_bf16(grad_output, "grad_output")
    _lib.require_device_bf16(w, "w")
    assert x.is_contiguous() and w.is_contiguous()
    dx = torch.empty_like(x)
    dw = torch.empty((n,), dtype=torch.float32, device=w.device)
    n_part = int(_lib.lib.fq_rmsnorm_bwd_num_partials(M, n))
    tmp_dw = torch.empty((n_part, n), dtype=torch.float32, device=w.device)
    with _lib.on_device(x.device):
        _lib.check(_lib.lib.fq_rmsnorm_bwd(_lib.ptr(grad_output), _lib.ptr(x), _lib.ptr(w), _lib.ptr(rms),
                                           _lib.ptr(dx), _lib.ptr(dw), _lib.ptr(tmp_dw), n_part, M, n,
                                           float(eps), _lib.stream_of(x)))
    return dx, dw


def triton_rms_norm_and_block_quant_forward(
    x: torch.Tensor,
    weight: torch.Tensor,
    eps: float = 1e-6,
    out: Optional[torch.Tensor] = None,
    scale: Optional[torch.Tensor] = None,
    rms: Optional[torch.Tensor] = None,
    round_scale: bool = False,
    output_mode: int = 2,
    *,
    fp8_dtype: torch.dtype = torch.float8_e4m3fn,
):
    """
    Fused RMSNorm forward and block quantization.
    Args:
        x: Input tensor, shape [M, N]
        weight: RMSNorm weight,  shape [N]
        eps: epsilon value for L2 normalization.
        out: output of quantization data
        scale: output of quantization scale.
        rms: output of rms (input when output_mode == 1)
        round_scale: Set whether to force power of 2 scales.
        output_mode: one of {0, 1, 2}.
            0: only output non-transpose tensor
            1: only output transposed tensor
            2: return both
        fp8_dtype: (extension, keyword only) float8_e4m3fn or float8_e5m2
    Returns:
        - out: quantization data [M, N].
        - scale: quantization scale [N/128, M].
        - rms: reciprocal of the root mean square of the input, [M].
        - transpose_output: quantization data of the transposed output [N, M].
        - transpose_scale: its quantization scale [ceil(M/128), N].
    """
    assert x.is_contiguous() and weight.is_contiguous()
    M, n = x.shape
    _check_hidden(n)
    assert n % 128 == 0, f"{n=} must be a multiple of 128"
    assert output_mode in (0, 1, 2)
    _lib.require_device_bf16(x, "x")
    _lib.require_device_bf16(weight, "weight")
    device = x.device
    kind = _lib.fp8_kind(fp8_dtype)

    if out is None and output_mode in (0, 2):
        out = torch.empty((M, n), device=device, dtype=fp8_dtype)
    if scale is None and output_mode in (0, 2):
        scale = torch.empty((n // 128, M), device=device, dtype=torch.float32)
    # the transposed buffers are always allocated, as in the reference
    transpose_output = torch.empty((n, M), device=device, dtype=fp8_dtype)
    transpose_scale = torch.empty(((M + 127) // 128, n), device=device, dtype=torch.float32)

    if output_mode == 0:
        assert rms is None
        rms = torch.empty((M,), dtype=torch.float32, device=device)
    elif output_mode == 1:
        assert rms is not None
    else:
        # a given rms is ignored and recomputed, as in the reference
        rms = torch.empty((M,), dtype=torch.float32, device=device)

    if M > 0:
        with _lib.on_device(device):
            _lib.check(_lib.lib.fq_rmsnorm_quant_fwd(
                _lib.ptr(x), _lib.ptr(weight),
                _lib.ptr(out) if output_mode != 1 else None,
                _lib.ptr(scale) if output_mode != 1 else None,
                _lib.ptr(rms), _lib.ptr(transpose_output), _lib.ptr(transpose_scale),
                M, n, float(eps), int(bool(round_scale)), output_mode, kind, _lib.stream_of(x)))
    return out, scale, rms, transpose_output, transpose_scale


def pack_route_weight(route_weight: torch.Tensor) -> torch.Tensor:
    """The router weight [N, K] (bf16 or fp32) in the operand order the RMSNorm + router GEMM
    kernels read it in, as a uint8 tensor to pass as `packed_route_weight=` of
    triton_rms_norm_fp32_gemm_block_quant_forward.  No counterpart in the reference, which
    re-reads route_weight on every call: re-pack after every update of the weight."""
    assert route_weight.is_contiguous() and route_weight.dim() == 2
    if route_weight.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"route_weight must be bfloat16 or float32, got {route_weight.dtype}")
    if not route_weight.is_cuda:
        raise RuntimeError("route_weight must live on the GPU: the HIP kernels are the only implementation")
    N, K = route_weight.size()
    assert K % 128 == 0 and N % 128 == 0
    w_fp32 = int(route_weight.dtype == torch.float32)
    packed = torch.empty(int(_lib.lib.fq_rmsnorm_router_scratch_bytes(K, N, w_fp32)), dtype=torch.uint8,
                         device=route_weight.device)
    with _lib.on_device(route_weight.device):
        _lib.check(_lib.lib.fq_pack_router_weight(_lib.ptr(route_weight), w_fp32, _lib.ptr(packed), K, N,
                                                  _lib.stream_of(route_weight)))
    return packed


def triton_rms_norm_fp32_gemm_block_quant_forward(
    x: torch.Tensor,
    norm_weight: torch.Tensor,
    route_weight: torch.Tensor,
    rms: Optional[torch.Tensor] = None,
    eps: float = 1e-6,
    output_mode: int = 0,
    round_scale=False,
    *,
    packed_route_weight: Optional[torch.Tensor] = None,
):
    """
    y = rms_norm(x)
    logits = y@w_route
    x_q, x_s, xt_q, xt_s = quantization(y)
    Args:
        x: input tensor, bf16 [M, K]
        norm weight: weight tensor of rms norm, bf16 [K]
        route_weight: moe router weight [N, K], bf16 or fp32, N a multiple of 128
        eps: epsilon of rms norm
        output_mode: 0 or 1
            0: only output non-transpose quantizatino tensor (and y, rms, logits)
            1: only output transposed quantizatino tensor (rms must be given)
        packed_route_weight: (keyword-only addition) the result of pack_route_weight(route_weight).
            The kernels read the router weight in matrix-core operand order; without this
            argument it is re-ordered on every call, with it the caller re-orders once per
            weight update.  Results are identical.

    Returns:
        - y: rms normed tensor
        - rms: 1/rms
        - logits: router logit
        - x_q:
        - x_s:
        - xt_q:
        - xt_s:
    """
    assert x.is_contiguous() and norm_weight.is_contiguous() and route_weight.is_contiguous()
    assert output_mode in (0, 1)
    M, K = x.size()
    N, K2 = route_weight.size()
    assert K2 == K
    assert M % 128 == 0 and K % 128 == 0 and N % 128 == 0
    _check_hidden(K)
    _lib.require_device_bf16(x, "x")
    _lib.require_device_bf16(norm_weight, "norm_weight")
    device = x.device
    y = torch.empty(M, K, dtype=x.dtype, device=device)
    if rms is None:
        assert output_mode == 0
        rms = torch.empty(M, dtype=torch.float32, device=device)
    logits = torch.empty(M, N, dtype=torch.float32, device=device)
    x_q = torch.empty((M, K), device=device, dtype=torch.float8_e4m3fn)
    x_s = torch.empty((K // 128, M), device=device, dtype=torch.float32)
    xt_q = torch.empty((K, M), device=device, dtype=torch.float8_e4m3fn)
    xt_s = torch.empty((M // 128, K), device=device, dtype=torch.float32)
    if M == 0:
        return y, rms, logits, x_q, x_s, xt_q, xt_s
    with _lib.on_device(device):
        if output_mode == 0:
            if route_weight.dtype not in (torch.bfloat16, torch.float32):
                raise TypeError(f"route_weight must be bfloat16 or float32, got {route_weight.dtype}")
            if not route_weight.is_cuda:
                raise RuntimeError("route_weight must live on the GPU: the HIP kernels are the only implementation")
            w_fp32 = int(route_weight.dtype == torch.float32)
            need = int(_lib.lib.fq_rmsnorm_router_scratch_bytes(K, N, w_fp32))
            if packed_route_weight is not None:
                assert packed_route_weight.is_cuda and packed_route_weight.dtype == torch.uint8
                assert packed_route_weight.numel() == need and packed_route_weight.is_contiguous()
                _lib.check(_lib.lib.fq_rmsnorm_router_quant_fwd_packed(
                    _lib.ptr(x), _lib.ptr(norm_weight), _lib.ptr(packed_route_weight), w_fp32, _lib.ptr(y),
                    _lib.ptr(rms), _lib.ptr(logits), _lib.ptr(x_q), _lib.ptr(x_s), M, K, N, float(eps),
                    int(bool(round_scale)), _lib.FQ_E4M3, _lib.stream_of(x)))
            else:
                # route_weight re-ordered for the matrix cores (an fp32 weight as two bf16 planes)
                scratch = torch.empty(need, dtype=torch.uint8, device=device)
                _lib.check(_lib.lib.fq_rmsnorm_router_quant_fwd(
                    _lib.ptr(x), _lib.ptr(norm_weight), _lib.ptr(route_weight), w_fp32, _lib.ptr(scratch),
                    _lib.ptr(y), _lib.ptr(rms), _lib.ptr(logits), _lib.ptr(x_q), _lib.ptr(x_s), M, K, N, float(eps),
                    int(bool(round_scale)), _lib.FQ_E4M3, _lib.stream_of(x)))
        else:
            _lib.check(_lib.lib.fq_rmsnorm_quant_fwd(
                _lib.ptr(x), _lib.ptr(norm_weight), None, None, _lib.ptr(rms), _lib.ptr(xt_q), _lib.ptr(xt_s),
                M, K, float(eps), int(bool(round_scale)), 1, _lib.FQ_E4M3, _lib.stream_of(x)))
    return y, rms, logits, x_q, x_s, xt_q, xt_s
