"""Row-wise 1x128 group quantiser (reference: linghe/quant/group.py:40-63)."""
from __future__ import annotations

import torch

from .. import _lib


def triton_group_quant(x, dtype=torch.float8_e4m3fn, group_size=128, round_scale=False):
    """
    groupwise quantize x, group is in under rowwise format
    Args:
        x: input tensor, bf16 [M, N]
        dtype: fp8 dtype of the codes; the scale is amax/448 for either dtype,
            as in the reference kernel (linghe/quant/group.py:27)
        group_size: group width (128 is the only supported value)
        round_scale: whether round scale to power of 2

    Returns:
        - y: quantized tensor [M, N]
        - s: quantization scale, float32 [M, N/128] (row-major)
    """
    M, N = x.shape
    assert group_size == 128, "only 1x128 groups are implemented"
    assert N % group_size == 0
    assert x.is_contiguous()
    _lib.require_device_bf16(x, "x")
    assert dtype in (torch.float8_e4m3fn, torch.float8_e5m2)
    y = torch.empty((M, N), device=x.device, dtype=dtype)
    s = torch.empty(M, N // group_size, device=x.device, dtype=torch.float32)
    if M > 0:
        with _lib.on_device(x.device):
            _lib.check(_lib.lib.fq_group_quant(_lib.ptr(x), _lib.ptr(y), _lib.ptr(s), M, N,
                                               int(bool(round_scale)),
                                               _lib.FQ_E4M3 if dtype == torch.float8_e4m3fn else _lib.FQ_E5M2_MAX448,
                                               _lib.stream_of(x)))
    return y, s
