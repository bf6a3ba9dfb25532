"""Shared plumbing of the autograd callers: the caller contract of the reference's
facade layer (linghe/facade/norm.py:49-112, linghe/facade/silu.py:11-170) stated
once.

* the recompute flag picks the kernel's output mode: None -> both layouts,
  False -> row-wise only, True -> transposed only;
* activations arrive as [s, b, h]; the kernels see [s*b, h]; row-wise codes go
  back out as [s, b, h'] and transposed codes as [h', s, b];
* the quantised result is handed to the caller's tensor class (TransformerEngine's
  Float8BlockwiseQTensor in Megatron) through one fixed set of keywords;
* the quantizer's dtype tag decides which FP8 format the kernel emits, so the
  label the tensor class receives and the bytes it wraps always agree.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

_OUTPUT_MODE = {None: 2, False: 0, True: 1}


def output_mode(is_recomputing) -> int:
    """output_mode of the quantising entry points for a layer that is (True) /
    is not (False) inside an activation recompute, or does not say (None)."""
    if is_recomputing is None:
        return 2
    return _OUTPUT_MODE[bool(is_recomputing)]


def kernel_fp8_dtype(tag) -> torch.dtype:
    """torch FP8 dtype for a quantizer's dtype tag: a torch dtype, or an enum member
    such as TransformerEngine's DType.kFloat8E5M2 (matched by name)."""
    if isinstance(tag, torch.dtype):
        if tag in (torch.float8_e4m3fn, torch.float8_e5m2):
            return tag
        raise TypeError(f"quantizer dtype {tag} is not an FP8 format of this path")
    name = str(getattr(tag, "name", tag)).upper()
    if "E5M2" in name:
        return torch.float8_e5m2
    if "E4M3" in name:
        return torch.float8_e4m3fn
    raise TypeError(f"cannot tell the FP8 format of quantizer dtype {tag!r}")


@dataclass
class Codes:
    """The four tensors a quantising entry point returns (absent layouts are None)."""
    row: Optional[torch.Tensor]
    row_scale: Optional[torch.Tensor]
    col: Optional[torch.Tensor]
    col_scale: Optional[torch.Tensor]


class Folded:
    """An activation [..., h] seen as the matrix [rows, h] the kernels take."""

    def __init__(self, t: torch.Tensor):
        self.shape = tuple(t.shape)
        self.lead = self.shape[:-1]
        self.rows = 1
        for d in self.lead:
            self.rows *= d

    def matrix(self, t: torch.Tensor) -> torch.Tensor:
        return t.view(self.rows, t.shape[-1])

    def unfold(self, codes: Codes, width: int) -> Codes:
        """row-wise codes back to [..., width], transposed codes to [width, ...]"""
        row = None if codes.row is None else codes.row.view(*self.lead, width)
        col = None if codes.col is None else codes.col.view(width, *self.lead)
        return Codes(row, codes.row_scale, col, codes.col_scale)


def wrap(cls, codes: Codes, *, shape, dtype, quantizer, fp8_tag, requires_grad):
    """Construct the caller's quantised-tensor class around `codes`
    (keywords of linghe/facade/norm.py:75-86)."""
    return cls(shape=shape, dtype=dtype, fp8_dtype=fp8_tag, rowwise_data=codes.row,
               rowwise_scale_inv=codes.row_scale, columnwise_data=codes.col,
               columnwise_scale_inv=codes.col_scale, quantizer=quantizer, requires_grad=requires_grad,
               is_2D_scaled=False)
