"""Acceptance rules used by the parity tests (TEST INFRASTRUCTURE ONLY).

* scales: distance in units in the last place, through the int32 view of the
  positive fp32 values;
* FP8 codes: number of codes that differ (at most 1e-4 of them, or one on a small
  tensor) and the largest distance in code steps (codes are mapped to a monotone
  integer line, so +0/-0 are 0 apart and neighbours are 1 apart);
* dequantisation bound: |q*s - v| <= half a code step at q's exponent, times s;
* ``output_check_like``: the reference's own, looser, elementwise rule
  (linghe/tools/check.py:11-129: |d| < rtol*|ref| + atol after upcasting).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch


def ulp_distance(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Elementwise distance in fp32 ulps (both finite, same sign expected)."""
    ai = a.detach().float().contiguous().view(torch.int32).to(torch.int64)
    bi = b.detach().float().contiguous().view(torch.int32).to(torch.int64)
    # map the sign-magnitude pattern to a monotone line
    ai = torch.where(ai < 0, -(ai & 0x7FFFFFFF), ai)
    bi = torch.where(bi < 0, -(bi & 0x7FFFFFFF), bi)
    return (ai - bi).abs()


def code_line(codes: torch.Tensor) -> torch.Tensor:
    """fp8 bit patterns (any fp8 dtype or uint8) -> signed monotone integers."""
    u = codes.detach().contiguous().view(torch.uint8).to(torch.int32)
    mag = u & 0x7F
    return torch.where(u >= 128, -mag, mag)


@dataclass
class CodeReport:
    total: int
    identical: int
    max_step: int

    @property
    def identical_frac(self) -> float:
        return 1.0 if self.total == 0 else self.identical / self.total


def compare_codes(ref: torch.Tensor, got: torch.Tensor) -> CodeReport:
    assert ref.shape == got.shape, (ref.shape, got.shape)
    if ref.numel() == 0:
        return CodeReport(0, 0, 0)
    d = (code_line(ref) - code_line(got)).abs()
    return CodeReport(int(d.numel()), int((d == 0).sum()), int(d.max()))


@dataclass
class ScaleReport:
    total: int
    exact: int
    within_1ulp: int
    max_ulp: int


def compare_scales(ref: torch.Tensor, got: torch.Tensor) -> ScaleReport:
    assert ref.shape == got.shape, (ref.shape, got.shape)
    if ref.numel() == 0:
        return ScaleReport(0, 0, 0, 0)
    d = ulp_distance(ref, got)
    return ScaleReport(int(d.numel()), int((d == 0).sum()), int((d <= 1).sum()), int(d.max()))


def allowed_mismatches(total: int, min_identical: float) -> int:
    """How many codes of `total` may differ.  The rule is a fraction (1 - min_identical, 1e-4 by
    default); on a tensor too small for the fraction to allow even one code it allows one, so
    that a single last-bit difference in a scale does not fail a small case while the fraction
    itself is never loosened.  min_identical = 1 means bit-exact: none."""
    if min_identical >= 1.0:
        return 0
    return max(1, math.ceil((1.0 - min_identical) * total - 1e-9))


def assert_codes(ref, got, name="codes", min_identical=0.9999, max_step=1):
    rep = compare_codes(ref, got)
    allowed = allowed_mismatches(rep.total, min_identical)
    assert rep.total - rep.identical <= allowed and rep.max_step <= max_step, (
        f"{name}: identical {rep.identical}/{rep.total} "
        f"({rep.identical_frac:.6f}; at most {allowed} may differ), max step {rep.max_step}")
    return rep


def assert_scales(ref, got, name="scales", max_ulp=1, min_within_1ulp=1.0, truth=None, bound=None):
    """All scales within max_ulp of the oracle's and at least min_within_1ulp of them
    within 1 ulp.

    truth / bound (optional, fp64, same layout as the scales): the real-number value
    of every scale and the first-order error bound of an fp32 evaluation of it.  With
    them a scale may be further than max_ulp from the oracle's only where the element
    that makes the group's amax is ill-conditioned (a cancellation): the group's own
    bound must exceed max_ulp / 2 ulps, and BOTH sides must lie within that bound of
    the true value.  Without them nothing may exceed max_ulp."""
    rep = compare_scales(ref, got)
    if rep.total == 0:
        return rep
    d = ulp_distance(ref, got)
    frac = rep.within_1ulp / rep.total
    beyond = d > max_ulp
    ok = frac >= min_within_1ulp
    n_ill = 0
    if bool(beyond.any()):
        if truth is None:
            ok = False
        else:
            t = truth.reshape(-1)[beyond.reshape(-1)]
            b = bound.reshape(-1)[beyond.reshape(-1)]
            ulp = torch.ldexp(torch.ones_like(t), torch.frexp(t.float().double())[1] - 24)
            ill = b > 0.5 * max_ulp * ulp
            g = got.detach().float().reshape(-1)[beyond.reshape(-1)].double()
            r = ref.detach().float().reshape(-1)[beyond.reshape(-1)].double()
            ok = ok and bool(ill.all()) and bool(((g - t).abs() <= b).all()) and bool(((r - t).abs() <= b).all())
            n_ill = int(ill.sum())
    assert ok, (f"{name}: exact {rep.exact}/{rep.total}, <=1ulp {rep.within_1ulp}, "
                f"max {rep.max_ulp} ulp, beyond {max_ulp} ulp: {int(beyond.sum())} "
                f"(of which ill-conditioned and within their bound: {n_ill})")
    return rep


def fp8_half_step(q: torch.Tensor, fp8_dtype) -> torch.Tensor:
    """Half the spacing of the fp8 grid at the value q (fp32 tensor of decoded
    codes).  e4m3: 3 mantissa bits, min normal exponent -6; e5m2: 2 bits, -14."""
    mant, emin = (3, -6) if fp8_dtype == torch.float8_e4m3fn else (2, -14)
    a = q.abs().clamp_min(2.0 ** emin)
    e = torch.floor(torch.log2(a))
    return torch.exp2(e - mant - 1)


def assert_dequant_bound(values, codes, scales_per_elem, fp8_dtype, name="dequant",
                         slack=1.0 + 2.0 ** -12):
    """|decode(code)*s - v| <= half a code step * s (small slack for the fp32
    rounding of the quotient)."""
    q = codes.float().double()
    s = scales_per_elem.double()
    err = (q * s - values.double()).abs()
    # at a power of two the grid below is finer than above, so the half step
    # taken at q's own exponent bounds both sides
    bound = fp8_half_step(q.float(), fp8_dtype).double() * s * slack
    bad = err > bound
    assert not bool(bad.any()), f"{name}: {int(bad.sum())} elements outside the quantisation bound"


def output_check_like(ref, got, rtol=None, atol=None):
    """The reference's elementwise acceptance (linghe/tools/check.py:43-69,114)."""
    assert ref.dtype == got.dtype and ref.shape == got.shape
    dt = ref.dtype
    defaults = {torch.float32: (1e-4, 1e-6), torch.bfloat16: (2e-2, 1e-3),
                torch.float8_e4m3fn: (0.125, 0.125), torch.float8_e5m2: (0.25, 0.25)}
    r, a = defaults[dt]
    rtol = r if rtol is None else rtol
    atol = a if atol is None else atol
    rf, gf = ref.float(), got.float()
    return int(((rf - gf).abs() >= rtol * rf.abs() + atol).sum())
