"""fp64 evaluation of the fused ops' mathematics, with first-order error bounds for
an fp32 evaluation of the same expressions (TEST INFRASTRUCTURE ONLY).

The torch oracle and the HIP kernels both evaluate these expressions in fp32, each
with its own exp, reduction order and rounding sequence, so their scales can
differ by a few units in the last place without either being wrong.  What the
mathematics fixes is the real-number value; this module computes it in fp64
(whose own error, ~1e-16, is nine orders below one fp32 ulp) together with a bound
on how far ANY fp32 evaluation with a stated number of roundings can be from it.

Notation: U = 2^-24 is the unit roundoff of fp32: one correctly rounded operation
has relative error <= U; one ulp of a result v is between U|v| and 2U|v|.

Rounding budgets (relative, in units of U):

* sigmoid.  exp2 to 1 ulp (<= 2U), the first-order tail correction (one fma, U),
  d = 1 + e (U, plus the error of e weighted by e/(1+e) < 1), a refined reciprocal
  (U): SIGMOID_K = 5.
* SwiGLU forward  y = ((s*x1)*x2)[*w]:  SIGMOID_K + 2 (+1 with the row weight).
* SwiGLU backward, with h = (g[*w])*x2:
    dx2 = (g[*w])*(s*x1):  SIGMOID_K + 2 (+1)
    dx1 = h*s + ((h*x1)*(1-s))*s.  d(dx1)/ds = h*(1 + x1*(1-2s)), so the sigmoid's
    error enters with that factor (|x1|-fold for large |x1|: no fp32 evaluation of
    this formula escapes it); the other roundings are bounded by
    4U*(|h*s| + |h*x1*(1-s)*s|) + U|dx1| + (error of h)*|dx1|.
* RMSNorm  y = (x*r)*g, r = 1/sqrt(sum(x^2)/n + eps):  the sum is <= 5U (four
  dot-product roundings inside a group of eight, the exact sum of the group sums
  rounded once), /n and +eps add 2U, the square root halves that and adds U, the
  reciprocal adds U: r <= 5.5U; two products: RMSNORM_K = 7.5.
* scale = amax/fmax: one more rounding (U), applied in ``scale_bounds``.
"""
from __future__ import annotations

import torch

U = 2.0 ** -24
SIGMOID_K = 5.0
RMSNORM_K = 7.5
GROUP = 128
FLOOR = 1e-30


def rmsnorm_values(x, gamma, eps):
    """(y fp64 [M, n], abs error bound fp64 [M, n], rstd fp64 [M])"""
    xd = x.double()
    n = x.shape[1]
    r = 1.0 / torch.sqrt((xd * xd).sum(1) / n + float(torch.tensor(eps, dtype=torch.float32)))
    y = xd * r[:, None] * gamma.double()[None, :]
    return y, RMSNORM_K * U * y.abs(), r


def swiglu_values(x, w=None):
    """(y fp64 [M, n], abs error bound)"""
    xd = x.double()
    n = x.shape[1] // 2
    x1, x2 = xd[:, :n], xd[:, n:]
    y = torch.sigmoid(x1) * x1 * x2
    k = SIGMOID_K + 2
    if w is not None:
        y = y * w.double().reshape(-1, 1)
        k += 1
    return y, k * U * y.abs()


def swiglu_grad_values(dy, x, w=None):
    """(dx fp64 [M, 2n] = dx1 | dx2, abs error bound fp64 [M, 2n], dw fp64 [M] or None)"""
    xd = x.double()
    n = x.shape[1] // 2
    x1, x2 = xd[:, :n], xd[:, n:]
    g = dy.double()
    s = torch.sigmoid(x1)
    gw, h_err = g, 1.0
    dw = None
    if w is not None:
        dw = (g * (s * x1 * x2)).sum(1)
        gw = g * w.double().reshape(-1, 1)
        h_err = 2.0
    h = gw * x2
    t1 = h * s
    t2 = h * x1 * (1.0 - s) * s
    dx1 = t1 + t2
    dx2 = gw * (s * x1)
    e1 = (SIGMOID_K * U) * (s * (h * (1.0 + x1 * (1.0 - 2.0 * s))).abs()) \
        + 4.0 * U * (t1.abs() + t2.abs()) + (1.0 + h_err) * U * dx1.abs()
    e2 = (SIGMOID_K + 2.0 + (h_err - 1.0)) * U * dx2.abs()
    return torch.cat([dx1, dx2], 1), torch.cat([e1, e2], 1), dw


def _scale_and_bound(amax, emax, fmax):
    s = torch.clamp_min(amax / fmax, FLOOR)
    # max is 1-Lipschitz in the sup norm: |amax' - amax| <= max_i |v'_i - v_i|; then one division
    b = emax / fmax + U * s
    return s, b


def scale_bounds(v, err, fmax=448.0):
    """Row-wise and column-wise scales of the matrix v [R, C] (R any, C % 128 == 0) in
    the single-matrix layouts, each with the largest distance an fp32 evaluation
    within `err` per element can have from it:
    (s_row [C/128, R], b_row, s_col [ceil(R/128), C], b_col), all fp64."""
    R, C = v.shape
    a = v.abs().reshape(R, C // GROUP, GROUP)
    e = err.reshape(R, C // GROUP, GROUP)
    s_row, b_row = _scale_and_bound(a.amax(2).t().contiguous(), e.amax(2).t().contiguous(), fmax)
    pad = (-R) % GROUP
    va, ea = v.abs(), err
    if pad:
        va = torch.nn.functional.pad(va, (0, 0, 0, pad))
        ea = torch.nn.functional.pad(ea, (0, 0, 0, pad))
    s_col, b_col = _scale_and_bound(va.reshape(-1, GROUP, C).amax(1), ea.reshape(-1, GROUP, C).amax(1), fmax)
    return s_row, b_row, s_col, b_col


def scale_bounds_per_expert(v, err, counts, fmax=448.0):
    """The same with the per-expert packing of the batched entry points: flat
    (s_row, b_row) = per expert [C/128, c_e] blocks, flat (s_col, b_col) = per expert
    [ceil(c_e/128), C] blocks, in expert order."""
    out = [[], [], [], []]
    start = 0
    for c in counts:
        if c:
            for k, t in enumerate(scale_bounds(v[start:start + c], err[start:start + c], fmax)):
                out[k].append(t.reshape(-1))
        start += c
    return tuple(torch.cat(t) if t else torch.empty(0, dtype=torch.float64) for t in out)


def ulps_from(truth64, got32):
    """distance of fp32 values from the fp64 truth in units of the truth's fp32 ulp"""
    t32 = truth64.float()
    ulp = torch.ldexp(torch.ones_like(truth64), torch.frexp(t32.double())[1] - 24)
    return (got32.double() - truth64).abs() / ulp


def report(name, truth64, bound64, kernel32, oracle32):
    """Compare kernel and oracle scales with the truth; returns a dict of figures and
    prints one line.  Distances are in fp32 ulps of the true value (fractional: the
    truth is not an fp32 number)."""
    truth64, bound64 = truth64.reshape(-1), bound64.reshape(-1)
    k, o = kernel32.reshape(-1).cpu(), oracle32.reshape(-1).cpu()
    dk, do = ulps_from(truth64, k), ulps_from(truth64, o)
    over = (k.double() - truth64).abs() > bound64
    over_o = (o.double() - truth64).abs() > bound64
    # how the two sides differ from EACH OTHER (what a parity test against the oracle sees)
    ki = k.view(torch.int32).to(torch.int64)
    oi = o.view(torch.int32).to(torch.int64)
    dko = (ki - oi).abs()
    fig = dict(groups=int(truth64.numel()),
               kernel_max=float(dk.max()), kernel_mean=float(dk.mean()),
               oracle_max=float(do.max()), oracle_mean=float(do.mean()),
               kernel_beyond_bound=int(over.sum()), oracle_beyond_bound=int(over_o.sum()),
               kernel_nearest=float((dk <= 0.5).double().mean()), oracle_nearest=float((do <= 0.5).double().mean()),
               vs_oracle_exact=float((dko == 0).double().mean()), vs_oracle_le1=float((dko <= 1).double().mean()),
               vs_oracle_max=int(dko.max()), bound_max_ulp=float((bound64 / (truth64 * U)).max()))
    print(f"[truth] {name}: groups {fig['groups']}; kernel vs truth mean {fig['kernel_mean']:.3f} max "
          f"{fig['kernel_max']:.2f} ulp (correctly rounded {100 * fig['kernel_nearest']:.1f} %); oracle vs truth mean "
          f"{fig['oracle_mean']:.3f} max {fig['oracle_max']:.2f} ulp (correctly rounded "
          f"{100 * fig['oracle_nearest']:.1f} %); kernel vs oracle exact {100 * fig['vs_oracle_exact']:.2f} % "
          f"<=1ulp {100 * fig['vs_oracle_le1']:.2f} % max {fig['vs_oracle_max']} ulp; beyond the derived bound: "
          f"kernel {fig['kernel_beyond_bound']}, oracle {fig['oracle_beyond_bound']}", flush=True)
    return fig
