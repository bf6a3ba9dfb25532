"""Scales of the fused ops against what the mathematics fixes.

A parity test against the torch oracle compares two fp32 evaluations, each a few
roundings away from the real-number value, so it cannot tell which side a 2-6 ulp
difference belongs to.  Here every group's scale is computed in fp64 (exact sum of
squares, exact sigmoid, exact products, amax/448) for the benchmark configurations
at full size, and per group:

  (i)  the kernel's scale is within the first-order bound of an fp32 evaluation of
       the expression (tests/truth.py states the rounding budget per op; for the
       SwiGLU backward the bound follows each element's own conditioning, so a
       group whose largest element suffered cancellation is allowed exactly what
       that cancellation amplifies and nothing more);
  (ii) the kernel is no further from the true value than the torch oracle is, in
       the mean and in the maximum over all groups (small margins below, in ulps).

The figures printed by report() are the per-config histogram quoted in the design
notes.  The reference's own acceptance for scales is rtol 1e-4
(linghe/tools/check.py:43-69), about 1700 ulp.
"""
import pytest
import torch

from linghe_amd import configs
from oracle import fq_oracle as O
from tests import truth as T
from tests.helpers import announce

pytestmark = pytest.mark.gpu

# (ii): the kernel's mean distance from the truth may exceed the oracle's by this
# factor, its maximum by this many ulps (both sides are samples of rounding noise)
MEAN_MARGIN = 1.05
MAX_MARGIN_ULP = 0.5


def _judge(name, truth, bound, kernel, oracle):
    fig = T.report(name, truth, bound, kernel, oracle)
    assert fig["kernel_beyond_bound"] == 0, (name, "kernel scale outside the fp32 error bound", fig)
    assert fig["oracle_beyond_bound"] == 0, (name, "oracle scale outside the fp32 error bound: the bound is wrong", fig)
    assert fig["kernel_mean"] <= fig["oracle_mean"] * MEAN_MARGIN, (name, fig)
    assert fig["kernel_max"] <= fig["oracle_max"] + MAX_MARGIN_ULP, (name, fig)
    return fig


@pytest.mark.parametrize("cfg", ["cfg1", "cfg5b"])
def test_rmsnorm_quant_scales_vs_fp64(gpu, cfg):
    from linghe_amd.utils.norm import triton_rms_norm_and_block_quant_forward as fwd

    announce("fp64 truth", cfg)
    d = configs.cfg1_rmsnorm_quant() if cfg == "cfg1" else configs.cfg5_rmsnorm_large()
    x, w, eps = d["x"], d["gamma"], d["eps"]
    _, s, r, _, st = fwd(x.to(gpu), w.to(gpu), eps, output_mode=2)
    torch.cuda.synchronize()
    s, r, st = s.cpu(), r.cpu(), st.cpu()
    ref = O.rms_norm_and_block_quant_forward(x, w, eps)
    o_s, o_r, o_st = ref[1], ref[2], ref[4]
    del ref
    y, err, r64 = T.rmsnorm_values(x, w, eps)
    # the statistic: 5.5 U by the budget in tests/truth.py
    _judge(cfg + ".rstd", r64, 5.5 * T.U * r64, r, o_r)
    sr, br, sc, bc = T.scale_bounds(y, err)
    del y, err
    _judge(cfg + ".row", sr, br, s, o_s)
    _judge(cfg + ".col", sc, bc, st, o_st)


def test_swiglu_fwd_scales_vs_fp64(gpu):
    from linghe_amd.utils.silu import triton_silu_and_block_quant_forward as fwd

    announce("fp64 truth cfg2")
    x = configs.cfg2_swiglu_fwd()["x"]
    _, s, _, st = fwd(x.to(gpu), output_mode=2)
    torch.cuda.synchronize()
    ref = O.silu_and_block_quant_forward(x, False)
    y, err = T.swiglu_values(x)
    sr, br, sc, bc = T.scale_bounds(y, err)
    _judge("cfg2.row", sr, br, s.cpu(), ref[1])
    _judge("cfg2.col", sc, bc, st.cpu(), ref[3])


@pytest.mark.parametrize("fp8", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_swiglu_bwd_scales_vs_fp64(gpu, fp8):
    from linghe_amd.utils.silu import triton_silu_and_block_quant_backward as bwd

    announce("fp64 truth cfg4", fp8)
    d = configs.cfg4_swiglu_bwd()
    _, ds, _, dst = bwd(d["dy"].to(gpu), d["x"].to(gpu), fp8_dtype=fp8)
    torch.cuda.synchronize()
    ref = O.silu_and_block_quant_backward(d["dy"], d["x"], False, fp8)
    v, err, _ = T.swiglu_grad_values(d["dy"], d["x"])
    sr, br, sc, bc = T.scale_bounds(v, err, O.fp8_max(fp8))
    tag = "cfg4." + str(fp8).split("_")[-1]
    _judge(tag + ".row", sr, br, ds.cpu(), ref[1])
    _judge(tag + ".col", sc, bc, dst.cpu(), ref[3])


def test_batched_swiglu_scales_vs_fp64(gpu):
    from linghe_amd.utils.silu import (triton_batch_weighted_silu_and_block_quant_backward as bwd,
                                       triton_batch_weighted_silu_and_block_quant_forward as fwd)

    announce("fp64 truth cfg3 forward and backward")
    d = configs.cfg3_batched_swiglu()
    x, w, counts, dy = d["x"], d["weight"], d["counts"], d["dy"]
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    xd, wd = x.to(gpu), w.to(gpu)
    _, s, _, st = fwd(xd, wd, cnt, counts, output_mode=2)
    _, ds, dw, _, dst = bwd(dy.to(gpu), xd, wd, cnt, splits=counts)
    torch.cuda.synchronize()
    ref = O.batch_weighted_silu_and_block_quant_forward(x, w, counts, False)
    y, err = T.swiglu_values(x, w)
    sr, br, sc, bc = T.scale_bounds_per_expert(y, err, counts)
    _judge("cfg3.row", sr, br, s.cpu().view(-1), ref[1])
    _judge("cfg3.col", sc, bc, st.cpu().view(-1), ref[3])
    rb = O.batch_weighted_silu_and_block_quant_backward(dy, x, w, counts, False)
    v, err, dw64 = T.swiglu_grad_values(dy, x, w)
    sr, br, sc, bc = T.scale_bounds_per_expert(v, err, counts)
    _judge("cfg3b.row", sr, br, ds.cpu().view(-1), rb[1])
    _judge("cfg3b.col", sc, bc, dst.cpu().view(-1), rb[4])
    # dw: a sum of n fp32 products per row; both sides against the fp64 sum
    n = x.shape[1] // 2
    mag = (dy.double().abs() * (torch.sigmoid(x.double()[:, :n]) * x.double()[:, :n] * x.double()[:, n:]).abs()).sum(1)
    tol = (T.SIGMOID_K + 3 + n / 128 + 7) * T.U * mag   # per-term roundings + the sums of 8 and of n/128 partials
    assert bool(((dw.cpu().view(-1).double() - dw64).abs() <= tol).all())
    k_err = float(((dw.cpu().view(-1).double() - dw64).abs() / mag.clamp_min(1e-300)).mean())
    o_err = float(((rb[2].view(-1).double() - dw64).abs() / mag.clamp_min(1e-300)).mean())
    print(f"[truth] cfg3b.dw: mean |err| / sum|terms| kernel {k_err:.3e}, oracle {o_err:.3e}", flush=True)
