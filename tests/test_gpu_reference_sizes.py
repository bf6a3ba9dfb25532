"""The shapes the reference's own test scripts run, at their own row counts
(reference tests/test_norm.py:329-331 and tests/test_silu.py:714-721): RMSNorm +
blockwise quant in its three output modes, SwiGLU + blockwise quant forward (three
modes) and backward, with the reference's input recipes (x = randn**2 / randn*coef,
weight = randn, round_scale as the reference's test passes it).  Inputs are drawn in
slabs so that the host never holds more than one fp32 slab beside the bf16 tensors.
Same oracle and tolerances as the smaller cases of tests/test_gpu_parity.py."""
import pytest
import torch

from oracle import fq_oracle as O
from tests import truth as T
from tests.helpers import announce, check_quant_pair
from tests.test_gpu_parity import EXACT, FUSED, FUSED_BWD, FUSED_NORM

pytestmark = pytest.mark.gpu


def _slabs(g, M, N, fn, rows=4096):
    out = torch.empty(M, N, dtype=torch.bfloat16)
    for r0 in range(0, M, rows):
        out[r0:r0 + rows] = fn(torch.randn(min(rows, M - r0), N, generator=g)).to(torch.bfloat16)
    return out


@pytest.mark.parametrize("M,N", [(4096, 2048), (8192, 1536), (16384, 1536)])
def test_rmsnorm_and_block_quant_reference_sizes(gpu, M, N):
    """reference tests/test_norm.py:189-220 as called at :329-331 (round_scale=True there;
    the unrounded scales are checked too)."""
    from linghe_amd.utils.norm import triton_rms_norm_and_block_quant_forward as fwd

    announce("rmsnorm+quant at the reference's size", M, N)
    g = torch.Generator().manual_seed(2200 + N)
    x = _slabs(g, M, N, lambda t: t ** 2)
    w = torch.randn(N, generator=g).to(torch.bfloat16)
    xd, wd = x.to(gpu), w.to(gpu)
    for round_scale in (True, False):
        ref = O.rms_norm_and_block_quant_forward(x, w, round_scale=round_scale)
        kw = dict(scale_max_ulp=0, scale_min_within1=1.0) if round_scale else dict(FUSED_NORM)
        q0, s0, rms, _, _ = fwd(xd, wd, round_scale=round_scale, output_mode=0)
        _, _, _, qt1, st1 = fwd(xd, wd, round_scale=round_scale, rms=rms, output_mode=1)
        q2, s2, rms2, qt2, st2 = fwd(xd, wd, round_scale=round_scale, output_mode=2)
        torch.cuda.synchronize()
        check_quant_pair("ref.rms.0.row", ref[0], ref[1], q0, s0, **kw)
        check_quant_pair("ref.rms.1.col", ref[3], ref[4], qt1, st1, **kw)
        check_quant_pair("ref.rms.2.row", ref[0], ref[1], q2, s2, **kw)
        check_quant_pair("ref.rms.2.col", ref[3], ref[4], qt2, st2, **kw)
        assert torch.equal(rms.cpu(), rms2.cpu())
        pinned = O.rms_norm_and_block_quant_forward(x, w, round_scale=round_scale, rstd=rms2.cpu())
        check_quant_pair("ref.rms.pinned.row", pinned[0], pinned[1], q2, s2, **EXACT)
        check_quant_pair("ref.rms.pinned.col", pinned[3], pinned[4], qt2, st2, **EXACT)


@pytest.mark.parametrize("M,N,coef,gcoef", [(16384, 1024, 1.0, 1.0), (8192, 4096, 1.0, 1.0), (16384, 1536, 1.0, 1.0),
                                            (4096, 1536 * 8, 1.0, 1.0), (4096, 1536 * 8, 100.0, 100.0),
                                            (4096, 1536 * 8, 0.0, 0.0)])
def test_silu_and_block_quant_reference_sizes(gpu, M, N, coef, gcoef):
    """reference tests/test_silu.py:405-446 as called at :714-721."""
    from linghe_amd.utils.silu import (triton_silu_and_block_quant_backward as bwd,
                                       triton_silu_and_block_quant_forward as fwd)

    announce("silu+quant fwd/bwd at the reference's size", M, N, coef, gcoef)
    g = torch.Generator().manual_seed(3100 + N + int(coef))
    x = _slabs(g, M, N, lambda t: t.to(torch.bfloat16) * coef)
    dy = _slabs(g, M, N // 2, lambda t: t.to(torch.bfloat16) * gcoef)
    xd, dyd = x.to(gpu), dy.to(gpu)
    ref = O.silu_and_block_quant_forward(x, False)
    for mode in (0, 1, 2):
        q, s, qt, st = fwd(xd, round_scale=False, output_mode=mode)
        torch.cuda.synchronize()
        if mode != 1:
            check_quant_pair(f"ref.silu.{mode}.row", ref[0], ref[1], q, s, **FUSED)
        if mode != 0:
            check_quant_pair(f"ref.silu.{mode}.col", ref[2], ref[3], qt, st, **FUSED)
    del ref
    rb = O.silu_and_block_quant_backward(dy, x, False)
    dq, ds, dqt, dst = bwd(dyd, xd, round_scale=False)
    torch.cuda.synchronize()
    v, err, _ = T.swiglu_grad_values(dy, x)
    sr, br, sc, bc = T.scale_bounds(v, err, 448.0)
    del v, err
    check_quant_pair("ref.silu.bwd.row", rb[0], rb[1], dq, ds, truth=sr, bound=br, **FUSED_BWD)
    check_quant_pair("ref.silu.bwd.col", rb[2], rb[3], dqt, dst, truth=sc, bound=bc, **FUSED_BWD)
