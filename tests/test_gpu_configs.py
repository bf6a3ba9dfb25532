"""The five benchmark configurations at full size: the GPU result of every timed
entry point against the CPU oracle on the same seeded inputs (the generators in
linghe_amd/configs.py are the ones bench.py times), plus properties that hold at
any size:
  * output_mode 0 and output_mode 1 together reproduce output_mode 2 bit for bit;
  * without scale rounding the largest code magnitude of every 1x128 / 128x1
    group is the format's maximum (the amax element divides to exactly fmax);
  * the row-wise and the column-wise quantisation of the same value dequantise to
    within the sum of their two half steps of each other.
"""
import pytest
import torch

from linghe_amd import configs
from oracle import compare as C
from oracle import fq_oracle as O
from tests.helpers import E4M3, E5M2, announce, check_quant_pair
from tests.test_gpu_parity import FUSED, FUSED_BWD, FUSED_NORM, check_bf16

pytestmark = pytest.mark.gpu


def _same_bits(a, b):
    return torch.equal(a.view(torch.uint8) if a.dtype != torch.float32 else a,
                       b.view(torch.uint8) if b.dtype != torch.float32 else b)


def _group_max_is_fmax(q, s_rowmajor_groups, fmax, name):
    """q: [R, K] codes quantised along K in groups of 128; s: [R, K/128]."""
    R, K = q.shape
    a = q.float().abs().reshape(R, K // 128, 128).amax(2)
    live = s_rowmajor_groups > 1e-30
    assert bool((a[live] == fmax).all()), name


def _row_col_consistent(q, s, qt, st, dtype, name, rows=1024):
    """dequantised row-wise and column-wise copies agree within their half steps
    (checked on the first `rows` rows)."""
    M, n = q.shape
    R = min(rows, M) // 128 * 128
    if R == 0:
        return
    qr = q[:R].float()
    sr = s[:, :R].t().repeat_interleave(128, 1)            # [R, n]
    qc = qt[:, :R].float().t()                             # [R, n]
    sc = st[: R // 128].repeat_interleave(128, 0)          # [R, n]
    hr = C.fp8_half_step(qr, dtype) * sr
    hc = C.fp8_half_step(qc, dtype) * sc
    gap = (qr * sr - qc * sc).abs()
    assert bool((gap <= (hr + hc) * (1 + 2.0 ** -12)).all()), name


def test_cfg1_rmsnorm_quant_full(gpu):
    from linghe_amd.utils.norm import triton_rms_norm_and_block_quant_forward as fwd

    announce("cfg1 full size")
    d = configs.cfg1_rmsnorm_quant()
    x, w = d["x"], d["gamma"]
    ref = O.rms_norm_and_block_quant_forward(x, w, d["eps"])
    xd, wd = x.to(gpu), w.to(gpu)
    q, s, r, qt, st = fwd(xd, wd, d["eps"], output_mode=2)
    q0, s0, r0, _, _ = fwd(xd, wd, d["eps"], output_mode=0)
    _, _, _, qt1, st1 = fwd(xd, wd, d["eps"], rms=r, output_mode=1)
    torch.cuda.synchronize()
    check_quant_pair("cfg1.row", ref[0], ref[1], q, s, **FUSED_NORM)
    check_quant_pair("cfg1.col", ref[3], ref[4], qt, st, **FUSED_NORM)
    C.assert_scales(ref[2], r.cpu(), "cfg1.rstd", max_ulp=4, min_within_1ulp=0.9)
    pinned = O.rms_norm_and_block_quant_forward(x, w, d["eps"], rstd=r.cpu())
    check_quant_pair("cfg1.pinned.row", pinned[0], pinned[1], q, s, scale_max_ulp=0, min_identical=1.0)
    check_quant_pair("cfg1.pinned.col", pinned[3], pinned[4], qt, st, scale_max_ulp=0, min_identical=1.0)
    for a, b in ((q, q0), (s, s0), (r, r0), (qt, qt1), (st, st1)):
        assert _same_bits(a.cpu(), b.cpu())
    qc, sc, qtc, stc = q.cpu(), s.cpu(), qt.cpu(), st.cpu()
    _group_max_is_fmax(qc, sc.t(), 448.0, "cfg1 row groups")
    _group_max_is_fmax(qtc, stc.t(), 448.0, "cfg1 column groups")
    _row_col_consistent(qc, sc, qtc, stc, E4M3, "cfg1 row/col")
    # dequantised codes sit within half a code step of the normalised value the
    # kernel quantised (the oracle's value evaluated with the kernel's statistic)
    y = (x.float() * r.cpu()[:, None]) * w.float()
    C.assert_dequant_bound(y, qc, sc.t().repeat_interleave(128, 1), E4M3, "cfg1 dequant")


def test_cfg2_swiglu_fwd_full(gpu):
    from linghe_amd.utils.silu import triton_silu_and_block_quant_forward as fwd

    announce("cfg2 full size")
    x = configs.cfg2_swiglu_fwd()["x"]
    ref = O.silu_and_block_quant_forward(x, False)
    xd = x.to(gpu)
    q, s, qt, st = fwd(xd, output_mode=2)
    q0, s0, _, _ = fwd(xd, output_mode=0)
    _, _, qt1, st1 = fwd(xd, output_mode=1)
    torch.cuda.synchronize()
    check_quant_pair("cfg2.row", ref[0], ref[1], q, s, **FUSED)
    check_quant_pair("cfg2.col", ref[2], ref[3], qt, st, **FUSED)
    for a, b in ((q, q0), (s, s0), (qt, qt1), (st, st1)):
        assert _same_bits(a.cpu(), b.cpu())
    qc, sc, qtc, stc = q.cpu(), s.cpu(), qt.cpu(), st.cpu()
    _group_max_is_fmax(qc, sc.t(), 448.0, "cfg2 row groups")
    _group_max_is_fmax(qtc, stc.t(), 448.0, "cfg2 column groups")
    _row_col_consistent(qc, sc, qtc, stc, E4M3, "cfg2 row/col")


def test_cfg3_batched_swiglu_full(gpu):
    from linghe_amd.utils.silu import (triton_batch_weighted_silu_and_block_quant_backward as bwd,
                                       triton_batch_weighted_silu_and_block_quant_forward as fwd)

    announce("cfg3 full size (forward and backward)")
    d = configs.cfg3_batched_swiglu()
    x, w, counts, dy = d["x"], d["weight"], d["counts"], d["dy"]
    assert sum(counts) == 65536 and min(counts) == 0 and len(counts) == 256
    ref = O.batch_weighted_silu_and_block_quant_forward(x, w, counts, False)
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    xd, wd, dyd = x.to(gpu), w.to(gpu), dy.to(gpu)
    q, s, qt, st = fwd(xd, wd, cnt, counts, output_mode=2)
    q0, s0, _, _ = fwd(xd, wd, cnt, counts, output_mode=0)
    _, _, qt1, st1 = fwd(xd, wd, cnt, counts, output_mode=1)
    torch.cuda.synchronize()
    check_quant_pair("cfg3.row", ref[0], ref[1], q, s.view(-1), **FUSED)
    check_quant_pair("cfg3.col", ref[2], ref[3], qt.view(-1), st.view(-1), **FUSED)
    for a, b in ((q, q0), (s, s0), (qt, qt1), (st, st1)):
        assert _same_bits(a.cpu(), b.cpu())
    rb = O.batch_weighted_silu_and_block_quant_backward(dy, x, w, counts, False)
    dq, ds, dw, dqt, dst = bwd(dyd, xd, wd, cnt, splits=counts)
    torch.cuda.synchronize()
    check_quant_pair("cfg3.bwd.row", rb[0], rb[1], dq, ds.view(-1), **FUSED_BWD)
    check_quant_pair("cfg3.bwd.col", rb[3], rb[4], dqt.view(-1), dst.view(-1), **FUSED_BWD)
    torch.testing.assert_close(dw.cpu(), rb[2], rtol=1e-4, atol=1e-4 * float(rb[2].abs().max()))
    # the same calls with the tiles read from a plan: every output byte for byte
    from linghe_amd.quant.block import triton_batch_blockwise_quant
    from linghe_amd.utils.silu import build_expert_plan

    plan = build_expert_plan(cnt, counts)
    planned = fwd(xd, wd, cnt, counts, output_mode=2, plan=plan) + bwd(dyd, xd, wd, cnt, splits=counts, plan=plan)
    torch.cuda.synchronize()
    for a, b in zip((q, s, qt, st, dq, ds, dw, dqt, dst), planned):
        assert _same_bits(a.cpu(), b.cpu())
    y = dyd  # 65536 x 512 bf16: the per-expert quantiser on a matrix of the activations' shape
    for a, b in zip(triton_batch_blockwise_quant(y, cnt, counts), triton_batch_blockwise_quant(y, cnt, counts, plan=plan)):
        assert _same_bits(a.cpu(), b.cpu())


@pytest.mark.parametrize("dtype", [E4M3, E5M2])
def test_cfg4_swiglu_bwd_full(gpu, dtype):
    from linghe_amd.utils.silu import triton_silu_and_block_quant_backward as bwd

    announce("cfg4 full size", dtype)
    d = configs.cfg4_swiglu_bwd()
    ref = O.silu_and_block_quant_backward(d["dy"], d["x"], False, dtype)
    dq, ds, dqt, dst = bwd(d["dy"].to(gpu), d["x"].to(gpu), fp8_dtype=dtype)
    torch.cuda.synchronize()
    check_quant_pair("cfg4.row", ref[0], ref[1], dq, ds, **FUSED_BWD)
    check_quant_pair("cfg4.col", ref[2], ref[3], dqt, dst, **FUSED_BWD)
    qc, sc, qtc, stc = dq.cpu(), ds.cpu(), dqt.cpu(), dst.cpu()
    fmax = O.fp8_max(dtype)
    _group_max_is_fmax(qc, sc.t(), fmax, "cfg4 row groups")
    _group_max_is_fmax(qtc, stc.t(), fmax, "cfg4 column groups")
    _row_col_consistent(qc, sc, qtc, stc, dtype, "cfg4 row/col")


def test_cfg5_rmsnorm_large_full(gpu):
    from linghe_amd.utils.norm import (triton_rms_norm_and_block_quant_forward as fwd,
                                       triton_rms_norm_backward as bwd)

    announce("cfg5 full size (backward, forward mode 2, recompute mode 1)")
    d = configs.cfg5_rmsnorm_large()
    x, w, dy, eps = d["x"], d["gamma"], d["dy"], d["eps"]
    xd, wd, dyd = x.to(gpu), w.to(gpu), dy.to(gpu)
    # 5b / 5c
    q, s, r, qt, st = fwd(xd, wd, eps, output_mode=2)
    _, _, _, qt1, st1 = fwd(xd, wd, eps, rms=r, output_mode=1)
    torch.cuda.synchronize()
    ref = O.rms_norm_and_block_quant_forward(x, w, eps)
    # 7168 heavy-tailed terms per row: torch's CPU sum is about one ulp from the exact
    # sum of squares (the kernel's is the exact sum rounded once), and 1/sqrt(ss/n + eps)
    # turns that into up to 2 ulps of the statistic in ~7 % of the rows
    tol = dict(FUSED_NORM)
    check_quant_pair("cfg5b.row", ref[0], ref[1], q, s, **tol)
    check_quant_pair("cfg5b.col", ref[3], ref[4], qt, st, **tol)
    C.assert_scales(ref[2], r.cpu(), "cfg5.rstd", max_ulp=4, min_within_1ulp=0.9)
    del ref
    pinned = O.rms_norm_and_block_quant_forward(x, w, eps, rstd=r.cpu())
    check_quant_pair("cfg5b.pinned.row", pinned[0], pinned[1], q, s, scale_max_ulp=0, min_identical=1.0)
    check_quant_pair("cfg5b.pinned.col", pinned[3], pinned[4], qt, st, scale_max_ulp=0, min_identical=1.0)
    del pinned
    assert _same_bits(qt.cpu(), qt1.cpu()) and _same_bits(st.cpu(), st1.cpu())
    del q, s, qt, st, qt1, st1
    # 5a
    dx, dg = bwd(dyd, xd, wd, eps)
    torch.cuda.synchronize()
    dx_ref, dg_ref = O.rms_norm_backward(x, w, dy, eps)
    check_bf16("cfg5a.dx", dx_ref, dx)
    torch.testing.assert_close(dg.cpu(), dg_ref, rtol=2e-4, atol=2e-4 * float(dg_ref.abs().max()))
    # linearity in the gradient: backward(2 dy) == 2 backward(dy) exactly (powers of
    # two commute with every rounding on the way)
    dx2, dg2 = bwd(dyd * 2, xd, wd, eps)
    torch.cuda.synchronize()
    assert torch.equal((dx.float() * 2).cpu(), dx2.float().cpu())
    assert torch.equal((dg * 2).cpu(), dg2.cpu())


def test_reference_batched_shape_32_experts(gpu):
    """The reference's own largest batched case (tests/test_silu.py:730-741): 32 experts of
    1024..3072 rows (multiples of 16), 8192-wide input.  The whole problem runs on the GPU;
    the oracle checks four experts (first, second, the smallest and the last), whose outputs
    are independent slices of the packed layouts, forward and backward."""
    import random

    from linghe_amd.utils.silu import (triton_batch_weighted_silu_and_block_quant_backward as bwd,
                                       triton_batch_weighted_silu_and_block_quant_forward as fwd)

    announce("reference batched shape: 32 experts x ~2048 rows x 8192")
    rnd = random.Random(7)
    M0, N, E = 2048, 8192, 32
    counts = [rnd.randint(M0 // 2, M0 // 2 * 3) // 16 * 16 for _ in range(E)]
    bs, n = sum(counts), N // 2
    g = torch.Generator().manual_seed(735)
    x = torch.empty(bs, N, dtype=torch.bfloat16)
    for r0 in range(0, bs, 8192):  # in slabs, to bound host memory
        x[r0:r0 + 8192] = torch.randn(min(8192, bs - r0), N, generator=g).to(torch.bfloat16)
    x[:3] = 0.0
    w = torch.randn(bs, 1, generator=g)
    dy = torch.empty(bs, n, dtype=torch.bfloat16)
    for r0 in range(0, bs, 8192):
        dy[r0:r0 + 8192] = torch.randn(min(8192, bs - r0), n, generator=g).to(torch.bfloat16)
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    xd, wd, dyd = x.to(gpu), w.to(gpu), dy.to(gpu)
    q, s, qt, st = fwd(xd, wd, cnt, counts, output_mode=2)
    dq, ds, dw, dqt, dst = bwd(dyd, xd, wd, cnt, splits=counts)
    torch.cuda.synchronize()
    assert q.shape == (bs, n) and dq.shape == (bs, N) and dw.shape == (bs, 1)
    q, s, qt, st = q.cpu(), s.cpu().view(-1), qt.cpu().view(-1), st.cpu().view(-1)
    dq, ds, dw, dqt, dst = dq.cpu(), ds.cpu().view(-1), dw.cpu(), dqt.cpu().view(-1), dst.cpu().view(-1)
    starts = [sum(counts[:e]) for e in range(E)]
    tblocks = [sum((c + 127) // 128 for c in counts[:e]) for e in range(E)]
    for e in sorted({0, 1, counts.index(min(counts)), E - 1}):
        si, ce, tb = starts[e], counts[e], tblocks[e]
        nblk = (ce + 127) // 128
        xe, we, dye = x[si:si + ce], w[si:si + ce], dy[si:si + ce]
        ref = O.batch_weighted_silu_and_block_quant_forward(xe, we, [ce], False)
        check_quant_pair(f"ref32.e{e}.row", ref[0], ref[1], q[si:si + ce], s[si * (n // 128):(si + ce) * (n // 128)],
                         **FUSED)
        check_quant_pair(f"ref32.e{e}.col", ref[2], ref[3], qt[si * n:(si + ce) * n], st[tb * n:(tb + nblk) * n],
                         **FUSED)
        rb = O.batch_weighted_silu_and_block_quant_backward(dye, xe, we, [ce], False)
        check_quant_pair(f"ref32.e{e}.bwd.row", rb[0], rb[1], dq[si:si + ce],
                         ds[si * (N // 128):(si + ce) * (N // 128)], **FUSED_BWD)
        check_quant_pair(f"ref32.e{e}.bwd.col", rb[3], rb[4], dqt[si * N:(si + ce) * N],
                         dst[tb * N:(tb + nblk) * N], **FUSED_BWD)
        torch.testing.assert_close(dw[si:si + ce], rb[2], rtol=1e-4, atol=1e-4 * float(rb[2].abs().max()))
    # every 1x128 group of every expert reaches the format's maximum: no group was skipped or
    # mis-scaled (the first three rows are zero rows)
    _group_max_is_fmax(q[3:], torch.ones(bs - 3, n // 128), 448.0, "ref32 row groups")
