"""GPU parity tests: every entry point of the hot path, called as the reference's
own tests call theirs (tests/test_norm.py, tests/test_silu.py,
tests/test_blockwise_quant.py, tests/test_group_quant.py of the reference),
compared with the CPU oracle on identical seeded inputs.

Acceptance (stricter than the reference's output_check):
  * FP8 codes: >= 99.99 % bit-identical, every mismatch exactly one code step;
  * fp32 scales of the plain quantisers: bit-identical;
  * fp32 scales of the fused ops: oracle and kernel are two fp32 evaluations of the
    same expression, each up to 3-5 ulp from the real-number value (measured
    against fp64 in tests/test_gpu_truth.py: the kernel is as close to it as the
    oracle, closer after an RMSNorm), so they differ from EACH OTHER by up to 6 ulp.
    The limits below are the largest differences measured over every shape here
    and the benchmark configurations:
      - SwiGLU forward: none beyond 5 ulp, >= 97 % within 1 ulp (99 % at the benchmark sizes) (torch's CPU sigmoid
        is 1/(1+exp(-x)) with a vectorised 2-ulp exp, the kernel's a hardware exp2);
      - SwiGLU backward: none beyond 6 ulp, >= 97 % within 1 ulp (99 % at the benchmark sizes), except where
        dx1 = h*s + h*x1*(1-s)*s cancels (x1 near -1.28) in the element that makes a
        group's amax - a group of one or two rows of a ragged expert: there both
        sides must lie within that element's own error bound of the fp64 value;
      - RMSNorm family against the pure oracle: none beyond 6 ulp, >= 90 % within
        1 ulp (torch's CPU sum of squares is itself about one ulp from the exact
        sum, and 1/sqrt turns that into 1-2 ulp of the statistic); against the
        oracle evaluated with the kernel's own statistic: bit-identical scales and
        codes;
  * bf16 outputs: >= 99.5 % identical, the rest within 2 bf16 ulps or, where
    dx = r*g*w - coef*x cancels, within 2^-9 of the tensor's largest magnitude.
"""
import pytest
import torch

from oracle import compare as C
from oracle import fq_oracle as O
from tests import truth as T
from tests.helpers import (E4M3, E5M2, announce, check_quant_pair, gamma_bf16, gen, randn_bf16,
                           zipf_counts)

pytestmark = pytest.mark.gpu

FUSED = dict(scale_max_ulp=5, scale_min_within1=0.97)        # SwiGLU forward
FUSED_BWD = dict(scale_max_ulp=6, scale_min_within1=0.97)    # SwiGLU backward (+ the conditioned escape, see above)
FUSED_NORM = dict(scale_max_ulp=6, scale_min_within1=0.9)    # RMSNorm vs pure oracle
EXACT = dict(scale_max_ulp=0, scale_min_within1=1.0, min_identical=1.0)


def _dev(t, gpu):
    return t.to(gpu)


def check_bf16(name, ref, got, min_identical=0.995):
    got = got.detach().cpu()
    assert ref.dtype == got.dtype == torch.bfloat16 and ref.shape == got.shape
    if ref.numel() == 0:
        return
    a = ref.view(torch.int16).to(torch.int32)
    b = got.view(torch.int16).to(torch.int32)
    a = torch.where(a < 0, -(a & 0x7FFF), a)
    b = torch.where(b < 0, -(b & 0x7FFF), b)
    d = (a - b).abs()
    frac = float((d == 0).float().mean())
    print(f"[parity] {name}: bf16 identical {frac:.6f}, max {int(d.max())} ulp", flush=True)
    far = d > 2
    absdiff = (ref.float() - got.float()).abs()
    assert frac >= min_identical, (name, frac)
    assert not bool(far.any()) or float(absdiff[far].max()) <= 2.0 ** -9 * float(ref.float().abs().max()), name


# ------------------------------------------------------------------ plain quantisers
@pytest.mark.parametrize("M,N", [(256, 256), (4096, 2048), (2064, 1536)])
@pytest.mark.parametrize("round_scale", [False, True])
def test_blockwise_quant(gpu, M, N, round_scale):
    from linghe_amd.quant.block import triton_blockwise_quant

    announce("blockwise_quant", M, N, round_scale)
    x = randn_bf16(gen(11), M, N)
    ref = O.blockwise_quant(x, round_scale)
    xd = _dev(x, gpu)
    for mode in (2, 0, 1):
        q, s, qt, st = triton_blockwise_quant(xd, round_scale=round_scale, output_mode=mode)
        torch.cuda.synchronize()
        assert q.shape == (M, N) and s.shape == (N // 128, M)
        assert qt.shape == (N, M) and st.shape == ((M + 127) // 128, N)
        if mode != 1:
            check_quant_pair(f"blockwise.m{mode}.row", ref[0], ref[1], q, s, **EXACT)
        if mode != 0:
            check_quant_pair(f"blockwise.m{mode}.col", ref[2], ref[3], qt, st, **EXACT)


@pytest.mark.parametrize("dtype", [E4M3, E5M2])
def test_blockwise_quant_dequant_bound(gpu, dtype):
    from linghe_amd.quant.block import triton_blockwise_quant

    announce("blockwise_quant dequant bound", dtype)
    M, N = 512, 384
    x = randn_bf16(gen(12), M, N, scale=3.0)
    x[5, 7] = 200.0  # outlier
    q, s, qt, st = triton_blockwise_quant(_dev(x, gpu), fp8_dtype=dtype)
    torch.cuda.synchronize()
    q, s, qt, st = q.cpu(), s.cpu(), qt.cpu(), st.cpu()
    xf = x.float()
    C.assert_dequant_bound(xf, q, s.t().repeat_interleave(128, 1), dtype, "row")
    C.assert_dequant_bound(xf.t(), qt, st.t().repeat_interleave(128, 1)[:, :M], dtype, "col")
    ref = O.blockwise_quant(x, False, dtype)
    check_quant_pair("blockwise.%s.row" % dtype, ref[0], ref[1], q, s, **EXACT)
    check_quant_pair("blockwise.%s.col" % dtype, ref[2], ref[3], qt, st, **EXACT)
    # the amax element of every group is the largest code
    fmax = O.fp8_max(dtype)
    assert float(q.float().abs().reshape(M, N // 128, 128).amax(2).min()) == fmax


@pytest.mark.parametrize("round_scale", [False, True])
def test_blockwise_quant_negative_zero(gpu, round_scale):
    """Inputs holding -0.0.  The reference's x / s keeps the sign of a zero (code 0x80); the kernel's
    two-operation division returns +0 or -0 depending on the sign of the reciprocal's correction term
    (with power-of-two scales the convert divides itself and keeps the sign).  Both codes decode to
    zero and the comparison rule counts them as identical; everything else stays bit-exact."""
    from linghe_amd.quant.block import triton_blockwise_quant

    announce("blockwise_quant with -0.0 inputs", round_scale)
    M, N = 256, 384
    x = randn_bf16(gen(14), M, N)
    x.view(torch.int16)[::3, ::5] = -32768  # bf16 -0.0
    x[128:, 128:256] = 0.0
    x.view(torch.int16)[130:140, 128:256] = -32768  # an all-zero group with negative zeros: scale = the floor
    assert bool((x.view(torch.int16) == -32768).any())
    ref = O.blockwise_quant(x, round_scale)
    q, s, qt, st = triton_blockwise_quant(_dev(x, gpu), round_scale=round_scale, output_mode=2)
    torch.cuda.synchronize()
    check_quant_pair("blockwise.negzero.row", ref[0], ref[1], q, s, **EXACT)
    check_quant_pair("blockwise.negzero.col", ref[2], ref[3], qt, st, **EXACT)
    zero = (x.float() == 0)
    assert bool(((q.cpu().view(torch.uint8)[zero] & 0x7F) == 0).all())
    assert bool(((qt.cpu().view(torch.uint8).t()[zero] & 0x7F) == 0).all())


@pytest.mark.parametrize("M,N", [(2049, 2048), (64, 128), (1000, 8192 + 128)])
@pytest.mark.parametrize("round_scale", [False, True])
def test_group_quant(gpu, M, N, round_scale):
    from linghe_amd.quant.group import triton_group_quant

    announce("group_quant", M, N, round_scale)
    x = randn_bf16(gen(13), M, N)
    rq, rs = O.group_quant_1x128(x, round_scale)
    q, s = triton_group_quant(_dev(x, gpu), round_scale=round_scale)
    torch.cuda.synchronize()
    assert s.shape == (M, N // 128)
    check_quant_pair("group", rq, rs, q, s, **EXACT)
    # e5m2 codes on the 448-based scale, as the reference kernel does
    q5, s5 = triton_group_quant(_dev(x, gpu), dtype=E5M2, round_scale=round_scale)
    torch.cuda.synchronize()
    ref5 = (x.float().reshape(M, N // 128, 128) / rs.unsqueeze(-1)).to(E5M2).reshape(M, N)
    check_quant_pair("group.e5m2", ref5, rs, q5, s5, **EXACT)


@pytest.mark.parametrize("counts", [[128, 0, 256, 16, 0, 144, 1, 127], [0, 0, 0, 0], [300],
                                    [33, 65, 7, 129, 513, 2, 0, 90, 128, 128, 77, 5, 0, 0, 250, 31],
                                    # every length of a ragged transposed row modulo 16, alone and after a full block
                                    list(range(1, 17)) + [128 + r for r in range(1, 16)] + [113, 120, 126]])
def test_batch_blockwise_quant(gpu, counts):
    from linghe_amd.quant.block import triton_batch_blockwise_quant

    announce("batch_blockwise_quant", counts)
    M, N = sum(counts), 384
    x = randn_bf16(gen(14), M, N)
    ref = O.batch_blockwise_quant(x, counts, False)
    for cdt in (torch.int32, torch.int64):
        cnt = torch.tensor(counts, dtype=cdt, device=gpu)
        q, s, qt, st = triton_batch_blockwise_quant(_dev(x, gpu), cnt, counts)
        torch.cuda.synchronize()
        assert s.shape == (M * N // 128,) and qt.shape == (M * N,)
        if M == 0:
            continue
        check_quant_pair("batch_blockwise.row", ref[0], ref[1], q, s, **EXACT)
        check_quant_pair("batch_blockwise.col", ref[2], ref[3], qt, st, **EXACT)


def test_batch_blockwise_quant_more_than_1024_experts(gpu):
    """The per-expert tile lookup fetches the counts of 1024 experts at a time: with more
    experts than that (most of them tiny or empty) it takes a second round."""
    from linghe_amd.quant.block import triton_batch_blockwise_quant

    announce("batch_blockwise_quant, 1300 experts")
    rng = torch.Generator().manual_seed(15)
    counts = [int(c) for c in torch.randint(0, 40, (1300,), generator=rng)]
    counts[5], counts[1029], counts[1299] = 300, 257, 129
    M, N = sum(counts), 256
    x = randn_bf16(gen(16), M, N)
    ref = O.batch_blockwise_quant(x, counts, False)
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    q, s, qt, st = triton_batch_blockwise_quant(_dev(x, gpu), cnt, counts)
    torch.cuda.synchronize()
    check_quant_pair("batch_blockwise.1300.row", ref[0], ref[1], q, s, **EXACT)
    check_quant_pair("batch_blockwise.1300.col", ref[2], ref[3], qt, st, **EXACT)


# ------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("M,N", [(1024, 2048), (1024, 1664), (208, 1664), (512, 4096), (256, 8192),
                                 (300, 512), (64, 7168), (130, 1536), (96, 1024), (40, 128), (3, 2048),
                                 (70, 3072), (50, 6144)])
def test_rmsnorm_fwd_bwd(gpu, M, N):
    """reference tests/test_norm.py:114-145 (inputs randn**3, weight randn)."""
    from linghe_amd.utils.norm import triton_rms_norm_backward, triton_rms_norm_forward

    announce("rmsnorm fwd/bwd", M, N)
    g = gen(21)
    x = (torch.randn(M, N, generator=g) ** 3).to(torch.bfloat16)
    w = torch.randn(N, generator=g).to(torch.bfloat16)
    dy = torch.randn(M, N, generator=g).to(torch.bfloat16)
    y_ref, r_ref = O.rms_norm_forward(x, w)
    xd, wd, dyd = _dev(x, gpu), _dev(w, gpu), _dev(dy, gpu)
    y, rms = triton_rms_norm_forward(xd, wd)
    torch.cuda.synchronize()
    check_bf16("rmsnorm.y", y_ref, y)
    C.assert_scales(r_ref, rms.cpu(), "rstd", max_ulp=4, min_within_1ulp=0.9)
    y2, _ = triton_rms_norm_forward(xd, wd, rms=rms)
    torch.cuda.synchronize()
    assert torch.equal(y2.cpu(), y.cpu())
    dx_ref, dw_ref = O.rms_norm_backward(x, w, dy)
    dx, dw = triton_rms_norm_backward(dyd, xd, wd)
    torch.cuda.synchronize()
    assert dw.dtype == torch.float32 and dw.shape == (N,)
    check_bf16("rmsnorm.dx", dx_ref, dx)
    torch.testing.assert_close(dw.cpu(), dw_ref, rtol=2e-4, atol=2e-4 * float(dw_ref.abs().max()))
    # with the saved statistic: the backward's own recomputation gives the same
    # fp32 value (the sum of squares is accumulated in double in every kernel, so
    # it does not depend on how a row is split over lanes), hence identical results
    dx2, dw2 = triton_rms_norm_backward(dyd, xd, wd, rms=rms)
    torch.cuda.synchronize()
    assert torch.equal(dx2.view(torch.int16).cpu(), dx.view(torch.int16).cpu())
    assert torch.equal(dw2.cpu(), dw.cpu())
    # 3-D input
    if M % 4 == 0:
        y3, _ = triton_rms_norm_forward(xd.view(4, M // 4, N), wd)
        torch.cuda.synchronize()
        assert y3.shape == (4, M // 4, N) and torch.equal(y3.view(M, N).cpu(), y.cpu())


@pytest.mark.parametrize("M,N", [(1024, 2048), (2048, 1536), (200, 512), (136, 7168), (128, 128), (256, 4096),
                                 (64, 6144), (128, 8192), (72, 2176),
                                 # rows a multiple of 1024: both passes of mode 2 hand out the rows by XCD
                                 (3072, 256), (5120, 640), (9216, 128)])
@pytest.mark.parametrize("round_scale", [True, False])
def test_rmsnorm_and_block_quant(gpu, M, N, round_scale):
    """reference tests/test_norm.py:189-220 (x = randn**2, weight randn, modes 0, 1, 2)."""
    from linghe_amd.utils.norm import triton_rms_norm_and_block_quant_forward as fwd

    announce("rmsnorm+quant", M, N, round_scale)
    g = gen(22)
    x = (torch.randn(M, N, generator=g) ** 2).to(torch.bfloat16)
    w = torch.randn(N, generator=g).to(torch.bfloat16)
    q_ref, s_ref, r_ref, qt_ref, st_ref = O.rms_norm_and_block_quant_forward(x, w, round_scale=round_scale)
    xd, wd = _dev(x, gpu), _dev(w, gpu)
    kw = dict(FUSED_NORM)
    if round_scale:
        # power-of-two scales absorb the last-bit noise, except when the raw scale
        # sits within a few ulps of a power of two (then the two sides may pick
        # neighbouring powers): none in these inputs
        kw = dict(scale_max_ulp=0, scale_min_within1=1.0)
    q, s, rms, qt0, st0 = fwd(xd, wd, round_scale=round_scale, output_mode=0)
    torch.cuda.synchronize()
    assert qt0.shape == (N, M) and st0.shape == ((M + 127) // 128, N)
    check_quant_pair("rms.0.row", q_ref, s_ref, q, s, **kw)
    C.assert_scales(r_ref, rms.cpu(), "rstd", max_ulp=4, min_within_1ulp=0.9)
    o1, s1, rms1, qt, st = fwd(xd, wd, round_scale=round_scale, rms=rms, output_mode=1)
    torch.cuda.synchronize()
    assert o1 is None and s1 is None and rms1 is rms
    check_quant_pair("rms.1.col", qt_ref, st_ref, qt, st, **kw)
    q2, s2, rms2, qt2, st2 = fwd(xd, wd, round_scale=round_scale, output_mode=2)
    torch.cuda.synchronize()
    # mode 0 and mode 2 agree in the statistic (same statistic kernel arithmetic)
    C.assert_scales(rms.cpu(), rms2.cpu(), "rstd mode0 vs mode2", max_ulp=4, min_within_1ulp=0.9)
    C.assert_scales(r_ref, rms2.cpu(), "rstd2", max_ulp=4, min_within_1ulp=0.9)
    check_quant_pair("rms.2.row", q_ref, s_ref, q2, s2, **kw)
    check_quant_pair("rms.2.col", qt_ref, st_ref, qt2, st2, **kw)
    # with the kernel's own statistic fed to the oracle everything is bit-exact
    p_ref = O.rms_norm_and_block_quant_forward(x, w, round_scale=round_scale, rstd=rms.cpu())
    check_quant_pair("rms.pinned.col(mode1)", p_ref[3], p_ref[4], qt, st, **EXACT)
    check_quant_pair("rms.pinned.row(mode0)", p_ref[0], p_ref[1], q, s, **EXACT)
    p_ref = O.rms_norm_and_block_quant_forward(x, w, round_scale=round_scale, rstd=rms2.cpu())
    check_quant_pair("rms.pinned.row", p_ref[0], p_ref[1], q2, s2, **EXACT)
    check_quant_pair("rms.pinned.col", p_ref[3], p_ref[4], qt2, st2, **EXACT)


# ------------------------------------------------------------------ SwiGLU
@pytest.mark.parametrize("M,N,coef", [(2048, 1024, 1.0), (1024, 4096, 1.0), (1000, 1536, 1.0),
                                      (512, 1536 * 8, 100.0), (512, 1536 * 8, 0.0)])
def test_silu_and_block_quant_fwd(gpu, M, N, coef):
    """reference tests/test_silu.py:405-436."""
    from linghe_amd.utils.silu import triton_silu_and_block_quant_forward as fwd

    announce("silu+quant fwd", M, N, coef)
    x = randn_bf16(gen(31), M, N, scale=coef)
    ref = O.silu_and_block_quant_forward(x, False)
    xd = _dev(x, gpu)
    for mode in (0, 1, 2):
        q, s, qt, st = fwd(xd, round_scale=False, output_mode=mode)
        torch.cuda.synchronize()
        if mode != 1:
            check_quant_pair(f"silu.{mode}.row", ref[0], ref[1], q, s, **FUSED)
        if mode != 0:
            check_quant_pair(f"silu.{mode}.col", ref[2], ref[3], qt, st, **FUSED)


@pytest.mark.parametrize("M,N,coef,gcoef", [(2048, 1024, 1.0, 1.0), (1024, 4096, 1.0, 1e-3),
                                            (512, 1536 * 8, 100.0, 100.0), (512, 1536 * 8, 0.0, 0.0)])
@pytest.mark.parametrize("dtype", [E4M3, E5M2])
def test_silu_and_block_quant_bwd(gpu, M, N, coef, gcoef, dtype):
    """reference tests/test_silu.py:437-446; e5m2 is this build's extension."""
    from linghe_amd.utils.silu import triton_silu_and_block_quant_backward as bwd

    announce("silu+quant bwd", M, N, coef, gcoef, dtype)
    g = gen(32)
    x = randn_bf16(g, M, N, scale=coef)
    dy = randn_bf16(g, M, N // 2, scale=gcoef)
    ref = O.silu_and_block_quant_backward(dy, x, False, dtype)
    dq, ds, dqt, dst = bwd(_dev(dy, gpu), _dev(x, gpu), round_scale=False, fp8_dtype=dtype)
    torch.cuda.synchronize()
    assert dq.shape == (M, N) and ds.shape == (N // 128, M) and dqt.shape == (N, M) and dst.shape == (M // 128, N)
    assert dq.dtype == dtype
    v, err, _ = T.swiglu_grad_values(dy, x)
    sr, br, sc, bc = T.scale_bounds(v, err, O.fp8_max(dtype))
    check_quant_pair("silu.bwd.row", ref[0], ref[1], dq, ds, truth=sr, bound=br, **FUSED_BWD)
    check_quant_pair("silu.bwd.col", ref[2], ref[3], dqt, dst, truth=sc, bound=bc, **FUSED_BWD)


def _batched_case(gpu, counts, N, coef, gcoef, seed, wdtype=torch.float32):
    from linghe_amd.utils.silu import (triton_batch_weighted_silu_and_block_quant_backward as bwd,
                                       triton_batch_weighted_silu_and_block_quant_forward as fwd)

    bs = sum(counts)
    g = gen(seed)
    x = randn_bf16(g, bs, N, scale=coef)
    if bs > 3:
        x[:3] = 0.0
    w = torch.randn(bs, 1, generator=g).to(wdtype)
    dy = randn_bf16(g, bs, N // 2, scale=gcoef)
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    ref = O.batch_weighted_silu_and_block_quant_forward(x, w, counts, False)
    xd, wd, dyd = _dev(x, gpu), _dev(w, gpu), _dev(dy, gpu)
    for mode in (2, 0, 1):
        q, s, qt, st = fwd(xd, wd, cnt, counts, round_scale=False, output_mode=mode)
        torch.cuda.synchronize()
        assert q.shape == (bs, N // 2) and s.shape == (bs, N // 256) and qt.shape == (bs, N // 2)
        if bs == 0:
            continue
        if mode != 1:
            check_quant_pair(f"batch.{mode}.row", ref[0], ref[1], q, s.view(-1), **FUSED)
        if mode != 0:
            check_quant_pair(f"batch.{mode}.col", ref[2], ref[3], qt.view(-1), st.view(-1), **FUSED)
    rb = O.batch_weighted_silu_and_block_quant_backward(dy, x, w, counts, False)
    dq, ds, dw, dqt, dst = bwd(dyd, xd, wd, cnt, splits=counts, round_scale=False)
    torch.cuda.synchronize()
    assert dq.shape == (bs, N) and dw.shape == w.shape and dw.dtype == w.dtype
    if bs == 0:
        return
    v, err, _ = T.swiglu_grad_values(dy, x, w.float())
    sr, br, sc, bc = T.scale_bounds_per_expert(v, err, counts)
    check_quant_pair("batch.bwd.row", rb[0], rb[1], dq, ds.view(-1), truth=sr, bound=br, **FUSED_BWD)
    check_quant_pair("batch.bwd.col", rb[3], rb[4], dqt.view(-1), dst.view(-1), truth=sc, bound=bc, **FUSED_BWD)
    tol = 2e-2 if wdtype == torch.bfloat16 else 1e-4
    torch.testing.assert_close(dw.cpu().float(), rb[2].float(), rtol=tol,
                               atol=tol * max(float(rb[2].abs().max()), 1e-30))


@pytest.mark.parametrize("counts,N,coef,gcoef", [
    ([0] * 8, 1536, 1.0, 1.0),
    ([160, 96, 0, 272, 16, 128, 0, 64], 1024, 1.0, 1.0),
    ([144, 80, 400, 16], 1536, 100.0, 100.0),
    ([144, 80, 400, 16], 1536, 0.0, 0.0),
    ([37, 0, 129, 1, 255, 3], 512, 1.0, 1e-3),   # counts that are not multiples of 16
    (list(range(1, 17)) + [128 + r for r in (1, 2, 3, 6, 9, 12, 15)], 256, 1.0, 1.0),   # every ragged tail
    ([64, 64], 8192, 1.0, 1.0),
])
def test_batch_weighted_silu_and_block_quant(gpu, counts, N, coef, gcoef):
    """reference tests/test_silu.py:588-649 (counts multiples of 16, first 3 rows zero,
    fp32 [bs,1] weights) plus ragged counts."""
    announce("batched silu+quant", counts, N, coef, gcoef)
    _batched_case(gpu, counts, N, coef, gcoef, seed=33)


def test_batch_weighted_silu_bf16_weight_many_experts(gpu):
    announce("batched silu+quant bf16 weight, 300 experts")
    counts = zipf_counts(6000, 300, seed=5, n_empty=7)
    _batched_case(gpu, counts, 512, 1.0, 1.0, seed=34, wdtype=torch.bfloat16)


# ------------------------------------------------------------------ bf16 SwiGLU, weight block quant
@pytest.mark.parametrize("M,N,coef", [(4096, 4096, 1.0), (1000, 1536, 1.0), (33, 256, 10.0), (512, 8192, 0.0)])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16, None])
def test_weighted_silu(gpu, M, N, coef, wdtype):
    """reference tests/test_silu.py:299-329 (x randn, weight randn [M,1], grad randn)."""
    from linghe_amd.utils.silu import triton_weighted_silu_backward as bwd, triton_weighted_silu_forward as fwd

    announce("weighted silu bf16", M, N, coef, wdtype)
    g = gen(41)
    x = randn_bf16(g, M, N, scale=coef)
    dy = randn_bf16(g, M, N // 2)
    w = None if wdtype is None else torch.randn(M, 1, generator=g).to(wdtype)
    y_ref = O.weighted_silu_forward(x, None if w is None else w.float())
    xd, dyd = _dev(x, gpu), _dev(dy, gpu)
    wd = None if w is None else _dev(w, gpu)
    y = fwd(xd, wd)
    y_asm = fwd(xd, wd, asm=True, out=torch.empty_like(y))
    torch.cuda.synchronize()
    assert y.shape == (M, N // 2) and y.dtype == torch.bfloat16
    check_bf16("wsilu.y", y_ref, y)
    assert torch.equal(y.cpu().view(torch.int16), y_asm.cpu().view(torch.int16))
    dx_ref, dw_ref = O.weighted_silu_backward(dy, x, None if w is None else w.float())
    dx, dw = bwd(dyd, xd, wd)
    torch.cuda.synchronize()
    assert dx.shape == (M, N)
    check_bf16("wsilu.dx", dx_ref, dx)
    if w is None:
        assert dw is None
    else:
        assert dw.shape == w.shape and dw.dtype == w.dtype
        tol = 2e-2 if wdtype == torch.bfloat16 else 1e-4
        torch.testing.assert_close(dw.cpu().float(), dw_ref.float(), rtol=tol,
                                   atol=tol * max(float(dw_ref.abs().max()), 1e-30))


@pytest.mark.parametrize("offset", [1, 2, 3])
def test_weighted_silu_bf16_weight_view(gpu, offset):
    """A bf16 weight that starts on an odd element of its storage (a slice of a longer vector): the row
    kernels read the weight as the aligned 4-byte word that holds it, so every alignment is tried."""
    from linghe_amd.utils.silu import triton_weighted_silu_backward as bwd, triton_weighted_silu_forward as fwd

    M, N = 257, 512
    announce("weighted silu bf16, weight view at element", offset)
    g = gen(47)
    x = randn_bf16(g, M, N)
    dy = randn_bf16(g, M, N // 2)
    w = torch.randn(M, 1, generator=g).to(torch.bfloat16)
    store = torch.zeros(M + 8, 1, dtype=torch.bfloat16, device=gpu)
    wd = store[offset:offset + M]
    wd.copy_(w)
    assert wd.data_ptr() == store.data_ptr() + 2 * offset and wd.is_contiguous()
    xd, dyd = _dev(x, gpu), _dev(dy, gpu)
    y = fwd(xd, wd)
    dx, dw = bwd(dyd, xd, wd)
    torch.cuda.synchronize()
    check_bf16("wsilu.view.y", O.weighted_silu_forward(x, w.float()), y)
    dx_ref, dw_ref = O.weighted_silu_backward(dy, x, w.float())
    check_bf16("wsilu.view.dx", dx_ref, dx)
    torch.testing.assert_close(dw.cpu().float(), dw_ref.float(), rtol=2e-2, atol=2e-2 * float(dw_ref.abs().max()))


@pytest.mark.parametrize("M,N", [(8192, 4096), (128, 128), (256, 1536)])
@pytest.mark.parametrize("round_scale", [True, False])
def test_block_quant(gpu, M, N, round_scale):
    """reference tests/test_blockwise_quant.py:46-56 (x = randn**3)."""
    from linghe_amd.quant.block import triton_block_quant

    announce("block_quant 128x128", M, N, round_scale)
    g = gen(42)
    x = (torch.randn(M, N, generator=g) ** 3).to(torch.bfloat16)
    if M >= 256:
        x[128:256, :128] = 0.0
    q_ref, s_ref = O.block_quant_128(x, round_scale)
    q, s = triton_block_quant(_dev(x, gpu), round_scale=round_scale)
    torch.cuda.synchronize()
    assert s.shape == (M // 128, N // 128)
    check_quant_pair("block128", q_ref, s_ref, q, s, **EXACT)
    q5, s5 = triton_block_quant(_dev(x, gpu), round_scale=round_scale, fp8_dtype=E5M2)
    torch.cuda.synchronize()
    r5 = O.block_quant_128(x, round_scale, E5M2)
    check_quant_pair("block128.e5m2", r5[0], r5[1], q5, s5, **EXACT)


# ------------------------------------------------------------------ RMSNorm + router GEMM + quant
@pytest.mark.parametrize("M,N,K,wdtype", [
    (8192, 256, 2048, torch.bfloat16), (256, 128, 1536, torch.bfloat16), (128, 512, 4096, torch.bfloat16),
    (384, 384, 7168, torch.bfloat16), (256, 128, 1024, torch.bfloat16), (128, 256, 1024, torch.bfloat16),
    (128, 128, 2048, torch.bfloat16),
    # an fp32 router weight (what Megatron keeps), as two bf16 planes: register-resident (2N = 256) and streamed forms
    (8192, 256, 2048, torch.float32), (256, 128, 2048, torch.float32), (128, 128, 1024, torch.float32),
    (256, 256, 1536, torch.float32),
    # more than 512 (virtual) columns: one launch per chunk of 512
    (256, 1024, 2048, torch.bfloat16), (128, 640, 1536, torch.bfloat16), (128, 384, 2048, torch.float32),
    (128, 1024, 1024, torch.float32),
    # the widest router the entry point accepts: 16 launches (bf16) / 32 virtual-column chunks (fp32)
    (128, 8192, 256, torch.bfloat16), (128, 8192, 128, torch.float32)])
@pytest.mark.parametrize("round_scale", [False, True])
def test_rms_norm_fp32_gemm_block_quant(gpu, M, N, K, wdtype, round_scale):
    """reference tests/test_norm.py:251-287 (x = randn**2, weights randn; the reference's
    router weight is whatever dtype the caller holds, loaded .to(float32))."""
    from linghe_amd.utils.norm import triton_rms_norm_fp32_gemm_block_quant_forward as fn

    announce("rmsnorm + router gemm + quant", M, N, K, wdtype, round_scale)
    g = gen(24)
    x = (torch.randn(M, K, generator=g) ** 2).to(torch.bfloat16)
    nw = torch.randn(K, generator=g).to(torch.bfloat16)
    rw = torch.randn(N, K, generator=g).to(wdtype)
    xd, nwd, rwd = _dev(x, gpu), _dev(nw, gpu), _dev(rw, gpu)
    y, rms, logits, q, s, qt0, st0 = fn(xd, nwd, rwd, round_scale=round_scale, output_mode=0)
    torch.cuda.synchronize()
    assert y.shape == (M, K) and logits.shape == (M, N) and logits.dtype == torch.float32
    assert s.shape == (K // 128, M) and qt0.shape == (K, M) and st0.shape == (M // 128, K)
    ref = O.rms_gemm_block_quant_forward(x, nw, rw, round_scale=round_scale)
    C.assert_scales(ref[1], rms.cpu(), "router.rstd", max_ulp=4, min_within_1ulp=0.9)
    check_bf16("router.y", ref[0], y)
    # with the kernel's own statistic everything but the GEMM is bit-exact
    pin = O.rms_gemm_block_quant_forward(x, nw, rw, round_scale=round_scale, rstd=rms.cpu())
    assert torch.equal(pin[0].view(torch.int16), y.cpu().view(torch.int16))
    check_quant_pair("router.row", pin[3], pin[4], q, s, **EXACT)
    # logits: fp32 GEMM accuracy (the two-term bf16 splits leave < 2^-17 of each |y| and of
    # each |w| of an fp32 weight; the reference's own check allows rtol 1e-3, atol 0.1).
    # Judged against the fp64 product of the fp32 y the oracle forms.
    y32 = (x.float() * rms.cpu()[:, None]) * nw.float()
    exact = y32.double() @ rw.double().t()
    scale = float((y32.abs().double() @ rw.double().abs().t()).max())
    err = float((logits.cpu().double() - exact).abs().max())
    err_oracle = float((pin[2].double() - exact).abs().max())
    print(f"[parity] router.logits vs fp64: kernel {err:.3e}, torch fp32 matmul {err_oracle:.3e}", flush=True)
    print(f"[parity] router.logits: max abs err {err:.3e}, sum|y||w| max {scale:.3e}", flush=True)
    assert err <= 2e-5 * scale
    torch.testing.assert_close(logits.cpu(), ref[2], rtol=1e-3, atol=0.1)
    # the weight re-ordered once by the caller: bit-identical results
    from linghe_amd.utils.norm import pack_route_weight
    packed = pack_route_weight(rwd)
    yp, rmsp, logitsp, qp, sp, _, _ = fn(xd, nwd, rwd, round_scale=round_scale, output_mode=0,
                                         packed_route_weight=packed)
    torch.cuda.synchronize()
    assert torch.equal(logitsp.cpu(), logits.cpu()) and torch.equal(rmsp.cpu(), rms.cpu())
    assert torch.equal(yp.cpu().view(torch.int16), y.cpu().view(torch.int16))
    assert torch.equal(qp.cpu().view(torch.uint8), q.cpu().view(torch.uint8)) and torch.equal(sp.cpu(), s.cpu())
    # output_mode 1: the transposed copy from the saved statistic
    _, rms1, _, _, _, qt, st = fn(xd, nwd, rwd, rms=rms, round_scale=round_scale, output_mode=1)
    torch.cuda.synchronize()
    assert rms1 is rms
    check_quant_pair("router.col", pin[5], pin[6], qt, st, **EXACT)
