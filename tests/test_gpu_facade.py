"""The autograd callers (reference linghe/facade/norm.py:15-112,
linghe/facade/silu.py:11-170) on the GPU: mode selection from is_recomputing,
3-D <-> 2-D views, what is saved and what the backward returns, compared at
autograd level with torch autograd of the fp32 formulas.

The quantised-tensor class the callers construct is external to the reference
(TransformerEngine's Float8BlockwiseQTensor); a stand-in wrapper subclass with
the same constructor keywords takes its place here.
"""
import pytest
import torch

from oracle import fq_oracle as O
from tests.helpers import E4M3, E5M2, announce, check_quant_pair, gamma_bf16, gen, randn_bf16
from tests.test_gpu_parity import FUSED, FUSED_BWD, FUSED_NORM, check_bf16

pytestmark = pytest.mark.gpu


class FakeQTensor(torch.Tensor):
    """Carries what the facades hand to the external class; no arithmetic."""

    @staticmethod
    def __new__(cls, *, shape, dtype, requires_grad=False, **kw):
        dev = None
        for k in ("rowwise_data", "columnwise_data"):
            if kw.get(k) is not None:
                dev = kw[k].device
        return torch.Tensor._make_wrapper_subclass(cls, tuple(shape), dtype=dtype, device=dev,
                                                   requires_grad=requires_grad)

    def __init__(self, **kw):
        self.kw = kw

    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        raise NotImplementedError(str(func))


class Quantizer:
    def __init__(self, pow2=False, dtype=E4M3):
        self.force_pow_2_scales = pow2
        self.dtype = dtype


class Capture(torch.autograd.Function):
    """identity whose backward keeps the incoming gradient object"""
    box = {}

    @staticmethod
    def forward(ctx, x):
        return x.view_as(x)

    @staticmethod
    def backward(ctx, g):
        Capture.box["grad"] = g
        return None


def test_rms_norm_function(gpu):
    from linghe_amd.facade.norm import rms_norm

    announce("facade rms_norm autograd")
    g = gen(51)
    x = randn_bf16(g, 512, 1536)
    w = gamma_bf16(g, 1536)
    dy = randn_bf16(g, 512, 1536)
    xd = x.to(gpu).requires_grad_()
    wd = w.to(gpu).requires_grad_()
    y = rms_norm(xd, wd)
    y.backward(dy.to(gpu))
    torch.cuda.synchronize()
    y_ref, _ = O.rms_norm_forward(x, w)
    dx_ref, dw_ref = O.rms_norm_backward(x, w, dy)
    check_bf16("facade.rms_norm.y", y_ref, y)
    check_bf16("facade.rms_norm.dx", dx_ref, xd.grad)
    # the weight gradient arrives in fp32 and autograd casts it to the bf16 parameter
    torch.testing.assert_close(wd.grad.float().cpu(), dw_ref, rtol=1e-2, atol=1e-2 * float(dw_ref.abs().max()))


@pytest.mark.parametrize("is_recomputing", [None, False, True])
@pytest.mark.parametrize("pow2", [False, True])
def test_block_rms_norm(gpu, is_recomputing, pow2):
    from linghe_amd.facade.norm import block_rms_norm

    announce("facade BlockRMSNorm", is_recomputing, pow2)
    S, B, H = 64, 4, 2048
    g = gen(52)
    x = randn_bf16(g, S, B, H)
    w = gamma_bf16(g, H)
    dy = randn_bf16(g, S, B, H)
    x2 = x.view(S * B, H)
    ref = O.rms_norm_and_block_quant_forward(x2, w, round_scale=pow2)
    xd = x.to(gpu).requires_grad_()
    wd = w.to(gpu).requires_grad_()
    rms_in = None
    if is_recomputing:
        rms_in = ref[2].to(gpu)  # the saved statistic of the first forward
    out, rms = block_rms_norm(xd, wd, rms_in, Quantizer(pow2), FakeQTensor, is_recomputing=is_recomputing)
    torch.cuda.synchronize()
    assert isinstance(out, FakeQTensor) and tuple(out.shape) == (S, B, H) and out.dtype == torch.bfloat16
    assert not rms.requires_grad and rms.shape == (S * B,)
    kw = out.kw
    assert kw["is_2D_scaled"] is False and kw["fp8_dtype"] == E4M3 and kw["requires_grad"] is True
    tol = dict(scale_max_ulp=0, scale_min_within1=1.0) if pow2 else FUSED_NORM
    if is_recomputing:  # transposed copy only; row-wise members stay None
        assert kw["rowwise_data"] is None and kw["rowwise_scale_inv"] is None
        assert rms is not None and torch.equal(rms.cpu(), ref[2])
        exact = dict(scale_max_ulp=0, scale_min_within1=1.0, min_identical=1.0)
        assert tuple(kw["columnwise_data"].shape) == (H, S, B)
        check_quant_pair("facade.rms.col", ref[3], ref[4], kw["columnwise_data"].reshape(H, S * B),
                         kw["columnwise_scale_inv"], **exact)
    else:
        assert tuple(kw["rowwise_data"].shape) == (S, B, H)
        check_quant_pair("facade.rms.row", ref[0], ref[1], kw["rowwise_data"].view(S * B, H),
                         kw["rowwise_scale_inv"], **tol)
        assert tuple(kw["columnwise_data"].shape) == (H, S, B)
        if is_recomputing is None:
            check_quant_pair("facade.rms.col", ref[3], ref[4], kw["columnwise_data"].reshape(H, S * B),
                             kw["columnwise_scale_inv"], **tol)
    # backward is the bf16 RMSNorm backward
    torch.autograd.backward([out], [dy.to(gpu)])
    torch.cuda.synchronize()
    dx_ref, dw_ref = O.rms_norm_backward(x2, w, dy.view(S * B, H))
    assert xd.grad.shape == (S, B, H)
    check_bf16("facade.rms.dx", dx_ref, xd.grad.view(S * B, H))
    torch.testing.assert_close(wd.grad.float().cpu(), dw_ref, rtol=1e-2, atol=1e-2 * float(dw_ref.abs().max()))


class TEDType:
    """stands in for TransformerEngine's DType enum members (matched by name)"""

    def __init__(self, name):
        self.name = name


@pytest.mark.parametrize("pow2", [False, True])
@pytest.mark.parametrize("gdtype,gtag", [(E4M3, E4M3), (E5M2, E5M2), (E5M2, TEDType("kFloat8E5M2"))])
def test_block_silu(gpu, pow2, gdtype, gtag):
    """The backward's codes are in the gradient quantizer's FP8 format (e5m2 is not
    in the reference, whose backward writes e4m3 bytes whatever the label says)."""
    from linghe_amd.facade.silu import block_silu_impl

    announce("facade BlockSiluFunction", pow2, gdtype)
    S, B, H = 128, 2, 2048
    g = gen(53)
    x = randn_bf16(g, S, B, H)
    dy = randn_bf16(g, S, B, H // 2, scale=1e-2)
    x2 = x.view(S * B, H)
    ref = O.silu_and_block_quant_forward(x2, pow2)
    leaf = x.to(gpu).requires_grad_()
    xin = Capture.apply(leaf)
    out = block_silu_impl(xin, Quantizer(pow2), Quantizer(pow2, gtag), FakeQTensor)
    torch.cuda.synchronize()
    assert isinstance(out, FakeQTensor) and tuple(out.shape) == (S, B, H // 2)
    kw = out.kw
    assert tuple(kw["rowwise_data"].shape) == (S, B, H // 2) and tuple(kw["columnwise_data"].shape) == (H // 2, S, B)
    tol = dict(scale_max_ulp=0, scale_min_within1=1.0) if pow2 else FUSED
    check_quant_pair("facade.silu.row", ref[0], ref[1], kw["rowwise_data"].view(S * B, H // 2),
                     kw["rowwise_scale_inv"], **tol)
    check_quant_pair("facade.silu.col", ref[2], ref[3], kw["columnwise_data"].reshape(H // 2, S * B),
                     kw["columnwise_scale_inv"], **tol)
    Capture.box.clear()
    torch.autograd.backward([out], [dy.to(gpu)])
    torch.cuda.synchronize()
    gq = Capture.box["grad"]
    assert isinstance(gq, FakeQTensor) and tuple(gq.shape) == (S, B, H)
    rb = O.silu_and_block_quant_backward(dy.view(S * B, H // 2), x2, pow2, gdtype)
    gk = gq.kw
    assert gk["fp8_dtype"] is gtag and gk["rowwise_data"].dtype == gdtype and gk["columnwise_data"].dtype == gdtype
    assert tuple(gk["rowwise_data"].shape) == (S, B, H) and tuple(gk["columnwise_data"].shape) == (H, S, B)
    tolb = dict(scale_max_ulp=0, scale_min_within1=1.0) if pow2 else FUSED_BWD
    check_quant_pair("facade.silu.bwd.row", rb[0], rb[1], gk["rowwise_data"].view(S * B, H),
                     gk["rowwise_scale_inv"], **tolb)
    check_quant_pair("facade.silu.bwd.col", rb[2], rb[3], gk["columnwise_data"].reshape(H, S * B),
                     gk["columnwise_scale_inv"], **tolb)


@pytest.mark.parametrize("with_plan", [False, True])
@pytest.mark.parametrize("is_recomputing,gdtype", [(None, E4M3), (False, E4M3), (True, E4M3), (None, E5M2)])
def test_block_batch_weighted_silu(gpu, is_recomputing, gdtype, with_plan):
    from linghe_amd.facade.silu import block_batch_weighted_silu_impl
    from linghe_amd.utils.silu import build_expert_plan

    announce("facade BlockBatchWeightedSiluFunction", is_recomputing, gdtype, with_plan)
    counts = [160, 0, 96, 272, 16, 128, 33, 64]
    bs, N = sum(counts), 1024
    g = gen(54)
    x = randn_bf16(g, bs, N)
    w = torch.rand(bs, 1, generator=g)
    dy = randn_bf16(g, bs, N // 2, scale=1e-2)
    ref = O.batch_weighted_silu_and_block_quant_forward(x, w, counts, False)
    leaf = x.to(gpu).requires_grad_()
    wd = w.to(gpu).requires_grad_()
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    qs = [Quantizer() for _ in counts]
    gqs = [Quantizer(dtype=gdtype) for _ in counts]
    # a tile plan built once from the counts serves the forward and, kept by the function, the backward
    plan = build_expert_plan(cnt, counts) if with_plan else None
    out = block_batch_weighted_silu_impl(Capture.apply(leaf), wd, cnt, counts, qs, gqs, FakeQTensor,
                                         is_recomputing=is_recomputing, plan=plan)
    torch.cuda.synchronize()
    assert isinstance(out, FakeQTensor) and tuple(out.shape) == (bs, N // 2)
    kw = out.kw
    assert kw["quantizer"] is qs
    if is_recomputing is not True:
        check_quant_pair("facade.batch.row", ref[0], ref[1], kw["rowwise_data"], kw["rowwise_scale_inv"].view(-1),
                         **FUSED)
    if is_recomputing is not False:
        check_quant_pair("facade.batch.col", ref[2], ref[3], kw["columnwise_data"].view(-1),
                         kw["columnwise_scale_inv"].view(-1), **FUSED)
    Capture.box.clear()
    torch.autograd.backward([out], [dy.to(gpu)])
    torch.cuda.synchronize()
    gq = Capture.box["grad"]
    rb = O.batch_weighted_silu_and_block_quant_backward(dy, x, w, counts, False, gdtype)
    assert isinstance(gq, FakeQTensor) and tuple(gq.shape) == (bs, N)
    assert gq.kw["quantizer"] is gqs and gq.kw["fp8_dtype"] == gdtype and gq.kw["rowwise_data"].dtype == gdtype
    check_quant_pair("facade.batch.bwd.row", rb[0], rb[1], gq.kw["rowwise_data"],
                     gq.kw["rowwise_scale_inv"].view(-1), **FUSED_BWD)
    check_quant_pair("facade.batch.bwd.col", rb[3], rb[4], gq.kw["columnwise_data"].view(-1),
                     gq.kw["columnwise_scale_inv"].view(-1), **FUSED_BWD)
    assert wd.grad.shape == (bs, 1) and wd.grad.dtype == torch.float32
    torch.testing.assert_close(wd.grad.cpu(), rb[2], rtol=1e-4, atol=1e-4 * float(rb[2].abs().max()))


def test_entry_points_under_graph_capture(gpu):
    """The library only enqueues work on the given stream, so its calls can be
    captured into a graph: every replay (with eager work and synchronisations in
    between) must reproduce the eager results bit for bit."""
    from linghe_amd.quant.block import triton_blockwise_quant
    from linghe_amd.utils.norm import triton_rms_norm_and_block_quant_forward, triton_rms_norm_backward
    from linghe_amd.utils.silu import (build_expert_plan, triton_batch_weighted_silu_and_block_quant_forward,
                                       triton_silu_and_block_quant_backward)

    announce("graph capture and replay")
    g = gen(55)
    M, N = 512, 1024
    x = randn_bf16(g, M, N).to(gpu)
    x2 = randn_bf16(g, M, N).to(gpu)
    w = gamma_bf16(g, N).to(gpu)
    dy = randn_bf16(g, M, N // 2).to(gpu)
    counts = [100, 0, 156, 256]
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    rw = torch.rand(M, 1, generator=g).to(gpu)

    def run(inp):
        a = triton_rms_norm_and_block_quant_forward(inp, w)
        b = triton_silu_and_block_quant_backward(dy, inp)
        c = triton_batch_weighted_silu_and_block_quant_forward(inp, rw, cnt, counts)
        d = triton_rms_norm_backward(inp, inp, w)
        e = triton_blockwise_quant(inp)
        # the tile plan is one more launch on the stream, and the planned kernels only read it
        plan = build_expert_plan(cnt, counts)
        f = triton_batch_weighted_silu_and_block_quant_forward(inp, rw, cnt, counts, plan=plan)
        return [t for grp in (a, b, c, d, e, f) for t in grp]

    def bits(ts):
        return [t.detach().clone().view(torch.uint8) if t.dtype != torch.float32 else t.detach().clone() for t in ts]

    eager1, eager2 = bits(run(x)), bits(run(x2))
    torch.cuda.synchronize()
    static_in = x.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(static_in)  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run(static_in)
    for rep, (src, want) in enumerate(((x, eager1), (x2, eager2), (x, eager1), (x2, eager2))):
        static_in.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        got = bits(outs)
        for k, (a, b) in enumerate(zip(want, got)):
            assert torch.equal(a, b), (rep, k)
        _ = (src.float() * 2).sum().item()  # eager work between the replays
