"""Consumer-side check of the emitted layouts: the (codes, scale_inv) pairs are
fed to a plain blockwise-scaled FP8 GEMM written with torch ops on the GPU
(the arithmetic of the reference's linghe/gemm/blockwise_fp8_gemm.py:106-183,
indexed for the layouts this path emits: activations 1x128 with scales
[K/128, M], weights 128x128 with scales [N/128, K/128], transposed copies 128x1
with scales [M/128, width]) and the products are compared with the fp32 GEMM of
the unquantised operands.  A transposed or mis-strided scale tensor fails this
by orders of magnitude; the bound itself is the FP8 quantisation noise."""
import pytest
import torch

from tests.helpers import announce, gen, randn_bf16

pytestmark = pytest.mark.gpu


def _rel(a, b):
    return float((a - b).norm() / b.norm())


def _fprop(x_q, x_s, w_q, w_s):
    """y[m, n] = sum over 128-wide k blocks of (x_q[m, kb] . w_q[n, kb]) * x_s[kb, m] * w_s[n/128, kb]"""
    M, K = x_q.shape
    N = w_q.shape[0]
    y = torch.zeros((M, N), device=x_q.device, dtype=torch.float32)
    for kb in range(K // 128):
        part = x_q[:, kb * 128:(kb + 1) * 128].float() @ w_q[:, kb * 128:(kb + 1) * 128].float().t()
        y += part * x_s[kb][:, None] * w_s[:, kb].repeat_interleave(128)[None, :]
    return y


def _wgrad(at_q, at_s, bt_q, bt_s):
    """(a^T b)[i, j] = sum over 128-row m blocks of (at_q[i, mb] . bt_q[j, mb]) * at_s[mb, i] * bt_s[mb, j]"""
    I, M = at_q.shape
    J = bt_q.shape[0]
    out = torch.zeros((I, J), device=at_q.device, dtype=torch.float32)
    for mb in range(M // 128):
        part = at_q[:, mb * 128:(mb + 1) * 128].float() @ bt_q[:, mb * 128:(mb + 1) * 128].float().t()
        out += part * at_s[mb][:, None] * bt_s[mb][None, :]
    return out


@pytest.mark.parametrize("round_scale", [False, True])
def test_blockwise_gemm_consumes_the_layouts(gpu, round_scale):
    from linghe_amd.quant.block import triton_block_quant, triton_blockwise_quant
    from linghe_amd.utils.norm import triton_rms_norm_and_block_quant_forward
    from linghe_amd.utils.silu import triton_silu_and_block_quant_backward, triton_silu_and_block_quant_forward

    announce("layout validation through a blockwise-scaled GEMM", round_scale)
    g = gen(71)
    M, K, N = 512, 1024, 768
    x = randn_bf16(g, M, K).to(gpu)
    w = randn_bf16(g, N, K, scale=0.05).to(gpu)
    dy = randn_bf16(g, M, N, scale=1e-2).to(gpu)
    x_q, x_s, xt_q, xt_s = triton_blockwise_quant(x, round_scale=round_scale)
    w_q, w_s = triton_block_quant(w, round_scale=round_scale)
    dy_q, dy_s, dyt_q, dyt_s = triton_blockwise_quant(dy, round_scale=round_scale)
    # fprop y = x w^T, dgrad dx = dy w (w^T quantised in 128x128 blocks again), wgrad dw = dy^T x
    y = _fprop(x_q, x_s, w_q, w_s)
    assert _rel(y, x.float() @ w.float().t()) < 0.05
    wt_q, wt_s = triton_block_quant(w.t().contiguous(), round_scale=round_scale)
    dx = _fprop(dy_q, dy_s, wt_q, wt_s)
    assert _rel(dx, dy.float() @ w.float()) < 0.05
    dw = _wgrad(dyt_q, dyt_s, xt_q, xt_s)
    assert _rel(dw, dy.float().t() @ x.float()) < 0.05
    # a transposed scale tensor must NOT pass (the check has teeth)
    bad = _fprop(x_q, x_s.t().contiguous().view(K // 128, M), w_q, w_s)
    assert _rel(bad, x.float() @ w.float().t()) > 0.05

    # the fused producers feed the same consumer
    gamma = (1 + 0.1 * torch.randn(K, generator=g)).to(torch.bfloat16).to(gpu)
    n_q, n_s, rstd, nt_q, nt_s = triton_rms_norm_and_block_quant_forward(x, gamma, round_scale=round_scale)
    xn = (x.float() * rstd[:, None]) * gamma.float()
    assert _rel(_fprop(n_q, n_s, w_q, w_s), xn @ w.float().t()) < 0.05
    assert _rel(_wgrad(dyt_q, dyt_s, nt_q, nt_s), dy.float().t() @ xn) < 0.05
    h = randn_bf16(g, M, 2 * K).to(gpu)
    a_q, a_s, at_q, at_s = triton_silu_and_block_quant_forward(h, round_scale=round_scale)
    act = (torch.sigmoid(h[:, :K].float()) * h[:, :K].float()) * h[:, K:].float()
    assert _rel(_fprop(a_q, a_s, w_q, w_s), act @ w.float().t()) < 0.05
    assert _rel(_wgrad(dyt_q, dyt_s, at_q, at_s), dy.float().t() @ act) < 0.05
    # SwiGLU backward: dh [M, 2K] (dx1 | dx2) and its transposed copy [2K, M]
    gact = randn_bf16(g, M, K, scale=1e-2).to(gpu)
    d_q, d_s, dt_q, dt_s = triton_silu_and_block_quant_backward(gact, h, round_scale=round_scale)
    hf = h.float().requires_grad_()
    ((torch.sigmoid(hf[:, :K]) * hf[:, :K]) * hf[:, K:]).backward(gact.float())
    w2 = randn_bf16(g, N, 2 * K, scale=0.05).to(gpu)
    w2_q, w2_s = triton_block_quant(w2, round_scale=round_scale)
    assert _rel(_fprop(d_q, d_s, w2_q, w2_s), hf.grad @ w2.float().t()) < 0.05
    assert _rel(_wgrad(dt_q, dt_s, xt_q, xt_s), hf.grad.t() @ x.float()) < 0.05
