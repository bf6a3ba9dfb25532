"""Pure-torch CPU restatement of the reference's torch oracles for the fused
1x128 / 128x1 blockwise-FP8 quantization path.

TEST INFRASTRUCTURE ONLY (checker, never the product): imported by ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``.

Every function names the reference lines it restates (paths relative to the
reference checkout).  All arithmetic is fp32 on the CPU through torch library
routines, exactly as the reference's own test oracles do.

How each function is pinned (no reference file is imported or run; the
reference holds no golden vectors for this path):

* ``group_quant_1x128``  - tests/test_oracle_pins.py: software RNE fp8 encoder
  written from the OCP FP8 spec (numpy, integer arithmetic) over random and
  boundary inputs; amax element maps to +-448; dequantisation bound; all-zero
  group -> scale 1e-30, code 0; per-element brute force over all 256 codes.
* ``blockwise_quant`` and the batched packers - element-by-element Python loops
  over the published index formulas (scale[b, r], qt[c, r], tscale[rb, c],
  per-expert packed offsets) on tiny ragged inputs.
* ``rms_norm_*`` - closed forms checked against torch.autograd in fp64
  (gradcheck) and against torch.nn.RMSNorm; a dropped 1/n, a wrong power of r
  or a transposed operand fails them.
* ``rms_gemm_block_quant_forward`` - composition of the pinned pieces; its GEMM is
  torch's fp32 matmul, checked against an fp64 product in the pins.
* ``swiglu_*`` - closed-form derivatives checked against fp64 autograd.
* ``block_quant_128`` - per-element loop over the block index formula on a tiny
  matrix with the same scale/code helpers.
* ``batch_block_pad_permute_with_indices`` / ``pad_indices`` - element-by-element
  loops over the kernel's published offsets (padded expert starts, padded
  strides, zero padding rows with the floor scale) on a tiny ragged case.
* e5m2 variants - parity unpinned by the reference (it has no e5m2 path);
  pinned only by the same software encoder and invariants.
"""
from __future__ import annotations

import torch

E4M3 = torch.float8_e4m3fn
E5M2 = torch.float8_e5m2
GROUP = 128
SCALE_FLOOR = 1e-30


def fp8_max(fp8_dtype) -> float:
    """Largest finite value of the code space the scales are derived from.

    The reference hard-codes 448 (linghe/tools/util.py:47-48) because it only
    ever emits e4m3fn; the e5m2 value is this build's keyword extension."""
    return 448.0 if fp8_dtype == E4M3 else 57344.0


def _pow2_ceil(scale: torch.Tensor) -> torch.Tensor:
    # linghe/tools/util.py:61-62 : exp2(ceil(log2(scale)))
    return torch.exp2(torch.ceil(torch.log2(scale)))


def group_quant_1x128(v: torch.Tensor, round_scale: bool = False, fp8_dtype=E4M3):
    """1x128 group quantisation along the last dim of a 2-D fp32 matrix.

    Restates torch_group_quant, linghe/tools/util.py:46-66: zero-pad the width
    to a multiple of 128, amax(|v|) per group in fp32, divide by fmax, floor at
    1e-30, optional power-of-two round-up, true division, RNE cast.

    Returns (codes [R, K] fp8, scales [R, ceil(K/128)] fp32)."""
    assert v.dim() == 2
    v = v.float()
    rows, width = v.shape
    padded = (width + GROUP - 1) // GROUP * GROUP
    if padded != width:
        v = torch.nn.functional.pad(v, (0, padded - width))
    g = v.reshape(rows, padded // GROUP, GROUP)
    scale = g.abs().amax(dim=2) / fp8_max(fp8_dtype)
    scale = torch.clamp_min(scale, torch.tensor(SCALE_FLOOR, dtype=torch.float32))
    if round_scale:
        scale = _pow2_ceil(scale)
    codes = (g / scale.unsqueeze(-1)).to(fp8_dtype).reshape(rows, padded)
    return codes[:, :width].contiguous(), scale


def blockwise_quant(y: torch.Tensor, round_scale: bool = False, fp8_dtype=E4M3):
    """Row-wise 1x128 and column-wise 128x1 quantisation of y [M, n].

    Restates torch_blockwise_quant (linghe/tools/util.py:69-82) and the
    ``y_q, y_scale.t(), yt_q, yt_scale.t()`` convention of
    tests/test_norm.py:81-84.

    Returns q [M, n], scale [n/128, M], qt [n, M], tscale [ceil(M/128), n]."""
    y = y.float()
    q, s = group_quant_1x128(y, round_scale, fp8_dtype)
    qt, st = group_quant_1x128(y.t(), round_scale, fp8_dtype)
    return q, s.t().contiguous(), qt, st.t().contiguous()


# ----------------------------------------------------------------------------
# RMSNorm
# ----------------------------------------------------------------------------
def rms_norm_fp32(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6):
    """fp32 RMSNorm through torch.nn.RMSNorm, as tests/test_norm.py:22-32,70-80
    build it; also returns rstd = rsqrt(sum(x^2)/n + eps) (tests/test_norm.py:80)."""
    xf = x.float()
    n = xf.shape[-1]
    mod = torch.nn.RMSNorm(normalized_shape=n, eps=eps, dtype=torch.float32)
    with torch.no_grad():
        mod.weight.copy_(weight.float())
        y = mod(xf)
    rstd = torch.rsqrt(torch.sum(xf ** 2, -1) / n + eps)
    return y, rstd


def rms_norm_forward(x, weight, eps: float = 1e-6):
    """bf16 RMSNorm forward oracle, tests/test_norm.py:22-32: fp32 math, result
    cast back to the input dtype."""
    y, rstd = rms_norm_fp32(x, weight, eps)
    return y.to(x.dtype), rstd


def rms_norm_backward(x, weight, dy, eps: float = 1e-6):
    """RMSNorm backward oracle, tests/test_norm.py:35-49: fp32 autograd through
    torch.nn.RMSNorm.  Returns (dx in x.dtype, dgamma fp32 [n]).

    The reference casts dgamma to bf16 only for its loose comparison; the kernel
    (linghe/utils/norm.py:179) returns fp32, so fp32 is kept here."""
    xf = x.float().clone().requires_grad_()
    n = xf.shape[-1]
    mod = torch.nn.RMSNorm(normalized_shape=n, eps=eps, dtype=torch.float32)
    with torch.no_grad():
        mod.weight.copy_(weight.float())
    mod(xf).backward(gradient=dy.float())
    return xf.grad.to(x.dtype), mod.weight.grad.detach()


def rms_norm_backward_closed_form(x, weight, dy, eps: float = 1e-6):
    """Closed form of the same gradient, linghe/utils/norm.py:131-135:
    dx = r*g*w - r^3*x*sum(x*g*w)/n ; dgamma = sum_rows x*g*r."""
    xf, wf, gf = x.float(), weight.float(), dy.float()
    n = xf.shape[-1]
    r = torch.rsqrt(torch.sum(xf * xf, -1, keepdim=True) / n + eps)
    dot = torch.sum(xf * gf * wf, -1, keepdim=True)
    dx = r * gf * wf - r * r * r * xf * dot / n
    dgamma = torch.sum(xf * gf * r, 0)
    return dx.to(x.dtype), dgamma


def rms_norm_and_block_quant_forward(x, weight, eps: float = 1e-6,
                                     round_scale: bool = False, fp8_dtype=E4M3, rstd=None):
    """tests/test_norm.py:70-84.  Returns q [M,n], scale [n/128,M], rstd [M],
    qt [n,M], tscale [ceil(M/128), n].

    With ``rstd`` given, the normalised value is (x * rstd[row]) * weight, the
    expression the reference evaluates when the caller passes a saved statistic
    (linghe/utils/norm.py:331-333, output_mode 1)."""
    if rstd is None:
        y, rstd = rms_norm_fp32(x, weight, eps)
    else:
        rstd = rstd.float()
        y = (x.float() * rstd.reshape(-1, 1)) * weight.float()
    q, s, qt, st = blockwise_quant(y, round_scale, fp8_dtype)
    return q, s, rstd, qt, st


# ----------------------------------------------------------------------------
# SwiGLU
# ----------------------------------------------------------------------------
def rms_gemm_block_quant_forward(x, norm_weight, route_weight, eps: float = 1e-6,
                                 round_scale: bool = False, rstd=None):
    """tests/test_norm.py:87-104: y = fp32 RMSNorm, logits = y @ route_weight^T in
    fp32, both quantisations of y.  Returns (y in x.dtype, rstd, logits fp32,
    codes [M,K], scale [K/128, M], transposed codes [K, M], scale [M/128, K])."""
    y, r = rms_norm_fp32(x, norm_weight, eps)
    if rstd is not None:  # the statistic the kernel used (see rms_norm_and_block_quant_forward)
        r = rstd
        y = (x.float() * r[:, None]) * norm_weight.float()
    logits = y @ route_weight.float().t()
    q, s, qt, st = blockwise_quant(y, round_scale)
    return y.to(x.dtype), r, logits, q, s, qt, st


def swiglu_fp32(x: torch.Tensor, row_weight: torch.Tensor | None = None):
    """y = sigmoid(x1) * x1 * x2 [* w_row] in fp32 with x1 | x2 the two halves
    of the last dim (tests/test_silu.py:29-43)."""
    xf = x.float()
    n = xf.shape[1] // 2
    x1, x2 = xf[:, :n], xf[:, n:]
    y = torch.sigmoid(x1) * x1 * x2
    if row_weight is not None:
        y = y * row_weight.float().reshape(-1, 1)
    return y


def swiglu_grad_fp32(dy, x, row_weight=None):
    """fp32 autograd of swiglu_fp32 (tests/test_silu.py:46-53,113-118).
    Returns (dx [M, 2n] fp32, dw [M,1] fp32 or None)."""
    xf = x.float().clone().requires_grad_()
    wf = None
    if row_weight is not None:
        wf = row_weight.float().clone().requires_grad_()
    swiglu_fp32(xf, wf).backward(gradient=dy.float())
    return xf.grad, (wf.grad if wf is not None else None)


def weighted_silu_forward(x, row_weight=None):
    """bf16 weighted SwiGLU, tests/test_silu.py:36-43 (result in x.dtype)."""
    return swiglu_fp32(x, row_weight).to(x.dtype)


def weighted_silu_backward(dy, x, row_weight=None):
    """tests/test_silu.py:46-53: dx cast to x.dtype, dw fp32."""
    dx, dw = swiglu_grad_fp32(dy, x, row_weight)
    return dx.to(x.dtype), dw


def silu_and_block_quant_forward(x, round_scale: bool = False, fp8_dtype=E4M3):
    """tests/test_silu.py:75-84, in the kernel's layouts: q [M,n],
    scale [n/128,M], qt [n,M], tscale [ceil(M/128), n]."""
    return blockwise_quant(swiglu_fp32(x), round_scale, fp8_dtype)


def silu_and_block_quant_backward(dy, x, round_scale: bool = False, fp8_dtype=E4M3):
    """tests/test_silu.py:113-123 in the kernel's layouts: dx codes [M,2n],
    scale [2n/128, M], dx^T codes [2n, M], tscale [ceil(M/128), 2n]."""
    dx, _ = swiglu_grad_fp32(dy, x)
    return blockwise_quant(dx, round_scale, fp8_dtype)


def block_quant_128(w, round_scale: bool = False, fp8_dtype=E4M3):
    """One scale per 128x128 block (linghe/tools/util.py:85-98): amax of the block
    / fmax, optional power-of-two rounding, true division, RNE cast.  The floor
    max(scale, 1e-30) is the kernel's (linghe/quant/block.py:24); the reference's
    torch helper has none and divides an all-zero block by zero.
    Returns (codes [M,N], scale [M/128, N/128])."""
    M, N = w.shape
    wp = w.float().reshape(M // GROUP, GROUP, N // GROUP, GROUP).permute(0, 2, 1, 3)
    scale = torch.amax(torch.amax(wp.abs(), dim=2), dim=2) / fp8_max(fp8_dtype)
    scale = torch.maximum(scale, torch.full((1,), SCALE_FLOOR, dtype=torch.float32))
    if round_scale:
        scale = _pow2_ceil(scale)
    q = (wp / scale[:, :, None, None]).to(fp8_dtype)
    return q.permute(0, 2, 1, 3).reshape(M, N).contiguous(), scale


# ----------------------------------------------------------------------------
# per-expert (batched) forms: outputs packed expert after expert
# ----------------------------------------------------------------------------
def _pack_experts(mats, counts, round_scale, fp8_dtype):
    """Per-expert blockwise quant with the flat packing of
    tests/test_silu.py:184-199 and tests/test_blockwise_quant.py:17-43:
    q rows concatenated; per expert the [nb, c] scale block, the [n, c]
    transposed codes and the [ceil(c/128), n] transposed scales, each
    flattened, in expert order."""
    width = mats.shape[1]
    qs, ss, qts, sts = [], [], [], []
    start = 0
    for c in counts:
        blk = mats[start:start + c]
        q, s, qt, st = blockwise_quant(blk, round_scale, fp8_dtype)
        qs.append(q)
        ss.append(s.reshape(-1))
        qts.append(qt.reshape(-1))
        sts.append(st.reshape(-1))
        start += c
    if start == 0:
        return (torch.empty((0, width), dtype=fp8_dtype),
                torch.empty((0,), dtype=torch.float32),
                torch.empty((0,), dtype=fp8_dtype),
                torch.empty((0,), dtype=torch.float32))
    return torch.cat(qs, 0), torch.cat(ss, 0), torch.cat(qts, 0), torch.cat(sts, 0)


def _as_count_list(counts):
    return [int(c) for c in (counts.tolist() if hasattr(counts, "tolist") else counts)]


def batch_blockwise_quant(xs, counts, round_scale: bool = False, fp8_dtype=E4M3):
    """tests/test_blockwise_quant.py:17-43."""
    return _pack_experts(xs.float(), _as_count_list(counts), round_scale, fp8_dtype)


def pad_indices(indices, counts, multiple: int = 16):
    """The index layout the gather kernel reads (linghe/utils/gather.py:871-875):
    expert e's entries start at the sum of the counts before it, each rounded up
    to `multiple`; the padding entries are zero and never used."""
    counts = _as_count_list(counts)
    out, s = [], 0
    for c in counts:
        pc = (c + multiple - 1) // multiple * multiple
        out.append(indices[s:s + c].to(torch.int32))
        out.append(torch.zeros(pc - c, dtype=torch.int32))
        s += c
    return torch.cat(out) if out else torch.zeros(0, dtype=torch.int32)


def batch_block_pad_permute_with_indices(x, indices, probs, counts, round_scale: bool = True,
                                         fp8_dtype=E4M3):
    """tests/test_gather.py:150-197: per expert (empty ones skipped) the rows
    x[indices[s:s+c]] in fp32, zero-padded to a multiple of 16 rows
    (linghe/tools/util.py:69-82, padding=True), blockwise quantised; the four
    results flattened and concatenated in expert order; probs[:, e][index]
    zero-padded likewise.  `indices` is the UNPADDED concatenation."""
    counts = _as_count_list(counts)
    qs, ss, qts, sts, ps = [], [], [], [], []
    s = 0
    for e, c in enumerate(counts):
        if c == 0:
            continue
        index = indices[s:s + c].long()
        y = x[index].float()
        pad = (c + 15) // 16 * 16 - c
        if pad:
            y = torch.nn.functional.pad(y, (0, 0, 0, pad))
        q, sc, qt, st = blockwise_quant(y, round_scale, fp8_dtype)
        qs.append(q.reshape(-1))
        ss.append(sc.reshape(-1))
        qts.append(qt.reshape(-1))
        sts.append(st.reshape(-1))
        if probs is not None:
            ps.append(torch.nn.functional.pad(probs[:, e][index], (0, pad)))
        s += c
    if not qs:
        z8, z32 = torch.empty((0,), dtype=fp8_dtype), torch.empty((0,), dtype=torch.float32)
        return z8, z32, z8.clone(), z32.clone(), (z32.clone() if probs is not None else None)
    return (torch.cat(qs), torch.cat(ss), torch.cat(qts), torch.cat(sts),
            torch.cat(ps) if probs is not None else None)


def batch_weighted_silu_and_block_quant_forward(xs, weight, counts,
                                                round_scale: bool = False,
                                                fp8_dtype=E4M3):
    """tests/test_silu.py:163-199.  The activation stays fp32 (the reference
    upcasts xs before its weighted-silu helper, so no bf16 rounding occurs)."""
    y = swiglu_fp32(xs, weight)
    return _pack_experts(y, _as_count_list(counts), round_scale, fp8_dtype)


def batch_weighted_silu_and_block_quant_backward(dy, xs, weight, counts,
                                                 round_scale: bool = False,
                                                 fp8_dtype=E4M3):
    """tests/test_silu.py:260-296.  Returns (dx codes [M,2n], flat scales,
    dw [M,1] fp32, flat dx^T codes, flat transposed scales)."""
    counts = _as_count_list(counts)
    if sum(counts) == 0:
        width = xs.shape[1]
        return (torch.empty((0, width), dtype=fp8_dtype),
                torch.empty((0,), dtype=torch.float32),
                torch.empty_like(weight, dtype=torch.float32),
                torch.empty((0,), dtype=fp8_dtype),
                torch.empty((0,), dtype=torch.float32))
    dx, dw = swiglu_grad_fp32(dy, xs, weight)
    q, s, qt, st = _pack_experts(dx, counts, round_scale, fp8_dtype)
    return q, s, dw, qt, st
