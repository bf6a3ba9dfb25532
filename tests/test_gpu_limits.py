"""Largest supported shapes: M = 2^24 rows and N = 2^22 columns.

The element counts (2^31 for the tall case) exceed what 32-bit indexing holds,
and the oracle cannot run on the whole tensor in reasonable time.  Every
128-row block (and every 128-column tile) is independent of the others, so the
kernel output of a slab must equal the oracle's output for that slab alone: the
first, the last and a few slabs around the 2^31-byte and 2^32-byte marks are
checked bit for bit.  Over the whole tensor the largest code of every group is
checked on the device: without scale rounding the group maximum maps to +-448
exactly, which a group that was never written (or written from the wrong rows)
does not do.
"""
from __future__ import annotations

import pytest
import torch

from oracle import fq_oracle as O
from tests.helpers import announce, check_quant_pair

pytestmark = pytest.mark.gpu

EXACT = dict(scale_max_ulp=0, scale_min_within1=1.0, min_identical=1.0)
FUSED = dict(scale_max_ulp=5, scale_min_within1=0.97)


def _every_group_hits_fmax(codes, name, fmax=448.0):
    """codes [..., L] fp8 with quantisation groups of 128 along the last dimension."""
    rows = codes.reshape(-1, codes.shape[-1])
    step = max(1, (1 << 26) // rows.shape[1])
    for a in range(0, rows.shape[0], step):
        part = rows[a:a + step].float().abs()
        top = part.reshape(part.shape[0], -1, 128).amax(2)
        assert float(top.min()) == fmax and float(top.max()) == fmax, f"{name}: a group without a +-{fmax} code"


def _fill(M, N, gpu, seed):
    """bf16 data generated on the device, 2^24 elements at a time (no 4x fp32 temporary
    of the whole tensor)."""
    g = torch.Generator(device=gpu).manual_seed(seed)
    x = torch.empty(M, N, dtype=torch.bfloat16, device=gpu)
    flat = x.view(-1)
    step = 1 << 24
    for a in range(0, flat.numel(), step):
        b = min(a + step, flat.numel())
        flat[a:b] = torch.randn(b - a, generator=g, device=gpu, dtype=torch.float32).to(torch.bfloat16)
    return x


def test_blockwise_quant_tallest(gpu):
    from linghe_amd.quant.block import triton_blockwise_quant

    M, N = 1 << 24, 128
    announce("blockwise_quant", M, N)
    x = _fill(M, N, gpu, 41)
    q, s, qt, st = triton_blockwise_quant(x, round_scale=False, output_mode=2)
    torch.cuda.synchronize()
    assert q.shape == (M, N) and s.shape == (1, M) and qt.shape == (N, M) and st.shape == (M // 128, N)
    # slabs: first, last, and around byte offsets 2^31 and 2^32 of x (2 bytes/element)
    blocks = [0, 1, (1 << 31) // (256 * 128) - 1, (1 << 31) // (256 * 128), (1 << 32) // (256 * 128) - 1,
              (1 << 32) // (256 * 128), M // 128 - 2, M // 128 - 1]
    for rb in blocks:
        r0 = rb * 128
        ref = O.blockwise_quant(x[r0:r0 + 128].cpu(), False)
        check_quant_pair(f"tall.rb{rb}.row", ref[0], ref[1], q[r0:r0 + 128], s[:, r0:r0 + 128], **EXACT)
        check_quant_pair(f"tall.rb{rb}.col", ref[2], ref[3], qt[:, r0:r0 + 128].contiguous(), st[rb:rb + 1], **EXACT)
    _every_group_hits_fmax(q, "tall.row")
    _every_group_hits_fmax(qt, "tall.col")
    assert float(st.min()) > 0.0 and float(s.min()) > 0.0


def test_blockwise_quant_widest(gpu):
    from linghe_amd.quant.block import triton_blockwise_quant

    M, N = 128, 1 << 22
    announce("blockwise_quant", M, N)
    x = _fill(M, N, gpu, 42)
    q, s, qt, st = triton_blockwise_quant(x, round_scale=False, output_mode=2)
    torch.cuda.synchronize()
    assert q.shape == (M, N) and s.shape == (N // 128, M) and qt.shape == (N, M) and st.shape == (1, N)
    for c0 in (0, 128, (1 << 21) - 128, 1 << 21, N - 256, N - 128):
        ref = O.blockwise_quant(x[:, c0:c0 + 128].contiguous().cpu(), False)
        cb = c0 // 128
        check_quant_pair(f"wide.c{c0}.row", ref[0], ref[1], q[:, c0:c0 + 128].contiguous(), s[cb:cb + 1], **EXACT)
        check_quant_pair(f"wide.c{c0}.col", ref[2], ref[3], qt[c0:c0 + 128], st[:, c0:c0 + 128].contiguous(), **EXACT)
    _every_group_hits_fmax(q, "wide.row")
    _every_group_hits_fmax(qt, "wide.col")


def test_group_quant_tallest(gpu):
    from linghe_amd.quant.group import triton_group_quant

    M, N = 1 << 24, 128
    announce("group_quant", M, N)
    x = _fill(M, N, gpu, 43)
    q, s = triton_group_quant(x)
    torch.cuda.synchronize()
    for r0 in (0, (1 << 23) - 64, (1 << 24) - 256):
        rq, rs = O.group_quant_1x128(x[r0:r0 + 256].cpu(), False)
        check_quant_pair(f"group.tall.r{r0}", rq, rs, q[r0:r0 + 256], s[r0:r0 + 256], **EXACT)
    # against the blockwise kernel on the same data: same codes, same scales
    from linghe_amd.quant.block import triton_blockwise_quant
    q2, s2, _, _ = triton_blockwise_quant(x, output_mode=0)
    torch.cuda.synchronize()
    assert torch.equal(q.view(torch.uint8), q2.view(torch.uint8))
    assert torch.equal(s.view(-1), s2.view(-1))


def test_swiglu_quant_tall(gpu):
    """2^23 rows x 256 input columns (2^31 input elements)."""
    from linghe_amd.utils.silu import triton_silu_and_block_quant_forward as fwd

    M, n = 1 << 23, 128
    announce("silu_and_block_quant_forward", M, 2 * n)
    x = _fill(M, 2 * n, gpu, 44)
    q, s, qt, st = fwd(x, round_scale=False, output_mode=2)
    torch.cuda.synchronize()
    assert q.shape == (M, n) and qt.shape == (n, M) and st.shape == (M // 128, n)
    for rb in (0, (1 << 31) // (512 * 128) - 1, (1 << 31) // (512 * 128), M // 128 - 1):
        r0 = rb * 128
        ref = O.silu_and_block_quant_forward(x[r0:r0 + 128].cpu(), False)
        check_quant_pair(f"silu.tall.rb{rb}.row", ref[0], ref[1], q[r0:r0 + 128], s[:, r0:r0 + 128], **FUSED)
        check_quant_pair(f"silu.tall.rb{rb}.col", ref[2], ref[3], qt[:, r0:r0 + 128].contiguous(), st[rb:rb + 1],
                         **FUSED)
    _every_group_hits_fmax(q, "silu.tall.row")
    _every_group_hits_fmax(qt, "silu.tall.col")


def test_batched_blockwise_quant_tallest(gpu):
    """2^24 rows over a few huge, ragged experts (and empty ones): the per-expert
    offsets si*nb, si*n + c*ce and the running block count all pass 2^31."""
    from linghe_amd.quant.block import triton_batch_blockwise_quant

    N = 128
    counts = [(1 << 22) + 5, 0, (1 << 23) - 77, 3, 0, (1 << 21) + 128, 0, 0]
    counts[-1] = (1 << 24) - sum(counts)
    M = sum(counts)
    assert M == 1 << 24 and counts[-1] > 0
    announce("batch_blockwise_quant", M, N, counts)
    x = _fill(M, N, gpu, 45)
    cnt = torch.tensor(counts, dtype=torch.int64, device=gpu)
    q, s, qt, st = triton_batch_blockwise_quant(x, cnt, counts, round_scale=False)
    torch.cuda.synchronize()
    nb = N // 128
    blocks = [(c + 127) // 128 for c in counts]
    assert st.numel() == sum(blocks) * N
    st = st.view(-1, N)
    si = tb = 0
    for e, ce in enumerate(counts):
        if ce:
            s_e = s[si * nb:(si + ce) * nb].view(nb, ce)
            qt_e = qt[si * N:(si + ce) * N].view(N, ce)
            for rb in sorted({0, blocks[e] // 2, blocks[e] - 1}):
                r0, r1 = rb * 128, min(rb * 128 + 128, ce)
                ref = O.blockwise_quant(x[si + r0:si + r1].cpu(), False)
                check_quant_pair(f"batch.tall.e{e}.rb{rb}.row", ref[0], ref[1], q[si + r0:si + r1], s_e[:, r0:r1],
                                 **EXACT)
                check_quant_pair(f"batch.tall.e{e}.rb{rb}.col", ref[2], ref[3], qt_e[:, r0:r1].contiguous(),
                                 st[tb + rb:tb + rb + 1], **EXACT)
        si += ce
        tb += blocks[e]
    _every_group_hits_fmax(q, "batch.tall.row")
    assert float(s.min()) > 0.0 and float(st.min()) > 0.0


def test_rms_norm_quant_tall(gpu):
    """2^23 rows x 512 columns: 8.6 GB of input, row and byte offsets beyond 2^32."""
    from linghe_amd.utils.norm import triton_rms_norm_and_block_quant_forward as fwd
    from tests.helpers import gamma_bf16, gen

    M, n = 1 << 23, 512
    announce("rms_norm_and_block_quant_forward", M, n)
    x = _fill(M, n, gpu, 46)
    w = gamma_bf16(gen(47), n)
    q, s, rms, qt, st = fwd(x, w.to(gpu), round_scale=False, output_mode=2)
    torch.cuda.synchronize()
    assert q.shape == (M, n) and s.shape == (n // 128, M) and qt.shape == (n, M) and st.shape == (M // 128, n)
    for rb in (0, (1 << 32) // (1024 * 128) - 1, (1 << 32) // (1024 * 128), M // 128 - 1):
        r0 = rb * 128
        xs = x[r0:r0 + 128].cpu()
        # with the kernel's own statistic the rest is bit-exact
        pin = O.rms_norm_and_block_quant_forward(xs, w, rstd=rms[r0:r0 + 128].cpu())
        check_quant_pair(f"rms.tall.rb{rb}.row", pin[0], pin[1], q[r0:r0 + 128], s[:, r0:r0 + 128], **EXACT)
        check_quant_pair(f"rms.tall.rb{rb}.col", pin[3], pin[4], qt[:, r0:r0 + 128].contiguous(), st[rb:rb + 1],
                         **EXACT)
        ref = O.rms_norm_and_block_quant_forward(xs, w)
        from oracle import compare as C
        C.assert_scales(ref[2], rms[r0:r0 + 128].cpu(), f"rms.tall.rb{rb}.rstd", max_ulp=4, min_within_1ulp=0.9)
    _every_group_hits_fmax(q, "rms.tall.row")
    _every_group_hits_fmax(qt, "rms.tall.col")
