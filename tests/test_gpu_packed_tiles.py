"""Per-expert kernels on the boundaries of the partial-tile packing: an expert's last row block of at most
32 / 64 rows is covered four / two column blocks to a workgroup, so every count around 32, 64 and 128 (plus a
multiple of 128) is run against every number of column blocks from one to six, where the run of column blocks
a workgroup takes ends inside, at, or beyond the matrix edge.  Same oracle and tolerances as the other
per-expert tests: bit-exact where no arithmetic precedes the quantisation."""
import pytest
import torch

from oracle import fq_oracle as O
from tests.helpers import announce, check_quant_pair, gen, randn_bf16
from tests.test_gpu_parity import EXACT, _batched_case

pytestmark = pytest.mark.gpu

# last-block sizes on both sides of every packing boundary, alone and behind full row blocks, with empty experts
BOUNDARY_COUNTS = [1, 15, 16, 31, 32, 33, 0, 48, 63, 64, 65, 96, 127, 128, 129, 0, 128 + 31, 128 + 32, 128 + 33,
                   128 + 64, 128 + 65, 256 + 17, 256, 384 + 64, 7]


@pytest.mark.parametrize("ncb", [1, 2, 3, 4, 5, 6])
def test_batch_blockwise_quant_packing_boundaries(gpu, ncb):
    from linghe_amd.quant.block import triton_batch_blockwise_quant

    counts = BOUNDARY_COUNTS
    N = 128 * ncb
    announce("packed tiles: batch_blockwise_quant", ncb)
    x = randn_bf16(gen(70 + ncb), sum(counts), N)
    ref = O.batch_blockwise_quant(x, counts, False)
    for cdt in (torch.int32, torch.int64):
        q, s, qt, st = triton_batch_blockwise_quant(x.to(gpu), torch.tensor(counts, dtype=cdt, device=gpu), counts)
        torch.cuda.synchronize()
        check_quant_pair("packed.blockwise.row", ref[0], ref[1], q, s, **EXACT)
        check_quant_pair("packed.blockwise.col", ref[2], ref[3], qt, st, **EXACT)


@pytest.mark.parametrize("ncb", [1, 2, 3, 4, 5])
def test_batched_swiglu_packing_boundaries(gpu, ncb):
    announce("packed tiles: batched swiglu fwd/bwd", ncb)
    _batched_case(gpu, BOUNDARY_COUNTS, 256 * ncb, 1.0, 1.0, seed=80 + ncb)


@pytest.mark.parametrize("ncb", [1, 2, 3, 4, 6])
def test_pad_permute_packing_boundaries(gpu, ncb):
    """the packing goes by the PADDED row count: 17..32 real rows pad to 32 (four column blocks), 33 to 48 (two)"""
    from linghe_amd.utils.gather import triton_batch_block_pad_permute_with_indices as fn

    counts = [1, 15, 16, 17, 31, 32, 33, 0, 47, 48, 49, 63, 64, 65, 113, 128, 129, 128 + 20, 256 + 50]
    m, N = 500, 128 * ncb
    announce("packed tiles: pad+permute+quant", ncb)
    g = gen(90 + ncb)
    x = randn_bf16(g, m, N)
    probs = torch.rand(m, len(counts), generator=g)
    idx = torch.cat([torch.randperm(m, generator=g)[:c] for c in counts])
    ref = O.batch_block_pad_permute_with_indices(x, idx, probs, counts, False)
    padded = O.pad_indices(idx, counts)
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    q, s, qt, st, p = fn(x.to(gpu), cnt, padded.to(gpu), counts, probs=probs.to(gpu))
    torch.cuda.synchronize()
    check_quant_pair("packed.gather.row", ref[0], ref[1], q.view(-1), s.view(-1), **EXACT)
    check_quant_pair("packed.gather.col", ref[2], ref[3], qt.view(-1), st.view(-1), **EXACT)
    assert torch.equal(p.cpu(), ref[4])
