"""gather + pad-to-16 + blockwise quant (reference tests/test_gather.py:597-634):
the GPU entry point against the CPU oracle; no arithmetic precedes the
quantisation, so scales and codes must be bit-identical."""
import pytest
import torch

from oracle import fq_oracle as O
from tests.helpers import E4M3, E5M2, announce, check_quant_pair, gen, randn_bf16, zipf_counts

pytestmark = pytest.mark.gpu

EXACT = dict(scale_max_ulp=0, scale_min_within1=1.0, min_identical=1.0)


def _routing(g, m, counts):
    """source row of every routed token, expert after expert (rows may repeat across experts)"""
    return torch.cat([torch.randperm(m, generator=g)[:c] if c <= m else torch.randint(0, m, (c,), generator=g)
                      for c in counts]) if sum(counts) else torch.zeros(0, dtype=torch.int64)


@pytest.mark.parametrize("counts,m,N", [
    ([5, 0, 130, 16, 127, 1, 129, 256], 300, 384),
    ([0, 0, 0], 64, 256),
    ([48], 48, 128),
    (None, 4096, 2048),          # 32 experts, top-2 of 4096 tokens, Zipf counts with empty experts
])
@pytest.mark.parametrize("round_scale", [True, False])
def test_batch_block_pad_permute_with_indices(gpu, counts, m, N, round_scale):
    from linghe_amd.utils.gather import triton_batch_block_pad_permute_with_indices as fn

    if counts is None:
        counts = zipf_counts(2 * m, 32, seed=9, n_empty=2)
    announce("pad+permute+quant", counts[:8], m, N, round_scale)
    g = gen(61)
    E = len(counts)
    x = randn_bf16(g, m, N)
    probs = torch.rand(m, E, generator=g)
    idx = _routing(g, m, counts)
    ref = O.batch_block_pad_permute_with_indices(x, idx, probs, counts, round_scale)
    padded = O.pad_indices(idx, counts)
    for cdt in (torch.int32, torch.int64):
        cnt = torch.tensor(counts, dtype=cdt, device=gpu)
        q, s, qt, st, p = fn(x.to(gpu), cnt, padded.to(gpu), counts, probs=probs.to(gpu), round_scale=round_scale)
        torch.cuda.synchronize()
        M = padded.numel()
        assert q.shape == (M, N) and s.shape == (M, N // 128) and qt.shape == (M, N)
        assert st.shape == (sum((c + 127) // 128 for c in counts), N) and p.shape == (M,)
        if M == 0:
            continue
        check_quant_pair("gather.row", ref[0], ref[1], q.view(-1), s.view(-1), **EXACT)
        check_quant_pair("gather.col", ref[2], ref[3], qt.view(-1), st.view(-1), **EXACT)
        assert torch.equal(p.cpu(), ref[4])
    # without probs, bf16 probs, e5m2 codes
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    out = fn(x.to(gpu), cnt, padded.to(gpu), counts, round_scale=round_scale)
    assert out[4] is None
    pb = probs.to(torch.bfloat16)
    out = fn(x.to(gpu), cnt, padded.to(gpu), counts, probs=pb.to(gpu), round_scale=round_scale, fp8_dtype=E5M2)
    torch.cuda.synchronize()
    ref5 = O.batch_block_pad_permute_with_indices(x, idx, pb, counts, round_scale, E5M2)
    if padded.numel():
        check_quant_pair("gather.e5m2.row", ref5[0], ref5[1], out[0].view(-1), out[1].view(-1), **EXACT)
        check_quant_pair("gather.e5m2.col", ref5[2], ref5[3], out[2].view(-1), out[3].view(-1), **EXACT)
        assert out[4].dtype == torch.bfloat16 and torch.equal(out[4].cpu(), ref5[4])


def test_pad_permute_ignores_bad_indices(gpu):
    """entries that do not name a source row (and the padding entries, whatever they hold) read as zero rows"""
    from linghe_amd.utils.gather import triton_batch_block_pad_permute_with_indices as fn

    announce("pad+permute+quant, out-of-range indices")
    g = gen(62)
    counts = [20, 7]
    m, N = 32, 256
    x = randn_bf16(g, m, N)
    idx = torch.randint(0, m, (27,), generator=g)
    padded = O.pad_indices(idx, counts)
    padded[20:32] = 10 ** 9       # padding of expert 0
    padded[3] = -5                # a corrupt entry inside expert 0
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    q, s, qt, st, _ = fn(x.to(gpu), cnt, padded.to(gpu), counts)
    torch.cuda.synchronize()
    x2 = torch.cat([x, torch.zeros(1, N, dtype=x.dtype)])
    idx2 = idx.clone()
    idx2[3] = m                   # the zero row
    ref = O.batch_block_pad_permute_with_indices(x2, idx2, None, counts, False)
    check_quant_pair("gather.bad.row", ref[0], ref[1], q.view(-1), s.view(-1), **EXACT)
    check_quant_pair("gather.bad.col", ref[2], ref[3], qt.view(-1), st.view(-1), **EXACT)
