"""Per-expert entry points with the tiles read from a plan (fq_build_expert_plan and the
*_planned forms): the plan's records against the host-side arithmetic on the counts, and every
output of the planned forms byte for byte against the forms that scan the counts (which the
parity tests hold against the oracle), plus the oracle itself on one case."""
import numpy as np
import pytest
import torch

from tests.helpers import announce, check_quant_pair, gen, randn_bf16, zipf_counts

pytestmark = pytest.mark.gpu

EXACT = dict(scale_max_ulp=0, scale_min_within1=1.0, min_identical=1.0)


def _dev(t, gpu):
    return t.to(gpu)


def _kind(rows):
    return 3 if rows <= 32 else 2 if rows <= 64 else 1


def _blocks(counts, pad):
    """(first row in the outputs, row block inside the expert, count, kind, expert) of every row block, expert order"""
    out, start = [], 0
    for e, c in enumerate(counts):
        pc = (c + pad - 1) // pad * pad
        for rb in range((c + 127) // 128):
            out.append((start + rb * 128, rb, c, _kind(min(128, pc - rb * 128)), e))
        start += pc
    return out


def _expected_shape(counts, pad=1):
    """row blocks in all, worked on whole (kind 1), in halves (2: a last block whose padded rows are 33..64), in
    quarters (3), and the padding itself"""
    kinds = [b[3] for b in _blocks(counts, pad)]
    return [len(kinds)] + [kinds.count(k) for k in (1, 2, 3)] + [pad]


def _expected_plan(counts, shape):
    """[blocks, 4] uint32 records - a row block's first row, its number inside the expert, the expert's
    count, kind << 30 | its number over all experts - and [blocks] int32 experts behind them; three sections
    (kinds 1, 2, 3) of the sizes in `shape`, each in expert order, what the counts do not fill left zero
    (expert -1) and what they have beyond a section's size dropped."""
    first = [0, shape[1], shape[1] + shape[2]]
    size = shape[1:4]
    fill = [0, 0, 0]
    table = np.zeros((shape[0], 4), dtype=np.int64)
    experts = np.full((shape[0],), -1, dtype=np.int32)
    for rbg, (row0, rb, c, kind, e) in enumerate(_blocks(counts, shape[4])):
        k = kind - 1
        if fill[k] < size[k]:
            table[first[k] + fill[k]] = [row0, rb, c, kind << 30 | rbg]
            experts[first[k] + fill[k]] = e
        fill[k] += 1
    return table.astype(np.uint32), experts


COUNT_SETS = {
    "mixed": [128, 0, 256, 16, 0, 144, 1, 127],
    "empty": [0, 0, 0, 0],
    "one": [300],
    "ragged": list(range(1, 17)) + [128 + r for r in range(1, 16)] + [113, 120, 126],
    "zipf300": zipf_counts(6000, 300, seed=5, n_empty=7),
}


def _many_experts():
    rng = torch.Generator().manual_seed(15)
    counts = [int(c) for c in torch.randint(0, 40, (2300,), generator=rng)]
    counts[5], counts[1029], counts[2299] = 300, 257, 129
    return counts


@pytest.mark.parametrize("name", sorted(COUNT_SETS) + ["many"])
@pytest.mark.parametrize("cdt,pad", [(torch.int32, 1), (torch.int64, 1), (torch.int32, 16)])
def test_plan_records(gpu, name, cdt, pad):
    import ctypes

    from linghe_amd import _lib

    counts = _many_experts() if name == "many" else COUNT_SETS[name]
    announce("expert plan records", name, cdt, pad)
    host = (ctypes.c_int64 * len(counts))(*counts)
    shape = (ctypes.c_int64 * 5)()
    _lib.check(_lib.lib.fq_expert_plan_shape(host, len(counts), pad, shape))
    assert list(shape) == _expected_shape(counts, pad)
    cnt = torch.tensor(counts, dtype=cdt, device=gpu)
    # the host's shape may disagree with the device's counts: sections are never overrun, their rest is empty
    for delta in ((0, 0, 0), (2, 1, 3), (-1, -1, -1)):
        sh = [max(0, shape[1 + i] + delta[i]) for i in range(3)]
        sh = [sum(sh)] + sh + [pad]
        if sh[0] == 0:
            continue
        cs = (ctypes.c_int64 * 5)(*sh)
        nbytes = int(_lib.lib.fq_expert_plan_bytes(cs))
        assert nbytes == 20 * sh[0]
        table = torch.full((nbytes,), 0x5A, dtype=torch.uint8, device=gpu)
        _lib.check(_lib.lib.fq_build_expert_plan(_lib.ptr(cnt), int(cdt == torch.int64), len(counts), cs,
                                                 _lib.ptr(table), _lib.stream_of(cnt)))
        torch.cuda.synchronize()
        raw = table.cpu().numpy()
        records, experts = _expected_plan(counts, sh)
        np.testing.assert_array_equal(raw[:16 * sh[0]].view(np.uint32).reshape(sh[0], 4), records)
        np.testing.assert_array_equal(raw[16 * sh[0]:].view(np.int32), experts)


@pytest.mark.parametrize("name", sorted(COUNT_SETS) + ["many"])
def test_planned_blockwise_quant(gpu, name):
    from linghe_amd.quant.block import triton_batch_blockwise_quant
    from linghe_amd.utils.silu import build_expert_plan

    counts = _many_experts() if name == "many" else COUNT_SETS[name]
    announce("planned batch_blockwise_quant", name)
    M, N = sum(counts), 384
    x = _dev(randn_bf16(gen(14), M, N), gpu)
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    plan = build_expert_plan(cnt, counts)
    a = triton_batch_blockwise_quant(x, cnt, counts)
    b = triton_batch_blockwise_quant(x, cnt, counts, plan=plan)
    torch.cuda.synchronize()
    for u, v in zip(a, b):
        assert torch.equal(u.view(torch.uint8), v.view(torch.uint8))


@pytest.mark.parametrize("name,N", [("mixed", 1024), ("empty", 1536), ("one", 512), ("ragged", 256),
                                    ("zipf300", 512), ("many", 256)])
@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
def test_planned_batch_weighted_silu(gpu, name, N, wdtype):
    from linghe_amd.utils.silu import (build_expert_plan,
                                       triton_batch_weighted_silu_and_block_quant_backward as bwd,
                                       triton_batch_weighted_silu_and_block_quant_forward as fwd)

    counts = _many_experts() if name == "many" else COUNT_SETS[name]
    announce("planned batched silu+quant", name, N, wdtype)
    bs = sum(counts)
    g = gen(35)
    x = _dev(randn_bf16(g, bs, N), gpu)
    w = _dev(torch.randn(bs, 1, generator=g).to(wdtype), gpu)
    dy = _dev(randn_bf16(g, bs, N // 2), gpu)
    cnt = torch.tensor(counts, dtype=torch.int64, device=gpu)
    plan = build_expert_plan(cnt, counts)
    for mode in (2, 0, 1):
        a = fwd(x, w, cnt, counts, output_mode=mode)
        b = fwd(x, w, cnt, counts, output_mode=mode, plan=plan)
        torch.cuda.synchronize()
        which = {2: (0, 1, 2, 3), 0: (0, 1), 1: (2, 3)}[mode]
        for i in which:
            assert torch.equal(a[i].view(torch.uint8), b[i].view(torch.uint8)), (mode, i)
    a = bwd(dy, x, w, cnt, splits=counts)
    b = bwd(dy, x, w, cnt, splits=counts, plan=plan)
    torch.cuda.synchronize()
    for i, (u, v) in enumerate(zip(a, b)):
        assert torch.equal(u.view(torch.uint8), v.view(torch.uint8)), i


def test_planned_blockwise_quant_against_oracle(gpu):
    from oracle import fq_oracle as O
    from linghe_amd.quant.block import triton_batch_blockwise_quant
    from linghe_amd.utils.silu import build_expert_plan

    counts = COUNT_SETS["ragged"]
    announce("planned batch_blockwise_quant against the oracle")
    M, N = sum(counts), 384
    x = randn_bf16(gen(14), M, N)
    ref = O.batch_blockwise_quant(x, counts, False)
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    q, s, qt, st = triton_batch_blockwise_quant(_dev(x, gpu), cnt, counts, plan=build_expert_plan(cnt, counts))
    torch.cuda.synchronize()
    check_quant_pair("planned.row", ref[0], ref[1], q, s, **EXACT)
    check_quant_pair("planned.col", ref[2], ref[3], qt, st, **EXACT)


def test_plan_of_other_splits_is_refused(gpu):
    from linghe_amd.quant.block import triton_batch_blockwise_quant
    from linghe_amd.utils.silu import build_expert_plan

    counts = [128, 256]
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    plan = build_expert_plan(cnt, counts)
    other = [384, 256]
    x = torch.zeros(sum(other), 128, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(ValueError):
        triton_batch_blockwise_quant(x, torch.tensor(other, dtype=torch.int32, device=gpu), other, plan=plan)


def test_planned_launch_with_larger_shape_than_the_counts(gpu):
    """A shape whose sections are larger than what the device-side counts fill: the records
    beyond are empty, their workgroups leave, the outputs are those of the exact shape."""
    import ctypes

    from linghe_amd import _lib
    from linghe_amd.quant.block import triton_batch_blockwise_quant

    counts = COUNT_SETS["ragged"]
    announce("planned batch_blockwise_quant, inflated shape")
    M, N = sum(counts), 384
    x = _dev(randn_bf16(gen(14), M, N), gpu)
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    ref = triton_batch_blockwise_quant(x, cnt, counts)
    exact = _expected_shape(counts)
    sh = [exact[1] + 2, exact[2] + 1, exact[3] + 3]
    shape = (ctypes.c_int64 * 5)(sum(sh), *sh, 1)
    table = torch.empty((int(_lib.lib.fq_expert_plan_bytes(shape)),), dtype=torch.uint8, device=gpu)
    L = _lib.lib
    _lib.check(L.fq_build_expert_plan(_lib.ptr(cnt), 0, len(counts), shape, _lib.ptr(table), _lib.stream_of(x)))
    out = [torch.zeros_like(t) for t in ref]
    _lib.check(L.fq_batched_blockwise_quant_planned(
        _lib.ptr(x), _lib.ptr(table), shape, _lib.ptr(out[0]), _lib.ptr(out[1]), _lib.ptr(out[2]), _lib.ptr(out[3]),
        M, N, 0, _lib.FQ_E4M3, _lib.stream_of(x)))
    torch.cuda.synchronize()
    for u, v in zip(ref, out):
        assert torch.equal(u.view(torch.uint8), v.view(torch.uint8))


@pytest.mark.parametrize("name", ["mixed", "ragged", "zipf300", "one"])
@pytest.mark.parametrize("with_probs", [True, False])
def test_planned_pad_permute_quant(gpu, name, with_probs):
    """gather + pad + quant with a plan of the padded layout: every output (the gathered
    probabilities included, which need the expert of a tile) byte for byte."""
    from linghe_amd.utils.gather import triton_batch_block_pad_permute_with_indices as permute
    from linghe_amd.utils.silu import build_expert_plan

    counts = COUNT_SETS[name]
    announce("planned gather + pad + quant", name, with_probs)
    g = gen(36)
    m, N = 700, 384
    x = _dev(randn_bf16(g, m, N), gpu)
    probs = _dev(torch.rand(m, len(counts), generator=g), gpu) if with_probs else None
    parts = []
    for c in counts:
        parts += [torch.randint(0, m, (c,), generator=g, dtype=torch.int32),
                  torch.zeros((c + 15) // 16 * 16 - c, dtype=torch.int32)]
    idx = _dev(torch.cat(parts), gpu)
    cnt = torch.tensor(counts, dtype=torch.int32, device=gpu)
    plan = build_expert_plan(cnt, counts, pad=16)
    a = permute(x, cnt, idx, counts, probs)
    b = permute(x, cnt, idx, counts, probs, plan=plan)
    torch.cuda.synchronize()
    for u, v in zip(a, b):
        assert (u is None) == (v is None)
        if u is not None:
            assert torch.equal(u.view(torch.uint8), v.view(torch.uint8))
    with pytest.raises(ValueError):  # a plan of the other layout
        permute(x, cnt, idx, counts, probs, plan=build_expert_plan(cnt, counts))
