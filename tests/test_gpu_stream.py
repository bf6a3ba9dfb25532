"""The no-work kernel behind the measured ceilings moves every byte it is asked to move exactly
once, in every variant: a ceiling taken from a variant that skipped part of the buffers would
be too low."""
from __future__ import annotations

import pytest
import torch

from linghe_amd import _lib
from tests.helpers import announce

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("order", [0, 1, 2, 3])
@pytest.mark.parametrize("chunks", [4, 8, 16])
@pytest.mark.parametrize("workgroups", [0, 96])
def test_stream_variant_copies_every_byte(gpu, order, chunks, workgroups):
    announce("no-work kernel", order, chunks, workgroups)
    L = _lib.lib
    # sizes that are not whole steps, tiles or blocks of rows; read and written sizes differ
    read_bytes = 16 * (3 * 65536 + 4097)
    write_bytes = 16 * (2 * 65536 + 771)
    g = torch.Generator(device=gpu).manual_seed(7)
    src = torch.randint(1, 1 << 30, (read_bytes // 4,), generator=g, device=gpu, dtype=torch.int32)
    dst = torch.full((write_bytes // 4 + 64,), -1, device=gpu, dtype=torch.int32)
    sink = torch.zeros(4, device=gpu, dtype=torch.int32)
    stream = torch.cuda.current_stream().cuda_stream
    for nt in (0, 1):
        dst.fill_(-1)
        _lib.check(L.fq_stream_rw_variant(src.data_ptr(), read_bytes, dst.data_ptr(), write_bytes, sink.data_ptr(),
                                          chunks, workgroups, order, nt, nt, stream))
        torch.cuda.synchronize()
        assert torch.equal(dst[:write_bytes // 4], src[:write_bytes // 4])
        assert bool((dst[write_bytes // 4:] == -1).all()), "wrote beyond write_bytes"
