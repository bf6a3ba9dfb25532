"""The allocation-free RMSNorm backward (fq_rmsnorm_bwd_noalloc) against the entry
point it is a variant of (fq_rmsnorm_bwd), through the C ABI: same inputs, outputs
bit for bit, on two calls in a row of which the second is smaller (the library's
fixed scratch array still holds the first call's partial rows then)."""
import pytest
import torch

from tests.helpers import announce, gamma_bf16, gen, randn_bf16

pytestmark = pytest.mark.gpu


def _both(L, stream, gpu, M, n, seed, with_rstd):
    g = gen(seed)
    x = (torch.randn(M, n, generator=g) ** 3).to(torch.bfloat16).to(gpu)
    dy = randn_bf16(g, M, n).to(gpu)
    w = gamma_bf16(g, n).to(gpu)
    rstd = None
    if with_rstd:
        rstd = torch.rsqrt(x.float().pow(2).mean(1) + 1e-6).contiguous()
    n_part = int(L.fq_rmsnorm_bwd_num_partials(M, n))
    part = torch.empty((n_part, n), device=gpu, dtype=torch.float32)
    dx_a = torch.empty_like(x)
    dg_a = torch.empty((n,), device=gpu, dtype=torch.float32)
    dx_b = torch.full_like(x, 7.0)
    dg_b = torch.full((n,), 7.0, device=gpu, dtype=torch.float32)
    rp = None if rstd is None else rstd.data_ptr()
    rc = L.fq_rmsnorm_bwd(dy.data_ptr(), x.data_ptr(), w.data_ptr(), rp, dx_a.data_ptr(), dg_a.data_ptr(),
                          part.data_ptr(), n_part, M, n, 1e-6, stream)
    assert rc == 0, L.fq_last_error()
    rc = L.fq_rmsnorm_bwd_noalloc(dy.data_ptr(), x.data_ptr(), w.data_ptr(), rp, dx_b.data_ptr(), dg_b.data_ptr(),
                                  M, n, 1e-6, stream)
    assert rc == 0, L.fq_last_error()
    torch.cuda.synchronize()
    return dx_a, dg_a, dx_b, dg_b


def test_rmsnorm_bwd_noalloc_matches_rmsnorm_bwd(gpu):
    from linghe_amd import _lib

    L = _lib.lib
    # two calls in a row: wide rows and many partial rows first, then a smaller, narrower input
    for M, n, with_rstd in ((4100, 7168, False), (520, 1536, True), (40, 128, False)):
        announce("rmsnorm_bwd_noalloc", M, n, with_rstd)
        x = torch.empty(1, device=gpu)  # make sure the stream handle is the current torch stream's
        stream = _lib.stream_of(x)
        dx_a, dg_a, dx_b, dg_b = _both(L, stream, gpu, M, n, 61, with_rstd)
        assert torch.equal(dx_a.view(torch.int16), dx_b.view(torch.int16))
        assert torch.equal(dg_a.view(torch.int32), dg_b.view(torch.int32))
        assert bool(torch.isfinite(dg_b).all())
    # the advertised property: the call itself allocates nothing on the device (the driver's count of
    # free device memory is the same before and after a call whose buffers all exist already)
    announce("rmsnorm_bwd_noalloc leaves the free-memory count unchanged")
    g = gen(62)
    M, n = 2048, 4096
    x = randn_bf16(g, M, n).to(gpu)
    dy = randn_bf16(g, M, n).to(gpu)
    w = gamma_bf16(g, n).to(gpu)
    dx = torch.empty_like(x)
    dg = torch.empty((n,), device=gpu, dtype=torch.float32)
    stream = _lib.stream_of(x)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(gpu)[0]
    for _ in range(3):
        rc = L.fq_rmsnorm_bwd_noalloc(dy.data_ptr(), x.data_ptr(), w.data_ptr(), None, dx.data_ptr(), dg.data_ptr(),
                                      M, n, 1e-6, stream)
        assert rc == 0, L.fq_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(gpu)[0] == free_before
    # beyond the fixed array (and the RMSNorm kernels' own limit): refused with a clear error, nothing launched
    rc = L.fq_rmsnorm_bwd_noalloc(None, None, None, None, None, None, 128, 8192 + 128, 1e-6, None)
    assert rc == -2 and L.fq_last_error()
    # no rows: dgamma is zeroed, nothing else is touched
    dg = torch.full((256,), 3.0, device=gpu, dtype=torch.float32)
    rc = L.fq_rmsnorm_bwd_noalloc(None, None, None, None, None, dg.data_ptr(), 0, 256, 1e-6,
                                  _lib.stream_of(dg))
    assert rc == 0, L.fq_last_error()
    torch.cuda.synchronize()
    assert float(dg.abs().max()) == 0.0
