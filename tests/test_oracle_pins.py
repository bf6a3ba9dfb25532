"""Pins of the CPU oracle (oracle/fq_oracle.py).  The reference holds no golden
vectors for this path, so each oracle function is checked against what the
mathematics fixes, chosen so that a plausible mistake (wrong fmax, dropped 1/n,
transposed scale, off-by-one block origin, round-half-up instead of
half-to-even) fails:

* an independent software FP8 encoder (integer arithmetic, from the OCP FP8
  spec) and a brute-force nearest-code search over all 256 codes;
* invariants: amax -> +-fmax, dequantisation bound, all-zero group -> 1e-30 / 0;
* element-by-element index formulas of the output layouts
  (linghe/utils/silu.py:248-276,507-554; linghe/quant/block.py:96-126,217-248);
* closed-form gradients against fp64 autograd (gradcheck).
"""
import math

import numpy as np
import pytest
import torch

from oracle import compare as C
from oracle import fq_oracle as O

E4M3, E5M2 = torch.float8_e4m3fn, torch.float8_e5m2


# ------------------------------------------------------------------ software fp8
def decode_table(kind):
    """value of each of the 256 codes (nan for NaN/inf codes), from the OCP spec."""
    mant, bias = (3, 7) if kind == "e4m3" else (2, 15)
    vals = np.zeros(256, dtype=np.float64)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        e = (code & 0x7F) >> mant
        m = code & ((1 << mant) - 1)
        if kind == "e4m3" and (code & 0x7F) == 0x7F:
            vals[code] = np.nan
        elif kind == "e5m2" and e == 31:
            vals[code] = np.nan
        elif e == 0:
            vals[code] = sign * m * 2.0 ** (1 - bias - mant)
        else:
            vals[code] = sign * (1 + m / (1 << mant)) * 2.0 ** (e - bias)
    return vals


def soft_encode(x, kind):
    """fp32 -> fp8 code, round to nearest even, integer arithmetic on the fp32
    bit pattern (inputs must be within the finite fp8 range)."""
    mant, bias = (3, 7) if kind == "e4m3" else (2, 15)
    bits = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.int64)
    sign = (bits >> 31) & 1
    e32 = ((bits >> 23) & 0xFF) - 127
    m32 = bits & 0x7FFFFF
    out = np.zeros(bits.shape, dtype=np.int64)
    emin = 1 - bias
    for idx in np.ndindex(bits.shape):
        e, m = int(e32[idx]), int(m32[idx])
        if e == -127:  # fp32 zero / subnormal -> 0
            code = 0
        else:
            sig = (1 << 23) | m                # 24-bit significand, value = sig * 2^(e-23)
            shift = 23 - mant                  # bits to drop for a normal result
            if e < emin:
                shift += emin - e              # subnormal: fixed exponent emin
                e_out = 0
            else:
                e_out = e + bias
            if shift > 40:
                q = 0
            else:
                q = sig >> shift
                rem = sig & ((1 << shift) - 1)
                half = 1 << (shift - 1)
                if rem > half or (rem == half and (q & 1)):
                    q += 1
            if e_out == 0:
                code = q                        # may carry into the first normal
            else:
                code = ((e_out - 1) << mant) + q  # q includes the hidden bit
        out[idx] = code | (int(sign[idx]) << 7)
    return out.astype(np.uint8)


@pytest.mark.parametrize("kind,dtype,fmax", [("e4m3", E4M3, 448.0), ("e5m2", E5M2, 57344.0)])
def test_torch_cast_matches_software_encoder(kind, dtype, fmax):
    table = decode_table(kind)
    finite = table[np.isfinite(table)]
    assert finite.max() == fmax == O.fp8_max(dtype)
    # every code decodes as torch decodes it
    tdec = torch.arange(256, dtype=torch.uint8).view(dtype).float().numpy().astype(np.float64)
    ok = np.isfinite(table)
    assert np.array_equal(tdec[ok], table[ok])
    rng = np.random.default_rng(0)
    pos = np.sort(np.unique(np.abs(finite)))
    mids = (pos[:-1] + pos[1:]) / 2                      # exact ties
    near = np.concatenate([np.nextafter(mids.astype(np.float32), np.float32(0)),
                           np.nextafter(mids.astype(np.float32), np.float32(1e9))])
    rnd = (rng.standard_normal(4000) * 10.0 ** rng.integers(-6, 2, 4000)).astype(np.float32)
    rnd = np.clip(rnd, -fmax, fmax)
    vals = np.concatenate([pos, -pos, mids, -mids, near, rnd]).astype(np.float32)
    got = torch.from_numpy(vals).to(dtype).view(torch.uint8).numpy()
    want = soft_encode(vals, kind)
    # +0 / -0 both acceptable for values that round to zero
    same = (got == want) | (((got & 0x7F) == 0) & ((want & 0x7F) == 0))
    assert same.all(), (vals[~same][:5], got[~same][:5], want[~same][:5])


@pytest.mark.parametrize("round_scale", [False, True])
@pytest.mark.parametrize("dtype,kind", [(E4M3, "e4m3"), (E5M2, "e5m2")])
def test_group_quant_is_nearest_code_of_exact_quotient(round_scale, dtype, kind):
    g = torch.Generator().manual_seed(3)
    v = torch.randn(5, 300, generator=g) * torch.tensor([1e-3, 1.0, 50.0, 1e4, 0.0]).reshape(5, 1)
    v[1, 17] = 77.0
    codes, scales = O.group_quant_1x128(v, round_scale, dtype)
    assert codes.shape == (5, 300) and scales.shape == (5, 3) and scales.dtype == torch.float32
    fmax = O.fp8_max(dtype)
    table = decode_table(kind)
    cand = np.where(np.isfinite(table), table, np.inf)
    vp = torch.nn.functional.pad(v, (0, 84)).reshape(5, 3, 128)
    for r in range(5):
        for b in range(3):
            amax = float(vp[r, b].abs().max())
            s = float(scales[r, b])
            raw = float(np.float32(max(np.float32(amax) / np.float32(fmax), np.float32(1e-30))))
            if round_scale:
                assert s >= raw and s < 2 * raw * (1 + 1e-6) and math.log2(s) == round(math.log2(s))
            else:
                assert s == raw
            for c in range(min(128, 300 - 128 * b)):
                x = float(vp[r, b, c])
                t = float(np.float32(x) / np.float32(s))   # the fp32 quotient the oracle rounds
                code = int(codes[r, 128 * b + c].view(torch.uint8))
                err = np.abs(cand - t)
                best = err.min()
                assert abs(table[code] - t) <= best * (1 + 1e-12), (r, b, c, x, s, code)
                if amax > 0 and abs(x) == amax and not round_scale:
                    assert abs(table[code]) == fmax
    # all-zero row: scale floor and zero codes
    floor = 2.0 ** -99 if round_scale else 1e-30   # ceil-to-power-of-two of 1e-30 is 2^-99
    assert torch.all(scales[4] == torch.tensor(floor, dtype=torch.float32))
    assert torch.all((codes[4].view(torch.uint8) & 0x7F) == 0)  # +0 or -0
    # dequantisation bound
    s_elem = scales.repeat_interleave(128, 1)[:, :300]
    C.assert_dequant_bound(v, codes, s_elem, dtype)


def test_pow2_round_matches_documented_torch_behaviour():
    # exact powers stay, anything clearly above goes to the next power
    s = torch.tensor([2.0 ** -10, 2.0 ** -10 * 1.5, 3.0, 1e-30, 0.75], dtype=torch.float32)
    r = O._pow2_ceil(s)
    assert r.tolist() == [2.0 ** -10, 2.0 ** -9, 4.0, 2.0 ** -99, 1.0]
    # values one fp32 ulp above a power of two are NOT rounded up by fp32 log2
    # (the property the device code reproduces with integer arithmetic)
    one_ulp_up = torch.tensor([2.0 ** -10], dtype=torch.float32).view(torch.int32) + 1
    assert float(O._pow2_ceil(one_ulp_up.view(torch.float32))) == 2.0 ** -10


# ------------------------------------------------------------------ layouts
def group_amax_scale(vals, fmax=448.0):
    a = np.float32(np.max(np.abs(np.asarray(vals, dtype=np.float32)))) if len(vals) else np.float32(0)
    return np.float32(max(a / np.float32(fmax), np.float32(1e-30)))


def test_blockwise_layouts_elementwise():
    """q[r*n+c], scale[b*M+r], qt[c*M+r], tscale[rb*n+c] on a ragged M."""
    M, n = 200, 256
    y = torch.randn(M, n, generator=torch.Generator().manual_seed(5))
    q, s, qt, st = O.blockwise_quant(y, False)
    assert q.shape == (M, n) and s.shape == (n // 128, M)
    assert qt.shape == (n, M) and st.shape == ((M + 127) // 128, n)
    yn = y.numpy()
    rng = np.random.default_rng(1)
    for _ in range(300):
        r, c = int(rng.integers(M)), int(rng.integers(n))
        b, rb = c // 128, r // 128
        s_row = group_amax_scale(yn[r, 128 * b:128 * b + 128])
        s_col = group_amax_scale(yn[128 * rb:min(M, 128 * rb + 128), c])
        assert float(s.reshape(-1)[b * M + r]) == s_row
        assert float(st.reshape(-1)[rb * n + c]) == s_col
        want_row = torch.tensor(np.float32(yn[r, c]) / s_row).to(E4M3).view(torch.uint8)
        want_col = torch.tensor(np.float32(yn[r, c]) / s_col).to(E4M3).view(torch.uint8)
        assert int(q.view(torch.uint8).reshape(-1)[r * n + c]) == int(want_row)
        assert int(qt.view(torch.uint8).reshape(-1)[c * M + r]) == int(want_col)
    # a transposed tail block (rows 128..199) only sees existing rows
    assert float(st[1, 0]) == group_amax_scale(yn[128:200, 0])


@pytest.mark.parametrize("counts", [[130, 0, 5, 128], [1], [0, 0], [300, 17]])
def test_batched_layouts_elementwise(counts):
    """per expert e: q[(si+i)*n+c], scale[si*nb + b*ce + i], qt[si*n + c*ce + i],
    tscale[(tb + i//128)*n + c]; column blocks restart at each expert."""
    n = 256
    nb = n // 128
    M = sum(counts)
    g = torch.Generator().manual_seed(6)
    x = torch.randn(M, 2 * n, generator=g).to(torch.bfloat16)
    w = torch.rand(M, 1, generator=g)
    q, s, qt, st = O.batch_weighted_silu_and_block_quant_forward(x, w, counts, False)
    blocks = sum((c + 127) // 128 for c in counts)
    assert q.shape == (M, n) and s.shape == (M * nb,) and qt.shape == (M * n,) and st.shape == (blocks * n,)
    if M == 0:
        return
    y = (torch.sigmoid(x.float()[:, :n]) * x.float()[:, :n] * x.float()[:, n:] * w).numpy()
    rng = np.random.default_rng(2)
    si = tb = 0
    for ce in counts:
        for _ in range(40 if ce else 0):
            i, c = int(rng.integers(ce)), int(rng.integers(n))
            b, rb = c // 128, i // 128
            s_row = group_amax_scale(y[si + i, 128 * b:128 * b + 128])
            lo = si + 128 * rb
            s_col = group_amax_scale(y[lo:min(si + ce, lo + 128), c])
            assert float(s[si * nb + b * ce + i]) == s_row
            assert float(st[(tb + rb) * n + c]) == s_col
            want_row = torch.tensor(np.float32(y[si + i, c]) / s_row).to(E4M3).view(torch.uint8)
            want_col = torch.tensor(np.float32(y[si + i, c]) / s_col).to(E4M3).view(torch.uint8)
            assert int(q.view(torch.uint8)[si + i, c]) == int(want_row)
            assert int(qt.view(torch.uint8)[si * n + c * ce + i]) == int(want_col)
        si += ce
        tb += (ce + 127) // 128
    # same packing for the plain batched quantiser
    xs = torch.randn(M, n, generator=g).to(torch.bfloat16)
    q2, s2, qt2, st2 = O.batch_blockwise_quant(xs, counts, False)
    e0 = next(k for k, c in enumerate(counts) if c)
    s0 = sum(counts[:e0])
    assert float(s2[s0 * nb]) == group_amax_scale(xs.float().numpy()[s0, :128])


def test_rms_gemm_logits_against_fp64():
    g = torch.Generator().manual_seed(79)
    x = (torch.randn(64, 256, generator=g) ** 2).to(torch.bfloat16)
    w = torch.randn(256, generator=g).to(torch.bfloat16)
    rw = torch.randn(128, 256, generator=g).to(torch.bfloat16)
    y16, r, logits, q, s, qt, st = O.rms_gemm_block_quant_forward(x, w, rw)
    xd = x.double()
    rd = torch.rsqrt((xd * xd).mean(1) + 1e-6)
    yd = xd * rd[:, None] * w.double()
    torch.testing.assert_close(logits.double(), yd @ rw.double().t(), rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(r.double(), rd, rtol=1e-6, atol=0)
    assert torch.equal(y16, yd.float().to(torch.bfloat16)) or (y16.float() - yd.float()).abs().max() < 2e-2
    ref = O.rms_norm_and_block_quant_forward(x, w)
    assert torch.equal(q.view(torch.uint8), ref[0].view(torch.uint8)) and torch.equal(s, ref[1])


def test_block_quant_128_elementwise():
    g = torch.Generator().manual_seed(78)
    w = (torch.randn(256, 384, generator=g) ** 3).to(torch.bfloat16)
    w[128:, 128:256] = 0.0  # an all-zero block: floor scale, zero codes
    q, s = O.block_quant_128(w, round_scale=False)
    assert s.shape == (2, 3)
    wf = w.float().numpy()
    qf = q.float().numpy()
    for rb in range(2):
        for cb in range(3):
            blk = wf[rb * 128:(rb + 1) * 128, cb * 128:(cb + 1) * 128]
            sc = group_amax_scale(blk.reshape(-1))
            assert float(s[rb, cb]) == sc
            for (i, j) in ((0, 0), (5, 127), (127, 64)):
                want = float(torch.tensor(blk[i, j] / sc).to(torch.float8_e4m3fn).float())
                assert qf[rb * 128 + i, cb * 128 + j] == want
    assert float(s[1, 1]) == np.float32(1e-30) and float(q[128:, 128:256].float().abs().max()) == 0.0
    q2, s2 = O.block_quant_128(w, round_scale=True)
    assert torch.equal(s2, O._pow2_ceil(s))


def test_pad_permute_layouts_elementwise():
    """gather + pad-to-16 + quant against the offsets the reference kernel writes
    (linghe/utils/gather.py:871-940): region start psi = sum of padded counts,
    strides = padded count, padding rows zero with the floor scale."""
    g = torch.Generator().manual_seed(77)
    counts = [5, 0, 130, 16]
    m, N, E = 40, 256, len(counts)
    nb = N // 128
    x = torch.randn(m, N, generator=g).to(torch.bfloat16)
    probs = torch.rand(m, E, generator=g)
    idx = torch.randint(0, m, (sum(counts),), generator=g)
    q, s, qt, st, p = O.batch_block_pad_permute_with_indices(x, idx, probs, counts, round_scale=False)
    padded = O.pad_indices(idx, counts)
    pcs = [(c + 15) // 16 * 16 for c in counts]
    assert padded.numel() == sum(pcs) == q.numel() // N == p.numel()
    qf = q.float().reshape(-1).numpy()
    qtf = qt.float().reshape(-1).numpy()
    sf, stf, pf = s.numpy(), st.numpy(), p.numpy()
    xf = x.float().numpy()
    psi = blk = src0 = 0
    for e, (c, pc) in enumerate(zip(counts, pcs)):
        for i in range(pc):
            row = xf[int(idx[src0 + i])] if i < c else np.zeros(N, dtype=np.float32)
            if i < c:
                assert int(padded[psi + i]) == int(idx[src0 + i])
                assert pf[psi + i] == float(probs[int(idx[src0 + i]), e])
            else:
                assert pf[psi + i] == 0.0
            for b in range(nb):
                sc = group_amax_scale(row[b * 128:(b + 1) * 128])
                assert sf[psi * nb + b * pc + i] == sc
                for c_ in (b * 128, b * 128 + 77):
                    want = float(torch.tensor(row[c_] / sc).to(torch.float8_e4m3fn).float())
                    assert qf[(psi + i) * N + c_] == want
            # transposed copy: column c_ of the padded [pc, N] block, 128-row groups
            rbk = i // 128
            rows = [xf[int(idx[src0 + k])] if k < c else np.zeros(N, dtype=np.float32)
                    for k in range(rbk * 128, min(pc, rbk * 128 + 128))]
            for c_ in (3, 200):
                sc = group_amax_scale([r[c_] for r in rows])
                assert stf[(blk + rbk) * N + c_] == sc
                want = float(torch.tensor(row[c_] / sc).to(torch.float8_e4m3fn).float())
                assert qtf[psi * N + c_ * pc + i] == want
        psi += pc
        blk += (c + 127) // 128
        src0 += c


def test_backward_layout_halves():
    """dx1 | dx2 share one [2n/128, M] scale tensor and one [2n, M] transposed
    tensor: rows 0..nb-1 / columns 0..n-1 belong to dx1 (linghe/utils/silu.py:382-420)."""
    M, n = 128, 128
    g = torch.Generator().manual_seed(7)
    x = torch.randn(M, 2 * n, generator=g).to(torch.bfloat16)
    dy = torch.randn(M, n, generator=g).to(torch.bfloat16)
    q, s, qt, st = O.silu_and_block_quant_backward(dy, x, False)
    assert q.shape == (M, 2 * n) and s.shape == (2, M) and qt.shape == (2 * n, M) and st.shape == (1, 2 * n)
    dx, _ = O.swiglu_grad_fp32(dy, x)
    assert float(s[0, 3]) == group_amax_scale(dx[3, :n].numpy())
    assert float(s[1, 3]) == group_amax_scale(dx[3, n:].numpy())
    assert float(st[0, n + 5]) == group_amax_scale(dx[:, n + 5].numpy())


# ------------------------------------------------------------------ gradients
def test_rmsnorm_matches_formula_and_fp64_autograd():
    g = torch.Generator().manual_seed(8)
    x = (torch.randn(9, 256, generator=g) ** 3).to(torch.bfloat16)
    w = torch.randn(256, generator=g).to(torch.bfloat16)
    dy = torch.randn(9, 256, generator=g).to(torch.bfloat16)
    y, rstd = O.rms_norm_fp32(x, w)
    xf, wf = x.double(), w.double()
    r64 = torch.rsqrt((xf * xf).mean(-1, keepdim=True) + 1e-6)
    torch.testing.assert_close(y.double(), xf * r64 * wf, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(rstd.double(), r64.squeeze(-1), rtol=1e-6, atol=0)
    # fp64 autograd of the definition
    x64 = xf.clone().requires_grad_()
    w64 = wf.clone().requires_grad_()
    (x64 * torch.rsqrt((x64 * x64).mean(-1, keepdim=True) + 1e-6) * w64).backward(dy.double())
    dx, dg = O.rms_norm_backward(x, w, dy)
    dxc, dgc = O.rms_norm_backward_closed_form(x, w, dy)
    assert dx.dtype == torch.bfloat16 and dg.dtype == torch.float32
    torch.testing.assert_close(dx.double(), x64.grad, rtol=1e-2, atol=1e-2 * float(x64.grad.abs().max()))
    torch.testing.assert_close(dg.double(), w64.grad, rtol=1e-4, atol=1e-4 * float(w64.grad.abs().max()))
    torch.testing.assert_close(dgc.double(), w64.grad, rtol=1e-4, atol=1e-4 * float(w64.grad.abs().max()))
    torch.testing.assert_close(dxc.float(), dx.float(), rtol=2e-2, atol=1e-2 * float(x64.grad.abs().max()))
    # gradcheck the closed form on a tiny fp64 problem
    def f(a, b):
        return a * torch.rsqrt((a * a).mean(-1, keepdim=True) + 1e-6) * b
    a = torch.randn(3, 8, dtype=torch.float64, requires_grad=True)
    b = torch.randn(8, dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(f, (a, b))


def test_swiglu_gradient_closed_form():
    """dx1 = s*g*x2*(1 + x1*(1-s)), dx2 = s*g*x1, dw = sum(s*x1*x2*g)
    (linghe/utils/silu.py:377-399,1148-1165) against the oracle's autograd."""
    g = torch.Generator().manual_seed(9)
    x = torch.randn(16, 256, generator=g).to(torch.bfloat16)
    dy = torch.randn(16, 128, generator=g).to(torch.bfloat16)
    w = torch.rand(16, 1, generator=g)
    dx, dw = O.swiglu_grad_fp32(dy, x, w)
    x1, x2, gg = x.double()[:, :128], x.double()[:, 128:], dy.double()
    s = torch.sigmoid(x1)
    wd = w.double()
    torch.testing.assert_close(dx.double()[:, :128], s * gg * x2 * wd * (1 + x1 * (1 - s)), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dx.double()[:, 128:], s * gg * x1 * wd, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dw.double(), (s * x1 * x2 * gg).sum(1, keepdim=True), rtol=1e-5, atol=1e-6)
    y = O.swiglu_fp32(x, w)
    torch.testing.assert_close(y.double(), s * x1 * x2 * wd, rtol=1e-6, atol=1e-7)
    assert O.weighted_silu_forward(x, w).dtype == torch.bfloat16


def test_compare_rules():
    a = torch.tensor([1.0, 2.0, 3.0])
    b = a.clone()
    b[1] = torch.nextafter(b[1], torch.tensor(9.0))
    rep = C.compare_scales(a, b)
    assert (rep.exact, rep.within_1ulp, rep.max_ulp) == (2, 3, 1)
    codes = torch.tensor([0x00, 0x80, 0x7E, 0x01, 0x81], dtype=torch.uint8)
    other = torch.tensor([0x80, 0x00, 0x7D, 0x81, 0x01], dtype=torch.uint8)
    rep = C.compare_codes(codes, other)
    assert rep.max_step == 2 and rep.identical == 2  # +0/-0 identical on the value line
    with pytest.raises(AssertionError):
        C.assert_codes(codes, other)


# ---------------------------------------------------------------------------
# the fp64 "truth" used by the GPU scale tests: the torch oracle must lie inside
# the fp32 error bound it derives, and a scale a few ulp further out must not
# ---------------------------------------------------------------------------
def test_truth_bounds_hold_for_the_oracle_and_reject_a_wrong_scale():
    from tests import truth as T

    g = torch.Generator().manual_seed(77)
    # RMSNorm + quant
    x = (torch.randn(256, 512, generator=g) ** 3).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(512, generator=g)).to(torch.bfloat16)
    ref = O.rms_norm_and_block_quant_forward(x, w, 1e-6)
    y, err, r64 = T.rmsnorm_values(x, w, 1e-6)
    sr, br, sc, bc = T.scale_bounds(y, err)
    assert bool(((ref[1].double() - sr).abs() <= br).all()) and bool(((ref[4].double() - sc).abs() <= bc).all())
    assert bool(((ref[2].double() - r64).abs() <= 5.5 * T.U * r64).all())
    # a scale 20 ulp away is outside the bound (the bound is not vacuous)
    off = (ref[1].view(torch.int32) + 20).view(torch.float32)
    assert not bool(((off.double() - sr).abs() <= br).all())
    # SwiGLU forward and backward, per-expert packing included
    x2 = torch.randn(300, 512, generator=g).to(torch.bfloat16)
    dy = (1e-2 * torch.randn(300, 256, generator=g)).to(torch.bfloat16)
    wt = torch.rand(300, 1, generator=g)
    counts = [130, 0, 7, 163]
    rf = O.batch_weighted_silu_and_block_quant_forward(x2, wt, counts, False)
    yv, ye = T.swiglu_values(x2, wt)
    sr, br, sc, bc = T.scale_bounds_per_expert(yv, ye, counts)
    assert bool(((rf[1].double() - sr).abs() <= br).all()) and bool(((rf[3].double() - sc).abs() <= bc).all())
    rb = O.batch_weighted_silu_and_block_quant_backward(dy, x2, wt, counts, False)
    dv, de, dw64 = T.swiglu_grad_values(dy, x2, wt)
    sr, br, sc, bc = T.scale_bounds_per_expert(dv, de, counts)
    assert bool(((rb[1].double() - sr).abs() <= br).all()) and bool(((rb[4].double() - sc).abs() <= bc).all())
    torch.testing.assert_close(rb[2].view(-1).double(), dw64, rtol=1e-5, atol=1e-7)
    # the fp64 derivative itself, against autograd in fp64
    xd = x2.double().requires_grad_()
    (torch.sigmoid(xd[:, :256]) * xd[:, :256] * xd[:, 256:] * wt.double()).backward(dy.double())
    torch.testing.assert_close(dv, xd.grad, rtol=1e-12, atol=1e-14)
    # a cancelling element gets a wider bound than its neighbours: x1 = -1.2785 makes 1 + x1 (1 - s) ~ 0
    xc = torch.tensor([[-1.2785, 0.5, 1.0, 1.0]], dtype=torch.float64)
    dvc, dec, _ = T.swiglu_grad_values(torch.ones(1, 2, dtype=torch.float64), xc)
    assert float(dec[0, 0] / dvc[0, 0].abs()) > 50 * float(dec[0, 1] / dvc[0, 1].abs())
