"""CPU checks of the drop-in boundary: the shared library loads and exports every
symbol include/fq_api.h declares (no compute is launched), the Python entry
points keep the reference's signatures, and host-side argument checks fire
before anything reaches a device."""
import ctypes
import inspect
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fq_api.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from linghe_amd import _lib

    names = declared_symbols()
    assert len(names) >= 13
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(raw, name), f"{name} declared in fq_api.h but not exported"
    bound = set(_lib.SIGNATURES) | set(_lib.OTHER_SYMBOLS)
    assert bound == set(names), bound ^ set(names)
    assert _lib.lib.fq_version() >= 100


def _ctype_of(decl: str):
    """C parameter declaration -> the ctypes type a binding must use for it."""
    decl = decl.strip()
    if "*" in decl:
        return ctypes.c_void_p
    words = [w for w in re.split(r"\s+", decl) if w not in ("const",)]
    base = " ".join(words[:-1])  # drop the parameter name
    return {"int": ctypes.c_int, "int64_t": ctypes.c_int64, "float": ctypes.c_float}[base]


def test_argument_types_match_header():
    """Every bound signature agrees with its declaration type by type: a pointer is a
    void pointer, int / int64_t / float map to the ctypes of the same width."""
    from linghe_amd import _lib

    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name, argtypes in _lib.SIGNATURES.items():
        m = re.search(r"\bint\s+" + name + r"\s*\((.*?)\)\s*;", text, flags=re.S)
        assert m, name
        declared = [_ctype_of(a) for a in m.group(1).split(",") if a.strip()]
        assert declared == list(argtypes), (name, declared, argtypes)
    m = re.search(r"\bint64_t\s+fq_rmsnorm_bwd_num_partials\s*\((.*?)\)\s*;", text, flags=re.S)
    assert [_ctype_of(a) for a in m.group(1).split(",")] == list(_lib.lib.fq_rmsnorm_bwd_num_partials.argtypes)
    assert _lib.lib.fq_rmsnorm_bwd_num_partials.restype is ctypes.c_int64


def test_c_side_validation_without_gpu():
    """Shape / flag errors are reported by return code before any HIP call."""
    from linghe_amd import _lib

    L = _lib.lib
    # width not a multiple of 128
    rc = L.fq_blockwise_quant(None, None, None, None, None, 16, 100, 0, 2, 0, None)
    assert rc == -2 and b"128" in L.fq_last_error()
    # bad mode
    rc = L.fq_swiglu_quant_fwd(None, None, None, None, None, 16, 128, 0, 7, 0, None)
    assert rc == -1
    # NULL outputs
    rc = L.fq_blockwise_quant(None, None, None, None, None, 16, 128, 0, 2, 0, None)
    assert rc == -1
    # unknown fp8 kind
    rc = L.fq_group_quant(None, None, None, 16, 128, 0, 9, None)
    assert rc == -1
    # hidden size too large for the row kernels
    rc = L.fq_rmsnorm_fwd(None, None, None, None, 4, 16384, 1e-6, 0, None)
    assert rc == -2
    # router weight packing: K not a multiple of 128, N beyond the limit, NULL buffers
    assert L.fq_pack_router_weight(None, 0, None, 100, 128, None) == -2
    assert L.fq_pack_router_weight(None, 0, None, 2048, 8192 + 128, None) == -2
    assert L.fq_pack_router_weight(None, 0, None, 2048, 256, None) == -1
    assert L.fq_rmsnorm_router_quant_fwd_packed(None, None, None, 0, None, None, None, None, None, 128, 2048, 100,
                                                1e-6, 0, 0, None) == -2
    # the no-work kernel's variants: chunks per lane 4 / 8 / 16 only, order 0..3
    assert L.fq_stream_rw_variant(None, 0, None, 0, None, 4, 0, 0, 0, 0, None) == -1          # no sink
    assert L.fq_stream_rw_variant(None, 16, None, 0, None, 5, 0, 0, 0, 0, None) == -1
    assert L.fq_stream_rw_variant(None, 24, None, 0, None, 4, 0, 0, 0, 0, None) == -2         # not a multiple of 16
    # 128x128 block quant needs whole blocks of rows
    rc = L.fq_block_quant(None, None, None, 100, 256, 0, 0, None)
    assert rc == -2 and b"128" in L.fq_last_error()
    # router GEMM: outputs in multiples of 128, rows in groups of 32
    rc = L.fq_rmsnorm_router_quant_fwd(None, None, None, 0, None, None, None, None, None, None, 128, 2048, 200, 1e-6,
                                       0, 0, None)
    assert rc == -2 and b"router" in L.fq_last_error()
    rc = L.fq_rmsnorm_router_quant_fwd(None, None, None, 1, None, None, None, None, None, None, 100, 2048, 256, 1e-6,
                                       0, 0, None)
    assert rc == -2
    assert L.fq_rmsnorm_router_scratch_bytes(2048, 256, 0) == 256 * 2048 * 2
    assert L.fq_rmsnorm_router_scratch_bytes(2048, 256, 1) == 256 * 2048 * 4
    # gather + pad: the output row count is a sum of multiples of 16; probs and prob_out go together
    rc = L.fq_batched_pad_permute_quant(None, None, 0, 4, 1, None, None, 0, None, None, None, None, None, 64, 100, 256,
                                        0, 0, None)
    assert rc == -2 and b"16" in L.fq_last_error()
    # more rows / wider than the 32-bit lane offsets of a tile allow
    rc = L.fq_blockwise_quant(None, None, None, None, None, (1 << 24) + 16, 128, 0, 2, 0, None)
    assert rc == -2
    # bf16 SwiGLU: weight and dw go together
    rc = L.fq_swiglu_bwd(None, None, None, 0, None, ctypes.c_void_p(16), 16, 128, None)
    assert rc == -1
    # RMSNorm backward: a wrong partial count is refused before anything else is looked at,
    # and with rows present every pointer must be there (no launch with a NULL gamma)
    n_part = L.fq_rmsnorm_bwd_num_partials(64, 256)
    rc = L.fq_rmsnorm_bwd(None, None, None, None, None, ctypes.c_void_p(256), ctypes.c_void_p(256), n_part + 1, 64,
                          256, 1e-6, None)
    assert rc == -2
    rc = L.fq_rmsnorm_bwd(ctypes.c_void_p(256), ctypes.c_void_p(256), None, None, ctypes.c_void_p(256),
                          ctypes.c_void_p(256), ctypes.c_void_p(256), n_part, 64, 256, 1e-6, None)
    assert rc == -1 and b"NULL" in L.fq_last_error()
    # ... and with no rows a NULL dgamma is still refused (it is the one output that is written)
    rc = L.fq_rmsnorm_bwd(None, None, None, None, None, None, None, L.fq_rmsnorm_bwd_num_partials(0, 256), 0, 256,
                          1e-6, None)
    assert rc == -1 and b"dgamma" in L.fq_last_error()
    # empty problem is a no-op
    assert L.fq_group_quant(None, None, None, 0, 128, 0, 0, None) == 0
    assert L.fq_swiglu_fwd(None, None, 0, None, 0, 128, None) == 0
    with pytest.raises(RuntimeError):
        _lib.check(-2)


REFERENCE_SIGNATURES = {
    # reference file:line -> (module, function, parameter names in order)
    "linghe/utils/norm.py:58": ("linghe_amd.utils.norm", "triton_rms_norm_forward",
                                ["x", "weight", "eps", "out", "rms"]),
    "linghe/utils/norm.py:144": ("linghe_amd.utils.norm", "triton_rms_norm_backward",
                                 ["grad_output", "x", "w", "eps", "rms"]),
    "linghe/utils/norm.py:343": ("linghe_amd.utils.norm", "triton_rms_norm_and_block_quant_forward",
                                 ["x", "weight", "eps", "out", "scale", "rms", "round_scale", "output_mode"]),
    "linghe/utils/silu.py:279": ("linghe_amd.utils.silu", "triton_silu_and_block_quant_forward",
                                 ["x", "out", "scale", "round_scale", "output_mode"]),
    "linghe/utils/silu.py:424": ("linghe_amd.utils.silu", "triton_silu_and_block_quant_backward",
                                 ["g", "x", "round_scale"]),
    "linghe/utils/silu.py:797": ("linghe_amd.utils.silu", "triton_batch_weighted_silu_and_block_quant_forward",
                                 ["x", "weight", "counts", "splits", "out", "scale", "round_scale", "output_mode"]),
    "linghe/utils/silu.py:1293": ("linghe_amd.utils.silu", "triton_batch_weighted_silu_and_block_quant_backward",
                                  ["g", "x", "weight", "counts", "splits", "round_scale"]),
    "linghe/quant/block.py:129": ("linghe_amd.quant.block", "triton_blockwise_quant",
                                  ["x", "round_scale", "output_mode"]),
    "linghe/quant/block.py:251": ("linghe_amd.quant.block", "triton_batch_blockwise_quant",
                                  ["xs", "token_count_per_expert", "splits", "round_scale"]),
    "linghe/quant/group.py:40": ("linghe_amd.quant.group", "triton_group_quant",
                                 ["x", "dtype", "group_size", "round_scale"]),
    "linghe/quant/block.py:32": ("linghe_amd.quant.block", "triton_block_quant",
                                 ["x", "block_size", "round_scale"]),
    "linghe/utils/silu.py:98": ("linghe_amd.utils.silu", "triton_weighted_silu_forward",
                                ["x", "weight", "out", "asm"]),
    "linghe/utils/silu.py:177": ("linghe_amd.utils.silu", "triton_weighted_silu_backward",
                                 ["g", "x", "weight"]),
    "linghe/utils/gather.py:960": ("linghe_amd.utils.gather", "triton_batch_block_pad_permute_with_indices",
                                   ["xs", "token_count_per_expert", "indices", "splits", "probs", "round_scale"]),
    "linghe/utils/norm.py:690": ("linghe_amd.utils.norm", "triton_rms_norm_fp32_gemm_block_quant_forward",
                                 ["x", "norm_weight", "route_weight", "rms", "eps", "output_mode", "round_scale"]),
}


@pytest.mark.parametrize("ref", sorted(REFERENCE_SIGNATURES))
def test_entry_points_keep_reference_signatures(ref):
    import importlib

    mod, fn, params = REFERENCE_SIGNATURES[ref]
    f = getattr(importlib.import_module(mod), fn)
    sig = inspect.signature(f)
    positional = [p.name for p in sig.parameters.values() if p.kind == p.POSITIONAL_OR_KEYWORD]
    assert positional == params, (ref, positional)
    extras = [p.name for p in sig.parameters.values() if p.kind == p.KEYWORD_ONLY]
    # additions are keyword-only: the FP8 format, the caller-packed router weight, and the per-expert tile plan
    assert set(extras) <= {"fp8_dtype", "packed_route_weight", "plan"}


def test_host_asserts_fire_on_cpu_tensors():
    """Reference assert conditions are checked in Python before the library is
    called, and CPU tensors are refused (there is no CPU path)."""
    import torch

    from linghe_amd.quant.block import triton_blockwise_quant
    from linghe_amd.utils.silu import (triton_batch_weighted_silu_and_block_quant_forward,
                                       triton_silu_and_block_quant_backward)

    x = torch.zeros(32, 256, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="GPU"):
        triton_blockwise_quant(x)
    with pytest.raises(AssertionError):
        triton_blockwise_quant(torch.zeros(17, 256, dtype=torch.bfloat16))  # M % 16
    with pytest.raises(AssertionError):
        triton_blockwise_quant(x.t())  # not contiguous
    with pytest.raises(AssertionError):
        from linghe_amd.quant.block import triton_block_quant
        triton_block_quant(torch.zeros(100, 256, dtype=torch.bfloat16))  # M % 128
    with pytest.raises(AssertionError, match="splits"):
        triton_batch_weighted_silu_and_block_quant_forward(x, torch.zeros(32, 1), torch.zeros(2, dtype=torch.int32))
    with pytest.raises(AssertionError):
        # M % 128 != 0 for the single-matrix backward
        triton_silu_and_block_quant_backward(torch.zeros(32, 128, dtype=torch.bfloat16).cuda()
                                             if torch.cuda.is_available() else
                                             torch.zeros(32, 128, dtype=torch.bfloat16), x)


def test_facade_contract_helpers():
    """The caller contract the autograd classes share (reference linghe/facade/norm.py:55-60,
    facade/silu.py:43-65): recompute flag -> output mode, and the quantizer's dtype tag ->
    the FP8 format the kernels are asked for."""
    import torch

    from linghe_amd.facade._qtensor import Codes, Folded, kernel_fp8_dtype, output_mode

    assert [output_mode(v) for v in (None, False, True)] == [2, 0, 1]
    assert kernel_fp8_dtype(torch.float8_e5m2) is torch.float8_e5m2
    assert kernel_fp8_dtype(torch.float8_e4m3fn) is torch.float8_e4m3fn

    class Tag:
        def __init__(self, name):
            self.name = name

    assert kernel_fp8_dtype(Tag("kFloat8E5M2")) is torch.float8_e5m2
    assert kernel_fp8_dtype(Tag("kFloat8E4M3")) is torch.float8_e4m3fn
    with pytest.raises(TypeError):
        kernel_fp8_dtype(torch.bfloat16)
    with pytest.raises(TypeError):
        kernel_fp8_dtype(Tag("kInt8"))
    act = Folded(torch.zeros(6, 5, 256))
    assert act.rows == 30 and act.matrix(torch.zeros(6, 5, 128)).shape == (30, 128)
    codes = act.unfold(Codes(torch.zeros(30, 128), None, torch.zeros(128, 30), None), 128)
    assert codes.row.shape == (6, 5, 128) and codes.col.shape == (128, 6, 5) and codes.row_scale is None
    none = act.unfold(Codes(None, None, None, None), 128)
    assert none.row is None and none.col is None


def test_expert_plan_shape_on_host():
    """fq_expert_plan_shape is host arithmetic on the caller's copy of the counts: row blocks in
    all, and how many are worked on whole, in halves (a last block of 33..64 rows) and in quarters
    (at most 32 rows).  The planned entry points refuse anything that is not such a shape."""
    from linghe_amd import _lib

    L = _lib.lib
    cases = {
        (): [0, 0, 0, 0],
        (0, 0): [0, 0, 0, 0],
        (128,): [1, 1, 0, 0],
        (129,): [2, 1, 0, 1],
        (32, 33, 64, 65): [4, 1, 2, 1],
        # 128+128+44 | - | 1 | 127 | 128+64 | 106*128+49
        (300, 0, 1, 127, 192, 13617): [3 + 1 + 1 + 2 + 107, 2 + 1 + 1 + 106, 3, 1],
    }
    for counts, want in cases.items():
        host = (ctypes.c_int64 * max(len(counts), 1))(*counts)
        shape = (ctypes.c_int64 * 5)(-1, -1, -1, -1, -1)
        assert L.fq_expert_plan_shape(host, len(counts), 1, shape) == 0
        assert list(shape) == want + [1], (counts, list(shape))
        assert L.fq_expert_plan_bytes(shape) == 20 * want[0]
    # the padded layout of gather + pad + quant classes a last block by its rows rounded up to 16
    host = (ctypes.c_int64 * 4)(32, 33, 64, 65)
    assert L.fq_expert_plan_shape(host, 4, 16, shape) == 0 and list(shape) == [4, 1, 2, 1, 16]
    host = (ctypes.c_int64 * 3)(17, 49, 129)   # 32 | 64 | 128 + 16
    assert L.fq_expert_plan_shape(host, 3, 16, shape) == 0 and list(shape) == [4, 1, 1, 2, 16]
    assert L.fq_expert_plan_shape(host, 3, 8, shape) == -1
    assert L.fq_expert_plan_shape(None, 3, 1, shape) == -1
    bad = (ctypes.c_int64 * 5)(5, 1, 1, 1, 1)  # the parts do not add up
    rc = L.fq_batched_blockwise_quant_planned(None, ctypes.c_void_p(256), bad, None, None, None, None, 640, 128, 0, 0,
                                              None)
    assert rc == -2 and b"plan shape" in L.fq_last_error()
    assert L.fq_build_expert_plan(None, 0, 4, bad, ctypes.c_void_p(256), None) == -2
    good = (ctypes.c_int64 * 5)(3, 1, 1, 1, 1)
    # more row blocks than rows
    rc = L.fq_batched_swiglu_quant_fwd_planned(ctypes.c_void_p(256), ctypes.c_void_p(256), 0, ctypes.c_void_p(256),
                                               good, ctypes.c_void_p(256), ctypes.c_void_p(256), ctypes.c_void_p(256),
                                               ctypes.c_void_p(256), 2, 128, 0, 2, 0, None)
    assert rc == -2 and b"inconsistent" in L.fq_last_error()
    # no plan
    rc = L.fq_batched_swiglu_quant_bwd_planned(ctypes.c_void_p(256), ctypes.c_void_p(256), ctypes.c_void_p(256), 0,
                                               None, good, ctypes.c_void_p(256), ctypes.c_void_p(256),
                                               ctypes.c_void_p(256), ctypes.c_void_p(256), ctypes.c_void_p(256),
                                               ctypes.c_void_p(256), 640, 128, 0, 0, None)
    assert rc == -1 and b"plan NULL" in L.fq_last_error()
    # a plan of the back-to-back layout handed to gather + pad + quant
    rc = L.fq_batched_pad_permute_quant_planned(None, ctypes.c_void_p(256), good, 4, None, None, 0, None, None, None,
                                                None, None, 64, 64, 256, 0, 0, None)
    assert rc == -2 and b"padded" in L.fq_last_error()
