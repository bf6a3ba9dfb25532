#!/usr/bin/env python3
"""Benchmark of the fused blockwise-FP8 quantisation path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--repeats R] [--configs all|cfg1,cfg2,...] [--no-cpu]

A "step" is one call of the entry point of a configuration on one batch of
synthetic (seeded) input that is already resident in HBM.  Calls go through
the C ABI with preallocated outputs; K steps are timed between two events on
the launch stream (HIP events without the system-scope fence), R times over,
and the median loop is reported (with the fastest and slowest); every timed
loop follows, in the stream, untimed calls of the same entry point that keep
the device busy for --settle-us (1.5 ms) first.  Buffers rotate over enough copies to exceed twice the
256 MB Infinity Cache, so the figure is an HBM figure ("cold"); the same loop
on one fixed set of buffers gives the cache-resident ("hot") figure.

Beside each configuration: the time a kernel that does no work needs to read
and write the configuration's algorithmic byte counts (`stream_us`, the
measured ceiling of this device for those bytes), the HBM traffic per call
measured with the profiler's counters (from profiles/hbm_traffic_per_config.md)
and the torch CPU oracle timed on the host cores.

Prints ONE short JSON line on stdout (under 4000 characters): the headline
metric is us/call of RMSNorm + 1x128 quant forward on bf16 [8192, 2048]
(output_mode 2) with its roofline and CPU baseline; the other configurations
appear as name -> [us, fraction of peak, fraction of the no-work kernel's rate].
Every field of every configuration goes to bench_full.json in the results folder
(RESULTS_DIR); stderr
carries one summary line per configuration.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
INFINITY_CACHE_BYTES = 256 << 20
FP8 = torch.float8_e4m3fn


def _p(t):
    return None if t is None else t.data_ptr()


class Case:
    """One configuration: `sets` buffer sets and a launcher taking a set index."""

    def __init__(self, name, entry, shape, rw_bytes, make_set, launch, cpu_fn):
        self.name, self.entry, self.shape = name, entry, shape
        self.read_bytes, self.write_bytes = rw_bytes          # algorithmic bytes read / written per call
        self.algo_bytes = self.read_bytes + self.write_bytes
        self.make_set, self.launch, self.cpu_fn = make_set, launch, cpu_fn
        self.sets = []

    def allocate(self):
        n_sets = max(2, min(16, (2 * INFINITY_CACHE_BYTES + 64 * (1 << 20)) // max(1, self.algo_bytes) + 1))
        self.sets = [self.make_set() for _ in range(n_sets)]


def build_cases(names, dev):
    from linghe_amd import _lib, configs
    L = _lib.lib
    stream = torch.cuda.current_stream(dev).cuda_stream
    cases = {}

    def add(name, **kw):
        if names is None or name in names:
            cases[name] = kw

    # ---------------------------------------------------------------- cfg1 / cfg5b / cfg5c
    def rms_quant_case(name, data, mode, pow2=False):
        x_cpu, g_cpu, eps = data["x"], data["gamma"], data["eps"]
        M, n = x_cpu.shape
        gd = g_cpu.to(dev)
        rstd_saved = None
        if mode == 1:
            from linghe_amd.utils.norm import triton_rms_norm_forward
            _, rstd_saved = triton_rms_norm_forward(x_cpu.to(dev), gd, eps)

        def make_set():
            s = dict(x=x_cpu.to(dev))
            if mode != 1:
                s["q"] = torch.empty((M, n), device=dev, dtype=FP8)
                s["s"] = torch.empty((n // 128, M), device=dev, dtype=torch.float32)
                s["rstd"] = torch.empty((M,), device=dev, dtype=torch.float32)
            else:
                s["q"], s["s"], s["rstd"] = None, None, rstd_saved.clone()
            if mode != 0:
                s["qt"] = torch.empty((n, M), device=dev, dtype=FP8)
                s["st"] = torch.empty(((M + 127) // 128, n), device=dev, dtype=torch.float32)
            else:
                s["qt"], s["st"] = None, None
            s["args"] = (_p(s["x"]), _p(gd), _p(s["q"]), _p(s["s"]), _p(s["rstd"]), _p(s["qt"]), _p(s["st"]),
                         M, n, float(eps), int(pow2), mode, _lib.FQ_E4M3, stream)
            return s

        def launch(s):
            _lib.check(L.fq_rmsnorm_quant_fwd(*s["args"]))

        def cpu_fn():
            from oracle import fq_oracle as O
            return O.rms_norm_and_block_quant_forward(x_cpu, g_cpu, eps, pow2)

        label = "triton_rms_norm_and_block_quant_forward(output_mode=%d)" % mode
        if mode == 2:
            label += " two passes"
        if pow2:
            label += ", round_scale=True"
        return Case(name, label, [M, n],
                    configs.rw_rmsnorm_quant(M, n, mode), make_set, launch, cpu_fn)

    lazy = {}

    def cfg5():
        if "cfg5" not in lazy:
            lazy["cfg5"] = configs.cfg5_rmsnorm_large()
        return lazy["cfg5"]

    add("cfg1", build=lambda: rms_quant_case("cfg1", configs.cfg1_rmsnorm_quant(), 2))
    # the same with power-of-two scales: what the autograd callers request when the
    # quantizer's recipe sets force_pow_2_scales (linghe/facade/norm.py:62-69)
    add("cfg1_pow2", build=lambda: rms_quant_case("cfg1_pow2", configs.cfg1_rmsnorm_quant(), 2, True))
    add("cfg5b", build=lambda: rms_quant_case("cfg5b", cfg5(), 2))
    add("cfg5c", build=lambda: rms_quant_case("cfg5c", cfg5(), 1))
    add("cfg5b_pow2", build=lambda: rms_quant_case("cfg5b_pow2", cfg5(), 2, True))
    # output_mode 0 (row-wise codes only: the first forward of a layer that will be recomputed)
    add("cfg1_mode0", build=lambda: rms_quant_case("cfg1_mode0", configs.cfg1_rmsnorm_quant(), 0))
    add("cfg5_mode0", build=lambda: rms_quant_case("cfg5_mode0", cfg5(), 0))
    # output_mode 1 at cfg1's size (cfg5c is the same at cfg5's): the recomputed forward
    add("cfg1_mode1", build=lambda: rms_quant_case("cfg1_mode1", configs.cfg1_rmsnorm_quant(), 1))

    # ---------------------------------------------------------------- bf16 RMSNorm forward (a2)
    def rms_fwd_case():
        d = cfg5()
        x_cpu, g_cpu, eps = d["x"], d["gamma"], d["eps"]
        M, n = x_cpu.shape
        gd = g_cpu.to(dev)

        def make_set():
            s = dict(x=x_cpu.to(dev), y=torch.empty((M, n), device=dev, dtype=torch.bfloat16),
                     r=torch.empty((M,), device=dev, dtype=torch.float32))
            s["args"] = (_p(s["x"]), _p(gd), _p(s["y"]), _p(s["r"]), M, n, float(eps), 0, stream)
            return s

        def launch(s):
            _lib.check(L.fq_rmsnorm_fwd(*s["args"]))

        def cpu_fn():
            from oracle import fq_oracle as O
            return O.rms_norm_forward(x_cpu, g_cpu, eps)

        return Case("a2_rmsnorm_fwd", "triton_rms_norm_forward", [M, n], (2 * M * n + 2 * n, 2 * M * n + 4 * M),
                    make_set, launch, cpu_fn)

    add("a2_rmsnorm_fwd", build=rms_fwd_case)

    # ---------------------------------------------------------------- cfg2
    def swiglu_fwd_case(name="cfg2", pow2=False, mode=2):
        x_cpu = configs.cfg2_swiglu_fwd()["x"]
        M, N = x_cpu.shape
        n = N // 2

        def make_set():
            s = dict(x=x_cpu.to(dev), q=None, s=None, qt=None, st=None)
            if mode != 1:
                s["q"] = torch.empty((M, n), device=dev, dtype=FP8)
                s["s"] = torch.empty((n // 128, M), device=dev, dtype=torch.float32)
            if mode != 0:
                s["qt"] = torch.empty((n, M), device=dev, dtype=FP8)
                s["st"] = torch.empty(((M + 127) // 128, n), device=dev, dtype=torch.float32)
            s["args"] = (_p(s["x"]), _p(s["q"]), _p(s["s"]), _p(s["qt"]), _p(s["st"]), M, n, int(pow2), mode,
                         _lib.FQ_E4M3, stream)
            return s

        def launch(s):
            _lib.check(L.fq_swiglu_quant_fwd(*s["args"]))

        def cpu_fn():
            from oracle import fq_oracle as O
            return O.silu_and_block_quant_forward(x_cpu, pow2)

        return Case(name, "triton_silu_and_block_quant_forward(output_mode=%d%s)" % (mode, ", round_scale=True" if pow2 else ""),
                    [M, N],
                    configs.rw_swiglu_fwd(M, n, mode), make_set, launch, cpu_fn)

    add("cfg2", build=swiglu_fwd_case)
    add("cfg2_pow2", build=lambda: swiglu_fwd_case("cfg2_pow2", True))
    # one layout only: what a recomputed layer asks for (row-wise in the forward, transposed in the recomputation)
    add("cfg2_mode0", build=lambda: swiglu_fwd_case("cfg2_mode0", False, 0))
    add("cfg2_mode1", build=lambda: swiglu_fwd_case("cfg2_mode1", False, 1))

    # ---------------------------------------------------------------- cfg3 (+ backward)
    def expert_plan(cnt, counts, pad=1):
        """the per-expert tile plan of a set of counts (table, shape), built once outside the timed region"""
        import ctypes
        host = (ctypes.c_int64 * len(counts))(*counts)
        shape = (ctypes.c_int64 * 5)()
        _lib.check(L.fq_expert_plan_shape(host, len(counts), pad, shape))
        table = torch.empty((max(int(L.fq_expert_plan_bytes(shape)), 16),), device=dev, dtype=torch.uint8)
        _lib.check(L.fq_build_expert_plan(_p(cnt), 0, len(counts), shape, _p(table), stream))
        return table, shape

    def batched_case(backward, planned=False):
        d = lazy.setdefault("cfg3", configs.cfg3_batched_swiglu())
        x_cpu, w_cpu, counts, dy_cpu = d["x"], d["weight"], d["counts"], d["dy"]
        M, N = x_cpu.shape
        n = N // 2
        E = len(counts)
        blocks = sum((c + 127) // 128 for c in counts)
        cnt = torch.tensor(counts, dtype=torch.int32, device=dev)
        plan, pshape = expert_plan(cnt, counts) if planned else (None, None)
        W = N if backward else n

        def make_set():
            s = dict(x=x_cpu.to(dev), w=w_cpu.to(dev), q=torch.empty((M, W), device=dev, dtype=FP8),
                     s=torch.empty((M, W // 128), device=dev, dtype=torch.float32),
                     qt=torch.empty((M, W), device=dev, dtype=FP8),
                     st=torch.empty((blocks, W), device=dev, dtype=torch.float32))
            if backward:
                s["dy"] = dy_cpu.to(dev)
                s["dw"] = torch.empty((M, 1), device=dev, dtype=torch.float32)
                s["dws"] = torch.empty((M, n // 128), device=dev, dtype=torch.float32)
                src = (_p(plan), pshape) if planned else (_p(cnt), 0, E, blocks)
                s["args"] = (_p(s["dy"]), _p(s["x"]), _p(s["w"]), 0) + src + (
                    _p(s["q"]), _p(s["s"]), _p(s["dw"]), _p(s["qt"]), _p(s["st"]), _p(s["dws"]), M, n, 0,
                    _lib.FQ_E4M3, stream)
            else:
                src = (_p(plan), pshape) if planned else (_p(cnt), 0, E, blocks)
                s["args"] = (_p(s["x"]), _p(s["w"]), 0) + src + (
                    _p(s["q"]), _p(s["s"]), _p(s["qt"]), _p(s["st"]), M, n, 0, 2, _lib.FQ_E4M3, stream)
            return s

        if backward:
            bwd_fn = L.fq_batched_swiglu_quant_bwd_planned if planned else L.fq_batched_swiglu_quant_bwd

            def launch(s):
                _lib.check(bwd_fn(*s["args"]))

            def cpu_fn():
                from oracle import fq_oracle as O
                return O.batch_weighted_silu_and_block_quant_backward(dy_cpu, x_cpu, w_cpu, counts, False)
            nbytes = configs.rw_batched_swiglu_bwd(M, n, counts)
            entry = "triton_batch_weighted_silu_and_block_quant_backward"
        else:
            fwd_fn = L.fq_batched_swiglu_quant_fwd_planned if planned else L.fq_batched_swiglu_quant_fwd

            def launch(s):
                _lib.check(fwd_fn(*s["args"]))

            def cpu_fn():
                from oracle import fq_oracle as O
                return O.batch_weighted_silu_and_block_quant_forward(x_cpu, w_cpu, counts, False)
            nbytes = configs.rw_batched_swiglu_fwd(M, n, counts)
            entry = "triton_batch_weighted_silu_and_block_quant_forward(output_mode=2)"
        if planned:
            entry += " with plan="
        c = Case(("cfg3b" if backward else "cfg3") + ("_planned" if planned else ""), entry, [M, N], nbytes,
                 make_set, launch, cpu_fn)
        c.extra = dict(n_experts=E, blocks=blocks, empty_experts=sum(1 for v in counts if v == 0),
                       max_count=max(counts))
        return c

    add("cfg3", build=lambda: batched_case(False))
    add("cfg3b", build=lambda: batched_case(True))
    # the same with every workgroup's tile read from a plan built once from the counts
    add("cfg3_planned", build=lambda: batched_case(False, True))
    add("cfg3b_planned", build=lambda: batched_case(True, True))

    # ---------------------------------------------------------------- cfg4
    def swiglu_bwd_case(kind, name, pow2=False):
        d = lazy.setdefault("cfg4", configs.cfg4_swiglu_bwd())
        dy_cpu, x_cpu = d["dy"], d["x"]
        M, N = x_cpu.shape
        n = N // 2
        dt = FP8 if kind == _lib.FQ_E4M3 else torch.float8_e5m2

        def make_set():
            s = dict(dy=dy_cpu.to(dev), x=x_cpu.to(dev), q=torch.empty((M, N), device=dev, dtype=dt),
                     s=torch.empty((N // 128, M), device=dev, dtype=torch.float32),
                     qt=torch.empty((N, M), device=dev, dtype=dt),
                     st=torch.empty((M // 128, N), device=dev, dtype=torch.float32))
            s["args"] = (_p(s["dy"]), _p(s["x"]), _p(s["q"]), _p(s["s"]), _p(s["qt"]), _p(s["st"]), M, n, int(pow2),
                         kind, stream)
            return s

        def launch(s):
            _lib.check(L.fq_swiglu_quant_bwd(*s["args"]))

        def cpu_fn():
            from oracle import fq_oracle as O
            return O.silu_and_block_quant_backward(dy_cpu, x_cpu, pow2, dt)

        return Case(name, "triton_silu_and_block_quant_backward(fp8=%s%s)" % (str(dt).split(".")[-1],
                                                                               ", round_scale=True" if pow2 else ""),
                    [M, N],
                    configs.rw_swiglu_bwd(M, n), make_set, launch, cpu_fn)

    add("cfg4", build=lambda: swiglu_bwd_case(_lib.FQ_E4M3, "cfg4"))
    add("cfg4_e5m2", build=lambda: swiglu_bwd_case(_lib.FQ_E5M2, "cfg4_e5m2"))
    add("cfg4_pow2", build=lambda: swiglu_bwd_case(_lib.FQ_E4M3, "cfg4_pow2", True))

    # ---------------------------------------------------------------- cfg5a
    def rms_bwd_case():
        d = cfg5()
        x_cpu, g_cpu, dy_cpu, eps = d["x"], d["gamma"], d["dy"], d["eps"]
        M, n = x_cpu.shape
        gd = g_cpu.to(dev)
        n_part = int(L.fq_rmsnorm_bwd_num_partials(M, n))

        def make_set():
            s = dict(x=x_cpu.to(dev), dy=dy_cpu.to(dev), dx=torch.empty((M, n), device=dev, dtype=torch.bfloat16),
                     dg=torch.empty((n,), device=dev, dtype=torch.float32),
                     part=torch.empty((n_part, n), device=dev, dtype=torch.float32))
            s["args"] = (_p(s["dy"]), _p(s["x"]), _p(gd), None, _p(s["dx"]), _p(s["dg"]), _p(s["part"]), n_part, M, n,
                         float(eps), stream)
            return s

        def launch(s):
            _lib.check(L.fq_rmsnorm_bwd(*s["args"]))

        def cpu_fn():
            from oracle import fq_oracle as O
            return O.rms_norm_backward(x_cpu, g_cpu, dy_cpu, eps)

        return Case("cfg5a", "triton_rms_norm_backward", [M, n], configs.rw_rmsnorm_bwd(M, n), make_set, launch,
                    cpu_fn)

    add("cfg5a", build=rms_bwd_case)

    # ---------------------------------------------------------------- next row: gather + pad + quant
    def permute_case(planned=False):
        d = lazy.setdefault("permute", configs.next_permute_pad_quant())
        x_cpu, probs_cpu, counts, idx_cpu = d["x"], d["probs"], d["counts"], d["indices"]
        m, N = x_cpu.shape
        M = idx_cpu.numel()
        E = len(counts)
        blocks = sum((c + 127) // 128 for c in counts)
        cnt = torch.tensor(counts, dtype=torch.int32, device=dev)
        idx = idx_cpu.to(dev)
        plan, pshape = expert_plan(cnt, counts, 16) if planned else (None, None)

        def make_set():
            s = dict(x=x_cpu.to(dev), probs=probs_cpu.to(dev), q=torch.empty((M, N), device=dev, dtype=FP8),
                     s=torch.empty((M, N // 128), device=dev, dtype=torch.float32),
                     qt=torch.empty((M, N), device=dev, dtype=FP8),
                     st=torch.empty((blocks, N), device=dev, dtype=torch.float32),
                     p=torch.empty((M,), device=dev, dtype=torch.float32))
            src = (_p(plan), pshape, E) if planned else (_p(cnt), 0, E, blocks)
            s["args"] = (_p(s["x"]),) + src + (_p(idx), _p(s["probs"]), 0, _p(s["p"]), _p(s["q"]), _p(s["s"]),
                                              _p(s["qt"]), _p(s["st"]), m, M, N, 0, _lib.FQ_E4M3, stream)
            return s

        fn = L.fq_batched_pad_permute_quant_planned if planned else L.fq_batched_pad_permute_quant

        def launch(s):
            _lib.check(fn(*s["args"]))

        def cpu_fn():
            from oracle import fq_oracle as O
            return O.batch_block_pad_permute_with_indices(x_cpu, d["indices_unpadded"], probs_cpu, counts, False)

        return Case("next_permute" + ("_planned" if planned else ""),
                    "triton_batch_block_pad_permute_with_indices" + (" with plan=" if planned else ""), [M, N],
                    configs.rw_permute_pad_quant(N, counts), make_set, launch, cpu_fn)

    add("next_permute", build=permute_case)
    add("next_permute_planned", build=lambda: permute_case(True))

    # ---------------------------------------------------------------- next rows: bf16 SwiGLU, weight block quant
    def wsilu_case(backward):
        M, N = 8192, 4096  # x [M, N] = gate | up
        g = torch.Generator().manual_seed(1102)
        x_cpu = torch.randn(M, N, generator=g).to(torch.bfloat16)
        w_cpu = torch.rand(M, 1, generator=g)
        dy_cpu = torch.randn(M, N // 2, generator=g).to(torch.bfloat16)

        def make_set():
            s = dict(x=x_cpu.to(dev), w=w_cpu.to(dev))
            if backward:
                s.update(dy=dy_cpu.to(dev), dx=torch.empty((M, N), device=dev, dtype=torch.bfloat16),
                         dw=torch.empty((M, 1), device=dev, dtype=torch.float32))
                s["args"] = (_p(s["dy"]), _p(s["x"]), _p(s["w"]), 0, _p(s["dx"]), _p(s["dw"]), M, N // 2, stream)
            else:
                s["y"] = torch.empty((M, N // 2), device=dev, dtype=torch.bfloat16)
                s["args"] = (_p(s["x"]), _p(s["w"]), 0, _p(s["y"]), M, N // 2, stream)
            return s

        def launch(s):
            _lib.check((L.fq_swiglu_bwd if backward else L.fq_swiglu_fwd)(*s["args"]))

        def cpu_fn():
            from oracle import fq_oracle as O
            return O.weighted_silu_backward(dy_cpu, x_cpu, w_cpu) if backward else O.weighted_silu_forward(x_cpu, w_cpu)

        nbytes = configs.rw_weighted_silu(M, N // 2, backward)
        return Case("next_wsilu_bwd" if backward else "next_wsilu_fwd",
                    "triton_weighted_silu_backward" if backward else "triton_weighted_silu_forward", [M, N], nbytes,
                    make_set, launch, cpu_fn)

    add("next_wsilu_fwd", build=lambda: wsilu_case(False))
    add("next_wsilu_bwd", build=lambda: wsilu_case(True))

    def block_quant_case():
        M, N = 8192, 4096
        g = torch.Generator().manual_seed(1103)
        x_cpu = (torch.randn(M, N, generator=g) ** 3).to(torch.bfloat16)

        def make_set():
            s = dict(x=x_cpu.to(dev), q=torch.empty((M, N), device=dev, dtype=FP8),
                     s=torch.empty((M // 128, N // 128), device=dev, dtype=torch.float32))
            s["args"] = (_p(s["x"]), _p(s["q"]), _p(s["s"]), M, N, 1, _lib.FQ_E4M3, stream)
            return s

        def launch(s):
            _lib.check(L.fq_block_quant(*s["args"]))

        def cpu_fn():
            from oracle import fq_oracle as O
            return O.block_quant_128(x_cpu, True)

        return Case("next_block_quant", "triton_block_quant(round_scale=True)", [M, N],
                    configs.rw_block_quant(M, N), make_set, launch, cpu_fn)

    add("next_block_quant", build=block_quant_case)

    # ---------------------------------------------------------------- the quantisers with no fused pre-op
    def plain_quant_case(name):
        g = torch.Generator().manual_seed(1105)
        planned = name == "a8_batch_blockwise_planned"
        if planned:
            name = "a8_batch_blockwise"
        if name == "a8_batch_blockwise":  # the activations of cfg3's experts: 65536 x 512, same Zipf counts
            d = lazy.setdefault("cfg3", configs.cfg3_batched_swiglu())
            counts = d["counts"]
            M, N = sum(counts), 512
        else:
            counts = None
            M, N = 8192, 2048
        x_cpu = torch.randn(M, N, generator=g).to(torch.bfloat16)
        blocks = sum((c + 127) // 128 for c in counts) if counts else (M + 127) // 128
        cnt = torch.tensor(counts, dtype=torch.int32, device=dev) if counts else None
        plan, pshape = expert_plan(cnt, counts) if planned else (None, None)

        def make_set():
            s = dict(x=x_cpu.to(dev), q=torch.empty((M, N), device=dev, dtype=FP8),
                     s=torch.empty((M * (N // 128),), device=dev, dtype=torch.float32))
            if name != "a8_group":
                s["qt"] = torch.empty((M * N,), device=dev, dtype=FP8)
                s["st"] = torch.empty((blocks * N,), device=dev, dtype=torch.float32)
            if name == "a8_blockwise":
                s["args"] = (_p(s["x"]), _p(s["q"]), _p(s["s"]), _p(s["qt"]), _p(s["st"]), M, N, 0, 2, _lib.FQ_E4M3,
                             stream)
            elif name == "a8_group":
                s["args"] = (_p(s["x"]), _p(s["q"]), _p(s["s"]), M, N, 0, _lib.FQ_E4M3, stream)
            elif planned:
                s["args"] = (_p(s["x"]), _p(plan), pshape, _p(s["q"]), _p(s["s"]), _p(s["qt"]), _p(s["st"]), M, N, 0,
                             _lib.FQ_E4M3, stream)
            else:
                s["args"] = (_p(s["x"]), _p(cnt), 0, len(counts), blocks, _p(s["q"]), _p(s["s"]), _p(s["qt"]),
                             _p(s["st"]), M, N, 0, _lib.FQ_E4M3, stream)
            return s

        fn = {"a8_blockwise": L.fq_blockwise_quant, "a8_group": L.fq_group_quant,
              "a8_batch_blockwise": L.fq_batched_blockwise_quant_planned if planned
              else L.fq_batched_blockwise_quant}[name]

        def launch(s):
            _lib.check(fn(*s["args"]))

        def cpu_fn():
            from oracle import fq_oracle as O
            if name == "a8_blockwise":
                return O.blockwise_quant(x_cpu, False)
            if name == "a8_group":
                return O.group_quant_1x128(x_cpu, False)
            return O.batch_blockwise_quant(x_cpu, counts, False)

        row = M * N + 4 * M * (N // 128)
        col = M * N + 4 * blocks * N
        entry = {"a8_blockwise": "triton_blockwise_quant(output_mode=2)", "a8_group": "triton_group_quant",
                 "a8_batch_blockwise": "triton_batch_blockwise_quant"}[name]
        c = Case(name + ("_planned" if planned else ""), entry + (" with plan=" if planned else ""), [M, N],
                 (2 * M * N, row + (0 if name == "a8_group" else col)), make_set, launch, cpu_fn)
        return c

    for _n in ("a8_blockwise", "a8_group", "a8_batch_blockwise", "a8_batch_blockwise_planned"):
        add(_n, build=lambda _n=_n: plain_quant_case(_n))

    # ---------------------------------------------------------------- next row: RMSNorm + router GEMM + quant
    def router_case(packed=False, shape=(8192, 256, 2048), name=None):
        M, N, K = shape
        g = torch.Generator().manual_seed(1104)
        x_cpu = (torch.randn(M, K, generator=g) ** 2).to(torch.bfloat16)
        nw_cpu = torch.randn(K, generator=g).to(torch.bfloat16)
        rw_cpu = torch.randn(N, K, generator=g).to(torch.bfloat16)
        nwd, rwd = nw_cpu.to(dev), rw_cpu.to(dev)

        def make_set():
            s = dict(x=x_cpu.to(dev), y=torch.empty((M, K), device=dev, dtype=torch.bfloat16),
                     r=torch.empty((M,), device=dev, dtype=torch.float32),
                     lg=torch.empty((M, N), device=dev, dtype=torch.float32),
                     q=torch.empty((M, K), device=dev, dtype=FP8),
                     s=torch.empty((K // 128, M), device=dev, dtype=torch.float32))
            s["ws"] = torch.empty_like(rwd)
            if packed:  # the weight re-ordered once, outside the timed calls
                _lib.check(L.fq_pack_router_weight(_p(rwd), 0, _p(s["ws"]), K, N, stream))
                s["args"] = (_p(s["x"]), _p(nwd), _p(s["ws"]), 0, _p(s["y"]), _p(s["r"]), _p(s["lg"]), _p(s["q"]),
                             _p(s["s"]), M, K, N, 1e-6, 0, _lib.FQ_E4M3, stream)
            else:
                s["args"] = (_p(s["x"]), _p(nwd), _p(rwd), 0, _p(s["ws"]), _p(s["y"]), _p(s["r"]), _p(s["lg"]),
                             _p(s["q"]), _p(s["s"]), M, K, N, 1e-6, 0, _lib.FQ_E4M3, stream)
            return s

        def launch(s):
            _lib.check((L.fq_rmsnorm_router_quant_fwd_packed if packed else L.fq_rmsnorm_router_quant_fwd)(*s["args"]))

        def cpu_fn():
            from oracle import fq_oracle as O
            return O.rms_gemm_block_quant_forward(x_cpu, nw_cpu, rw_cpu)

        c = Case(name or ("next_router_packed" if packed else "next_router"),
                 "triton_rms_norm_fp32_gemm_block_quant_forward(output_mode=0%s)"
                 % (", packed_route_weight=..." if packed else ""), [M, N, K],
                 configs.rw_router(M, N, K), make_set, launch, cpu_fn)
        c.extra = {"gemm_flops": 2 * M * N * K}
        return c

    add("next_router", build=router_case)
    add("next_router_packed", build=lambda: router_case(True))
    # a wide router: more than 512 logits run as one launch per 512 (virtual) columns, x re-read by each
    add("next_router_wide", build=lambda: router_case(False, (2048, 2048, 2048), "next_router_wide"))

    # ---------------------------------------------------------------- the per-expert tile plan of cfg3's counts
    def plan_case():
        import ctypes
        d = lazy.setdefault("cfg3", configs.cfg3_batched_swiglu())
        counts = d["counts"]
        cnt = torch.tensor(counts, dtype=torch.int32, device=dev)
        host = (ctypes.c_int64 * len(counts))(*counts)
        shape = (ctypes.c_int64 * 5)()
        _lib.check(L.fq_expert_plan_shape(host, len(counts), 1, shape))
        nbytes = int(L.fq_expert_plan_bytes(shape))

        def make_set():
            s = dict(plan=torch.empty((nbytes,), device=dev, dtype=torch.uint8))
            s["args"] = (_p(cnt), 0, len(counts), shape, _p(s["plan"]), stream)
            return s

        def launch(s):
            _lib.check(L.fq_build_expert_plan(*s["args"]))

        return Case("expert_plan", "fq_build_expert_plan (one launch per set of counts)", [len(counts)],
                    (4 * len(counts), nbytes), make_set, launch, None)

    add("expert_plan", build=plan_case)

    # ---------------------------------------------------------------- the no-work stream kernel on a known size
    # (the read / copy rates of the memory system, and the calibration of FETCH_SIZE / WRITE_SIZE)
    def stream_case(name, read_mib, write_mib):
        rb, wb = read_mib << 20, write_mib << 20
        sink = torch.zeros(16, device=dev, dtype=torch.uint8)

        def make_set():
            s = dict(src=torch.zeros(max(rb, 16), device=dev, dtype=torch.uint8),
                     dst=torch.empty(max(wb, 16), device=dev, dtype=torch.uint8))
            s["args"] = (_p(s["src"]), rb, _p(s["dst"]), wb, _p(sink), 0, stream)
            return s

        def launch(s):
            _lib.check(L.fq_stream_rw(*s["args"]))

        return Case(name, "fq_stream_rw: read %d MiB, write %d MiB, no arithmetic" % (read_mib, write_mib),
                    [rb, wb], (rb, wb), make_set, launch, None)

    add("stream_read", build=lambda: stream_case("stream_read", 256, 0))
    add("stream_copy", build=lambda: stream_case("stream_copy", 256, 256))
    return cases


class TimingEvents:
    """A pair of HIP events created with hipEventDisableSystemFence and recorded on the launch
    stream.  A default event performs a system-scope fence (cache write-back and invalidation)
    when it is recorded; HIP documents this flag for events that only measure time.  With default
    events every timed loop carries 25-85 us of fence work that is not the kernels' (a 20-call loop
    of the SwiGLU backward reads 37.2 us per call where the kernel trace of the same loop shows
    20 dispatches of 33.3-34.9 us back to back)."""
    _hip = None

    def __init__(self, stream):
        import ctypes
        if TimingEvents._hip is None:
            TimingEvents._hip = ctypes.CDLL("libamdhip64.so")
        self.c, self.hip, self.stream = ctypes, TimingEvents._hip, ctypes.c_void_p(stream)
        self.a, self.b = ctypes.c_void_p(), ctypes.c_void_p()
        for e in (self.a, self.b):
            self._ok(self.hip.hipEventCreateWithFlags(ctypes.byref(e), ctypes.c_uint(0x20000000)))

    def _ok(self, rc):
        if rc != 0:
            raise RuntimeError("HIP event call failed with error %d" % rc)

    def start(self):
        self._ok(self.hip.hipEventRecord(self.a, self.stream))

    def stop(self):
        self._ok(self.hip.hipEventRecord(self.b, self.stream))

    def elapsed_us(self):
        ms = self.c.c_float()
        self._ok(self.hip.hipEventSynchronize(self.b))
        self._ok(self.hip.hipEventElapsedTime(self.c.byref(ms), self.a, self.b))
        return ms.value * 1000.0

    def close(self):
        for e in (self.a, self.b):
            self.hip.hipEventDestroy(e)


SETTLE_US = 1500.0  # see time_loop; --settle-us 0 turns it off


def time_loop(launch, sets, steps, warmup, repeats, settle_us=None, idle_gap_s=0.0):
    """us per call, one figure per repeat: `steps` back-to-back launches between two
    events on the launch stream (the current torch stream), rotating over `sets`.

    Every repeat is: synchronize, pre-roll, start event, exactly `steps` calls, stop event,
    synchronize.  The pre-roll is untimed calls of the same entry point, enqueued right in
    front of the start event, enough of them to keep the device busy for `settle_us`: a loop
    that starts on a device that has been mostly idle runs at a lower rate for its first
    millisecond or so (20 calls of the SwiGLU backward read 36-39 us per call that way, 33.7-34.0
    behind a pre-roll of 30 calls or more, and 33.9 in loops of 100-300 calls with no pre-roll at
    all; the kernel trace of a slow loop shows the same 33-35 us dispatches, so the difference is
    not inside the kernels), so what a short loop measures from idle is the device waking up, not
    the steady state the path runs in."""
    k = len(sets)
    for i in range(warmup):
        launch(sets[i % k])
    ev = TimingEvents(torch.cuda.current_stream().cuda_stream)
    settle_us = SETTLE_US if settle_us is None else settle_us
    preroll = 0
    if settle_us > 0:
        torch.cuda.synchronize()
        ev.start()
        for i in range(8):
            launch(sets[i % k])
        ev.stop()
        torch.cuda.synchronize()
        preroll = max(warmup, min(2000, int(settle_us / max(ev.elapsed_us() / 8, 0.5)) + 1))
    out = []
    for _ in range(repeats):
        torch.cuda.synchronize()
        if idle_gap_s > 0:
            time.sleep(idle_gap_s)  # let the device go idle: the from-idle figure
        for i in range(preroll):
            launch(sets[i % k])
        ev.start()
        for i in range(steps):
            launch(sets[(preroll + i) % k])
        ev.stop()
        torch.cuda.synchronize()
        out.append(ev.elapsed_us() / steps)
    ev.close()
    time_loop.last_preroll = preroll
    return sorted(out)


def median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2] if len(xs) % 2 else 0.5 * (xs[len(xs) // 2 - 1] + xs[len(xs) // 2])


def time_single_calls(case, sets, calls, warmup):
    """(median, trimmed mean) in us of event pairs around single calls, the
    protocol of the reference's own harness (linghe/tools/benchmark.py:32-70:
    one event pair per call, sorted, max(1, n/100) dropped at either end).  The
    events' own cost is inside every sample, so these read a few us above the
    back-to-back figure."""
    k = len(sets)
    for i in range(warmup):
        case.launch(sets[i % k])
    torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(calls)]
    for i, (a, b) in enumerate(pairs):
        a.record()
        case.launch(sets[i % k])
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) * 1000.0 for a, b in pairs)
    clip = max(1, calls // 100)
    kept = t[clip:-clip] if 2 * clip < calls else t
    return t[len(t) // 2], sum(kept) / len(kept)


def time_cpu(case):
    """the oracle on the host cores: 1 warm-up, then the minimum of 3 runs (us)."""
    case.cpu_fn()
    runs = []
    for _ in range(3):
        t0 = time.perf_counter()
        case.cpu_fn()
        runs.append(time.perf_counter() - t0)
    return min(runs) * 1e6


# Variants of the no-work kernel the ceiling is taken over: (chunks per lane, workgroups, order, hint on
# loads, hint on stores); workgroups 0 = one step per workgroup.  The short list is what came out on top
# somewhere in the full sweep (`--stream-sweep`, table in profiles/stream_ceiling_sweep.md).
STREAM_VARIANTS = [
    (4, 16384, 0, 0, 0), (4, 16384, 0, 1, 1),            # the plain form, without and with the hints
    (8, 2048, 0, 1, 1), (8, 0, 0, 1, 1), (8, 0, 1, 1, 1), (8, 0, 0, 1, 0), (8, 2048, 1, 1, 0),
    (8, 2048, 0, 1, 0), (8, 0, 1, 1, 0),                 # the other two of the best four on a 2:1 read:write mix
    (4, 0, 0, 1, 0),                                     # the best on the SwiGLU backward's mix
    (4, 0, 0, 1, 1), (4, 512, 0, 1, 1), (16, 0, 0, 1, 1),
]


def _stream_sets(dev, rb, wb):
    n_sets = max(2, min(16, (2 * INFINITY_CACHE_BYTES + (64 << 20)) // max(1, rb + wb) + 1))
    return [(torch.zeros(max(rb, 16), device=dev, dtype=torch.uint8),
             torch.empty(max(wb, 16), device=dev, dtype=torch.uint8)) for _ in range(n_sets)]


def _time_stream_variant(variant, sets, sink, rb, wb, stream, steps, warmup, repeats):
    from linghe_amd import _lib
    cpl, wgs, order, ntl, nts = variant

    def launch(s):
        _lib.check(_lib.lib.fq_stream_rw_variant(s[0].data_ptr(), rb, s[1].data_ptr(), wb, sink.data_ptr(), cpl, wgs,
                                                 order, ntl, nts, stream))
    return median(time_loop(launch, sets, steps, warmup, repeats))


def stream_ceiling(case, dev, stream, steps, warmup, repeats):
    """(us, variant) for the no-work kernel to read and write this configuration's algorithmic byte
    counts, cold buffers: what the memory system alone takes for the same bytes.  The fastest of
    STREAM_VARIANTS."""
    rb, wb = (case.read_bytes + 15) // 16 * 16, (case.write_bytes + 15) // 16 * 16
    sink = torch.zeros(16, device=dev, dtype=torch.uint8)
    sets = _stream_sets(dev, rb, wb)
    best = None
    for v in STREAM_VARIANTS:
        t = _time_stream_variant(v, sets, sink, rb, wb, stream, steps, warmup, repeats)
        if best is None or t < best[0]:
            best = (t, v)
    return best


def stream_sweep(dev, stream, steps, warmup, repeats):
    """Every variant of the no-work kernel on the byte counts of cfg1, cfg2, cfg4 and cfg5a (read MB, write MB),
    cold buffers: a markdown table on stdout (the basis of STREAM_VARIANTS)."""
    from linghe_amd import configs
    sizes = [("cfg1", configs.rw_rmsnorm_quant(8192, 2048, 2)), ("cfg2", configs.rw_swiglu_fwd(8192, 2048, 2)),
             ("cfg4", configs.rw_swiglu_bwd(8192, 2048)), ("cfg5a", configs.rw_rmsnorm_bwd(16384, 7168))]
    variants = [(c, w, o, l, st) for c in (4, 8, 16) for w in (256, 512, 1024, 2048, 0) for o in (0, 1, 2)
                for l in (0, 1) for st in (0, 1)]
    # order 3: the access pattern of the tile kernels (steps are tiles of 256-byte row segments)
    variants += [(c, w, 3, l, st) for c in (4, 8, 16) for w in (2048, 0) for l in (0, 1) for st in (0, 1)]
    variants.insert(0, (4, 16384, 0, 0, 0))
    variants.insert(1, (4, 16384, 0, 1, 1))
    cols = {}
    for name, (rb, wb) in sizes:
        rb, wb = (rb + 15) // 16 * 16, (wb + 15) // 16 * 16
        sink = torch.zeros(16, device=dev, dtype=torch.uint8)
        sets = _stream_sets(dev, rb, wb)
        cols[name] = [_time_stream_variant(v, sets, sink, rb, wb, stream, steps, warmup, repeats) for v in variants]
        print("[sweep] %s done" % name, file=sys.stderr, flush=True)
        del sets
        torch.cuda.empty_cache()
    print("| chunks/lane | workgroups | order | nt loads | nt stores | " + " | ".join(
        "%s us (%.1f + %.1f MB)" % (n, r / 1e6, w / 1e6) for n, (r, w) in sizes) + " |")
    print("|---|---|---|---|---|" + "---|" * len(sizes))
    for i, v in enumerate(variants):
        print("| %d | %s | %d | %d | %d | " % (v[0], v[1] or "one step each", v[2], v[3], v[4])
              + " | ".join("%.2f" % cols[n][i] for n, _ in sizes) + " |")
    for n, (r, w) in sizes:
        best = min(range(len(variants)), key=lambda i: cols[n][i])
        print("best %s: %s %.2f us = %.0f GB/s (%.3f of 8 TB/s)" % (n, variants[best], cols[n][best],
                                                                  (r + w) / cols[n][best] / 1e3,
                                                                  (r + w) / cols[n][best] / 1e3 / HBM_PEAK_GBS))


def load_traffic_table():
    """Measured HBM bytes per call and configuration, from the tracked profiler summary
    (rows `| config | fetched MB | written MB | total MB |`): the digits printed here are
    the digits of that file.  Absent file or row -> None."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic_per_config.md")
    table = {}
    if os.path.exists(path):
        for line in open(path):
            cells = [c.strip() for c in line.strip().strip("|").split("|")]
            if len(cells) >= 4:
                try:
                    table[cells[0]] = dict(fetched=float(cells[1]) * 1e6, written=float(cells[2]) * 1e6,
                                           total=float(cells[3]) * 1e6)
                except ValueError:
                    pass
    return table


ALL = ["cfg1", "cfg2", "cfg3", "cfg3b", "cfg4", "cfg4_e5m2", "cfg5a", "cfg5b", "cfg5c",
       "cfg1_pow2", "cfg2_pow2", "cfg4_pow2", "cfg5b_pow2", "cfg1_mode0", "cfg5_mode0", "cfg1_mode1", "cfg2_mode0", "cfg2_mode1", "a2_rmsnorm_fwd", "a8_blockwise", "a8_group", "a8_batch_blockwise",
       "cfg3_planned", "cfg3b_planned", "a8_batch_blockwise_planned", "expert_plan",
       "next_permute", "next_permute_planned", "next_wsilu_fwd", "next_wsilu_bwd", "next_block_quant", "next_router", "next_router_packed", "next_router_wide",
       "stream_read", "stream_copy"]


def main():
    global SETTLE_US
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--repeats", type=int, default=7, help="timed loops of --steps calls per figure; the median is reported")
    ap.add_argument("--settle-us", type=float, default=SETTLE_US,
                    help="untimed pre-roll in front of every timed loop, in us of device time (0: loops start on an idle device)")
    ap.add_argument("--configs", default="all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the no-work stream kernel on each config's bytes")
    ap.add_argument("--no-headline", action="store_true",
                    help="profiling aid: run only the named configs and print their results without the headline line")
    ap.add_argument("--hot-only", action="store_true", help="profiling aid: one buffer set, no rotation")
    ap.add_argument("--stream-sweep", action="store_true",
                    help="time every variant of the no-work kernel on three configurations' byte counts and print a table")
    args = ap.parse_args()
    SETTLE_US = max(0.0, args.settle_us)
    if args.gpus != 1:
        print("bench.py: this path is measured on ONE GPU (every row block / expert is independent, "
              "there is no collective to time); --gpus must be 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    names = ALL if args.configs == "all" else [c.strip() for c in args.configs.split(",")]
    if "cfg1" not in names and not args.no_headline:
        names = ["cfg1"] + names
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    if args.stream_sweep:
        stream_sweep(dev, stream, args.steps, args.warmup, min(3, args.repeats))
        return
    builders = build_cases(set(names), dev)
    traffic = load_traffic_table()
    results = {}
    for name in names:
        case = builders[name]["build"]()
        case.allocate()
        if args.hot_only:
            case.sets = case.sets[:1]
        # the cache-resident loops and the single-call samples run first: by the time the
        # headline (cold) loops start the device has been busy for a few milliseconds and
        # its clocks have settled (the first loop after host-side set-up reads up to 10 % slow)
        # for the record, the eight headline configurations are also timed the plain way first: warm-up,
        # then loops of `steps` calls that each start on a device left idle for 20 ms
        idle = None
        if name in HEADLINE_CONFIGS and not args.hot_only and SETTLE_US > 0:
            idle = time_loop(case.launch, case.sets, args.steps, args.warmup, min(5, args.repeats), settle_us=0,
                             idle_gap_s=0.02)
        hot = None if args.hot_only else time_loop(case.launch, case.sets[:1], args.steps, args.warmup,
                                                   min(3, args.repeats))
        med, trimmed = time_single_calls(case, case.sets, max(10, min(args.steps, 200)), min(args.warmup, 10))
        cold = time_loop(case.launch, case.sets, args.steps, args.warmup, args.repeats)
        preroll = time_loop.last_preroll
        if hot is None:
            hot = cold
        us = median(cold)
        gbs = case.algo_bytes / us / 1e3
        r = dict(entry=case.entry, shape=case.shape, algorithmic_bytes=case.algo_bytes,
                 algorithmic_bytes_read=case.read_bytes, algorithmic_bytes_written=case.write_bytes,
                 us_per_call=round(us, 3), us_per_call_min=round(cold[0], 3), us_per_call_max=round(cold[-1], 3),
                 timed_loops=len(cold), preroll_calls=preroll,
                 gb_per_s=round(gbs, 1), frac_of_hbm_peak=round(gbs / HBM_PEAK_GBS, 4),
                 us_per_call_hot=round(median(hot), 3), gb_per_s_hot=round(case.algo_bytes / median(hot) / 1e3, 1),
                 us_single_call_median=round(med, 3), us_single_call_trimmed_mean=round(trimmed, 3),
                 buffer_sets=len(case.sets))
        if idle is not None:
            r["us_per_call_from_idle"] = round(median(idle), 3)
        if hasattr(case, "extra"):
            r.update(case.extra)
        # the buffers of the case are released before the ceiling and the CPU leg allocate theirs
        case.sets = []
        torch.cuda.empty_cache()
        if not args.no_ceiling and not name.startswith("stream_"):
            ceil_us, ceil_variant = stream_ceiling(case, dev, stream, args.steps, args.warmup, min(3, args.repeats))
            r["stream_us"] = round(ceil_us, 3)
            r["stream_variant"] = list(ceil_variant)
            r["stream_gb_per_s"] = round(case.algo_bytes / ceil_us / 1e3, 1)
            r["frac_of_stream"] = round(ceil_us / us, 4)
            torch.cuda.empty_cache()
        if name in traffic:
            r["hbm_traffic_bytes"] = traffic[name]["total"]
            r["hbm_fetched_bytes"] = traffic[name]["fetched"]
            r["hbm_written_bytes"] = traffic[name]["written"]
        if not args.no_cpu and case.cpu_fn is not None:
            r["cpu_us_per_call"] = round(time_cpu(case), 1)
            r["cpu_threads"] = torch.get_num_threads()
        results[name] = r
        print(f"[bench] {name}: {us:.2f} us cold [{cold[0]:.2f} .. {cold[-1]:.2f}] ({gbs:.0f} GB/s, "
              f"{100 * gbs / HBM_PEAK_GBS:.1f}% of peak"
              + (f", {100 * r['frac_of_stream']:.0f}% of the no-work kernel's rate" if "stream_us" in r else "")
              + f"), {median(hot):.2f} us hot", file=sys.stderr, flush=True)
        del case
        torch.cuda.empty_cache()

    if args.no_headline:
        print(json.dumps({"configs": results}))
        return
    write_full_results(results, args)
    line = headline_line(results, args.steps, args.warmup, SETTLE_US)
    print(encode_line(line), flush=True)


def encode_line(line):
    """JSON text of the headline line, kept under MAX_LINE_CHARS: if it ever grows beyond, the
    per-configuration extras go first (they are in the full results anyway), never the headline."""
    text = json.dumps(line, separators=(",", ":"))
    for drop in ("from_idle_us", "configs"):
        if len(text) < MAX_LINE_CHARS:
            break
        line = {k: v for k, v in line.items() if k != drop}
        text = json.dumps(line, separators=(",", ":"))
    return text


RESULTS_DIR = "gpurun_out"  # folder, beside this file, that side results are written to
MAX_LINE_CHARS = 4000  # the last stdout line must fit the window a harness keeps of stdout
HEADLINE_CONFIGS = ("cfg1", "cfg2", "cfg3", "cfg3b", "cfg4", "cfg5a", "cfg5b", "cfg5c")


def write_full_results(results, args):
    """Every field of every configuration: to bench_full.json in the results folder, or, when that
    cannot be written, as one JSON object per configuration on stderr.  The stdout line stays short."""
    out_dir = os.path.join(ROOT, RESULTS_DIR)
    try:
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, "bench_full.json"), "w") as f:
            json.dump({"steps": args.steps, "warmup": args.warmup, "repeats": args.repeats,
                       "settle_us": SETTLE_US, "configs": results}, f, indent=1)
    except OSError as e:  # a read-only tree
        print("[bench] bench_full.json not written: %s" % e, file=sys.stderr)
        for name, r in results.items():
            print("[bench-full] " + json.dumps({name: r}), file=sys.stderr)


def headline_line(results, steps, warmup, settle_us):
    """The ONE stdout line, built from the per-configuration results: cfg1 is the headline
    (BASELINE metric), `configs` maps every measured configuration to
    [us per call, fraction of the 8 TB/s peak, fraction of the no-work kernel's rate on the same
    bytes (null when not measured)], `from_idle_us` the same loops started on an idle device."""
    head = results["cfg1"]
    roofline = {"bound": "hbm", "achieved": head["gb_per_s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": head["frac_of_hbm_peak"], "traffic": head.get("hbm_traffic_bytes")}
    if "stream_us" in head:
        # what a kernel that only moves cfg1's bytes reaches on this device, and cfg1 against it
        roofline["copy_ceiling"] = head["stream_gb_per_s"]
        roofline["frac_of_copy_ceiling"] = head["frac_of_stream"]
    line = {
        "metric": "us/call and achieved HBM GB/s (% of peak), RMSNorm+quant fwd 8192x2048",
        "value": head["us_per_call"],
        "unit": "us/call",
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "preroll_calls": head.get("preroll_calls", 0),
        "ms_per_step": round(head["us_per_call"] / 1000.0, 6),
        "us_per_call_from_idle": head.get("us_per_call_from_idle"),
        "higher_is_better": False,
        "scaling": "weak",
        # the reference publishes 72.4 us for "RMSNorm+Quantization, forward" on an H800 at batch 8192, hidden 2048
        # (its README; tensor shapes, output_mode and round_scale are not stated): context, not a like-for-like
        # baseline, so vs_baseline stays null
        "vs_baseline": None,
        "reference_published": {"value": 72.4, "unit": "us/call", "hardware": "H800", "exact_config": "not stated"},
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "cfg1: RMSNorm + 1x128/128x1 e4m3 blockwise quant forward, x bf16 [8192,2048], "
                               "output_mode 2, buffers rotated beyond the Infinity Cache; value = median of %d "
                               "loops of %d calls, each behind preroll_calls untimed calls (%.1f ms of device "
                               "time); us_per_call_from_idle = same loops on a device idle for 20 ms"
                               % (head.get("timed_loops", 0), steps, settle_us / 1000.0),
                   "entry": head["entry"]},
        "roofline": roofline,
    }
    if "cpu_us_per_call" in head:
        line["cpu_baseline"] = {"value": head["cpu_us_per_call"], "unit": "us/call",
                                "cores": head["cpu_threads"], "kind": "port",
                                "sample": "cfg1 at full size, torch CPU oracle, 1 warm-up + min of 3 calls"}
    line["configs"] = {name: [r["us_per_call"], r["frac_of_hbm_peak"], r.get("frac_of_stream")]
                       for name, r in results.items()}
    line["from_idle_us"] = {name: r["us_per_call_from_idle"] for name, r in results.items()
                            if "us_per_call_from_idle" in r}
    line["full_results"] = RESULTS_DIR + "/bench_full.json"
    return line


if __name__ == "__main__":
    main()
