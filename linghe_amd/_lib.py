"""ctypes binding of libfq_gfx950.so (declared in include/fq_api.h).

The library is the only compute path: if it is missing or fails to load, the
import of any operator module raises; there is no eager / CPU fallback.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libfq_gfx950.so"
# LINGHE_FQ_LIB names another build of the same library (same ABI), e.g. one compiled with other tuning macros
LIB_PATH = os.environ.get("LINGHE_FQ_LIB") or os.path.join(_HERE, LIB_NAME)

FQ_E4M3 = 0
FQ_E5M2 = 1
FQ_E5M2_MAX448 = 2

_P = ctypes.c_void_p
_I = ctypes.c_int
_L = ctypes.c_int64
_F = ctypes.c_float

# name -> argtypes, exactly the declarations of include/fq_api.h
SIGNATURES = {
    "fq_stream_rw": [_P, _L, _P, _L, _P, _I, _P],
    "fq_stream_rw_variant": [_P, _L, _P, _L, _P, _I, _L, _I, _I, _I, _P],
    "fq_blockwise_quant": [_P, _P, _P, _P, _P, _L, _L, _I, _I, _I, _P],
    "fq_batched_blockwise_quant": [_P, _P, _I, _I, _L, _P, _P, _P, _P, _L, _L, _I, _I, _P],
    "fq_batched_blockwise_quant_planned": [_P, _P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _P],
    "fq_expert_plan_shape": [_P, _I, _I, _P],
    "fq_batched_pad_permute_quant_planned": [_P, _P, _P, _I, _P, _P, _I, _P, _P, _P, _P, _P, _L, _L, _L, _I, _I, _P],
    "fq_build_expert_plan": [_P, _I, _I, _P, _P, _P],
    "fq_batched_pad_permute_quant": [_P, _P, _I, _I, _L, _P, _P, _I, _P, _P, _P, _P, _P, _L, _L, _L, _I, _I, _P],
    "fq_block_quant": [_P, _P, _P, _L, _L, _I, _I, _P],
    "fq_swiglu_fwd": [_P, _P, _I, _P, _L, _L, _P],
    "fq_swiglu_bwd": [_P, _P, _P, _I, _P, _P, _L, _L, _P],
    "fq_group_quant": [_P, _P, _P, _L, _L, _I, _I, _P],
    "fq_rmsnorm_fwd": [_P, _P, _P, _P, _L, _L, _F, _I, _P],
    "fq_rmsnorm_bwd": [_P, _P, _P, _P, _P, _P, _P, _L, _L, _L, _F, _P],
    "fq_rmsnorm_bwd_noalloc": [_P, _P, _P, _P, _P, _P, _L, _L, _F, _P],
    "fq_rmsnorm_quant_fwd": [_P, _P, _P, _P, _P, _P, _P, _L, _L, _F, _I, _I, _I, _P],
    "fq_rmsnorm_router_quant_fwd": [_P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _L, _L, _L, _F, _I, _I, _P],
    "fq_pack_router_weight": [_P, _I, _P, _L, _L, _P],
    "fq_rmsnorm_router_quant_fwd_packed": [_P, _P, _P, _I, _P, _P, _P, _P, _P, _L, _L, _L, _F, _I, _I, _P],
    "fq_swiglu_quant_fwd": [_P, _P, _P, _P, _P, _L, _L, _I, _I, _I, _P],
    "fq_swiglu_quant_bwd": [_P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _P],
    "fq_batched_swiglu_quant_fwd": [_P, _P, _I, _P, _I, _I, _L, _P, _P, _P, _P, _L, _L, _I, _I, _I, _P],
    "fq_batched_swiglu_quant_bwd": [_P, _P, _P, _I, _P, _I, _I, _L, _P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _P],
    "fq_batched_swiglu_quant_fwd_planned": [_P, _P, _I, _P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _I, _P],
    "fq_batched_swiglu_quant_bwd_planned": [_P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _P, _L, _L, _I, _I, _P],
}
OTHER_SYMBOLS = ["fq_version", "fq_last_error", "fq_rmsnorm_bwd_num_partials", "fq_rmsnorm_router_scratch_bytes",
                 "fq_expert_plan_bytes"]


def _load() -> ctypes.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m linghe_amd.build` "
            "(hipcc, gfx950). There is no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _I
    lib.fq_version.argtypes = []
    lib.fq_version.restype = _I
    lib.fq_last_error.argtypes = []
    lib.fq_last_error.restype = ctypes.c_char_p
    lib.fq_rmsnorm_bwd_num_partials.argtypes = [_L, _L]
    lib.fq_rmsnorm_bwd_num_partials.restype = _L
    lib.fq_rmsnorm_router_scratch_bytes.argtypes = [_L, _L, _I]
    lib.fq_rmsnorm_router_scratch_bytes.restype = _L
    lib.fq_expert_plan_bytes.argtypes = [_P]
    lib.fq_expert_plan_bytes.restype = _L
    return lib


lib = _load()


def check(rc: int) -> None:
    if rc != 0:
        msg = lib.fq_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"libfq_gfx950 error {rc}: {msg}")


def ptr(t):
    """Device address of a tensor (None -> NULL)."""
    return None if t is None else t.data_ptr()


# torch's raw-stream accessor costs 0.3 us, torch.cuda.current_stream(...).cuda_stream 4 us
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_of(t: torch.Tensor):
    """Handle of the current stream on t's device."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def on_device(device: torch.device):
    """Context that makes `device` current for a launch; free when it already is."""
    if torch.cuda.current_device() == device.index:
        return _NO_GUARD
    return torch.cuda.device(device)


def fp8_kind(dtype) -> int:
    if dtype == torch.float8_e4m3fn:
        return FQ_E4M3
    if dtype == torch.float8_e5m2:
        return FQ_E5M2
    raise ValueError(f"unsupported fp8 dtype {dtype}")


def require_device_bf16(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU: the HIP kernels are the only implementation")
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{name} must be bfloat16, got {t.dtype}")
