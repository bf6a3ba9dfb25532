from linghe_amd.utils.norm import (  # noqa: F401
    triton_rms_norm_and_block_quant_forward,
    triton_rms_norm_backward,
    triton_rms_norm_forward,
    triton_rms_norm_fp32_gemm_block_quant_forward,
)
