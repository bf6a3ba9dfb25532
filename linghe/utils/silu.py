from linghe_amd.utils.silu import (  # noqa: F401
    ExpertPlan,
    build_expert_plan,
    triton_batch_weighted_silu_and_block_quant_backward,
    triton_batch_weighted_silu_and_block_quant_forward,
    triton_silu_and_block_quant_backward,
    triton_silu_and_block_quant_forward,
    triton_weighted_silu_backward,
    triton_weighted_silu_forward,
)
