from linghe_amd.quant.block import (  # noqa: F401
    triton_batch_blockwise_quant,
    triton_block_quant,
    triton_blockwise_quant,
)
