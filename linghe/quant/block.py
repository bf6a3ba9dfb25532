from linghe_amd.quant.block import triton_batch_blockwise_quant, triton_blockwise_quant  # noqa: F401
