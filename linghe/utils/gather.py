from linghe_amd.utils.gather import triton_batch_block_pad_permute_with_indices  # noqa: F401
