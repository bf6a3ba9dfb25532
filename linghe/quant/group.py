from linghe_amd.quant.group import triton_group_quant  # noqa: F401
