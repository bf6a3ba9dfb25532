from linghe_amd.facade.norm import BlockRMSNorm, RMSNormFunction, block_rms_norm, rms_norm  # noqa: F401
