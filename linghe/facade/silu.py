from linghe_amd.facade.silu import (  # noqa: F401
    BlockBatchWeightedSiluFunction,
    BlockSiluFunction,
    block_batch_weighted_silu_impl,
    block_silu_impl,
)
