"""MI355X-native (gfx950) fused blockwise-FP8 quantisation path.

Python entry points keep the names, argument order and return tuples of the
reference's wrappers (linghe.utils.norm, linghe.utils.silu, linghe.quant.block,
linghe.quant.group) and call hand-written HIP kernels through the C ABI of
libfq_gfx950.so (include/fq_api.h).
"""
__version__ = "0.2.0"
