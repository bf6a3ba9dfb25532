"""Drop-in import paths: ``from linghe.utils.norm import triton_rms_norm_and_block_quant_forward``
(and the other entry points of the fused blockwise-FP8 quantisation path) resolve
to the MI355X implementations in ``linghe_amd``.  Only that path is provided."""
