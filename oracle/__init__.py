"""CPU oracle for the fused blockwise-FP8 quantization path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``linghe_amd/`` may import this
package: it is the checker for the HIP kernels (tests, the smoke check and the
CPU-baseline leg of the benchmark), never the thing that is shipped or timed
as the product.
"""
