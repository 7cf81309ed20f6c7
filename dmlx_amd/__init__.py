"""dmlx_amd — MI355X (gfx950) implementation of dmlx's quantized MoE expert-FFN path.

capi      ctypes binding of libdmoe.so (the C ABI in include/dmoe.h)
quantize  weight quantizers (MLX affine 4/8-bit, MXFP4, FP8 per-row) for data preparation
workloads seeded synthetic inputs of the five benchmark configurations
"""
