"""MI355X-native quantized linear path behind PyTorch/XLA's operator interface.

Importing `xla_amd.experimental.xla_quantized_matmul` (or
`xla_amd.experimental.custom_kernel`) defines `torch.ops.xla.quantized_matmul`
and `torch.ops.xla.quantized_matmul_int8` for ROCm tensors; the arithmetic
runs in hand-written gfx950 HIP kernels reached through the C ABI of
libxla_amd_qmm.so (include/xla_amd_qmm.h).
"""
__version__ = "0.1.0"
