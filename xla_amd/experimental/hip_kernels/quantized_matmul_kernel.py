"""Tuned workgroup tiles of the gfx950 W8A8 GEMM, by problem shape.

Plays the role of TUNED_BLOCK_SIZES / get_tuned_block_sizes in
torch_xla/experimental/pallas_kernels/quantized_matmul_kernel.py:326-555: a
table from (device generation, batch, out features, in features, activation
dtype, quantize_activation) to the block sizes the kernel is launched with.
Here a "block" is the output tile of one workgroup (batch_block x out_block)
and the K extent of one LDS pipeline stage (in_block).
"""
import torch

_ARCH = "gfx950"

# key:   (arch, batch_size, n_output_features, n_input_features, activation_dtype, quantize_activation)
# value: (batch_block_size, out_block_size, in_block_size)
TUNED_BLOCK_SIZES = {}


def _add(batches, n_out, n_in, blocks):
  for bs in batches:
    for dtype in ("bfloat16", "float16", "float32"):
      TUNED_BLOCK_SIZES[(_ARCH, bs, n_out, n_in, dtype, True)] = blocks


# Fastest measured tile per shape (MI355X, one sweep over the four tile classes; ties
# within 3 % go to what the library would pick by itself).  Shapes: the Llama-3-8B
# linears (q/o, k/v, gate+up fused and single, qkv fused, down) and two square ones; launches of at most 128
# 64 x 64 tiles take the 32-wide tiles measured afterwards (15-45 % faster there).
# (n_out, n_in): {batch: (batch_block, out_block)}
_MEASURED = {
    (4096, 4096): {32: (32, 32), 64: (64, 32), 128: (64, 32), 256: (64, 64), 512: (64, 64), 1024: (128, 128),
                   2048: (128, 256), 4096: (256, 256), 8192: (256, 256)},
    (1024, 4096): {32: (32, 32), 64: (64, 32), 128: (64, 32), 256: (64, 32), 512: (64, 32), 1024: (64, 64),
                   2048: (64, 64), 4096: (64, 64), 8192: (128, 256)},
    (14336, 4096): {32: (64, 64), 64: (64, 64), 128: (64, 64), 256: (128, 128), 512: (128, 256), 1024: (256, 256),
                    2048: (256, 256), 4096: (256, 256), 8192: (256, 256)},
    (4096, 14336): {32: (32, 32), 64: (64, 32), 128: (64, 32), 256: (64, 64), 512: (64, 64), 1024: (128, 128),
                    2048: (128, 256), 4096: (256, 256), 8192: (256, 256)},
    (6144, 4096): {32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (64, 64), 1024: (128, 256),
                   2048: (256, 256), 4096: (256, 256), 8192: (256, 256)},
    (28672, 4096): {32: (64, 64), 64: (64, 64), 128: (128, 128), 256: (128, 256), 512: (256, 256), 1024: (256, 256),
                    2048: (256, 256), 4096: (256, 256), 8192: (256, 256)},
    (8192, 8192): {32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (128, 128), 1024: (128, 256),
                   2048: (256, 256), 4096: (256, 256), 8192: (256, 256)},
    (2048, 2048): {32: (32, 32), 64: (64, 32), 128: (64, 32), 256: (64, 32), 512: (64, 64), 1024: (64, 64),
                   2048: (64, 64), 4096: (128, 256), 8192: (256, 256)},
}
for (_n_out, _n_in), _by_batch in _MEASURED.items():
  for _bs, (_bm, _bn) in _by_batch.items():
    _add((_bs,), _n_out, _n_in, (_bm, _bn, 128))


def get_device_arch(device=None) -> str:
  """Architecture name of the GPU ("gfx950" on MI355X), or "" without one."""
  if not torch.cuda.is_available():
    return ""
  name = getattr(torch.cuda.get_device_properties(device or 0), "gcnArchName", "")
  return name.split(":")[0]


def get_tuned_block_sizes(block_table, batch_size, n_output_features, n_input_features,
                          activation_dtype, quantize_activation, arch=None):
  """(batch_block_size, out_block_size, in_block_size) for a shape, or
  (None, None, None) when the shape has not been tuned."""
  key = (arch if arch is not None else get_device_arch(), batch_size, n_output_features,
         n_input_features, activation_dtype, quantize_activation)
  return block_table.get(key, (None, None, None))
