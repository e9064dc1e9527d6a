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


# Llama-3-8B linears (q/o, k/v, gate/up, down) at prefill batch sizes.
for _n_out, _n_in in ((4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336), (6144, 4096),
                      (28672, 4096)):
  _add((1024, 2048, 4096, 8192), _n_out, _n_in, (256, 256, 128))
  # (128 x 256 once it still gives >= 160 workgroups)
  _add((512,), _n_out, _n_in, (128, 256, 128) if _n_out >= 10240 else (128, 128, 128))
  _add((256,), _n_out, _n_in, (128, 256, 128) if _n_out >= 20480 else (128, 128, 128))
  _add((64, 128), _n_out, _n_in, (64, 64, 128))


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
