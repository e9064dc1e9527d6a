"""The dedicated int8 kernel and its tuned workgroup tiles, by problem shape.

Counterpart of torch_xla/experimental/pallas_kernels/quantized_matmul_kernel.py:
`quantized_matmul_int8` (:171-310) launches the gfx950 kernels with the
arithmetic of the Pallas `matmul_kernel` (:88-124), and TUNED_BLOCK_SIZES /
get_tuned_block_sizes (:326-555) map (device generation, batch, out features,
in features, activation dtype, quantize_activation) to the block sizes the
kernel is launched with.  Here a "block" is the output tile of one workgroup
(batch_block x out_block) and the K extent of one LDS pipeline stage (in_block).
"""
import torch

from xla_amd import _lib


def quantized_matmul_int8(
    x: torch.Tensor,  # [bs, n_input_features]
    w: torch.Tensor,  # [n_output_features, n_input_features] int8
    scalar: torch.Tensor,  # [n_output_features]
    zero_point=None,
    quant_block_size=None,
    quantize_activation: bool = False,
    *,
    batch_block_size=None,
    out_block_size=None,
    in_block_size=None,
):
  """int8-weight matmul with the arithmetic of the reference's dedicated kernel; result in x.dtype.

  quantize_activation: row abs-max, activation scale and quotient in x.dtype
  (:10-18, :199-200), int32 accumulation, then `acc * w_scale * x_scale` in
  float32 and one cast (:117-121).  Otherwise the float branch (:108-112,
  :246): float32 accumulation over all of K, `acc * w_scale` in float32, one
  cast.  The weight scale is always taken as float32 (:219-221).

  All three block sizes must be given, as in the reference (:194).  A
  (batch, out) pair the GEMM has no workgroup tile for, and `in_block_size`
  (the K extent of a pipeline stage is fixed at 128), act as hints only: the
  library then chooses the tile by shape; block sizes never change a value.
  """
  from xla_amd.experimental import xla_quantized_matmul as _qmm
  assert zero_point is None, "Not implemented: zero_point is not supported."
  assert quant_block_size is None, "Not implemented: quant_block_size is not supported."
  assert batch_block_size is not None and out_block_size is not None and in_block_size is not None
  assert x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], (
      f"x.shape[1] ({x.shape[1]}) must be equal to w.shape[1] ({w.shape[1]})")
  assert w.shape[0] == scalar.shape[0], (
      f"w.shape[0] ({w.shape[0]}) must be equal to scalar.shape[0] ({scalar.shape[0]})")
  x2 = x.contiguous()
  w = w.contiguous()
  scalar32 = scalar.to(torch.float32).contiguous()
  if quantize_activation:
    if (batch_block_size, out_block_size) not in _SUPPORTED_TILES:
      batch_block_size = out_block_size = 0
    return _qmm.w8a8_linear_gpu(x2, w, scalar32, None, x_scale_dtype=torch.float32, cvt_dtype=torch.float32,
                                mid_dtype=torch.float32, out_dtype=x.dtype, block_m=batch_block_size,
                                block_n=out_block_size)
  return _qmm._weight_only_gpu(x2, w, scalar32, None, -1, False, torch.float32, dot_dtype=torch.float32,
                               store_dtype=x.dtype)


# workgroup tiles (batch_block, out_block) the W8A8 GEMM is built for
_SUPPORTED_TILES = ((32, 32), (64, 32), (64, 64), (128, 128), (128, 256), (256, 256))

_ARCH = "gfx950"

# key:   (arch, batch_size, n_output_features, n_input_features, activation_dtype, quantize_activation)
# value: (batch_block_size, out_block_size, in_block_size)
TUNED_BLOCK_SIZES = {}


def _add(batches, n_out, n_in, blocks):
  for bs in batches:
    for dtype in ("bfloat16", "float16", "float32"):
      TUNED_BLOCK_SIZES[(_ARCH, bs, n_out, n_in, dtype, True)] = blocks


# Fastest measured tile per shape (MI355X, one sweep over the six workgroup tiles, quantized Gaussian operands,
# graph replays; a tile within 3 % of the fastest goes to what the library would pick by itself, which leaves four
# entries that differ from the shape rule: (5120, 640) at 2048 / 4096 rows and (5120, 1280) at 2048 rows, where a
# short K favours 128 x 128, and (37888, 3584) at 128 rows).  Shapes: the (out, in) pairs of the reference's table
# (Llama-3-8B; Llama-3-70B, Qwen2.5-7B and a 5120-wide model sharded over devices) plus the single projections
# and two square ones; batches as in the reference's table, 16 ... 16384 (where the result fits 700 M elements).
# (n_out, n_in): {batch: (batch_block, out_block)}
_MEASURED = {
    (6144, 4096): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (64, 64),
                   1024: (128, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (4096, 4096): {16: (32, 32), 32: (32, 32), 64: (32, 32), 128: (64, 32), 256: (64, 64), 512: (64, 64),
                   1024: (128, 128), 2048: (128, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (28672, 4096): {16: (64, 64), 32: (64, 64), 64: (64, 64), 128: (128, 128), 256: (128, 256), 512: (256, 256),
                    1024: (256, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (4096, 14336): {16: (32, 32), 32: (32, 32), 64: (32, 32), 128: (64, 32), 256: (64, 64), 512: (64, 64),
                    1024: (128, 128), 2048: (128, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (1024, 4096): {16: (32, 32), 32: (32, 32), 64: (32, 32), 128: (32, 32), 256: (32, 32), 512: (64, 32),
                   1024: (64, 64), 2048: (64, 64), 4096: (128, 128), 8192: (128, 256), 16384: (256, 256)},
    (14336, 4096): {16: (64, 64), 32: (64, 64), 64: (64, 64), 128: (64, 64), 256: (128, 128), 512: (128, 256),
                    1024: (256, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (8192, 8192): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (128, 128),
                   1024: (128, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (2048, 2048): {16: (32, 32), 32: (32, 32), 64: (32, 32), 128: (32, 32), 256: (64, 32), 512: (64, 64),
                   1024: (64, 64), 2048: (128, 128), 4096: (128, 256), 8192: (256, 256), 16384: (256, 256)},
    (1280, 8192): {16: (32, 32), 32: (32, 32), 64: (32, 32), 128: (32, 32), 256: (64, 32), 512: (64, 64),
                   1024: (64, 64), 2048: (64, 64), 4096: (128, 256), 8192: (256, 256), 16384: (256, 256)},
    (8192, 1024): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (128, 128),
                   1024: (128, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (7168, 8192): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (128, 128),
                   1024: (128, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (8192, 3584): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (128, 128),
                   1024: (128, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (4608, 3584): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (64, 64),
                   1024: (128, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (3584, 3584): {16: (32, 32), 32: (32, 32), 64: (32, 32), 128: (64, 32), 256: (64, 64), 512: (64, 64),
                   1024: (128, 128), 2048: (128, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (37888, 3584): {16: (64, 64), 32: (64, 64), 64: (64, 64), 128: (128, 128), 256: (256, 256), 512: (256, 256),
                    1024: (256, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (3584, 18944): {16: (32, 32), 32: (32, 32), 64: (32, 32), 128: (64, 32), 256: (64, 64), 512: (64, 64),
                    1024: (128, 128), 2048: (128, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (896, 5120): {16: (32, 32), 32: (32, 32), 64: (32, 32), 128: (32, 32), 256: (32, 32), 512: (64, 32),
                  1024: (64, 64), 2048: (64, 64), 4096: (128, 128), 8192: (128, 256), 16384: (256, 256)},
    (5120, 640): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (64, 64),
                  1024: (128, 256), 2048: (128, 128), 4096: (128, 128), 8192: (256, 256), 16384: (256, 256)},
    (5120, 1280): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (64, 64),
                   1024: (128, 256), 2048: (128, 128), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (1792, 5120): {16: (32, 32), 32: (32, 32), 64: (32, 32), 128: (32, 32), 256: (64, 32), 512: (64, 64),
                   1024: (64, 64), 2048: (128, 128), 4096: (128, 256), 8192: (256, 256), 16384: (256, 256)},
    (13824, 5120): {16: (64, 64), 32: (64, 64), 64: (64, 64), 128: (64, 64), 256: (128, 128), 512: (128, 256),
                    1024: (256, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (5120, 6912): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (64, 64),
                   1024: (128, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (6912, 5120): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (128, 128),
                   1024: (128, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
    (5120, 3456): {16: (32, 32), 32: (32, 32), 64: (64, 32), 128: (64, 64), 256: (64, 64), 512: (64, 64),
                   1024: (128, 256), 2048: (256, 256), 4096: (256, 256), 8192: (256, 256), 16384: (256, 256)},
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
