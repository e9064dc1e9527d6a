"""CPU restatement of the affine quantize / dequantize operators (TEST INFRASTRUCTURE ONLY).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; the product never does.

What the reference binds (torch_xla/experimental/quantized.py:7-41) lowers to
StableHLO uniform quantize / dequantize ops; its tests check the exported text
only (test/stablehlo/test_pt2e_qdq.py), never values, so values are pinned
here against torch's own decomposition of the same operators
(torch/ao/quantization/fx/_decomposed.py, a library routine) in
tests/test_oracle_pins.py.  Against the reference's PJRT execution of those
StableHLO ops: parity unpinned.

numpy float32 arithmetic, op by op.
"""
import numpy as np


def _bcast(p, shape, axis):
  p = np.asarray(p)
  if axis == -1 or p.size == 1:
    return p.reshape(-1)[0]
  view = [1] * len(shape)
  view[axis] = shape[axis]
  return p.reshape(view)


def quantize_affine(x, inv_scale, zero_point, quant_min, quant_max, np_dtype, axis=-1):
  """q = cast(clamp(rint(f32(x) * inv_scale) + zp, qmin, qmax)); NaN -> 0."""
  x = np.asarray(x, dtype=np.float32)
  inv = np.float32(_bcast(np.asarray(inv_scale, dtype=np.float32), x.shape, axis))
  zp = np.float32(_bcast(np.asarray(zero_point, dtype=np.float32), x.shape, axis))
  with np.errstate(invalid="ignore", over="ignore"):
    r = np.rint(x * inv).astype(np.float32) + zp  # np.rint: half to even
    r = np.clip(r, np.float32(quant_min), np.float32(quant_max))
    r = np.where(np.isnan(x), np.float32(0), r)
  return r.astype(np_dtype)


def dequantize_per_channel(q, scale, zero_point, axis):
  """f32(q - zp) * scale (integer subtraction first)."""
  q = np.asarray(q).astype(np.int64)
  zp = 0 if zero_point is None else _bcast(np.asarray(zero_point, dtype=np.int64), q.shape, axis)
  sc = _bcast(np.asarray(scale, dtype=np.float32), q.shape, axis)
  return ((q - zp).astype(np.float32) * sc).astype(np.float32)


def dequantize_per_tensor_f32(q, scale, zero_point):
  """(f32(q) - zp) * scale, both ops in f32."""
  q = np.asarray(q).astype(np.float32)
  return ((q - np.float32(zero_point)).astype(np.float32) * np.float32(scale)).astype(np.float32)
