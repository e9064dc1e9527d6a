"""`quantized_decomposed` quantize / dequantize operators on ROCm GPUs.

Counterpart of torch_xla/experimental/quantized.py:7-41, which binds the four
operators to the XLA dispatch key (there they lower to StableHLO uniform
quantize / dequantize ops whose parameters live in the tensor type).  Here
they are bound to the CUDA key (ROCm tensors) and run as HIP elementwise
kernels through libxla_amd_qmm.so; values follow torch's own decomposition
(torch/ao/quantization/fx/_decomposed.py), which is what the operators denote.
The argument checks are the reference's `_check_scale_zp` (:52-70) plus its
"all scales > 0" assertion (:86-87).
"""
import weakref

import torch
from torch.library import impl
# defines the quantized_decomposed operators and their CPU / Meta implementations
from torch.ao.quantization.fx._decomposed import quantized_decomposed_lib

from xla_amd import _lib

_QDT = {torch.int8: _lib.QDT_I8, torch.uint8: _lib.QDT_U8, torch.int16: _lib.QDT_I16, torch.int32: _lib.QDT_I32}


# Parameter tensors whose values have been checked: (id(scale), id(zero_point), dtype) ->
# (versions and storage pointers at the time).  The value checks need the numbers on the host,
# which synchronises the device for GPU parameters; they run once per pair of parameter tensors,
# so that repeated calls with the same parameters launch without a synchronisation and can be
# captured into a HIP graph.
_validated = {}


def _param_state(t):
  try:
    v = t._version
  except RuntimeError:
    v = -1
  return (v, t.data_ptr(), t.numel())


def _check_scale_zp(input, scale, zero_point, axis, dtype):
  # 1. scale, zp are 1-D; 2. their length matches the (de)quant dim or is 1;
  # 3. dtype is an integer type; 4. zero points lie within dtype's range
  assert len(scale.shape) == 1 and len(zero_point.shape) == 1
  assert 'int' in str(dtype)
  assert dtype in _QDT, f"xla_amd: quantized dtype {dtype} is not supported on the GPU path"
  if axis == -1:
    assert scale.numel() == 1 and zero_point.numel() == 1
  else:
    assert axis >= 0 and axis < len(input.shape)
    qdq_dim_size = input.shape[axis]
    assert qdq_dim_size == scale.numel() or scale.numel() == 1
    assert qdq_dim_size == zero_point.numel() or zero_point.numel() == 1
  key = (id(scale), id(zero_point), dtype)
  state = (_param_state(scale), _param_state(zero_point))
  if _validated.get(key) == state:
    return
  if (scale.is_cuda or zero_point.is_cuda) and torch.cuda.is_current_stream_capturing():
    raise RuntimeError("xla_amd: quantization parameters are checked on the host the first time they are "
                       "seen; call the operator once with these parameter tensors before capturing a graph")
  info = torch.iinfo(dtype)
  zp_host = zero_point.cpu()
  assert torch.equal(zp_host, torch.clamp(zp_host, info.min, info.max))
  # all scales must be greater than 0 (StableHLO qdq constraint the reference enforces)
  assert bool((scale.cpu() > 0).all())
  if len(_validated) > 1024:
    _validated.clear()
  _validated[key] = state
  for t in (scale, zero_point):
    weakref.finalize(t, _validated.pop, key, None)


def _check_scalar(scale, zero_point, dtype):
  # the same conditions for host scalars
  assert 'int' in str(dtype)
  assert dtype in _QDT, f"xla_amd: quantized dtype {dtype} is not supported on the GPU path"
  info = torch.iinfo(dtype)
  assert info.min <= zero_point <= info.max
  assert scale > 0


def _per_channel_params(input, axis, scale, zero_point):
  """scale and zero_point with one entry per channel of `axis` (either may come with a single entry),
  or both with a single entry."""
  n = max(scale.numel(), 1 if zero_point is None else zero_point.numel())
  if n > 1:
    assert n == input.shape[axis]
    scale = scale.expand(n)
    if zero_point is not None:
      zero_point = zero_point.expand(n)
  return scale, zero_point


def _geometry(input, axis, n_params):
  """[outer, channels, inner] view of a contiguous tensor for parameters along `axis`."""
  if axis == -1 or n_params == 1:
    return 1, 1, input.numel()
  outer = 1
  for d in input.shape[:axis]:
    outer *= d
  inner = 1
  for d in input.shape[axis + 1:]:
    inner *= d
  return outer, input.shape[axis], inner


def _quantize(input, inv_scale, zero_point, quant_min, quant_max, dtype, axis):
  lib = _lib.load()
  x = input.contiguous()
  outer, channels, inner = _geometry(x, axis, inv_scale.numel())
  q = torch.empty(x.shape, dtype=dtype, device=x.device)
  inv = inv_scale.to(device=x.device, dtype=torch.float32).contiguous()
  zp = zero_point.to(device=x.device, dtype=torch.int32).contiguous()
  _lib.check(
      lib.xla_amd_qmm_quantize_affine(x.data_ptr(), q.data_ptr(), inv.data_ptr(), zp.data_ptr(), outer, channels,
                                      inner, _lib.dt(x.dtype), _QDT[dtype], quant_min, quant_max,
                                      _lib.stream_of(x)), "quantize_affine")
  return q


def _dequantize(input, scale, zero_point, dtype, out_dtype, axis, int_subtract):
  lib = _lib.load()
  assert input.dtype == dtype, f"Expecting input to have dtype: {dtype}, but got {input.dtype}"
  out_dtype = out_dtype or torch.float32
  q = input.contiguous()
  outer, channels, inner = _geometry(q, axis, scale.numel())
  out = torch.empty(q.shape, dtype=out_dtype, device=q.device)
  sc = scale.to(device=q.device, dtype=torch.float32).contiguous()
  zp = None if zero_point is None else zero_point.to(device=q.device, dtype=torch.int32).contiguous()
  _lib.check(
      lib.xla_amd_qmm_dequantize_affine(q.data_ptr(), out.data_ptr(), sc.data_ptr(), _lib.ptr(zp), outer, channels,
                                        inner, _QDT[dtype], _lib.dt(out_dtype), int_subtract, _lib.stream_of(q)),
      "dequantize_affine")
  return out


# per-tensor parameters are host scalars: their one-element device tensors are kept, so that a call
# does not pay two host-to-device copies
_scalar_cache = {}


def _scalar_params(device, a: float, z: int):
  key = (str(device), a, z)
  hit = _scalar_cache.get(key)
  if hit is None:
    if len(_scalar_cache) > 256:
      _scalar_cache.clear()
    hit = (torch.tensor([a], dtype=torch.float64).to(torch.float32).to(device),
           torch.tensor([z], dtype=torch.int32).to(device))
    _scalar_cache[key] = hit
  return hit


def _float_input(input):
  assert input.dtype in (torch.float32, torch.bfloat16, torch.float16), \
      f"Expecting input to have dtype torch.float32, but got dtype: {input.dtype}"


@impl(quantized_decomposed_lib, "quantize_per_tensor", "CUDA")
def rocm_quantize_per_tensor(input: torch.Tensor, scale: float, zero_point: int, quant_min: int, quant_max: int,
                             dtype: torch.dtype):
  _float_input(input)
  _check_scalar(scale, zero_point, dtype)
  # torch: inv_scale = 1.0 / scale in double, then multiplied into an f32 tensor as an f32 scalar
  inv, zp = _scalar_params(input.device, 1.0 / scale, zero_point)
  return _quantize(input, inv, zp, quant_min, quant_max, dtype, -1)


@impl(quantized_decomposed_lib, "quantize_per_channel", "CUDA")
def rocm_quantize_per_channel(input: torch.Tensor, scales: torch.Tensor, zero_points: torch.Tensor, axis: int,
                              quant_min: int, quant_max: int, dtype: torch.dtype):
  _float_input(input)
  assert axis < input.dim(), f"Expecting axis to be < {input.dim()}"
  _check_scale_zp(input, scales, zero_points, axis, dtype)
  scales, zero_points = _per_channel_params(input, axis, scales, zero_points)
  inv = 1.0 / scales.to(torch.float32) if scales.dtype != torch.float64 else (1.0 / scales).to(torch.float32)
  return _quantize(input, inv, zero_points, quant_min, quant_max, dtype, axis)


@impl(quantized_decomposed_lib, "dequantize_per_tensor", "CUDA")
def rocm_dequantize_per_tensor(input: torch.Tensor, scale: float, zero_point: int, quant_min: int, quant_max: int,
                               dtype: torch.dtype, *, out_dtype=None):
  _check_scalar(scale, zero_point, dtype)
  sc, zp = _scalar_params(input.device, scale, zero_point)
  return _dequantize(input, sc, zp, dtype, out_dtype, -1, 0)


@impl(quantized_decomposed_lib, "dequantize_per_channel", "CUDA")
def rocm_dequantize_per_channel(input: torch.Tensor, scales: torch.Tensor, zero_points, axis: int, quant_min: int,
                                quant_max: int, dtype: torch.dtype, *, out_dtype=None):
  assert axis < input.dim(), f"Expecting axis to be < {input.dim()}"
  zp_check = zero_points if zero_points is not None else torch.zeros_like(scales, dtype=torch.int64)
  _check_scale_zp(input, scales, zp_check, axis, dtype)
  scales, zero_points = _per_channel_params(input, axis, scales, zero_points)
  return _dequantize(input, scales, zero_points, dtype, out_dtype, axis, 1)
