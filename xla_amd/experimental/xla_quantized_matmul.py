"""`torch.ops.xla.quantized_matmul` and `XlaQuantizedLinear` for ROCm tensors.

Drop-in for torch_xla/experimental/xla_quantized_matmul.py: same operator
schema (:7-9), same shape/dtype checks and messages (:12-53), same module
(:186-243).  Tensors on a ROCm GPU run hand-written gfx950 kernels through
libxla_amd_qmm.so; there is no fallback for them.  CPU tensors take the
reference's own eager formulation (:139-183), which the reference documents
as its debugging path; meta tensors only get shapes and dtypes.
"""
import os
import weakref

import torch
import torch.nn.functional as F
from torch.library import impl

from xla_amd import _lib
from xla_amd.core.xla_model import XLA_LIB

XLA_LIB.define(
    "quantized_matmul(Tensor x, Tensor w, Tensor scale, Tensor? zero_point=None, int? block_size=-1, bool? int4_weight=False, bool? quantize_activation=False) -> Tensor"
)

# What float -> int8 does with a rounded quotient of +-128 (possible because
# the scale itself is rounded to x's dtype): "saturate" clamps like XLA's
# convert on the device path, "wrap" reproduces torch's CPU cast.
_OVERFLOW = {"saturate": _lib.OVERFLOW_SATURATE, "wrap": _lib.OVERFLOW_WRAP}


def _overflow_policy() -> str:
  p = os.environ.get("XLA_AMD_QMM_OVERFLOW", "saturate")
  if p not in _OVERFLOW:
    raise RuntimeError(f"XLA_AMD_QMM_OVERFLOW must be 'saturate' or 'wrap', got {p!r}")
  return p


# Dispatch decisions, for tests and profiling (kernel id -> calls).
counters = {"skinny_mfma": 0, "generic": 0, "w8a8_mfma": 0, "w8a8_generic": 0, "pack": 0, "pack_hit": 0}


def _check_per_channel_quant_weight_dtype_shapes(input_dim, output_dim, w, w_scaler, zero_point):
  assert w.dtype == torch.int8, f"Weight dtype is expected to be torch.int8, got {w.dtype}."
  assert w.dim() == 2, f"Weight tensor is expected to be 2D, got {w.dim()}D Tensor."
  w_shape = list(w.shape)
  assert output_dim == w_shape[0] and input_dim == w_shape[
      1], f"Weight shape is expected to be [output_dim, input_dim], output_dim: {output_dim}, input_dim: {input_dim}, but got {w_shape}."
  assert w_scaler.dim() == 1 and w_scaler.shape[0] == w_shape[
      0], f"weight scaler shape is expect to be [out_channel,], got {w_scaler.shape}, weight shape {w_shape}."
  if zero_point is not None:
    assert zero_point.dim() == 1 and w_scaler.shape[0] == w_shape[
        0], f"zero point shape is expect to be [out_channel,], got {zero_point.shape}, weight shape {w_shape}."


def _check_blockwise_quant_weight_dtype_shapes(input_dim, output_dim, block_size, w, w_scaler,
                                               zero_point):
  assert w.dtype == torch.int8, (f"Weight dtype is expected to be torch.int8, got {w.dtype}.")
  assert w.dim() == 3, (f"Weight tensor is expected to be 3D, got {w.dim()}D Tensor.")
  w_shape = list(w.shape)
  assert input_dim % block_size == 0, (f"input_dim should be divisible by block_size, "
                                       f"got input_dim: {input_dim}, block_size: {block_size}.")
  assert w_shape[0] == input_dim / block_size and w_shape[1] == block_size, (
      f"Weight shape is expected to be [input_dim / block_size, block_size, output_dim], "
      f"input_dim: {input_dim}, block_size: {block_size}, output_dim: {output_dim}, "
      f"but got {w_shape}.")
  assert w_scaler.dim() == 2, (f"weight scaler is expected to be 2D, got {w_scaler.dim()}D Tensor.")
  assert w_scaler.shape[0] == w_shape[0] and w_scaler.shape[1] == w_shape[-1], (
      f"weight scaler shape is expect to be [in_channel / block_size, out_channel], "
      f"got {w_scaler.shape}, weight shape {w_shape}.")
  if zero_point is not None:
    assert zero_point.dim() == 2, (f"zero_point is expected to be 2D, got {zero_point.dim()}D Tensor.")
    assert zero_point.shape[0] == w_shape[0] and zero_point.shape[1] == w_shape[-1], (
        f"zero_point shape is expect to be [in_channel / block_size, out_channel], "
        f"got {zero_point.shape}, weight shape {w_shape}.")


def _check_args(x, w, scaler, zero_point, block_size, quantize_activation):
  if block_size == -1:
    _check_per_channel_quant_weight_dtype_shapes(x.shape[-1], scaler.shape[0], w, scaler, zero_point)
  else:
    assert quantize_activation == False, (
        "Blockwise quantization does not support activation quantization.")
    _check_blockwise_quant_weight_dtype_shapes(x.shape[-1], w.shape[-1], block_size, w, scaler,
                                               zero_point)


def _result_dtype(x, scaler, quantize_activation):
  """dtype the reference's op sequence ends in (torch type promotion)."""
  if quantize_activation:
    # int32 * scaler -> scaler.dtype; ... * x_scale (x.dtype) -> promotion of the two
    return torch.promote_types(scaler.dtype, x.dtype)
  return torch.promote_types(x.dtype, scaler.dtype)


# ---- one-time re-layouts of weights ----------------------------------------------
# key (id(w), kind) -> (version, data_ptr, bits, copy); dropped when w dies.
_pack_cache = {}


def _relayout(w: torch.Tensor, bits: int, layout: int, kind: str) -> torch.Tensor:
  key = (id(w), kind)
  hit = _pack_cache.get(key)
  if hit is not None and hit[0] == w._version and hit[1] == w.data_ptr() and hit[2] == bits:
    counters["pack_hit"] += 1
    return hit[3]
  if layout == _lib.W_NK:
    n, k = w.shape
    s, c = 1, k
  else:
    s, c, n = w.shape
    k = s * c
  lib = _lib.load()
  size_fn, copy_fn = ((lib.xla_amd_qmm_tiled_bytes, lib.xla_amd_qmm_tile_weight) if kind == "tiled" else
                      (lib.xla_amd_qmm_packed_bytes, lib.xla_amd_qmm_pack_weight))
  nbytes = size_fn(n, k, bits)
  if nbytes == 0:
    raise RuntimeError(f"xla_amd: cannot re-lay out weight of shape {tuple(w.shape)} to {bits} bits ({kind})")
  out = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
  _lib.check(copy_fn(w.data_ptr(), out.data_ptr(), s, c, n, layout, bits, _lib.stream_of(w)), f"{kind} weight")
  counters["pack"] += 1
  if hit is None:
    weakref.finalize(w, _pack_cache.pop, key, None)
  _pack_cache[key] = (w._version, w.data_ptr(), bits, out)
  return out


def _packed_weight(w: torch.Tensor, bits: int, layout: int) -> torch.Tensor:
  """Plain K-major copy of w (int8 [N,K] or int4 nibbles [N,K/2])."""
  return _relayout(w, bits, layout, "packed")


def _tiled_weight(w: torch.Tensor, bits: int, layout: int) -> torch.Tensor:
  """Tiled copy of w for the streaming kernel (blocks of 16 channels x 128 columns in MFMA operand order).

  The copy is made once per weight tensor and reused while the tensor is alive
  and unmodified (same object, same storage pointer, same version counter); it
  costs as much device memory again as the weight itself.
  """
  return _relayout(w, bits, layout, "tiled")


def _weight_only_gpu(x2, w, scaler, zero_point, block_size, int4_weight, out_dtype):
  lib = _lib.load()
  m, k = x2.shape
  blockwise = block_size != -1
  n = w.shape[-1] if blockwise else w.shape[0]
  c = block_size if blockwise else k
  if blockwise and (scaler.dtype != x2.dtype or (zero_point is not None and zero_point.dtype != x2.dtype)):
    # torch.einsum / torch.matmul of the reference raise on mixed dtypes here
    raise RuntimeError(
        f"expected scalar type {x2.dtype} for blockwise scaler/zero_point, got {scaler.dtype}"
        f"{'' if zero_point is None else '/' + str(zero_point.dtype)}")
  out = torch.empty((m, n), dtype=out_dtype, device=x2.device)
  if m == 0:
    return out
  bits = 4 if int4_weight else 8
  kern = lib.xla_amd_qmm_dispatch(m, n, k, c, bits, _lib.dt(x2.dtype), 0)
  layout = _lib.W_SCN if blockwise else _lib.W_NK
  stream = _lib.stream_of(x2)
  zp_dt = _lib.dt(zero_point.dtype) if zero_point is not None else _lib.dt(x2.dtype)
  if kern == _lib.KERNEL_SKINNY_MFMA:
    wk = _tiled_weight(w, bits, layout)
    counters["skinny_mfma"] += 1
    _lib.check(
        lib.xla_amd_qmm_weight_only_skinny(x2.data_ptr(), wk.data_ptr(), scaler.data_ptr(),
                                           _lib.ptr(zero_point), out.data_ptr(), m, n, k, c, bits,
                                           _lib.dt(x2.dtype), _lib.dt(scaler.dtype), zp_dt,
                                           _lib.dt(out_dtype), stream), "weight_only_skinny")
  else:
    counters["generic"] += 1
    _lib.check(
        lib.xla_amd_qmm_weight_only_generic(x2.data_ptr(), w.data_ptr(), scaler.data_ptr(),
                                            _lib.ptr(zero_point), out.data_ptr(), m, n, k, c, layout,
                                            _lib.dt(x2.dtype), _lib.dt(scaler.dtype), zp_dt,
                                            _lib.dt(out_dtype), stream), "weight_only_generic")
  return out


def quantize_per_token_gpu(x2: torch.Tensor, scale_dtype=None, want_sum=False, overflow=None):
  """`_quantize_tensor` (:56-73) on the GPU: returns (x_q int8 [M,K], scale [M,1], x_sum|None)."""
  lib = _lib.load()
  m, k = x2.shape
  scale_dtype = scale_dtype or x2.dtype
  x_q = torch.empty((m, k), dtype=torch.int8, device=x2.device)
  x_scale = torch.empty((m, 1), dtype=scale_dtype, device=x2.device)
  x_sum = torch.empty((m,), dtype=torch.int32, device=x2.device) if want_sum else None
  policy = _OVERFLOW[overflow or _overflow_policy()]
  _lib.check(
      lib.xla_amd_qmm_quantize_per_token(x2.data_ptr(), x_q.data_ptr(), x_scale.data_ptr(),
                                         _lib.ptr(x_sum), m, k, _lib.dt(x2.dtype),
                                         _lib.dt(scale_dtype), policy, _lib.stream_of(x2)),
      "quantize_per_token")
  return x_q, x_scale, x_sum


def w8a8_gemm_gpu(x_q, w, x_scale, w_scale, zero_point, x_sum, *, cvt_dtype, mid_dtype, out_dtype,
                  want_acc=False, block_m=0, block_n=0):
  """int8 GEMM + epilogue; returns (out, acc|None)."""
  lib = _lib.load()
  m, k = x_q.shape
  n = w.shape[0]
  out = torch.empty((m, n), dtype=out_dtype, device=x_q.device)
  acc = torch.empty((m, n), dtype=torch.int32, device=x_q.device) if want_acc else None
  if m == 0:
    return out, acc
  kern = lib.xla_amd_qmm_dispatch(m, n, k, k, 8, _lib.DT_F32, 1)
  counters["w8a8_mfma" if kern == _lib.KERNEL_W8A8_MFMA else "w8a8_generic"] += 1
  zp_dt = _lib.dt(zero_point.dtype) if zero_point is not None else _lib.DT_F32
  _lib.check(
      lib.xla_amd_qmm_w8a8_gemm(x_q.data_ptr(), w.data_ptr(), x_scale.data_ptr(), w_scale.data_ptr(),
                                _lib.ptr(zero_point), _lib.ptr(x_sum), out.data_ptr(), _lib.ptr(acc),
                                m, n, k, _lib.dt(x_scale.dtype), _lib.dt(w_scale.dtype), zp_dt,
                                _lib.dt(cvt_dtype), _lib.dt(mid_dtype), zp_dt, _lib.dt(out_dtype),
                                block_m, block_n, _lib.stream_of(x_q)), "w8a8_gemm")
  return out, acc


@impl(XLA_LIB, "quantized_matmul", "CUDA")
def quantized_matmul_rocm(x: torch.Tensor,
                          w: torch.Tensor,
                          scaler: torch.Tensor,
                          zero_point: torch.Tensor = None,
                          block_size: int = -1,
                          int4_weight: bool = False,
                          quantize_activation: bool = False):
  """Quantized matrix multiply on a ROCm GPU (arguments as xla_quantized_matmul.py:84-100).

      x: activation [..., in_channel] (float32, bfloat16 or float16).
      w: int8 weight; per-channel [out_channel, in_channel]; blockwise
         [in_channel / block_size, block_size, out_channel].
      scaler: per-channel [out_channel]; blockwise [in_channel / block_size, out_channel].
      zero_point: optional, same shape as scaler, in real units (integer zero
         point times scale).
      int4_weight: the int8 container holds int4 values; they are packed two
         per byte once per weight tensor.
      quantize_activation: per-token dynamic int8 quantization of x (W8A8).
  """
  block_size = -1 if block_size is None else block_size
  int4_weight = bool(int4_weight)
  quantize_activation = bool(quantize_activation)
  _check_args(x, w, scaler, zero_point, block_size, quantize_activation)
  if not (x.is_floating_point() and scaler.is_floating_point()):
    raise RuntimeError(f"xla_amd quantized_matmul: x and scaler must be floating point, got {x.dtype}, {scaler.dtype}")
  out_dtype = _result_dtype(x, scaler, quantize_activation)
  x2 = x.reshape(-1, x.shape[-1]).contiguous()
  w = w.contiguous()
  scaler = scaler.contiguous()
  if zero_point is not None:
    zero_point = zero_point.contiguous()
  if quantize_activation:
    x_q, x_scale, x_sum = quantize_per_token_gpu(x2, want_sum=zero_point is not None)
    out, _ = w8a8_gemm_gpu(x_q, w, x_scale, scaler, zero_point, x_sum, cvt_dtype=scaler.dtype,
                           mid_dtype=scaler.dtype, out_dtype=out_dtype)
  else:
    out = _weight_only_gpu(x2, w, scaler, zero_point, block_size, int4_weight, out_dtype)
  return out.reshape(*x.shape[:-1], out.shape[-1])


def _quantize_tensor(x: torch.Tensor, n_bits: int = 8, dim: int = -1):
  """Eager form of the activation quantizer (:56-73), used for CPU tensors."""
  max_val = torch.amax(torch.abs(x), dim=dim, keepdim=True)
  int_max = 2**(n_bits - 1) - 1
  scale = max_val / int_max
  x_int = torch.round(x / scale).to(torch.int8)
  return x_int, scale.to(x.dtype)


@impl(XLA_LIB, "quantized_matmul", "CPU")
def quantized_matmul(x: torch.Tensor,
                     w: torch.Tensor,
                     scaler: torch.Tensor,
                     zero_point: torch.Tensor = None,
                     block_size: int = -1,
                     int4_weight: bool = False,
                     quantize_activation: bool = False):
  """CPU tensors only: the reference's eager debugging path (:139-183)."""
  block_size = -1 if block_size is None else block_size
  _check_args(x, w, scaler, zero_point, block_size, quantize_activation)
  if block_size == -1:
    w = w.to(x.dtype)
    if quantize_activation:
      x, x_scale = _quantize_tensor(x)
      x = x.to(torch.int32)
      w = w.to(torch.int32)
    out = F.linear(x, w)
    out = out * scaler
  else:
    x = x.reshape(*x.shape[:-1], x.shape[-1] // block_size, block_size)
    w = w.to(x.dtype)
    out = torch.einsum('scn,...sc->...sn', w, x)
    out = torch.einsum('sn,...sn->...n', scaler, out)
  if zero_point is not None:
    if block_size == -1:
      zp_out = torch.einsum("...c,z->...z", x, zero_point)
    else:
      zp_out = torch.matmul(x.sum(dim=-1), zero_point)
    out -= zp_out
  if quantize_activation:
    out = out * x_scale
  return out


@impl(XLA_LIB, "quantized_matmul", "Meta")
def quantized_matmul_meta(x, w, scaler, zero_point=None, block_size=-1, int4_weight=False,
                          quantize_activation=False):
  block_size = -1 if block_size is None else block_size
  _check_args(x, w, scaler, zero_point, block_size, bool(quantize_activation))
  n = w.shape[0] if block_size == -1 else w.shape[-1]
  return torch.empty(*x.shape[:-1], n, dtype=_result_dtype(x, scaler, bool(quantize_activation)),
                     device=x.device)


class XlaQuantizedLinear(torch.nn.Module):
  """Linear layer over a quantized weight (xla_quantized_matmul.py:186-243).

  State-dict keys and buffer shapes are the reference's: `weight` int8
  [out, in], `weight_scaler` [out], and `zero_point` [out] unless symmetric;
  `load_quantized_weight` replaces them (blockwise weights are 3-D).
  """

  def __init__(self,
               input_dim,
               output_dim,
               is_symmetric: bool = False,
               block_size: int = -1,
               int4_weight: bool = False,
               quantize_activation: bool = False):
    super().__init__()
    self.input_dim = input_dim
    self.output_dim = output_dim
    self.is_symmetric = is_symmetric
    self.block_size = block_size
    self.int4_weight = int4_weight
    self.quantize_activation = quantize_activation
    self.register_buffer('weight', torch.zeros(output_dim, input_dim).to(torch.int8))
    self.register_buffer('weight_scaler', torch.zeros(output_dim))
    if not self.is_symmetric:
      self.register_buffer('zero_point', torch.zeros(output_dim))
    else:
      self.zero_point = None

  def load_quantized_weight(self, weight, weight_scaler, zero_point=None):
    '''
    weight: per-channel [out_channel, in_channel];
            blockwise [in_channel / block_size, block_size, out_channel].
    weight_scaler: per-channel [out_channel]; blockwise [in_channel / block_size, out_channel].
    '''
    if self.block_size == -1:
      _check_per_channel_quant_weight_dtype_shapes(self.input_dim, self.output_dim, weight,
                                                   weight_scaler, zero_point)
    else:
      _check_blockwise_quant_weight_dtype_shapes(self.input_dim, self.output_dim, self.block_size,
                                                 weight, weight_scaler, zero_point)
    self.weight = weight
    self.weight_scaler = weight_scaler
    self.zero_point = zero_point

  def forward(self, x):
    return torch.ops.xla.quantized_matmul(
        x,
        self.weight,
        self.weight_scaler,
        self.zero_point,
        block_size=self.block_size,
        int4_weight=self.int4_weight,
        quantize_activation=self.quantize_activation)
