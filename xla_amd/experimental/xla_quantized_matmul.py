"""`torch.ops.xla.quantized_matmul` and `XlaQuantizedLinear` for ROCm tensors.

Drop-in for torch_xla/experimental/xla_quantized_matmul.py: same operator
schema (:7-9), same shape/dtype checks and messages (:12-53), same module
(:186-243).  Tensors on a ROCm GPU run hand-written gfx950 kernels through
libxla_amd_qmm.so; there is no fallback for them.  CPU tensors take an eager
formulation with the rounding points of the reference's (:139-183), which the
reference documents as its debugging path; meta tensors only get shapes and
dtypes.
"""
import os
import weakref

import torch
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
counters = {"skinny_mfma": 0, "wo_gemm": 0, "generic": 0, "w8a8_mfma": 0, "w8a8_generic": 0, "pack": 0, "pack_hit": 0}


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
# The streaming kernel reads a tiled copy of the weight (blocks of 16 channels x
# 128 columns in MFMA operand order).  It is made once per weight tensor, either
# explicitly (`prepare_weight`, `XlaQuantizedLinear.prepare`) or on the first call
# that needs it, and kept in `_pack_cache` while the tensor object is alive.
#
# key (id(w), kind) -> (version, data_ptr, bits, copy)
_pack_cache = {}


def _version_of(w: torch.Tensor) -> int:
  try:
    return w._version
  except RuntimeError:  # inference tensors do not track a version counter
    return -1


def invalidate_weight_cache(w: torch.Tensor = None):
  """Drops the cached re-layouts of `w` (of every weight when `w` is None).

  The cache notices in-place operations on the weight through torch's version
  counter.  Writes that bypass the counter are invisible to it and need this
  call: `w.data.copy_(...)` / `w.data[...] = ...`, anything written into an
  inference-mode tensor, and writes from outside torch to the same memory.
  """
  if w is None:
    _pack_cache.clear()
    return
  for kind in ("tiled", "packed"):
    _pack_cache.pop((id(w), kind), None)


def _relayout(w: torch.Tensor, bits: int, layout: int, kind: str) -> torch.Tensor:
  key = (id(w), kind)
  hit = _pack_cache.get(key)
  if hit is not None and hit[0] == _version_of(w) and hit[1] == w.data_ptr() and hit[2] == bits:
    counters["pack_hit"] += 1
    return hit[3]
  if torch.cuda.is_current_stream_capturing():
    # The copy would only be recorded, not made: the buffer would stay empty until the first
    # replay and every replay would repeat the re-layout.
    raise RuntimeError(
        "xla_amd: the weight of a quantized_matmul call has no device-side copy yet and the current "
        "stream is being captured into a HIP graph; call xla_amd.experimental.xla_quantized_matmul."
        "prepare_weight(w, ...) or XlaQuantizedLinear.prepare() (or run the call once) before the capture")
  if layout == _lib.W_NK:
    n, k = w.shape
    s, c = 1, k
  else:
    s, c, n = w.shape
    k = s * c
  lib = _lib.load()
  if kind == "tiled":
    copy_fn, nbytes = lib.xla_amd_qmm_tile_weight, lib.xla_amd_qmm_tiled_bytes(n, k, c, bits)
  else:
    copy_fn, nbytes = lib.xla_amd_qmm_pack_weight, lib.xla_amd_qmm_packed_bytes(n, k, bits)
  if nbytes == 0:
    raise RuntimeError(f"xla_amd: cannot re-lay out weight of shape {tuple(w.shape)} to {bits} bits ({kind})")
  out = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
  # (the copy is keyed on the caller's tensor; a strided weight is read through a contiguous temporary, once)
  src = w if w.is_contiguous() else w.contiguous()
  _lib.check(copy_fn(src.data_ptr(), out.data_ptr(), s, c, n, layout, bits, _lib.stream_of(w)), f"{kind} weight")
  counters["pack"] += 1
  if hit is None:
    weakref.finalize(w, _pack_cache.pop, key, None)
  _pack_cache[key] = (_version_of(w), w.data_ptr(), bits, out)
  return out


def _packed_weight(w: torch.Tensor, bits: int, layout: int) -> torch.Tensor:
  """Plain K-major copy of w (int8 [N,K] or int4 nibbles [N,K/2])."""
  return _relayout(w, bits, layout, "packed")


def _tiled_weight(w: torch.Tensor, bits: int, layout: int) -> torch.Tensor:
  """Tiled copy of w for the streaming kernel (blocks of a channel group x 128 columns in MFMA operand order).

  The copy is made once per weight tensor and reused while the tensor is alive
  and unmodified (same object, same storage pointer, same version counter); it
  costs as much device memory again as the weight itself (half for int4).
  """
  return _relayout(w, bits, layout, "tiled")


def _weight_geometry(w, block_size):
  """(n, k, c, layout) of an operator weight."""
  if block_size == -1:
    n, k = w.shape
    return n, k, k, _lib.W_NK
  s, c, n = w.shape
  return n, s * c, c, _lib.W_SCN


def prepare_weight(w: torch.Tensor, block_size: int = -1, int4_weight: bool = False, x_dtype=torch.bfloat16):
  """Makes the device-side copy of `w` that `quantized_matmul(x, w, ...)` will read, now.

  Returns True when the weight-only call for this weight runs the streaming
  kernel (which reads a tiled copy), False when it reads `w` itself and there is
  nothing to prepare.  Call it before capturing a HIP graph: the first call for a
  weight otherwise makes the copy lazily, which a capture must not record.
  """
  if not w.is_cuda:
    return False
  n, k, c, layout = _weight_geometry(w, block_size)
  bits = 4 if int4_weight else 8
  if _lib.load().xla_amd_qmm_dispatch(1, n, k, c, bits, _lib.dt(x_dtype), 0) != _lib.KERNEL_SKINNY_MFMA:
    return False
  _tiled_weight(w, bits, layout)
  return True


def _weight_only_launch(x2, w, w_tiled, n, k, c, layout, bits, scaler, zero_point, out_dtype, dot_dtype, store_dtype):
  """One weight-only launch; `w` (operator layout) or `w_tiled` may be None, not both."""
  lib = _lib.load()
  m = x2.shape[0]
  blockwise = c != k
  if blockwise and (scaler.dtype != x2.dtype or (zero_point is not None and zero_point.dtype != x2.dtype)):
    # torch.einsum / torch.matmul of the reference raise on mixed dtypes here
    raise RuntimeError(
        f"expected scalar type {x2.dtype} for blockwise scaler/zero_point, got {scaler.dtype}"
        f"{'' if zero_point is None else '/' + str(zero_point.dtype)}")
  dot_dtype = dot_dtype or x2.dtype
  store_dtype = store_dtype or out_dtype
  out = torch.empty((m, n), dtype=store_dtype, device=x2.device)
  if m == 0:
    return out
  kern = lib.xla_amd_qmm_dispatch(m, n, k, c, bits, _lib.dt(x2.dtype), 0)
  stream = _lib.stream_of(x2)
  zp_dt = _lib.dt(zero_point.dtype) if zero_point is not None else _lib.dt(x2.dtype)
  dts = (_lib.dt(x2.dtype), _lib.dt(scaler.dtype), zp_dt, _lib.dt(dot_dtype), _lib.dt(out_dtype),
         _lib.dt(store_dtype))
  if kern == _lib.KERNEL_WEIGHT_ONLY_GEMM and (c != k or bits == 4) and m > 32:
    # the tiled GEMM for blockwise / int4 weights computes in one dtype throughout
    same = (scaler.dtype == x2.dtype and (zero_point is None or zero_point.dtype == x2.dtype) and
            dot_dtype == x2.dtype and out_dtype == x2.dtype and store_dtype == x2.dtype)
    if not same:
      kern = _lib.KERNEL_SKINNY_MFMA
  if kern == _lib.KERNEL_WEIGHT_ONLY_GEMM and x2.dtype == torch.float32:
    if store_dtype != torch.float32 or dot_dtype != torch.float32:
      kern = _lib.KERNEL_SKINNY_MFMA  # (f32 rows with a narrower stored result: no caller; the streaming kernel does it)
    else:
      # f32 rows: split into three bf16 parts in a workspace, then the bf16 GEMM with f32 accumulation throughout
      wk = w_tiled if w_tiled is not None else _tiled_weight(w, bits, layout)
      counters["wo_gemm"] += 1
      nbytes = lib.xla_amd_qmm_weight_only_gemm_f32_workspace_bytes(m, n, k)
      workspace = torch.empty(nbytes, dtype=torch.uint8, device=x2.device)
      x2 = x2.contiguous()
      _lib.check(
          lib.xla_amd_qmm_weight_only_gemm_f32(x2.data_ptr(), wk.data_ptr(), scaler.data_ptr(), _lib.ptr(zero_point),
                                               out.data_ptr(), workspace.data_ptr(), nbytes, m, n, k,
                                               _lib.dt(scaler.dtype), zp_dt, stream), "weight_only_gemm_f32")
      return out
  if kern == _lib.KERNEL_WEIGHT_ONLY_GEMM:
    wk = w_tiled if w_tiled is not None else _tiled_weight(w, bits, layout)
    counters["wo_gemm"] += 1
    nbytes = lib.xla_amd_qmm_weight_only_gemm_workspace_bytes(m, n, k, c, bits)
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=x2.device) if nbytes else None
    _lib.check(
        lib.xla_amd_qmm_weight_only_gemm(x2.data_ptr(), wk.data_ptr(), scaler.data_ptr(), _lib.ptr(zero_point),
                                         out.data_ptr(), _lib.ptr(workspace), nbytes, m, n, k, c, bits, *dts, stream),
        "weight_only_gemm")
  elif kern == _lib.KERNEL_SKINNY_MFMA:
    wk = w_tiled if w_tiled is not None else _tiled_weight(w, bits, layout)
    counters["skinny_mfma"] += 1
    _lib.check(
        lib.xla_amd_qmm_weight_only_skinny(x2.data_ptr(), wk.data_ptr(), scaler.data_ptr(),
                                           _lib.ptr(zero_point), out.data_ptr(), m, n, k, c, bits,
                                           *dts, stream), "weight_only_skinny")
  else:
    if w is None:
      raise RuntimeError("xla_amd: this shape runs the generic kernel, which reads the operator's weight layout")
    counters["generic"] += 1
    w = w.contiguous()
    _lib.check(
        lib.xla_amd_qmm_weight_only_generic(x2.data_ptr(), w.data_ptr(), scaler.data_ptr(),
                                            _lib.ptr(zero_point), out.data_ptr(), m, n, k, c, layout,
                                            *dts, stream), "weight_only_generic")
  return out


def _weight_only_gpu(x2, w, scaler, zero_point, block_size, int4_weight, out_dtype, dot_dtype=None,
                     store_dtype=None):
  n, k, c, layout = _weight_geometry(w, block_size)
  return _weight_only_launch(x2, w, None, n, k, c, layout, 4 if int4_weight else 8, scaler, zero_point,
                             out_dtype, dot_dtype, store_dtype)


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


def quantized_matmul_gpu(x, w, scaler, zero_point=None, block_size=-1, int4_weight=False,
                         quantize_activation=False, store_dtype=None):
  """`quantized_matmul` on ROCm tensors; `store_dtype` fuses a final `.to(store_dtype)` of the result."""
  block_size = -1 if block_size is None else block_size
  int4_weight = bool(int4_weight)
  quantize_activation = bool(quantize_activation)
  _check_args(x, w, scaler, zero_point, block_size, quantize_activation)
  if not (x.is_floating_point() and scaler.is_floating_point()):
    raise RuntimeError(f"xla_amd quantized_matmul: x and scaler must be floating point, got {x.dtype}, {scaler.dtype}")
  out_dtype = _result_dtype(x, scaler, quantize_activation)
  x2 = x.reshape(-1, x.shape[-1]).contiguous()
  scaler = scaler.contiguous()
  if zero_point is not None:
    zero_point = zero_point.contiguous()
  if quantize_activation:
    out = w8a8_linear_gpu(x2, w.contiguous(), scaler, zero_point, x_scale_dtype=x2.dtype, cvt_dtype=scaler.dtype,
                          mid_dtype=scaler.dtype, out_dtype=out_dtype)
    if store_dtype is not None and store_dtype != out_dtype:
      out = out.to(store_dtype)
  else:
    out = _weight_only_gpu(x2, w, scaler, zero_point, block_size, int4_weight, out_dtype, store_dtype=store_dtype)
  return out.reshape(*x.shape[:-1], out.shape[-1])


def w8a8_linear_gpu(x2, w, w_scale, zero_point, *, x_scale_dtype, cvt_dtype, mid_dtype, out_dtype, overflow=None,
                    block_m=0, block_n=0):
  """Per-token quantization + int8 GEMM in one library call; the quantized activations live in a workspace
  that is only needed during the call (the caching allocator hands the same block to the next call)."""
  lib = _lib.load()
  m, k = x2.shape
  n = w.shape[0]
  out = torch.empty((m, n), dtype=out_dtype, device=x2.device)
  if m == 0:
    return out
  nbytes = lib.xla_amd_qmm_w8a8_linear_workspace_bytes(m, n, k)
  workspace = torch.empty(nbytes, dtype=torch.uint8, device=x2.device)
  kern = lib.xla_amd_qmm_dispatch(m, n, k, k, 8, _lib.DT_F32, 1)
  counters["w8a8_mfma" if kern == _lib.KERNEL_W8A8_MFMA else "w8a8_generic"] += 1
  zp_dt = _lib.dt(zero_point.dtype) if zero_point is not None else _lib.DT_F32
  _lib.check(
      lib.xla_amd_qmm_w8a8_linear(x2.data_ptr(), w.data_ptr(), w_scale.data_ptr(), _lib.ptr(zero_point),
                                  out.data_ptr(), workspace.data_ptr(), nbytes, m, n, k, _lib.dt(x2.dtype),
                                  _lib.dt(w_scale.dtype), zp_dt, _lib.dt(x_scale_dtype), _lib.dt(cvt_dtype),
                                  _lib.dt(mid_dtype), _lib.dt(out_dtype), _OVERFLOW[overflow or _overflow_policy()],
                                  block_m, block_n, _lib.stream_of(x2)), "w8a8_linear")
  return out


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
  return quantized_matmul_gpu(x, w, scaler, zero_point, block_size, int4_weight, quantize_activation)


# ---- CPU tensors --------------------------------------------------------------------
# The reference documents calls with CPU tensors as its debugging path
# (docs/source/perf/quantized_ops.md:48-49) and its CI compares the device against it.
# The formulation below is this package's own; it rounds to the tensor dtype at exactly
# the points where the reference's op sequence (:139-183) materialises a tensor, and it
# applies the same explicit float -> int8 overflow policy as the GPU kernels, so that a
# CPU tensor and a GPU tensor give the same answer.


def _quantize_tensor(x: torch.Tensor, n_bits: int = 8, dim: int = -1, overflow: str = None):
  """Per-token symmetric quantizer (:56-73): every step is one torch op in x's dtype.

  Returns (int8 values, scale in x's dtype, kept dim).  A quotient that rounds to
  +-2^(n_bits-1) (the scale is itself rounded) follows the overflow policy; an
  all-zero row gives zeros with scale 0, a row with a NaN gives zeros with scale NaN.
  """
  qmax = (1 << (n_bits - 1)) - 1
  scale = x.abs().amax(dim=dim, keepdim=True) / qmax
  r = torch.nan_to_num((x / scale).round().float(), nan=0.0, posinf=0.0, neginf=0.0)
  policy = overflow or _overflow_policy()
  if policy == "saturate":
    q = r.clamp(-qmax - 1, qmax).to(torch.int8)
  else:
    q = r.to(torch.int32).to(torch.int8)  # modulo 256, what torch's own cast does
  return q, scale.to(x.dtype)


def _cpu_per_channel(x2, w, scaler, zero_point, quantize_activation):
  if quantize_activation:
    x_q, x_scale = _quantize_tensor(x2)
    acc = torch.mm(x_q.to(torch.int32), w.to(torch.int32).t())  # exact
    out = acc * scaler  # integer tensor times float tensor: converted to scaler's dtype first
    if zero_point is not None:
      row_sum = x_q.to(torch.int32).sum(dim=-1, keepdim=True)
      out.sub_(row_sum * zero_point)
    return out * x_scale
  out = torch.mm(x2, w.to(x2.dtype).t()) * scaler
  if zero_point is not None:
    out.sub_(x2.sum(dim=-1, keepdim=True) * zero_point)
  return out


def _cpu_blockwise(x2, w, scaler, zero_point, block_size):
  m = x2.shape[0]
  s, c, n = w.shape
  xb = x2.reshape(m, s, c)
  # per block: [s, m, c] @ [s, c, n] -> [s, m, n], rounded to x's dtype
  p = torch.bmm(xb.transpose(0, 1), w.to(x2.dtype))
  # sum over blocks of scaler[s, n] * p[s, m, n] as one contraction per channel (a single rounding)
  out = torch.bmm(p.permute(2, 1, 0), scaler.t().unsqueeze(-1)).squeeze(-1).t()
  if zero_point is not None:
    out = out.contiguous()
    out.sub_(torch.mm(xb.sum(dim=-1), zero_point))
  return out


@impl(XLA_LIB, "quantized_matmul", "CPU")
def quantized_matmul(x: torch.Tensor,
                     w: torch.Tensor,
                     scaler: torch.Tensor,
                     zero_point: torch.Tensor = None,
                     block_size: int = -1,
                     int4_weight: bool = False,
                     quantize_activation: bool = False):
  """CPU tensors (the reference's debugging path, :139-183); `int4_weight` only concerns storage."""
  block_size = -1 if block_size is None else block_size
  quantize_activation = bool(quantize_activation)
  _check_args(x, w, scaler, zero_point, block_size, quantize_activation)
  x2 = x.reshape(-1, x.shape[-1])
  if block_size == -1:
    out = _cpu_per_channel(x2, w, scaler, zero_point, quantize_activation)
  else:
    out = _cpu_blockwise(x2, w, scaler, zero_point, block_size)
  return out.reshape(*x.shape[:-1], out.shape[-1])


@impl(XLA_LIB, "quantized_matmul", "Meta")
def quantized_matmul_meta(x, w, scaler, zero_point=None, block_size=-1, int4_weight=False,
                          quantize_activation=False):
  block_size = -1 if block_size is None else block_size
  _check_args(x, w, scaler, zero_point, block_size, bool(quantize_activation))
  n = w.shape[0] if block_size == -1 else w.shape[-1]
  return torch.empty(*x.shape[:-1], n, dtype=_result_dtype(x, scaler, bool(quantize_activation)),
                     device=x.device)


# ---- weight-only matmul on a tiled weight alone ----------------------------------------
# Not part of the reference's interface: the operator a module calls once it keeps only the
# tiled form of its weight on the device (XlaQuantizedLinear.prepare(release_weight=True)).
XLA_AMD_LIB = torch.library.Library("xla_amd", "DEF")
XLA_AMD_LIB.define(
    "weight_only_tiled(Tensor x, Tensor w_tiled, Tensor scale, Tensor? zero_point, int out_features, "
    "int block_size, bool int4_weight) -> Tensor")


@impl(XLA_AMD_LIB, "weight_only_tiled", "CUDA")
def weight_only_tiled_rocm(x, w_tiled, scaler, zero_point, out_features, block_size, int4_weight):
  if not (x.is_floating_point() and scaler.is_floating_point()):
    raise RuntimeError(f"xla_amd weight_only_tiled: x and scaler must be floating point, got {x.dtype}, {scaler.dtype}")
  k = x.shape[-1]
  c = k if block_size == -1 else block_size
  bits = 4 if int4_weight else 8
  need = _lib.load().xla_amd_qmm_tiled_bytes(out_features, k, c, bits)
  assert need > 0 and w_tiled.numel() * w_tiled.element_size() == need, (
      f"tiled weight of {w_tiled.numel() * w_tiled.element_size()} bytes does not belong to a "
      f"[{out_features}, {k}] weight of {bits} bits")
  x2 = x.reshape(-1, k).contiguous()
  out = _weight_only_launch(x2, None, w_tiled, out_features, k, c, _lib.W_NK if c == k else _lib.W_SCN, bits,
                            scaler.contiguous(), None if zero_point is None else zero_point.contiguous(),
                            _result_dtype(x, scaler, False), None, None)
  return out.reshape(*x.shape[:-1], out_features)


@impl(XLA_AMD_LIB, "weight_only_tiled", "Meta")
def weight_only_tiled_meta(x, w_tiled, scaler, zero_point, out_features, block_size, int4_weight):
  return torch.empty(*x.shape[:-1], out_features, dtype=_result_dtype(x, scaler, False), device=x.device)


class XlaQuantizedLinear(torch.nn.Module):
  """Linear layer over a quantized weight (xla_quantized_matmul.py:186-243).

  State-dict keys and buffer shapes are the reference's: `weight` int8
  [out, in], `weight_scaler` [out], and `zero_point` [out] unless symmetric;
  `load_quantized_weight` replaces them (blockwise weights are 3-D).

  On a ROCm GPU, `prepare()` makes the tiled copy of the weight that the
  streaming kernel reads ahead of the first forward, and can drop the
  reference-layout buffer from device memory; `state_dict()` still returns it.
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
    # tiled copy owned by the module (set by prepare(); moves with .to()/.cuda(), never saved)
    self.register_buffer('_weight_tiled', None, persistent=False)
    self._released_shape = None  # shape of `weight` while only the tiled form is kept
    self._tiled_from = None      # (version, storage pointer) of `weight` when the tiled copy was made
    self._register_state_dict_hook(XlaQuantizedLinear._restore_weight_in_state_dict)

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
    self._weight_tiled = None
    self._released_shape = None

  # -- device-side weight layout ----------------------------------------------------------
  def prepare(self, release_weight: bool = False) -> bool:
    """Makes the tiled copy of the weight now instead of on the first forward.

    Needed before a HIP-graph capture (the lazy copy must not be recorded), and
    after writes to `weight` that torch's version counter cannot see
    (`weight.data.copy_`).  Returns False when this layer does not use a tiled
    copy (CPU tensors, activation quantization, shapes of the generic kernel).
    With `release_weight=True` the reference-layout `weight` buffer is freed on
    the device and only the tiled form is kept (half the weight memory);
    `state_dict()` rebuilds `weight` from it, `load_state_dict()` brings the
    buffer back (call `prepare` again afterwards).
    """
    if self._released_shape is not None:
      return True
    w = self.weight
    if not w.is_cuda or self.quantize_activation:
      return False
    n, k, c, layout = _weight_geometry(w, self.block_size)
    bits = 4 if self.int4_weight else 8
    if _lib.load().xla_amd_qmm_dispatch(1, n, k, c, bits, _lib.DT_BF16, 0) != _lib.KERNEL_SKINNY_MFMA:
      return False
    invalidate_weight_cache(w)
    self._weight_tiled = _tiled_weight(w, bits, layout)
    self._tiled_from = (_version_of(w), w.data_ptr())
    if release_weight:
      invalidate_weight_cache(w)  # the module's own reference keeps the copy alive
      self._released_shape = tuple(w.shape)
      self.weight = torch.empty(0, dtype=torch.int8, device=w.device)
    return True

  def _rebuilt_weight(self):
    shape = self._released_shape
    if len(shape) == 2:
      (n, k), s, c, layout = shape, 1, shape[1], _lib.W_NK
    else:
      (s, c, n), layout = shape, _lib.W_SCN
    w = torch.empty(shape, dtype=torch.int8, device=self._weight_tiled.device)
    _lib.check(
        _lib.load().xla_amd_qmm_untile_weight(self._weight_tiled.data_ptr(), w.data_ptr(), s, c, n, layout,
                                              4 if self.int4_weight else 8, _lib.stream_of(w)), "untile_weight")
    return w

  @staticmethod
  def _restore_weight_in_state_dict(module, state_dict, prefix, local_metadata):
    if module._released_shape is not None:
      state_dict[prefix + "weight"] = module._rebuilt_weight()
    return state_dict

  def _restore_weight(self):
    """Brings the operator-layout `weight` back from the tiled form (undoes `release_weight`)."""
    if self._released_shape is not None:
      self.weight = self._rebuilt_weight()
      self._released_shape = None
      self._weight_tiled = None

  def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
    # A dict without this layer's `weight` (a partial or scaler-only checkpoint, strict=False) leaves the
    # weight as it is, tiled copy included.  A dict with one is copied into a buffer that already holds the
    # current values (rebuilt from the tiled form when that was all the module kept), so that a load which
    # fails half-way - a shape mismatch is only reported, not copied - still leaves a valid weight.
    if prefix + "weight" in state_dict:
      self._restore_weight()
      self._weight_tiled = None
    return super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

  def _apply(self, fn, recurse=True):
    # .cpu() / .to(other device) of a module that kept only the tiled form: the operator layout can only be
    # rebuilt where the tiled copy lives, so it is rebuilt before the move (and the module needs a new
    # prepare() afterwards).  Casts and moves that stay on the device keep the released state.
    if self._released_shape is not None:
      here = self._weight_tiled.device
      if fn(torch.empty(0, dtype=torch.uint8, device=here)).device != here:
        self._restore_weight()
    return super()._apply(fn, recurse)

  def _tiled_is_current(self):
    if self._weight_tiled is None:
      return False
    if self._released_shape is not None:
      return True
    # `weight` is still there: the copy stands while torch has seen no write to it (an in-place
    # operation or a new tensor sends the call back to the operator, which re-tiles)
    return self._tiled_from == (_version_of(self.weight), self.weight.data_ptr())

  def forward(self, x):
    if x.is_cuda and self._tiled_is_current():
      return torch.ops.xla_amd.weight_only_tiled(x, self._weight_tiled, self.weight_scaler, self.zero_point,
                                                 self.output_dim, self.block_size, self.int4_weight)
    return torch.ops.xla.quantized_matmul(
        x,
        self.weight,
        self.weight_scaler,
        self.zero_point,
        block_size=self.block_size,
        int4_weight=self.int4_weight,
        quantize_activation=self.quantize_activation)
