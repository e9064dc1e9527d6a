"""CPU restatement of PyTorch/XLA's quantized matmul.  TEST INFRASTRUCTURE ONLY.

This file is the checker for the HIP kernels; the shipped package never
imports it.  It restates, op for op and in the reference's order and dtypes,
what the reference executes for CPU tensors (the implementation its own CI
compares the XLA device against), so every intermediate is rounded to the
dtype the reference rounds it to.

Reference statements followed (paths relative to the pytorch/xla tree):
  quantize_tensor            torch_xla/experimental/xla_quantized_matmul.py:56-73
  quantized_matmul           torch_xla/experimental/xla_quantized_matmul.py:139-183
                             (device variant :76-136 differs only in where
                             dtypes are converted, noted inline)
  pallas_quantize_array      torch_xla/experimental/pallas_kernels/quantized_matmul_kernel.py:10-18,199-200
  quantized_matmul_int8      torch_xla/experimental/pallas_kernels/quantized_matmul_kernel.py:88-124,171-310
                             and the wrapper torch_xla/experimental/custom_kernel.py:1066-1106
  int32_accumulators         csrc/ops/dot_general.cpp:16-37 (s8 x s8 -> s32 contraction)

How each function is pinned (tests/test_oracle_*.py):
  quantize_tensor        all 65536 bf16 bit patterns against an independent
                         exact-rational model (oracle/bitexact_model.py) plus
                         invariants (odd symmetry, |q| <= 127 unless the 127.5
                         band is hit, argmax maps to +-127/128).
  int32_accumulators     int64 numpy matmul; the reference's own exactness
                         case (test/quantized_ops/test_dot_general.py:44-57).
  quantized_matmul       closed forms (scale==1, w==1 -> row sums, one-hot x),
                         the reference's fake-quant identity
                         (test/quantized_ops/test_quantized_matmul.py:210-218),
                         blockwise with S==1 equals per-channel, fp64 dense
                         matmul on dequantized weights within the reference's
                         thresholds, and the committed tests/golden fixtures.
  quantized_matmul_int8  same integer model + f32 epilogue closed form; the
                         float branch (quantize_activation=False) against
                         bf16(f64 dot * scale) within one ulp, w == 1 (row sums)
                         and one-hot x; the reference pins the kernel only on
                         TPU, only with quantize_activation=True, within
                         rel-err 2e-2.
Parity unpinned (cannot be decided offline, see the policy argument):
  float->int8 conversion of a rounded value of +-128 on the PJRT CPU device
  (`overflow`), and whether XLA-CPU keeps bf16 round trips between the
  elementwise ops of the quantizer.
  quantized_matmul_int8(quantize_activation=False) with bf16/f16 x: the Pallas
  kernel calls lax.dot_general on (x, int8 w) without preferred_element_type
  (quantized_matmul_kernel.py:108-112); whether each in-block dot comes back in
  float32 or rounded to x's dtype is decided by jax 0.8.0.dev20251001 / Mosaic,
  which are not part of the reference tree.  This restatement keeps the float32
  accumulator the kernel declares (acc_dtype, :246) over all of K.
"""
import torch
import torch.nn.functional as F

INT8_MIN, INT8_MAX = -128, 127


def _to_int8(r: torch.Tensor, overflow: str) -> torch.Tensor:
  """float -> int8 of an already rounded tensor.

  'wrap'     : torch's CPU cast (what `.to(torch.int8)` does in eager mode).
  'saturate' : clamp to [-128,127] (XLA ConvertElementType, TPU behaviour).
  NaN (an all-zero row gives 0/0) maps to 0 under both policies.
  """
  r = torch.nan_to_num(r.float(), nan=0.0, posinf=0.0, neginf=0.0)
  if overflow == "saturate":
    return r.clamp(INT8_MIN, INT8_MAX).to(torch.int8)
  if overflow == "wrap":
    return r.to(torch.int32).to(torch.int8)
  raise ValueError(overflow)


def quantize_tensor(x: torch.Tensor, n_bits: int = 8, dim: int = -1, overflow: str = "saturate"):
  """xla_quantized_matmul.py:56-73.  All arithmetic in x.dtype, op by op."""
  max_val = torch.amax(torch.abs(x), dim=dim, keepdim=True)
  int_max = 2**(n_bits - 1) - 1
  scale = max_val / int_max
  r = torch.round(x / scale)
  x_int = _to_int8(r, overflow)
  # (an all-zero row gives scale 0 and quotients 0/0 -> 0; a row that holds a NaN keeps its NaN scale)
  return x_int, scale.to(x.dtype)


def int32_accumulators(x_int: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
  """s8 x s8 -> s32 contraction over the last dims (dot_general.cpp:16-37)."""
  return F.linear(x_int.to(torch.int32), w.to(torch.int32))


def quantized_matmul(x, w, scaler, zero_point=None, block_size=-1, int4_weight=False,
                     quantize_activation=False, overflow="saturate"):
  """xla_quantized_matmul.py:139-183 (int4_weight only changes storage, :101-103)."""
  if block_size == -1:
    w = w.to(x.dtype)
    if quantize_activation:
      x, x_scale = quantize_tensor(x, overflow=overflow)
      x = x.to(torch.int32)
      w = w.to(torch.int32)
    out = F.linear(x, w)
    out = out * scaler
  else:
    assert not quantize_activation
    x = x.reshape(*x.shape[:-1], x.shape[-1] // block_size, block_size)
    w = w.to(x.dtype)
    out = torch.einsum('scn,...sc->...sn', w, x)
    out = torch.einsum('sn,...sn->...n', scaler, out)
  if zero_point is not None:
    if block_size == -1:
      zp_out = torch.einsum("...c,z->...z", x, zero_point)
    else:
      zp_out = x.sum(dim=-1)
      zp_out = torch.matmul(zp_out, zero_point)
    out -= zp_out
  if quantize_activation:
    out = out * x_scale
  return out


def pallas_quantize_array(x: torch.Tensor, overflow: str = "saturate"):
  """quantized_matmul_kernel.py:199-200 (row abs-max in x.dtype, outside the
  kernel) and :10-18 (scale and quotient in x.dtype; scale returned as f32)."""
  x_abs_max = torch.amax(torch.abs(x), dim=-1, keepdim=True)
  scale = x_abs_max / 127
  r = torch.round(x / scale)
  x_int = _to_int8(r, overflow)
  return x_int, scale.to(torch.float32)


def quantized_matmul_int8(x, w, scalar, quantize_activation=False, overflow="saturate"):
  """Pallas kernel semantics (quantized_matmul_kernel.py:88-124,219-221,297,310):
  f32 weight scale, int32 (W8A8) or f32 (weight-only) accumulation,
  `acc *= w_scale; acc *= x_scale; out = acc.astype(x.dtype)`.
  Tile sizes only change the padding, never the value of an output element."""
  scalar = scalar.to(torch.float32)
  if quantize_activation:
    x_q, x_scale = pallas_quantize_array(x, overflow=overflow)
    acc = int32_accumulators(x_q, w).to(torch.float32)
    acc = acc * scalar
    acc = acc * x_scale
  else:
    acc = F.linear(x.to(torch.float32), w.to(torch.float32))
    acc = acc * scalar
  return acc.to(x.dtype)


def quantized_matmul_int8_fallback(x, w, scalar, quantize_activation=False, overflow="saturate"):
  """Table-miss route of the wrapper (custom_kernel.py:1101-1106)."""
  return quantized_matmul(
      x, w, scalar, quantize_activation=quantize_activation, overflow=overflow).to(x.dtype)
