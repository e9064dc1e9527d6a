"""`torch.ops.xla.quantized_matmul_int8` for ROCm tensors.

Drop-in for the wrapper and operator in torch_xla/experimental/custom_kernel.py
(:1066-1106, :1742-1782): a shape table chooses the launch configuration of the
dedicated int8 kernel; a shape that is not in the table takes the
`quantized_matmul` route and is cast to x's dtype, with the same warning.
"""
import logging
import warnings

import torch
from torch.library import impl

from xla_amd import _lib
from xla_amd.core.xla_model import XLA_LIB
from xla_amd.experimental import xla_quantized_matmul as _qmm

XLA_LIB.define(
    "quantized_matmul_int8(Tensor x, Tensor w, Tensor scalar, Tensor? zero_point=None, Tensor? quant_block_size=None, bool quantize_activation=False, int? batch_block_size=None, int? out_block_size=None, int? in_block_size=None) -> Tensor",
)

_DTYPE_NAME = {torch.bfloat16: "bfloat16", torch.float16: "float16", torch.float32: "float32"}


def quantized_matmul_int8(
    x: torch.Tensor,
    w: torch.Tensor,
    scalar: torch.Tensor,
    zero_point: torch.Tensor | None = None,
    quant_block_size: torch.Tensor | None = None,
    quantize_activation: bool = False,
    batch_block_size: int | None = None,
    out_block_size: int | None = None,
    in_block_size: int | None = None,
) -> torch.Tensor:
  """int8 weight (and optionally int8 activation) matmul, result in x.dtype.

  x [bs, in] float, w int8 [out, in], scalar [out].  The arithmetic is that of
  the reference's dedicated kernel (pallas_kernels/quantized_matmul_kernel.py:
  88-124, 199-221): row abs-max and activation scale in x.dtype, weight scale
  and epilogue in float32, int32 accumulation, one final cast to x.dtype.
  """
  from xla_amd.experimental.hip_kernels.quantized_matmul_kernel import (
      get_tuned_block_sizes,
      TUNED_BLOCK_SIZES,
  )
  assert zero_point is None, "Not implemented: zero_point is not supported."
  assert quant_block_size is None, "Not implemented: quant_block_size is not supported."
  bs, n_in_features = x.shape
  n_out_features, _ = w.shape
  if x.dtype not in _DTYPE_NAME:
    raise RuntimeError(f"xla_amd quantized_matmul_int8: unsupported activation dtype {x.dtype}")
  if batch_block_size is None or out_block_size is None or in_block_size is None:
    batch_block_size, out_block_size, in_block_size = get_tuned_block_sizes(
        TUNED_BLOCK_SIZES, bs, n_out_features, n_in_features, _DTYPE_NAME[x.dtype],
        quantize_activation)
  if batch_block_size is not None and out_block_size is not None and in_block_size is not None:
    x2 = x.contiguous()
    w = w.contiguous()
    scalar32 = scalar.to(torch.float32).contiguous()
    if quantize_activation:
      x_q, x_scale, _ = _qmm.quantize_per_token_gpu(x2, scale_dtype=torch.float32)
      out, _ = _qmm.w8a8_gemm_gpu(x_q, w, x_scale, scalar32, None, None, cvt_dtype=torch.float32,
                                  mid_dtype=torch.float32, out_dtype=x.dtype,
                                  block_m=batch_block_size, block_n=out_block_size)
      return out
    # weight-only: float32 accumulation, float32 scale, one cast to x.dtype
    return _qmm._weight_only_gpu(x2, w, scalar32, None, -1, False,
                                 torch.promote_types(x.dtype, torch.float32)).to(x.dtype)
  logging.warning(
      f"Couldn't find w8a8 quantized matmul kernel block sizes for {bs=}, {n_out_features=}, {n_in_features=}, {_DTYPE_NAME[x.dtype]=}, {quantize_activation=}, falling back to XLA quantized matmul kernel."
  )
  return _qmm.quantized_matmul_rocm(x, w, scalar, quantize_activation=quantize_activation).to(x.dtype)


@impl(XLA_LIB, "quantized_matmul_int8", "CUDA")
def quantized_matmul_int8_rocm(
    x: torch.Tensor,
    w: torch.Tensor,
    scalar: torch.Tensor,
    zero_point: torch.Tensor | None = None,
    quant_block_size: torch.Tensor | None = None,
    quantize_activation: bool = False,
    batch_block_size: int | None = None,
    out_block_size: int | None = None,
    in_block_size: int | None = None,
) -> torch.Tensor:
  return quantized_matmul_int8(x, w, scalar, zero_point, quant_block_size, quantize_activation,
                               batch_block_size, out_block_size, in_block_size)


@impl(XLA_LIB, "quantized_matmul_int8", "CompositeExplicitAutograd")
def quantized_matmul_int8_non_gpu(
    x: torch.Tensor,
    w: torch.Tensor,
    scalar: torch.Tensor,
    zero_point: torch.Tensor | None = None,
    quant_block_size: torch.Tensor | None = None,
    quantize_activation: bool = False,
    batch_block_size: int | None = None,
    out_block_size: int | None = None,
    in_block_size: int | None = None,
) -> torch.Tensor:
  # Fake/meta tensors only need the output's shape and dtype; like the
  # reference (:1764-1782) any other non-device tensor gets a warning and an
  # uninitialised result of the right shape.
  if x.device != torch.device("meta"):
    warnings.warn('xla_amd quantized_matmul_int8 should only be applied to tensors on a ROCm GPU')
  return torch.empty(x.shape[0], w.shape[0], device=x.device, dtype=x.dtype)
