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

  x [bs, in] float, w int8 [out, in], scalar [out].  As in the reference
  (:1088-1106) the block sizes always come from the tuned table, whatever the
  caller passed: a shape in the table runs the dedicated kernel
  (hip_kernels/quantized_matmul_kernel.py), any other shape takes the
  `quantized_matmul` route, cast to x.dtype, with the reference's warning.
  """
  from xla_amd.experimental.hip_kernels.quantized_matmul_kernel import (
      quantized_matmul_int8 as kernel,
      get_tuned_block_sizes,
      TUNED_BLOCK_SIZES,
  )
  bs, n_in_features = x.shape
  n_out_features, _ = w.shape
  if x.dtype not in _DTYPE_NAME:
    raise RuntimeError(f"xla_amd quantized_matmul_int8: unsupported activation dtype {x.dtype}")
  batch_block_size, out_block_size, in_block_size = get_tuned_block_sizes(
      TUNED_BLOCK_SIZES, bs, n_out_features, n_in_features, _DTYPE_NAME[x.dtype], quantize_activation)
  if batch_block_size is not None and out_block_size is not None and in_block_size is not None:
    return kernel(x, w, scalar, zero_point, quant_block_size, quantize_activation,
                  batch_block_size=batch_block_size, out_block_size=out_block_size,
                  in_block_size=in_block_size)
  logging.warning(
      f"Couldn't find w8a8 quantized matmul kernel block sizes for {bs=}, {n_out_features=}, {n_in_features=}, {_DTYPE_NAME[x.dtype]=}, {quantize_activation=}, falling back to XLA quantized matmul kernel."
  )
  return _qmm.quantized_matmul_gpu(x, w, scalar, quantize_activation=quantize_activation, store_dtype=x.dtype)


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
