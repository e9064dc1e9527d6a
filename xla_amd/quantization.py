"""Round-to-nearest weight quantizer and module swap for XlaQuantizedLinear.

Produces weights in the layouts `torch.ops.xla.quantized_matmul` takes:
per-channel `w_int [out, in]`, `scaler [out]`, `zero_point [out]`; blockwise
`w_int [in/block, block, out]`, `scaler [in/block, out]`, `zero_point
[in/block, out]`.  The zero point is returned in real units (integer zero
point times scale), the convention of the reference's own test helper
(test/quantized_ops/test_quantized_matmul.py:25-74) and of the operator
(xla_quantized_matmul.py:125-133).  The swap utility follows the usage shown in
docs/source/perf/quantized_ops.md:92-109.
"""
import torch

from xla_amd.experimental.xla_quantized_matmul import XlaQuantizedLinear


def quantize_weight_rtn(w_fp: torch.Tensor, n_bits: int = 8, block_size: int = -1,
                        symmetric: bool = True, scale_dtype=None):
  """Round-to-nearest quantization of a linear weight `w_fp [out, in]`.

  symmetric : scale = absmax / (2^(n_bits-1) - 1), w_int = clamp(round(w/scale), -qmax, qmax).
  asymmetric: scale = (max - min) / (2^n_bits - 1), zp_int = qmin - round(min/scale),
              w_int = clamp(round(w/scale) + zp_int, qmin, qmax); dequantization is
              w_int * scale - zero_point with zero_point = zp_int * scale.
  Statistics are per output channel, or per (output channel, block of
  `block_size` input features).
  Returns (w_int int8, scaler, zero_point or None) in the operator's layouts.
  """
  assert w_fp.dim() == 2
  out_dim, in_dim = w_fp.shape
  w = w_fp.detach().to(torch.float32)
  if block_size != -1:
    assert in_dim % block_size == 0
    w = w.reshape(out_dim * in_dim // block_size, block_size)
  qmin, qmax = -2**(n_bits - 1), 2**(n_bits - 1) - 1
  mn, mx = torch.aminmax(w, dim=1)
  if symmetric:
    scale = torch.maximum(mx.abs(), mn.abs()) / qmax
    scale = torch.clamp(scale, min=1e-10)
    w_int = torch.clamp(torch.round(w / scale[:, None]), -qmax, qmax)
    zp = None
  else:
    mn = torch.minimum(mn, torch.zeros_like(mn))
    mx = torch.maximum(mx, torch.zeros_like(mx))
    scale = torch.clamp((mx - mn) / (qmax - qmin), min=1e-10)
    zp_int = torch.clamp(qmin - torch.round(mn / scale), qmin, qmax)
    w_int = torch.clamp(torch.round(w / scale[:, None]) + zp_int[:, None], qmin, qmax)
    zp = zp_int * scale
  w_int = w_int.to(torch.int8)
  scale_dtype = scale_dtype or w_fp.dtype
  if block_size != -1:
    s = in_dim // block_size
    w_int = w_int.reshape(out_dim, s, block_size).permute(1, 2, 0).contiguous()
    scale = scale.reshape(out_dim, s).permute(1, 0).contiguous()
    if zp is not None:
      zp = zp.reshape(out_dim, s).permute(1, 0).contiguous()
  scale = scale.to(scale_dtype)
  if zp is not None:
    zp = zp.to(scale_dtype)
  return w_int, scale, zp


def quantize_linear(linear: torch.nn.Linear, n_bits: int = 8, block_size: int = -1,
                    symmetric: bool = True, quantize_activation: bool = False,
                    scale_dtype=None) -> XlaQuantizedLinear:
  """XlaQuantizedLinear holding the RTN-quantized weight of `linear` (bias-free)."""
  assert linear.bias is None, "XlaQuantizedLinear has no bias"
  w_int, scale, zp = quantize_weight_rtn(linear.weight.data, n_bits, block_size, symmetric,
                                         scale_dtype)
  q = XlaQuantizedLinear(linear.in_features, linear.out_features, is_symmetric=symmetric,
                         block_size=block_size, int4_weight=(n_bits == 4),
                         quantize_activation=quantize_activation)
  q.load_quantized_weight(w_int, scale, zp)
  return q


def replace_linear_with_quantized(module: torch.nn.Module, predicate=None, **kwargs) -> torch.nn.Module:
  """Replaces every bias-free nn.Linear under `module` (for which `predicate(name,
  layer)` holds, if given) by its quantized counterpart, in place."""
  for name, child in list(module.named_children()):
    if isinstance(child, torch.nn.Linear) and child.bias is None and (predicate is None or predicate(name, child)):
      setattr(module, name, quantize_linear(child, **kwargs))
    else:
      replace_linear_with_quantized(child, predicate, **kwargs)
  return module


def fuse_quantized_linears(linears) -> XlaQuantizedLinear:
  """One XlaQuantizedLinear that computes several of them side by side.

  The layers must read the same input (same in_features) and share their
  quantization settings; their output channels are concatenated in the order
  given, so `fused(x).split([l.output_dim for l in linears], dim=-1)` equals
  `[l(x) for l in linears]` exactly (every output channel keeps its own weight
  row, scale and zero point).  Meant for the q/k/v and gate/up pairs of a
  decoder layer: one launch streams all the weights, instead of one launch
  (with its fixed cost) per projection.
  """
  linears = list(linears)
  first = linears[0]
  for l in linears[1:]:
    assert (l.input_dim, l.is_symmetric, l.block_size, l.int4_weight, l.quantize_activation) == \
        (first.input_dim, first.is_symmetric, first.block_size, first.int4_weight, first.quantize_activation), \
        "fused layers must share input size and quantization settings"
    assert l.weight.dtype == first.weight.dtype and l.weight_scaler.dtype == first.weight_scaler.dtype
  out_dim = sum(l.output_dim for l in linears)
  fused = XlaQuantizedLinear(first.input_dim, out_dim, first.is_symmetric, first.block_size, first.int4_weight,
                             first.quantize_activation)
  cat_dim = 0 if first.block_size == -1 else -1  # per-channel [out, in] / [out]; blockwise [.., out]
  weight = torch.cat([l.weight for l in linears], dim=cat_dim).contiguous()
  scaler = torch.cat([l.weight_scaler for l in linears], dim=cat_dim).contiguous()
  zero_point = None
  if first.zero_point is not None:
    zero_point = torch.cat([l.zero_point for l in linears], dim=cat_dim).contiguous()
  fused.load_quantized_weight(weight, scaler, zero_point)
  return fused
