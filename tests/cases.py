"""Seeded synthetic inputs of the benchmark configurations (CPU tensors)."""
import torch

from xla_amd.quantization import quantize_weight_rtn


def gen(seed):
  return torch.Generator().manual_seed(seed)


def per_channel_int8(m, n, k, x_dtype, scale_dtype, seed=0, std=0.02):
  """x [m,k] ~ N(0,1); w = per-row absmax/127 RTN of an N(0,std) weight [n,k]."""
  g = gen(seed)
  x = torch.randn(m, k, generator=g).to(x_dtype)
  w_fp = torch.randn(n, k, generator=g) * std
  w_int, scale, _ = quantize_weight_rtn(w_fp, 8, -1, True, scale_dtype)
  return x, w_int, scale, w_fp


def uniform_int8(m, n, k, x_dtype, scale_dtype, seed=0):
  """Config 1: w uniform in [-127,127], scaler from an independent N(0,0.02) weight."""
  g = gen(seed)
  x = torch.randn(m, k, generator=g).to(x_dtype)
  w_int = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int32).to(torch.int8)
  w_fp = torch.randn(n, k, generator=g) * 0.02
  scale = (w_fp.abs().amax(1) / 127).to(scale_dtype)
  return x, w_int, scale


def blockwise(m, n, k, block, n_bits, x_dtype, symmetric=False, seed=0, std=0.02):
  """Config 3: blockwise (a)symmetric RTN; w [k/block, block, n], scale/zp [k/block, n]."""
  g = gen(seed)
  x = torch.randn(m, k, generator=g).to(x_dtype)
  w_fp = torch.randn(n, k, generator=g) * std
  w_int, scale, zp = quantize_weight_rtn(w_fp, n_bits, block, symmetric, x_dtype)
  return x, w_int, scale, zp, w_fp


def outlier_activations(m, k, x_dtype, seed=1234, frac=0.01, factor=20.0):
  """Config 4 activations: N(0,1) with 1% of the channels scaled by 20."""
  g = gen(seed)
  x = torch.randn(m, k, generator=g)
  idx = torch.randperm(k, generator=g)[:max(1, int(round(k * frac)))]
  x[:, idx] *= factor
  return x.to(x_dtype)


def rel_l2(a, b):
  a = a.double()
  b = b.double()
  return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def within_tolerance(actual, expected):
  """Output tolerance of the floating-point paths: max-abs-err <= 1e-2 * ||row||_inf for every row, or rel-L2 <= 2e-3."""
  a, e = actual.double(), expected.double()
  row_ok = ((a - e).abs().amax(-1) <= 1e-2 * e.abs().amax(-1)).all().item()
  return row_ok or rel_l2(a, e) <= 2e-3
