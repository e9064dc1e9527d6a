"""Independent exact models used to pin the oracle.  TEST INFRASTRUCTURE ONLY.

Nothing here shares code with oracle/quantized_matmul_oracle.py: bf16 and f16
are modelled with integer/float64 arithmetic in numpy and an explicit
round-to-nearest-even, so that a mistake in the torch restatement (a rounding
done in the wrong dtype, a missing round, a wrong tie rule) shows up as a
mismatch.  Mathematics restated: IEEE-754 division and RNE rounding, the
quantizer formula of torch_xla/experimental/xla_quantized_matmul.py:69-73 and
the s8 x s8 -> s32 contraction of csrc/ops/dot_general.cpp:16-37.
"""
import numpy as np

_FMT = {  # name -> (significand bits incl. hidden one, min normal exponent, max exponent)
    "bf16": (8, -126, 127),
    "f16": (11, -14, 15),
    "f32": (24, -126, 127),
}


def round_to_format(v, fmt: str):
  """RNE-round float64 values to the grid of `fmt`, returned as float64.

  Exact as long as v itself is exact in float64 (all uses here: quotients and
  products of numbers with <= 24 significant bits are correctly rounded by
  float64 far below the target's half-ulp, so no double-rounding can occur
  unless the exact value is itself a tie, which float64 then represents).
  """
  p, emin, emax = _FMT[fmt]
  v = np.asarray(v, dtype=np.float64)
  out = np.zeros_like(v)
  fin = np.isfinite(v) & (v != 0)
  m, e = np.frexp(v[fin])  # v = m * 2**e, 0.5 <= |m| < 1
  e_eff = np.maximum(e, emin + 1)  # subnormal range shares the exponent of the smallest normal
  q = np.ldexp(1.0, (e_eff - p).astype(np.int64))  # one ulp: 2**(e_eff - p)
  r = np.rint(v[fin] / q) * q  # np.rint is half-to-even; v/q is exact (power of two)
  big = np.ldexp(2.0 - np.ldexp(1.0, 1 - p), emax)
  r = np.where(np.abs(r) > big, np.sign(r) * np.inf, r)
  out[fin] = r
  out[~np.isfinite(v)] = v[~np.isfinite(v)]
  return out


def bf16_bits_to_f64(bits):
  bits = np.asarray(bits, dtype=np.uint32)
  return (bits << 16).astype(np.uint32).view(np.float32).astype(np.float64)


def f64_to_bf16_bits(v):
  """float64 values already on the bf16 grid -> their 16-bit patterns."""
  f = np.asarray(v, dtype=np.float64).astype(np.float32)
  return (f.view(np.uint32) >> 16).astype(np.uint16)


def quantize_rows(x, fmt: str, overflow: str = "saturate"):
  """Exact model of `_quantize_tensor` for a 2-D array of values on `fmt`'s grid.

  max = amax(|x|) (exact); scale = RN_fmt(max / 127); r = RN_fmt(x / scale);
  q = round_half_even(r) -> int8 by `overflow`.  Returns (q int64 array with
  int8 values, scale float64 on the grid, r_rounded float64 before the cast).
  """
  x = np.asarray(x, dtype=np.float64)
  mx = np.max(np.abs(x), axis=-1, keepdims=True)
  scale = round_to_format(mx / 127.0, fmt)
  with np.errstate(divide="ignore", invalid="ignore"):
    r = round_to_format(x / scale, fmt)
  r = np.where(np.isfinite(r), r, 0.0)
  rr = np.rint(r)
  if overflow == "saturate":
    q = np.clip(rr, -128, 127).astype(np.int64)
  elif overflow == "wrap":
    q = ((rr.astype(np.int64) + 128) % 256) - 128
  else:
    raise ValueError(overflow)
  return q, scale[..., 0], rr


def int_matmul(xq, w):
  """Exact integer contraction out[m,n] = sum_k xq[m,k] * w[n,k] in int64."""
  return np.asarray(xq, dtype=np.int64) @ np.asarray(w, dtype=np.int64).T


def dense_fake_quant(x, w_nk, scale_sn, zp_sn, block):
  """float64 x @ (w*scale - zp): the reference's fake-quant identity
  (test/quantized_ops/test_quantized_matmul.py:210-218) with a pre-scaled
  zero point (:62-64).  w_nk [N,K] ints, scale_sn/zp_sn [S,N], block = K//S."""
  x = np.asarray(x, dtype=np.float64)
  w = np.asarray(w_nk, dtype=np.float64)
  n, k = w.shape
  s = np.repeat(np.asarray(scale_sn, dtype=np.float64), block, axis=0)  # [K,N]
  wdq = w.T * s
  if zp_sn is not None:
    wdq = wdq - np.repeat(np.asarray(zp_sn, dtype=np.float64), block, axis=0)
  return x @ wdq
