"""Writes the golden fixtures of this directory.

Every expected value here comes from exact arithmetic that shares no code with
the CPU oracle or the GPU kernels: integer/rational models in
oracle/bitexact_model.py (numpy int64 / float64 with explicit round-to-nearest-
even) or values worked out by hand below.  The reference implementation
cannot be imported here (it needs the torch_xla extension), so its own tests'
procedures are restated as data: the int8 x int8 -> int32 exactness case of
test/quantized_ops/test_dot_general.py:44-57 and the fake-quant identity of
test/quantized_ops/test_quantized_matmul.py:210-218.

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import bitexact_model as bx  # noqa: E402


def bf16_grid(v):
  return bx.round_to_format(np.asarray(v, dtype=np.float64), "bf16")


def main():
  rng = np.random.default_rng(20251125)
  out = {}

  # 1. hand-computable per-channel case: w = identity-like rows, scale = powers of two
  x = np.array([[1.0, -2.0, 3.0, 0.5], [0.0, 4.0, -1.0, 2.0]])
  w = np.array([[1, 0, 0, 0], [0, 1, 0, 0], [1, 1, 1, 1], [-1, 2, -3, 4], [127, -128, 0, 0]], dtype=np.int64)
  scale = np.array([1.0, 0.5, 2.0, 0.25, 0.125])
  zp = np.array([0.0, 1.0, -0.5, 2.0, 0.0])
  dot = x @ w.T
  expect = dot * scale
  expect_zp = expect - x.sum(-1, keepdims=True) * zp
  assert expect[0].tolist() == [1.0, -1.0, 5.0, -3.0, 47.875]  # worked by hand
  out["hand_per_channel"] = dict(x=x.tolist(), w=w.tolist(), scale=scale.tolist(), zp=zp.tolist(),
                                 expect=expect.tolist(), expect_zp=expect_zp.tolist())

  # 2. blockwise hand case: K = 4, block 2 -> S = 2; w [S, C, N]
  wb = np.array([[[1, -1], [2, 0]], [[0, 3], [-2, 1]]], dtype=np.int64)  # [2,2,2]
  sb = np.array([[1.0, 0.5], [2.0, 0.25]])  # [S,N]
  zb = np.array([[0.5, 0.0], [0.0, 1.0]])
  xb = np.array([[1.0, 2.0, 3.0, 4.0], [-1.0, 0.5, 0.0, 2.0]])
  xr = xb.reshape(2, 2, 2)
  p = np.einsum("scn,msc->msn", wb.astype(np.float64), xr)
  eb = np.einsum("sn,msn->mn", sb, p)
  ezb = eb - xr.sum(-1) @ zb
  assert eb[0].tolist() == [1 * (1 + 4) + 2 * (0 - 8), 0.5 * (-1 + 0) + 0.25 * (9 + 4)]
  out["hand_blockwise"] = dict(x=xb.tolist(), w=wb.tolist(), scale=sb.tolist(), zp=zb.tolist(),
                               block_size=2, expect=eb.tolist(), expect_zp=ezb.tolist())

  # 3. quantizer: every bf16 row maximum in [1, 4) (2 binades x 128 mantissas): q of the maximum
  #    element itself under both overflow policies (the 127.5 -> 128 band)
  maxima = np.array([(1.0 + m / 128.0) * e for e in (1.0, 2.0) for m in range(128)])
  q_sat, sc, rr = bx.quantize_rows(maxima[:, None], "bf16", "saturate")
  q_wrap, _, _ = bx.quantize_rows(maxima[:, None], "bf16", "wrap")
  counts = {int(v): int((rr[:, 0] == v).sum()) for v in (126, 127, 128)}
  assert sum(counts.values()) == 256
  out["bf16_overflow_band"] = dict(maxima_bits=bx.f64_to_bf16_bits(maxima).tolist(),
                                   scale_bits=bx.f64_to_bf16_bits(sc).tolist(),
                                   rounded=rr[:, 0].astype(int).tolist(), q_saturate=q_sat[:, 0].tolist(),
                                   q_wrap=q_wrap[:, 0].tolist(), counts=counts)

  # 4. seeded W8A8 case [4,256] x [64,256]: bf16 activations with an outlier column
  xa = bf16_grid(rng.standard_normal((4, 256)))
  xa[:, 7] = bf16_grid(xa[:, 7] * 20.0)
  wq = rng.integers(-127, 128, size=(64, 256))
  q, s, _ = bx.quantize_rows(xa, "bf16", "saturate")
  acc = bx.int_matmul(q, wq)
  assert np.abs(acc).max() < 2**31
  out["w8a8_seeded"] = dict(x_bits=bx.f64_to_bf16_bits(xa).tolist(), w=wq.tolist(), x_q=q.tolist(),
                            x_scale_bits=bx.f64_to_bf16_bits(s).tolist(), acc=acc.tolist())

  # 5. int8 x int8 -> int32 exactness, values in [-15, 15), batch (10,3,4) x (10,4,5)
  a = rng.integers(-15, 15, size=(10, 3, 4))
  b = rng.integers(-15, 15, size=(10, 4, 5))
  out["dot_general_int32"] = dict(a=a.tolist(), b=b.tolist(), expect=np.einsum("bij,bjk->bik", a, b).tolist())

  # 6. int4 nibble packing of all 16 values in all 8 positions of a word
  P = [0, 2, 4, 6, 1, 3, 5, 7]
  rows = []
  for v in range(-8, 8):
    vals = [((v + 8 + 3 * k) % 16) - 8 for k in range(8)]
    word = 0
    for j in range(8):
      word |= ((vals[P[j]] + 8) & 15) << (4 * j)
    rows.append(dict(values=vals, word=word))
  out["int4_pack"] = rows

  # 7. the five bf16 rounding points of the blockwise path with a zero point
  #    (xla_quantized_matmul.py:119-133: p = einsum('scn,...sc->...sn'), out = einsum('sn,...sn->...n'),
  #    zsum = x.sum(-1), zpo = zsum @ zp, out - zpo; every result is a bf16 tensor).  Inputs are chosen so
  #    that every sum is exact in f32 whatever the order (x multiples of 1/16, |w| <= 8), hence the only
  #    inexact operations are the five roundings, done here with the exact model's round_to_format.
  def blockwise_bf16_case(m, s_, c, n, tag):
    xq = rng.integers(-255, 256, size=(m, s_ * c)) / 16.0                    # bf16-exact (8 significant bits)
    wq4 = rng.integers(-8, 8, size=(s_, c, n))
    sc_ = bf16_grid((1.0 + rng.integers(0, 128, size=(s_, n)) / 128.0) * 2.0 ** rng.integers(-9, -5, size=(s_, n)))
    zp_ = bf16_grid(rng.integers(-8, 8, size=(s_, n)) * sc_)
    xr_ = xq.reshape(m, s_, c)

    def run(r_p=True, r_o1=True, r_zs=True, r_zpo=True, r_o2=True):
      rnd = lambda v, on: bf16_grid(v) if on else v
      p_ = rnd(np.einsum("scn,msc->msn", wq4.astype(np.float64), xr_), r_p)
      o_ = rnd(np.einsum("sn,msn->mn", sc_, p_), r_o1)
      zs = rnd(xr_.sum(-1), r_zs)
      zo = rnd(zs @ zp_, r_zpo)
      return rnd(o_ - zo, r_o2), rnd(o_, True)

    full, no_zp = run()
    # a formulation that skips any one of the five roundings must fail this fixture
    for k in range(5):
      flags = [True] * 5
      flags[k] = False
      other, _ = run(*flags)
      assert (other != full).any(), f"{tag}: rounding point {k} does not show in this fixture"
    out[tag] = dict(m=m, s=s_, c=c, n=n, x_bits=bx.f64_to_bf16_bits(xq).tolist(), w=wq4.tolist(),
                    scale_bits=bx.f64_to_bf16_bits(sc_).tolist(), zp_bits=bx.f64_to_bf16_bits(zp_).tolist(),
                    expect_bits=bx.f64_to_bf16_bits(no_zp).tolist(), expect_zp_bits=bx.f64_to_bf16_bits(full).tolist())

  blockwise_bf16_case(2, 3, 4, 4, "blockwise_bf16_roundings")          # any kernel that takes odd shapes
  blockwise_bf16_case(3, 3, 128, 8, "blockwise_bf16_roundings_c128")   # a shape the streaming kernel takes

  with open(os.path.join(HERE, "quantized_matmul_golden.json"), "w") as f:
    json.dump(out, f)
  print("wrote", os.path.join(HERE, "quantized_matmul_golden.json"), "overflow band counts", counts)


if __name__ == "__main__":
  main()
