"""Pins the CPU oracle: golden fixtures, an independent exact model, closed forms
and the procedures of the reference's own tests (no GPU)."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import bitexact_model as bx
from oracle import quantized_matmul_oracle as oracle
from tests import cases

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "quantized_matmul_golden.json")))


def bf16_from_bits(bits):
  return torch.tensor(np.asarray(bits, dtype=np.uint16).astype(np.int32)).to(torch.int16).view(torch.bfloat16)


# ---- golden fixtures ---------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_hand_per_channel(dtype):
  g = GOLD["hand_per_channel"]
  x, w = torch.tensor(g["x"], dtype=dtype), torch.tensor(g["w"], dtype=torch.int8)
  s, z = torch.tensor(g["scale"], dtype=dtype), torch.tensor(g["zp"], dtype=dtype)
  assert torch.equal(oracle.quantized_matmul(x, w, s), torch.tensor(g["expect"], dtype=dtype))
  assert torch.equal(oracle.quantized_matmul(x, w, s, z), torch.tensor(g["expect_zp"], dtype=dtype))


def test_hand_blockwise():
  g = GOLD["hand_blockwise"]
  x, w = torch.tensor(g["x"]), torch.tensor(g["w"], dtype=torch.int8)
  s, z = torch.tensor(g["scale"]), torch.tensor(g["zp"])
  assert torch.equal(oracle.quantized_matmul(x, w, s, block_size=2), torch.tensor(g["expect"]))
  assert torch.equal(oracle.quantized_matmul(x, w, s, z, block_size=2), torch.tensor(g["expect_zp"]))


def test_bf16_overflow_band():
  g = GOLD["bf16_overflow_band"]
  x = bf16_from_bits(g["maxima_bits"]).reshape(-1, 1)
  for policy in ("saturate", "wrap"):
    q, s = oracle.quantize_tensor(x, overflow=policy)
    assert q.flatten().tolist() == g["q_" + policy]
    assert torch.equal(s.flatten(), bf16_from_bits(g["scale_bits"]))
  # 42 of the 256 possible row maxima per pair of binades round to 128
  assert g["counts"] == {"126": 26, "127": 188, "128": 42}


def test_w8a8_seeded_fixture():
  g = GOLD["w8a8_seeded"]
  x = bf16_from_bits(np.asarray(g["x_bits"])).reshape(4, 256)
  w = torch.tensor(g["w"], dtype=torch.int8)
  q, s = oracle.quantize_tensor(x)
  assert torch.equal(q.long(), torch.tensor(g["x_q"]))
  assert torch.equal(s.flatten(), bf16_from_bits(g["x_scale_bits"]))
  assert torch.equal(oracle.int32_accumulators(q, w).long(), torch.tensor(g["acc"]))


def test_dot_general_int32_exact():
  # the reference's exactness case (test/quantized_ops/test_dot_general.py:44-57)
  g = GOLD["dot_general_int32"]
  a, b = torch.tensor(g["a"], dtype=torch.int8), torch.tensor(g["b"], dtype=torch.int8)
  for i in range(a.shape[0]):
    got = oracle.int32_accumulators(a[i], b[i].T.contiguous())
    assert got.dtype == torch.int32
    assert torch.equal(got.long(), torch.tensor(g["expect"][i]))


def _blockwise_bf16_fixture(tag):
  g = GOLD[tag]
  m, s_, c, n = g["m"], g["s"], g["c"], g["n"]
  x = bf16_from_bits(np.asarray(g["x_bits"])).reshape(m, s_ * c)
  w = torch.tensor(g["w"], dtype=torch.int8)
  scale, zp = bf16_from_bits(np.asarray(g["scale_bits"])).reshape(s_, n), bf16_from_bits(np.asarray(g["zp_bits"])).reshape(s_, n)
  return x, w, scale, zp, c, bf16_from_bits(np.asarray(g["expect_bits"])).reshape(m, n), bf16_from_bits(
      np.asarray(g["expect_zp_bits"])).reshape(m, n)


@pytest.mark.parametrize("tag", ["blockwise_bf16_roundings", "blockwise_bf16_roundings_c128"])
def test_blockwise_bf16_rounding_points(tag):
  """The five points where the blockwise path rounds to bf16 (every sum of the fixture is exact in f32,
  so the roundings are the only inexact operations; the generator checks that dropping any one of them
  changes the result): oracle and the operator's CPU formulation, bit for bit."""
  import xla_amd.experimental.xla_quantized_matmul  # noqa: F401  (registers the CPU key)
  x, w, scale, zp, c, expect, expect_zp = _blockwise_bf16_fixture(tag)
  assert torch.equal(oracle.quantized_matmul(x, w, scale, block_size=c), expect)
  assert torch.equal(oracle.quantized_matmul(x, w, scale, zp, block_size=c), expect_zp)
  assert torch.equal(torch.ops.xla.quantized_matmul(x, w, scale, block_size=c), expect)
  assert torch.equal(torch.ops.xla.quantized_matmul(x, w, scale, zp, block_size=c), expect_zp)
  assert torch.equal(torch.ops.xla.quantized_matmul(x, w, scale, zp, block_size=c, int4_weight=True), expect_zp)


# ---- quantizer against the independent exact model ---------------------------------
@pytest.mark.parametrize("policy", ["saturate", "wrap"])
def test_quantizer_all_bf16_values(policy):
  bits = np.arange(65536, dtype=np.uint32)
  vals = bx.bf16_bits_to_f64(bits)
  vals = vals[np.isfinite(vals)]
  for mx in (1.0, 1.5, 3.140625, 100.0, 2.0**-20, 2.0**60):
    row = vals[np.abs(vals) <= mx]
    row = np.concatenate([row, [mx]])[None, :]
    q_ref, s_ref, _ = bx.quantize_rows(row, "bf16", policy)
    x = torch.tensor(row, dtype=torch.float64).to(torch.bfloat16)
    assert torch.equal(x.double(), torch.tensor(row))  # every value is on the bf16 grid
    q, s = oracle.quantize_tensor(x, overflow=policy)
    assert np.array_equal(q.numpy().astype(np.int64), q_ref), (mx, policy)
    assert s.double().item() == s_ref[0]


@pytest.mark.parametrize("fmt,dtype", [("f16", torch.float16), ("f32", torch.float32)])
def test_quantizer_other_dtypes(fmt, dtype):
  x = cases.outlier_activations(64, 512, dtype, seed=3)
  q_ref, s_ref, _ = bx.quantize_rows(x.double().numpy(), fmt, "saturate")
  q, s = oracle.quantize_tensor(x)
  assert np.array_equal(q.numpy().astype(np.int64), q_ref)
  assert np.array_equal(s.double().numpy()[:, 0], s_ref)


def test_quantizer_invariants():
  x = cases.outlier_activations(256, 1024, torch.bfloat16, seed=5)
  q, s = oracle.quantize_tensor(x)
  qn, _ = oracle.quantize_tensor(-x)
  inner = q.int().abs() < 127  # odd symmetry away from the saturating band
  assert torch.equal(qn.int()[inner], -q.int()[inner])
  amax_idx = x.abs().float().argmax(-1)
  top = q.int().abs().gather(1, amax_idx[:, None])
  assert ((top >= 126) & (top <= 128)).all()
  # scale * 127 is within one bf16 ulp (2^-8 relative) of the row maximum
  rel = (s.float()[:, 0] * 127 / x.abs().float().amax(-1) - 1).abs()
  assert rel.max() < 2**-7
  z, zs = oracle.quantize_tensor(torch.zeros(2, 8, dtype=torch.bfloat16))
  assert z.abs().sum() == 0 and zs.abs().sum() == 0


# ---- closed forms of the matmul ------------------------------------------------------
def test_closed_forms():
  g = cases.gen(1)
  x = torch.randn(5, 64, generator=g)
  ones = torch.ones(7, 64, dtype=torch.int8)
  s = torch.rand(7, generator=g)
  out = oracle.quantized_matmul(x, ones, s)  # w == 1 -> row sums times scale
  assert torch.allclose(out, x.sum(-1, keepdim=True) * s, atol=1e-5)
  w = torch.randint(-128, 128, (7, 64), generator=g, dtype=torch.int32).to(torch.int8)
  e = torch.zeros(1, 64)
  e[0, 9] = 1.0  # one-hot x picks a weight column
  assert torch.equal(oracle.quantized_matmul(e, w, torch.ones(7))[0], w[:, 9].float())
  z = torch.randn(7, generator=g)
  assert torch.allclose(oracle.quantized_matmul(x, w, s, z), oracle.quantized_matmul(x, w, s) - x.sum(-1, keepdim=True) * z,
                        atol=1e-4)


@pytest.mark.parametrize("n_bits", [4, 8])
def test_fake_quant_identity(n_bits):
  # x @ (w*scale - zp): test/quantized_ops/test_quantized_matmul.py:210-218 with a pre-scaled zero point (:62-64)
  x, w, s, z, _ = cases.blockwise(6, 24, 64, 16, n_bits, torch.float32, symmetric=False, seed=2)
  w_nk = w.permute(2, 0, 1).reshape(24, 64)
  ref = bx.dense_fake_quant(x.numpy(), w_nk.numpy(), s.numpy(), z.numpy(), 16)
  out = oracle.quantized_matmul(x, w, s, z, block_size=16)
  assert np.abs(out.double().numpy() - ref).max() < 1e-5
  # per-channel is the one-block special case
  xs, ws, ss, _ = cases.per_channel_int8(4, 10, 32, torch.float32, torch.float32, seed=3)
  zz = torch.randn(10, generator=cases.gen(4)) * 0.01
  blk = oracle.quantized_matmul(xs, ws.T.reshape(1, 32, 10).contiguous(), ss[None], zz[None], block_size=32)
  assert torch.allclose(blk, oracle.quantized_matmul(xs, ws, ss, zz), atol=1e-6)


def test_bf16_rounding_points():
  # dot -> bf16, then * scaler -> bf16 (two roundings), fp32 accumulation inside the dot
  x, w, s, _ = cases.per_channel_int8(16, 256, 1024, torch.bfloat16, torch.bfloat16, seed=6)
  out = oracle.quantized_matmul(x, w, s)
  dot = (x.double() @ w.double().T)
  two = (dot.to(torch.bfloat16).float() * s.float()).to(torch.bfloat16)
  assert cases.rel_l2(out, two) < 3e-4  # only fp32-vs-exact accumulation differences remain
  one = (dot * s.double()).to(torch.bfloat16)
  assert cases.rel_l2(out, one) > cases.rel_l2(out, two)


def test_w8a8_integer_model():
  x = cases.outlier_activations(32, 512, torch.bfloat16, seed=7)
  _, w, s, _ = cases.per_channel_int8(1, 48, 512, torch.bfloat16, torch.float32, seed=8)
  q, xs = oracle.quantize_tensor(x)
  acc = bx.int_matmul(q.numpy(), w.numpy())
  assert np.array_equal(oracle.int32_accumulators(q, w).numpy().astype(np.int64), acc)
  out = oracle.quantized_matmul(x, w, s, quantize_activation=True)
  assert out.dtype == torch.float32
  expect = (torch.tensor(acc).float() * s) * xs.float()
  assert torch.equal(out, expect)
  p = oracle.quantized_matmul_int8(x, w, s, quantize_activation=True)
  assert p.dtype == torch.bfloat16 and torch.equal(p, expect.to(torch.bfloat16))


def test_dedicated_kernel_float_branch():
  # oracle.quantized_matmul_int8(quantize_activation=False), the float branch of the reference's dedicated kernel
  # (quantized_matmul_kernel.py:108-121, :246): float32 accumulation, * float32 scale, ONE cast to x.dtype
  x, w, s, _ = cases.per_channel_int8(16, 256, 1024, torch.bfloat16, torch.bfloat16, seed=6)
  out = oracle.quantized_matmul_int8(x, w, s)
  assert out.dtype == torch.bfloat16
  exact = (x.double() @ w.double().T) * s.float().double()  # the scale enters as float32 (:219-221)
  one = exact.to(torch.bfloat16)
  # bf16(f64 dot * scale) within one ulp everywhere (f32 accumulation can flip a tie), equal almost everywhere
  ulp = torch.ldexp(torch.ones_like(exact), torch.frexp(exact.abs().clamp_min(1e-30))[1].to(torch.int32) - 8)
  assert ((out.double() - exact).abs() <= ulp).all()
  assert (out == one).float().mean() > 0.99
  # one rounding, not two: closer to the exact result than the quantized_matmul sequence (dot -> bf16, * scale -> bf16)
  two = oracle.quantized_matmul(x, w, s)
  assert cases.rel_l2(out, exact) < 0.8 * cases.rel_l2(two, exact)
  # w == 1: row sums times scale; one-hot x: a weight column times scale, exactly
  ones = torch.ones(7, 1024, dtype=torch.int8)
  s7 = torch.rand(7, generator=cases.gen(2))
  rs = oracle.quantized_matmul_int8(x, ones, s7)
  assert torch.equal(rs, ((x.double().sum(-1, keepdim=True)).float() * s7).to(torch.bfloat16))
  e = torch.zeros(1, 1024, dtype=torch.bfloat16)
  e[0, 9] = 1.0
  assert torch.equal(oracle.quantized_matmul_int8(e, w, s)[0], (w[:, 9].float() * s.float()).to(torch.bfloat16))
  # float32 activations: nothing is rounded in between, both operators agree
  xf, wf, sf, _ = cases.per_channel_int8(5, 48, 256, torch.float32, torch.float32, seed=4)
  assert torch.equal(oracle.quantized_matmul_int8(xf, wf, sf), oracle.quantized_matmul(xf, wf, sf))


def test_quantizer_nan_and_zero_rows():
  x = torch.tensor([[1.0, float("nan"), -2.0, 0.5], [0.0, 0.0, 0.0, 0.0], [1.0, 2.0, -4.0, 0.25]]).bfloat16()
  q, s = oracle.quantize_tensor(x)
  assert q[0].abs().sum() == 0 and torch.isnan(s[0]).all()      # NaN row: scale NaN (torch.amax), values 0
  assert q[1].abs().sum() == 0 and s[1].item() == 0.0           # zero row
  assert q[2].tolist() == [32, 64, -127, 8]


def test_output_dtypes():
  x = torch.randn(3, 8).bfloat16()
  w = torch.randint(-8, 8, (5, 8), dtype=torch.int8)
  assert oracle.quantized_matmul(x, w, torch.rand(5).bfloat16()).dtype == torch.bfloat16
  assert oracle.quantized_matmul(x, w, torch.rand(5)).dtype == torch.float32
  assert oracle.quantized_matmul(x, w, torch.rand(5), quantize_activation=True).dtype == torch.float32
  assert oracle.quantized_matmul(x, w, torch.rand(5).bfloat16(), quantize_activation=True).dtype == torch.bfloat16


# ---- the reference's own module-level tests, restated ----------------------------------
def _rtn_like_reference(w_fp, n_bits=8, block_size=-1, symmetric=True):
  """The RTN helper of test/quantized_ops/test_quantized_matmul.py:25-74 (determine_qparams conventions)."""
  from torch.ao.quantization.utils import determine_qparams
  import torch.ao.quantization.fx._decomposed  # noqa: F401  registers quantized_decomposed
  out_dim, in_dim = w_fp.shape
  w = w_fp if block_size == -1 else w_fp.reshape(out_dim * in_dim // block_size, block_size)
  mn, mx = torch.aminmax(w, dim=1)
  qmin, qmax = -2**(n_bits - 1), 2**(n_bits - 1) - 1
  scheme = torch.per_channel_symmetric if symmetric else torch.per_channel_affine
  scaler, zp = determine_qparams(mn, mx, qmin, qmax, dtype=torch.int8, eps=torch.Tensor([1e-5]),
                                 has_customized_qrange=False, qscheme=scheme)
  w_int = torch.ops.quantized_decomposed.quantize_per_channel(w, scaler, zp, 0, qmin, qmax, torch.int8)
  scaler = scaler.to(w_fp.dtype)
  zp = None if symmetric else zp.to(w_fp.dtype) * scaler
  if block_size != -1:
    s = in_dim // block_size
    w_int = w_int.reshape(out_dim, s, block_size).permute(1, 2, 0)
    scaler = scaler.reshape(out_dim, s).permute(1, 0)
    if zp is not None:
      zp = zp.reshape(out_dim, s).permute(1, 0)
  return w_int, scaler, zp


def _cos(a, b):
  a, b = a.flatten().float(), b.flatten().float()
  return (torch.dot(a, b) / (a.norm() * b.norm())).item()


@pytest.mark.parametrize("qa", [False, True])
def test_reference_q_linear_per_channel(qa):
  torch.manual_seed(123456)
  lin = torch.nn.Linear(5, 8, bias=False)
  x = torch.randn(3, 5)
  w, s, _ = _rtn_like_reference(lin.weight.data)
  out = oracle.quantized_matmul(x, w, s, quantize_activation=qa)
  assert torch.allclose(lin(x), out, atol=0.01)  # test_quantized_matmul.py:125


@pytest.mark.parametrize("n_bits,block,sym,qa", [(4, -1, True, False), (8, 2, True, False), (8, -1, False, False),
                                                 (8, -1, False, True), (4, -1, False, False), (8, 2, False, False)])
def test_reference_variants_cosine(n_bits, block, sym, qa):
  torch.manual_seed(123456)
  lin = torch.nn.Linear(6, 8, bias=False)
  x = torch.randn(3, 6)
  w, s, z = _rtn_like_reference(lin.weight.data, n_bits, block, sym)
  out = oracle.quantized_matmul(x, w, s, z, block_size=block, quantize_activation=qa)
  assert _cos(lin(x), out) > (0.97 if n_bits == 4 else 0.99)  # the reference asserts 0.99 on its seed


# ---- quantized_decomposed quantize / dequantize (oracle/quantized_decomposed_oracle.py) -------------

def _qdq_cases():
  g = torch.Generator().manual_seed(5)
  x = torch.randn(6, 10, 16, generator=g) * 3
  x[0, 0, :8] = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, 1e9, -1e9, 0.0])  # ties and saturation
  return x


def test_qdq_oracle_hand_values():
  from oracle import quantized_decomposed_oracle as qo
  # rint is half-to-even; zero point added after rounding; clamp last
  q = qo.quantize_affine(np.array([0.5, 1.5, 2.5, -0.5, -1.5, 300.0, -300.0], dtype=np.float32), 1.0, 3, -128, 127,
                         np.int8)
  assert q.tolist() == [3, 5, 5, 3, 1, 127, -128]
  assert qo.dequantize_per_tensor_f32(np.array([3, 5, -128], dtype=np.int8), 0.5, 3).tolist() == [0.0, 1.0, -65.5]
  assert qo.dequantize_per_channel(np.array([[3, 5], [7, 9]], dtype=np.int8), [0.5, 2.0], [1, 2], 0).tolist() == \
      [[1.0, 2.0], [10.0, 14.0]]


def test_qdq_oracle_matches_torch_decomposition():
  import torch.ao.quantization.fx._decomposed  # noqa: F401  (defines the CPU implementations)
  from oracle import quantized_decomposed_oracle as qo
  qd = torch.ops.quantized_decomposed
  x = _qdq_cases()
  for xdt in (torch.float32, torch.bfloat16, torch.float16):
    xi = x.to(xdt)
    for (scale, zp, lo, hi, dt, ndt) in [(0.037, -5, -128, 127, torch.int8, np.int8), (0.11, 128, 0, 255, torch.uint8, np.uint8),
                                         (0.5, 0, -7, 7, torch.int8, np.int8), (0.01, 10, -32768, 32767, torch.int16, np.int16)]:
      ref = qd.quantize_per_tensor(xi, scale, zp, lo, hi, dt)
      inv = np.float32(1.0 / scale)
      got = qo.quantize_affine(xi.float().numpy(), inv, zp, lo, hi, ndt)
      assert np.array_equal(got, ref.numpy()), (xdt, scale)
      deq = qd.dequantize_per_tensor(ref, scale, zp, lo, hi, dt)
      assert np.array_equal(qo.dequantize_per_tensor_f32(ref.numpy(), scale, zp), deq.numpy())
    for axis in (0, 1, 2):
      c = x.shape[axis]
      g = torch.Generator().manual_seed(axis)
      scales = torch.rand(c, generator=g) * 0.1 + 0.01
      zps = torch.randint(-20, 20, (c,), generator=g)
      ref = qd.quantize_per_channel(xi, scales, zps, axis, -128, 127, torch.int8)
      got = qo.quantize_affine(xi.float().numpy(), (1.0 / scales).numpy(), zps.numpy(), -128, 127, np.int8, axis)
      assert np.array_equal(got, ref.numpy()), (xdt, axis)
      deq = qd.dequantize_per_channel(ref, scales, zps, axis, -128, 127, torch.int8)
      assert np.array_equal(qo.dequantize_per_channel(ref.numpy(), scales.numpy(), zps.numpy(), axis), deq.numpy())
      deq0 = qd.dequantize_per_channel(ref, scales, None, axis, -128, 127, torch.int8)
      assert np.array_equal(qo.dequantize_per_channel(ref.numpy(), scales.numpy(), None, axis), deq0.numpy())
