"""GPU parity: HIP kernels (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

from tests import cases
from oracle import quantized_matmul_oracle as oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
  import xla_amd.experimental.custom_kernel  # noqa: F401  (defines both ops)
  import xla_amd.experimental.xla_quantized_matmul as qmm
  return qmm


def dev(*ts):
  return [None if t is None else t.cuda() for t in ts]


def check(actual, expected, what=""):
  assert actual.dtype == expected.dtype, f"{what}: dtype {actual.dtype} vs {expected.dtype}"
  assert actual.shape == expected.shape
  a = actual.cpu()
  assert torch.isfinite(a.float()).all()
  rl2 = cases.rel_l2(a, expected)
  assert cases.within_tolerance(a, expected), f"{what}: rel-L2 {rl2:.3e} outside tolerance"
  return rl2


# ---- config 1: fp32 per-channel -------------------------------------------------
def test_config1_fp32_per_channel(ops):
  x, w, s = cases.uniform_int8(8, 1024, 1024, torch.float32, torch.float32, seed=1)
  exp = oracle.quantized_matmul(x, w, s)
  xd, wd, sd = dev(x, w, s)
  out = torch.ops.xla.quantized_matmul(xd, wd, sd)
  rl2 = check(out, exp, "cfg1")
  assert rl2 < 1e-5  # fp32 path: summation order only
  assert ops.counters["skinny_mfma"] >= 1


# ---- config 2: decode GEMV, bf16 ---------------------------------------------------
@pytest.mark.parametrize("m", [1, 4, 16])
def test_config2_decode_gemv(ops, m):
  x, w, s, _ = cases.per_channel_int8(m, 14336, 4096, torch.bfloat16, torch.bfloat16, seed=2)
  exp = oracle.quantized_matmul(x, w, s)
  xd, wd, sd = dev(x, w, s)
  out = torch.ops.xla.quantized_matmul(xd, wd, sd)
  rl2 = check(out, exp, f"cfg2 M={m}")
  # two-rounding epilogue reproduced: only summation-order ulp flips remain
  assert rl2 < 5e-4, rl2


@pytest.mark.parametrize("m,n,k", [(3, 50, 128), (17, 100, 256), (33, 16, 384), (70, 31, 128)])
@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("zp", [False, True])
def test_skinny_per_channel_shapes(ops, m, n, k, xdt, zp):
  x, w, s, _ = cases.per_channel_int8(m, n, k, xdt, xdt, seed=m + n)
  z = (torch.randn(n, generator=cases.gen(5)) * 0.01).to(xdt) if zp else None
  exp = oracle.quantized_matmul(x, w, s, z)
  xd, wd, sd, zd = dev(x, w, s, z)
  # more than 32 rows of bf16/f16 go to the tiled GEMM, everything else here to the weight-streaming kernel
  which = "wo_gemm" if (m > 32 and xdt != torch.float32) else "skinny_mfma"
  before = ops.counters[which]
  out = torch.ops.xla.quantized_matmul(xd, wd, sd, zd)
  assert ops.counters[which] == before + 1
  check(out, exp, "skinny per-channel")


@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("zp", [False, True])
def test_skinny_wide_outputs(ops, xdt, zp):
  # more than 16384 channels: workgroups of eight computing waves (128 channels); one and two x tiles,
  # a channel tail that ends inside a workgroup, inside a wave, and a whole number of workgroups
  for (m, n, k) in [(16, 16400, 512), (32, 16500, 1024), (5, 20480, 640), (17, 16385, 128)]:
    x, w, s, _ = cases.per_channel_int8(m, n, k, xdt, xdt, seed=m + n)
    z = (torch.randn(n, generator=cases.gen(5)) * 0.01).to(xdt) if zp else None
    exp = oracle.quantized_matmul(x, w, s, z)
    before = ops.counters["skinny_mfma"]
    out = torch.ops.xla.quantized_matmul(*dev(x, w, s, z))
    assert ops.counters["skinny_mfma"] == before + 1
    check(out, exp, f"wide output {m, n, k, xdt, zp}")


def test_per_channel_mixed_scale_dtype(ops):
  x, w, s, _ = cases.per_channel_int8(5, 64, 256, torch.bfloat16, torch.float32, seed=3)
  z = torch.randn(64, generator=cases.gen(6)) * 0.01
  exp = oracle.quantized_matmul(x, w, s, z)
  out = torch.ops.xla.quantized_matmul(*dev(x, w, s, z))
  assert out.dtype == torch.float32
  check(out, exp, "bf16 x, f32 scale/zp")


# ---- small odd shapes: generic kernel ----------------------------------------------
@pytest.mark.parametrize("xdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("zp", [False, True])
def test_generic_small(ops, xdt, zp):
  g = cases.gen(7)
  x = torch.randn(3, 5, generator=g).to(xdt)
  w = torch.randint(-128, 128, (8, 5), generator=g, dtype=torch.int32).to(torch.int8)
  s = torch.rand(8, generator=g).to(xdt)
  z = torch.randn(8, generator=g).to(xdt) if zp else None
  exp = oracle.quantized_matmul(x, w, s, z)
  before = ops.counters["generic"]
  out = torch.ops.xla.quantized_matmul(*dev(x, w, s, z))
  assert ops.counters["generic"] == before + 1
  check(out, exp, "generic")
  # batch dims
  x3 = torch.randn(2, 3, 5, generator=g).to(xdt)
  exp = oracle.quantized_matmul(x3, w, s, z)
  out = torch.ops.xla.quantized_matmul(*dev(x3, w, s, z))
  check(out, exp, "generic 3-D x")


# ---- config 3: blockwise int4 ----------------------------------------------------------
@pytest.mark.parametrize("bits,int4", [(4, True), (4, False), (8, False)])
@pytest.mark.parametrize("sym", [False, True])
def test_config3_blockwise(ops, bits, int4, sym):
  x, w, s, z, _ = cases.blockwise(16, 4096, 4096, 128, bits, torch.bfloat16, symmetric=sym, seed=4)
  exp = oracle.quantized_matmul(x, w, s, z, block_size=128)
  out = torch.ops.xla.quantized_matmul(*dev(x, w, s, z), block_size=128, int4_weight=int4)
  rl2 = check(out, exp, "cfg3")
  assert rl2 < 1e-3, rl2


@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("bits", [4, 8])
def test_blockwise_shapes(ops, xdt, bits):
  # (n = 22: no 16-byte scale loads, generic kernel; k = 8192: the x columns are replaced mid-way, k-split waves)
  for (m, n, k, c) in [(2, 24, 256, 128), (19, 40, 512, 256), (3, 8, 6, 2), (5, 16, 96, 32), (4, 22, 256, 128),
                       (16, 256, 8192, 128), (20, 4096, 2048, 512)]:
    x, w, s, z, _ = cases.blockwise(m, n, k, c, bits, xdt, symmetric=False, seed=m)
    exp = oracle.quantized_matmul(x, w, s, z, block_size=c)
    out = torch.ops.xla.quantized_matmul(*dev(x, w, s, z), block_size=c, int4_weight=(bits == 4))
    check(out, exp, f"blockwise {m,n,k,c}")


@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("sym", [False, True])
def test_blockwise_int4_eight_wave_k_split(ops, xdt, sym):
  """Packed int4, K = 4096, at most 256 channel groups, up to 16 rows: eight computing waves split K
  (256 weight bytes per row and step); block sizes that divide the 512 columns of a step."""
  for (m, n, c) in [(16, 4096, 128), (1, 4096, 256), (7, 1000, 512), (16, 24, 128), (3, 4080, 128)]:
    x, w, s, z, _ = cases.blockwise(m, n, 4096, c, 4, xdt, symmetric=sym, seed=100 + m)
    exp = oracle.quantized_matmul(x, w, s, z, block_size=c, int4_weight=True)
    before = ops.counters["skinny_mfma"]
    out = torch.ops.xla.quantized_matmul(*dev(x, w, s, z), block_size=c, int4_weight=True)
    check(out, exp, f"blockwise int4 {m,n,c}")
    assert ops.counters["skinny_mfma"] == before + 1


def test_int4_per_channel(ops):
  g = cases.gen(9)
  x = torch.randn(7, 512, generator=g).bfloat16()
  w = torch.randint(-8, 8, (48, 512), generator=g, dtype=torch.int32).to(torch.int8)
  s = torch.rand(48, generator=g).bfloat16()
  exp = oracle.quantized_matmul(x, w, s)
  out = torch.ops.xla.quantized_matmul(*dev(x, w, s), int4_weight=True)
  check(out, exp, "int4 per-channel")


# ---- activation quantizer: bit exact ---------------------------------------------------
@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("policy", ["saturate", "wrap"])
def test_quantize_per_token_bit_exact(ops, xdt, policy):
  # rows kept in registers (2, 4, 8 vector steps per thread), one-element steps, and a row read twice (K > 16384)
  for (m, k) in [(64, 4096), (5, 37), (3, 8), (1, 16384), (4, 8192), (3, 14336), (2, 20480)]:
    x = cases.outlier_activations(m, k, xdt, seed=11 + m)
    if m >= 3:
      x[1] = 0  # all-zero row
    q_ref, s_ref = oracle.quantize_tensor(x, overflow=policy)
    q, s, xs = ops.quantize_per_token_gpu(x.cuda(), want_sum=True, overflow=policy)
    assert torch.equal(q.cpu(), q_ref), f"{xdt} {policy} {(m, k)}: {(q.cpu() != q_ref).sum().item()} mismatches"
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(xs.cpu().long(), q_ref.long().sum(-1))


def test_quantize_all_bf16_values(ops):
  bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
  vals = bits.view(torch.bfloat16)
  finite = torch.isfinite(vals.float())
  vals = vals[finite]
  rows = []
  for mx in [1.0, 1.5, 3.140625, 100.0, 2.0**-20, 2.0**60]:
    v = vals[vals.float().abs() <= mx]
    row = torch.zeros(65536, dtype=torch.bfloat16)
    row[:v.numel()] = v
    row[-1] = mx
    rows.append(row)
  x = torch.stack(rows)
  for policy in ("saturate", "wrap"):
    q_ref, s_ref = oracle.quantize_tensor(x, overflow=policy)
    q, s, _ = ops.quantize_per_token_gpu(x.cuda(), overflow=policy)
    assert torch.equal(q.cpu(), q_ref)
    assert torch.equal(s.cpu(), s_ref)


@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16])
def test_quantize_every_pair_of_row_maximum_and_value(ops, xdt):
  """Every positive finite value of the dtype as a row's maximum, against every value of the dtype no larger
  than it: the whole domain of the quotient x / scale for 2-byte activations (the kernel divides by the row's
  scale through a refined reciprocal and one correction step; this is the check that the result is the
  division's, bit for bit).  The checker for all rows is the oracle's op sequence run by torch on the GPU
  (a library division); every 499th row is also checked against the oracle on the CPU."""
  bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).cuda()
  vals = bits.view(xdt)
  vals = torch.where(torch.isfinite(vals.float()), vals, torch.zeros_like(vals))
  maxima = vals[(vals.float() > 0)]
  maxima = maxima[torch.argsort(maxima.float())]
  assert maxima.numel() in (0x7f7f, 0x7bff)  # positive finite values, denormals included
  chunk = 2048
  for at in range(0, maxima.numel(), chunk):
    mx = maxima[at:at + chunk].reshape(-1, 1)
    x = torch.where(vals.float().abs().reshape(1, -1) <= mx.float(), vals.reshape(1, -1), torch.zeros((), dtype=xdt, device="cuda"))
    for policy in ("wrap", "saturate"):  # (an f16 scale rounded in the subnormal range gives quotients up to 190)
      q_ref, s_ref = oracle.quantize_tensor(x, overflow=policy)
      q, s, _ = ops.quantize_per_token_gpu(x, overflow=policy)
      bad = (q != q_ref).any(dim=1) | (s.view(torch.int16) != s_ref.view(torch.int16)).any(dim=1)
      assert not bad.any(), f"{xdt} {policy}: rows with maximum {mx[bad][:4].flatten().tolist()} differ"
    rows = torch.arange(at % 499, x.shape[0], 499)
    if rows.numel():
      q_cpu, s_cpu = oracle.quantize_tensor(x[rows.cuda()].cpu())
      assert torch.equal(q[rows.cuda()].cpu(), q_cpu) and torch.equal(s[rows.cuda()].cpu(), s_cpu)


# ---- W8A8: int32 accumulators bit exact, epilogue within tolerance ------------------------
@pytest.mark.parametrize("m,n,k", [(64, 64, 64), (100, 130, 256), (256, 512, 128), (300, 700, 1024),
                                   (2048, 1024, 512), (7, 9, 80), (5, 8, 5), (512, 4096, 4096)])
def test_w8a8_int32_exact(ops, m, n, k):
  g = cases.gen(m + n + k)
  xq = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int32).to(torch.int8)
  w = torch.randint(-128, 128, (n, k), generator=g, dtype=torch.int32).to(torch.int8)
  xs = torch.rand(m, 1, generator=g)
  ws = torch.rand(n, generator=g)
  _, acc = ops.w8a8_gemm_gpu(xq.cuda(), w.cuda(), xs.cuda(), ws.cuda(), None, None,
                             cvt_dtype=torch.float32, mid_dtype=torch.float32,
                             out_dtype=torch.float32, want_acc=True)
  ref = torch.from_numpy(xq.numpy().astype(np.int64) @ w.numpy().astype(np.int64).T)
  assert torch.equal(acc.cpu().long(), ref)


@pytest.mark.parametrize("xdt,sdt", [(torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16),
                                     (torch.float32, torch.float32), (torch.float16, torch.float32)])
@pytest.mark.parametrize("zp", [False, True])
def test_w8a8_quantized_matmul(ops, xdt, sdt, zp):
  m, n, k = 200, 384, 512
  x = cases.outlier_activations(m, k, xdt, seed=21)
  _, w, s, _ = cases.per_channel_int8(1, n, k, xdt, sdt, seed=22)
  z = (torch.randn(n, generator=cases.gen(23)) * 0.01).to(sdt) if zp else None
  exp = oracle.quantized_matmul(x, w, s, z, quantize_activation=True)
  out = torch.ops.xla.quantized_matmul(*dev(x, w, s, z), quantize_activation=True)
  rl2 = check(out, exp, "w8a8")
  assert rl2 < 1e-6 or xdt != torch.float32, rl2


def test_config4_w8a8_prefill(ops):
  m, n, k = 2048, 14336, 4096
  x = cases.outlier_activations(m, k, torch.bfloat16, seed=1234)
  _, w, s, _ = cases.per_channel_int8(1, n, k, torch.bfloat16, torch.float32, seed=31)
  xd, wd, sd = dev(x, w, s)
  out = torch.ops.xla.quantized_matmul(xd, wd, sd, quantize_activation=True)
  assert out.dtype == torch.float32 and out.shape == (m, n)
  # exact int32 accumulators on a sample of rows/columns + the row-checksum identity
  xq_ref, xs_ref = oracle.quantize_tensor(x)
  xq, xs, _ = ops.quantize_per_token_gpu(xd)
  assert torch.equal(xq.cpu(), xq_ref) and torch.equal(xs.cpu(), xs_ref)
  _, acc = ops.w8a8_gemm_gpu(xq, wd, xs, sd, None, None, cvt_dtype=torch.float32,
                             mid_dtype=torch.float32, out_dtype=torch.float32, want_acc=True)
  acc = acc.cpu()
  rows = torch.arange(0, m, 37)
  ref_rows = oracle.int32_accumulators(xq_ref[rows], w)
  assert torch.equal(acc[rows], ref_rows)
  cols = torch.arange(0, n, 101)
  ref_cols = oracle.int32_accumulators(xq_ref, w[cols])
  assert torch.equal(acc[:, cols], ref_cols)
  # checksum: sum_n acc[m,n] == x_q[m,:] . sum_n w[n,:]
  wsum = w.long().sum(0)
  assert torch.equal(acc.long().sum(1), xq_ref.long() @ wsum)
  exp_rows = oracle.quantized_matmul(x[rows], w, s, quantize_activation=True)
  check(out[rows.cuda()], exp_rows, "cfg4 rows")


def test_quantized_matmul_int8_op(ops):
  for (m, n, k, hit) in [(256, 4096, 4096, True), (192, 320, 256, False)]:
    x = cases.outlier_activations(m, k, torch.bfloat16, seed=41)
    _, w, s, _ = cases.per_channel_int8(1, n, k, torch.bfloat16, torch.float32, seed=42)
    exp = oracle.quantized_matmul_int8(x, w, s, quantize_activation=True) if hit else \
        oracle.quantized_matmul_int8_fallback(x, w, s, quantize_activation=True)
    out = torch.ops.xla.quantized_matmul_int8(*dev(x, w, s), quantize_activation=True)
    assert out.dtype == torch.bfloat16
    check(out, exp, "quantized_matmul_int8")


def _reference_int8_case(dtype, bs, n_in, n_out, seed):
  """Inputs and float result of _test_quantized_matmul_int8 (test_pallas.py:886-919): symmetric per-channel
  qparams from determine_qparams, weights through quantized_decomposed.quantize_per_channel, f32 scalar."""
  import torch.ao.quantization.fx._decomposed  # noqa: F401  (defines quantized_decomposed for CPU tensors)
  from torch.ao.quantization.utils import determine_qparams
  g = cases.gen(seed)
  x = torch.randn(bs, n_in, generator=g).to(dtype)
  w = torch.randn(n_out, n_in, generator=g).to(dtype)
  min_val, max_val = torch.aminmax(w, dim=1)
  scalar, zero_point = determine_qparams(min_val, max_val, -128, 127, dtype=torch.int8, eps=torch.Tensor([1e-5]),
                                         has_customized_qrange=False, qscheme=torch.per_channel_symmetric)
  w_int = torch.ops.quantized_decomposed.quantize_per_channel(w, scalar, zero_point, 0, -128, 127, torch.int8)
  return x, w_int, scalar.to(torch.float32), torch.nn.functional.linear(x, w)


def _rel_error(x, q_x):  # test_pallas.py:882-884
  abs_error = torch.sqrt(torch.mean(torch.square(q_x - x), axis=1))
  return torch.mean(abs_error) / torch.sqrt(torch.mean(torch.square(x)))


@pytest.mark.parametrize("use_compile", [False, True])
def test_quantized_matmul_int8_wrapper_like_reference(ops, use_compile):
  # test_pallas.py:951-1026: shapes in the tuned table (dedicated-kernel semantics) and outside it (fallback +
  # cast to x.dtype), bf16 and f32, called directly and through torch.compile; bar: rel. error < 3e-2 against
  # the float linear, result in x's dtype
  from xla_amd.experimental.hip_kernels.quantized_matmul_kernel import TUNED_BLOCK_SIZES
  fn = torch.ops.xla.quantized_matmul_int8
  if use_compile:
    torch._dynamo.reset()
    fn = torch.compile(lambda x, w_int, scalar, quantize_activation: torch.ops.xla.quantized_matmul_int8(
        x, w_int, scalar, quantize_activation=quantize_activation), backend="aot_eager")
  shapes = [(torch.bfloat16, 256, 4096, 4096), (torch.bfloat16, 512, 4096, 1024)]  # (dtype, bs, n_in, n_out): hits
  assert all(("gfx950", bs, n_out, n_in, "bfloat16", True) in TUNED_BLOCK_SIZES for _, bs, n_in, n_out in shapes)
  shapes += [(dt, bs, n_in, n_out) for dt in (torch.bfloat16, torch.float32) for bs in (256, 512)
             for n_in in (256, 512) for n_out in (256, 512)]  # misses
  for (dt, bs, n_in, n_out) in shapes:
    x, w_int, scalar, expected = _reference_int8_case(dt, bs, n_in, n_out, seed=bs + n_in + n_out)
    actual = fn(x.cuda(), w_int.cuda(), scalar.cuda(), quantize_activation=True).cpu()
    assert actual.shape == expected.shape and actual.dtype == x.dtype
    assert _rel_error(expected.float(), actual.float()) < 3e-2, (dt, bs, n_in, n_out)


# ---- committed golden fixtures through the HIP path ----------------------------------------
import json
import os

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "quantized_matmul_golden.json")))


def _bf16_from_bits(bits):
  return torch.tensor(np.asarray(bits, dtype=np.uint16).astype(np.int32)).to(torch.int16).view(torch.bfloat16)


def test_golden_hand_cases(ops):
  g = GOLD["hand_per_channel"]
  x, w = torch.tensor(g["x"]), torch.tensor(g["w"], dtype=torch.int8)
  s, z = torch.tensor(g["scale"]), torch.tensor(g["zp"])
  assert torch.equal(torch.ops.xla.quantized_matmul(*dev(x, w, s)).cpu(), torch.tensor(g["expect"]))
  assert torch.equal(torch.ops.xla.quantized_matmul(*dev(x, w, s, z)).cpu(), torch.tensor(g["expect_zp"]))
  g = GOLD["hand_blockwise"]
  x, w = torch.tensor(g["x"]), torch.tensor(g["w"], dtype=torch.int8)
  s, z = torch.tensor(g["scale"]), torch.tensor(g["zp"])
  assert torch.equal(torch.ops.xla.quantized_matmul(*dev(x, w, s), block_size=2).cpu(), torch.tensor(g["expect"]))
  assert torch.equal(torch.ops.xla.quantized_matmul(*dev(x, w, s, z), block_size=2).cpu(), torch.tensor(g["expect_zp"]))


def test_golden_overflow_band_and_w8a8(ops):
  g = GOLD["bf16_overflow_band"]
  x = _bf16_from_bits(g["maxima_bits"]).reshape(-1, 1).contiguous()
  for policy in ("saturate", "wrap"):
    q, s, _ = ops.quantize_per_token_gpu(x.cuda(), overflow=policy)
    assert q.cpu().flatten().tolist() == g["q_" + policy]
    assert torch.equal(s.cpu().flatten(), _bf16_from_bits(g["scale_bits"]))
  g = GOLD["w8a8_seeded"]
  x = _bf16_from_bits(np.asarray(g["x_bits"])).reshape(4, 256).contiguous()
  w = torch.tensor(g["w"], dtype=torch.int8)
  q, s, _ = ops.quantize_per_token_gpu(x.cuda())
  assert torch.equal(q.cpu().long(), torch.tensor(g["x_q"]))
  assert torch.equal(s.cpu().flatten(), _bf16_from_bits(g["x_scale_bits"]))
  _, acc = ops.w8a8_gemm_gpu(q, w.cuda(), s, torch.ones(64).cuda(), None, None, cvt_dtype=torch.float32,
                             mid_dtype=torch.float32, out_dtype=torch.float32, want_acc=True)
  assert torch.equal(acc.cpu().long(), torch.tensor(g["acc"]))


@pytest.mark.parametrize("tag", ["blockwise_bf16_roundings", "blockwise_bf16_roundings_c128"])
def test_golden_blockwise_bf16_rounding_points(ops, tag):
  """The five bf16 rounding points of the blockwise path, fixed by the exact model (every sum of the fixture is
  exact in f32, so the kernels' summation order cannot show): generic kernel (C = 4), streaming kernel (C = 128,
  int8 container and packed int4), bit for bit."""
  g = GOLD[tag]
  m, s_, c, n = g["m"], g["s"], g["c"], g["n"]
  x = _bf16_from_bits(np.asarray(g["x_bits"])).reshape(m, s_ * c).contiguous()
  w = torch.tensor(g["w"], dtype=torch.int8)
  scale = _bf16_from_bits(np.asarray(g["scale_bits"])).reshape(s_, n).contiguous()
  zp = _bf16_from_bits(np.asarray(g["zp_bits"])).reshape(s_, n).contiguous()
  expect = _bf16_from_bits(np.asarray(g["expect_bits"])).reshape(m, n)
  expect_zp = _bf16_from_bits(np.asarray(g["expect_zp_bits"])).reshape(m, n)
  before = dict(ops.counters)
  assert torch.equal(torch.ops.xla.quantized_matmul(*dev(x, w, scale), block_size=c).cpu(), expect)
  assert torch.equal(torch.ops.xla.quantized_matmul(*dev(x, w, scale, zp), block_size=c).cpu(), expect_zp)
  assert torch.equal(torch.ops.xla.quantized_matmul(*dev(x, w, scale, zp), block_size=c, int4_weight=True).cpu(), expect_zp)
  kernel = "skinny_mfma" if c % 128 == 0 else "generic"
  assert ops.counters[kernel] == before[kernel] + 3, "the fixture did not reach the kernel it is meant for"


def test_golden_dot_general_and_int4_pack(ops):
  from xla_amd import _lib
  g = GOLD["dot_general_int32"]
  a, b = torch.tensor(g["a"], dtype=torch.int8), torch.tensor(g["b"], dtype=torch.int8)
  for i in range(a.shape[0]):
    _, acc = ops.w8a8_gemm_gpu(a[i].contiguous().cuda(), b[i].T.contiguous().cuda(), torch.ones(3, 1).cuda(),
                               torch.ones(5).cuda(), None, None, cvt_dtype=torch.float32,
                               mid_dtype=torch.float32, out_dtype=torch.float32, want_acc=True)
    assert torch.equal(acc.cpu().long(), torch.tensor(g["expect"][i]))
  rows = GOLD["int4_pack"]
  w = torch.tensor([r["values"] for r in rows], dtype=torch.int8)  # [16, 8]
  for layout, src in ((_lib.W_NK, w), (_lib.W_SCN, w.T.reshape(1, 8, 16).contiguous())):
    packed = ops._packed_weight(src.cuda(), 4, layout).cpu().numpy().view(np.uint32)
    assert packed.tolist() == [r["word"] for r in rows]


def _tiled_expected(wn, bits, G):
  """The tiled copy by its written definition (include/xla_amd_qmm.h): groups of G channels."""
  n, k = wn.shape
  groups, n_blk = (n + G - 1) // G, k // 128
  blk = 128 * G if bits == 8 else 64 * G
  expect = np.zeros(groups * n_blk * blk, dtype=np.uint8)
  P = [0, 2, 4, 6, 1, 3, 5, 7]
  for p in range(groups):
    for t in range(n_blk):
      base = (p * n_blk + t) * blk
      for q in range(4):
        for r in range(G):
          ch, k0 = G * p + r, 128 * t + 32 * q
          if ch >= n:
            continue
          if bits == 8:
            for h in range(2):
              at = base + ((h * 4 + q) * G + r) * 16
              expect[at:at + 16] = wn[ch, k0 + 16 * h:k0 + 16 * h + 16] & 0xFF
          else:
            for i in range(4):
              word = 0
              for j in range(8):
                word |= ((int(wn[ch, k0 + 8 * i + P[j]]) + 8) & 15) << (4 * j)
              for b in range(4):
                expect[base + (q * G + r) * 16 + 4 * i + b] = (word >> (8 * b)) & 0xFF
  return expect


def test_tile_weight_layout(ops):
  # the tiled copy against its written definition (include/xla_amd_qmm.h), both source layouts, N tail
  from xla_amd import _lib
  n, k = 40, 256
  g = cases.gen(7)
  for bits in (8, 4):
    lo, hi = (-128, 128) if bits == 8 else (-8, 8)
    w = torch.randint(lo, hi, (n, k), generator=g, dtype=torch.int32).to(torch.int8)
    expect = _tiled_expected(w.numpy().astype(np.int64), bits, 16)
    for layout, src in ((_lib.W_NK, w), (_lib.W_SCN, w.T.reshape(2, 128, n).contiguous())):
      got = ops._tiled_weight(src.cuda(), bits, layout).cpu().numpy()
      assert got.shape == expect.shape and (got == expect).all(), f"bits {bits} layout {layout}"


@pytest.mark.parametrize("n,group", [(4100, 10), (6144, 12), (7165, 14), (7166, 14)])
def test_tile_weight_layout_narrow_groups(ops, n, group):
  # per-channel int8 weights of many channels are tiled in groups of 14 / 12 / 10 channels: layout by its
  # definition, and the way back to the operator's layout
  from xla_amd import _lib
  lib = _lib.load()
  k = 256
  assert lib.xla_amd_qmm_tile_group(n, k, k, 8) == group
  w = torch.randint(-128, 128, (n, k), generator=cases.gen(11), dtype=torch.int32).to(torch.int8)
  expect = _tiled_expected(w.numpy().astype(np.int64), 8, group)
  tiled = ops._tiled_weight(w.cuda(), 8, _lib.W_NK)
  got = tiled.cpu().numpy()
  assert got.shape == expect.shape and (got == expect).all()
  back = torch.empty_like(w, device="cuda")
  _lib.check(lib.xla_amd_qmm_untile_weight(tiled.data_ptr(), back.data_ptr(), 1, k, n, _lib.W_NK, 8, _lib.stream_of(back)),
             "untile_weight")
  assert torch.equal(back.cpu(), w)


@pytest.mark.parametrize("n", [4100, 6144, 7165, 7166, 14336])
@pytest.mark.parametrize("m", [1, 16, 32, 80, 200])
@pytest.mark.parametrize("zp", [False, True])
def test_narrow_channel_groups_parity(ops, n, m, zp):
  """Per-channel int8 weights whose tiled copy has groups of 10 / 12 / 14 / 14 / 14 channels: the streaming
  kernel (m <= 32) and the tiled GEMM (more rows) against the oracle; 4100, 7166 and 7165 channels also take
  the stores of rows that are not a multiple of four (of two) channels long."""
  k = 512
  x, w, s, _ = cases.per_channel_int8(m, n, k, torch.bfloat16, torch.bfloat16, seed=n + m)
  z = (torch.randn(n, generator=cases.gen(3)) * 0.01).to(torch.bfloat16) if zp else None
  expected = oracle.quantized_matmul(x, w, s, z)
  got = torch.ops.xla.quantized_matmul(*dev(x, w, s, z))
  check(got, expected, f"n={n} m={m} zp={zp}")


@pytest.mark.parametrize("n,k", [(36864, 1024), (33002, 512), (40000, 4096), (128256, 512)])
@pytest.mark.parametrize("m", [1, 5, 16])
@pytest.mark.parametrize("zp", [False, True])
def test_streaming_kernel_with_resident_x(ops, n, k, m, zp):
  """More channel groups than wave slots and up to 16 rows: persistent waves that each stream a run of groups,
  x resident in LDS (one and two copy chunks of x, group widths 10 / 16, a channel count that is not a multiple
  of the group), against the oracle."""
  x, w, s, _ = cases.per_channel_int8(m, n, k, torch.bfloat16, torch.bfloat16, seed=n + m)
  z = (torch.randn(n, generator=cases.gen(3)) * 0.01).to(torch.bfloat16) if zp else None
  expected = oracle.quantized_matmul(x, w, s, z)
  got = torch.ops.xla.quantized_matmul(*dev(x, w, s, z))
  check(got, expected, f"n={n} k={k} m={m} zp={zp}")
  if m == 16 and not zp:
    x16 = x.half()
    got16 = torch.ops.xla.quantized_matmul(*dev(x16, w, s.half()))
    check(got16, oracle.quantized_matmul(x16, w, s.half()), f"f16 n={n} k={k}")


def test_w8a8_tiles_and_tails(ops):
  # every workgroup tile the kernel offers, on shapes with M/N/K tails
  for bm, bn in ((32, 32), (64, 32), (64, 64), (128, 128), (128, 256), (256, 256)):
    for (m, n, k) in [(bm + 3, 2 * bn + 5, 144), (17, 33, 64), (bm, bn, 4096)]:
      g = cases.gen(bm + m + n)
      xq = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int32).to(torch.int8)
      w = torch.randint(-128, 128, (n, k), generator=g, dtype=torch.int32).to(torch.int8)
      _, acc = ops.w8a8_gemm_gpu(xq.cuda(), w.cuda(), torch.ones(m, 1).cuda(), torch.ones(n).cuda(), None, None,
                                 cvt_dtype=torch.float32, mid_dtype=torch.float32, out_dtype=torch.float32,
                                 want_acc=True, block_m=bm, block_n=bn)
      ref = torch.from_numpy(xq.numpy().astype(np.int64) @ w.numpy().astype(np.int64).T)
      assert torch.equal(acc.cpu().long(), ref), (bm, bn, m, n, k)


@pytest.mark.parametrize("quantize_activation", [False, True])
def test_q_linear_module_compile_on_gpu(ops, quantize_activation):
  # test_quantized_matmul.py:128-143 (test_q_linear_module_dynamo): the compiled module runs the HIP kernels
  from xla_amd.quantization import quantize_linear
  torch.manual_seed(0)
  with torch.no_grad():
    lin = torch.nn.Linear(512, 256, bias=False)
    x = torch.randn(3, 512)
    q = quantize_linear(lin, n_bits=8, quantize_activation=quantize_activation)
    out_quant = q(x)  # CPU tensors: the eager formulation
    assert torch.allclose(lin(x), out_quant, atol=0.05)
    qd = q.cuda()
    before = dict(ops.counters)
    torch._dynamo.reset()
    out_compiled = torch.compile(qd, backend="aot_eager", fullgraph=True)(x.cuda())
    assert sum(ops.counters.values()) > sum(before.values())  # a HIP kernel ran
    assert torch.allclose(out_compiled.cpu(), out_quant, atol=4e-3)


def test_w8a8_pipeline_depths_and_k_steps(ops):
  # 64 x 64 tiles run with three LDS stages up to 512 tiles and with two above, and with two K groups per
  # workgroup up to 256 tiles when K >= 1024; K from less than one step (128) to several, with and without a
  # partial last step, even and odd step counts, crosses every prologue/drain case
  # (32 x 32 tiles: four K groups of one wave each when K >= 1024: 1, 2, 3 or 4 of them have a last step)
  for (m, n, blk, bn) in ((70, 130, 64, 64), (64 * 24, 64 * 24, 64, 64), (64 * 20, 64 * 20, 64, 64), (20, 100, 32, 32),
                          (70, 100, 64, 32)):  # 6, 576, 400, 4, 8 tiles
    for k in (16, 112, 128, 144, 256, 272, 384, 400, 1024, 1040, 1152, 1296, 1408, 1536):
      g = cases.gen(m + k)
      xq = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int32).to(torch.int8)
      w = torch.randint(-128, 128, (n, k), generator=g, dtype=torch.int32).to(torch.int8)
      _, acc = ops.w8a8_gemm_gpu(xq.cuda(), w.cuda(), torch.ones(m, 1).cuda(), torch.ones(n).cuda(), None, None,
                                 cvt_dtype=torch.float32, mid_dtype=torch.float32, out_dtype=torch.float32,
                                 want_acc=True, block_m=blk, block_n=bn)
      ref = (xq.double() @ w.double().T).long()  # exact: |sum| < 2^53
      assert torch.equal(acc.cpu().long(), ref), (m, n, k)
  # the short epilogue (whole tiles, f32 scales, no accumulator output) behind two K groups and behind one
  for (m, n, k, blk, bn) in ((128, 192, 1152, 64, 64), (128, 192, 896, 64, 64), (32, 96, 1152, 32, 32), (32, 96, 896, 32, 32),
                             (128, 96, 1152, 64, 32), (128, 96, 896, 64, 32)):
    g = cases.gen(k)
    xq = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int32).to(torch.int8)
    w = torch.randint(-128, 128, (n, k), generator=g, dtype=torch.int32).to(torch.int8)
    xs, ws = torch.rand(m, 1, generator=g) + 0.5, torch.rand(n, generator=g) + 0.5
    expect = ((xq.double() @ w.double().T).float() * ws[None, :]) * xs
    for odt in (torch.float32, torch.bfloat16, torch.float16):
      out, _ = ops.w8a8_gemm_gpu(xq.cuda(), w.cuda(), xs.cuda(), ws.cuda(), None, None, cvt_dtype=torch.float32,
                                 mid_dtype=torch.float32, out_dtype=odt, block_m=blk, block_n=bn)
      assert torch.equal(out.cpu(), expect.to(odt)), (m, n, k, blk, bn, odt)


def test_w8a8_column_split_two_tile_widths(ops):
  # a shape whose 256-wide tiles would leave the last round of workgroups mostly empty: the library covers the
  # columns with 32 256-wide and 32 192-wide tiles in two launches; ragged last tile, partial last K step
  m, n, k = 2048, 14300, 1088
  g = cases.gen(99)
  xq = torch.randint(-128, 128, (m, k), generator=g, dtype=torch.int32).to(torch.int8)
  w = torch.randint(-128, 128, (n, k), generator=g, dtype=torch.int32).to(torch.int8)
  xs, ws = torch.rand(m, 1, generator=g) + 0.5, torch.rand(n, generator=g) + 0.5
  ref = (xq.double() @ w.double().T).long()  # exact: |sum| < 2^53
  out, acc = ops.w8a8_gemm_gpu(xq.cuda(), w.cuda(), xs.cuda(), ws.cuda(), None, None, cvt_dtype=torch.float32,
                               mid_dtype=torch.float32, out_dtype=torch.float32, want_acc=True)
  assert torch.equal(acc.cpu().long(), ref)
  expect = (ref.float() * ws[None, :]) * xs
  assert torch.equal(out.cpu(), expect)
  # short epilogue (no accumulator output), bf16
  out16, _ = ops.w8a8_gemm_gpu(xq.cuda(), w.cuda(), xs.cuda(), ws.cuda(), None, None, cvt_dtype=torch.float32,
                               mid_dtype=torch.float32, out_dtype=torch.bfloat16)
  assert torch.equal(out16.cpu(), expect.to(torch.bfloat16))


def test_skinny_k_splits_and_long_k(ops):
  # small N takes k-split workgroups; K = 14336 is the down projection; M > 32 takes two passes
  for (m, n, k, xdt) in [(16, 256, 4096, torch.bfloat16), (5, 4096, 14336, torch.bfloat16), (40, 1024, 1024, torch.bfloat16),
                         (8, 2048, 2048, torch.float32), (16, 4096, 640, torch.float16)]:
    x, w, s, _ = cases.per_channel_int8(m, n, k, xdt, xdt, seed=n + k)
    exp = oracle.quantized_matmul(x, w, s)
    out = torch.ops.xla.quantized_matmul(*dev(x, w, s))
    check(out, exp, f"skinny {m, n, k, xdt}")
  # blockwise with blocks wider than a step (C = 1024) and K tail of the last step
  x, w, s, z, _ = cases.blockwise(16, 512, 3072, 1024, 8, torch.bfloat16, symmetric=False, seed=9)
  check(torch.ops.xla.quantized_matmul(*dev(x, w, s, z), block_size=1024),
        oracle.quantized_matmul(x, w, s, z, block_size=1024), "blockwise C=1024")
  x, w, s, z, _ = cases.blockwise(16, 512, 640, 128, 4, torch.bfloat16, symmetric=False, seed=10)
  check(torch.ops.xla.quantized_matmul(*dev(x, w, s, z), block_size=128, int4_weight=True),
        oracle.quantized_matmul(x, w, s, z, block_size=128), "blockwise int4 K=640")


def test_module_and_state_dict_on_gpu(ops):
  from xla_amd.quantization import quantize_linear
  lin = torch.nn.Linear(256, 64, bias=False)
  x = torch.randn(3, 7, 256)
  for kw in (dict(n_bits=8), dict(n_bits=8, symmetric=False), dict(n_bits=4, block_size=128, symmetric=False),
             dict(n_bits=8, quantize_activation=True)):
    q = quantize_linear(lin, **kw)
    exp = oracle.quantized_matmul(x, q.weight, q.weight_scaler, q.zero_point, block_size=q.block_size,
                                  quantize_activation=q.quantize_activation)
    qd = q.cuda()
    out = qd(x.cuda())
    assert out.shape == (3, 7, 64)
    check(out, exp, f"module {kw}")
    assert qd.weight.is_cuda and set(qd.state_dict()) >= {"weight", "weight_scaler"}


def _cosine(x, y):  # _calc_cosine_dist, test_quantized_matmul.py:106-109
  x, y = x.flatten().to(torch.float32), y.flatten().to(torch.float32)
  return (torch.sum(x * y) / (torch.norm(x) * torch.norm(y))).item()


def test_linear_modules_at_the_reference_tests_shapes(ops):
  # test_quantized_matmul.py:111-126 (per channel), :182-196 (int4), :228-244 (blockwise), :246-267 (asymmetric
  # per channel, with and without activation quantization), :269-286 (asymmetric blockwise): tiny layers,
  # quantized output close to the float one, device output equal to the CPU-tensor one
  from xla_amd.quantization import quantize_linear
  torch.manual_seed(0)
  cases_ = [((5, 8), dict(n_bits=8)), ((5, 8), dict(n_bits=8, quantize_activation=True)), ((5, 8), dict(n_bits=4)),
            ((6, 8), dict(n_bits=8, block_size=2)), ((6, 8), dict(n_bits=4, block_size=2)),
            ((6, 8), dict(n_bits=4, symmetric=False)), ((6, 8), dict(n_bits=8, symmetric=False)),
            ((6, 8), dict(n_bits=4, symmetric=False, quantize_activation=True)),
            ((6, 8), dict(n_bits=8, symmetric=False, quantize_activation=True)),
            ((6, 8), dict(n_bits=8, block_size=2, symmetric=False))]
  with torch.no_grad():
    for (n_in, n_out), kw in cases_:
      lin = torch.nn.Linear(n_in, n_out, bias=False)
      x = torch.randn(3, n_in)
      out_fp = lin(x)
      q = quantize_linear(lin, **kw)
      out_quant = q(x)
      assert _cosine(out_fp, out_quant) > (0.95 if kw["n_bits"] == 4 else 0.99), kw
      out_dev = q.cuda()(x.cuda()).cpu()
      assert _cosine(out_dev, out_quant) > 0.99999, kw
      assert torch.allclose(out_dev, out_quant, atol=2e-3), kw


# ---- quantized_decomposed quantize / dequantize on the GPU ------------------------------------------

def test_qdq_ops_match_oracle_and_torch_cpu(ops):
  import xla_amd.experimental.quantized  # noqa: F401  (binds the CUDA key)
  from oracle import quantized_decomposed_oracle as qo
  qd = torch.ops.quantized_decomposed
  g = torch.Generator().manual_seed(5)
  x = torch.randn(6, 10, 16, generator=g) * 3
  x[0, 0, :8] = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, 1e9, -1e9, 0.0])
  for xdt in (torch.float32, torch.bfloat16, torch.float16):
    xi = x.to(xdt)
    for (scale, zp, lo, hi, dt, ndt) in [(0.037, -5, -128, 127, torch.int8, np.int8), (0.11, 128, 0, 255, torch.uint8, np.uint8),
                                         (0.01, 10, -32768, 32767, torch.int16, np.int16)]:
      q = qd.quantize_per_tensor(xi.cuda(), scale, zp, lo, hi, dt)
      assert q.dtype == dt and q.is_cuda
      expect = qo.quantize_affine(xi.float().numpy(), np.float32(1.0 / scale), zp, lo, hi, ndt)
      assert np.array_equal(q.cpu().numpy(), expect), (xdt, scale)
      assert torch.equal(q.cpu(), qd.quantize_per_tensor(xi, scale, zp, lo, hi, dt))
      d = qd.dequantize_per_tensor(q, scale, zp, lo, hi, dt)
      assert np.array_equal(d.cpu().numpy(), qo.dequantize_per_tensor_f32(expect, scale, zp))
      d16 = qd.dequantize_per_tensor(q, scale, zp, lo, hi, dt, out_dtype=torch.bfloat16)
      assert torch.equal(d16.cpu(), qd.dequantize_per_tensor(q.cpu(), scale, zp, lo, hi, dt, out_dtype=torch.bfloat16))
    for axis in (0, 1, 2):
      c = x.shape[axis]
      g2 = torch.Generator().manual_seed(axis)
      scales = torch.rand(c, generator=g2) * 0.1 + 0.01
      zps = torch.randint(-20, 20, (c,), generator=g2)
      q = qd.quantize_per_channel(xi.cuda(), scales.cuda(), zps.cuda(), axis, -128, 127, torch.int8)
      expect = qo.quantize_affine(xi.float().numpy(), (1.0 / scales).numpy(), zps.numpy(), -128, 127, np.int8, axis)
      assert np.array_equal(q.cpu().numpy(), expect), (xdt, axis)
      d = qd.dequantize_per_channel(q, scales.cuda(), zps.cuda(), axis, -128, 127, torch.int8)
      assert np.array_equal(d.cpu().numpy(), qo.dequantize_per_channel(expect, scales.numpy(), zps.numpy(), axis))
      d0 = qd.dequantize_per_channel(q, scales.cuda(), None, axis, -128, 127, torch.int8)
      assert np.array_equal(d0.cpu().numpy(), qo.dequantize_per_channel(expect, scales.numpy(), None, axis))
  # a weight-sized tensor through the vector path: quantize -> dequantize stays within half a step
  w = torch.randn(4096, 4096, generator=g).bfloat16()
  q = qd.quantize_per_tensor(w.cuda(), 0.05, 0, -128, 127, torch.int8)
  assert torch.equal(q.cpu(), qd.quantize_per_tensor(w, 0.05, 0, -128, 127, torch.int8))
  back = qd.dequantize_per_tensor(q, 0.05, 0, -128, 127, torch.int8).cpu()
  inside = w.float().abs() <= 127 * 0.05
  assert ((back - w.float()).abs()[inside] <= 0.025 + 1e-6).all()


def test_fused_linears_on_gpu(ops):
  # q/k/v-style N-concatenation: one launch, outputs identical to the separate layers
  from xla_amd.quantization import quantize_linear, fuse_quantized_linears
  torch.manual_seed(11)
  for kwargs, xdt in ((dict(n_bits=8, scale_dtype=torch.bfloat16), torch.bfloat16),
                      (dict(n_bits=8, quantize_activation=True), torch.bfloat16),
                      (dict(n_bits=4, block_size=128, symmetric=False, scale_dtype=torch.bfloat16), torch.bfloat16)):
    lins = [quantize_linear(torch.nn.Linear(512, n, bias=False), **kwargs).cuda() for n in (256, 64, 128)]
    fused = fuse_quantized_linears(lins)
    x = torch.randn(9, 512).to(xdt).cuda()
    outs = fused(x).split([l.output_dim for l in lins], dim=-1)
    for l, o in zip(lins, outs):
      assert torch.equal(l(x), o), kwargs


def test_w8a8_f16_scaler_overflow_like_the_reference(ops):
  """With an f16 scaler the reference converts the int32 sums to f16 before it scales them: sums beyond 65504
  become inf there, and here at the same places with the same sign."""
  for (m, n, k, zp) in [(7, 512, 640, True), (31, 16, 256, False), (300, 333, 8704, True)]:
    x = cases.outlier_activations(m, k, torch.float16, seed=5)
    _, w, s, _ = cases.per_channel_int8(1, n, k, torch.float16, torch.float16, seed=5)
    z = (torch.randn(n, generator=cases.gen(6)) * 0.01).half() if zp else None
    exp = oracle.quantized_matmul(x, w, s, z, quantize_activation=True)
    out = torch.ops.xla.quantized_matmul(x.cuda(), w.cuda(), s.cuda(), None if z is None else z.cuda(), -1, False, True).cpu()
    fin = torch.isfinite(exp)
    assert (~fin).any() and not exp.isnan().any()
    assert torch.equal(torch.isfinite(out), fin) and torch.equal(out[~fin], exp[~fin]), (m, n, k)
    zero = torch.zeros_like(out)
    assert cases.within_tolerance(torch.where(fin, out, zero), torch.where(fin, exp, zero)), (m, n, k)
