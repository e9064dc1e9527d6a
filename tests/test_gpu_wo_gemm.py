"""GPU parity of the weight-only tiled GEMM (many rows of x, or few channels with a long K) against the CPU oracle."""
import pytest
import torch

from tests import cases
from oracle import quantized_matmul_oracle as oracle
from xla_amd import _lib

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
  import xla_amd.experimental.custom_kernel  # noqa: F401
  import xla_amd.experimental.xla_quantized_matmul as qmm
  return qmm


def check(actual, expected, what=""):
  assert actual.dtype == expected.dtype, f"{what}: dtype {actual.dtype} vs {expected.dtype}"
  assert actual.shape == expected.shape
  a = actual.cpu()
  assert torch.isfinite(a.float()).all(), what
  rl2 = cases.rel_l2(a, expected)
  assert cases.within_tolerance(a, expected), f"{what}: rel-L2 {rl2:.3e} outside tolerance"
  return rl2


def wo_gemm(ops, x, w, s, z, dot_dtype=None, store_dtype=None):
  """Calls xla_amd_qmm_weight_only_gemm directly (whatever the dispatcher would choose)."""
  lib = _lib.load()
  m, k = x.shape
  n = w.shape[0]
  wt = ops._tiled_weight(w, 8, _lib.W_NK)
  out_dtype = torch.promote_types(x.dtype, s.dtype)
  store_dtype = store_dtype or out_dtype
  out = torch.empty(m, n, dtype=store_dtype, device=x.device)
  nbytes = lib.xla_amd_qmm_weight_only_gemm_workspace_bytes(m, n, k, k, 8)
  ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
  zp_dt = _lib.dt(z.dtype) if z is not None else _lib.dt(x.dtype)
  rc = lib.xla_amd_qmm_weight_only_gemm(x.data_ptr(), wt.data_ptr(), s.data_ptr(), _lib.ptr(z), out.data_ptr(), ws.data_ptr(),
                                        nbytes, m, n, k, k, 8, _lib.dt(x.dtype), _lib.dt(s.dtype), zp_dt,
                                        _lib.dt(dot_dtype or x.dtype), _lib.dt(out_dtype), _lib.dt(store_dtype),
                                        torch.cuda.current_stream().cuda_stream)
  _lib.check(rc, "weight_only_gemm")
  return out


@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("zp", [False, True])
def test_wo_gemm_shapes(ops, xdt, zp):
  # every row-tile height (32 / 64 / 128 rows), both tile widths, with and without a K split, M / N tails,
  # one to many K steps, several chunks of x
  for (m, n, k) in [(33, 256, 512), (64, 100, 1024), (17, 4096, 14336), (32, 1024, 4096), (128, 512, 128), (200, 333, 2560),
                    (300, 700, 1024), (48, 64, 8192), (2, 16, 128), (130, 2048, 2048),
                    # K slices of 3, 4 + 1, 4 + 3 and 4 + 4 + 3 steps (the two-deep weight ring's tails)
                    (40, 96, 384), (64, 128, 640), (50, 200, 896), (64, 64, 1408),
                    # more work items than compute units: workgroups walk several of them
                    (60, 33024, 256),
                    # few rows against a long K: the weight-streaming kernel over K slices (N tail, M tail, 28 and 16 steps)
                    (32, 200, 8192), (9, 4096, 14336), (24, 1000, 8192),
                    # a narrow output with two x tiles: K slices at K = 4096 too
                    (32, 1024, 4096), (17, 520, 4096)]:
    x, w, s, _ = cases.per_channel_int8(m, n, k, xdt, xdt, seed=m + n)
    z = (torch.randn(n, generator=cases.gen(5)) * 0.01).to(xdt) if zp else None
    exp = oracle.quantized_matmul(x, w, s, z)
    out = wo_gemm(ops, x.cuda(), w.cuda(), s.cuda(), None if z is None else z.cuda())
    rl2 = check(out, exp, f"wo_gemm {m, n, k, xdt, zp}")
    assert rl2 < 1e-3, (m, n, k, rl2)


def test_wo_gemm_mixed_dtypes_and_float_branch(ops):
  x, w, s, _ = cases.per_channel_int8(100, 384, 1024, torch.bfloat16, torch.float32, seed=3)
  z = torch.randn(384, generator=cases.gen(6)) * 0.01
  out = wo_gemm(ops, x.cuda(), w.cuda(), s.cuda(), z.cuda())
  assert out.dtype == torch.float32
  check(out, oracle.quantized_matmul(x, w, s, z), "bf16 x, f32 scale / zp")
  # the dedicated kernel's float branch: f32 accumulation, f32 scale, one cast
  out = wo_gemm(ops, x.cuda(), w.cuda(), s.cuda(), None, dot_dtype=torch.float32, store_dtype=torch.bfloat16)
  rl2 = check(out, oracle.quantized_matmul_int8(x, w, s), "float branch")
  assert rl2 < 3e-4


def test_weight_only_prefill_through_the_operator(ops):
  # cfg2's shape with a prefill-sized M: the operator takes the tiled GEMM above 32 rows
  m, n, k = 2048, 14336, 4096
  x, w, s, _ = cases.per_channel_int8(m, n, k, torch.bfloat16, torch.bfloat16, seed=2)
  before = ops.counters["wo_gemm"]
  out = torch.ops.xla.quantized_matmul(x.cuda(), w.cuda(), s.cuda())
  assert ops.counters["wo_gemm"] == before + 1
  rows = torch.arange(0, m, 29)
  rl2 = check(out[rows.cuda()], oracle.quantized_matmul(x[rows], w, s), "weight-only prefill rows")
  assert rl2 < 5e-4
  # size-independent: a row of the result depends on that row of x only
  out2 = torch.ops.xla.quantized_matmul(x[rows].cuda(), w.cuda(), s.cuda())
  assert cases.rel_l2(out2.cpu(), out[rows.cuda()].cpu()) < 1e-3
  # the module and 3-D activations take the same route
  from xla_amd.experimental.xla_quantized_matmul import XlaQuantizedLinear
  lin = XlaQuantizedLinear(k, n, is_symmetric=True)
  lin.load_quantized_weight(w.cuda(), s.cuda())
  x3 = x[:96].reshape(2, 48, k)
  check(lin(x3.cuda()), oracle.quantized_matmul(x3, w, s), "module, 3-D x")


@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16])
def test_blockwise_and_int4_gemm(ops, xdt):
  """More than 32 rows against blockwise or int4 weights: the tiled GEMM with per-block rounding points."""
  op = torch.ops.xla.quantized_matmul
  # (m, n, k, block, bits, asymmetric): one and several steps per block, block = chunk, row / channel tails,
  # several chunks, more tiles than compute units
  for (m, n, k, c, bits, asym) in [(65, 128, 256, 128, 8, False), (100, 200, 1024, 128, 4, True), (128, 4096, 4096, 128, 4, True),
                                   (130, 60, 1536, 512, 8, True), (300, 1000, 2048, 256, 4, False), (65, 4, 128, 128, 4, True),
                                   (70, 132, 2560, 640, 8, False), (513, 8192, 1024, 128, 4, True),
                                   # blocks of 128 columns (the kernel that rounds a block during the next one's MFMAs):
                                   # 5 and 11 steps (an odd count, a last chunk of one and of three steps), int4 without
                                   # and int8 with a zero point (the latter keeps the other kernel), several items
                                   (90, 264, 640, 128, 4, False), (200, 136, 1408, 128, 8, False), (80, 128, 384, 128, 8, True),
                                   (700, 5000, 1152, 128, 4, True)]:
    x, w, s, z, _ = cases.blockwise(m, n, k, c, bits, xdt, symmetric=not asym, seed=m + n)
    exp = oracle.quantized_matmul(x, w, s, z if asym else None, block_size=c, int4_weight=bits == 4)
    before = ops.counters["wo_gemm"]
    out = op(x.cuda(), w.cuda(), s.cuda(), z.cuda() if asym else None, c, bits == 4)
    assert ops.counters["wo_gemm"] == before + 1
    rl2 = check(out, exp, f"blockwise GEMM {m, n, k, c, bits, asym, xdt}")
    assert rl2 < 1e-3, (m, n, k, c, bits, rl2)
  # per-channel int4 (one block)
  for (m, n, k, zp) in [(77, 512, 1024, False), (200, 100, 384, True)]:
    x, w, s, _ = cases.per_channel_int8(m, n, k, xdt, xdt, seed=m)
    w = w.clamp(-8, 7)
    z = (torch.randn(n, generator=cases.gen(5)) * 0.01).to(xdt) if zp else None
    exp = oracle.quantized_matmul(x, w, s, z, int4_weight=True)
    before = ops.counters["wo_gemm"]
    out = op(x.cuda(), w.cuda(), s.cuda(), None if z is None else z.cuda(), -1, True)
    assert ops.counters["wo_gemm"] == before + 1
    check(out, exp, f"per-channel int4 GEMM {m, n, k, zp, xdt}")
  # mixed dtypes (f32 scale with 2-byte x) keep the streaming kernel
  x, w, s, _ = cases.per_channel_int8(80, 64, 256, xdt, torch.float32, seed=9)
  before = ops.counters["skinny_mfma"]
  out = op(x.cuda(), w.clamp(-8, 7).cuda(), s.cuda(), None, -1, True)
  assert ops.counters["skinny_mfma"] == before + 1
  check(out, oracle.quantized_matmul(x, w.clamp(-8, 7), s, int4_weight=True), "int4, f32 scale")


@pytest.mark.parametrize("zp", [False, True])
def test_int4_per_channel_k_slices(ops, zp):
  """Few rows, few channels, long K with per-channel int4 weights: the streaming kernel over K slices (steps of 1024 columns)."""
  op = torch.ops.xla.quantized_matmul
  for (m, n, k, sdt) in [(32, 4096, 14336, torch.bfloat16), (9, 1000, 8192, torch.bfloat16), (16, 2048, 10240, torch.float32)]:
    x, w, s, _ = cases.per_channel_int8(m, n, k, torch.bfloat16, sdt, seed=n)
    w = w.clamp(-8, 7)
    z = (torch.randn(n, generator=cases.gen(5)) * 0.01).to(sdt) if zp else None
    exp = oracle.quantized_matmul(x, w, s, z, int4_weight=True)
    before = ops.counters["wo_gemm"]
    out = op(x.cuda(), w.cuda(), s.cuda(), None if z is None else z.cuda(), -1, True)
    assert ops.counters["wo_gemm"] == before + 1
    check(out, exp, f"int4 K slices {m, n, k, sdt, zp}")


@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16])
def test_blockwise_k_slices(ops, xdt):
  """Few rows, few channels, long K with blockwise weights: K slices of whole quantization blocks; the second kernel adds
  the slices' scaled sums (and zero-point sums) and does the final roundings."""
  op = torch.ops.xla.quantized_matmul
  lib = _lib.load()
  # (m, n, k, block, bits, asymmetric): blocks shorter than, equal to and longer than a step of the streaming kernel
  # (512 columns of int8, 1024 of int4), a last slice shorter than the others, row tails, one and two row tiles
  for (m, n, k, c, bits, asym) in [(32, 4096, 14336, 128, 4, True), (16, 4096, 14336, 128, 8, False), (9, 1000, 8192, 256, 4, True),
                                   (32, 2048, 14336, 2048, 8, True), (24, 512, 10240, 1024, 4, False), (8, 64, 16384, 512, 8, True),
                                   (32, 200, 8192, 128, 4, True)]:
    assert lib.xla_amd_qmm_weight_only_gemm_workspace_bytes(m, n, k, c, bits) > 0, (m, n, k, c, bits)
    x, w, s, z, _ = cases.blockwise(m, n, k, c, bits, xdt, symmetric=not asym, seed=m + n)
    exp = oracle.quantized_matmul(x, w, s, z if asym else None, block_size=c, int4_weight=bits == 4)
    before = ops.counters["wo_gemm"]
    out = op(x.cuda(), w.cuda(), s.cuda(), z.cuda() if asym else None, c, bits == 4)
    assert ops.counters["wo_gemm"] == before + 1
    rl2 = check(out, exp, f"blockwise K slices {m, n, k, c, bits, asym, xdt}")
    assert rl2 < 1e-3, (m, n, k, c, bits, rl2)


@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16])
def test_wo_gemm_several_rounds_of_tiles(ops, xdt):
  """More 128 x 256 tiles than compute units, the last round part full: persistent workgroups walk two items or
  one (also: a last column tile narrower than 256, rows whose count is no multiple of 16 or of 128)."""
  for (m, n, k) in [(1056, 7680, 256), (1100, 7500, 384), (2048, 14336, 128)]:
    assert -(-m // 128) * -(-n // 256) > 256
    x, w, s, _ = cases.per_channel_int8(m, n, k, xdt, xdt, seed=m)
    exp = oracle.quantized_matmul(x, w, s)
    out = wo_gemm(ops, x.cuda(), w.cuda(), s.cuda(), None)
    check(out, exp, f"several rounds {m,n,k}")


@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16])
def test_wo_gemm_results_written_out_by_the_copying_waves(ops, xdt):
  """From 12 steps of K up, with one 2-byte dtype throughout and N a multiple of 8, the 128 x 256 tile leaves its
  results in LDS and the copying waves scale them and write them out during the next item: exactly 12 and 13 steps,
  one item per workgroup and several, row and column tails."""
  for (m, n, k) in [(1024, 8192, 1536), (1100, 7496, 1664), (2048, 14336, 1536)]:
    x, w, s, _ = cases.per_channel_int8(m, n, k, xdt, xdt, seed=m + k)
    exp = oracle.quantized_matmul(x, w, s)
    out = wo_gemm(ops, x.cuda(), w.cuda(), s.cuda(), None)
    check(out, exp, f"results through LDS {m,n,k}")
    if m == 1100:  # the same with a scale vector that does not start on 16 bytes: the computing waves store
      out2 = torch.empty(m, n, dtype=xdt, device="cuda")
      s2 = torch.empty(n + 4, dtype=xdt, device="cuda")[4:].copy_(s)
      assert s2.data_ptr() % 16 != 0
      lib = _lib.load()
      assert lib.xla_amd_qmm_weight_only_gemm_workspace_bytes(m, n, k, k, 8) == 0
      wt = ops._tiled_weight(w.cuda(), 8, _lib.W_NK)
      rc = lib.xla_amd_qmm_weight_only_gemm(x.cuda().data_ptr(), wt.data_ptr(), s2.data_ptr(), None, out2.data_ptr(), None, 0,
                                            m, n, k, k, 8, _lib.dt(xdt), _lib.dt(xdt), _lib.dt(xdt), _lib.dt(xdt), _lib.dt(xdt),
                                            _lib.dt(xdt), torch.cuda.current_stream().cuda_stream)
      _lib.check(rc, "weight_only_gemm")
      assert torch.equal(out2, out)


@pytest.mark.parametrize("sdt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("zp", [False, True])
def test_f32_rows_through_the_tiled_gemm(ops, sdt, zp):
  """128 rows of f32 x or more: split into three bf16 parts (exact), bf16 MFMA GEMM with f32 accumulation; against
  the f32 oracle to summation-order accuracy (the tolerance of the f32 streaming kernel's test)."""
  for (m, n, k) in [(128, 64, 128), (300, 700, 1024), (130, 4096, 2048), (1000, 520, 384)]:
    x, w, s, _ = cases.per_channel_int8(m, n, k, torch.float32, sdt, seed=m)
    z = (torch.randn(n, generator=cases.gen(m + 1)) * 0.5).to(sdt) if zp else None
    exp = oracle.quantized_matmul(x, w, s, z)
    before = ops.counters["wo_gemm"]
    out = torch.ops.xla.quantized_matmul(x.cuda(), w.cuda(), s.cuda(), None if z is None else z.cuda())
    assert ops.counters["wo_gemm"] == before + 1, "f32 rows did not take the tiled GEMM"
    rl2 = check(out, exp, f"f32 rows {m,n,k,sdt,zp}")
    assert rl2 < 1e-5, rl2
