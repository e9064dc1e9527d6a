"""The entry point that allocates nothing (xla_amd_qmm_w8a8_linear_noalloc) against the workspace variant it
derives from, through the C ABI.  Collected last: it must also pass after every other GPU test has run."""
import ctypes

import pytest
import torch

from tests import cases
from oracle import quantized_matmul_oracle as oracle
from xla_amd import _lib

pytestmark = pytest.mark.gpu


def _call(noalloc, x, w, s, z, out, sdt):
  lib = _lib.load()
  m, k = x.shape
  n = w.shape[0]
  zp_dt = _lib.dt(z.dtype) if z is not None else _lib.DT_F32
  tail = (m, n, k, _lib.dt(x.dtype), _lib.dt(s.dtype), zp_dt, _lib.dt(x.dtype), _lib.dt(sdt), _lib.dt(sdt),
          _lib.dt(out.dtype), _lib.OVERFLOW_SATURATE, 0, 0, torch.cuda.current_stream().cuda_stream)
  if noalloc:
    rc = lib.xla_amd_qmm_w8a8_linear_noalloc(x.data_ptr(), w.data_ptr(), s.data_ptr(), _lib.ptr(z), out.data_ptr(), *tail)
  else:
    nbytes = lib.xla_amd_qmm_w8a8_linear_workspace_bytes(m, n, k)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    rc = lib.xla_amd_qmm_w8a8_linear(x.data_ptr(), w.data_ptr(), s.data_ptr(), _lib.ptr(z), out.data_ptr(),
                                     ws.data_ptr(), nbytes, *tail)
  _lib.check(rc, "w8a8_linear" + ("_noalloc" if noalloc else ""))
  torch.cuda.synchronize()


def test_no_alloc_entry_point_matches_the_workspace_variant():
  lib = _lib.load()
  rows, elems = ctypes.c_int64(), ctypes.c_int64()
  lib.xla_amd_qmm_w8a8_linear_noalloc_limits(ctypes.byref(rows), ctypes.byref(elems))
  assert rows.value == 8192 and elems.value == 16 << 20
  _lib.check(lib.xla_amd_qmm_init(), "init")  # set-up of this device: the scratch array gets its memory here
  torch.cuda.synchronize()
  # two calls in a row on the shared scratch, the second smaller, with and without a zero point
  for (m, n, k, sdt, zp) in [(2048, 1024, 4096, torch.float32, False), (300, 700, 1024, torch.bfloat16, True),
                             (7, 9, 80, torch.float32, True)]:
    x = cases.outlier_activations(m, k, torch.bfloat16, seed=m)
    _, w, s, _ = cases.per_channel_int8(1, n, k, torch.bfloat16, sdt, seed=n)
    z = (torch.randn(n, generator=cases.gen(3)) * 0.01).to(sdt) if zp else None
    xd, wd, sd = x.cuda(), w.cuda(), s.cuda()
    zd = None if z is None else z.cuda()
    odt = torch.promote_types(sdt, torch.bfloat16)
    ref = torch.empty(m, n, dtype=odt, device="cuda")
    got = torch.full((m, n), float("nan"), dtype=odt, device="cuda")
    _call(False, xd, wd, sd, zd, ref, sdt)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info()[0]
    _call(True, xd, wd, sd, zd, got, sdt)
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before  # nothing from torch's allocator
    assert torch.cuda.mem_get_info()[0] == free_before                     # nothing from the device either
    assert torch.equal(got, ref), (m, n, k)
    rows_ = torch.arange(0, m, max(1, m // 16))
    exp = oracle.quantized_matmul(x[rows_], w, s, z, quantize_activation=True)
    assert cases.within_tolerance(got[rows_.cuda()].cpu(), exp)


def test_no_alloc_entry_point_rejects_oversized_activations():
  lib = _lib.load()
  one = torch.zeros(256, dtype=torch.uint8, device="cuda")
  p = one.data_ptr()
  args = lambda m, k: (p, p, p, None, p, m, 8, k, _lib.DT_BF16, _lib.DT_F32, _lib.DT_F32, _lib.DT_BF16, _lib.DT_F32,
                       _lib.DT_F32, _lib.DT_F32, _lib.OVERFLOW_SATURATE, 0, 0, None)
  assert lib.xla_amd_qmm_w8a8_linear_noalloc(*args(8193, 16)) == _lib.EUNSUPPORTED
  assert b"exceeds the fixed scratch" in lib.xla_amd_qmm_last_error()
  assert lib.xla_amd_qmm_w8a8_linear_noalloc(*args(4096, 4097)) == _lib.EUNSUPPORTED
