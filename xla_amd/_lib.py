"""ctypes binding of libxla_amd_qmm.so (include/xla_amd_qmm.h).

There is no fallback: if the library is missing or a symbol cannot be bound,
loading raises, and every GPU operator of this package raises with it.
"""
import ctypes
import os
import threading

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libxla_amd_qmm.so")

OK, EINVAL, EUNSUPPORTED, EHIP = 0, -1, -2, -3
DT_F32, DT_BF16, DT_F16 = 0, 1, 2
OVERFLOW_SATURATE, OVERFLOW_WRAP = 0, 1
W_NK, W_SCN = 0, 1
QDT_I8, QDT_U8, QDT_I16, QDT_I32 = 0, 1, 2, 3
KERNEL_GENERIC, KERNEL_SKINNY_MFMA, KERNEL_W8A8_MFMA, KERNEL_W8A8_GENERIC, KERNEL_WEIGHT_ONLY_GEMM = 0, 1, 2, 3, 4
ABI_VERSION = 5

_DT = {torch.float32: DT_F32, torch.bfloat16: DT_BF16, torch.float16: DT_F16}

_c_i64, _c_int, _c_vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p

# name -> (restype, argtypes); must list every function include/xla_amd_qmm.h declares.
SIGNATURES = {
    "xla_amd_qmm_abi_version": (_c_int, []),
    "xla_amd_qmm_last_error": (ctypes.c_char_p, []),
    "xla_amd_qmm_packed_bytes": (ctypes.c_size_t, [_c_i64, _c_i64, _c_int]),
    "xla_amd_qmm_pack_weight": (_c_int, [_c_vp, _c_vp, _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_vp]),
    "xla_amd_qmm_tile_group": (_c_int, [_c_i64, _c_i64, _c_i64, _c_int]),
    "xla_amd_qmm_tiled_bytes": (ctypes.c_size_t, [_c_i64, _c_i64, _c_i64, _c_int]),
    "xla_amd_qmm_tile_weight": (_c_int, [_c_vp, _c_vp, _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_vp]),
    "xla_amd_qmm_untile_weight": (_c_int, [_c_vp, _c_vp, _c_i64, _c_i64, _c_i64, _c_int, _c_int, _c_vp]),
    "xla_amd_qmm_weight_only_skinny": (_c_int, [_c_vp] * 5 + [_c_i64] * 4 + [_c_int] * 7 + [_c_vp]),
    "xla_amd_qmm_weight_only_gemm_workspace_bytes": (ctypes.c_size_t, [_c_i64] * 4 + [_c_int]),
    "xla_amd_qmm_weight_only_gemm": (_c_int, [_c_vp] * 6 + [ctypes.c_size_t] + [_c_i64] * 4 + [_c_int] * 7 + [_c_vp]),
    "xla_amd_qmm_weight_only_gemm_f32_workspace_bytes": (ctypes.c_size_t, [_c_i64] * 3),
    "xla_amd_qmm_weight_only_gemm_f32": (_c_int, [_c_vp] * 6 + [ctypes.c_size_t] + [_c_i64] * 3 + [_c_int] * 2 + [_c_vp]),
    "xla_amd_qmm_weight_only_generic": (_c_int, [_c_vp] * 5 + [_c_i64] * 4 + [_c_int] * 7 + [_c_vp]),
    "xla_amd_qmm_quantize_per_token": (_c_int, [_c_vp] * 4 + [_c_i64] * 2 + [_c_int] * 3 + [_c_vp]),
    "xla_amd_qmm_w8a8_gemm": (_c_int, [_c_vp] * 8 + [_c_i64] * 3 + [_c_int] * 9 + [_c_vp]),
    "xla_amd_qmm_w8a8_linear_workspace_bytes": (ctypes.c_size_t, [_c_i64] * 3),
    "xla_amd_qmm_w8a8_linear": (_c_int, [_c_vp] * 6 + [ctypes.c_size_t] + [_c_i64] * 3 + [_c_int] * 10 + [_c_vp]),
    "xla_amd_qmm_init": (_c_int, []),
    "xla_amd_qmm_w8a8_linear_noalloc": (_c_int, [_c_vp] * 5 + [_c_i64] * 3 + [_c_int] * 10 + [_c_vp]),
    "xla_amd_qmm_w8a8_linear_noalloc_limits": (None, [ctypes.POINTER(_c_i64)] * 2),
    "xla_amd_qmm_dispatch": (_c_int, [_c_i64] * 4 + [_c_int] * 3),
    "xla_amd_qmm_w8a8_tile": (_c_int, [_c_i64] * 3 + [ctypes.POINTER(ctypes.c_int32)]),
    "xla_amd_qmm_quantize_affine": (_c_int, [_c_vp] * 4 + [_c_i64] * 3 + [_c_int] * 2 + [ctypes.c_int32] * 2 + [_c_vp]),
    "xla_amd_qmm_dequantize_affine": (_c_int, [_c_vp] * 4 + [_c_i64] * 3 + [_c_int] * 3 + [_c_vp]),
}

_lib = None
_lock = threading.Lock()


def lib_path() -> str:
  return _LIB_PATH


def load():
  """Loads the shared library once and binds every entry point."""
  global _lib
  if _lib is not None:
    return _lib
  with _lock:
    if _lib is not None:
      return _lib
    if not os.path.exists(_LIB_PATH):
      raise RuntimeError(
          f"{_LIB_PATH} is not built; run `python -m xla_amd.build` (needs hipcc). "
          "There is no fallback implementation for GPU tensors.")
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
      fn = getattr(lib, name)  # AttributeError if the symbol is missing
      fn.restype = res
      fn.argtypes = args
    got = lib.xla_amd_qmm_abi_version()
    if got != ABI_VERSION:
      raise RuntimeError(f"libxla_amd_qmm.so has ABI version {got}, expected {ABI_VERSION}")
    _lib = lib
  return _lib


def dt(dtype: torch.dtype) -> int:
  try:
    return _DT[dtype]
  except KeyError:
    raise RuntimeError(f"xla_amd: unsupported floating dtype {dtype}") from None


def check(rc: int, what: str):
  if rc != OK:
    msg = load().xla_amd_qmm_last_error().decode("utf-8", "replace")
    raise RuntimeError(f"{what} failed (code {rc}): {msg}")


def ptr(t):
  return None if t is None else t.data_ptr()


def stream_of(t: torch.Tensor):
  return torch.cuda.current_stream(t.device).cuda_stream
