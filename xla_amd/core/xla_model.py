"""Operator namespace `xla` (reference: torch_xla/core/xla_model.py:40)."""
import torch

try:
  XLA_LIB = torch.library.Library("xla", "DEF")
except RuntimeError as e:  # a real torch_xla in the same process owns the namespace
  raise RuntimeError(
      "xla_amd defines the `xla` operator namespace itself and cannot be imported "
      "next to another package that already defined it (is torch_xla loaded?)") from e
