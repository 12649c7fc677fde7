"""Quantization backend selector; same names and aliases as the reference
(src/cache_dit/quantization/backend.py:4-51). The backend the reference calls
TORCHAO (online FP8 quantization of nn.Linear) is served here by the HIP kernels
of this package; CACHE_DIT (SVDQuant W4A4) is not built."""
from __future__ import annotations

from enum import Enum


class QuantizeBackend(Enum):
  AUTO = "AUTO"
  TORCHAO = "TORCHAO"  # online FP8 path: served by libcdit_hip.so here
  CACHE_DIT = "CACHE_DIT"  # SVDQuant: not built
  NONE = "NONE"

  @classmethod
  def from_str(cls, backend_str: str) -> "QuantizeBackend":
    key = backend_str.lower()
    aliases = {
        "ao": cls.TORCHAO,
        "torchao": cls.TORCHAO,
        "cache_dit": cls.CACHE_DIT,
        "cache-dit": cls.CACHE_DIT,
        "cachedit": cls.CACHE_DIT,
        "auto": cls.AUTO,
        "none": cls.NONE,
    }
    if key in aliases:
      return aliases[key]
    for member in cls:
      if member.value.lower() == key:
        return member
    raise ValueError(f"Unsupported quantization backend: {backend_str}.")

  @classmethod
  def is_supported(cls, backend: "QuantizeBackend") -> bool:
    if backend in (cls.AUTO, cls.TORCHAO):
      # The kernels are built in-tree; whether a gfx950 is present is checked
      # when quantize() runs, as the reference checks its platform there.
      return True
    if backend == cls.CACHE_DIT:
      return False
    if backend == cls.NONE:
      raise ValueError("QuantizeBackend.NONE is not a valid backend")
    return False
