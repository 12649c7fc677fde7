"""`QuantizeConfig`: the user-facing quantization configuration.

Field names, defaults and helper methods follow the reference's dataclass
(src/cache_dit/quantization/config.py:329-449 fields, :451-465 __post_init__,
:588-705 update / strify / component_quant_types / expand_configs /
from_kwargs), restricted to what the FP8 path reads. SVDQuant-only fields are
kept so that existing configs and YAML files still construct, but an `svdq*`
quant_type is refused: that mode is not built here.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable, Dict, List, Optional, Union

from .backend import QuantizeBackend

#: quant types the reference's online path accepts (quantize_ao.py:16-27)
ALLOWED_QUANTIZE_TYPES = [
    "float8_per_row",
    "float8_per_tensor",
    "float8_per_block",
    "float8_weight_only",
    "nvfp4",
    "nvfp4_weight_only",
    "int8_per_row",
    "int8_per_tensor",
    "int8_weight_only",
    "int4_weight_only",
]
#: the ones with MI355X kernels behind them
BUILT_QUANTIZE_TYPES = ["float8_per_row", "float8_per_tensor", "float8_weight_only"]

_DEFAULT_EXCLUDE = ("embedder", "embed", "modulation", "mod")


@dataclasses.dataclass
class QuantizeConfig:
  backend: Union[str, QuantizeBackend] = QuantizeBackend.AUTO
  quant_type: str = "float8_per_row"
  # substrings of layer names that are never quantized
  exclude_layers: Optional[list] = dataclasses.field(default_factory=lambda: list(_DEFAULT_EXCLUDE))
  # quantize only inside the transformer's repeated block classes
  regional_quantize: bool = True
  repeated_blocks: List[str] = dataclasses.field(default_factory=list)
  filter_fn: Optional[Any] = None
  # None -> the transformer; list of names -> each with quant_type;
  # dict name -> {"quant_type": ..., ...} -> each with its own settings
  components_to_quantize: Optional[Union[List[str], Dict[str, Dict[str, str]]]] = None
  per_tensor_fallback: bool = True
  # {layer-name substring: quant_type}
  precision_plan: Optional[Dict[str, str]] = None
  # SVDQuant-only fields (accepted, unused)
  calibrate_fn: Optional[Callable[..., Any]] = None
  serialize_to: Optional[str] = None
  svdq_kwargs: Optional[Dict[str, Any]] = None
  verbose: bool = False

  def __post_init__(self):
    if isinstance(self.quant_type, str):
      self.quant_type = self.quant_type.lower()
    if isinstance(self.backend, str):
      self.backend = QuantizeBackend.from_str(self.backend)
    if self.backend == QuantizeBackend.AUTO:
      self.backend = (QuantizeBackend.CACHE_DIT
                      if self.is_svdq() else QuantizeBackend.TORCHAO)
    if self.is_svdq() or self.backend == QuantizeBackend.CACHE_DIT:
      raise NotImplementedError(
          f"quant_type {self.quant_type!r} (SVDQuant, backend CACHE_DIT) is not built in this "
          "MI355X implementation; built quant types: " + ", ".join(BUILT_QUANTIZE_TYPES))
    assert QuantizeBackend.is_supported(
        self.backend), f"Quantization backend {self.backend} is not supported in this environment."

  # -- predicates --------------------------------------------------------------
  def is_svdq(self) -> bool:
    return isinstance(self.quant_type, str) and self.quant_type.lower().startswith("svdq")

  # -- helpers mirrored from the reference ------------------------------------
  def update(self, **kwargs) -> "QuantizeConfig":
    """Sets the given non-None fields in place and re-validates."""
    for key, value in kwargs.items():
      if hasattr(self, key) and value is not None:
        setattr(self, key, value)
    if "backend" not in kwargs:
      self.backend = QuantizeBackend.AUTO
    self.__post_init__()
    return self

  def strify(self) -> str:
    """Short description used in logs and summaries."""
    if self.components_to_quantize is None or isinstance(self.components_to_quantize, list):
      return self.quant_type.lower()
    parts = []
    for component, d in self.components_to_quantize.items():
      parts.append(f"<{component}:{d.get('quant_type', self.quant_type).lower()}>")
    return "".join(parts)

  def component_quant_types(self) -> Dict[str, str]:
    c = self.components_to_quantize
    if c is None:
      return {"transformer": self.quant_type}
    if isinstance(c, list):
      return {name: self.quant_type for name in c}
    if isinstance(c, dict):
      return {name: d.get("quant_type", self.quant_type) for name, d in c.items()}
    raise ValueError("components_to_quantize should be either a list or a dict.")

  @classmethod
  def expand_configs(cls, config: "QuantizeConfig") -> List["QuantizeConfig"]:
    """One config per target component."""
    c = config.components_to_quantize
    if c is None:
      return [config]
    if isinstance(c, list):
      return [dataclasses.replace(config, components_to_quantize=[name]) for name in c]
    if isinstance(c, dict):
      overridable = ("backend", "quant_type", "exclude_layers", "regional_quantize",
                     "repeated_blocks", "filter_fn", "per_tensor_fallback", "precision_plan",
                     "calibrate_fn", "serialize_to", "svdq_kwargs", "verbose")
      out = []
      for name, d in c.items():
        changes = {k: d.get(k, getattr(config, k)) for k in overridable}
        out.append(dataclasses.replace(config, components_to_quantize=[name], **changes))
      return out
    raise ValueError("components_to_quantize should be either a list or a dict.")

  @classmethod
  def from_kwargs(cls, **kwargs) -> "QuantizeConfig":
    """Builds a config from legacy keyword arguments; unknown keys are dropped
    silently (so `quantize(m, config=...)` falls back to the defaults, as it does
    in the reference)."""
    known = {k: v for k, v in kwargs.items() if k in cls.__dataclass_fields__}
    return cls(**known)
