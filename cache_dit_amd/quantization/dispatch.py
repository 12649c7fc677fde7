"""`quantize()` / `remove_quantization_stats()`: the public entry points
(reference: src/cache_dit/quantization/dispatch.py:11-60 and :93-136)."""
from __future__ import annotations

import copy
from typing import Optional

import torch

from ..logger import init_logger
from .backend import QuantizeBackend
from .config import QuantizeConfig

logger = init_logger(__name__)


def quantize(
    module: torch.nn.Module,
    quantize_config: Optional[QuantizeConfig] = None,
    **kwargs,
) -> torch.nn.Module:
  """Quantizes `module` in place and returns it.

  Accepts the config positionally or as `quantize_config=`; without a config the
  legacy keyword form `quantize(m, quant_type=..., exclude_layers=[...])` is
  converted with `QuantizeConfig.from_kwargs` (with a deprecation warning) and no
  arguments at all is a ValueError.
  """
  if quantize_config is None:
    if not kwargs:
      raise ValueError("quantize_config should be specified for quantization.")
    logger.warning("The quantization arguments in kwargs will be deprecated, "
                   "please use QuantizeConfig to specify quantization configurations.")
    quantize_config = QuantizeConfig.from_kwargs(**kwargs)
  elif kwargs:
    logger.warning("The quantization arguments in kwargs will be ignored since "
                   "quantize_config is specified, please use QuantizeConfig to "
                   "specify quantization configurations.")

  if quantize_config.backend == QuantizeBackend.TORCHAO:
    from .policy import quantize_ao

    return quantize_ao(module, quantize_config, **kwargs)
  raise ValueError(f"backend: {quantize_config.backend} is not supported now!")


def load(module: torch.nn.Module, quantize_config_or_path) -> torch.nn.Module:
  """Serialized quantized checkpoints exist only for SVDQuant in the reference
  (dispatch.py:63-90); the FP8 modes are always quantized online."""
  raise NotImplementedError("load() serves SVDQuant checkpoints only, which are not built here; "
                            "the FP8 modes quantize online with quantize().")


_STAT_ATTRS = ("_quantize_config", "_is_quantized", "_quantize_type", "_exclude_layers")


def remove_quantization_stats(module: torch.nn.Module) -> torch.nn.Module:
  """Deletes the bookkeeping attributes quantize() leaves on a module (and, one
  level deep, on the extra components its config named)."""
  components = None
  if hasattr(module, "_quantize_config"):
    components = copy.deepcopy(module._quantize_config.components_to_quantize)

  def strip(m: torch.nn.Module) -> None:
    for attr in _STAT_ATTRS:
      if hasattr(m, attr):
        delattr(m, attr)

  strip(module)
  if components is not None:
    from ..utils import parse_extra_modules

    for extra in parse_extra_modules(module, components):
      strip(extra)
  return module
