"""The part of `enable_cache()` and of the YAML loader that this path owns: the
`quantize_config` plumbing.

`enable_cache(pipe_or_adapter, cache_config=..., parallelism_config=...,
quantize_config=...)` in the reference applies, in this order, cache hooks, the
attention backend, parallelism and then quantization
(src/cache_dit/caching/cache_interface.py:339-464). Caching, attention and
parallelism are not part of this package: they are refused loudly rather than
ignored, so that nobody believes DBCache is active when it is not. What is
reproduced is the quantization step (:433-464): by default every discovered
transformer is quantized; with `components_to_quantize` the config is expanded
into one config per named pipeline component.
"""
from __future__ import annotations

import copy
from typing import Any, List, Optional

import torch

from .logger import init_logger
from .quantization import QuantizeConfig, quantize
from .utils import parse_extra_modules

logger = init_logger(__name__)


def _find_transformers(obj: Any) -> List[tuple]:
  """(owner, attribute name, module) of the transformer(s) of a pipeline-like
  object, the way the reference discovers them (cache_interface.py:377-407):
  `transformer`, then `transformer_2` (Wan 2.2 style two-expert pipelines)."""
  pipe = getattr(obj, "pipe", obj)
  found = []
  for name in ("transformer", "transformer_2"):
    m = getattr(pipe, name, None)
    if isinstance(m, torch.nn.Module):
      found.append((pipe, name, m))
  return found


def enable_cache(pipe_or_adapter: Any,
                 cache_config: Optional[Any] = None,
                 calibrator_config: Optional[Any] = None,
                 params_modifiers: Optional[Any] = None,
                 parallelism_config: Optional[Any] = None,
                 attention_backend: Optional[str] = None,
                 quantize_config: Optional[QuantizeConfig] = None,
                 **kwargs) -> Any:
  """Applies `quantize_config` to a pipeline, a block adapter or a bare
  transformer module and returns the same object. The parameter list is the
  reference's (src/cache_dit/caching/cache_interface.py:26-47), positions included."""
  refused = {
      "cache_config": cache_config,
      "calibrator_config": calibrator_config,
      "params_modifiers": params_modifiers,
      "parallelism_config": parallelism_config,
      "attention_backend": attention_backend,
  }
  given = [k for k, v in refused.items() if v is not None]
  if given or kwargs:
    raise NotImplementedError(
        f"enable_cache: {given + sorted(kwargs)} belong to cache-dit's caching / parallelism / "
        "attention layers, which this package leaves to cache-dit itself; only quantize_config "
        "is handled here.")
  if quantize_config is None:
    return pipe_or_adapter
  assert isinstance(quantize_config, QuantizeConfig), (
      "quantize_config should be an instance of QuantizeConfig.")

  if isinstance(pipe_or_adapter, torch.nn.Module) and not _find_transformers(pipe_or_adapter):
    if quantize_config.components_to_quantize is not None:
      raise ValueError("components_to_quantize needs a pipeline, got a bare module")
    quantize(pipe_or_adapter, quantize_config=quantize_config)
    return pipe_or_adapter

  pipe = getattr(pipe_or_adapter, "pipe", pipe_or_adapter)
  if quantize_config.components_to_quantize is None:
    transformers = _find_transformers(pipe_or_adapter)
    if not transformers:
      raise ValueError("enable_cache: no transformer module found to quantize")
    for owner, name, module in transformers:
      setattr(owner, name, quantize(module, quantize_config=quantize_config))
    return pipe_or_adapter

  for config in QuantizeConfig.expand_configs(quantize_config):
    names = config.components_to_quantize
    components = parse_extra_modules(pipe, names)
    assert len(components) == len(names), (
        f"Some components in quantize_config.components_to_quantize: {names} are not found in "
        "the pipeline, please check the component names or directly pass the actual modules in "
        "components_to_quantize.")
    for component, name in zip(components, names):
      name = getattr(component, "_actual_module_name", name)
      quantized = quantize(component, quantize_config=config)
      if isinstance(name, str):
        setattr(pipe, name, quantized)
  return pipe_or_adapter


def load_quantize_config(path_or_dict, **kwargs) -> Optional[QuantizeConfig]:
  """Reads the `quantize_config` section of a YAML file or dict; keys that are not
  QuantizeConfig fields and None values are dropped; no section -> None
  (reference: src/cache_dit/caching/load_configs.py:359-386)."""
  if isinstance(path_or_dict, str):
    import yaml

    try:
      with open(path_or_dict, "r") as f:
        data = yaml.safe_load(f)
    except FileNotFoundError:
      raise FileNotFoundError(f"Configuration file not found: {path_or_dict}")
    except yaml.YAMLError as e:
      raise yaml.YAMLError(f"YAML file parsing error: {str(e)}")
  elif isinstance(path_or_dict, dict):
    data = copy.deepcopy(path_or_dict)
  else:
    raise ValueError("Input must be a file path (str) or a configuration dictionary (dict).")
  if not data or "quantize_config" not in data:
    return None
  section = data["quantize_config"]
  fields = QuantizeConfig.__dataclass_fields__
  return QuantizeConfig(**{k: v for k, v in section.items() if k in fields and v is not None})
