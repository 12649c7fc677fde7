"""Small host-side helpers the quantization path reads
(reference: src/cache_dit/utils.py:153-170 check_quantized, :232-289
parse_extra_modules, :307-318 maybe_empty_cache)."""
from __future__ import annotations

import gc
from typing import Any, List, Union

import torch


def _is_quantized(module: torch.nn.Module) -> bool:
  return bool(getattr(module, "_is_quantized", False))


def check_quantized(module: Union[torch.nn.Module, Any]) -> bool:
  """True if `module` (an nn.Module), or any nn.Module attribute of a pipeline-like
  object (or of its `.pipe`), carries the `_is_quantized` mark."""
  if isinstance(module, torch.nn.Module):
    return _is_quantized(module)
  pipe = getattr(module, "pipe", module)
  if pipe is None:
    return False
  for name in dir(pipe):
    try:
      attr = getattr(pipe, name)
    except Exception:
      continue
    if isinstance(attr, torch.nn.Module) and _is_quantized(attr):
      return True
  return False


def parse_extra_modules(pipe_or_adapter: Any,
                        extra_modules: List[Union[str, torch.nn.Module]]) -> List[torch.nn.Module]:
  """Resolves component names (or module objects) against a pipeline-like object.
  Names that the pipeline does not have are skipped."""
  if isinstance(extra_modules, dict):
    extra_modules = list(extra_modules.keys())
  pipe = getattr(pipe_or_adapter, "pipe", pipe_or_adapter)
  if not extra_modules or pipe is None:
    return []
  found: List[torch.nn.Module] = []
  for item in extra_modules:
    if isinstance(item, torch.nn.Module):
      found.append(item)
    elif isinstance(item, str) and isinstance(getattr(pipe, item, None), torch.nn.Module):
      found.append(getattr(pipe, item))
  return found


def maybe_empty_cache() -> None:
  try:
    gc.collect()
    if torch.cuda.is_available():
      torch.cuda.empty_cache()
  except Exception:
    pass
