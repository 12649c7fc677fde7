"""Which nn.Linear gets which quantization: the policy layer of `quantize()`.

Restates the behaviour of the reference's torchao policy module,
src/cache_dit/quantization/torchao/quantize_ao.py -- passes (`quantize_ao`
:74-163), the per-call context (`QuantizeAOContext` :182-512), the guards
(:515-535) and the two layer filters (`_basic_filter_fn` :666-775,
`_fallback_filter_fn` :778-821) -- with the conversion itself done by this
package's HIP-backed Linears instead of `torchao.quantize_`.
"""
from __future__ import annotations

import copy
import dataclasses
import logging
import os
from typing import Callable, Dict, List, Optional

import torch
from torch import nn

from ..logger import init_logger
from ..utils import check_quantized, maybe_empty_cache
from .config import ALLOWED_QUANTIZE_TYPES, BUILT_QUANTIZE_TYPES, QuantizeConfig

logger = init_logger(__name__)

# Order in which the quant types of a precision plan are applied
# (quantize_ao.py:29-40): per-tensor first so that it also takes fallback layers.
PRECISION_PLAN_ORDER = [
    "float8_per_tensor",
    "float8_per_row",
    "float8_per_block",
    "float8_weight_only",
    "nvfp4",
    "nvfp4_weight_only",
    "int8_per_tensor",
    "int8_per_row",
    "int8_weight_only",
    "int4_weight_only",
]

FALLBACK_QUANT_TYPE = "float8_per_tensor"

#: (linear, quant_type) -> None; replaces the Linear's weight in place
ConvertFn = Callable[[nn.Linear, str], None]


def _default_convert(linear: nn.Linear, quant_type: str) -> None:
  from ..nn import convert_linear_

  convert_linear_(linear, quant_type)


def _env_flag(name: str) -> bool:
  return os.environ.get(name, "0").lower() in ("1", "true", "yes", "on")


@dataclasses.dataclass
class QuantizeContext:
  """State of one quantize() call: normalised settings plus the statistics the
  summary prints."""
  module_ref: Optional[nn.Module] = None
  quant_type: str = "float8_per_row"
  regional_quantize: bool = True
  repeated_blocks: Optional[List[str]] = None
  exclude_layers: List[str] = dataclasses.field(default_factory=list)
  per_tensor_fallback: bool = True
  precision_plan: Optional[Dict[str, str]] = None
  verbose: bool = False
  kwargs: dict = dataclasses.field(default_factory=dict)
  # statistics
  num_linear_layers: int = 0
  fallback_layers: List[str] = dataclasses.field(default_factory=list)
  rowwise_layers: List[str] = dataclasses.field(default_factory=list)
  quantized_map: Dict[str, int] = dataclasses.field(
      default_factory=lambda: {t: 0
                               for t in ALLOWED_QUANTIZE_TYPES})
  skipped_map: Dict[str, List[str]] = dataclasses.field(
      default_factory=lambda: {t: []
                               for t in ALLOWED_QUANTIZE_TYPES})
  # precision plan, inverted: quant_type -> [layer-name substrings]
  reverse_precision_plan: Dict[str, List[str]] = dataclasses.field(default_factory=dict)
  layers_allowed_to_quantize: Optional[List[str]] = None
  precision_plan_pass_applied: bool = False
  first_quantize_pass_applied: bool = False

  def __post_init__(self):
    self.quant_type = self.quant_type.lower()
    assert self.quant_type in ALLOWED_QUANTIZE_TYPES, (
        f"quant_type {self.quant_type} is not supported, allowed quantization "
        f"types: {ALLOWED_QUANTIZE_TYPES}.")
    if self.exclude_layers is None:
      self.exclude_layers = []

  # -- construction -----------------------------------------------------------
  @staticmethod
  def from_config(quantize_config: QuantizeConfig, module: nn.Module,
                  **kwargs) -> "QuantizeContext":
    return QuantizeContext(
        module_ref=module,
        quant_type=quantize_config.quant_type,
        regional_quantize=quantize_config.regional_quantize,
        repeated_blocks=quantize_config.repeated_blocks,
        exclude_layers=quantize_config.exclude_layers,
        precision_plan=quantize_config.precision_plan,
        per_tensor_fallback=quantize_config.per_tensor_fallback,
        verbose=quantize_config.verbose,
        kwargs=copy.deepcopy(kwargs),
    ).normalize()

  def normalize(self) -> "QuantizeContext":
    if self.precision_plan:
      inverted: Dict[str, List[str]] = {}
      for layer_name, qt in self.precision_plan.items():
        qt = qt.lower()
        assert qt in ALLOWED_QUANTIZE_TYPES, (
            f"quant_type {qt} in precision_plan is not supported, allowed "
            f"quantization types: {ALLOWED_QUANTIZE_TYPES}.")
        inverted.setdefault(qt, [])
        if layer_name not in inverted[qt]:
          inverted[qt].append(layer_name)
      self.reverse_precision_plan = {k: v for k, v in inverted.items() if v}

    self._collect_rowwise_layers()

    # a diffusers transformer names its repeated block classes itself
    self.repeated_blocks = getattr(self.module_ref, "_repeated_blocks",
                                   self.repeated_blocks if self.repeated_blocks else None)
    if self.repeated_blocks is None:
      self.regional_quantize = False

    if self.module_ref is not None and self.is_float8_per_row():
      for name, sub in self.module_ref.named_modules():
        if isinstance(sub, nn.Linear) and not getattr(sub, "_is_inner_quantized", False):
          assert sub.weight.dtype == torch.bfloat16, (
              f"Per-row quantization is only supported for linear layers with "
              f"weight dtype of bfloat16, but found dtype {sub.weight.dtype} "
              f"in layer {name}.")

    if self.required_fallback() and self.fallback_layers and self.precision_plan is not None:
      # with a precision plan the fallback layers simply join the per-tensor plan
      merged = self.reverse_precision_plan.get(FALLBACK_QUANT_TYPE, []) + self.fallback_layers
      self.reverse_precision_plan[FALLBACK_QUANT_TYPE] = list(dict.fromkeys(merged))
      self.fallback_layers = []
      logger.info("precision_plan is specified, the fallback layers will be merged "
                  "into the float8_per_tensor plan.")
    return self

  def _collect_rowwise_layers(self) -> None:
    """Layers a tensor-parallel planner marked row-parallel (`_rowwise_layers` on
    the module) cannot take per-row scales in the reference: they fall back to
    per-tensor, or are excluded when the fallback is off. Single-GPU modules
    never carry the attribute."""
    exclude = list(self.exclude_layers)
    fallback = list(self.fallback_layers)
    rowwise: List[str] = list(self.rowwise_layers)
    if self.module_ref is not None and (self.is_float8_per_row()
                                        or self.precision_plan is not None):
      if not _env_flag("CACHE_DIT_DISABLE_EXCLUDE_FOR_QUANTIZE_AFTER_TP"):
        rowwise = list(getattr(self.module_ref, "_rowwise_layers", []))
        if rowwise:
          if self.per_tensor_fallback:
            fallback = fallback + rowwise
          else:
            exclude = exclude + rowwise
    self.rowwise_layers = rowwise
    self.exclude_layers = exclude
    self.fallback_layers = fallback

  # -- predicates --------------------------------------------------------------
  def is_float8_per_row(self) -> bool:
    return self.quant_type == "float8_per_row"

  def is_float8(self) -> bool:
    return "float8" in self.quant_type

  def is_weight_only(self) -> bool:
    return "weight_only" in self.quant_type

  def required_fallback(self) -> bool:
    return bool(self.per_tensor_fallback
                and self.quant_type in ("float8_per_row", "float8_per_tensor", "float8_per_block")
                and self.regional_quantize and self.fallback_layers)

  @staticmethod
  def _matches(name: str, patterns: Optional[List[str]]) -> Optional[str]:
    for p in patterns or []:
      if p in name:
        return p
    return None

  def is_fallback_layer(self, name: str) -> bool:
    return self.required_fallback() and self._matches(name, self.fallback_layers) is not None

  def is_exclude_layer(self, name: str) -> bool:
    return self._matches(name, self.exclude_layers) is not None

  def is_rowwise_layer(self, name: str) -> bool:
    return self._matches(name, self.rowwise_layers) is not None

  @staticmethod
  def is_quantized_layer(m: nn.Module) -> bool:
    return bool(getattr(m, "_is_inner_quantized", False))

  def get_exclude_name(self, name: str) -> Optional[str]:
    if self.is_rowwise_layer(name):
      return "RowwiseParallel"
    return self._matches(name, self.exclude_layers)

  # -- reporting ----------------------------------------------------------------
  @property
  def quantized_region(self) -> str:
    if self.regional_quantize and self.repeated_blocks is not None:
      shown = list(self.repeated_blocks[:2])
      if len(self.repeated_blocks) > 2:
        shown.append("...")
      return str(shown)
    return self.module_ref.__class__.__name__ if self.module_ref is not None else "Module"

  def summary_lines(self) -> List[str]:
    """The summary table, one string per row (same rows and column layout as the
    reference logs at quantize_ao.py:274-334)."""
    total_q = sum(self.quantized_map.values())
    total_s = sum(len(v) for v in self.skipped_map.values())
    wk = max(len(k) for k in self.quantized_map)
    wc = max(len(str(v)) for v in self.quantized_map.values()) + 3
    rows = [f"Quantized        Region: {self.quantized_region}"]
    for qt, n in self.quantized_map.items():
      if n > 0:
        rows.append(f"Quantized Linear Layers: {n:<{wc}} {qt:<{wk}} "
                    f"{len(self.skipped_map.get(qt, []))} (skipped)")
    rows.append(f"Quantized Linear Layers: {total_q:<{wc}} (total)")
    rows.append(f"Skipped   Linear Layers: {total_s:<{wc}} (total)")
    rows.append(f"Linear           Layers: {self.num_linear_layers:<{wc}} (total)")
    if self.verbose and logger.isEnabledFor(logging.DEBUG):
      rows.append(f"Skipped        Patterns: {self.exclude_layers}")
    return rows

  def skipped_reason_lines(self) -> List[str]:
    """Per (quant type, skip pattern) counts, shown in verbose mode."""
    counts: Dict[str, int] = {}
    for qt, reasons in self.skipped_map.items():
      for reason in reasons:
        key = f"{qt}, {reason}"
        counts[key] = counts.get(key, 0) + 1
    if not counts:
      return []
    split = {k: [p.strip() for p in k.split("->")] for k in counts}
    wn = max(len(v[0]) for v in split.values())
    wp = max(len(v[1]) for v in split.values())
    return [f"{split[k][0].ljust(wn)}: {split[k][1].ljust(wp)}: {n:<4} layers"
            for k, n in counts.items()]

  def summary(self) -> None:

    def box(lines: List[str]) -> None:
      width = max(len(s) for s in lines) + 2
      logger.info("-" * width)
      logger.info("\n".join(s.ljust(width) + "|" for s in lines))
      logger.info("-" * width)

    box(self.summary_lines())
    if self.verbose:
      reasons = self.skipped_reason_lines()
      if reasons:
        box(reasons)


# ------------------------------------------------------------------------------- filters


def basic_filter(m: nn.Module, name: str, ctx: QuantizeContext,
                 override_quant_type: Optional[str] = None) -> bool:
  """True if Linear `m` (block-relative name `name`) is to be quantized in the
  current pass; records statistics and skip reasons as it goes."""
  qt = override_quant_type if override_quant_type is not None else ctx.quant_type
  if ctx.is_quantized_layer(m) or not isinstance(m, nn.Linear):
    return False

  def skip(pattern: str) -> bool:
    reason = f"skip: {name} -> pattern<{pattern}>"
    ctx.skipped_map[qt].append(reason)
    logger.debug(reason)
    return False

  if not ctx.first_quantize_pass_applied:
    ctx.num_linear_layers += 1

  # A plan pass only takes the layers its quant type names; layers outside every
  # plan wait for the default pass (and are not reported as skipped here).
  if ctx.precision_plan is not None and not ctx.precision_plan_pass_applied:
    allowed = ctx.layers_allowed_to_quantize
    if allowed and ctx._matches(name, allowed) is None:
      return False

  if ctx.is_exclude_layer(name) or ctx.is_fallback_layer(name):
    if not ctx.is_fallback_layer(name):  # fallback layers are taken by the second pass
      return skip(str(ctx.get_exclude_name(name)))
    return False

  if qt == "float8_per_row" and m.weight.dtype != torch.bfloat16:
    return skip(f"dtype({m.weight.dtype})!=bfloat16")

  if qt in ("nvfp4", "nvfp4_weight_only"):
    shape = tuple(m.weight.shape)
    if shape[-2] % 16 != 0 or shape[-1] % 16 != 0:
      return skip(f"weight_shape{shape}%16!=0")
    if qt == "nvfp4" and (shape[-2] <= 64 or (shape[-1] <= 1024 and shape[-2] <= 1024)):
      return skip(f"weight_shape{shape} is too small")

  if qt == "float8_per_block":
    shape = tuple(m.weight.shape)
    if shape[-2] % 128 != 0 or shape[-1] % 128 != 0:
      return skip(f"w{shape} % blocksize(128, 128) != 0")

  if qt in ("float8_per_row", "float8_per_tensor", "float8_per_block") and not _bias_ok(m):
    return skip("_scaled_mm: DTensor + bias NOT supported")

  incompatible = _kernel_incompatibility(m, qt)
  if incompatible is not None:
    return skip(incompatible)

  m._is_inner_quantized = True
  ctx.quantized_map[qt] += 1
  return True


def fallback_filter(m: nn.Module, name: str, ctx: QuantizeContext) -> bool:
  """Second pass: takes exactly the fallback layers the first pass left alone."""
  if ctx.is_quantized_layer(m) or not isinstance(m, nn.Linear):
    return False
  if not ctx.is_fallback_layer(name):
    if not ctx.is_exclude_layer(name):
      reason = f"fallback: {name} -> pattern<NOT in fallback layers>"
      ctx.skipped_map[FALLBACK_QUANT_TYPE].append(reason)
      logger.debug(reason)
    return False
  if not _bias_ok(m):
    reason = f"fallback: {name} -> pattern<_scaled_mm: DTensor + bias NOT supported>"
    ctx.skipped_map[FALLBACK_QUANT_TYPE].append(reason)
    logger.debug(reason)
    return False
  incompatible = _kernel_incompatibility(m, FALLBACK_QUANT_TYPE)
  if incompatible is not None:
    reason = f"fallback: {name} -> pattern<{incompatible}>"
    ctx.skipped_map[FALLBACK_QUANT_TYPE].append(reason)
    logger.debug(reason)
    return False
  m._is_inner_quantized = True
  ctx.quantized_map[FALLBACK_QUANT_TYPE] += 1
  return True


def _kernel_incompatibility(m: nn.Linear, qt: str) -> Optional[str]:
  """Why the FP8 kernels cannot take Linear `m` under quant type `qt` (None if they
  can). The reference hands every layer to torchao, whose FP8 configs leave a layer
  they cannot run unquantized without raising; here such a layer is skipped with a
  reason before anything about it is recorded, for every quant type that has a
  kernel: both weight dimensions multiples of 16, bf16 weight and bias."""
  if qt not in BUILT_QUANTIZE_TYPES:
    return None
  shape = tuple(m.weight.shape)
  if shape[-2] % 16 != 0 or shape[-1] % 16 != 0:
    return f"weight_shape{shape}%16!=0"
  if m.weight.dtype != torch.bfloat16:
    return f"dtype({m.weight.dtype})!=bfloat16"
  bias = getattr(m, "bias", None)
  if bias is not None and bias.dtype != torch.bfloat16:
    return f"bias_dtype({bias.dtype})!=bfloat16"
  return None


def _bias_ok(m: nn.Linear) -> bool:
  """A DTensor weight or bias together with a bias is refused (distributed only)."""
  if not (torch.distributed.is_available() and torch.distributed.is_initialized()):
    return True
  if getattr(m, "bias", None) is None:
    return True
  from torch.distributed.tensor import DTensor

  return not isinstance(m.weight, DTensor) and not isinstance(m.bias, DTensor)


# ------------------------------------------------------------------------------- passes


def _apply(root: nn.Module, quant_type: str, filter_fn: Callable[[nn.Module, str], bool],
           convert: ConvertFn) -> None:
  """Walks `root` depth first with names relative to it (the root itself has the
  empty name) and converts every module the filter accepts."""

  def walk(m: nn.Module, fqn: str) -> None:
    if filter_fn(m, fqn):
      convert(m, quant_type)  # type: ignore[arg-type]
      return
    for child_name, child in m.named_children():
      walk(child, f"{fqn}.{child_name}" if fqn else child_name)

  walk(root, "")


def _check_can_quantize(module: nn.Module) -> bool:
  if check_quantized(module):
    logger.warning(f"Module {module.__class__.__name__} is already quantized, skipping. ")
    return False
  assert isinstance(module, nn.Module)
  return True


def _check_platform(ctx: QuantizeContext) -> None:
  """The reference asserts a CUDA platform (quantize_ao.py:527-528), an importable
  backend (:529-533) and, for FP8, compute capability >= (8, 9) (:231-236). On
  ROCm PyTorch the device type is "cuda" as well; gfx950 reports (9, 5)."""
  from .. import _native

  assert torch.cuda.is_available(), (
      "Quantization functionality with the HIP backend is only supported on GPU devices.")
  if not _native.is_built():
    raise ImportError("Quantization needs libcdit_hip.so; build it with "
                      "`python -m cache_dit_amd.csrc.build`.")
  if ctx.is_float8():
    cap = torch.cuda.get_device_capability()
    assert cap >= (8, 9), f"FP8 requires a GPU with FP8 matrix cores, but got capability {cap}"
    _native.device_arch()  # raises unless the device is a gfx950


def _check_dtype_overrides(kwargs: dict) -> None:
  """`weight_dtype` / `activation_dtype` reach torchao's FP8 configs in the reference
  (quantize_ao.py:548-555, :565-572, :604-607; default float8_e4m3fn). The kernels
  here encode OCP e4m3fn only, so any other request is refused instead of being
  quietly served as e4m3fn."""
  for key in ("weight_dtype", "activation_dtype"):
    dt = kwargs.get(key, torch.float8_e4m3fn)
    if dt is None or dt == torch.float8_e4m3fn or dt == "float8_e4m3fn":
      continue
    raise NotImplementedError(
        f"{key}={dt} is not built in this MI355X implementation: the quantizer and the GEMMs "
        "encode torch.float8_e4m3fn only")


def quantize_ao(module: nn.Module, quantize_config: QuantizeConfig,
                _convert_fn: Optional[ConvertFn] = None, **kwargs) -> nn.Module:
  """Applies `quantize_config` to `module` in place.

  `_convert_fn` replaces the Linear conversion (tests use it to exercise the
  policy without a GPU); when it is given the platform checks are skipped too.
  """
  if not _check_can_quantize(module):
    return module
  ctx = QuantizeContext.from_config(quantize_config, module, **kwargs)
  _check_dtype_overrides(ctx.kwargs)
  convert_impl = _convert_fn
  if convert_impl is None:
    _check_platform(ctx)

    def convert_impl(linear: nn.Linear, qt: str) -> None:
      if qt not in BUILT_QUANTIZE_TYPES:
        raise NotImplementedError(
            f"quant_type {qt!r} has no MI355X kernel in this build (built: "
            f"{BUILT_QUANTIZE_TYPES})")
      _default_convert(linear, qt)

  def convert(linear: nn.Linear, qt: str) -> None:
    # the filter has already booked the layer as quantized: take that back when the
    # conversion fails, so that a caller who catches the error sees true bookkeeping
    try:
      convert_impl(linear, qt)
    except BaseException:
      if getattr(linear, "_is_inner_quantized", False):
        del linear._is_inner_quantized
      ctx.quantized_map[qt] -= 1
      raise

  def basic(qt_override: Optional[str] = None):
    return lambda m, name: basic_filter(m, name, ctx, qt_override)

  def regions():
    return [m for m in module.modules() if m.__class__.__name__ in ctx.repeated_blocks]

  if ctx.regional_quantize:
    assert ctx.repeated_blocks is not None, (
        "repeated_blocks must be specified when regional_quantize is True.")
    touched = False
    if ctx.precision_plan is not None:
      logger.debug(f"Precision plan is enabled with the following plan: {ctx.precision_plan}")
      for qt in PRECISION_PLAN_ORDER:
        names = ctx.reverse_precision_plan.get(qt, [])
        if not names:
          continue
        ctx.layers_allowed_to_quantize = names
        for block in regions():
          _apply(block, qt, basic(qt), convert)
          touched = True
        ctx.first_quantize_pass_applied = True
      # default pass: everything no plan entry named
      ctx.precision_plan_pass_applied = True
      ctx.layers_allowed_to_quantize = None
      for block in regions():
        _apply(block, ctx.quant_type, basic(), convert)
        touched = True
    else:
      for block in regions():
        _apply(block, ctx.quant_type, basic(), convert)
        touched = True
      ctx.first_quantize_pass_applied = True
      if ctx.required_fallback():
        for block in regions():
          _apply(block, FALLBACK_QUANT_TYPE, lambda m, name: fallback_filter(m, name, ctx),
                 convert)
          touched = True
    if not touched:
      raise ValueError(f"Regional quantization failed because {ctx.repeated_blocks} "
                       "classes are not found in the module.")
  else:
    _apply(module, ctx.quant_type, basic(), convert)

  maybe_empty_cache()
  ctx.summary()

  module._is_quantized = True
  module._quantize_config = quantize_config
  module._quantize_type = ctx.quant_type
  module._exclude_layers = ctx.exclude_layers
  module._quantize_context = ctx
  return module
