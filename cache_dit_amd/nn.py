"""Quantized nn.Linear modules: the counterpart of torchao's Float8Tensor
`aten.linear` override that cache-dit installs with `quantize_`
(src/cache_dit/quantization/torchao/quantize_ao.py:166-179).

Conversion is in place: the nn.Linear object keeps its identity (parents, hooks
and block adapters that hold a reference keep working, and
`isinstance(m, nn.Linear)` stays true, which the reference's filter relies on);
its class is switched to a subclass whose forward calls the HIP kernels, its
`weight` becomes the e4m3 codes [N,K] and a `weight_scale` buffer [N,1] holds
the per-output-channel fp32 scales.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from . import _native, ops

FP8 = torch.float8_e4m3fn

#: scale rounding used for activations and weights (see ops.fp8_rowwise_quant)
DEFAULT_SCALE_MODE = "bf16div"


def _quantize_weight(weight: torch.Tensor, scale_mode: str, per_tensor: bool = False):
  """W bf16 [N,K] -> (codes e4m3 [N,K], scale fp32 [N,1]) with the HIP quantizer.

  The reference quantizes the weight wherever it lives, and its CLI flow does so
  before `pipe.to(device)` (src/cache_dit/_utils/utils.py:2419,2459). There is no
  CPU kernel here, so a CPU weight makes a round trip through the GPU.
  """
  if weight.dtype != torch.bfloat16:
    raise ValueError(f"weight must be bfloat16 to be quantized to FP8, got {weight.dtype}")
  src = weight.detach()
  if not src.is_cuda:
    if not torch.cuda.is_available():
      raise RuntimeError("quantizing a CPU weight needs a GPU to run the quantizer kernel on; "
                         "there is no CPU path")
    src = src.to("cuda")
  quant = ops.fp8_tensorwise_quant if per_tensor else ops.fp8_rowwise_quant
  q, s = quant(src.contiguous(), scale_mode)
  return q.to(weight.device), s.to(weight.device)


class _Fp8LinearBase(nn.Linear):
  """Common state of the two quantized Linears. Never constructed directly:
  `convert_linear_` re-classes an existing nn.Linear."""

  weight_scale: torch.Tensor
  share_input_quant: bool = False
  epilogue: int
  scale_mode: str
  quant_type: str

  def extra_repr(self) -> str:
    return (f"in_features={self.in_features}, out_features={self.out_features}, "
            f"bias={self.bias is not None}, quant_type={self.quant_type}, "
            f"epilogue={'gelu_tanh' if self.epilogue & _native.EPI_GELU_TANH else 'none'}")

  def _check_input(self, x: torch.Tensor) -> None:
    if x.dtype != torch.bfloat16:
      raise ValueError(f"{type(self).__name__} takes bfloat16 activations, got {x.dtype}")
    if not x.is_cuda:
      raise RuntimeError(f"{type(self).__name__}: input is on {x.device}; there is no CPU path")


class Fp8DynamicLinear(_Fp8LinearBase):
  """`float8_per_row` (w8a8 dynamic): per-token e4m3 activation quantization,
  e4m3 x e4m3 GEMM with fp32 accumulate, per-token x per-channel scales, bias,
  optional fused GELU-tanh, bf16 out.

  Every forward is one `torch.ops.cdit.*` call, so Dynamo and Inductor see a single
  opaque node with a fake implementation, the way the reference keeps this path
  traceable (src/cache_dit/quantization/torchao/_scaled_mm.py:94-137, :338-357)."""

  def forward(self, x: torch.Tensor) -> torch.Tensor:
    self._check_input(x)
    # sharing keeps the last activation's codes alive between calls; a compiled graph gets
    # the stateless form (its front end owns the memory its graphs are captured into)
    share = self.share_input_quant and not torch.compiler.is_compiling()
    return torch.ops.cdit.linear_w8a8(x, self.weight, self.weight_scale, self.bias,
                                      self._scale_mode_id, self.epilogue,
                                      ops.GRANULARITY_PER_ROW, share)


class Fp8DynamicLinearPerTensor(_Fp8LinearBase):
  """`float8_per_tensor` (w8a8 dynamic, one scale per tensor): the activation is
  quantized with a single scale computed from its global amax, the weight likewise
  at conversion time; `weight_scale` [N,1] then holds N copies of the weight's scale
  and the GEMM is the per-row one fed with constant scales."""

  def forward(self, x: torch.Tensor) -> torch.Tensor:
    self._check_input(x)
    return torch.ops.cdit.linear_w8a8(x, self.weight, self.weight_scale, self.bias,
                                      self._scale_mode_id, self.epilogue,
                                      ops.GRANULARITY_PER_TENSOR, False)


class Fp8WeightOnlyLinear(_Fp8LinearBase):
  """`float8_weight_only` (w8a16): bf16 activations, e4m3 weights dequantized in
  the GEMM mainloop, per-channel scale in the epilogue."""

  def forward(self, x: torch.Tensor) -> torch.Tensor:
    self._check_input(x)
    return torch.ops.cdit.w8a16_mm(x, self.weight.t(), self.weight_scale, self.bias,
                                   _native.DT_BF16, self.epilogue)


_CLASS_OF = {
    "float8_per_row": Fp8DynamicLinear,
    "float8_per_tensor": Fp8DynamicLinearPerTensor,
    "float8_weight_only": Fp8WeightOnlyLinear,
}


def convert_linear_(linear: nn.Linear,
                    quant_type: str,
                    scale_mode: str = DEFAULT_SCALE_MODE,
                    gelu_tanh: bool = False) -> nn.Linear:
  """Quantizes `linear` in place and returns it (same object)."""
  cls = _CLASS_OF.get(quant_type)
  if cls is None:
    raise NotImplementedError(
        f"quant_type {quant_type!r} is not built in this MI355X implementation; built: "
        f"{sorted(_CLASS_OF)}")
  if isinstance(linear, _Fp8LinearBase):
    return linear
  if type(linear) is not nn.Linear and type(linear).forward is not nn.Linear.forward:
    raise TypeError(f"cannot convert {type(linear).__name__}: it overrides nn.Linear.forward")
  if linear.in_features % 16 != 0 or linear.out_features % 16 != 0:
    raise ValueError(f"FP8 matmul needs in/out features that are multiples of 16, got "
                     f"{linear.in_features}x{linear.out_features}")
  q, s = _quantize_weight(linear.weight, scale_mode, per_tensor=quant_type == "float8_per_tensor")
  bias = linear.bias
  del linear.weight
  linear.weight = nn.Parameter(q, requires_grad=False)
  linear.register_buffer("weight_scale", s.reshape(-1, 1).contiguous())
  if bias is not None:
    if bias.dtype != torch.bfloat16:
      raise ValueError(f"bias must be bfloat16, got {bias.dtype}")
    linear.bias = nn.Parameter(bias.detach().contiguous(), requires_grad=False)
  linear.epilogue = _native.EPI_GELU_TANH if gelu_tanh else _native.EPI_NONE
  linear.scale_mode = scale_mode
  linear._scale_mode_id = _native.SCALE_MODE_IDS[scale_mode]
  linear.quant_type = quant_type
  linear.__class__ = cls
  return linear


def fuse_gelu_tanh_(linear: nn.Linear, act: nn.Module) -> None:
  """Moves a following nn.GELU(approximate="tanh") into `linear`'s epilogue and
  turns `act` into an identity, the way the reference wires its fused GELU MLP
  (src/cache_dit/quantization/svdquant/passes.py:489-511). The fused result
  applies GELU to the fp32 accumulator, one bf16 rounding less than the unfused
  pair."""
  if not isinstance(linear, _Fp8LinearBase):
    raise TypeError("fuse_gelu_tanh_ expects an already quantized Linear")
  if not (isinstance(act, nn.GELU) and act.approximate == "tanh"):
    raise TypeError("fuse_gelu_tanh_ expects nn.GELU(approximate='tanh')")
  linear.epilogue |= _native.EPI_GELU_TANH
  act.forward = lambda x: x  # type: ignore[method-assign]
  act._cdit_fused_into_linear = True  # type: ignore[attr-defined]


def share_activation_quant_(module: nn.Module, enable: bool = True) -> int:
  """Lets every `float8_per_row` Linear under `module` reuse the activation codes of
  the previous Linear on the stream when it is handed the very same, unmodified
  input buffer (q/k/v projections, FLUX `proj_mlp` + q/k/v): one quantizer launch
  per distinct input instead of one per Linear, with bit-identical outputs. Returns
  the number of Linears switched."""
  n = 0
  for m in module.modules():
    if isinstance(m, Fp8DynamicLinear):
      m.share_input_quant = bool(enable)
      n += 1
  if not enable:
    ops.clear_shared_activation_quant()
  return n


def dequantize_weight(linear: _Fp8LinearBase) -> torch.Tensor:
  """bf16 view of the quantized weight (for inspection and tests)."""
  return (linear.weight.to(torch.float32) * linear.weight_scale).to(torch.bfloat16)
