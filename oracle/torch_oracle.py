"""CPU oracle in eager PyTorch ops. TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Restates, with ordinary CPU tensor ops, what cache-dit's `float8_per_row` and
`float8_weight_only` modes compute. cache-dit holds only the call sites; the
arithmetic is torchao's (>= 0.17, not vendored: /root/reference/pyproject.toml:30-34)
and torch._scaled_mm's. Each function cites the call site it serves.

Parity status: the e4m3 cast, clamp, amax, matmul and GELU are PyTorch library
routines here, so they are pinned by construction; the one choice the
reference's text does not fix -- whether `amax / 448` is rounded to bf16 before
it is widened to fp32 -- is "parity unpinned" and selectable through
``scale_mode`` ("bf16div", the eager behaviour of an un-upcast bf16 division,
is the default; "fp32div" keeps the quotient in fp32).

This module is also what bench.py times as the CPU baseline ("port").
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

FP8_MAX = 448.0
SCALE_MODES = ("bf16div", "fp32div")


def choose_scale_rowwise(x: torch.Tensor, scale_mode: str = "bf16div") -> torch.Tensor:
  """Per-row scale [..., 1] fp32 of a bf16 tensor.

  torchao `_choose_scale_float8(x, block_size=(1,..,1,K), float8_e4m3fn)` wrapped
  by cache-dit's zero-scale patch
  (src/cache_dit/quantization/torchao/quantize_ao.py:43-71).
  """
  assert scale_mode in SCALE_MODES, scale_mode
  amax = x.abs().amax(dim=-1, keepdim=True)  # in x's dtype: exact
  if scale_mode == "bf16div":
    scale = (amax / FP8_MAX).to(torch.float32)  # bf16 / python scalar stays bf16
  else:
    scale = amax.to(torch.float32) / FP8_MAX
  return torch.where(scale == 0, torch.ones_like(scale), scale)


def quantize_affine_float8(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
  """torchao `_quantize_affine_float8`: true division, clamp, RNE cast.

  Reached through `Float8Tensor.from_hp(...)`, call site
  tests/kernels/test_opaque_scaled_mm.py:68-73.
  """
  y = x.to(torch.float32) / scale
  y = y.clamp(min=-FP8_MAX, max=FP8_MAX)
  return y.to(torch.float8_e4m3fn)


def quantize_rowwise(x: torch.Tensor,
                     scale_mode: str = "bf16div") -> Tuple[torch.Tensor, torch.Tensor]:
  """x bf16 [..., K] -> (codes float8_e4m3fn [..., K], scale fp32 [..., 1])."""
  scale = choose_scale_rowwise(x, scale_mode)
  return quantize_affine_float8(x, scale), scale


def choose_scale_tensorwise(x: torch.Tensor, scale_mode: str = "bf16div") -> torch.Tensor:
  """One fp32 scale (shape [1, 1]) for the whole bf16 tensor: torchao
  `_choose_scale_float8` with `PerTensor()` granularity, the config built at
  src/cache_dit/quantization/torchao/quantize_ao.py:559-575, under the same
  zero-scale patch (:43-71)."""
  assert scale_mode in SCALE_MODES, scale_mode
  amax = x.abs().amax().reshape(1, 1)
  if scale_mode == "bf16div":
    scale = (amax / FP8_MAX).to(torch.float32)
  else:
    scale = amax.to(torch.float32) / FP8_MAX
  return torch.where(scale == 0, torch.ones_like(scale), scale)


def quantize_tensorwise(x: torch.Tensor,
                        scale_mode: str = "bf16div") -> Tuple[torch.Tensor, torch.Tensor]:
  """x bf16 [M, K] -> (codes float8_e4m3fn [M, K], scale fp32 [M, 1] with every
  entry equal to the tensor's scale: the layout the GEMM entry point takes)."""
  scale = choose_scale_tensorwise(x, scale_mode)
  return quantize_affine_float8(x, scale), scale.expand(x.shape[0], 1).contiguous()


def ln_modulate(x: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor,
                eps: float = 1e-6) -> torch.Tensor:
  """The modulated activation of a DiT block as eager bf16 tensor ops compute it:
  LayerNorm without affine parameters (fp32 statistics, bf16 result), then
  `* (1 + scale) + shift` with every bf16 op rounding its result -- diffusers'
  AdaLayerNormZeroSingle / AdaLayerNormZero, whose output feeds proj_mlp and
  attn.to_q/k/v (src/cache_dit/caching/patch_functors/functor_flux.py:60-67).
  x bf16 [..., K]; shift, scale bf16 broadcastable to x."""
  K = x.shape[-1]
  n = torch.nn.functional.layer_norm(x.to(torch.float32), (K, ), eps=eps).to(x.dtype)
  return n * (1 + scale) + shift


def ln_modulate_quant(x: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor, eps: float = 1e-6,
                      scale_mode: str = "bf16div"):
  """(y, codes, scales): the modulated activation and its per-row quantization."""
  y = ln_modulate(x, shift, scale, eps)
  q, s = quantize_rowwise(y, scale_mode)
  return y, q, s


def gelu_tanh(v: torch.Tensor) -> torch.Tensor:
  return torch.nn.functional.gelu(v, approximate="tanh")


def scaled_mm_rowwise(a_q: torch.Tensor,
                      a_scale: torch.Tensor,
                      b_q: torch.Tensor,
                      b_scale: torch.Tensor,
                      bias: Optional[torch.Tensor] = None,
                      gelu: Optional[str] = None,
                      out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
  """Row-wise scaled FP8 matmul, fp32 accumulate, out_dtype (bf16, fp16 or fp32) out.

  `torch._scaled_mm(a, b.t(), scale_a[M,1], scale_b[1,N], bias, out_dtype=bf16)` as
  called at src/cache_dit/quantization/torchao/_scaled_mm.py:62-91 (the CPU backend
  of _scaled_mm only takes per-tensor scales, so the scales are applied outside).
  a_q [M,K], b_q [N,K] float8_e4m3fn; a_scale [M,1], b_scale [N,1] or [N] fp32.
  gelu: None, "fused" (on the fp32 value) or "unfused" (on the rounded output, as a
  separate nn.GELU module does).
  An fp32 output gets its bias the way the reference adds it, after the matmul
  (`output + bias`, _scaled_mm.py:71-81): the same value, the sum of two fp32 numbers
  rounded once.
  """
  acc = a_q.to(torch.float32) @ b_q.to(torch.float32).t()
  y = acc * a_scale.reshape(-1, 1) * b_scale.reshape(1, -1)
  if bias is not None:
    y = y + bias.to(torch.float32)
  if gelu == "fused":
    y = gelu_tanh(y)
  out = y.to(out_dtype)
  if gelu == "unfused":
    out = gelu_tanh(out.to(torch.float32)).to(out_dtype)
  return out


def w8a8_linear(x: torch.Tensor,
                w_q: torch.Tensor,
                w_scale: torch.Tensor,
                bias: Optional[torch.Tensor] = None,
                gelu: Optional[str] = None,
                scale_mode: str = "bf16div") -> torch.Tensor:
  """torchao Float8Tensor `aten.linear` for PerRow dynamic activation quant:
  flatten, quantize the activation per token, scaled matmul, reshape back."""
  lead = x.shape[:-1]
  x2 = x.reshape(-1, x.shape[-1])
  x_q, x_s = quantize_rowwise(x2, scale_mode)
  out = scaled_mm_rowwise(x_q, x_s, w_q, w_scale, bias, gelu)
  return out.reshape(*lead, w_q.shape[0])


def w8a16_linear(x: torch.Tensor,
                 w_q: torch.Tensor,
                 w_scale: torch.Tensor,
                 bias: Optional[torch.Tensor] = None,
                 gelu: Optional[str] = None,
                 fused: bool = False) -> torch.Tensor:
  """Weight-only: `F.linear(x, W.dequantize(), b)` with W.dequantize() =
  (q.float() * scale).to(bf16) (Float8WeightOnlyConfig, selected at
  src/cache_dit/quantization/torchao/quantize_ao.py:604-610). `fused=True` skips
  the bf16 rounding of the dequantized weight (scale applied to the accumulator)."""
  lead = x.shape[:-1]
  x2 = x.reshape(-1, x.shape[-1]).to(torch.float32)
  ws = w_scale.reshape(-1, 1).to(torch.float32)
  if fused:
    y = (x2 @ w_q.to(torch.float32).t()) * ws.reshape(1, -1)
  else:
    wd = (w_q.to(torch.float32) * ws).to(torch.bfloat16)
    y = x2 @ wd.to(torch.float32).t()
  if bias is not None:
    y = y + bias.to(torch.float32)
  if gelu == "fused":
    y = gelu_tanh(y)
  out = y.to(torch.bfloat16)
  if gelu == "unfused":
    out = gelu_tanh(out.to(torch.float32)).to(torch.bfloat16)
  return out.reshape(*lead, w_q.shape[0])
