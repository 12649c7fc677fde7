"""Shared input recipes and error metrics for the tests."""
from __future__ import annotations

import numpy as np
import torch

FP8 = torch.float8_e4m3fn


def config1_inputs(M=4608, K=3072, N=3072, seed=0):
  """benchmark config 1: x ~N(0,1) with 0.1% of channels x20, W ~N(0,0.02),
  bias ~N(0,0.01), all drawn in fp32 on the CPU generator and cast to bf16."""
  g = torch.Generator().manual_seed(seed)
  x = torch.randn(1, M, K, generator=g)
  n_out = max(1, int(0.001 * K))
  idx = torch.randperm(K, generator=g)[:n_out]
  x[..., idx] *= 20.0
  w = torch.randn(N, K, generator=g) * 0.02
  b = torch.randn(N, generator=g) * 0.01
  return x.to(torch.bfloat16), w.to(torch.bfloat16), b.to(torch.bfloat16)


def all_finite_bf16() -> torch.Tensor:
  """Every finite bf16 value (both zeros included), as a 1-D bf16 tensor."""
  bits = np.arange(65536, dtype=np.uint16)
  keep = (bits & 0x7f80) != 0x7f80
  return torch.from_numpy(bits[keep].view(np.int16).copy()).view(torch.bfloat16)


def bits_u8(t: torch.Tensor) -> np.ndarray:
  return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def bits_u32(t: torch.Tensor) -> np.ndarray:
  return t.detach().cpu().contiguous().view(torch.int32).numpy().view(np.uint32)


def max_rel_err(y: torch.Tensor, ref: torch.Tensor) -> float:
  """max |y - ref| / max |ref|: the tensor-level relative error."""
  y = y.detach().float().cpu()
  ref = ref.detach().float().cpu()
  return float((y - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def elementwise_ok(y: torch.Tensor, ref: torch.Tensor, rel: float = 1e-2, abs_floor=None) -> bool:
  """|y - ref| <= rel * |ref| + floor everywhere; floor defaults to rel * rms(ref)
  (bf16 outputs near zero make a bare element-wise relative error meaningless)."""
  y = y.detach().float().cpu()
  ref = ref.detach().float().cpu()
  if abs_floor is None:
    abs_floor = rel * float(ref.pow(2).mean().sqrt())
  return bool(((y - ref).abs() <= rel * ref.abs() + abs_floor).all())


def cosine(y: torch.Tensor, ref: torch.Tensor) -> float:
  y = y.detach().double().cpu().flatten()
  ref = ref.detach().double().cpu().flatten()
  return float((y @ ref) / (y.norm() * ref.norm()).clamp_min(1e-300))
