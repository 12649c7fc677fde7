"""FP8 quantizers for activations that cross GPUs, scale packed behind each row.

Same names, shapes and dtypes as the reference's Triton ops
(src/cache_dit/kernels/triton/_ops_registery.py:52-185, kernels
src/cache_dit/kernels/triton/_float8_comm.py:5-148), backed by HIP kernels in
libcdit_hip.so and registered as `torch.ops.cdit.fp8_comm_*` with fake
implementations. On one GPU they are plain tensor -> tensor functions; what would use
them (Ulysses all-to-all with FP8 payloads) is outside this package.
"""
from __future__ import annotations

import torch

from . import _native
from .ops import FP8, _DeviceOf, _require_cuda, _stream_ptr

torch.library.define("cdit::fp8_comm_per_token_quant", "(Tensor x) -> Tensor")
torch.library.define("cdit::fp8_comm_per_token_dequant", "(Tensor x) -> Tensor")
torch.library.define("cdit::fp8_comm_qkv_permute_quant", "(Tensor x) -> Tensor")
torch.library.define("cdit::fp8_comm_qkv_permute_dequant", "(Tensor quant_x) -> Tensor")


@torch.library.impl("cdit::fp8_comm_per_token_quant", "CUDA")
def _per_token_quant(x: torch.Tensor) -> torch.Tensor:
  assert x.dtype == torch.bfloat16, f"expected bfloat16 but got {x.dtype}"
  *shape, H = x.shape
  x2 = x.reshape(-1, H).contiguous()
  M = x2.shape[0]
  y = torch.empty((M, H + 2), dtype=FP8, device=x.device)
  with _DeviceOf(x2):
    _native.check(_native.load().cdit_fp8_comm_per_token_quant(x2.data_ptr(), M, H, y.data_ptr(),
                                                               _stream_ptr(x2)))
  return y.reshape(*shape, H + 2)


@torch.library.register_fake("cdit::fp8_comm_per_token_quant")
def _fake_per_token_quant(x):
  assert x.dtype == torch.bfloat16
  *shape, H = x.shape
  return x.new_empty((*shape, H + 2), dtype=FP8)


@torch.library.impl("cdit::fp8_comm_per_token_dequant", "CUDA")
def _per_token_dequant(x: torch.Tensor) -> torch.Tensor:
  assert x.dtype == FP8, f"expected float8_e4m3fn but got {x.dtype}"
  *shape, H2 = x.shape
  if H2 < 2:
    raise ValueError(f"fp8_comm_per_token_dequant: rows of {H2} bytes hold no scale")
  x2 = x.reshape(-1, H2).contiguous()
  M, H = x2.shape[0], H2 - 2
  y = torch.empty((M, H), dtype=torch.bfloat16, device=x.device)
  with _DeviceOf(x2):
    _native.check(_native.load().cdit_fp8_comm_per_token_dequant(x2.data_ptr(), M, H, y.data_ptr(),
                                                                 _stream_ptr(x2)))
  return y.reshape(*shape, H)


@torch.library.register_fake("cdit::fp8_comm_per_token_dequant")
def _fake_per_token_dequant(x):
  assert x.dtype == FP8
  *shape, H = x.shape
  return x.new_empty((*shape, H - 2), dtype=torch.bfloat16)


@torch.library.impl("cdit::fp8_comm_qkv_permute_quant", "CUDA")
def _qkv_permute_quant(x: torch.Tensor) -> torch.Tensor:
  assert x.dtype == torch.bfloat16, f"expected bfloat16 but got {x.dtype}"
  B, S, P, N, D = x.shape
  if x.stride(4) != 1 or x.stride(3) != D:  # heads and channels contiguous, as the kernel reads
    x = x.contiguous()
  quant_x = torch.empty((P, S, B, N, D + 4), dtype=FP8, device=x.device)
  with _DeviceOf(x):
    _native.check(_native.load().cdit_fp8_comm_qkv_permute_quant(
        x.data_ptr(), B, S, P, N, D, x.stride(0), x.stride(1), x.stride(2), quant_x.data_ptr(),
        _stream_ptr(x)))
  return quant_x


@torch.library.register_fake("cdit::fp8_comm_qkv_permute_quant")
def _fake_qkv_permute_quant(x):
  B, S, P, N, D = x.shape
  return x.new_empty((P, S, B, N, D + 4), dtype=FP8)


@torch.library.impl("cdit::fp8_comm_qkv_permute_dequant", "CUDA")
def _qkv_permute_dequant(quant_x: torch.Tensor) -> torch.Tensor:
  assert quant_x.dtype == FP8, f"expected float8_e4m3fn but got {quant_x.dtype}"
  S, B, N, D4 = quant_x.shape
  D = D4 - 4
  if quant_x.stride(3) != 1:
    quant_x = quant_x.contiguous()
  x = torch.empty((B, S, N, D), dtype=torch.bfloat16, device=quant_x.device)
  with _DeviceOf(quant_x):
    _native.check(_native.load().cdit_fp8_comm_qkv_permute_dequant(
        quant_x.data_ptr(), S, B, N, D, quant_x.stride(0), quant_x.stride(1), quant_x.stride(2),
        x.data_ptr(), _stream_ptr(quant_x)))
  return x


@torch.library.register_fake("cdit::fp8_comm_qkv_permute_dequant")
def _fake_qkv_permute_dequant(quant_x):
  S, B, N, D4 = quant_x.shape
  return quant_x.new_empty((B, S, N, D4 - 4), dtype=torch.bfloat16)


def fp8_comm_per_token_quant(x: torch.Tensor) -> torch.Tensor:
  """bf16 [..., H] -> float8_e4m3fn [..., H + 2] (codes, then the row's scale as bf16)."""
  _require_cuda("fp8_comm_per_token_quant", x)
  return torch.ops.cdit.fp8_comm_per_token_quant(x)


def fp8_comm_per_token_dequant(x: torch.Tensor) -> torch.Tensor:
  """float8_e4m3fn [..., H + 2] -> bf16 [..., H]."""
  _require_cuda("fp8_comm_per_token_dequant", x)
  return torch.ops.cdit.fp8_comm_per_token_dequant(x)


def fp8_comm_qkv_permute_quant(x: torch.Tensor) -> torch.Tensor:
  """bf16 [B, S, P, N, D] -> float8_e4m3fn [P, S, B, N, D + 4] (codes, then the head row's
  fp32 scale)."""
  _require_cuda("fp8_comm_qkv_permute_quant", x)
  return torch.ops.cdit.fp8_comm_qkv_permute_quant(x)


def fp8_comm_qkv_permute_dequant(quant_x: torch.Tensor) -> torch.Tensor:
  """float8_e4m3fn [S, B, N, D + 4] -> bf16 [B, S, N, D]."""
  _require_cuda("fp8_comm_qkv_permute_dequant", quant_x)
  return torch.ops.cdit.fp8_comm_qkv_permute_dequant(quant_x)
