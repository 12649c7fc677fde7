"""CPU restatement of the reference's FP8 comm quantizers in eager PyTorch ops.
TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Follows /root/reference/src/cache_dit/kernels/triton/_float8_comm.py:5-148 and the op
wrappers src/cache_dit/kernels/triton/_ops_registery.py:52-185 statement by statement.
The reference kernels are Triton (not runnable here: no NVIDIA backend, and on AMD its
`/` and the fp32 -> e4m3 cast are whatever the backend lowers them to), so the
restatement fixes IEEE fp32 arithmetic and round-to-nearest-even casts. Pinned by: the
reference's own round-trip bounds (tests/kernels/test_triton_ops.py:111-160), closed
forms (amax = 448 * 2^k gives scale 2^k and exact codes; the eps floors), brute force
over every e4m3 code, and the packed layouts read back with plain views
(tests/test_oracle_comm.py).
"""
from __future__ import annotations

import torch

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0


def per_token_quant(x: torch.Tensor) -> torch.Tensor:
  """_fp8_comm_per_token_quant_kernel (_float8_comm.py:5-40), eps = 1e-4
  (_ops_registery.py:67): bf16 [..., H] -> e4m3 [..., H + 2]."""
  *shape, H = x.shape
  xf = x.reshape(-1, H).to(torch.float32)
  M = xf.shape[0]
  absmax = xf.abs().amax(dim=1, keepdim=True).clamp_min(1e-4) if H else torch.full((M, 1), 1e-4)
  x_s = absmax / FP8_MAX
  x_s_inv = 1.0 / x_s
  codes = (xf * x_s_inv).clamp(-FP8_MAX, FP8_MAX).to(FP8)
  y = torch.empty((M, H + 2), dtype=torch.uint8)
  y[:, :H] = codes.view(torch.uint8)
  y[:, H:] = x_s.to(torch.bfloat16).view(torch.uint8)  # 2 bytes per row, little endian
  return y.view(FP8).reshape(*shape, H + 2)


def per_token_dequant(y: torch.Tensor) -> torch.Tensor:
  """_fp8_comm_per_token_dequant_kernel (_float8_comm.py:43-62): e4m3 [..., H + 2] ->
  bf16 [..., H]."""
  *shape, H2 = y.shape
  H = H2 - 2
  y2 = y.reshape(-1, H2)
  x_s = y2[:, H:].contiguous().view(torch.bfloat16).to(torch.float32)  # [M, 1]
  x = y2[:, :H].to(torch.float32) * x_s
  return x.to(torch.bfloat16).reshape(*shape, H)


def qkv_permute_quant(x: torch.Tensor) -> torch.Tensor:
  """_fp8_comm_qkv_permute_quant_kernel (_float8_comm.py:66-113), EPS = 1e-6
  (_ops_registery.py:118): bf16 [B, S, P, N, D] -> e4m3 [P, S, B, N, D + 4]."""
  B, S, P, N, D = x.shape
  xf = x.permute(2, 1, 0, 3, 4).to(torch.float32)  # [P, S, B, N, D]
  scale = (xf.abs().amax(dim=-1, keepdim=True) / FP8_MAX).clamp_min(1e-6)
  codes = (xf / scale).clamp(-FP8_MAX, FP8_MAX).to(FP8)
  out = torch.empty((P, S, B, N, D + 4), dtype=torch.uint8)
  out[..., :D] = codes.view(torch.uint8)
  out[..., D:] = scale.contiguous().view(torch.uint8)  # 4 bytes per head row
  return out.view(FP8)


def qkv_permute_dequant(quant_x: torch.Tensor) -> torch.Tensor:
  """_fp8_comm_qkv_dequant_permute_kernel (_float8_comm.py:116-148): e4m3 [S, B, N, D + 4]
  -> bf16 [B, S, N, D], x[b, s] = dequant(quant_x[s, b]): the inverse of qkv_permute_quant's
  permutation, which is what the output's declared shape says.

  DEVIATION for B > 1, parity unpinned there: the reference kernel as written stores the
  dequantized row of program `bs_id = s * B + b` at `x_ptr + bs_id * x.stride(1)`
  (_float8_comm.py:130-139; the wrapper passes x.stride(1) of the [B, S, N, D] output,
  _ops_registery.py:160-170), i.e. at flat row s * B + b of a buffer whose flat row b * S + s
  is x[b, s]. For B = 1 the two agree; for B > 1 and S > 1 the reference leaves the rows in
  [S, B] order inside a tensor declared [B, S, N, D], so that dequant(quant(x)[p]) is not
  x[:, :, p]. Its own test (tests/kernels/test_triton_ops.py:132-160, B = 2) only asks that
  the result be nearer to slice p than to the other slices, which both layouts satisfy.
  This restatement, and the HIP kernel, implement the true permutation (round trip =
  identity up to quantization error); `qkv_permute_dequant_as_written` below restates the
  literal behaviour for comparison."""
  S, B, N, D4 = quant_x.shape
  D = D4 - 4
  scale = quant_x[..., D:].contiguous().view(torch.float32)  # [S, B, N, 1]
  x = quant_x[..., :D].to(torch.float32) * scale
  return x.to(torch.bfloat16).permute(1, 0, 2, 3).contiguous()


def qkv_permute_dequant_as_written(quant_x: torch.Tensor) -> torch.Tensor:
  """The reference kernel's literal store pattern (see qkv_permute_dequant): flat row
  s * B + b of the [B, S, N, D] output receives dequant(quant_x[s, b]). Equal to
  qkv_permute_dequant for B = 1 only. Not used by the product; kept so that a test can state
  which of the two layouts this build follows."""
  S, B, N, D4 = quant_x.shape
  D = D4 - 4
  scale = quant_x[..., D:].contiguous().view(torch.float32)
  x = (quant_x[..., :D].to(torch.float32) * scale).to(torch.bfloat16)  # [S, B, N, D]
  return x.reshape(S * B, N, D).reshape(B, S, N, D).contiguous()
