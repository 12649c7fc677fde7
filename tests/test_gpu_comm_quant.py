"""GPU parity of the FP8 comm quantizers (packed trailing scales) against the CPU
restatement of the reference's Triton kernels: bit-exact codes, scales and dequantized
values on the same seeded inputs; the reference's own round-trip bounds
(tests/kernels/test_triton_ops.py:111-160 of the reference) on its shapes."""
import pytest
import torch

from helpers import bits_u8
from oracle import comm_oracle as co

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _x(shape, seed, outliers=True):
  g = torch.Generator().manual_seed(seed)
  x = torch.randn(*shape, generator=g)
  if outliers:
    x.view(-1)[torch.randperm(x.numel(), generator=g)[:max(1, x.numel() // 500)]] *= 30
  return x.to(torch.bfloat16)


@pytest.mark.parametrize("shape", [(2, 3, 128), (7, 3072), (3, 16384), (5, 20), (4, 1000), (9, 8),
                                   (1, 1, 4104), (6, 17), (300, 1536)])
def test_per_token_quant_and_dequant_bit_exact(shape):
  from cache_dit_amd import comm_quant as cq
  x = _x(shape, seed=sum(shape))
  x.view(-1, shape[-1])[0] = 0  # a zero row: the eps floor
  q = cq.fp8_comm_per_token_quant(x.cuda())
  q_ref = co.per_token_quant(x)
  assert q.shape == q_ref.shape and q.dtype == FP8
  assert (bits_u8(q) == bits_u8(q_ref)).all()
  d = cq.fp8_comm_per_token_dequant(q)
  d_ref = co.per_token_dequant(q_ref)
  assert d.shape == x.shape and d.dtype == torch.bfloat16
  assert torch.equal(d.cpu().view(torch.int16), d_ref.view(torch.int16))


def test_per_token_reference_round_trip_bounds():
  from cache_dit_amd import comm_quant as cq
  torch.manual_seed(0)
  x = torch.randn((2, 3, 128), device="cuda", dtype=torch.bfloat16)
  with torch.inference_mode():
    quantized = cq.fp8_comm_per_token_quant(x)
    dequantized = cq.fp8_comm_per_token_dequant(quantized)
    torch.cuda.synchronize()
  diff = (dequantized.float() - x.float()).abs()
  assert quantized.shape == (2, 3, 130) and quantized.dtype == torch.float8_e4m3fn
  assert dequantized.shape == x.shape and dequantized.dtype == torch.bfloat16
  assert torch.isfinite(quantized.float()).all() and torch.isfinite(dequantized).all()
  assert diff.mean().item() < 0.05 and diff.max().item() < 0.2


@pytest.mark.parametrize("shape", [(2, 4, 3, 5, 64), (1, 37, 3, 24, 128), (2, 5, 2, 3, 256),
                                   (1, 6, 3, 4, 96), (2, 3, 1, 2, 512), (1, 4, 3, 2, 20),
                                   (1, 3, 2, 1, 1024)])
def test_qkv_permute_quant_and_dequant_bit_exact(shape):
  from cache_dit_amd import comm_quant as cq
  x = _x(shape, seed=sum(shape))
  x[0, 0, 0, 0] = 0  # a zero head row: the eps floor on the scale
  q = cq.fp8_comm_qkv_permute_quant(x.cuda())
  q_ref = co.qkv_permute_quant(x)
  assert q.shape == q_ref.shape and q.dtype == FP8
  assert (bits_u8(q) == bits_u8(q_ref)).all()
  for p in range(shape[2]):  # a slice along P is not contiguous: strides reach the kernel
    d = cq.fp8_comm_qkv_permute_dequant(q[p])
    d_ref = co.qkv_permute_dequant(q_ref[p])
    assert d.shape == (shape[0], shape[1], shape[3], shape[4]) and d.dtype == torch.bfloat16
    assert torch.equal(d.cpu().view(torch.int16), d_ref.view(torch.int16))


@pytest.mark.parametrize("D", [64, 128, 256, 512])
def test_qkv_permute_quant_over_the_range_of_row_magnitudes(D):
  """Head rows from far below the 1e-6 floor of the scale to the top of the bf16 range,
  neighbours in one wavefront: the kernel's exact fast division (rows whose scale is
  amax / 448 inside its proven window) and its fallback (floored or very large scales)
  must both give the oracle's codes, whichever the other rows of the wavefront take."""
  from cache_dit_amd import comm_quant as cq
  B, S, P, N = 1, 23, 3, 6
  g = torch.Generator().manual_seed(D)
  x = torch.randn(B, S, P, N, D, generator=g)
  mags = torch.tensor([1e-30, 1e-9, 3e-7, 4.4e-4, 4.6e-4, 1e-3, 1.0, 77.0, 1e9, 1e30, 3e38])
  pick = torch.randint(0, len(mags), (B, S, P, N, 1), generator=g)
  x = (x * mags[pick]).clamp(-3e38, 3e38).to(torch.bfloat16)
  q = cq.fp8_comm_qkv_permute_quant(x.cuda())
  q_ref = co.qkv_permute_quant(x)
  assert (bits_u8(q) == bits_u8(q_ref)).all()
  for p in range(P):
    d = cq.fp8_comm_qkv_permute_dequant(q[p])
    assert torch.equal(d.cpu().view(torch.int16), co.qkv_permute_dequant(q_ref[p]).view(torch.int16))


def test_per_token_quant_over_the_range_of_row_magnitudes():
  from cache_dit_amd import comm_quant as cq
  g = torch.Generator().manual_seed(5)
  x = torch.randn(64, 1536, generator=g)
  mags = torch.tensor([1e-30, 1e-9, 1e-5, 9e-5, 1.1e-4, 1.0, 1e9, 1e30, 3e38])
  x = (x * mags[torch.randint(0, len(mags), (64, 1), generator=g)]).clamp(-3e38, 3e38).to(torch.bfloat16)
  q = cq.fp8_comm_per_token_quant(x.cuda())
  assert (bits_u8(q) == bits_u8(co.per_token_quant(x))).all()


def _same_bf16_up_to_nan(got, want):
  """Bit for bit, except that a NaN only has to be a NaN (its sign and payload are whatever
  the converting hardware or library leaves)."""
  nan = torch.isnan(want)
  assert torch.equal(torch.isnan(got), nan)
  assert torch.equal(got.view(torch.int16)[~nan], want.view(torch.int16)[~nan])


def test_dequant_of_arbitrary_code_bytes_including_nan_codes():
  """The dequantizers take whatever bytes arrive: every code value, the two NaN codes among
  them, next to rows without any in the same wavefront."""
  from cache_dit_amd import comm_quant as cq
  g = torch.Generator().manual_seed(11)
  for H in (64, 1536, 3072):
    raw = torch.randint(0, 256, (37, H + 2), dtype=torch.uint8, generator=g)
    raw[::3] &= 0x77  # rows without a NaN code (the low seven bits never all ones)
    raw[:, H:] = torch.tensor([0x80, 0x3c], dtype=torch.uint8)  # scale 2^-6 (bf16 0x3c80), low byte first
    q = raw.view(FP8)
    _same_bf16_up_to_nan(cq.fp8_comm_per_token_dequant(q.cuda()).cpu(), co.per_token_dequant(q))
  for D in (64, 128, 512):
    raw = torch.randint(0, 256, (5, 2, 3, D + 4), dtype=torch.uint8, generator=g)
    raw[::2] &= 0x77
    raw[..., D:] = torch.tensor([0, 0, 0x80, 0x3c], dtype=torch.uint8)  # fp32 scale 2^-6
    q = raw.view(FP8)
    _same_bf16_up_to_nan(cq.fp8_comm_qkv_permute_dequant(q.cuda()).cpu(), co.qkv_permute_dequant(q))


def test_qkv_permute_quant_takes_a_strided_input():
  """x as a view of a packed [B, S, 3 * N * D] qkv projection output with padding."""
  from cache_dit_amd import comm_quant as cq
  B, S, P, N, D = 2, 9, 3, 4, 128
  base = _x((B, S, P * N * D + 64), seed=3)
  x = base[..., :P * N * D].view(B, S, P, N, D)
  assert not x.is_contiguous()
  xg = base.cuda()[..., :P * N * D].view(B, S, P, N, D)
  assert not xg.is_contiguous()
  q = cq.fp8_comm_qkv_permute_quant(xg)
  assert (bits_u8(q) == bits_u8(co.qkv_permute_quant(x))).all()


def test_qkv_reference_round_trip_tracks_selected_slice():
  from cache_dit_amd import comm_quant as cq
  torch.manual_seed(0)
  x = torch.randn((2, 4, 3, 5, 64), device="cuda", dtype=torch.bfloat16)
  with torch.inference_mode():
    quantized = cq.fp8_comm_qkv_permute_quant(x)
    torch.cuda.synchronize()
  assert quantized.shape == (3, 4, 2, 5, 68) and quantized.dtype == torch.float8_e4m3fn
  assert torch.isfinite(quantized[..., :64].float()).all()
  with torch.inference_mode():
    for p_index in range(x.shape[2]):
      dequantized = cq.fp8_comm_qkv_permute_dequant(quantized[p_index])
      torch.cuda.synchronize()
      distances = [(dequantized.float() - x[:, :, r].float()).abs().mean().item()
                   for r in range(x.shape[2])]
      assert dequantized.shape == (2, 4, 5, 64) and dequantized.dtype == torch.bfloat16
      assert torch.isfinite(dequantized).all()
      assert min(range(len(distances)), key=lambda i: distances[i]) == p_index


def test_comm_ops_fake_and_error_paths():
  from cache_dit_amd import _native, comm_quant as cq
  from torch._subclasses.fake_tensor import FakeTensorMode
  with FakeTensorMode():
    x = torch.empty(2, 3, 128, dtype=torch.bfloat16, device="cuda")
    q = torch.ops.cdit.fp8_comm_per_token_quant(x)
    assert q.shape == (2, 3, 130) and q.dtype == FP8
    assert torch.ops.cdit.fp8_comm_per_token_dequant(q).shape == (2, 3, 128)
    x5 = torch.empty(2, 4, 3, 5, 64, dtype=torch.bfloat16, device="cuda")
    q5 = torch.ops.cdit.fp8_comm_qkv_permute_quant(x5)
    assert q5.shape == (3, 4, 2, 5, 68)
    assert torch.ops.cdit.fp8_comm_qkv_permute_dequant(q5[0]).shape == (2, 4, 5, 64)
  L = _native.load()
  one = 256
  assert L.cdit_fp8_comm_qkv_permute_quant(one, 1, 1, 1, 1, 6, 6, 6, 6, one, None) == 1
  assert b"multiple of 4" in L.cdit_last_error()
  assert L.cdit_fp8_comm_per_token_quant(None, 3, 8, one, None) == 1
  assert b"null pointer" in L.cdit_last_error()
  assert L.cdit_fp8_comm_per_token_quant(None, 0, 8, None, None) == 0
  assert cq.fp8_comm_per_token_quant(torch.zeros(0, 16, dtype=torch.bfloat16, device="cuda")).shape == (0, 18)
  with pytest.raises(RuntimeError, match="no CPU path"):
    cq.fp8_comm_per_token_quant(torch.zeros(2, 16, dtype=torch.bfloat16))
