"""Pins the per-tensor quantizer of the oracle (CPU only). The reference routes
`float8_per_tensor` to torchao's PerTensor granularity
(src/cache_dit/quantization/torchao/quantize_ao.py:559-575); it holds no golden
vector for it, so the restatement is pinned against what the arithmetic fixes."""
import numpy as np
import pytest
import torch

from oracle import c_oracle, torch_oracle as to

FP8 = torch.float8_e4m3fn


def _bits(x):
  return x.view(torch.int16).numpy().astype(np.uint16)


@pytest.mark.parametrize("mode", ["bf16div", "fp32div"])
def test_equals_rowwise_when_all_rows_share_the_amax(mode):
  g = torch.Generator().manual_seed(3)
  x = torch.randn(37, 96, generator=g).to(torch.bfloat16)
  x[:, 5] = 7.5  # every row's amax, hence the tensor's
  x = x.clamp(-7.5, 7.5)
  qt, st = to.quantize_tensorwise(x, mode)
  qr, sr = to.quantize_rowwise(x, mode)
  assert torch.equal(st, sr) and torch.equal(qt.view(torch.uint8), qr.view(torch.uint8))


@pytest.mark.parametrize("mode", ["bf16div", "fp32div"])
def test_closed_forms(mode):
  # amax = 448 * 2^k: scale = 2^k exactly in both modes, codes = e4m3(x / 2^k)
  x = torch.tensor([[448.0 * 4, 3.0, -1.5], [0.25, -448.0 * 4, 96.0]]).to(torch.bfloat16)
  q, s = to.quantize_tensorwise(x, mode)
  assert s.shape == (2, 1) and torch.all(s == 4.0)
  assert torch.equal(q.float(), (x.float() / 4.0).to(FP8).float())
  # all-zero tensor: scale 1 (the zero-scale patch), codes 0
  q, s = to.quantize_tensorwise(torch.zeros(3, 8, dtype=torch.bfloat16), mode)
  assert torch.all(s == 1.0) and torch.all(q.view(torch.uint8) == 0)
  # the largest element maps to +-448, nothing exceeds it
  g = torch.Generator().manual_seed(5)
  x = (torch.randn(64, 128, generator=g) * 3).to(torch.bfloat16)
  q, s = to.quantize_tensorwise(x, mode)
  assert q.float().abs().max() <= 448.0
  i = x.float().abs().argmax()
  assert abs(q.float().flatten()[i]) >= 416.0  # within one e4m3 step of 448


@pytest.mark.parametrize("mode", [0, 1])
def test_c_restatement_matches_torch_restatement(mode):
  g = torch.Generator().manual_seed(17 + mode)
  for scale in (1e-3, 1.0, 300.0, 3e4):
    x = (torch.randn(48, 160, generator=g) * scale).to(torch.bfloat16)
    q, s = to.quantize_tensorwise(x, to.SCALE_MODES[mode])
    qc, sc = c_oracle.quant_tensorwise(_bits(x), mode)
    assert np.array_equal(qc, q.view(torch.uint8).numpy())
    assert np.array_equal(sc, s.reshape(-1).numpy())


def test_scale_power_of_two_equivariance():
  g = torch.Generator().manual_seed(9)
  x = torch.randn(16, 64, generator=g).to(torch.bfloat16)
  q1, s1 = to.quantize_tensorwise(x)
  q2, s2 = to.quantize_tensorwise((x.float() * 8).to(torch.bfloat16))
  assert torch.equal(q1.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s1 * 8, s2)
