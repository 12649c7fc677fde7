"""Pins oracle.torch_oracle.ln_modulate (LayerNorm + AdaLN modulation as eager bf16 ops):
a closed form, and a scalar restatement with every rounding step written out."""
import numpy as np
import torch

from oracle import torch_oracle as to


def _bf16(v: np.ndarray) -> np.ndarray:
  """fp32 -> nearest-even bf16 -> fp32, on the bit pattern."""
  u = np.asarray(v, dtype=np.float32).view(np.uint32).astype(np.uint64)
  u = (u + 0x7fff + ((u >> 16) & 1)) & 0xffff0000
  return u.astype(np.uint32).view(np.float32)


def test_closed_form_plus_minus_a():
  """x = (+a, -a, ...): mean 0, variance a^2, so with eps = 0 the normalised row is +-1
  exactly; scale 1 and shift 3 then give 5 and 1."""
  for a in (0.5, 3.0, 96.0):
    x = torch.tensor([a, -a] * 8, dtype=torch.bfloat16).reshape(1, 16)
    y = to.ln_modulate(x, torch.full((16,), 3.0, dtype=torch.bfloat16),
                       torch.ones(16, dtype=torch.bfloat16), eps=0.0)
    assert torch.equal(y.float(), torch.tensor([5.0, 1.0] * 8).reshape(1, 16))
  # a constant row has variance 0: eps alone sets rstd, the normalised row is 0, y = shift
  x = torch.full((1, 16), 7.0, dtype=torch.bfloat16)
  sh = torch.arange(16, dtype=torch.float32).to(torch.bfloat16)
  assert torch.equal(to.ln_modulate(x, sh, torch.ones(16, dtype=torch.bfloat16)), sh.reshape(1, 16))


def test_every_rounding_step_written_out():
  """(x - mean) * rstd, 1 + scale, their product and the sum with shift are each rounded
  to bf16: a numpy restatement with the roundings explicit gives the same bits, given
  the same fp32 mean and rstd."""
  g = torch.Generator().manual_seed(0)
  M, K = 5, 64
  x = (torch.randn(M, K, generator=g) * 3 + 1).to(torch.bfloat16)
  sh = torch.randn(K, generator=g).to(torch.bfloat16)
  sc = (torch.randn(K, generator=g) * 0.3).to(torch.bfloat16)
  y = to.ln_modulate(x, sh, sc, eps=1e-6)
  xf = x.float().numpy()
  mean = xf.astype(np.float64).mean(1, keepdims=True)
  var = ((xf.astype(np.float64) - mean)**2).mean(1, keepdims=True)
  rstd = (1.0 / np.sqrt(var + 1e-6)).astype(np.float32)
  n = _bf16((xf - mean.astype(np.float32)) * rstd)
  t = _bf16(np.float32(1.0) + sc.float().numpy())
  want = _bf16(_bf16(n * t) + sh.float().numpy())
  got = y.float().numpy()
  # fp32 statistics against float64 ones: a bf16 result may sit on the other side of a
  # rounding boundary for a rare element; everything else must agree to the bit
  assert (got != want).mean() <= 0.01
  assert np.allclose(got, want, rtol=2**-7, atol=2**-7)
  y2, q, s = to.ln_modulate_quant(x, sh, sc)
  q_ref, s_ref = to.quantize_rowwise(y)
  assert torch.equal(y2, y) and torch.equal(q.view(torch.uint8), q_ref.view(torch.uint8))
  assert torch.equal(s, s_ref)
