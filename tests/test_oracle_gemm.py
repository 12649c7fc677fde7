"""Pins the GEMM / linear oracles: C (double accumulation) vs PyTorch ops vs
closed forms vs the committed golden vectors."""
import os

import numpy as np
import pytest
import torch

from helpers import bits_u8, max_rel_err
from oracle import c_oracle
from oracle import torch_oracle as to

GOLD = os.path.join(os.path.dirname(__file__), "golden")
FP8 = torch.float8_e4m3fn


def _bf(a):
  return torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)


def _u16(t):
  return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_golden_linear_vectors():
  z = np.load(os.path.join(GOLD, "linear_vectors.npz"))
  x, w, b = _bf(z["x"]), _bf(z["w"]), _bf(z["bias"])
  wq, ws = to.quantize_rowwise(w)
  assert (bits_u8(wq) == z["wq"]).all() and (ws.reshape(-1).numpy() == z["ws"]).all()
  assert (_u16(to.w8a8_linear(x, wq, ws, b)) == z["y_w8a8"]).all()
  assert (_u16(to.w8a8_linear(x, wq, ws, b, gelu="fused")) == z["y_w8a8_gelu_fused"]).all()
  assert (_u16(to.w8a8_linear(x, wq, ws, b, gelu="unfused")) == z["y_w8a8_gelu_unfused"]).all()
  assert (_u16(to.w8a16_linear(x, wq, ws, b, fused=False)) == z["y_w8a16_ref"]).all()
  assert (_u16(to.w8a16_linear(x, wq, ws, b, fused=True)) == z["y_w8a16_fused"]).all()
  # the C restatement reproduces them to the last-bit-or-one of bf16 (it sums in double)
  y = _bf(c_oracle.gemm_rowwise(z["xq"], z["xs"], z["wq"], z["ws"], z["bias"]))
  assert max_rel_err(y, _bf(z["y_w8a8"])) <= 2.0**-7
  y = _bf(c_oracle.w8a16(z["x"], z["wq"], z["ws"], z["bias"], dequant_bf16=True))
  assert max_rel_err(y, _bf(z["y_w8a16_ref"])) <= 2.0**-7


def test_exact_on_small_integers():
  g = torch.Generator().manual_seed(1)
  a = torch.randint(-4, 5, (33, 128), generator=g).float()
  w = torch.randint(-4, 5, (17, 128), generator=g).float()
  ones_a, ones_w = torch.ones(33, 1), torch.ones(17, 1)
  expect = (a @ w.t()).to(torch.bfloat16)  # integers < 2^8... exact in fp32, then bf16
  y = to.scaled_mm_rowwise(a.to(FP8), ones_a, w.to(FP8), ones_w)
  assert torch.equal(y, expect)
  yc = _bf(c_oracle.gemm_rowwise(bits_u8(a.to(FP8)), ones_a.numpy(), bits_u8(w.to(FP8)),
                                 ones_w.numpy()))
  assert torch.equal(yc, expect)


def test_scales_bias_and_gelu_closed_forms():
  a = torch.tensor([[1.0, 2.0] + [0.0] * 14]).to(FP8)
  w = torch.tensor([[3.0, 0.5] + [0.0] * 14, [-1.0, 1.0] + [0.0] * 14]).to(FP8)
  a_s, w_s = torch.tensor([[0.5]]), torch.tensor([[2.0], [4.0]])
  bias = torch.tensor([0.25, -1.0]).to(torch.bfloat16)
  y = to.scaled_mm_rowwise(a, a_s, w, w_s, bias)
  # (1*3 + 2*0.5) * 0.5 * 2 + 0.25 = 4.25 ; (-1 + 2) * 0.5 * 4 - 1 = 1.0
  assert y.float().tolist() == [[4.25, 1.0]]
  yg = to.scaled_mm_rowwise(a, a_s, w, w_s, bias, gelu="fused").float()
  for got, v in zip(yg[0].tolist(), (4.25, 1.0)):
    import math
    expect = 0.5 * v * (1 + math.tanh(0.7978845608 * (v + 0.044715 * v**3)))
    assert abs(got - expect) <= 2.0**-8 * abs(expect)
    assert abs(c_oracle.lib().oracle_gelu_tanh(v) - expect) <= 1e-6
  yc = _bf(c_oracle.gemm_rowwise(bits_u8(a), a_s.numpy(), bits_u8(w), w_s.numpy(), _u16(bias)))
  assert yc.float().tolist() == [[4.25, 1.0]]


@pytest.mark.parametrize("M,N,K", [(64, 48, 256), (7, 16, 3072)])
def test_c_vs_torch_random(M, N, K):
  g = torch.Generator().manual_seed(M + N + K)
  x = torch.randn(M, K, generator=g).to(torch.bfloat16)
  w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
  b = (torch.randn(N, generator=g) * 0.01).to(torch.bfloat16)
  xq, xs = to.quantize_rowwise(x)
  wq, ws = to.quantize_rowwise(w)
  for gelu_c, gelu_t in ((0, None), (1, "fused"), (2, "unfused")):
    y = to.scaled_mm_rowwise(xq, xs, wq, ws, b, gelu=gelu_t)
    yc = _bf(c_oracle.gemm_rowwise(bits_u8(xq), xs.numpy(), bits_u8(wq), ws.numpy(), _u16(b),
                                   gelu=gelu_c))
    assert max_rel_err(yc, y) <= 2.0**-7  # at most one bf16 ulp of the largest value apart
  for fused in (True, False):
    y = to.w8a16_linear(x, wq, ws, b, fused=fused)
    yc = _bf(c_oracle.w8a16(_u16(x), bits_u8(wq), ws.numpy(), _u16(b), dequant_bf16=not fused))
    assert max_rel_err(yc, y) <= 2.0**-7


def test_w8a8_tracks_the_unquantized_linear():
  """End-to-end sanity of the whole restatement: FP8 w8a8 output close to the bf16
  linear it replaces (cosine > 0.999 on config-1-like data)."""
  g = torch.Generator().manual_seed(3)
  x = torch.randn(256, 1024, generator=g).to(torch.bfloat16)
  w = (torch.randn(512, 1024, generator=g) * 0.02).to(torch.bfloat16)
  wq, ws = to.quantize_rowwise(w)
  y = to.w8a8_linear(x, wq, ws).float().flatten()
  ref = (x.float() @ w.float().t()).flatten()
  assert float(y @ ref / (y.norm() * ref.norm())) > 0.999


def test_output_dtypes_are_one_rounding_of_the_fp32_result():
  """fp16 / bf16 outputs are the fp32-output result rounded once (the GEMM accumulates and
  applies scales and bias in fp32 whatever the output dtype), and an fp32 output with bias
  equals the reference's `matmul(out_dtype=fp32) + bias` (_scaled_mm.py:71-81)."""
  g = torch.Generator().manual_seed(21)
  x = torch.randn(40, 64, generator=g).to(torch.bfloat16)
  w = (torch.randn(24, 64, generator=g) * 0.1).to(torch.bfloat16)
  aq, a_s = to.quantize_rowwise(x)
  wq, w_s = to.quantize_rowwise(w)
  b = (torch.randn(24, generator=g) * 0.1).to(torch.bfloat16)
  f32 = to.scaled_mm_rowwise(aq, a_s, wq, w_s, b, out_dtype=torch.float32)
  assert f32.dtype == torch.float32
  for dt in (torch.float16, torch.bfloat16):
    out = to.scaled_mm_rowwise(aq, a_s, wq, w_s, b.to(dt), out_dtype=dt)
    if dt == torch.bfloat16:
      assert torch.equal(out, f32.to(dt))
    assert out.dtype == dt
    assert (out.float() - to.scaled_mm_rowwise(aq, a_s, wq, w_s, b.to(dt), out_dtype=torch.float32)
            ).abs().max() <= f32.abs().max() * 2.0**-8
  no_bias = to.scaled_mm_rowwise(aq, a_s, wq, w_s, None, out_dtype=torch.float32)
  assert torch.equal(f32, no_bias + b)
