"""Writes tests/golden/*.npz from the CPU oracle. Run from the repo root:
    python tests/golden/make_golden.py
Deterministic: CPU generator seeds only."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import torch_oracle as to  # noqa: E402


def u16(t):
  return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def u8(t):
  return t.contiguous().view(torch.uint8).numpy()


def main():
  g = torch.Generator().manual_seed(1234)
  # quantizer: 48 rows x 512 with outlier channels, a zero row, tiny and huge rows
  x = torch.randn(48, 512, generator=g)
  x[:, [7, 300]] *= 20
  x[5] = 0
  x[6] *= 1e-20
  x[7] *= 1e20
  x[8, ::2] = -0.0
  x = x.to(torch.bfloat16)
  out = {"x": u16(x)}
  for mode in to.SCALE_MODES:
    q, s = to.quantize_rowwise(x, mode)
    out[f"q_{mode}"] = u8(q)
    out[f"s_{mode}"] = s.reshape(-1).numpy()
  np.savez_compressed(os.path.join(HERE, "quant_vectors.npz"), **out)

  # linear: x [40, 256], W [96, 256], bias; w8a8 (fused / unfused gelu) and w8a16
  x = torch.randn(40, 256, generator=g)
  x[:, 11] *= 20
  x = x.to(torch.bfloat16)
  w = (torch.randn(96, 256, generator=g) * 0.05).to(torch.bfloat16)
  b = (torch.randn(96, generator=g) * 0.1).to(torch.bfloat16)
  wq, ws = to.quantize_rowwise(w)
  xq, xs = to.quantize_rowwise(x)
  lin = {
      "x": u16(x), "w": u16(w), "bias": u16(b), "wq": u8(wq), "ws": ws.reshape(-1).numpy(),
      "xq": u8(xq), "xs": xs.reshape(-1).numpy(),
      "y_w8a8": u16(to.w8a8_linear(x, wq, ws, b)),
      "y_w8a8_gelu_fused": u16(to.w8a8_linear(x, wq, ws, b, gelu="fused")),
      "y_w8a8_gelu_unfused": u16(to.w8a8_linear(x, wq, ws, b, gelu="unfused")),
      "y_w8a16_ref": u16(to.w8a16_linear(x, wq, ws, b, fused=False)),
      "y_w8a16_fused": u16(to.w8a16_linear(x, wq, ws, b, fused=True)),
  }
  np.savez_compressed(os.path.join(HERE, "linear_vectors.npz"), **lin)
  print("wrote", os.listdir(HERE))


if __name__ == "__main__":
  main()
