"""Pins the oracle's e4m3fn encode/decode against the format's definition and
against PyTorch's own CPU float8_e4m3fn cast (a library routine)."""
import numpy as np
import torch

from helpers import all_finite_bf16
from oracle import c_oracle

FP8 = torch.float8_e4m3fn


def _enc(vals):
  L = c_oracle.lib()
  return np.array([L.oracle_e4m3_encode(float(v)) for v in vals], dtype=np.uint8)


def test_known_answers():
  # value -> code, from the format definition (S.EEEE.MMM, bias 7)
  kat = [(0.0, 0x00), (-0.0, 0x80)] + list({
      1.0: 0x38, -1.0: 0xB8, 0.5: 0x30, 448.0: 0x7E, -448.0: 0xFE,
      2.0**-6: 0x08, 2.0**-9: 0x01, 2.0**-10: 0x00, 1.5 * 2.0**-9: 0x02, 2.5 * 2.0**-9: 0x02,
      3.5 * 2.0**-9: 0x04, 17.0: 0x58, 19.0: 0x5A, 18.0: 0x59, 432.0: 0x7E, 464.0: 0x7E,
      240.0: 0x77, 0.875 * 2.0**-6: 0x07, 0.9375 * 2.0**-6: 0x08,
  }.items())
  for v, code in kat:
    got = c_oracle.lib().oracle_e4m3_encode(v)
    assert got == code, f"{v}: {got:#x} != {code:#x}"
    t = int(torch.tensor([v], dtype=torch.float32).to(FP8).view(torch.uint8))
    assert t == code, f"torch {v}: {t:#x} != {code:#x}"
  # beyond the tie at 464 the cast is NaN, in torch and in the oracle
  for v in (465.0, 480.0, 1000.0, float("inf")):
    assert c_oracle.lib().oracle_e4m3_encode(v) == 0x7F
    assert int(torch.tensor([v]).to(FP8).view(torch.uint8)) == 0x7F


def test_decode_every_code_matches_torch_and_closed_form():
  L = c_oracle.lib()
  codes = torch.arange(256, dtype=torch.uint8)
  tv = codes.view(FP8).float().numpy()
  for c in range(256):
    v = L.oracle_e4m3_decode(c)
    if (c & 0x7F) == 0x7F:
      assert np.isnan(v) and np.isnan(tv[c])
      continue
    e, m = (c >> 3) & 0xF, c & 7
    closed = (m / 8.0) * 2.0**-6 if e == 0 else (1 + m / 8.0) * 2.0**(e - 7)
    closed = -closed if c & 0x80 else closed
    assert v == closed == tv[c]
  # positive codes are strictly increasing
  pos = [L.oracle_e4m3_decode(c) for c in range(0x7F)]
  assert all(a < b for a, b in zip(pos, pos[1:])) and pos[-1] == 448.0


def test_encode_decode_round_trip():
  L = c_oracle.lib()
  for c in range(256):
    if (c & 0x7F) == 0x7F:
      continue
    assert L.oracle_e4m3_encode(L.oracle_e4m3_decode(c)) == c


def test_encode_all_bf16_values_matches_torch_cast():
  v = all_finite_bf16().float()
  t = v.clamp(-448, 448).to(FP8).view(torch.uint8).numpy()
  c = _enc(v.clamp(-448, 448).numpy())
  assert (t == c).all()


def test_encode_random_fp32_and_midpoints_matches_torch_cast():
  g = torch.Generator().manual_seed(0)
  v = (torch.rand(200000, generator=g) * 2 - 1) * 470
  v = torch.cat([v, torch.randn(100000, generator=g) * 0.01, torch.randn(50000, generator=g) * 1e-3])
  # exact midpoints between neighbouring codes and their fp32 neighbours
  codes = torch.arange(0x7F, dtype=torch.uint8).view(FP8).float()
  mid = (codes[:-1] + codes[1:]) / 2
  mids = torch.cat([mid, torch.nextafter(mid, torch.tensor(1e9)), torch.nextafter(mid, torch.tensor(-1e9))])
  v = torch.cat([v, mids, -mids])
  t = v.to(FP8).view(torch.uint8).numpy()
  c = _enc(v.numpy())
  assert (t == c).all()
