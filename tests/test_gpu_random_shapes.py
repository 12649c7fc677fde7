"""Seeded random sweeps over shapes, row strides and value ranges, through the launchers'
own kernel choice (no variant forced):

* GEMMs (w8a8, w8a16, and the batched forms with random membership) on small-integer operands
  with power-of-two scales: every product, sum and scaling is exact in fp32, so the bf16 output
  must equal an fp32 matmul bit for bit whatever tile, kernel or order of accumulation the
  launcher picks; outputs are windows of sentinel-filled buffers that must stay untouched
  outside;
* the quantizers (per row, per tensor, on a concatenation, fused into the LayerNorm producer)
  against the CPU oracle bit for bit, over rows scaled across 120 binades, zero rows, outlier
  columns and, outside the bit-exact contract, Inf / NaN elements (NaN scales and codes only
  have to be NaN on both sides).
"""
import random

import pytest
import torch

from helpers import bits_u8
from oracle import torch_oracle as to

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
DEV = "cuda"


def _untouched(full, n_cols):
  return bool((full[0] == 777).all() and (full[-1] == 777).all() and (full[:, n_cols:] == 777).all())


def _gemm_shape(rng):
  r = rng.random()
  M = rng.randint(1, 16) if r < 0.15 else rng.randint(17, 700) if r < 0.4 else rng.randint(700, 9000)
  N = rng.choice([16, 8]) * rng.randint(2, 900)
  K = 16 * rng.randint(1, 8) if rng.random() < 0.1 else 16 * rng.randint(8, 1000)
  while M * N * K > 1.5e11:
    K = max(128, K // 2 // 16 * 16)
  return M, N, K


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_exact_integer_gemms_over_random_shapes_and_strides(seed):
  from cache_dit_amd import ops
  rng = random.Random(seed)
  for case in range(14):
    M, N, K = _gemm_shape(rng)
    pad_a, pad_w, pad_o = rng.choice([0, 0, 16, 64]), rng.choice([0, 0, 16, 128]), rng.choice([0, 0, 8, 24])
    g = torch.Generator(device=DEV).manual_seed(1000 * seed + case)
    a = torch.randint(-3, 4, (M, K + pad_a), generator=g, device=DEV).float().to(FP8)[:, :K]
    w = torch.randint(-3, 4, (N, K + pad_w), generator=g, device=DEV).float().to(FP8)[:, :K]
    sa = torch.pow(2.0, torch.randint(-3, 3, (M,), generator=g, device=DEV).float())
    sw = torch.pow(2.0, torch.randint(-3, 3, (N,), generator=g, device=DEV).float())
    b = (torch.randint(-8, 9, (N,), generator=g, device=DEV).to(torch.bfloat16)
         if rng.random() < 0.7 else None)
    full = torch.full((M + 2, N + pad_o), 777.0, dtype=torch.bfloat16, device=DEV)
    out = full[1:M + 1, :N]
    what = (seed, case, M, N, K, pad_a, pad_w, pad_o, b is not None)
    ops.gemm_rowwise_into(a, sa, w, sw, b, out, 0)
    ref = (a.float() @ w.float().t()) * sa[:, None] * sw[None, :]
    ref = (ref if b is None else ref + b.float()[None, :]).to(torch.bfloat16)
    torch.cuda.synchronize()
    assert torch.equal(out, ref), ("w8a8",) + what
    assert _untouched(full, N), ("w8a8 wrote outside",) + what
    if rng.random() < 0.6:
      x = torch.randint(-4, 5, (M, K + pad_a), generator=g, device=DEV).to(torch.bfloat16)[:, :K]
      full.fill_(777.0)
      ops.w8a16_into(x, w, sw, b, out, 0)
      ref = (x.float() @ w.float().t()) * sw[None, :]
      ref = (ref if b is None else ref + b.float()[None, :]).to(torch.bfloat16)
      torch.cuda.synchronize()
      assert torch.equal(out, ref), ("w8a16",) + what
      assert _untouched(full, N), ("w8a16 wrote outside",) + what


@pytest.mark.parametrize("seed", [21, 22])
def test_exact_integer_batched_gemms_with_random_membership(seed):
  from cache_dit_amd import ops
  rng = random.Random(seed)
  for case in range(12):
    K = 16 * rng.randint(8, 400) if rng.random() < 0.5 else 128 * rng.randint(1, 40)
    n_acts, left = rng.randint(1, 4), 8
    g = torch.Generator(device=DEV).manual_seed(1000 * seed + case)
    acts8, acts16, refs8, refs16, fulls = [], [], [], [], []
    for s in range(n_acts):
      M = rng.choice([rng.randint(1, 16), rng.randint(17, 600), rng.randint(600, 4000)])
      members = rng.randint(1, max(1, min(4, left - (n_acts - s - 1))))
      left -= members
      a = torch.randint(-3, 4, (M, K), generator=g, device=DEV).float().to(FP8)
      x = torch.randint(-4, 5, (M, K), generator=g, device=DEV).to(torch.bfloat16)
      sa = torch.pow(2.0, torch.randint(-3, 3, (M,), generator=g, device=DEV).float())
      ws, wss, bs, o8, o16 = [], [], [], [], []
      for _ in range(members):
        N = 8 * rng.randint(2, 500) if rng.random() < 0.7 else 16 * rng.randint(100, 700)
        w = torch.randint(-3, 4, (N, K), generator=g, device=DEV).float().to(FP8)
        sw = torch.pow(2.0, torch.randint(-3, 3, (N,), generator=g, device=DEV).float())
        b = (torch.randint(-8, 9, (N,), generator=g, device=DEV).to(torch.bfloat16)
             if rng.random() < 0.6 else None)
        f8 = torch.full((M + 2, N + 8), 777.0, dtype=torch.bfloat16, device=DEV)
        f16 = torch.full((M + 2, N + 8), 777.0, dtype=torch.bfloat16, device=DEV)
        ws.append(w), wss.append(sw), bs.append(b), o8.append(f8[1:M + 1, :N]), o16.append(f16[1:M + 1, :N])
        fulls += [(f8, N), (f16, N)]
        r8 = (a.float() @ w.float().t()) * sa[:, None] * sw[None, :]
        r16 = (x.float() @ w.float().t()) * sw[None, :]
        if b is not None:
          r8, r16 = r8 + b.float()[None, :], r16 + b.float()[None, :]
        refs8.append(r8.to(torch.bfloat16)), refs16.append(r16.to(torch.bfloat16))
      acts8.append((a, sa, ws, wss, bs, o8, [0] * members))
      acts16.append((x, ws, wss, bs, o16, [0] * members))
    what = (seed, case, K, [(t[0].shape[0], [w.shape[0] for w in t[2]]) for t in acts8])
    ops.gemm_rowwise_batched_into(acts8)
    ops.w8a16_batched_into(acts16)
    torch.cuda.synchronize()
    for i, (o, r) in enumerate(zip([o for t in acts8 for o in t[5]], refs8)):
      assert torch.equal(o, r), ("w8a8 member", i) + what
    for i, (o, r) in enumerate(zip([o for t in acts16 for o in t[4]], refs16)):
      assert torch.equal(o, r), ("w8a16 member", i) + what
    assert all(_untouched(f, n) for f, n in fulls), ("wrote outside",) + what


def _activation(rng, M, K, g):
  x = torch.randn(M, K, generator=g)
  kind = rng.random()
  if kind < 0.2:
    x = x * torch.pow(2.0, torch.randint(-60, 60, (M, 1), generator=g).float())
  elif kind < 0.3:
    x = x * torch.pow(2.0, torch.randint(-130, -100, (M, 1), generator=g).float())
  elif kind < 0.4:
    x = x * 1e30
  if rng.random() < 0.3 and M > 2:
    x[rng.randrange(M)] = 0
  if rng.random() < 0.15:
    x[rng.randrange(M), rng.randrange(K)] = float("inf")
  if rng.random() < 0.15:
    x[rng.randrange(M), rng.randrange(K)] = float("nan")
  if rng.random() < 0.3:
    x[:, rng.randrange(K)] *= 50
  return x.to(torch.bfloat16)


def _same_codes_and_scales(q, s, q_ref, s_ref, what):
  s, s_ref = s.cpu().reshape(-1), s_ref.reshape(-1)
  both_nan = torch.isnan(s) & torch.isnan(s_ref)
  assert torch.equal(torch.where(both_nan, torch.zeros_like(s), s).view(torch.int32),
                     torch.where(both_nan, torch.zeros_like(s_ref), s_ref).view(torch.int32)), what
  qb, rb = torch.from_numpy(bits_u8(q)), torch.from_numpy(bits_u8(q_ref))
  nan_both = ((qb & 0x7f) == 0x7f) & ((rb & 0x7f) == 0x7f)  # 0x7f and 0xff are both NaN
  assert not ((qb != rb) & ~nan_both).any(), what


@pytest.mark.parametrize("seed", [31, 32, 33])
def test_quantizers_over_random_shapes_and_value_ranges(seed):
  from cache_dit_amd import _native, ops
  rng = random.Random(seed)
  for case in range(14):
    mode = rng.choice(["bf16div", "fp32div"])
    mid = _native.SCALE_MODE_IDS[mode]
    M = rng.randint(1, 40) if rng.random() < 0.3 else rng.randint(40, 2500)
    K = 8 * rng.randint(1, 64) if rng.random() < 0.3 else 8 * rng.randint(64, 2500)
    if rng.random() < 0.15:
      K = rng.randint(1, 5000)  # any K: the element-wise kernels
    while M * K > 1.2e7:
      M = max(1, M // 2)
    pad = rng.choice([0, 0, 8, 40]) if K % 8 == 0 else rng.choice([0, 3])
    g = torch.Generator().manual_seed(1000 * seed + case)
    x_cpu = _activation(rng, M, K, g)
    xf = torch.zeros(M, K + pad, dtype=torch.bfloat16)
    xf[:, :K] = x_cpu
    x = xf.to(DEV)[:, :K]
    qf = torch.full((M + 1, K + pad), 0x55, dtype=torch.uint8, device=DEV).view(FP8)
    q, s = qf[:M, :K], torch.empty(M, dtype=torch.float32, device=DEV)
    what = (seed, case, M, K, pad, mode)
    ops.quant_rowwise_into(x, q, s, mid, gemm_follows=rng.random() < 0.5)
    torch.cuda.synchronize()
    _same_codes_and_scales(q, s, *to.quantize_rowwise(x_cpu, mode), ("per row",) + what)
    assert (qf[M].view(torch.uint8) == 0x55).all() and (qf[:, K:].view(torch.uint8) == 0x55).all(), what
    ops.quant_tensorwise_into(x, q, s, torch.zeros(1, dtype=torch.int32, device=DEV), mid)
    torch.cuda.synchronize()
    q_ref, s_ref = to.quantize_tensorwise(x_cpu, mode)
    _same_codes_and_scales(q, s, q_ref, s_ref.reshape(-1).expand(M).contiguous(), ("per tensor",) + what)
    if K % 16 == 0 and 32 <= K <= 16384:
      k1 = 8 * rng.randint(1, K // 8 - 1)
      x1, x2 = x_cpu[:, :k1].contiguous().to(DEV), x_cpu[:, k1:].contiguous().to(DEV)
      if ops.cat2_quant_ok(x1, x2):
        ops.quant_rowwise_cat2_into(x1, x2, q, s, mid)
        torch.cuda.synchronize()
        _same_codes_and_scales(q, s, *to.quantize_rowwise(x_cpu, mode), ("cat2", k1) + what)
    if K % 8 == 0 and K >= 16:
      xm = (torch.randn(M, K, generator=g) * 2 + 0.3).to(torch.bfloat16)
      shift = (torch.randn(K, generator=g) * 0.5).to(torch.bfloat16)
      scl = (torch.randn(K, generator=g) * 0.3).to(torch.bfloat16)
      y, q2, s2 = torch.ops.cdit.ln_modulate_quant(xm.to(DEV).reshape(1, M, K), shift.to(DEV), scl.to(DEV),
                                                   1e-6, mid, True)
      torch.cuda.synchronize()
      _same_codes_and_scales(q2.reshape(M, K), s2.reshape(M), *to.quantize_rowwise(y.cpu().reshape(M, K), mode),
                             ("fused producer",) + what)
      y_ref = to.ln_modulate(xm.reshape(1, M, K), shift, scl, 1e-6)
      assert (y.cpu() != y_ref).float().mean().item() <= 2e-3, ("fused producer y",) + what
