"""GPU parity of the weight-only (w8a16) GEMM against the CPU oracle."""
import numpy as np
import pytest
import torch

from helpers import bits_u8, elementwise_ok, max_rel_err
from oracle import c_oracle
from oracle import torch_oracle as to

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
REL_TOL = 1e-2


@pytest.fixture(autouse=True)
def _auto_variant():
  from cache_dit_amd import _native
  _native.set_gemm_variant(-1)
  yield
  _native.set_gemm_variant(-1)


def _problem(M, N, K, seed, bias=True):
  g = torch.Generator().manual_seed(seed)
  x = torch.randn(M, K, generator=g).to(torch.bfloat16)
  w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
  b = (torch.randn(N, generator=g) * 0.01).to(torch.bfloat16) if bias else None
  wq, ws = to.quantize_rowwise(w)
  return x, wq, ws, b


def _run(x, wq, ws, b, epilogue=0):
  from cache_dit_amd import ops
  out = ops.w8a16_mm(x.cuda(), wq.cuda().t(), ws.cuda(), None if b is None else b.cuda(),
                     torch.bfloat16, epilogue)
  torch.cuda.synchronize()
  return out


def _assert_close(out, ref):
  assert out.dtype == torch.bfloat16 and out.shape == ref.shape
  e = max_rel_err(out, ref)
  assert e <= REL_TOL, f"max rel err {e:.3e}"
  assert elementwise_ok(out, ref, REL_TOL)


@pytest.mark.parametrize("variant", [0, 3, 7, 8, 9, 10, 11, 12, 100])
@pytest.mark.parametrize("M,N,K", [(512, 768, 1024), (300, 520, 192), (1, 264, 64), (257, 8, 384)])
def test_variants_with_tails(variant, M, N, K):
  from cache_dit_amd import _native
  p = _problem(M, N, K, seed=M + N + K)
  _native.set_gemm_variant(variant)
  out = _run(*p)
  _assert_close(out, to.w8a16_linear(*p, fused=True))
  _assert_close(out, to.w8a16_linear(*p, fused=False))  # the reference's dequantize-first form


@pytest.mark.parametrize("variant", [0, 3, 7, 8, 9, 10, 11, 12, 100])
def test_exact_small_integers(variant):
  from cache_dit_amd import _native
  g = torch.Generator().manual_seed(12)
  M, N, K = 320, 264, 512
  x = torch.randint(-4, 5, (M, K), generator=g).to(torch.bfloat16)
  w = torch.randint(-4, 5, (N, K), generator=g).float().to(FP8)
  ws = torch.full((N, 1), 0.25)
  _native.set_gemm_variant(variant)
  out = _run(x, w, ws, None)
  assert torch.equal(out.cpu(), to.w8a16_linear(x, w, ws, fused=True))


@pytest.mark.parametrize("M,N,K", [(1, 18432, 3072), (1, 9216, 3072), (3, 264, 384), (16, 512, 128)])
@pytest.mark.parametrize("gelu", [0, 1])
def test_skinny_kernel(M, N, K, gelu):
  from cache_dit_amd import _native
  x, wq, ws, b = _problem(M, N, K, seed=M * 5 + N + K)
  ws = ws * (8 if gelu else 1)
  ref = to.w8a16_linear(x, wq, ws, b, gelu="fused" if gelu else None, fused=True)
  _assert_close(_run(x, wq, ws, b, epilogue=gelu), ref)
  _native.set_gemm_variant(50)
  _assert_close(_run(x, wq, ws, b, epilogue=gelu), ref)


ONE_ROW_SHAPES = [(18432, 3072), (9216, 3072), (1008, 2048), (24, 128), (6160, 4096), (3088, 1024),
                  (528, 1152), (272, 3968)]


@pytest.mark.parametrize("N,K", ONE_ROW_SHAPES)
@pytest.mark.parametrize("gelu", [0, 1])
def test_one_row_kernel(N, K, gelu):
  """M = 1 with K <= 4096 runs a kernel of its own (whole weight rows per wavefront, K walked
  in an interleaved order): automatic choice, forced (51), against the oracle and the 16-row
  kernel (50); row counts that leave partial wavefronts, K with a partial last KiB."""
  from cache_dit_amd import _native
  x, wq, ws, b = _problem(1, N, K, seed=N + K)
  ws = ws * (8 if gelu else 1)
  ref = to.w8a16_linear(x, wq, ws, b, gelu="fused" if gelu else None, fused=True)
  auto = _run(x, wq, ws, b, epilogue=gelu)
  _assert_close(auto, ref)
  _native.set_gemm_variant(51)
  assert torch.equal(_run(x, wq, ws, b, epilogue=gelu), auto)
  _native.set_gemm_variant(50)
  _assert_close(_run(x, wq, ws, b, epilogue=gelu), ref)


@pytest.mark.parametrize("N,K", ONE_ROW_SHAPES)
def test_one_row_kernel_exact_and_k_positions(N, K):
  """Integer operands: bit-equal to the oracle. Then a single 1 in the activation on both
  sides of every boundary of the kernel's K walk (16-byte lane pieces, the two MFMAs of a
  piece, 1 KiB loads) against weights whose value encodes the K index."""
  from cache_dit_amd import _native
  _native.set_gemm_variant(51)
  g = torch.Generator().manual_seed(N + K)
  x = torch.randint(-4, 5, (1, K), generator=g).to(torch.bfloat16)
  w = torch.randint(-4, 5, (N, K), generator=g).float().to(FP8)
  ws = torch.full((N, 1), 0.25)
  assert torch.equal(_run(x, w, ws, None).cpu(), to.w8a16_linear(x, w, ws, fused=True))
  w = ((((torch.arange(K) * 7) % 15) + 1).float().repeat(N, 1) * (1 + (torch.arange(N) % 2)).reshape(-1, 1)).to(FP8)
  ones = torch.ones(N, 1)
  for pos in (0, 7, 8, 15, 16, 31, 127, 128, 1007, 1023, 1024, 1040, 2047, 2048, 3071, 3072, K - 17, K - 1):
    if pos >= K:
      continue
    x = torch.zeros(1, K)
    x[0, pos] = 1.0
    out = _run(x.to(torch.bfloat16), w, ones, None)
    assert torch.equal(out.cpu(), to.w8a16_linear(x.to(torch.bfloat16), w, ones, fused=True)), pos


def test_one_row_kernel_writes_only_its_row():
  from cache_dit_amd import _native
  N, K = 1040, 3072
  x, wq, ws, b = _problem(1, N, K, seed=9)
  ref = to.w8a16_linear(x, wq, ws, b, fused=True)
  buf = torch.full((2, N + 24), 7.0, dtype=torch.bfloat16, device="cuda")
  L = _native.load()
  xg, w, sw, bias = x.cuda(), wq.cuda(), ws.cuda().reshape(-1).contiguous(), b.cuda()
  rc = L.cdit_w8a16_gemm(xg.data_ptr(), w.data_ptr(), sw.data_ptr(), bias.data_ptr(), buf.data_ptr(),
                         1, N, K, K, K, buf.stride(0), 0, _native.DT_BF16, None)
  assert rc == 0, L.cdit_last_error()
  torch.cuda.synchronize()
  assert max_rel_err(buf[0, :N].cpu(), ref[0]) <= REL_TOL
  assert (buf[0, N:] == 7.0).all() and (buf[1] == 7.0).all()


def test_skinny_exact_and_every_code():
  from cache_dit_amd import _native
  g = torch.Generator().manual_seed(14)
  M, N, K = 5, 272, 1024
  x = torch.randint(-4, 5, (M, K), generator=g).to(torch.bfloat16)
  w = torch.randint(-4, 5, (N, K), generator=g).float().to(FP8)
  ws = torch.full((N, 1), 0.25)
  _native.set_gemm_variant(50)
  assert torch.equal(_run(x, w, ws, None).cpu(), to.w8a16_linear(x, w, ws, fused=True))
  # K positions: one-hot activations pick single weights whose value encodes K
  x = torch.zeros(M, K)
  x[torch.arange(M), torch.tensor([0, 33, 130, 517, 1023])] = 1.0
  w = ((torch.arange(K) % 15) + 1).float().repeat(N, 1).to(FP8)
  ones = torch.ones(N, 1)
  assert torch.equal(_run(x.to(torch.bfloat16), w, ones, None).cpu(),
                     to.w8a16_linear(x.to(torch.bfloat16), w, ones, fused=True))


def test_k_position_sensitivity():
  M, N, K = 256, 256, 256
  x = torch.zeros(M, K)
  x[torch.arange(M), torch.arange(M) % K] = 1.0
  w = ((torch.arange(K) % 15) + 1).float().repeat(N, 1)
  ones = torch.ones(N, 1)
  out = _run(x.to(torch.bfloat16), w.to(FP8), ones, None)
  assert torch.equal(out.cpu(), to.w8a16_linear(x.to(torch.bfloat16), w.to(FP8), ones, fused=True))


def test_every_e4m3_code_dequantizes_exactly():
  """x = identity picks out single weights: out[m, n] = float(code) for all 256 codes
  (NaN codes excluded), so the in-loop e4m3 -> bf16 conversion is checked value by value."""
  codes = torch.arange(256, dtype=torch.uint8)
  keep = (codes & 0x7f) != 0x7f
  codes = codes[keep]
  K = 256
  N = 256
  w = torch.zeros(N, K, dtype=torch.uint8)
  w[torch.arange(codes.numel()), torch.arange(codes.numel())] = codes
  wq = w.view(FP8)
  x = torch.eye(K).to(torch.bfloat16)
  out = _run(x, wq, torch.ones(N, 1), None)
  expect = wq.float().t().to(torch.bfloat16)  # exact: every e4m3 value is a bf16 value
  assert torch.equal(out.cpu(), expect)


@pytest.mark.parametrize("K,N", [(3072, 3072), (3072, 9216), (3072, 12288), (12288, 3072),
                                 (15360, 3072)])
def test_flux_shapes_m4608(K, N):
  M = 4608
  x, wq, ws, b = _problem(M, N, K, seed=K + N)
  out = _run(x, wq, ws, b)
  rows = torch.arange(0, M, 37)  # every 37th row against the oracle
  ref = to.w8a16_linear(x[rows], wq, ws, b, fused=True)
  _assert_close(out[rows.cuda()], ref)
  # and against the reference's own definition of the mode, F.linear(x, W.dequantize(), b)
  # with the dequantized weight rounded to bf16 first
  # (src/cache_dit/quantization/torchao/quantize_ao.py:604-610): the kernel applies the
  # scale to the accumulator instead, one rounding less per weight; within max rel err 1e-2
  ref_unfused = to.w8a16_linear(x[rows], wq, ws, b, fused=False)
  assert max_rel_err(out[rows.cuda()], ref_unfused) <= 1e-2


def test_against_c_oracle_and_gelu():
  x, wq, ws, b = _problem(200, 256, 512, seed=8)
  xb = x.view(torch.int16).numpy().view(np.uint16)
  bb = b.view(torch.int16).numpy().view(np.uint16)
  for gelu in (0, 1):
    ref_bits = c_oracle.w8a16(xb, bits_u8(wq), ws.numpy(), bb, gelu=gelu, dequant_bf16=False)
    ref = torch.from_numpy(ref_bits.view(np.int16)).view(torch.bfloat16)
    _assert_close(_run(x, wq, ws * (8 if gelu else 1), b, epilogue=gelu), ref if not gelu else
                  to.w8a16_linear(x, wq, ws * 8, b, gelu="fused", fused=True))


@pytest.mark.parametrize("variant", [7, 8, 9, 10, 11, 12])
def test_wide_kernels_every_short_k_loop(variant):
  """K loops of 3 to 9 steps of 64, more tiles than CUs: every split of a short K loop
  between the steps before a tile's last ones and those last ones, where the DMA stream
  moves on to the next tile and the conversions that a step does for the next one are
  of no use. Exact small-integer data, sampled rows bit for bit."""
  from cache_dit_amd import _native, ops
  M, N = 5000, 3088
  for steps in range(3, 10):
    K = 64 * steps
    g = torch.Generator(device="cuda").manual_seed(steps)
    x = torch.randint(-3, 4, (M, K), generator=g, device="cuda").to(torch.bfloat16)
    w = torch.randint(-3, 4, (N, K), generator=g, device="cuda").float().to(FP8)
    sw = torch.full((N,), 0.25, device="cuda")
    b = torch.randint(-8, 9, (N,), generator=g, device="cuda").to(torch.bfloat16)
    out = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    _native.set_gemm_variant(variant)
    ops.w8a16_into(x, w, sw, b, out, 0)
    torch.cuda.synchronize()
    rows = torch.cat([torch.arange(0, M, 53), torch.arange(M - 5, M)])
    ref = to.w8a16_linear(x[rows.cuda()].cpu(), w.cpu(), sw.cpu().reshape(-1, 1), b.cpu(), fused=True)
    assert torch.equal(out[rows.cuda()].cpu(), ref), (variant, K)


@pytest.mark.parametrize("variant", [7, 8, 9, 10, 11, 12])
def test_wide_kernels_random_shapes_many_tiles_per_workgroup(variant):
  """Random shapes with edge tiles in M and N and more tiles than CUs (persistent
  workgroups run several tiles each), exact small-integer data: sampled rows must
  match the oracle bit for bit."""
  from cache_dit_amd import _native, ops
  rng = torch.Generator().manual_seed(200 + variant)
  for _ in range(6):
    M = int(torch.randint(2000, 9000, (1,), generator=rng))
    N = int(torch.randint(130, 600, (1,), generator=rng)) * 16
    K = int(torch.randint(2, 17, (1,), generator=rng)) * 64
    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    x = torch.randint(-3, 4, (M, K), generator=g, device="cuda").to(torch.bfloat16)
    w = torch.randint(-3, 4, (N, K), generator=g, device="cuda").float().to(FP8)
    sw = torch.full((N,), 0.25, device="cuda")
    b = torch.randint(-8, 9, (N,), generator=g, device="cuda").to(torch.bfloat16)
    out = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    _native.set_gemm_variant(variant)
    ops.w8a16_into(x, w, sw, b, out, 0)
    torch.cuda.synchronize()
    rows = torch.cat([torch.arange(0, M, 61), torch.arange(M - 5, M)])
    ref = to.w8a16_linear(x[rows.cuda()].cpu(), w.cpu(), sw.cpu().reshape(-1, 1), b.cpu(), fused=True)
    assert torch.equal(out[rows.cuda()].cpu(), ref), (M, N, K)


@pytest.mark.parametrize("variant", [-1, 0, 3, 7, 8, 9, 10, 11, 12, 100])
def test_nothing_is_written_outside_the_output(variant):
  """The output is a window of a larger buffer holding a sentinel (ldo > N, rows below),
  M and N leave partial tiles: the window equals the contiguous result, no sentinel changes."""
  from cache_dit_amd import _native, ops
  for M, N, K in [(300, 528, 256), (70, 1040, 384), (5, 272, 640)]:
    g = torch.Generator().manual_seed(M + N)
    x = torch.randint(-3, 4, (M, K), generator=g).to(torch.bfloat16).cuda()
    w = torch.randint(-3, 4, (N, K), generator=g).float().to(FP8).cuda()
    sw = torch.full((N,), 0.25, device="cuda")
    b = torch.randint(-8, 9, (N,), generator=g).to(torch.bfloat16).cuda()
    _native.set_gemm_variant(variant)
    plain = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    ops.w8a16_into(x, w, sw, b, plain, 0)
    buf = torch.full((M + 40, N + 24), -7.0, dtype=torch.bfloat16, device="cuda")
    ops.w8a16_into(x, w, sw, b, buf[:M, :N], 0)
    torch.cuda.synchronize()
    assert torch.equal(buf[:M, :N], plain), (M, N, K)
    assert bool((buf[M:] == -7.0).all()) and bool((buf[:, N:] == -7.0).all()), (M, N, K)
    ref = to.w8a16_linear(x.cpu(), w.cpu(), sw.cpu().reshape(-1, 1), b.cpu(), fused=True)
    assert torch.equal(plain.cpu(), ref), (M, N, K)


def test_very_large_output_stride_takes_a_kernel_with_64_bit_offsets():
  from cache_dit_amd import ops
  g = torch.Generator().manual_seed(9)
  M, N, K, ldo = 5, 272, 640, 1_100_000
  x = torch.randint(-3, 4, (M, K), generator=g).to(torch.bfloat16).cuda()
  w = torch.randint(-3, 4, (N, K), generator=g).float().to(FP8).cuda()
  sw = torch.full((N,), 0.25, device="cuda")
  buf = torch.full((M, ldo), -7.0, dtype=torch.bfloat16, device="cuda")
  for variant in (-1, 7, 12):
    from cache_dit_amd import _native
    _native.set_gemm_variant(variant)
    buf.fill_(-7.0)
    ops.w8a16_into(x, w, sw, None, buf[:, :N], 0)
    ref = to.w8a16_linear(x.cpu(), w.cpu(), sw.cpu().reshape(-1, 1), None, fused=True)
    assert torch.equal(buf[:, :N].cpu(), ref)
    assert bool((buf[:, N:] == -7.0).all())


def _stage(spec, seed, integer=False):
  """spec: list of (M, K, [N...], [epilogue...]). Returns the `acts` list of
  ops.w8a16_batched_into with NaN-filled outputs."""
  acts = []
  for s, (M, K, Ns, epis) in enumerate(spec):
    g = torch.Generator(device="cuda").manual_seed(seed + 17 * s)
    if integer:
      x = torch.randint(-3, 4, (M, K), generator=g, device="cuda").to(torch.bfloat16)
    else:
      x = torch.randn(M, K, generator=g, device="cuda").to(torch.bfloat16)
    ws, wss, bs = [], [], []
    for i, N in enumerate(Ns):
      if integer:
        ws.append(torch.randint(-3, 4, (N, K), generator=g, device="cuda").float().to(FP8))
        wss.append(torch.full((N,), 0.25, device="cuda"))
        b = torch.randint(-8, 9, (N,), generator=g, device="cuda").float().to(torch.bfloat16)
      else:
        ws.append(torch.randn(N, K, generator=g, device="cuda").to(FP8))
        wss.append(torch.rand(N, generator=g, device="cuda") * 0.01 + 0.001)
        b = (torch.randn(N, generator=g, device="cuda") * 0.1).to(torch.bfloat16)
      bs.append(None if i == 1 else b)
    outs = [torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda") for N in Ns]
    acts.append((x, ws, wss, bs, outs, list(epis)))
  return acts


def _one_by_one(x, ws, wss, bs, epis):
  from cache_dit_amd import ops
  outs = []
  for w, s, b, e in zip(ws, wss, bs, epis):
    o = torch.empty((x.shape[0], w.shape[0]), dtype=torch.bfloat16, device="cuda")
    ops.w8a16_into(x, w, s, b, o, e)
    outs.append(o)
  return outs


@pytest.mark.parametrize("spec", [
    # FLUX single block: proj_mlp (GELU) + q/k/v on one activation
    [(4608, 3072, [12288, 3072, 3072, 3072], [1, 0, 0, 0])],
    # FLUX double block, stage by stage: image stream (4096 tokens) + text stream (512 tokens)
    [(4096, 3072, [3072] * 3, [0] * 3), (512, 3072, [3072] * 3, [0] * 3)],
    [(4096, 3072, [3072], [0]), (512, 3072, [3072], [0])],
    [(4096, 3072, [12288], [1]), (512, 3072, [12288], [1])],
    [(4096, 12288, [3072], [0]), (512, 12288, [3072], [0])],
    # ragged everything, three activations
    [(300, 512, [528, 272], [0, 1]), (77, 512, [80], [0]), (1000, 512, [144, 16, 208], [1, 0, 0])],
    # what the tile stream does not take runs as single calls: N not a multiple of 16, M <= 16
    [(300, 512, [520, 264], [0, 0])],
    [(300, 512, [528], [0]), (9, 512, [272], [0])],
])
def test_batched_equals_one_launch_per_member(spec):
  from cache_dit_amd import ops
  acts = _stage(spec, seed=spec[0][0])
  ops.w8a16_batched_into(acts)
  torch.cuda.synchronize()
  for s, (x, ws, wss, bs, outs, epis) in enumerate(acts):
    want = _one_by_one(x, ws, wss, bs, epis)
    for p, (g, w) in enumerate(zip(outs, want)):
      assert torch.equal(g.view(torch.int16), w.view(torch.int16)), f"activation {s} member {p}"


@pytest.mark.parametrize("variant", [7, 8, 9, 10, 11, 12])
def test_batched_every_tile_shape_exact_integers_against_the_oracle(variant):
  from cache_dit_amd import _native, ops
  spec = [(2100, 640, [1104, 528], [0, 0]), (333, 640, [3088], [0]), (40, 640, [272, 80], [0, 0])]
  acts = _stage(spec, seed=variant, integer=True)
  _native.set_gemm_variant(variant)
  ops.w8a16_batched_into(acts)
  torch.cuda.synchronize()
  for s, (x, ws, wss, bs, outs, epis) in enumerate(acts):
    for p, (w, sc, b, o) in enumerate(zip(ws, wss, bs, outs)):
      ref = to.w8a16_linear(x.cpu(), w.cpu(), sc.cpu(), None if b is None else b.cpu(), fused=True)
      assert torch.equal(o.cpu().view(torch.int16), ref.view(torch.int16)), (variant, s, p)


@pytest.mark.parametrize("seed", range(16))
def test_batched_random_shapes_exact_against_the_oracle(seed):
  """Randomly drawn batches (1 to 4 activations of 17 to 700 rows, 1 to 3 members each with N
  a multiple of 16 up to 608, K of 3 to 8 steps of 64, a randomly forced tile shape or the
  automatic choice) on integer-valued data: bit-equal to the CPU oracle, nothing written
  outside the outputs (windows of sentinel-filled buffers)."""
  import random
  from cache_dit_amd import _native, ops
  rnd = random.Random(seed)
  K = 64 * rnd.randint(6, 16)
  n_act = rnd.randint(1, 4)
  budget = 8
  acts, bufs = [], []
  for s in range(n_act):
    M = rnd.choice([17, 33, 64, 100, 255, 256, 257, 300, 511, 700])
    n_mem = rnd.randint(1, min(3, budget - (n_act - s - 1)))
    budget -= n_mem
    Ns = [16 * rnd.randint(1, 38) for _ in range(n_mem)]
    (x, ws, wss, bs, _, _), = _stage([(M, K, Ns, [0] * n_mem)], seed=1000 * seed + s, integer=True)
    outs = []
    for N in Ns:
      buf = torch.full((M + 1, N + 8), 7.0, dtype=torch.bfloat16, device="cuda")
      bufs.append((buf, M, N))
      outs.append(buf[:M, :N])
    acts.append((x, ws, wss, bs, outs, [0] * n_mem))
  variant = rnd.choice([-1, -1, 7, 8, 9, 10, 11, 12])
  _native.set_gemm_variant(variant)
  ops.w8a16_batched_into(acts)
  torch.cuda.synchronize()
  for s, (x, ws, wss, bs, outs, epis) in enumerate(acts):
    for p, (w, sc, b, o) in enumerate(zip(ws, wss, bs, outs)):
      ref = to.w8a16_linear(x.cpu(), w.cpu(), sc.cpu(), None if b is None else b.cpu(), fused=True)
      assert torch.equal(o.cpu().view(torch.int16), ref.view(torch.int16)), (seed, variant, s, p)
  for buf, M, N in bufs:
    assert (buf[M] == 7.0).all() and (buf[:, N:] == 7.0).all(), (seed, variant)


def test_weight_only_sibling_groups_and_stream_batches_in_a_model():
  """float8_weight_only model: group_sibling_linears_ and the stream-batched block forwards
  give the bits of the plain forwards, eager and under graph capture."""
  import logging
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  logging.getLogger("CACHE_DIT_AMD").setLevel(logging.WARNING)
  torch.manual_seed(0)
  kw = dict(dim=512, heads=4, mlp=2048, n_double=2, n_single=3, in_channels=64, text_dim=256,
            pooled_dim=128)
  model = ds.FluxLikeTransformer(**kw).to(torch.bfloat16).cuda()
  cache_dit.quantize(model, cache_dit.QuantizeConfig(quant_type="float8_weight_only"))
  ds.fuse_gelu_epilogues(model)
  inputs = ds.flux_like_inputs("cuda", n_img=320, n_txt=64, in_channels=64, text_dim=256,
                               pooled_dim=128)
  with torch.no_grad():
    y0 = model(**inputs)
    assert cache_dit.group_sibling_linears_(model, lambda: model(**inputs)) == 2 * 2 + 3 * 1
    blk = model.single_transformer_blocks[0]
    assert len(blk.proj_mlp.sibling_group.members) == 4 and blk.proj_mlp.sibling_group.weight_only
    assert torch.equal(model(**inputs), y0)
    assert ds.batch_streams(model) == 2
    assert torch.equal(model(**inputs), y0)
    static = {k: v.clone() for k, v in inputs.items()}
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
      model(**static)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
      ys = model(**static)
    other = ds.flux_like_inputs("cuda", n_img=320, n_txt=64, in_channels=64, text_dim=256,
                                pooled_dim=128, seed=5)
    for src in (other, inputs):
      want = model(**src)
      torch.cuda.synchronize()
      for k in static:
        static[k].copy_(src[k])
      graph.replay()
      torch.cuda.synchronize()
      assert torch.equal(ys, want)
    ds.batch_streams(model, False)
    assert cache_dit.group_sibling_linears_(model, enable=False) == 0
    assert torch.equal(model(**inputs), y0)

  # Qwen-Image- and Wan-shaped toy models: stream batches and sibling groups of weight-only Linears
  qwen = ds.QwenImageLikeTransformer(dim=256, heads=2, mlp=512, n_layers=2, in_channels=64,
                                     text_dim=128).to(torch.bfloat16).cuda()
  cache_dit.quantize(qwen, cache_dit.QuantizeConfig(quant_type="float8_weight_only"))
  qin = ds.qwen_image_like_inputs("cuda", n_img=200, n_txt=24, in_channels=64, text_dim=128)
  wan = ds.WanLikeTransformer(dim=256, heads=2, ffn=512, n_layers=2, in_channels=64,
                              text_dim=128).to(torch.bfloat16).cuda()
  cache_dit.quantize(wan, cache_dit.QuantizeConfig(quant_type="float8_weight_only"))
  winp = ds.wan_like_inputs("cuda", n_tokens=200, n_txt=48, in_channels=64, text_dim=128)
  with torch.no_grad():
    q0 = qwen(**qin)
    assert ds.batch_streams(qwen) == 2
    assert torch.equal(qwen(**qin), q0)
    w0 = wan(**winp)
    assert cache_dit.group_sibling_linears_(wan, lambda: wan(**winp)) == 2 * 2
    assert wan.blocks[0].attn1.to_q.sibling_group.weight_only
    assert torch.equal(wan(**winp), w0)
