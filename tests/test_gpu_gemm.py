"""GPU parity of the row-wise scaled FP8 GEMM (w8a8) against the CPU oracle."""
import numpy as np
import pytest
import torch

from helpers import bits_u8, config1_inputs, elementwise_ok, max_rel_err
from oracle import c_oracle
from oracle import torch_oracle as to

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
REL_TOL = 1e-2  # target: max relative error 1e-2, bf16 out, fp32 accumulate


@pytest.fixture(autouse=True)
def _auto_variant():
  from cache_dit_amd import _native
  _native.set_gemm_variant(-1)
  yield
  _native.set_gemm_variant(-1)


def _rand_problem(M, N, K, seed, bias=True, outliers=True):
  g = torch.Generator().manual_seed(seed)
  x = torch.randn(M, K, generator=g)
  if outliers and K >= 16:
    x[:, torch.randperm(K, generator=g)[:max(1, K // 1000)]] *= 20
  w = torch.randn(N, K, generator=g) * 0.02
  b = (torch.randn(N, generator=g) * 0.01).to(torch.bfloat16) if bias else None
  xq, xs = to.quantize_rowwise(x.to(torch.bfloat16))
  wq, ws = to.quantize_rowwise(w.to(torch.bfloat16))
  return xq, xs, wq, ws, b


def _run(xq, xs, wq, ws, b, epilogue=0):
  from cache_dit_amd import ops
  out = ops.float8_inference_scaled_mm(xq.cuda(), xs.cuda(), wq.cuda().t(), ws.cuda().t(),
                                       torch.bfloat16, bias=None if b is None else b.cuda(),
                                       use_fast_accum=True, epilogue=epilogue)
  torch.cuda.synchronize()
  return out


def _assert_close(out, ref):
  assert out.dtype == torch.bfloat16 and out.shape == ref.shape
  assert torch.isfinite(out.float()).all()
  e = max_rel_err(out, ref)
  assert e <= REL_TOL, f"max rel err {e:.3e} > {REL_TOL}"
  assert elementwise_ok(out, ref, REL_TOL)


TILED_VARIANTS = [0, 1, 6, 7, 12, 14, 15, 16, 17, 18, 20, 21]


@pytest.mark.parametrize("variant", TILED_VARIANTS + [100])
@pytest.mark.parametrize("M,N,K", [(512, 768, 1024), (300, 520, 256), (1, 264, 128),
                                   (257, 8, 384)])
def test_variants_with_tails(variant, M, N, K):
  from cache_dit_amd import _native
  p = _rand_problem(M, N, K, seed=M + N + K)
  ref = to.scaled_mm_rowwise(*p)
  _native.set_gemm_variant(variant)
  _assert_close(_run(*p), ref)


@pytest.mark.parametrize("variant", TILED_VARIANTS + [100])
def test_exact_small_integers(variant):
  """Integer-valued codes and power-of-two scales: every partial sum is exact in
  fp32 whatever the order, so the output must equal the oracle bit for bit."""
  from cache_dit_amd import _native
  g = torch.Generator().manual_seed(11)
  M, N, K = 320, 264, 512
  a = torch.randint(-4, 5, (M, K), generator=g).float().to(FP8)
  w = torch.randint(-4, 5, (N, K), generator=g).float().to(FP8)
  a_s = torch.full((M, 1), 0.5)
  w_s = torch.full((N, 1), 0.25)
  ref = to.scaled_mm_rowwise(a, a_s, w, w_s)
  _native.set_gemm_variant(variant)
  out = _run(a, a_s, w, w_s, None)
  assert torch.equal(out.cpu(), ref)


@pytest.mark.parametrize("M,N,K", [(1, 18432, 3072), (1, 9216, 3072), (3, 264, 384), (16, 512, 128),
                                   (7, 3072, 15360)])
@pytest.mark.parametrize("gelu", [0, 1])
def test_skinny_kernel(M, N, K, gelu):
  """M <= 16 (the M = 1 modulation Linears): automatic choice and forced variant."""
  from cache_dit_amd import _native
  p = _rand_problem(M, N, K, seed=M * 7 + N + K)
  ref = to.scaled_mm_rowwise(*p, gelu="fused" if gelu else None)
  _assert_close(_run(*p, epilogue=gelu), ref)
  _native.set_gemm_variant(50)
  _assert_close(_run(*p, epilogue=gelu), ref)


def test_skinny_exact_and_k_positions():
  from cache_dit_amd import _native
  g = torch.Generator().manual_seed(13)
  M, N, K = 5, 272, 1024
  a = torch.randint(-4, 5, (M, K), generator=g).float().to(FP8)
  w = torch.randint(-4, 5, (N, K), generator=g).float().to(FP8)
  a_s, w_s = torch.full((M, 1), 0.5), torch.full((N, 1), 0.25)
  _native.set_gemm_variant(50)
  assert torch.equal(_run(a, a_s, w, w_s, None).cpu(), to.scaled_mm_rowwise(a, a_s, w, w_s))
  a = torch.zeros(M, K)
  a[torch.arange(M), torch.tensor([0, 33, 130, 517, 1023])] = 1.0
  w = ((torch.arange(K) % 15) + 1).float().repeat(N, 1)
  ones_m, ones_n = torch.ones(M, 1), torch.ones(N, 1)
  assert torch.equal(_run(a.to(FP8), ones_m, w.to(FP8), ones_n, None).cpu(),
                     to.scaled_mm_rowwise(a.to(FP8), ones_m, w.to(FP8), ones_n))


ONE_ROW_SHAPES = [(18432, 3072), (9216, 3072), (1000, 2048), (24, 128), (6152, 4096), (3080, 1024),
                  (520, 1152), (264, 3968)]


@pytest.mark.parametrize("N,K", ONE_ROW_SHAPES)
@pytest.mark.parametrize("gelu", [0, 1])
def test_one_row_kernel(N, K, gelu):
  """M = 1 with K <= 4096 runs a kernel of its own (a wavefront reads whole weight rows, 1 KiB
  per load, and walks K in an interleaved order): automatic choice, forced (51), against the
  oracle and against the 16-row kernel (50); row counts that leave partial wavefronts and
  workgroups, K with a partial last KiB."""
  from cache_dit_amd import _native
  p = _rand_problem(1, N, K, seed=N + K)
  ref = to.scaled_mm_rowwise(*p, gelu="fused" if gelu else None)
  auto = _run(*p, epilogue=gelu)
  _assert_close(auto, ref)
  _native.set_gemm_variant(51)
  forced = _run(*p, epilogue=gelu)
  assert torch.equal(forced, auto)
  _native.set_gemm_variant(50)
  _assert_close(_run(*p, epilogue=gelu), ref)


@pytest.mark.parametrize("N,K", ONE_ROW_SHAPES)
def test_one_row_kernel_exact_and_k_positions(N, K):
  """Integer codes and power-of-two scales make every partial sum exact: bit-equal to the
  oracle. Then a single 1 in the activation, at positions on both sides of every boundary
  of the kernel's K walk (16-byte lane pieces, 1 KiB loads, the pair of loads of one MFMA),
  against weights whose value encodes the K index: a mismatch between the positions the
  weight and the activation operands are fetched from gives a wrong answer."""
  from cache_dit_amd import _native
  _native.set_gemm_variant(51)
  g = torch.Generator().manual_seed(N + K)
  a = torch.randint(-4, 5, (1, K), generator=g).float().to(FP8)
  w = torch.randint(-4, 5, (N, K), generator=g).float().to(FP8)
  a_s, w_s = torch.full((1, 1), 0.5), torch.full((N, 1), 0.25)
  assert torch.equal(_run(a, a_s, w, w_s, None).cpu(), to.scaled_mm_rowwise(a, a_s, w, w_s))
  w = (((torch.arange(K) * 7) % 15) + 1).float().repeat(N, 1) * (1 + (torch.arange(N) % 2)).reshape(-1, 1)
  ones_n = torch.ones(N, 1)
  for pos in (0, 15, 16, 31, 127, 128, 1007, 1023, 1024, 1040, 2047, 2048, 3071, 3072, K - 17, K - 1):
    if pos >= K:
      continue
    a = torch.zeros(1, K)
    a[0, pos] = 1.0
    out = _run(a.to(FP8), torch.ones(1, 1), w.to(FP8), ones_n, None)
    assert torch.equal(out.cpu(), to.scaled_mm_rowwise(a.to(FP8), torch.ones(1, 1), w.to(FP8), ones_n)), pos


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_one_row_kernel_writes_only_its_row(out_dtype):
  """M = 1 into the first row of a larger buffer holding a sentinel, N that leaves a partial
  wavefront: the other elements keep the sentinel, for every output type."""
  from cache_dit_amd import _native
  N, K = 1030, 3072
  xq, xs, wq, ws, b = _rand_problem(1, N, K, seed=5)
  if out_dtype == torch.float16:  # the bias has the output's type; an fp32 output takes none
    b = b.to(torch.float16)
  elif out_dtype == torch.float32:
    b = None
  ref = to.scaled_mm_rowwise(xq, xs, wq, ws, b, out_dtype=out_dtype)
  buf = torch.full((2, N + 26), 7.0, dtype=out_dtype, device="cuda")
  L = _native.load()
  a, sa, w, sw = xq.cuda(), xs.cuda().reshape(-1), wq.cuda(), ws.cuda().reshape(-1).contiguous()
  bias = None if b is None else b.cuda()
  dt_id = {torch.bfloat16: _native.DT_BF16, torch.float16: _native.DT_F16, torch.float32: _native.DT_F32}[out_dtype]
  rc = L.cdit_fp8_gemm_rowwise(a.data_ptr(), sa.data_ptr(), w.data_ptr(), sw.data_ptr(),
                               None if bias is None else bias.data_ptr(), buf.data_ptr(), 1, N, K, K, K,
                               buf.stride(0), 0, dt_id, None)
  assert rc == 0, L.cdit_last_error()
  torch.cuda.synchronize()
  assert max_rel_err(buf[0, :N].cpu(), ref[0]) <= REL_TOL
  assert (buf[0, N:] == 7.0).all() and (buf[1] == 7.0).all()


@pytest.mark.parametrize("scale_mode", [0, 1])
@pytest.mark.parametrize("kind", ["normal", "zero", "tiny", "huge", "nan", "inf"])
def test_one_row_fused_linear_matches_the_two_calls(kind, scale_mode):
  """cdit_fp8_linear_w8a8 at M = 1 (the row quantized inside the GEMM kernel) against the
  quantizer and the GEMM called one after the other, bit for bit: also for a zero row, scales
  outside the fast-division window and rows that hold a NaN or an infinity."""
  from cache_dit_amd import _native, ops
  N, K = 3080, 3072  # not a multiple of the 12 rows of a workgroup
  g = torch.Generator(device="cuda").manual_seed(3 + scale_mode)
  x = (torch.randn(1, K, generator=g, device="cuda") * 2).to(torch.bfloat16)
  if kind == "zero":
    x.zero_()
  elif kind == "tiny":
    x *= 1e-32
  elif kind == "huge":
    x *= 1e32
  elif kind == "nan":
    x[0, 1500] = float("nan")
  elif kind == "inf":
    x[0, 77] = float("inf")
  w = (torch.randn(N, K, generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  wq, w_s = ops.fp8_rowwise_quant(w)
  w_s = w_s.reshape(-1).contiguous()
  bias = (torch.randn(N, generator=g, device="cuda") * 0.1).to(torch.bfloat16)
  L = _native.load()
  q_ws = torch.full((1, K), 0x55, dtype=torch.uint8, device="cuda").view(FP8)
  s_ws = torch.full((1,), -1.0, dtype=torch.float32, device="cuda")
  out = torch.empty(1, N, dtype=torch.bfloat16, device="cuda")
  rc = L.cdit_fp8_linear_w8a8(x.data_ptr(), wq.data_ptr(), w_s.data_ptr(), bias.data_ptr(),
                              out.data_ptr(), q_ws.data_ptr(), s_ws.data_ptr(), 1, N, K, K, K, N,
                              scale_mode, 0, 1, None)
  assert rc == 0, L.cdit_last_error()
  q2 = torch.empty(1, K, dtype=FP8, device="cuda")
  s2 = torch.empty(1, dtype=torch.float32, device="cuda")
  out2 = torch.empty(1, N, dtype=torch.bfloat16, device="cuda")
  ops.quant_rowwise_into(x, q2, s2, scale_mode)
  ops.gemm_rowwise_into(q2, s2, wq, w_s, bias, out2, 0)
  torch.cuda.synchronize()
  assert torch.equal(q_ws.view(torch.uint8), q2.view(torch.uint8))
  assert torch.equal(s_ws.view(torch.int32), s2.view(torch.int32))
  assert torch.equal(out.view(torch.int16), out2.view(torch.int16))
  if kind in ("nan", "inf"):
    assert torch.isnan(out.float()).all()
  else:
    assert torch.isfinite(out.float()).all()


def test_k_position_sensitivity():
  """One non-zero per row of A at a different K position per row against a weight
  whose value encodes its K index: a K-permutation mismatch between the A and B
  operand layouts would show up as a wrong (not just noisy) answer."""
  M, N, K = 256, 256, 256
  a = torch.zeros(M, K)
  a[torch.arange(M), torch.arange(M) % K] = 1.0
  w = ((torch.arange(K) % 15) + 1).float().repeat(N, 1) * (1 + (torch.arange(N) % 2)).reshape(-1, 1)
  ones_m, ones_n = torch.ones(M, 1), torch.ones(N, 1)
  ref = to.scaled_mm_rowwise(a.to(FP8), ones_m, w.to(FP8), ones_n)
  out = _run(a.to(FP8), ones_m, w.to(FP8), ones_n, None)
  assert torch.equal(out.cpu(), ref)


def test_reference_smoke_shape_w32x64_x4x64():
  # tests/kernels/test_opaque_scaled_mm.py:67-74 of the reference: W[32,64], x[4,64], seed 0
  torch.manual_seed(0)
  w = torch.randn(32, 64).to(torch.bfloat16)
  x = torch.randn(4, 64).to(torch.bfloat16)
  xq, xs = to.quantize_rowwise(x)
  wq, ws = to.quantize_rowwise(w)
  ref = to.scaled_mm_rowwise(xq, xs, wq, ws)
  out = _run(xq, xs, wq, ws, None)
  assert out.shape == (4, 32)
  _assert_close(out, ref)


def test_reference_partition_shape_m512_k3072_n3072():
  # tests/kernels/test_rowwise_cudagraph_partition.py:35-37 of the reference
  p = _rand_problem(512, 3072, 3072, seed=2)
  _assert_close(_run(*p), to.scaled_mm_rowwise(*p))


@pytest.mark.parametrize("M,N,K", [
    (6889, 3072, 3072), (6889, 12288, 3072), (6889, 3072, 12288),  # Qwen-Image image stream
    (256, 3072, 3072), (256, 12288, 3072), (256, 3072, 12288),  # Qwen-Image text stream
    (32760, 5120, 5120), (32760, 13824, 5120), (32760, 5120, 13824),  # Wan2.1-14B
    (512, 5120, 5120),  # Wan cross-attention to_k / to_v (text tokens)
    (4608, 3072, 15360), (4608, 12288, 3072),  # FLUX proj_out and the headline shape
])
def test_qwen_and_wan_shapes_sampled_rows(M, N, K):
  """Every (M, N, K) of the Qwen-Image and Wan2.1-14B blocks (odd token counts: 6889 =
  83 x 83, 32760 = 8 x 4095) and the FLUX headline shape, at full size: every 97th row
  plus the last rows against the CPU oracle."""
  from cache_dit_amd import ops
  g = torch.Generator(device="cuda").manual_seed(M + N)
  x = torch.randn(M, K, generator=g, device="cuda").to(torch.bfloat16)
  w = (torch.randn(N, K, generator=g, device="cuda") * 0.02).to(torch.bfloat16)
  b = (torch.randn(N, generator=g, device="cuda") * 0.01).to(torch.bfloat16)
  xq, xs = ops.fp8_rowwise_quant(x)
  wq, ws = ops.fp8_rowwise_quant(w)
  out = ops.float8_inference_scaled_mm(xq, xs, wq.t(), ws.t(), torch.bfloat16, bias=b)
  rows = torch.cat([torch.arange(0, M, 97), torch.arange(M - 3, M)])
  ref = to.scaled_mm_rowwise(xq[rows.cuda()].cpu(), xs[rows.cuda()].cpu(), wq.cpu(), ws.cpu(),
                             b.cpu())
  _assert_close(out[rows.cuda()], ref)
  assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("variant", [12, 14, 15, 16, 17, 18])
def test_wide_kernels_every_short_k_loop(variant):
  """K loops of 3 to 9 steps, more tiles than CUs: the K loop runs its steps in two
  loops (the last steps of a tile, where the DMA stream moves on to the next tile, apart
  from those before them), so every split of a short loop between the two is covered,
  and the steps a tile needs before it may use the kernel at all. Exact small-integer
  data, sampled rows bit for bit."""
  from cache_dit_amd import _native, ops
  M, N = 5000, 3080
  for steps in range(3, 10):
    K = 128 * steps
    g = torch.Generator(device="cuda").manual_seed(steps)
    a = torch.randint(-3, 4, (M, K), generator=g, device="cuda").float().to(FP8)
    w = torch.randint(-3, 4, (N, K), generator=g, device="cuda").float().to(FP8)
    sa = torch.full((M,), 0.5, device="cuda")
    sw = torch.full((N,), 0.25, device="cuda")
    b = torch.randint(-8, 9, (N,), generator=g, device="cuda").to(torch.bfloat16)
    out = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    _native.set_gemm_variant(variant)
    ops.gemm_rowwise_into(a, sa, w, sw, b, out, 0)
    torch.cuda.synchronize()
    rows = torch.cat([torch.arange(0, M, 53), torch.arange(M - 5, M)])
    ref = to.scaled_mm_rowwise(a[rows.cuda()].cpu(), sa[rows.cuda()].cpu().reshape(-1, 1), w.cpu(),
                               sw.cpu().reshape(-1, 1), b.cpu())
    assert torch.equal(out[rows.cuda()].cpu(), ref), (variant, K)


@pytest.mark.parametrize("variant", [12, 14, 15, 16, 17, 18])
def test_wide_kernels_random_shapes_many_tiles_per_workgroup(variant):
  """Random shapes with edge tiles in M and N and more tiles than CUs (a persistent
  workgroup then runs several tiles, the DMA stream crossing tile boundaries), exact
  small-integer data: sampled rows must match the oracle bit for bit."""
  from cache_dit_amd import _native, ops
  rng = torch.Generator().manual_seed(100 + variant)
  for _ in range(6):
    M = int(torch.randint(2000, 9000, (1,), generator=rng))
    N = int(torch.randint(250, 1200, (1,), generator=rng)) * 8
    K = int(torch.randint(2, 13, (1,), generator=rng)) * 128
    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    a = torch.randint(-3, 4, (M, K), generator=g, device="cuda").float().to(FP8)
    w = torch.randint(-3, 4, (N, K), generator=g, device="cuda").float().to(FP8)
    sa = torch.full((M,), 0.5, device="cuda")
    sw = torch.full((N,), 0.25, device="cuda")
    b = torch.randint(-8, 9, (N,), generator=g, device="cuda").to(torch.bfloat16)
    out = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    _native.set_gemm_variant(variant)
    ops.gemm_rowwise_into(a, sa, w, sw, b, out, 0)
    torch.cuda.synchronize()
    rows = torch.cat([torch.arange(0, M, 61), torch.arange(M - 5, M)])
    ref = to.scaled_mm_rowwise(a[rows.cuda()].cpu(), sa[rows.cuda()].cpu().reshape(-1, 1), w.cpu(),
                               sw.cpu().reshape(-1, 1), b.cpu())
    assert torch.equal(out[rows.cuda()].cpu(), ref), (M, N, K)


def test_config1_full():
  x, w, b = config1_inputs()
  xq, xs = to.quantize_rowwise(x[0])
  wq, ws = to.quantize_rowwise(w)
  ref = to.scaled_mm_rowwise(xq, xs, wq, ws, b)
  _assert_close(_run(xq, xs, wq, ws, b), ref)


@pytest.mark.parametrize("M,N,K", [(333, 512, 1024), (64, 256, 3072)])
def test_against_c_oracle(M, N, K):
  """The plain-C restatement (double accumulation) as a second checker."""
  xq, xs, wq, ws, b = _rand_problem(M, N, K, seed=5)
  ref_bits = c_oracle.gemm_rowwise(bits_u8(xq), xs.numpy(), bits_u8(wq), ws.numpy(),
                                   b.view(torch.int16).numpy().view(np.uint16))
  ref = torch.from_numpy(ref_bits.view(np.int16)).view(torch.bfloat16)
  _assert_close(_run(xq, xs, wq, ws, b), ref)


@pytest.mark.parametrize("variant", [0, 1, 12, 14, 17, 21, 100])
def test_gelu_tanh_epilogue(variant):
  from cache_dit_amd import _native
  p = _rand_problem(384, 512, 1024, seed=9)
  # make the pre-activation O(1) so that GELU is exercised away from zero
  p = (p[0], p[1] * 8, p[2], p[3], p[4])
  fused = to.scaled_mm_rowwise(*p, gelu="fused")
  unfused = to.scaled_mm_rowwise(*p, gelu="unfused")
  _native.set_gemm_variant(variant)
  out = _run(*p, epilogue=1)
  _assert_close(out, fused)
  _assert_close(out, unfused)  # one bf16 rounding apart: inside the same bar


def test_against_torch_scaled_mm_on_gpu():
  """torch._scaled_mm (hipBLASLt row-wise FP8, a library routine) fed with the same
  codes and scales: a second witness for the GEMM at the FLUX MLP shape."""
  M, N, K = 4608, 12288, 3072
  g = torch.Generator(device="cuda").manual_seed(3)
  a = torch.randn(M, K, generator=g, device="cuda").to(torch.bfloat16)
  w = (torch.randn(N, K, generator=g, device="cuda") * 0.02).to(torch.bfloat16)
  b = (torch.randn(N, generator=g, device="cuda") * 0.01).to(torch.bfloat16)
  from cache_dit_amd import ops
  aq, a_s = ops.fp8_rowwise_quant(a)
  wq, w_s = ops.fp8_rowwise_quant(w)
  out = ops.float8_inference_scaled_mm(aq, a_s, wq.t(), w_s.t(), torch.bfloat16, bias=b)
  try:
    ref = torch._scaled_mm(aq, wq.t(), scale_a=a_s, scale_b=w_s.t(), bias=b,
                           out_dtype=torch.bfloat16)
  except Exception as e:  # pragma: no cover - depends on the box's hipBLASLt
    pytest.skip(f"torch._scaled_mm row-wise not available here: {e}")
  assert max_rel_err(out, ref) <= REL_TOL
  # linearity in the scales (size-independent property at the full shape)
  out2 = ops.float8_inference_scaled_mm(aq, a_s * 2, wq.t(), w_s.t() * 0.5, torch.bfloat16,
                                        bias=b)
  assert torch.equal(out2, out)


def test_scalar_scales_and_misaligned_scale_slices():
  """Tensor-wise (one-element) scales are taken as the reference's op takes them, and a
  scale vector that is a slice starting off a 16-byte boundary gives the same bits as an
  aligned copy."""
  from cache_dit_amd import ops
  xq, xs, wq, ws, b = (t.cuda() if t is not None else None for t in _rand_problem(300, 520, 512, 11))
  sa, sb = torch.tensor([[0.03125]], device="cuda"), torch.tensor([[0.5]], device="cuda")
  out = ops.float8_inference_scaled_mm(xq, sa, wq.t(), sb, torch.bfloat16, bias=b)
  ref = to.scaled_mm_rowwise(xq.cpu(), sa.cpu().expand(300, 1), wq.cpu(), sb.cpu().expand(520, 1),
                             b.cpu())
  _assert_close(out, ref)
  pad_a = torch.cat([torch.zeros(1, device="cuda"), xs.reshape(-1)])
  pad_b = torch.cat([torch.zeros(3, device="cuda"), ws.reshape(-1)])
  assert pad_a[1:].data_ptr() % 16 != 0 and pad_b[3:].data_ptr() % 16 != 0
  want = ops.float8_inference_scaled_mm(xq, xs, wq.t(), ws.t(), torch.bfloat16, bias=b)
  got = ops.float8_inference_scaled_mm(xq, pad_a[1:].reshape(-1, 1), wq.t(), pad_b[3:].reshape(1, -1),
                                       torch.bfloat16, bias=b)
  assert torch.equal(got, want)


def test_error_paths():
  from cache_dit_amd import ops
  a = torch.zeros(4, 64, device="cuda").to(FP8)
  w = torch.zeros(32, 64, device="cuda").to(FP8)
  s_a, s_w = torch.ones(4, 1, device="cuda"), torch.ones(1, 32, device="cuda")
  with pytest.raises(NotImplementedError):
    ops.float8_inference_scaled_mm(a, s_a, w.t(), s_w, torch.bfloat16, output_scale=s_a)
  with pytest.raises(ValueError):
    ops.float8_inference_scaled_mm(a, s_a, w.t(), s_w, torch.float64)
  with pytest.raises(ValueError):
    ops.float8_inference_scaled_mm(a, s_a[:2], w.t(), s_w, torch.bfloat16)
  from cache_dit_amd import _native
  L = _native.load()
  o = torch.zeros(4, 32, dtype=torch.bfloat16, device="cuda")
  rc = L.cdit_fp8_gemm_rowwise(a.data_ptr(), s_a.data_ptr(), w.data_ptr(), s_w.data_ptr(), None,
                               o.data_ptr(), 4, 32, 40, 64, 64, 32, 0, 1, None)
  assert rc == 1 and b"multiple of 16" in L.cdit_last_error()
  rc = L.cdit_fp8_gemm_rowwise(a.data_ptr(), s_a.data_ptr(), w.data_ptr(), s_w.data_ptr(), None,
                               o.data_ptr(), 0, 32, 64, 64, 64, 32, 0, 1, None)
  assert rc == 0  # empty M is a no-op


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K,variant", [(300, 520, 1024, -1), (2100, 1800, 512, 15),
                                           (2100, 1800, 1024, 17), (5, 264, 256, -1),
                                           (64, 48, 64, -1), (257, 72, 384, 100)])
def test_output_dtypes(out_dtype, M, N, K, variant):
  """The op's three out_dtype ids (reference _scaled_mm.py:38-59): fp16 and fp32 outputs
  through the wide kernel (both tiles built for them), the skinny and the generic kernel,
  against the oracle; an fp32 output with bias is the matmul plus a separate add."""
  from cache_dit_amd import _native, ops
  g = torch.Generator().manual_seed(M + N + K)
  x = torch.randn(M, K, generator=g).to(torch.bfloat16)
  w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16)
  b = (torch.randn(N, generator=g) * 0.1).to(out_dtype)
  aq, a_s = to.quantize_rowwise(x)
  wq, w_s = to.quantize_rowwise(w)
  ref = to.scaled_mm_rowwise(aq, a_s, wq, w_s, b, out_dtype=out_dtype)
  _native.set_gemm_variant(variant)
  out = ops.float8_inference_scaled_mm(aq.cuda(), a_s.cuda(), wq.cuda().t(), w_s.cuda().t(),
                                       out_dtype, bias=b.cuda())
  torch.cuda.synchronize()
  assert out.dtype == out_dtype and out.shape == ref.shape
  assert max_rel_err(out, ref) <= REL_TOL
  assert elementwise_ok(out, ref, REL_TOL)
  # GELU in the epilogue (no bias for fp32: the separate add would come after it)
  bias = None if out_dtype == torch.float32 else b
  ref = to.scaled_mm_rowwise(aq, a_s * 4, wq, w_s, bias, gelu="fused", out_dtype=out_dtype)
  out = ops.float8_inference_scaled_mm(aq.cuda(), a_s.cuda() * 4, wq.cuda().t(), w_s.cuda().t(),
                                       out_dtype, bias=None if bias is None else bias.cuda(),
                                       epilogue=1)
  assert max_rel_err(out, ref) <= REL_TOL


def test_output_dtypes_exact():
  """Small integers: every product and sum is exact, so fp16 / fp32 outputs must equal the
  oracle bit for bit."""
  from cache_dit_amd import ops
  g = torch.Generator().manual_seed(5)
  M, N, K = 700, 392, 768
  a = torch.randint(-4, 5, (M, K), generator=g).float().to(FP8)
  w = torch.randint(-4, 5, (N, K), generator=g).float().to(FP8)
  s_a = torch.full((M, 1), 0.5)
  s_w = torch.full((N, 1), 0.25)
  for dt in (torch.float16, torch.float32):
    b = torch.randint(-8, 9, (N,), generator=g).to(dt)
    ref = to.scaled_mm_rowwise(a, s_a, w, s_w, b, out_dtype=dt)
    out = ops.float8_inference_scaled_mm(a.cuda(), s_a.cuda(), w.cuda().t(), s_w.cuda().t(), dt,
                                         bias=b.cuda())
    assert torch.equal(out.cpu(), ref)


def test_output_dtypes_second_witness():
  """torch._scaled_mm on the same codes at fp16 / fp32 output, where the vendor library
  offers it (on ROCm its row-wise FP8 matmul may only build bf16 outputs: then skipped)."""
  from cache_dit_amd import ops
  g = torch.Generator(device="cuda").manual_seed(6)
  x = torch.randn(1024, 1024, generator=g, device="cuda").to(torch.bfloat16)
  wt = (torch.randn(768, 1024, generator=g, device="cuda") * 0.03).to(torch.bfloat16)
  aq, a_s = ops.fp8_rowwise_quant(x)
  wq, w_s = ops.fp8_rowwise_quant(wt)
  for dt in (torch.float16, torch.float32):
    out = ops.float8_inference_scaled_mm(aq, a_s, wq.t(), w_s.t(), dt)
    try:
      ref = torch._scaled_mm(aq, wq.t(), scale_a=a_s, scale_b=w_s.t(), out_dtype=dt)
    except Exception as e:  # pragma: no cover - depends on the box's hipBLASLt
      pytest.skip(f"torch._scaled_mm row-wise {dt} not available here: {e}")
    assert max_rel_err(out, ref) <= REL_TOL


@pytest.mark.parametrize("out_dtype", [torch.float16, torch.float32])
def test_fused_linear_entry_point_with_other_output_dtypes(out_dtype):
  """cdit_fp8_linear_w8a8 (quantizer + GEMM in one call) passes out_dtype_id through:
  same result as the two entry points called one after the other."""
  from cache_dit_amd import _native, ops
  M, N, K = 640, 384, 768
  g = torch.Generator(device="cuda").manual_seed(31)
  x = torch.randn(M, K, generator=g, device="cuda").to(torch.bfloat16)
  w = (torch.randn(N, K, generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  wq, w_s = ops.fp8_rowwise_quant(w)
  w_s = w_s.reshape(-1).contiguous()
  bias = None if out_dtype == torch.float32 else (torch.randn(N, generator=g, device="cuda") * 0.1).to(out_dtype)
  q_ws = torch.empty(M, K, dtype=FP8, device="cuda")
  s_ws = torch.empty(M, dtype=torch.float32, device="cuda")
  out = torch.empty(M, N, dtype=out_dtype, device="cuda")
  L = _native.load()
  rc = L.cdit_fp8_linear_w8a8(x.data_ptr(), wq.data_ptr(), w_s.data_ptr(),
                              None if bias is None else bias.data_ptr(), out.data_ptr(),
                              q_ws.data_ptr(), s_ws.data_ptr(), M, N, K, K, K, N, 0, 0,
                              ops.encode_output_dtype(out_dtype), None)
  assert rc == 0, L.cdit_last_error()
  torch.cuda.synchronize()
  aq, a_s = ops.fp8_rowwise_quant(x)
  assert torch.equal(q_ws.view(torch.uint8), aq.view(torch.uint8))
  ref = ops.float8_inference_scaled_mm(aq, a_s, wq.t(), w_s.reshape(1, -1), out_dtype, bias=bias)
  assert torch.equal(out, ref)
  cpu = to.scaled_mm_rowwise(aq.cpu(), a_s.cpu(), wq.cpu(), w_s.cpu(),
                             None if bias is None else bias.cpu(), out_dtype=out_dtype)
  assert max_rel_err(out, cpu) <= REL_TOL


def test_wide_variants_agree_bit_for_bit_on_random_data():
  """All tiles of the wide kernel accumulate K in the same order with the same MFMA, so on the
  same (random, non-integer) operands they must give identical outputs, edge tiles included."""
  from cache_dit_amd import _native, ops
  g = torch.Generator(device="cuda").manual_seed(77)
  for (M, N, K) in [(1000, 1160, 1024), (2345, 520, 768), (333, 2056, 2048)]:
    bits = torch.randint(0, 256, (M, K), dtype=torch.uint8, device="cuda", generator=g)
    a = (bits & 0xBF).view(FP8)
    bits = torch.randint(0, 256, (N, K), dtype=torch.uint8, device="cuda", generator=g)
    w = (bits & 0xBF).view(FP8)
    sa = torch.rand(M, device="cuda", generator=g) + 0.5
    sw = torch.rand(N, device="cuda", generator=g) * 1e-3
    b = torch.randn(N, device="cuda", generator=g).to(torch.bfloat16)
    outs = []
    for variant in (12, 14, 15, 16, 17, 18):
      _native.set_gemm_variant(variant)
      for epi in (0, 1):
        out = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
        ops.gemm_rowwise_into(a, sa, w, sw, b, out, epi)
        outs.append((variant, epi, out))
    torch.cuda.synchronize()
    for variant, epi, out in outs[2:]:
      assert torch.equal(out, outs[epi][2]), (M, N, K, variant, epi)


@pytest.mark.parametrize("scale_mode", [0, 1])
@pytest.mark.parametrize("M,N,K", [(1, 18432, 3072), (1, 9216, 3072), (3, 264, 256), (15, 520, 3072),
                                   (16, 512, 3072), (16, 72, 128), (2, 4096, 15360)])
def test_fused_linear_for_few_rows_matches_the_two_calls(M, N, K, scale_mode):
  """cdit_fp8_linear_w8a8 at M <= 16 runs one kernel that quantizes the rows itself (when
  M (K + 16) bytes of codes fit in 48 KiB of LDS; (16, ., 3072) does not and takes the two
  kernels): codes, scales and outputs must equal those of the quantizer and the GEMM called
  one after the other, bit for bit, including zero rows and scales outside the fast-division
  window."""
  from cache_dit_amd import _native, ops
  g = torch.Generator(device="cuda").manual_seed(M * 7 + N + K + scale_mode)
  x = (torch.randn(M, K, generator=g, device="cuda") * 2).to(torch.bfloat16)
  if M >= 3:
    x[0] = 0
    x[1] = x[1] * 1e-32
    x[2] = x[2] * 1e32
  w = (torch.randn(N, K, generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  wq, w_s = ops.fp8_rowwise_quant(w)
  w_s = w_s.reshape(-1).contiguous()
  bias = (torch.randn(N, generator=g, device="cuda") * 0.1).to(torch.bfloat16)
  L = _native.load()
  for epi in (0, 1):
    q_ws = torch.full((M, K), 0x55, dtype=torch.uint8, device="cuda").view(FP8)
    s_ws = torch.full((M,), -1.0, dtype=torch.float32, device="cuda")
    out = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    rc = L.cdit_fp8_linear_w8a8(x.data_ptr(), wq.data_ptr(), w_s.data_ptr(), bias.data_ptr(),
                                out.data_ptr(), q_ws.data_ptr(), s_ws.data_ptr(), M, N, K, K, K, N,
                                scale_mode, epi, 1, None)
    assert rc == 0, L.cdit_last_error()
    q2 = torch.empty(M, K, dtype=FP8, device="cuda")
    s2 = torch.empty(M, dtype=torch.float32, device="cuda")
    out2 = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
    ops.quant_rowwise_into(x, q2, s2, scale_mode)
    ops.gemm_rowwise_into(q2, s2, wq, w_s, bias, out2, epi)
    torch.cuda.synchronize()
    assert torch.equal(q_ws.view(torch.uint8), q2.view(torch.uint8))
    assert torch.equal(s_ws.view(torch.int32), s2.view(torch.int32))
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))


@pytest.mark.parametrize("variant", [-1] + TILED_VARIANTS + [100])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16, torch.float32])
def test_nothing_is_written_outside_the_output(variant, dt):
  """The output is a window of a larger buffer (rows below it, columns to its right, ldo > N)
  holding a sentinel, with M and N that leave partial tiles in both directions: the window
  must equal the result of the contiguous call and not one sentinel may change."""
  from cache_dit_amd import _native, ops
  for M, N, K in [(300, 528, 256), (70, 1040, 384), (5, 272, 640)]:
    g = torch.Generator().manual_seed(M + N)
    a = torch.randint(-4, 5, (M, K), generator=g).float().to(FP8).cuda()
    w = torch.randint(-4, 5, (N, K), generator=g).float().to(FP8).cuda()
    s_a = torch.full((M,), 0.5, device="cuda")
    s_w = torch.full((N,), 0.25, device="cuda")
    b = None if dt == torch.float32 else torch.randint(-8, 9, (N,), generator=g).to(dt).cuda()
    _native.set_gemm_variant(variant)
    plain = torch.empty(M, N, dtype=dt, device="cuda")
    ops.gemm_rowwise_into(a, s_a, w, s_w, b, plain, 0)
    buf = torch.full((M + 40, N + 24), -7.0, dtype=dt, device="cuda")
    ops.gemm_rowwise_into(a, s_a, w, s_w, b, buf[:M, :N], 0)
    torch.cuda.synchronize()
    assert torch.equal(buf[:M, :N], plain), (M, N, K)
    assert bool((buf[M:] == -7.0).all()) and bool((buf[:, N:] == -7.0).all()), (M, N, K)
    ref = to.scaled_mm_rowwise(a.cpu(), s_a.cpu().reshape(-1, 1), w.cpu(), s_w.cpu().reshape(-1, 1),
                               None if b is None else b.cpu(), out_dtype=dt)
    assert torch.equal(plain.cpu(), ref), (M, N, K)


def test_very_large_output_stride_takes_a_kernel_with_64_bit_offsets():
  """The wide kernels address a block of output rows with 32-bit byte offsets and are only
  chosen when 512 * ldo fits; a window of a very wide buffer must still come out right."""
  from cache_dit_amd import ops
  g = torch.Generator().manual_seed(9)
  M, N, K, ldo = 5, 272, 640, 1_100_000
  a = torch.randint(-4, 5, (M, K), generator=g).float().to(FP8).cuda()
  w = torch.randint(-4, 5, (N, K), generator=g).float().to(FP8).cuda()
  s_a = torch.full((M,), 0.5, device="cuda")
  s_w = torch.full((N,), 0.25, device="cuda")
  buf = torch.full((M, ldo), -7.0, dtype=torch.bfloat16, device="cuda")
  ops.gemm_rowwise_into(a, s_a, w, s_w, None, buf[:, :N], 0)
  ref = to.scaled_mm_rowwise(a.cpu(), s_a.cpu().reshape(-1, 1), w.cpu(), s_w.cpu().reshape(-1, 1))
  assert torch.equal(buf[:, :N].cpu(), ref)
  assert bool((buf[:, N:] == -7.0).all())


def test_scales_and_bias_at_odd_offsets():
  """a_scale, b_scale and bias that are only 4-byte (2-byte) aligned: the kernels that fetch
  them in 16-byte pieces must not be chosen; the result is the same."""
  from cache_dit_amd import ops
  g = torch.Generator().manual_seed(10)
  M, N, K = 600, 400, 512
  a = torch.randint(-4, 5, (M, K), generator=g).float().to(FP8).cuda()
  w = torch.randint(-4, 5, (N, K), generator=g).float().to(FP8).cuda()
  s_a = (torch.rand(M + 1, generator=g) + 0.5).cuda()
  s_w = (torch.rand(N + 1, generator=g) * 0.01).cuda()
  b = torch.randint(-8, 9, (N + 1,), generator=g).to(torch.bfloat16).cuda()
  ref = to.scaled_mm_rowwise(a.cpu(), s_a[1:].cpu().reshape(-1, 1), w.cpu(), s_w[1:].cpu().reshape(-1, 1),
                             b[1:].cpu())
  out = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
  ops.gemm_rowwise_into(a, s_a[1:], w, s_w[1:], b[1:], out, 0)
  torch.cuda.synchronize()
  _assert_close(out, ref)
  aligned = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
  ops.gemm_rowwise_into(a, s_a[1:].clone(), w, s_w[1:].clone(), b[1:].clone(), aligned, 0)
  assert torch.equal(out, aligned) or max_rel_err(out, aligned.cpu()) <= REL_TOL


@pytest.mark.parametrize("M,N,K", [(4608, 12288, 3072), (1000, 840, 512)])
def test_measurement_instance_with_time_stamps_gives_the_same_bits(M, N, K):
  """cdit_debug_gemm_stamps runs the 288 x 192 kernel with four stamps per workgroup added:
  the output must be the ordinary kernel's bit for bit, every workgroup that the launcher
  reports must have written a start before its end, a hardware XCD id below 8 and a tile
  count, and the tile counts must add up to the tiles of the problem."""
  import ctypes
  from cache_dit_amd import _native
  L = _native.load()
  g = torch.Generator().manual_seed(M + K)
  a = (torch.randn(M, K, generator=g) * 40).cuda().to(FP8)
  w = (torch.randn(N, K, generator=g) * 40).cuda().to(FP8)
  sa = (torch.rand(M, 1, generator=g) + 0.5).cuda()
  sw = (torch.rand(1, N, generator=g) * 1e-3).cuda()
  b = torch.randn(N, generator=g).to(torch.bfloat16).cuda()
  ref = torch.full((M, N), 7.0, dtype=torch.bfloat16, device="cuda")
  out = torch.full((M, N), -7.0, dtype=torch.bfloat16, device="cuda")
  _native.set_gemm_variant(14)
  _native.check(L.cdit_fp8_gemm_rowwise(a.data_ptr(), sa.data_ptr(), w.data_ptr(), sw.data_ptr(),
                                        b.data_ptr(), ref.data_ptr(), M, N, K, K, K, N, 0, 1, None))
  stamps = torch.zeros(4 * 512, dtype=torch.int64, device="cuda")
  n_wg = ctypes.c_int(0)
  _native.check(L.cdit_debug_gemm_stamps(a.data_ptr(), sa.data_ptr(), w.data_ptr(), sw.data_ptr(),
                                         b.data_ptr(), out.data_ptr(), M, N, K, K, K, N,
                                         stamps.data_ptr(), ctypes.byref(n_wg), None))
  torch.cuda.synchronize()
  assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
  assert 0 < n_wg.value <= 512
  st = stamps.view(-1, 4).cpu()
  used, rest = st[:n_wg.value], st[n_wg.value:]
  assert (rest == 0).all()
  assert (used[:, 1] > used[:, 0]).all() and (used[:, 0] > 0).all()
  assert ((used[:, 2] >= 0) & (used[:, 2] < 8)).all()
  assert int(used[:, 3].sum()) == ((M + 287) // 288) * ((N + 191) // 192)
  # too small for this kernel: refused with a message, nothing launched
  rc = L.cdit_debug_gemm_stamps(a.data_ptr(), sa.data_ptr(), w.data_ptr(), sw.data_ptr(),
                                b.data_ptr(), out.data_ptr(), 16, N, K, K, K, N,
                                stamps.data_ptr(), ctypes.byref(n_wg), None)
  assert rc != 0 and b"288 x 192" in L.cdit_last_error()
