"""GPU parity of the per-row FP8 quantizer: codes and scales bit-exact against
the CPU oracle, called through the C ABI (ctypes) and through the torch op."""
import numpy as np
import pytest
import torch

from helpers import all_finite_bf16, bits_u32, bits_u8, config1_inputs
from oracle import torch_oracle as to

pytestmark = pytest.mark.gpu
MODES = ["bf16div", "fp32div"]


def _check(x_cpu: torch.Tensor, mode: str, x_gpu=None):
  from cache_dit_amd import ops

  xg = x_cpu.cuda() if x_gpu is None else x_gpu
  q, s = ops.fp8_rowwise_quant(xg, mode)
  torch.cuda.synchronize()
  q_ref, s_ref = to.quantize_rowwise(x_cpu, mode)
  assert q.shape == x_cpu.shape and s.shape == (*x_cpu.shape[:-1], 1)
  assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
  s_bad = int((bits_u32(s) != bits_u32(s_ref)).sum())
  q_bad = int((bits_u8(q) != bits_u8(q_ref)).sum())
  assert s_bad == 0, f"{s_bad} scales differ"
  assert q_bad == 0, f"{q_bad} of {q_ref.numel()} codes differ"


@pytest.mark.parametrize("mode", MODES)
def test_config1_bit_exact(mode):
  x, _, _ = config1_inputs()
  _check(x, mode)


@pytest.mark.parametrize("mode", MODES)
def test_every_bf16_value_grouped_by_magnitude(mode):
  # rows of 256 neighbouring magnitudes: quotients cover the whole code range
  v = all_finite_bf16()
  order = torch.argsort(v.float().abs(), stable=True)
  v = v[order]
  n = (v.numel() // 256) * 256
  _check(v[:n].reshape(-1, 256).contiguous(), mode)


@pytest.mark.parametrize("mode", MODES)
def test_every_bf16_value_times_scales(mode):
  # each row: a random sample of all values below a per-row cap -> many amax values
  g = torch.Generator().manual_seed(1)
  v = all_finite_bf16()
  rows = []
  for i in range(512):
    cap = float(2.0**((i % 64) - 32)) * (1.0 + (i // 64) / 8.0)
    pool = v[v.float().abs() <= cap]
    pick = pool[torch.randint(pool.numel(), (1024, ), generator=g)]
    pick[i % 1024] = torch.tensor(cap).to(torch.bfloat16)
    rows.append(pick)
  _check(torch.stack(rows), mode)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("M,K", [(1, 3072), (3, 16), (7, 8), (5, 100), (2, 1000), (4, 4096 + 8),
                                 (2, 16384), (2, 20000), (33, 5120), (9, 15360), (257, 512)])
def test_shapes(mode, M, K):
  g = torch.Generator().manual_seed(M * 1000 + K)
  x = (torch.randn(M, K, generator=g) * 3).to(torch.bfloat16)
  _check(x, mode)


@pytest.mark.parametrize("mode", MODES)
def test_zero_rows_signed_zero_and_extremes(mode):
  g = torch.Generator().manual_seed(3)
  x = torch.randn(8, 1024, generator=g).to(torch.bfloat16)
  x[0] = 0  # all-zero row: scale 1, codes 0
  x[1] = -0.0  # negative zeros: codes 0x80
  x[2, 1:] = 0  # single non-zero element
  x[3] = x[3] * 1e-30  # scale below the fast-division window
  x[4] = x[4] * 1e30  # ... and above it
  x[5] = x[5] * 1e-38  # bf16 subnormals
  x[6, ::2] = -x[6, ::2].abs() * 1e-6  # tiny negatives next to large values
  x[7, 0] = 3.0e38
  _check(x, mode)
  from cache_dit_amd import ops
  q, s = ops.fp8_rowwise_quant(x.cuda(), mode)
  assert float(s[0]) == 1.0 and int(bits_u8(q[0]).max()) == 0
  assert (bits_u8(q[1]) == 0x80).all()


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("K", [512, 4096 + 8])
def test_non_finite_rows_stay_in_their_row(mode, K):
  """Rows with Inf or NaN are outside the bit-exact contract; what is checked is that they
  neither hang the kernel nor leak into their neighbours: every other row is bit-exact, an
  Inf row gets an infinite scale (amax/448) and a NaN row a NaN scale, as in the reference
  arithmetic (torch.amax propagates NaN)."""
  g = torch.Generator().manual_seed(5 + K)
  x = torch.randn(12, K, generator=g).to(torch.bfloat16)
  x[3, 7] = float("inf")
  x[5, K - 1] = float("-inf")
  x[8, 100] = float("nan")
  from cache_dit_amd import ops
  q, s = ops.fp8_rowwise_quant(x.cuda(), mode)
  torch.cuda.synchronize()
  q_ref, s_ref = to.quantize_rowwise(x, mode)
  good = torch.tensor([r not in (3, 5, 8) for r in range(12)])
  assert (bits_u8(q)[good] == bits_u8(q_ref)[good]).all()
  assert (bits_u32(s).reshape(-1)[good] == bits_u32(s_ref).reshape(-1)[good]).all()
  s = s.reshape(-1).cpu()
  assert torch.isinf(s[3]) and torch.isinf(s[5]) and torch.isnan(s[8])
  assert torch.isinf(s_ref.reshape(-1)[3]) and torch.isnan(s_ref.reshape(-1)[8])
  # the codes of those rows follow the reference arithmetic too: finite / Inf = +-0,
  # Inf / Inf = NaN, anything / NaN = NaN, and torch.clamp keeps NaN
  qb, qr = bits_u8(q), bits_u8(q_ref)
  is_nan = lambda c: (c & 0x7f) == 0x7f  # noqa: E731  (0x7f / 0xff are e4m3fn's NaNs)
  for row, col in ((3, 7), (5, K - 1)):
    others = np.arange(K) != col
    assert (qb[row][others] == qr[row][others]).all() and (qb[row][others] & 0x7f == 0).all()
    assert is_nan(qb[row][col]) and is_nan(qr[row][col])
  assert is_nan(qb[8]).all() and is_nan(qr[8]).all()


@pytest.mark.parametrize("mode", MODES)
def test_strided_rows_and_leading_dims(mode):
  g = torch.Generator().manual_seed(4)
  base = torch.randn(6, 20, 640, generator=g).to(torch.bfloat16)
  from cache_dit_amd import ops
  xg = base.cuda()[:, :, :512]  # row stride 640, K = 512
  q, s = ops.fp8_rowwise_quant(xg, mode)
  q_ref, s_ref = to.quantize_rowwise(base[:, :, :512], mode)
  assert (bits_u8(q) == bits_u8(q_ref)).all() and (bits_u32(s) == bits_u32(s_ref)).all()


def test_c_abi_direct_with_leading_dimension():
  """Calls cdit_fp8_quant_rowwise through ctypes with ld_x > K and ld_q > K."""
  from cache_dit_amd import _native
  L = _native.load()
  g = torch.Generator().manual_seed(5)
  M, K, ldx, ldq = 37, 1024, 1536, 1280
  x = torch.randn(M, ldx, generator=g).to(torch.bfloat16)
  xg = x.cuda()
  q = torch.zeros(M, ldq, dtype=torch.uint8, device="cuda")
  s = torch.empty(M, dtype=torch.float32, device="cuda")
  rc = L.cdit_fp8_quant_rowwise(xg.data_ptr(), M, K, ldx, q.data_ptr(), ldq, s.data_ptr(), 0,
                                torch.cuda.current_stream().cuda_stream)
  assert rc == 0, _native.last_error()
  torch.cuda.synchronize()
  q_ref, s_ref = to.quantize_rowwise(x[:, :K], "bf16div")
  assert (q[:, :K].cpu().numpy() == bits_u8(q_ref)).all()
  assert (q[:, K:].cpu().numpy() == 0).all(), "wrote outside the row"
  assert (bits_u32(s) == bits_u32(s_ref.reshape(-1))).all()


def test_c_abi_error_paths():
  from cache_dit_amd import _native
  L = _native.load()
  x = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda")
  q = torch.zeros(4, 64, dtype=torch.uint8, device="cuda")
  s = torch.zeros(4, dtype=torch.float32, device="cuda")
  assert L.cdit_fp8_quant_rowwise(x.data_ptr(), 4, 64, 32, q.data_ptr(), 64, s.data_ptr(), 0,
                                  None) == 1
  assert b"leading dimension" in L.cdit_last_error()
  assert L.cdit_fp8_quant_rowwise(x.data_ptr(), 4, 64, 64, q.data_ptr(), 64, s.data_ptr(), 7,
                                  None) == 1
  assert L.cdit_fp8_quant_rowwise(None, 4, 64, 64, q.data_ptr(), 64, s.data_ptr(), 0, None) == 1
  assert L.cdit_fp8_quant_rowwise(x.data_ptr(), 0, 64, 64, q.data_ptr(), 64, s.data_ptr(), 0,
                                  None) == 0  # empty input is a no-op


def test_full_size_properties_wan_shape():
  """At the largest benchmark activation (Wan: 32760 x 5120) the oracle is too slow
  for every row, so: a random sample of rows is checked bit-exactly against the
  oracle, and the whole tensor through size-independent properties -- every row
  reaches code 0x7E or one below, no NaN code, exact equivariance under scaling by
  a power of two and under negation."""
  from cache_dit_amd import ops
  g = torch.Generator(device="cuda").manual_seed(6)
  x = torch.randn(32760, 5120, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
  for mode in MODES:
    q, s = ops.fp8_rowwise_quant(x, mode)
    qb = q.view(torch.uint8)
    assert int(((qb & 0x7f) == 0x7f).sum()) == 0
    top = (qb & 0x7f).amax(dim=-1)
    assert int((top < 0x7d).sum()) == 0 and int((top > 0x7e).sum()) == 0
    rows = torch.randint(0, x.shape[0], (96, ), generator=torch.Generator().manual_seed(7))
    rows[0], rows[1] = 0, x.shape[0] - 1
    q_ref, s_ref = to.quantize_rowwise(x[rows.cuda()].cpu(), mode)
    assert (bits_u8(q[rows.cuda()]) == bits_u8(q_ref)).all()
    assert (bits_u32(s[rows.cuda()]) == bits_u32(s_ref)).all()
    q2, s2 = ops.fp8_rowwise_quant((x.float() * 2.0**-7).to(torch.bfloat16), mode)
    assert bool((q2.view(torch.uint8) == qb).all()) and bool((s2 == s * 2.0**-7).all())
    q3, s3 = ops.fp8_rowwise_quant(-x, mode)
    assert bool((q3.view(torch.uint8) == (qb ^ 0x80)).all()) and bool((s3 == s).all())


@pytest.mark.parametrize("mode", MODES)
def test_gemm_follows_hint_changes_nothing(mode):
  """CDIT_QUANT_GEMM_FOLLOWS is a cache hint: codes and scales are the same bits."""
  from cache_dit_amd import _native, ops
  g = torch.Generator().manual_seed(21)
  x = (torch.randn(300, 3072, generator=g) * 2).to(torch.bfloat16).cuda()
  m = _native.SCALE_MODE_IDS[mode]
  q0 = torch.empty(300, 3072, dtype=torch.float8_e4m3fn, device="cuda")
  q1 = torch.empty_like(q0)
  s0 = torch.empty(300, dtype=torch.float32, device="cuda")
  s1 = torch.empty_like(s0)
  ops.quant_rowwise_into(x, q0, s0, m)
  ops.quant_rowwise_into(x, q1, s1, m, gemm_follows=True)
  torch.cuda.synchronize()
  assert (bits_u8(q0) == bits_u8(q1)).all() and (bits_u32(s0) == bits_u32(s1)).all()
  q_ref, s_ref = to.quantize_rowwise(x.cpu(), mode)
  assert (bits_u8(q1) == bits_u8(q_ref)).all() and (bits_u32(s1) == bits_u32(s_ref.reshape(-1))).all()
  L = _native.load()  # an unknown mode stays an error with the flag set
  assert L.cdit_fp8_quant_rowwise(x.data_ptr(), 4, 64, 64, q0.data_ptr(), 64, s0.data_ptr(),
                                  0x100 | 5, None) == 1


def _batched_case(shapes, K, mode_id, seed, specials=True):
  """Activations [M_s, K] with outliers; a zero row, rows with scales outside the
  fast-division window and a row that holds a NaN among them."""
  g = torch.Generator(device="cuda").manual_seed(seed)
  xs = []
  for s, M in enumerate(shapes):
    x = (torch.randn(M, K, generator=g, device="cuda") * (1 + s)).to(torch.bfloat16)
    if specials and M >= 5 and K > 0:
      x[0] = 0
      x[1] *= 1e-32
      x[2] *= 1e32
      x[3, K // 2] = float("nan")
      x[4, 0] = 100.0
    xs.append(x)
  return xs


@pytest.mark.parametrize("mode_id", [0, 1])
@pytest.mark.parametrize("shapes,K", [
    ((4096, 512), 3072),          # FLUX double block: image + text stream
    ((4096, 512), 12288),         # ... inputs of ff.net.2
    ((6889, 256), 3072),          # Qwen-Image
    ((5, 1, 77, 300), 1024),      # four activations, a single row among them
    ((7, 0, 9), 640),             # an empty activation is skipped
    ((33, 21), 16384),            # the longest row the register-resident kernel holds
    ((33, 21), 16896),            # beyond it: runs as one launch per activation
    ((12, 40), 200),              # K not a multiple of 8 in bytes of 16: likewise
])
def test_batched_quantizer_equals_one_launch_per_activation(shapes, K, mode_id):
  """cdit_fp8_quant_rowwise_batched against cdit_fp8_quant_rowwise per activation: codes and
  scales bit for bit, nothing written outside (outputs are windows of sentinel buffers)."""
  from cache_dit_amd import ops
  xs = _batched_case(shapes, K, mode_id, seed=sum(shapes) + K)
  items, bufs = [], []
  for x in xs:
    M = x.shape[0]
    qb = torch.full((M + 1, K + 16), 0x55, dtype=torch.uint8, device="cuda")
    sb = torch.full((M + 1, ), -1.0, dtype=torch.float32, device="cuda")
    bufs.append((qb, sb))
    items.append((x, qb[:M, :K].view(torch.float8_e4m3fn), sb[:M]))
  ops.quant_rowwise_batched_into(items, mode_id)
  torch.cuda.synchronize()
  for x, (qb, sb) in zip(xs, bufs):
    M = x.shape[0]
    q1 = torch.empty(M, K, dtype=torch.float8_e4m3fn, device="cuda")
    s1 = torch.empty(M, dtype=torch.float32, device="cuda")
    if M:
      ops.quant_rowwise_into(x, q1, s1, mode_id)
    torch.cuda.synchronize()
    assert torch.equal(qb[:M, :K], q1.view(torch.uint8))
    assert torch.equal(sb[:M].view(torch.int32), s1.view(torch.int32))
    assert (qb[:, K:] == 0x55).all() and (qb[M] == 0x55).all() and sb[M] == -1.0


def test_batched_quantizer_against_the_oracle_and_strided_inputs():
  """Activations that are column windows of wider buffers (ld_x > K), against the CPU oracle."""
  from cache_dit_amd import ops
  K = 1536
  g = torch.Generator().manual_seed(3)
  wide = [torch.randn(M, K + 64, generator=g).to(torch.bfloat16) for M in (130, 70, 19)]
  items = []
  for w in wide:
    x = w.cuda()[:, 8:8 + K]
    items.append((x, torch.empty(x.shape, dtype=torch.float8_e4m3fn, device="cuda"),
                  torch.empty(x.shape[0], dtype=torch.float32, device="cuda")))
  ops.quant_rowwise_batched_into(items, 0)
  torch.cuda.synchronize()
  for w, (_, q, s) in zip(wide, items):
    q_ref, s_ref = to.quantize_rowwise(w[:, 8:8 + K].contiguous(), "bf16div")
    assert int((bits_u8(q) != bits_u8(q_ref)).sum()) == 0
    assert int((bits_u32(s) != bits_u32(s_ref.reshape(-1))).sum()) == 0


def test_batched_quantizer_argument_checks():
  import ctypes
  from cache_dit_amd import _native
  L = _native.load()
  x = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda")
  q = torch.empty(4, 64, dtype=torch.uint8, device="cuda")
  s = torch.empty(4, dtype=torch.float32, device="cuda")
  vp, i64 = ctypes.c_void_p, ctypes.c_int64
  EINVAL = 1  # CDIT_EINVAL

  def call(n, M=4, K=64, ld=64, mode=0, xs=None):
    k = max(n, 1)
    return L.cdit_fp8_quant_rowwise_batched(
        n, (vp * k)(*([x.data_ptr()] * k if xs is None else xs)), (i64 * k)(*[M] * k), K,
        (i64 * k)(*[ld] * k), (vp * k)(*[q.data_ptr()] * k), (i64 * k)(*[64] * k),
        (vp * k)(*[s.data_ptr()] * k), mode, None)

  assert call(1) == 0 and call(2) == 0
  assert call(0) == EINVAL and b"activations" in L.cdit_last_error()
  assert call(5) == EINVAL
  assert call(2, M=-1) == EINVAL and b"bad shape" in L.cdit_last_error()
  assert call(2, ld=32) == EINVAL and b"leading dimension" in L.cdit_last_error()
  assert call(2, mode=7) == EINVAL and b"scale_mode" in L.cdit_last_error()
  assert call(2, xs=[x.data_ptr(), None]) == EINVAL and b"null pointer" in L.cdit_last_error()
  torch.cuda.synchronize()


@pytest.mark.parametrize("mode_id", [0, 1])
@pytest.mark.parametrize("M,K1,K2", [(4608, 3072, 12288), (300, 512, 2048), (77, 8, 8), (33, 4096, 12288),
                                     (5, 1000, 24)])
def test_concatenating_quantizer_equals_the_quantizer_on_the_concatenation(M, K1, K2, mode_id):
  """cdit_fp8_quant_rowwise_cat2 on [x1 | x2] (column windows of wider buffers) against
  cdit_fp8_quant_rowwise on torch.cat: codes and scales bit for bit, nothing written outside;
  rows with a zero block, scales outside the fast-division window and a NaN among them."""
  from cache_dit_amd import ops
  g = torch.Generator(device="cuda").manual_seed(M + K1 + K2)
  w1 = (torch.randn(M, K1 + 16, generator=g, device="cuda") * 3).to(torch.bfloat16)
  w2 = torch.randn(M, K2 + 8, generator=g, device="cuda").to(torch.bfloat16)
  x1, x2 = w1[:, 8:8 + K1], w2[:, :K2]
  if M >= 5:
    x1[0] = 0
    x1[1] *= 1e-32
    x2[1] *= 1e-32
    x2[2] *= 1e32
    x2[3, K2 // 2] = float("nan")
    x1[4] = 0
    x2[4] = 0
  K = K1 + K2
  qb = torch.full((M + 1, K + 16), 0x55, dtype=torch.uint8, device="cuda")
  sb = torch.full((M + 1, ), -1.0, dtype=torch.float32, device="cuda")
  ops.quant_rowwise_cat2_into(x1, x2, qb[:M, :K].view(torch.float8_e4m3fn), sb[:M], mode_id)
  cat = torch.cat([x1, x2], dim=1)
  q1 = torch.empty(M, K, dtype=torch.float8_e4m3fn, device="cuda")
  s1 = torch.empty(M, dtype=torch.float32, device="cuda")
  ops.quant_rowwise_into(cat, q1, s1, mode_id)
  torch.cuda.synchronize()
  assert torch.equal(qb[:M, :K], q1.view(torch.uint8))
  assert torch.equal(sb[:M].view(torch.int32), s1.view(torch.int32))
  assert (qb[:, K:] == 0x55).all() and (qb[M] == 0x55).all() and sb[M] == -1.0


def test_concatenating_quantizer_argument_checks():
  from cache_dit_amd import _native
  L = _native.load()
  x = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda")
  q = torch.empty(4, 128, dtype=torch.uint8, device="cuda")
  s = torch.empty(4, dtype=torch.float32, device="cuda")

  def call(K1=64, K2=64, ld1=64, ld2=64, ldq=128, mode=0, x2=x):
    return L.cdit_fp8_quant_rowwise_cat2(x.data_ptr(), K1, ld1, x2.data_ptr() if x2 is not None else None,
                                         K2, ld2, 4, q.data_ptr(), ldq, s.data_ptr(), mode, None)

  assert call() == 0
  assert call(K1=0) == 1 and b"bad shape" in L.cdit_last_error()
  assert call(ldq=100) == 1 and b"leading dimension" in L.cdit_last_error()
  assert call(mode=5) == 1 and b"scale_mode" in L.cdit_last_error()
  assert call(x2=None) == 1 and b"null pointer" in L.cdit_last_error()
  assert call(K1=60, ld1=64) == 1 and b"multiples of 8" in L.cdit_last_error()
  torch.cuda.synchronize()
