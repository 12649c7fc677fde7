"""Sibling GEMMs on one activation as one launch (cdit_fp8_gemm_rowwise_grouped): equal,
bit for bit, to one launch per member, and to the CPU oracle on exact small-integer
data; tails, a null bias, per-member epilogues, outputs that are column slices of one
buffer, every tile shape."""
import pytest
import torch

from helpers import max_rel_err
from oracle import torch_oracle as to

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


@pytest.fixture(autouse=True)
def _auto_variant():
  from cache_dit_amd import _native
  _native.set_gemm_variant(-1)
  yield
  _native.set_gemm_variant(-1)


def _members(M, K, Ns, seed, integer=False, no_bias=()):
  g = torch.Generator(device="cuda").manual_seed(seed)
  if integer:
    a = torch.randint(-3, 4, (M, K), generator=g, device="cuda").float().to(FP8)
    a_s = torch.full((M,), 0.5, device="cuda")
  else:
    a = torch.randn(M, K, generator=g, device="cuda").to(FP8)
    a_s = torch.rand(M, generator=g, device="cuda") * 0.1 + 0.01
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
    bs.append(None if i in no_bias else b)
  return a, a_s, ws, wss, bs


def _separate(a, a_s, ws, wss, bs, epis):
  from cache_dit_amd import ops
  outs = []
  for w, s, b, e in zip(ws, wss, bs, epis):
    o = torch.empty((a.shape[0], w.shape[0]), dtype=torch.bfloat16, device="cuda")
    ops.gemm_rowwise_into(a, a_s, w, s, b, o, e)
    outs.append(o)
  return outs


def _grouped(a, a_s, ws, wss, bs, epis, outs=None):
  from cache_dit_amd import ops
  if outs is None:
    outs = [torch.full((a.shape[0], w.shape[0]), float("nan"), dtype=torch.bfloat16, device="cuda")
            for w in ws]
  ops.gemm_rowwise_grouped_into(a, a_s, ws, wss, bs, outs, epis)
  torch.cuda.synchronize()
  return outs


@pytest.mark.parametrize("M,K,Ns,epis", [
    (4608, 3072, [12288, 3072, 3072, 3072], [1, 0, 0, 0]),  # FLUX single block: proj_mlp + q/k/v
    (4096, 3072, [3072, 3072, 3072], [0, 0, 0]),  # FLUX double block q/k/v
    (512, 3072, [3072, 3072, 3072], [0, 0, 0]),  # text stream
    (6889, 3072, [3072, 3072, 3072], [0, 0, 0]),  # Qwen-Image q/k/v
    (300, 512, [520, 264, 72], [0, 1, 0]),  # ragged everything
    (1000, 1024, [192, 2048], [1, 1]),
])
def test_grouped_equals_separate_launches(M, K, Ns, epis):
  args = _members(M, K, Ns, seed=M + K, no_bias=(1,))
  want = _separate(*args, epis)
  got = _grouped(*args, epis)
  for p, (g, w) in enumerate(zip(got, want)):
    assert torch.equal(g.view(torch.int16), w.view(torch.int16)), f"member {p}"


@pytest.mark.parametrize("variant", [12, 14, 15, 16, 17, 18])
def test_every_tile_shape_exact_integers_against_the_oracle(variant):
  """Small-integer codes and power-of-two scales: every product and sum is exact, so the
  result must equal the oracle's bit for bit, whatever the tile shape; more tiles than
  CUs, tails in M and in every member's N, outputs as column slices of one buffer."""
  from cache_dit_amd import _native
  M, K, Ns = 2100, 640, [1096, 520, 3080]
  a, a_s, ws, wss, bs = _members(M, K, Ns, seed=variant, integer=True, no_bias=(2,))
  epis = [0, 0, 0]
  whole = torch.full((M, sum(Ns) + 8), float("nan"), dtype=torch.bfloat16, device="cuda")
  outs, c = [], 0
  for N in Ns:
    outs.append(whole[:, c:c + N])
    c += N
  _native.set_gemm_variant(variant)
  _grouped(a, a_s, ws, wss, bs, epis, outs)
  _native.set_gemm_variant(-1)
  assert torch.isnan(whole[:, c:]).all()  # nothing written past the last member
  for p in range(3):
    ref = to.scaled_mm_rowwise(a.cpu(), a_s.cpu(), ws[p].cpu(), wss[p].cpu(),
                               None if bs[p] is None else bs[p].cpu())
    assert torch.equal(outs[p].cpu().view(torch.int16), ref.view(torch.int16)), f"member {p}"


def test_groups_the_grouped_kernel_does_not_take_still_run():
  """A single member, M <= 16 and a misaligned scale run member by member."""
  for M, Ns in ((7, [264, 520]), (300, [520])):
    args = _members(M, 512, Ns, seed=M)
    epis = [0] * len(Ns)
    for g, w in zip(_grouped(*args, epis), _separate(*args, epis)):
      assert torch.equal(g.view(torch.int16), w.view(torch.int16))
  a, a_s, ws, wss, bs = _members(300, 512, [520, 264], seed=3)
  pad = torch.cat([torch.zeros(1, device="cuda"), wss[1]])
  wss[1] = pad[1:]
  assert wss[1].data_ptr() % 16 != 0
  for g, w in zip(_grouped(a, a_s, ws, wss, bs, [0, 0]), _separate(a, a_s, ws, wss, bs, [0, 0])):
    assert torch.equal(g.view(torch.int16), w.view(torch.int16))
  from cache_dit_amd import _native
  L = _native.load()
  assert L.cdit_fp8_gemm_rowwise_grouped(None, None, 4, 64, 64, 5, None, None, None, None, None, 64,
                                         None, None, None) == 1
  assert b"a group holds" in L.cdit_last_error()


def test_grouped_random_data_against_the_oracle_sampled_rows():
  M, K, Ns = 4608, 3072, [12288, 3072, 3072, 3072]
  a, a_s, ws, wss, bs = _members(M, K, Ns, seed=9)
  got = _grouped(a, a_s, ws, wss, bs, [1, 0, 0, 0])
  rows = torch.cat([torch.arange(0, M, 211), torch.arange(M - 2, M)]).cuda()
  for p in range(4):
    ref = to.scaled_mm_rowwise(a[rows].cpu(), a_s[rows].cpu(), ws[p].cpu(), wss[p].cpu(), bs[p].cpu(),
                               gelu="fused" if p == 0 else None)
    assert max_rel_err(got[p][rows], ref) <= 1e-2, p
