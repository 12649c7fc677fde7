"""The allocation-free Linear entry point (cdit_fp8_linear_w8a8_static: activation codes
and scales in an array inside the library) against cdit_fp8_linear_w8a8 with the
caller's workspaces, through the C ABI. Same kernels, so outputs must be equal bit for
bit; both also go against the CPU oracle."""
import pytest
import torch

from helpers import max_rel_err
from oracle import torch_oracle as to

FP8 = torch.float8_e4m3fn


def _problem(M, K, N, seed, device="cuda"):
  g = torch.Generator().manual_seed(seed)
  x = torch.randn(M, K, generator=g)
  x[:, torch.randperm(K, generator=g)[:3]] *= 20
  x = x.to(torch.bfloat16)
  w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
  b = (torch.randn(N, generator=g) * 0.01).to(torch.bfloat16)
  wq, ws = to.quantize_rowwise(w)
  return x, wq, ws.reshape(-1).contiguous(), b


def _call(fn_name, x, wq, ws, b, epilogue, workspaces):
  from cache_dit_amd import _native
  L = _native.load()
  M, K = x.shape
  N = wq.shape[0]
  out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=x.device)
  stream = torch.cuda.current_stream().cuda_stream
  head = (x.data_ptr(), wq.data_ptr(), ws.data_ptr(), b.data_ptr(), out.data_ptr())
  tail = (M, N, K, x.stride(0), wq.stride(0), out.stride(0), 0, epilogue, _native.DT_BF16, stream)
  if fn_name == "static":
    rc = L.cdit_fp8_linear_w8a8_static(*head, *tail)
  else:
    q, s = workspaces
    rc = L.cdit_fp8_linear_w8a8(*head, q.data_ptr(), s.data_ptr(), *tail)
  assert rc == 0, L.cdit_last_error()
  return out


@pytest.mark.gpu
def test_static_workspace_linear_equals_the_workspace_form_twice_in_a_row():
  """Two calls in a row on one stream, the second with a smaller input (fewer rows,
  shorter rows, and the single-kernel M <= 16 form): what the first call left in the
  library's array must not show in the second result."""
  print("no-alloc entry point: shapes (700,1024,768) then (300,512,520) then (3,256,264)",
        flush=True)
  shapes = [(700, 1024, 768, 0), (300, 512, 520, 1), (3, 256, 264, 0)]
  problems = [tuple(t.cuda() for t in _problem(M, K, N, seed=M)) for M, K, N, _ in shapes]
  outs = []
  for (M, K, N, epi), p in zip(shapes, problems):  # back to back, no synchronisation between
    outs.append(_call("static", *p, epi, None))
  torch.cuda.synchronize()
  for (M, K, N, epi), p, got in zip(shapes, problems, outs):
    q = torch.empty((M, K), dtype=FP8, device="cuda")
    s = torch.empty((M,), dtype=torch.float32, device="cuda")
    want = _call("workspace", *p, epi, (q, s))
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, K, N)
    x, wq, ws, b = (t.cpu() for t in p)
    ref = to.w8a8_linear(x, wq, ws, b, gelu="fused" if epi else None)
    assert max_rel_err(got, ref) <= 1e-2, (M, K, N)


@pytest.mark.gpu
def test_static_workspace_linear_rejects_what_does_not_fit():
  from cache_dit_amd import _native
  L = _native.load()
  one = 256  # never dereferenced: the size check comes first
  K = 4096
  M = _native.STATIC_WS_CODE_BYTES // K + 1
  rc = L.cdit_fp8_linear_w8a8_static(one, one, one, None, one, M, 64, K, K, K, 64, 0, 0, 1, None)
  assert rc == 1 and b"exceeds the built-in workspace" in L.cdit_last_error()
  rc = L.cdit_fp8_linear_w8a8_static(one, one, one, None, one, _native.STATIC_WS_ROWS + 1, 64, 16,
                                     16, 16, 64, 0, 0, 1, None)
  assert rc == 1 and b"exceeds the built-in workspace" in L.cdit_last_error()
  # the largest FLUX / Qwen-Image activation fits, the Wan one does not
  assert 6889 * 12288 <= _native.STATIC_WS_CODE_BYTES < 32760 * 5120
