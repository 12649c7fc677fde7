"""GPU parity of the per-tensor FP8 path (`float8_per_tensor`) through the C ABI:
quantizer codes and scales bit-exact against the oracle, Linear forward within the
GEMM tolerance, hipGraph capture."""
import pytest
import torch
from torch import nn

from oracle import torch_oracle as to

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _dev():
  return torch.device("cuda", 0)


@pytest.mark.parametrize("mode", ["bf16div", "fp32div"])
@pytest.mark.parametrize("M,K", [(1, 16), (7, 200), (64, 3072), (300, 520), (4608, 3072), (33, 15360),
                                 (5, 17)])
def test_quantizer_bit_exact(M, K, mode):
  from cache_dit_amd import ops
  g = torch.Generator().manual_seed(M * 31 + K)
  x = (torch.randn(M, K, generator=g) * (0.1 + (M % 5))).to(torch.bfloat16)
  x[M // 2, K // 3] = 37.0  # one outlier sets the tensor's scale
  q_ref, s_ref = to.quantize_tensorwise(x, mode)
  q, s = ops.fp8_tensorwise_quant(x.to(_dev()), mode)
  torch.cuda.synchronize()
  assert torch.equal(s.cpu(), s_ref)
  assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))


@pytest.mark.parametrize("mode", ["bf16div", "fp32div"])
def test_quantizer_edge_cases(mode):
  from cache_dit_amd import ops
  # all zeros -> scale 1; strided rows; huge and tiny magnitudes (cold division path)
  z = torch.zeros(9, 64, dtype=torch.bfloat16)
  q, s = ops.fp8_tensorwise_quant(z.to(_dev()), mode)
  assert torch.all(s.cpu() == 1.0) and torch.all(q.cpu().view(torch.uint8) == 0)
  for mag in (1e-30, 1e30):
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(12, 256, generator=g) * mag).to(torch.bfloat16)
    q_ref, s_ref = to.quantize_tensorwise(x, mode)
    q, s = ops.fp8_tensorwise_quant(x.to(_dev()), mode)
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))
  base = torch.randn(20, 512, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16)
  xs = base.to(_dev())[:, :384]  # row stride 512, K 384
  q_ref, s_ref = to.quantize_tensorwise(base[:, :384].contiguous(), mode)
  q, s = ops.fp8_tensorwise_quant(xs, mode)
  assert torch.equal(s.cpu(), s_ref) and torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))


def test_repeated_calls_do_not_keep_the_previous_amax():
  from cache_dit_amd import ops
  big = torch.full((8, 64), 100.0, dtype=torch.bfloat16, device=_dev())
  small = torch.full((8, 64), 0.5, dtype=torch.bfloat16, device=_dev())
  _, s1 = ops.fp8_tensorwise_quant(big)
  _, s2 = ops.fp8_tensorwise_quant(small)
  assert torch.all(s1.cpu() == to.choose_scale_tensorwise(big.cpu()))
  assert torch.all(s2.cpu() == to.choose_scale_tensorwise(small.cpu()))


def _ref_linear(x, lin_w, bias, mode="bf16div"):
  xq, xs = to.quantize_tensorwise(x, mode)
  wq, ws = to.quantize_tensorwise(lin_w, mode)
  return to.scaled_mm_rowwise(xq, xs, wq, ws, bias)


@pytest.mark.parametrize("M,K,N", [(1, 256, 512), (77, 384, 264 + 8), (4096, 3072, 3072)])
def test_linear_forward_matches_oracle(M, K, N):
  import cache_dit_amd
  N = (N // 16) * 16
  torch.manual_seed(M + K)
  lin = nn.Linear(K, N, bias=True).to(torch.bfloat16)
  x = torch.randn(M, K).to(torch.bfloat16)
  ref = _ref_linear(x, lin.weight.detach(), lin.bias.detach()).float()
  m = nn.Sequential(lin).to(_dev())
  cache_dit_amd.quantize(m, cache_dit_amd.QuantizeConfig(quant_type="float8_per_tensor",
                                                         regional_quantize=False))
  assert type(m[0]).__name__ == "Fp8DynamicLinearPerTensor"
  assert torch.all(m[0].weight_scale == m[0].weight_scale[0])
  out = m(x.to(_dev())).float().cpu()
  err = (out - ref).abs().max() / ref.abs().max()
  assert err <= 1e-2, err


def test_forward_under_hip_graph_capture():
  import cache_dit_amd
  torch.manual_seed(0)
  m = nn.Sequential(nn.Linear(512, 1024).to(torch.bfloat16)).to(_dev())
  cache_dit_amd.quantize(m, cache_dit_amd.QuantizeConfig(quant_type="float8_per_tensor",
                                                         regional_quantize=False))
  x = torch.randn(96, 512, device=_dev()).to(torch.bfloat16)
  eager = m(x).clone()
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side):
    m(x)
  torch.cuda.current_stream().wait_stream(side)
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.graph(graph):
    y = m(x)
  for scale in (1.0, 3.0, 0.25):  # the amax scratch must be re-zeroed on every replay
    x.copy_((torch.randn(96, 512, device=_dev()) * scale).to(torch.bfloat16))
    expect = m(x).clone()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(y, expect)
  assert eager.shape == y.shape
