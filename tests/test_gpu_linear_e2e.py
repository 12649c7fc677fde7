"""GPU end-to-end: quantize() on real modules, golden vectors, and the single-step
transformer output against the same model run with the oracle's ops."""
import copy
import logging
import os

import numpy as np
import pytest
import torch
from torch import nn

from helpers import bits_u8, cosine, max_rel_err
from oracle import torch_oracle as to

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
logging.getLogger("CACHE_DIT_AMD").setLevel(logging.WARNING)


def _bf(a):
  return torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)


def test_golden_vectors_on_gpu():
  from cache_dit_amd import ops
  z = np.load(os.path.join(GOLD, "quant_vectors.npz"))
  x = _bf(z["x"]).cuda()
  for mode in ("bf16div", "fp32div"):
    q, s = ops.fp8_rowwise_quant(x, mode)
    assert (bits_u8(q) == z[f"q_{mode}"]).all()
    assert (s.reshape(-1).cpu().numpy().view(np.uint32) == z[f"s_{mode}"].view(np.uint32)).all()
  z = np.load(os.path.join(GOLD, "linear_vectors.npz"))
  x, b = _bf(z["x"]).cuda(), _bf(z["bias"]).cuda()
  wq = torch.from_numpy(z["wq"]).view(torch.float8_e4m3fn).cuda()
  ws = torch.from_numpy(z["ws"]).cuda()
  xq, xs = ops.fp8_rowwise_quant(x)
  assert (bits_u8(xq) == z["xq"]).all() and (xs.reshape(-1).cpu().numpy() == z["xs"]).all()
  y = ops.float8_inference_scaled_mm(xq, xs, wq.t(), ws.reshape(1, -1), torch.bfloat16, bias=b)
  assert max_rel_err(y, _bf(z["y_w8a8"])) <= 1e-2
  yg = ops.float8_inference_scaled_mm(xq, xs, wq.t(), ws.reshape(1, -1), torch.bfloat16, bias=b,
                                      epilogue=1)
  assert max_rel_err(yg, _bf(z["y_w8a8_gelu_fused"])) <= 1e-2
  assert max_rel_err(yg, _bf(z["y_w8a8_gelu_unfused"])) <= 1e-2
  yw = ops.w8a16_mm(x, wq.t(), ws, b)
  assert max_rel_err(yw, _bf(z["y_w8a16_ref"])) <= 1e-2
  assert max_rel_err(yw, _bf(z["y_w8a16_fused"])) <= 1e-2


class _Blk(nn.Module):

  def __init__(self, d):
    super().__init__()
    self.to_q = nn.Linear(d, d)
    self.proj_mlp = nn.Linear(d, 4 * d)
    self.act_mlp = nn.GELU(approximate="tanh")
    self.proj_out = nn.Linear(4 * d, d, bias=False)
    self.mod = nn.Linear(d, d)

  def forward(self, x):
    return x + self.proj_out(self.act_mlp(self.proj_mlp(self.to_q(x) + self.mod(x))))


class _Net(nn.Module):
  _repeated_blocks = ["_Blk"]

  def __init__(self, d=256):
    super().__init__()
    self.blocks = nn.ModuleList([_Blk(d), _Blk(d)])

  def forward(self, x):
    for b in self.blocks:
      x = b(x)
    return x


@pytest.mark.parametrize("quant_type", ["float8_per_row", "float8_weight_only"])
@pytest.mark.parametrize("where", ["gpu", "cpu_then_gpu"])
def test_quantize_module_in_place(quant_type, where):
  """Weights quantized on the GPU, or on the CPU before `.to(device)` as the
  reference's CLI flow does: same codes either way, equal to the oracle's."""
  import cache_dit_amd as cache_dit
  from cache_dit_amd.nn import Fp8DynamicLinear, Fp8WeightOnlyLinear
  torch.manual_seed(0)
  net = _Net().to(torch.bfloat16)
  ref = copy.deepcopy(net)
  if where == "gpu":
    net = net.cuda()
  out = cache_dit.quantize(net, cache_dit.QuantizeConfig(quant_type=quant_type))
  assert out is net and net._is_quantized
  net = net.cuda()
  cls = Fp8DynamicLinear if quant_type == "float8_per_row" else Fp8WeightOnlyLinear
  for blk, rblk in zip(net.blocks, ref.blocks):
    assert type(blk.mod) is nn.Linear and blk.mod.weight.dtype == torch.bfloat16  # excluded
    for name in ("to_q", "proj_mlp", "proj_out"):
      lin, rlin = getattr(blk, name), getattr(rblk, name)
      assert isinstance(lin, cls) and isinstance(lin, nn.Linear) and lin._is_inner_quantized
      wq, ws = to.quantize_rowwise(rlin.weight.detach())
      assert lin.weight.dtype == torch.float8_e4m3fn and not lin.weight.requires_grad
      assert (bits_u8(lin.weight) == bits_u8(wq)).all()
      assert torch.equal(lin.weight_scale.cpu(), ws)
  x = torch.randn(2, 50, 256, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
  y = net(x.cuda())
  assert y.shape == x.shape and y.dtype == torch.bfloat16
  # the same network with the oracle's ops on the CPU
  f = to.w8a8_linear if quant_type == "float8_per_row" else to.w8a16_linear
  h = x
  for rblk in ref.blocks:
    q = {n: to.quantize_rowwise(getattr(rblk, n).weight.detach()) for n in ("to_q", "proj_mlp",
                                                                           "proj_out")}
    t = f(h, *q["to_q"], rblk.to_q.bias.detach()) + rblk.mod(h)
    t = rblk.act_mlp(f(t, *q["proj_mlp"], rblk.proj_mlp.bias.detach()))
    h = h + f(t, *q["proj_out"], None)
  assert cosine(y, h) >= 0.9999 and max_rel_err(y, h) <= 2e-2
  assert "quant_type=" + quant_type in repr(net.blocks[0].to_q)
  sd = net.state_dict()
  assert sd["blocks.0.to_q.weight"].dtype == torch.float8_e4m3fn
  assert sd["blocks.0.to_q.weight_scale"].shape == (256, 1)


def test_input_checks_of_the_quantized_linear():
  import cache_dit_amd as cache_dit
  net = _Net().to(torch.bfloat16).cuda()
  cache_dit.quantize(net, cache_dit.QuantizeConfig())
  lin = net.blocks[0].to_q
  with pytest.raises(ValueError, match="bfloat16"):
    lin(torch.zeros(4, 256, device="cuda"))
  with pytest.raises(RuntimeError, match="no CPU path"):
    lin(torch.zeros(4, 256, dtype=torch.bfloat16))
  assert lin(torch.zeros(0, 256, dtype=torch.bfloat16, device="cuda")).shape == (0, 256)
  y = lin(torch.zeros(3, 5, 256, dtype=torch.bfloat16, device="cuda"))  # zero rows: scale 1
  assert torch.equal(y, lin.bias.expand(3, 5, 256))
  xs = torch.randn(8, 512, device="cuda").to(torch.bfloat16)[:, ::2]  # non-contiguous input
  assert torch.equal(lin(xs), lin(xs.contiguous()))


def _oracle_ops_forward(model, inputs, device):
  """Runs `model` with every quantized Linear replaced by the oracle's w8a8
  arithmetic written in plain torch ops on `device`. On a GPU device this comparator is the
  oracle's op sequence executed by PyTorch's GPU kernels, NOT the CPU oracle bit for bit (GPU
  eager evaluates `bf16 / 448.0` as a multiply by the reciprocal, its matmul sums in another
  order): good for the cosine bar of the full-size step tests, which is all they use it
  for; bit-exact parity is checked against the CPU oracle at sizes it finishes in seconds."""
  from cache_dit_amd.nn import _Fp8LinearBase

  def fwd(self, x):
    return to.w8a8_linear(x, self.weight, self.weight_scale, self.bias,
                          gelu="fused" if self.epilogue else None)

  saved = _Fp8LinearBase.forward
  from cache_dit_amd import nn as cnn
  old = cnn.Fp8DynamicLinear.forward
  cnn.Fp8DynamicLinear.forward = fwd
  try:
    with torch.inference_mode():
      return model(**inputs)
  finally:
    cnn.Fp8DynamicLinear.forward = old


def test_small_flux_like_step_cosine_vs_oracle_ops():
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  torch.manual_seed(0)
  kw = dict(dim=512, heads=4, mlp=2048, n_double=2, n_single=3, in_channels=64, text_dim=256,
            pooled_dim=128)
  model = ds.FluxLikeTransformer(**kw).to(torch.bfloat16).cuda()
  bf16_model = copy.deepcopy(model)
  cache_dit.quantize(model, cache_dit.QuantizeConfig())
  inputs = ds.flux_like_inputs("cuda", n_img=320, n_txt=64, in_channels=64, text_dim=256,
                               pooled_dim=128)
  with torch.inference_mode():
    y = model(**inputs)
    y_bf16 = bf16_model(**inputs)
  y_ref = _oracle_ops_forward(model, inputs, "cuda")
  assert torch.isfinite(y.float()).all()
  assert cosine(y, y_ref) >= 0.999, cosine(y, y_ref)
  assert cosine(y, y_bf16) >= 0.99, cosine(y, y_bf16)
  # fusing GELU into the epilogue keeps the output inside the same bar
  n = ds.fuse_gelu_epilogues(model)
  assert n == 2 * 2 + 3
  with torch.inference_mode():
    y_fused = model(**inputs)
  assert cosine(y_fused, y_ref) >= 0.999


def test_shared_activation_quant_is_bit_identical_and_saves_launches():
  import cache_dit_amd as cache_dit
  from cache_dit_amd import ops
  from cache_dit_amd.testing import dit_shapes as ds
  torch.manual_seed(0)
  kw = dict(dim=512, heads=4, mlp=2048, n_double=2, n_single=3, in_channels=64, text_dim=256,
            pooled_dim=128)
  model = ds.FluxLikeTransformer(**kw).to(torch.bfloat16).cuda()
  cache_dit.quantize(model, cache_dit.QuantizeConfig())
  inputs = ds.flux_like_inputs("cuda", n_img=320, n_txt=64, in_channels=64, text_dim=256,
                               pooled_dim=128)
  with torch.inference_mode():
    y0 = model(**inputs)
  n = cache_dit.share_activation_quant_(model)
  assert n == 2 * 14 + 3 * 6
  ops.quant_launches = 0
  with torch.no_grad():
    y1 = model(**inputs)
    y2 = model(**inputs)
  assert torch.equal(y0, y1) and torch.equal(y0, y2)
  # per double block: q/k/v share (img), add_q/k/v share (txt), the other 8 do not: 10 of 14;
  # per single block: proj_mlp + q/k/v share, proj_out and norm.linear do not: 3 of 6
  assert ops.quant_launches == 2 * (2 * 10 + 3 * 3), ops.quant_launches
  ops.quant_launches = 0
  with torch.inference_mode():  # no version counters there: nothing is shared
    y3 = model(**inputs)
  assert torch.equal(y0, y3) and ops.quant_launches == 2 * 14 + 3 * 6
  # an in-place change of the shared input must not reuse stale codes
  lin = model.single_transformer_blocks[0].attn.to_q
  x = torch.randn(64, 512, device="cuda").to(torch.bfloat16)
  with torch.no_grad():
    a = lin(x)
    x.mul_(2.0)
    b = lin(x)
  cache_dit.share_activation_quant_(model, False)
  assert torch.equal(b, lin(x)) and not torch.equal(a, b)


def test_linear_forward_under_hip_graph_capture():
  """A captured forward replays correctly with new input data (no allocation-order or
  stream assumptions in the launch path); every replay is checked against eager, with
  eager work and synchronisation between the replays."""
  import cache_dit_amd as cache_dit
  torch.manual_seed(0)
  net = _Net().to(torch.bfloat16).cuda()
  cache_dit.quantize(net, cache_dit.QuantizeConfig())
  static_x = torch.randn(3, 70, 256, device="cuda").to(torch.bfloat16)
  with torch.no_grad():
    net(static_x)  # warm-up outside capture (sets kernel attributes)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
      net(static_x)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
      static_y = net(static_x)
    for seed in range(4):
      new_x = torch.randn(3, 70, 256, device="cuda",
                          generator=torch.Generator(device="cuda").manual_seed(seed)).to(torch.bfloat16)
      expect = net(new_x)  # eager, also between replays
      torch.cuda.synchronize()
      static_x.copy_(new_x)
      graph.replay()
      torch.cuda.synchronize()
      assert torch.equal(static_y, expect), f"replay {seed} differs from eager"


def test_full_flux_shaped_step_cosine():
  """benchmark config 2 at full size (19 + 38 blocks, 4096 + 512 tokens): the HIP
  path against the oracle's arithmetic in torch ops on the same GPU, and against
  the unquantized bf16 model."""
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  torch.manual_seed(0)
  with torch.device("cuda"):
    model = ds.FluxLikeTransformer().to(torch.bfloat16)
  inputs = ds.flux_like_inputs("cuda")
  with torch.inference_mode():
    y_bf16 = model(**inputs)
  cache_dit.quantize(model, cache_dit.QuantizeConfig())
  total, quantized = ds.count_linears(model)
  assert quantized == 494
  with torch.inference_mode():
    y = model(**inputs)
  y_ref = _oracle_ops_forward(model, inputs, "cuda")
  c_ref, c_bf16 = cosine(y, y_ref), cosine(y, y_bf16)
  print(f"full FLUX-shaped step: cosine vs oracle ops {c_ref:.6f}, vs bf16 {c_bf16:.6f}")
  assert torch.isfinite(y.float()).all()
  assert c_ref >= 0.999, c_ref
  assert c_bf16 >= 0.99, c_bf16
  # The stage patch on this unmodified model at full size: the launches of a forward are
  # those of the step the benchmark times as its headline (per step 152 quantizer launches,
  # 114 batched GEMM calls -- 171 launches where the tile cost model splits a stage --, 38
  # proj_out and 76 M = 1 Linears), and the output keeps its bits.
  from test_gpu_patch_functors import _Launches
  with torch.no_grad():
    y_plain = model(**inputs)
    cache_dit.apply_stage_patch(model)
    with _Launches() as staged:
      y_staged = model(**inputs)
    cache_dit.remove_stage_patch(model)
  assert torch.equal(y_staged, y_plain)
  assert staged.n["batched"] == 19 * 4 + 38 and staged.n["single"] == 19 * 2 + 38 * 2
  assert staged.n["shared_quant"] + staged.n["cat2"] == 152 and staged.n["cat2"] == 38


def _full_size_step(model_cls, inputs_fn, n_quantized, n_skipped):
  """One full-size step of a benchmark model: the HIP path against the oracle's
  arithmetic in torch ops on the same GPU, and against the unquantized bf16 model."""
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  torch.manual_seed(0)
  with torch.device("cuda"):
    model = model_cls().to(torch.bfloat16)
  inputs = inputs_fn("cuda")
  with torch.inference_mode():
    y_bf16 = model(**inputs)
  cache_dit.quantize(model, cache_dit.QuantizeConfig(verbose=True))
  ctx = model._quantize_context
  total, quantized = ds.count_linears(model)
  assert quantized == n_quantized == ctx.quantized_map["float8_per_row"]
  assert sum(len(v) for v in ctx.skipped_map.values()) == n_skipped
  with torch.inference_mode():
    y = model(**inputs)
  y_ref = _oracle_ops_forward(model, inputs, "cuda")
  c_ref, c_bf16 = cosine(y, y_ref), cosine(y, y_bf16)
  print(f"{model_cls.__name__} full-size step: cosine vs oracle ops {c_ref:.6f}, vs bf16 "
        f"{c_bf16:.6f}", flush=True)
  assert torch.isfinite(y.float()).all()
  assert c_ref >= 0.999, c_ref
  assert c_bf16 >= 0.99, c_bf16
  # with GELU-tanh folded into the producing Linear and shared activation quantization,
  # as the benchmark runs the model
  ds.fuse_gelu_epilogues(model)
  cache_dit.share_activation_quant_(model)
  with torch.no_grad():
    y_fast = model(**inputs)
  cache_dit.share_activation_quant_(model, False)
  assert cosine(y_fast, y_ref) >= 0.999
  return model


def test_full_qwen_image_shaped_step_cosine():
  """benchmark config 4 at full size: 60 blocks, 6889 image + 256 text tokens, hidden
  3072, MLP 12288; 12 quantized Linears per block, `img_mod.1` / `txt_mod.1` skipped by
  the default "mod" pattern (layer inventory:
  src/cache_dit/distributed/transformers/qwen_image.py:119-134)."""
  from cache_dit_amd.testing import dit_shapes as ds
  model = _full_size_step(ds.QwenImageLikeTransformer, ds.qwen_image_like_inputs, 720, 120)
  blk = model.transformer_blocks[0]
  assert type(blk.img_mod[1]) is nn.Linear and blk.img_mod[1].weight.dtype == torch.bfloat16


def test_full_wan_shaped_step_cosine():
  """benchmark config 5 at full size: 40 layers, 32760 video + 512 text tokens, hidden
  5120, FFN 13824; 10 quantized Linears per block (layer inventory:
  src/cache_dit/distributed/transformers/wan.py:284-293)."""
  from cache_dit_amd.testing import dit_shapes as ds
  _full_size_step(ds.WanLikeTransformer, ds.wan_like_inputs, 400, 0)


class _OneLinear(nn.Module):

  def __init__(self, k, n):
    super().__init__()
    self.proj = nn.Linear(k, n)

  def forward(self, x):
    return self.proj(x)


@pytest.mark.parametrize("quant_type", ["float8_per_row", "float8_per_tensor", "float8_weight_only"])
@pytest.mark.parametrize("M,K,N", [(4, 64, 32), (512, 3072, 3072)])
def test_torch_compile_fullgraph_equals_eager(quant_type, M, K, N):
  """torch.compile(fullgraph=True) of a quantized Linear: Dynamo traces the module
  forward into the one opaque cdit op (fake implementation), Inductor calls it; the
  output equals eager bit for bit. Shapes: the reference's opaque-op test W[32,64] /
  x[4,64] (tests/kernels/test_opaque_scaled_mm.py:46-94) and its CUDA-graph partition
  test M=512, K=N=3072; like the former, also with Inductor's own graph capture."""
  import cache_dit_amd as cache_dit
  torch.manual_seed(0)
  net = _OneLinear(K, N).to(torch.bfloat16).cuda()
  cache_dit.quantize(net, cache_dit.QuantizeConfig(quant_type=quant_type, exclude_layers=[]))
  assert net.proj._is_inner_quantized
  x = torch.randn(M, K, device="cuda").to(torch.bfloat16)
  with torch.no_grad():
    eager = net(x)
    torch._dynamo.reset()
    compiled = torch.compile(net, fullgraph=True)
    assert torch.equal(compiled(x), eager)
    x3 = torch.randn(2, M, K, device="cuda").to(torch.bfloat16)  # another rank: recompiles
    assert torch.equal(compiled(x3), net(x3))
    graphed = torch.compile(net, fullgraph=True, options={"triton.cudagraphs": True})
    graphed(x)
    out = graphed(x)
    torch.cuda.synchronize()
    assert torch.equal(out, eager)
  torch._dynamo.reset()


def test_merged_stream_attention_projections_under_graph_capture():
  """The reference's merged-stream case at its own size
  (tests/kernels/test_rowwise_cudagraph_partition.py:82-128: B=1, 12288 image + 512 text
  tokens, 24 heads of 128): one set of row-wise quantized q/k/v Linears applied to both
  streams, the results merged text-first, SDPA on top -- replayed from a hipGraph and run
  under torch.compile(options={"triton.cudagraphs": True}); both must reproduce eager."""
  import torch.nn.functional as F
  from cache_dit_amd import nn as cnn
  B, SI, ST, H, D = 1, 12288, 512, 24, 128
  S, C = SI + ST, H * D
  torch.manual_seed(0)
  lins = [nn.Linear(C, C, bias=False, dtype=torch.bfloat16).cuda() for _ in range(3)]
  for lin in lins:
    cnn.convert_linear_(lin, "float8_per_row")
  qw, kw, vw = lins
  g = torch.Generator(device="cuda").manual_seed(1)
  x_img = torch.randn(B, SI, C, device="cuda", generator=g).to(torch.bfloat16)
  x_txt = torch.randn(B, ST, C, device="cuda", generator=g).to(torch.bfloat16)

  def fn(img, txt):
    merged = []
    for lin in (qw, kw, vw):
      t = torch.empty((B, S, H, D), device=img.device, dtype=img.dtype)
      t[:, :ST] = lin(txt).view(B, ST, H, D)
      t[:, ST:] = lin(img).view(B, SI, H, D)
      merged.append(t)
    q, k, v = (t.permute(0, 2, 1, 3).contiguous() for t in merged)
    return F.scaled_dot_product_attention(q, k, v), merged[0]

  with torch.no_grad():
    out, q_merged = fn(x_img, x_txt)
    torch.cuda.synchronize()
    assert out.shape == (B, H, S, D) and torch.isfinite(out.float()).all()
    # hipGraph capture and replays, also on other data in the static inputs
    s_img, s_txt = x_img.clone(), x_txt.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
      fn(s_img, s_txt)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
      g_out, g_q = fn(s_img, s_txt)
    other_img = torch.randn(B, SI, C, device="cuda", generator=g).to(torch.bfloat16)
    for img in (other_img, x_img, other_img):
      want_out, want_q = fn(img, x_txt)
      s_img.copy_(img)
      graph.replay()
      torch.cuda.synchronize()
      assert torch.equal(g_q, want_q) and torch.equal(g_out, want_out)
    del graph
    # the reference's own form: compiled, with Inductor's graph capture around the opaque ops
    torch._dynamo.reset()
    try:
      compiled = torch.compile(fn, options={"triton.cudagraphs": True})
      c1 = compiled(x_img, x_txt)
      c_out, c_q = c1[0].clone(), c1[1].clone()
      c2 = compiled(x_img, x_txt)
      torch.cuda.synchronize()
    except Exception as e:  # no Inductor back end on the box
      torch._dynamo.reset()
      pytest.skip(f"torch.compile unavailable: {str(e)[:80]}")
    assert torch.equal(c_q, q_merged) and torch.equal(c2[1], q_merged)
    assert cosine(c_out, out) >= 0.99999 and cosine(c2[0], out) >= 0.99999
  torch._dynamo.reset()


def test_torch_compile_of_a_block_with_glue_ops():
  """A block with element-wise glue around three quantized Linears (one with GELU-tanh
  folded into its epilogue) compiles without graph breaks: Dynamo records three cdit
  nodes."""
  import cache_dit_amd as cache_dit
  from cache_dit_amd.nn import fuse_gelu_tanh_
  torch.manual_seed(0)
  net = _Net().to(torch.bfloat16).cuda()
  cache_dit.quantize(net, cache_dit.QuantizeConfig())
  for blk in net.blocks:
    fuse_gelu_tanh_(blk.proj_mlp, blk.act_mlp)
  x = torch.randn(3, 70, 256, device="cuda").to(torch.bfloat16)
  seen = []

  def backend(gm, example_inputs):
    seen.extend(str(n.target) for n in gm.graph.nodes if n.op == "call_function")
    return gm.forward

  with torch.no_grad():
    eager = net(x)
    torch._dynamo.reset()
    out = torch.compile(net, fullgraph=True, backend=backend)(x)
  torch._dynamo.reset()
  assert torch.equal(out, eager)
  assert sum(t.startswith("cdit.linear_w8a8") for t in seen) == 2 * 3, seen


def test_shared_activation_quant_across_two_graph_captures():
  """Codes cached inside one graph capture must not be handed to another capture: two
  graphs of a share-enabled model, captured one after the other from the same static
  input, both replay correctly with new data."""
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  torch.manual_seed(0)
  kw = dict(dim=256, heads=2, mlp=512, n_double=1, n_single=1, in_channels=64, text_dim=128,
            pooled_dim=64)
  model = ds.FluxLikeTransformer(**kw).to(torch.bfloat16).cuda()
  cache_dit.quantize(model, cache_dit.QuantizeConfig())
  cache_dit.share_activation_quant_(model)
  lin_q, lin_k = model.single_transformer_blocks[0].attn.to_q, model.single_transformer_blocks[0].attn.to_k
  static_x = torch.randn(96, 256, device="cuda").to(torch.bfloat16)

  def pair():
    return lin_q(static_x), lin_k(static_x)

  with torch.no_grad():
    pair()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
      pair()
    torch.cuda.current_stream().wait_stream(side)
    graphs = []
    for _ in range(2):  # same capture stream, same static input, unchanged _version
      g = torch.cuda.CUDAGraph()
      with torch.cuda.graph(g):
        outs = pair()
      graphs.append((g, outs))
    for seed in range(3):
      new_x = torch.randn(96, 256, device="cuda",
                          generator=torch.Generator(device="cuda").manual_seed(seed)).to(torch.bfloat16)
      cache_dit.share_activation_quant_(model, False)
      want = (lin_q(new_x), lin_k(new_x))
      cache_dit.share_activation_quant_(model)
      torch.cuda.synchronize()
      static_x.copy_(new_x)
      for g, outs in reversed(graphs):  # the second graph must carry its own quantizer node
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(outs[0], want[0]) and torch.equal(outs[1], want[1]), seed
        outs[0].zero_(), outs[1].zero_()
  cache_dit.share_activation_quant_(model, False)


class _PlanBlk(nn.Module):

  def __init__(self, d):
    super().__init__()
    self.to_q, self.to_k, self.to_v = nn.Linear(d, d), nn.Linear(d, d), nn.Linear(d, d)
    self.to_out = nn.ModuleList([nn.Linear(d, d), nn.Dropout(0.0)])
    self.ff_in, self.ff_out = nn.Linear(d, 2 * d), nn.Linear(2 * d, d, bias=False)


class _PlanNet(nn.Module):
  _repeated_blocks = ["_PlanBlk"]

  def __init__(self, d=128):
    super().__init__()
    self.blocks = nn.ModuleList([_PlanBlk(d), _PlanBlk(d)])


def _oracle_linear(kind, x, weight, bias):
  """x, weight bf16 on the CPU -> the oracle's output for a Linear of quant type `kind`."""
  if kind == "float8_per_row":
    return to.w8a8_linear(x, *to.quantize_rowwise(weight), bias)
  if kind == "float8_weight_only":
    return to.w8a16_linear(x, *to.quantize_rowwise(weight), bias)
  assert kind == "float8_per_tensor"
  wq, ws = to.quantize_tensorwise(weight)
  xq, xs = to.quantize_tensorwise(x.reshape(-1, x.shape[-1]))
  return to.scaled_mm_rowwise(xq, xs, wq, ws, bias).reshape(*x.shape[:-1], weight.shape[0])


@pytest.mark.parametrize("with_plan", [True, False])
def test_mixed_precision_plan_and_fallback_on_device(with_plan):
  """A precision plan mixing per-row, per-tensor and weight-only Linears, with a
  row-parallel layer that falls back to per-tensor (merged into the plan when there is
  one, taken by the second pass when there is none), converted for real on the GPU:
  every layer has the class its quant type asks for, its weight codes are the oracle's
  and its forward agrees with the oracle's arithmetic for that type
  (reference passes: src/cache_dit/quantization/torchao/quantize_ao.py:100-148)."""
  import cache_dit_amd as cache_dit
  from cache_dit_amd import nn as cnn
  torch.manual_seed(0)
  net = _PlanNet().to(torch.bfloat16)
  ref = copy.deepcopy(net)
  net = net.cuda()
  net._rowwise_layers = ["ff_out"]
  plan = {"to_k": "float8_per_tensor", "to_v": "float8_weight_only"} if with_plan else None
  cache_dit.quantize(net, cache_dit.QuantizeConfig(precision_plan=plan))
  want = {"to_q": "float8_per_row", "to_out.0": "float8_per_row", "ff_in": "float8_per_row",
          "to_k": "float8_per_tensor" if with_plan else "float8_per_row",
          "to_v": "float8_weight_only" if with_plan else "float8_per_row",
          "ff_out": "float8_per_tensor"}
  classes = {"float8_per_row": cnn.Fp8DynamicLinear, "float8_per_tensor": cnn.Fp8DynamicLinearPerTensor,
             "float8_weight_only": cnn.Fp8WeightOnlyLinear}
  ctx = net._quantize_context
  for kind in classes:
    assert ctx.quantized_map[kind] == 2 * sum(v == kind for v in want.values()), (kind, ctx.quantized_map)
  g = torch.Generator().manual_seed(1)
  for blk, rblk in zip(net.blocks, ref.blocks):
    for name, kind in want.items():
      lin, rlin = blk.get_submodule(name), rblk.get_submodule(name)
      assert type(lin) is classes[kind] and lin.quant_type == kind, (name, type(lin))
      w = rlin.weight.detach()
      wq, ws = (to.quantize_tensorwise if kind == "float8_per_tensor" else to.quantize_rowwise)(w)
      assert (bits_u8(lin.weight) == bits_u8(wq)).all(), name
      assert torch.equal(lin.weight_scale.cpu().reshape(-1), ws.reshape(-1)), name
      x = torch.randn(3, 37, lin.in_features, generator=g).to(torch.bfloat16)
      y = lin(x.cuda())
      y_ref = _oracle_linear(kind, x, w, None if rlin.bias is None else rlin.bias.detach())
      assert max_rel_err(y, y_ref) <= 1e-2, (name, kind, max_rel_err(y, y_ref))


def test_linear_on_cat_equals_the_linear_on_the_concatenation():
  """linear_on_cat(proj_out, [attn, mlp]) against proj_out(torch.cat(...)): same bits, eager,
  compiled (fullgraph) and for the cases that fall back to concatenating (another quant type,
  three sources, few rows); and a FLUX-shaped model with fuse_cat_quant equals itself without."""
  import logging
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  logging.getLogger("CACHE_DIT_AMD").setLevel(logging.WARNING)
  torch.manual_seed(0)
  lin = torch.nn.Linear(512 + 2048, 512).to(torch.bfloat16).cuda()
  holder = torch.nn.Sequential(lin)
  cache_dit.quantize(holder, cache_dit.QuantizeConfig())
  a = torch.randn(2, 300, 512, device="cuda").to(torch.bfloat16)
  b = torch.randn(2, 300, 2048, device="cuda").to(torch.bfloat16)
  with torch.no_grad():
    want = lin(torch.cat([a, b], dim=-1))
    assert torch.equal(cache_dit.linear_on_cat(lin, [a, b]), want)
    compiled = torch.compile(lambda u, v: cache_dit.linear_on_cat(lin, [u, v]), fullgraph=True)
    assert torch.equal(compiled(a, b), want)
    # few rows, three sources: the plain expression
    assert torch.equal(cache_dit.linear_on_cat(lin, [a[:1, :4], b[:1, :4]]),
                       lin(torch.cat([a[:1, :4], b[:1, :4]], dim=-1)))
    assert torch.equal(cache_dit.linear_on_cat(lin, [a, b[..., :1024], b[..., 1024:]]), want)
  wo = torch.nn.Sequential(torch.nn.Linear(512 + 2048, 512).to(torch.bfloat16).cuda())
  cache_dit.quantize(wo, cache_dit.QuantizeConfig(quant_type="float8_weight_only"))
  with torch.no_grad():
    assert torch.equal(cache_dit.linear_on_cat(wo[0], [a, b]), wo[0](torch.cat([a, b], dim=-1)))

  kw = dict(dim=512, heads=4, mlp=2048, n_double=1, n_single=3, in_channels=64, text_dim=256,
            pooled_dim=128)
  model = ds.FluxLikeTransformer(**kw).to(torch.bfloat16).cuda()
  cache_dit.quantize(model, cache_dit.QuantizeConfig())
  inputs = ds.flux_like_inputs("cuda", n_img=320, n_txt=64, in_channels=64, text_dim=256,
                               pooled_dim=128)
  with torch.no_grad():
    y0 = model(**inputs)
    assert ds.fuse_cat_quant(model) == 3
    assert torch.equal(model(**inputs), y0)


def test_compiled_blocks_run_the_batched_ops():
  """Blocks of a FLUX-shaped toy model under torch.compile(fullgraph=True) with the Linears of
  a stage handed to linear_batch: inside a compiled graph a stage is one cdit::linear_w8a8_batch
  (or cdit::w8a16_batch) op; the op equals the per-Linear ops bit for bit, the compiled model
  agrees with the eager one to the accuracy of the re-fused glue."""
  import logging
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  logging.getLogger("CACHE_DIT_AMD").setLevel(logging.WARNING)
  for quant_type in ("float8_per_row", "float8_weight_only"):
    torch.manual_seed(0)
    lins = [torch.nn.Linear(512, n).to(torch.bfloat16).cuda() for n in (512, 1024, 256, 512)]
    holder = torch.nn.ModuleList(lins)
    cache_dit.quantize(holder, cache_dit.QuantizeConfig(quant_type=quant_type))
    x = torch.randn(2, 150, 512, device="cuda").to(torch.bfloat16)
    e = torch.randn(2, 40, 512, device="cuda").to(torch.bfloat16)
    op = (torch.ops.cdit.linear_w8a8_batch if quant_type == "float8_per_row"
          else torch.ops.cdit.w8a16_batch)
    with torch.no_grad():
      outs = op([x, e], [l.weight for l in lins], [l.weight_scale.reshape(-1) for l in lins],
                [l.bias for l in lins], [3, 1], [0, 1, 0, 0])
      lins[1].epilogue = 1
      want = [lins[0](x), lins[1](x), lins[2](x), lins[3](e)]
      for o, w in zip(outs, want):
        assert torch.equal(o, w)
      fn = torch.compile(lambda a, b: cache_dit.linear_batch([(a, lins[:3]), (b, lins[3:])]),
                         fullgraph=True)
      (o0, o1, o2), (o3, ) = fn(x, e)
      for o, w in zip((o0, o1, o2, o3), want):
        assert torch.equal(o, w)

    kw = dict(dim=512, heads=4, mlp=2048, n_double=2, n_single=2, in_channels=64, text_dim=256,
              pooled_dim=128)
    model = ds.FluxLikeTransformer(**kw).to(torch.bfloat16).cuda()
    cache_dit.quantize(model, cache_dit.QuantizeConfig(quant_type=quant_type))
    ds.fuse_gelu_epilogues(model)
    inputs = ds.flux_like_inputs("cuda", n_img=320, n_txt=64, in_channels=64, text_dim=256,
                                 pooled_dim=128)
    with torch.no_grad():
      y0 = model(**inputs)
      ds.batch_streams(model, single_blocks=True)
      assert torch.equal(model(**inputs), y0)  # eager: the stateful batched path
      for blk in list(model.transformer_blocks) + list(model.single_transformer_blocks):
        blk.compile(fullgraph=True)
      y1 = model(**inputs)
    assert cosine(y1, y0) >= 0.999
