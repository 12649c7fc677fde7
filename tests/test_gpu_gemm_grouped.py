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


def _acts(spec, seed, integer=False):
  """spec: list of (M, [N...]); one K for all. Returns the `acts` list for
  gemm_rowwise_batched_into (outputs NaN-filled) and the per-member epilogue flags."""
  out = []
  for s, (M, K, Ns, epis) in enumerate(spec):
    a, a_s, ws, wss, bs = _members(M, K, Ns, seed=seed + 17 * s, integer=integer, no_bias=(1,))
    outs = [torch.full((M, N), float("nan"), dtype=torch.bfloat16, device="cuda") for N in Ns]
    out.append((a, a_s, ws, wss, bs, outs, list(epis)))
  return out


@pytest.mark.parametrize("spec", [
    # FLUX double block, stage by stage: image stream (4096 tokens) + text stream (512 tokens)
    [(4096, 3072, [3072] * 3, [0] * 3), (512, 3072, [3072] * 3, [0] * 3)],
    [(4096, 3072, [3072], [0]), (512, 3072, [3072], [0])],
    [(4096, 3072, [12288], [1]), (512, 3072, [12288], [1])],
    [(4096, 12288, [3072], [0]), (512, 12288, [3072], [0])],
    # Qwen-Image: 6889 + 256 tokens
    [(6889, 3072, [3072] * 3, [0] * 3), (256, 3072, [3072] * 3, [0] * 3)],
    # ragged everything, three activations
    [(300, 512, [520, 264], [0, 1]), (77, 512, [72], [0]), (1000, 512, [136, 8, 200], [1, 0, 0])],
])
def test_batched_equals_separate_launches(spec):
  from cache_dit_amd import ops
  acts = _acts(spec, seed=spec[0][0])
  ops.gemm_rowwise_batched_into(acts)
  torch.cuda.synchronize()
  for s, (a, a_s, ws, wss, bs, outs, epis) in enumerate(acts):
    want = _separate(a, a_s, ws, wss, bs, epis)
    for p, (g, w) in enumerate(zip(outs, want)):
      assert torch.equal(g.view(torch.int16), w.view(torch.int16)), f"activation {s} member {p}"


def test_batched_launch_is_deterministic_over_repeats():
  """The same batch twenty times over, alternating with other launches: every run gives
  the same bits as the first and as the members on their own (a timing-dependent fault in
  the tile stream would show as a run that differs)."""
  from cache_dit_amd import ops
  spec = [(6889, 3072, [3072] * 3, [0] * 3), (256, 3072, [3072] * 3, [0] * 3)]
  acts = _acts(spec, seed=6889)
  want = [_separate(a, a_s, ws, wss, bs, epis) for a, a_s, ws, wss, bs, outs, epis in acts]
  other = _acts([(300, 512, [520, 264], [0, 1]), (77, 512, [72], [0])], seed=1)
  for rep in range(20):
    for _, _, _, _, _, outs, _ in acts:
      for o in outs:
        o.fill_(float("nan"))
    ops.gemm_rowwise_batched_into(acts)
    if rep % 3 == 0:
      ops.gemm_rowwise_batched_into(other)
    torch.cuda.synchronize()
    for s, (_, _, _, _, _, outs, _) in enumerate(acts):
      for p, (g, w) in enumerate(zip(outs, want[s])):
        assert torch.equal(g.view(torch.int16), w.view(torch.int16)), (rep, s, p)


@pytest.mark.parametrize("variant", [12, 14, 15, 16, 17, 18])
def test_batched_every_tile_shape_exact_integers_against_the_oracle(variant):
  from cache_dit_amd import _native, ops
  spec = [(2100, 640, [1096, 520], [0, 0]), (333, 640, [3080], [0]), (40, 640, [264, 72], [0, 0])]
  acts = _acts(spec, seed=variant, integer=True)
  _native.set_gemm_variant(variant)
  ops.gemm_rowwise_batched_into(acts)
  torch.cuda.synchronize()
  _native.set_gemm_variant(-1)
  for s, (a, a_s, ws, wss, bs, outs, epis) in enumerate(acts):
    for p in range(len(ws)):
      ref = to.scaled_mm_rowwise(a.cpu(), a_s.cpu(), ws[p].cpu(), wss[p].cpu(),
                                 None if bs[p] is None else bs[p].cpu())
      assert torch.equal(outs[p].cpu().view(torch.int16), ref.view(torch.int16)), (s, p)


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
  assert L.cdit_fp8_gemm_rowwise_grouped(None, None, 4, 64, 64, 9, None, None, None, None, None, 64,
                                         None, None, None) == 1
  assert b"a batch holds" in L.cdit_last_error()
  # a batch with an M <= 16 activation runs member by member
  from cache_dit_amd import ops
  acts = _acts([(300, 512, [520], [0]), (5, 512, [264], [0])], seed=8)
  ops.gemm_rowwise_batched_into(acts)
  torch.cuda.synchronize()
  for a, a_s, ws, wss, bs, outs, epis in acts:
    for g, w in zip(outs, _separate(a, a_s, ws, wss, bs, epis)):
      assert torch.equal(g.view(torch.int16), w.view(torch.int16))


def test_grouped_random_data_against_the_oracle_sampled_rows():
  M, K, Ns = 4608, 3072, [12288, 3072, 3072, 3072]
  a, a_s, ws, wss, bs = _members(M, K, Ns, seed=9)
  got = _grouped(a, a_s, ws, wss, bs, [1, 0, 0, 0])
  rows = torch.cat([torch.arange(0, M, 211), torch.arange(M - 2, M)]).cuda()
  for p in range(4):
    ref = to.scaled_mm_rowwise(a[rows].cpu(), a_s[rows].cpu(), ws[p].cpu(), wss[p].cpu(), bs[p].cpu(),
                               gelu="fused" if p == 0 else None)
    assert max_rel_err(got[p][rows], ref) <= 1e-2, p


def test_sibling_groups_in_a_model_are_found_and_bit_identical():
  """group_sibling_linears_ on FLUX- and Wan-shaped toy models: the groups are the runs of
  Linears fed the same buffer (q/k/v, add_q/k/v, proj_mlp + q/k/v; in Wan's cross
  attention only to_k / to_v, which read the text), the output equals the ungrouped
  model's bit for bit, also under graph capture and with the fused producer."""
  import logging
  import cache_dit_amd as cache_dit
  from cache_dit_amd import ops
  from cache_dit_amd.testing import dit_shapes as ds
  logging.getLogger("CACHE_DIT_AMD").setLevel(logging.WARNING)
  torch.manual_seed(0)
  kw = dict(dim=512, heads=4, mlp=2048, n_double=2, n_single=3, in_channels=64, text_dim=256,
            pooled_dim=128)
  model = ds.FluxLikeTransformer(**kw).to(torch.bfloat16).cuda()
  cache_dit.quantize(model, cache_dit.QuantizeConfig())
  ds.fuse_gelu_epilogues(model)
  inputs = ds.flux_like_inputs("cuda", n_img=320, n_txt=64, in_channels=64, text_dim=256,
                               pooled_dim=128)
  with torch.no_grad():
    y0 = model(**inputs)
  n = cache_dit.group_sibling_linears_(model, lambda: model(**inputs))
  assert n == 2 * 2 + 3 * 1
  blk = model.single_transformer_blocks[0]
  assert blk.proj_mlp.sibling_group is blk.attn.to_v.sibling_group
  assert len(blk.proj_mlp.sibling_group.members) == 4 and blk.proj_out.sibling_group is None
  with torch.no_grad():
    ops.quant_launches = 0
    y1 = model(**inputs)
    # per double block 14 Linears, 6 of them in two groups; per single block 6, 4 in one group
    assert ops.quant_launches == 2 * 2 + 3 * 1  # only the groups go through the shared lookup
    assert torch.equal(y1, y0)
    assert torch.equal(model(**inputs), y0)
    # the fused producer hands its codes to the groups as well
    ds.fuse_norm_quant(model)
    ops.quant_launches = 0
    y2 = model(**inputs)
    assert ops.quant_launches == 0 and torch.isfinite(y2.float()).all()
    ds.fuse_norm_quant(model, False)
    # graph capture: the siblings' outputs live in the graph's pool
    static = {k: v.clone() for k, v in inputs.items()}
    model(**static)
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
  with torch.inference_mode():  # no version counters: members compute on their own
    assert torch.equal(model(**inputs), y0)
  assert cache_dit.group_sibling_linears_(model, enable=False) == 0
  assert blk.proj_mlp.sibling_group is None

  wan = ds.WanLikeTransformer(dim=256, heads=2, ffn=512, n_layers=2, in_channels=64,
                              text_dim=128).to(torch.bfloat16).cuda()
  cache_dit.quantize(wan, cache_dit.QuantizeConfig())
  winp = ds.wan_like_inputs("cuda", n_tokens=200, n_txt=48, in_channels=64, text_dim=128)
  with torch.no_grad():
    w0 = wan(**winp)
    assert cache_dit.group_sibling_linears_(wan, lambda: wan(**winp)) == 2 * 2
    b0 = wan.blocks[0]
    assert len(b0.attn1.to_q.sibling_group.members) == 3
    assert b0.attn2.to_q.sibling_group is None and len(b0.attn2.to_k.sibling_group.members) == 2
    assert torch.equal(wan(**winp), w0)


def test_stream_batched_block_forwards_are_bit_identical():
  """FLUX- and Qwen-Image-shaped toy models with the image- and text-stream Linears of a
  stage handed to linear_batch (one launch per stage): same bits as the plain forwards,
  also combined with the fused producer, under graph capture, and for models that are
  not quantized at all (then the Linears just run one by one)."""
  import logging
  import cache_dit_amd as cache_dit
  from cache_dit_amd import ops
  from cache_dit_amd.testing import dit_shapes as ds
  logging.getLogger("CACHE_DIT_AMD").setLevel(logging.WARNING)
  torch.manual_seed(0)
  kw = dict(dim=512, heads=4, mlp=2048, n_double=2, n_single=2, in_channels=64, text_dim=256,
            pooled_dim=128)
  model = ds.FluxLikeTransformer(**kw).to(torch.bfloat16).cuda()
  inputs = ds.flux_like_inputs("cuda", n_img=320, n_txt=64, in_channels=64, text_dim=256,
                               pooled_dim=128)
  with torch.no_grad():
    y_bf16 = model(**inputs)
    assert ds.batch_streams(model) == 2
    assert torch.equal(model(**inputs), y_bf16)  # unquantized: plain Linears, one by one
    ds.batch_streams(model, False)
  cache_dit.quantize(model, cache_dit.QuantizeConfig())
  ds.fuse_gelu_epilogues(model)
  with torch.no_grad():
    y0 = model(**inputs)
    ds.batch_streams(model)
    ops.quant_launches = 0
    y1 = model(**inputs)
    # per double block 4 stages go through the shared lookup, each one quantizer launch for
    # its two streams; nothing else does
    assert ops.quant_launches == 2 * 4
    assert torch.equal(y1, y0)
    ds.fuse_norm_quant(model)  # the modulated activations arrive with their codes
    ops.quant_launches = 0
    y2 = model(**inputs)
    assert ops.quant_launches == 2 * 2 and torch.isfinite(y2.float()).all()
    ds.fuse_norm_quant(model, False)
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
                                pooled_dim=128, seed=3)
    want = model(**other)
    for k in static:
      static[k].copy_(other[k])
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(ys, want)
  with torch.inference_mode():
    assert torch.equal(model(**inputs), y0)

  qwen = ds.QwenImageLikeTransformer(dim=256, heads=2, mlp=512, n_layers=2, in_channels=64,
                                     text_dim=128).to(torch.bfloat16).cuda()
  cache_dit.quantize(qwen, cache_dit.QuantizeConfig())
  qin = ds.qwen_image_like_inputs("cuda", n_img=200, n_txt=24, in_channels=64, text_dim=128)
  with torch.no_grad():
    q0 = qwen(**qin)
    assert ds.batch_streams(qwen) == 2
    assert torch.equal(qwen(**qin), q0)


@pytest.mark.parametrize("seed", range(24))
def test_batched_random_shapes_exact_against_the_oracle(seed):
  """Randomly drawn batches -- 1 to 4 activations of 17 to 700 rows, 1 to 3 members each with
  N a multiple of 8 up to 600, K of 3 to 8 steps, random epilogue flags and missing biases,
  a randomly forced tile shape or the automatic choice -- on integer-valued data, where every
  partial sum is exact: the outputs must equal the CPU oracle bit for bit, and nothing but
  the outputs may be written (each is a window of a sentinel-filled buffer)."""
  import random
  from cache_dit_amd import _native, ops
  rnd = random.Random(seed)
  K = 128 * rnd.randint(3, 8)
  n_act = rnd.randint(1, 4)
  budget = 8
  acts, bufs = [], []
  for s in range(n_act):
    M = rnd.choice([17, 33, 64, 100, 255, 256, 257, 300, 511, 700])
    n_mem = rnd.randint(1, min(3, budget - (n_act - s - 1)))
    budget -= n_mem
    Ns = [8 * rnd.randint(1, 75) for _ in range(n_mem)]
    no_bias = tuple(i for i in range(n_mem) if rnd.random() < 0.3)
    a, a_s, ws, wss, bs = _members(M, K, Ns, seed=1000 * seed + s, integer=True, no_bias=no_bias)
    epis = [rnd.randint(0, 1) for _ in Ns]
    outs = []
    for N in Ns:
      buf = torch.full((M + 1, N + 8), 7.0, dtype=torch.bfloat16, device="cuda")
      bufs.append((buf, M, N))
      outs.append(buf[:M, :N])
    acts.append((a, a_s, ws, wss, bs, outs, epis))
  variant = rnd.choice([-1, -1, 12, 14, 15, 16, 17, 18])
  _native.set_gemm_variant(variant)
  if n_act == 1 and len(acts[0][2]) == 1:
    a, a_s, ws, wss, bs, outs, epis = acts[0]
    ops.gemm_rowwise_into(a, a_s, ws[0], wss[0], bs[0], outs[0], epis[0])
  else:
    ops.gemm_rowwise_batched_into(acts)
  torch.cuda.synchronize()
  for s, (a, a_s, ws, wss, bs, outs, epis) in enumerate(acts):
    for p, (w, sc, b, o, e) in enumerate(zip(ws, wss, bs, outs, epis)):
      ref = to.scaled_mm_rowwise(a.cpu(), a_s.cpu(), w.cpu(), sc.cpu(), None if b is None else b.cpu(),
                                 gelu="fused" if e else None)
      if e:  # the GELU is not exact arithmetic: the oracle's tolerance
        assert max_rel_err(o.cpu(), ref) <= 1e-2, (seed, variant, s, p)
      else:
        assert torch.equal(o.cpu().view(torch.int16), ref.view(torch.int16)), (seed, variant, s, p)
  for buf, M, N in bufs:
    assert (buf[M] == 7.0).all() and (buf[:, N:] == 7.0).all(), (seed, variant)
