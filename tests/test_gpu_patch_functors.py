"""Stage patch functors (cache_dit_amd.patch_functors): an UNMODIFIED block -- the class's own
forward, diffusers attribute names and signatures -- patched in place runs every stage of
its Linears as one quantizer launch and one batched GEMM launch, with the bits of the plain
forward; launch counts are those of the hand-batched step the benchmark times."""
import logging

import pytest
import torch

from helpers import cosine

pytestmark = pytest.mark.gpu
logging.getLogger("CACHE_DIT_AMD").setLevel(logging.WARNING)


class _Launches:
  """Counts the library calls of a forward: batched / grouped GEMM launches, single GEMMs
  (fused quantizer + GEMM of one Linear, or a GEMM on shared codes), quantizer launches."""

  def __enter__(self):
    from cache_dit_amd import ops
    self.ops = ops
    self.n = {"batched": 0, "single": 0, "cat2": 0}
    self.saved = {}

    def wrap(name, key):
      fn = getattr(ops, name)
      self.saved[name] = fn

      def counted(*a, **k):
        self.n[key] += 1
        return fn(*a, **k)

      setattr(ops, name, counted)

    wrap("gemm_rowwise_batched_into", "batched")
    wrap("w8a16_batched_into", "batched")
    wrap("linear_w8a8_into", "single")
    wrap("gemm_rowwise_into", "single")
    wrap("w8a16_into", "single")
    wrap("quant_rowwise_cat2_into", "cat2")
    ops.quant_launches = 0
    return self

  def __exit__(self, *exc):
    for name, fn in self.saved.items():
      setattr(self.ops, name, fn)
    self.n["shared_quant"] = self.ops.quant_launches


def _flux(quant_type="float8_per_row", n_double=2, n_single=3):
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  torch.manual_seed(0)
  kw = dict(dim=512, heads=4, mlp=2048, n_double=n_double, n_single=n_single, in_channels=64,
            text_dim=256, pooled_dim=128)
  model = ds.FluxLikeTransformer(**kw).to(torch.bfloat16).cuda()
  cache_dit.quantize(model, cache_dit.QuantizeConfig(quant_type=quant_type))
  ds.fuse_gelu_epilogues(model)
  inputs = ds.flux_like_inputs("cuda", n_img=320, n_txt=64, in_channels=64, text_dim=256,
                               pooled_dim=128)
  return model, inputs


@pytest.mark.parametrize("quant_type", ["float8_per_row", "float8_weight_only"])
def test_flux_blocks_patched_in_place_run_stage_by_stage(quant_type):
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  model, inputs = _flux(quant_type)
  double, single = model.transformer_blocks[0], model.single_transformer_blocks[0]
  with torch.no_grad():
    with _Launches() as plain:
      y0 = model(**inputs)
    # 14 Linears per double block, 6 per single block, each a call of its own (what lies
    # outside the repeated blocks is not quantized)
    assert plain.n["batched"] == 0 and plain.n["single"] == 2 * 14 + 3 * 6
    assert cache_dit.apply_stage_patch(model) is model and model._cdit_stage_patched
    # the model's code is what it was: the class forwards are untouched, the instances rebound
    assert type(double).forward is ds.FluxTransformerBlock.forward
    assert type(single).forward is ds.FluxSingleTransformerBlock.forward
    assert type(double.attn).forward is ds.FluxAttention.forward and not double.attn._forward_pre_hooks
    with _Launches() as staged:
      y1 = model(**inputs)
    assert torch.equal(y1, y0)
    # double block: q/k/v + add_q/k/v, to_out + to_add_out, the two ff.net.0.proj, the two
    # ff.net.2: four batched launches; its two M = 1 norm Linears on their own. Single block:
    # proj_mlp + q/k/v one batched launch; norm.linear and proj_out on their own.
    assert staged.n["batched"] == 2 * 4 + 3 * 1
    assert staged.n["single"] == 2 * 2 + 3 * 2
    if quant_type == "float8_per_row":
      assert staged.n["shared_quant"] == 2 * 4 + 3 * 1  # one quantizer launch per stage
      assert staged.n["cat2"] == 3                       # proj_out reads [attn | mlp] in place
    assert torch.equal(model(**inputs), y0)
    # the fused modulated norms on top: the stages fed by one arrive with their codes
    if quant_type == "float8_per_row":
      cache_dit.apply_stage_patch(model, fuse_norm_quant=True, materialize=False)
      with _Launches() as fused:
        y2 = model(**inputs)
      assert fused.n["shared_quant"] == 2 * 2  # to_out / to_add_out and ff.net.2 of the double blocks
      assert torch.isfinite(y2.float()).all() and cosine(y2, y0) >= 0.9999
    cache_dit.remove_stage_patch(model)
    assert "forward" not in double.__dict__ and "forward" not in single.__dict__
    assert "forward" not in double.attn.__dict__ and "forward" not in double.attn.to_out[0].__dict__
    assert "_cdit_joint_attn" not in double.attn.to_out[0].__dict__
    with _Launches() as again:
      assert torch.equal(model(**inputs), y0)
    assert again.n["batched"] == 0


def test_qwen_image_and_wan_blocks_patched_in_place():
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  torch.manual_seed(0)
  qwen = ds.QwenImageLikeTransformer(dim=256, heads=2, mlp=512, n_layers=2, in_channels=64,
                                     text_dim=128).to(torch.bfloat16).cuda()
  cache_dit.quantize(qwen, cache_dit.QuantizeConfig())
  ds.fuse_gelu_epilogues(qwen)
  qin = ds.qwen_image_like_inputs("cuda", n_img=200, n_txt=24, in_channels=64, text_dim=128)
  wan = ds.WanLikeTransformer(dim=256, heads=2, ffn=512, n_layers=2, in_channels=64,
                              text_dim=128).to(torch.bfloat16).cuda()
  cache_dit.quantize(wan, cache_dit.QuantizeConfig())
  win = ds.wan_like_inputs("cuda", n_tokens=200, n_txt=48, in_channels=64, text_dim=128)
  with torch.no_grad():
    q0, w0 = qwen(**qin), wan(**win)
    cache_dit.apply_stage_patch(qwen)
    with _Launches() as staged:
      assert torch.equal(qwen(**qin), q0)
    # 12 quantized Linears per block in four stages of two streams; img_mod / txt_mod stay bf16
    assert staged.n["batched"] == 2 * 4 and staged.n["single"] == 0
    assert staged.n["shared_quant"] == 2 * 4
    cache_dit.apply_stage_patch(qwen, fuse_norm_quant=True)
    with _Launches() as fused:
      q2 = qwen(**qin)
    assert fused.n["shared_quant"] == 2 * 2 and cosine(q2, q0) >= 0.9999
    cache_dit.apply_stage_patch(wan)
    with _Launches() as staged:
      assert torch.equal(wan(**win), w0)
    # per block: q/k/v of the self-attention, the query next to k / v of the cross-attention
    # (two activations, one launch); the two output projections and the FFN on their own
    assert staged.n["batched"] == 2 * 2 and staged.n["single"] == 2 * 4
    cache_dit.apply_stage_patch(wan, fuse_norm_quant=True)
    w2 = wan(**win)
    assert cosine(w2, w0) >= 0.9999
    cache_dit.remove_stage_patch(wan)
    assert torch.equal(wan(**win), w0)


def test_single_block_that_takes_both_streams_and_graph_capture():
  """Newer diffusers hand FLUX single blocks the two streams; the functor picks the rebound
  forward by the original's parameters. And a patched model under hipGraph capture."""
  import cache_dit_amd as cache_dit
  from cache_dit_amd import patch_functors as pf
  from cache_dit_amd.testing import dit_shapes as ds

  class FluxSingleTransformerBlock(ds.FluxSingleTransformerBlock):  # same class name on purpose

    def forward(self, hidden_states, encoder_hidden_states, temb, image_rotary_emb=None,
                joint_attention_kwargs=None):
      n_txt = encoder_hidden_states.shape[1]
      h = torch.cat([encoder_hidden_states, hidden_states], dim=1)
      h = super().forward(h, temb, image_rotary_emb, joint_attention_kwargs)
      return h[:, :n_txt], h[:, n_txt:]

  torch.manual_seed(0)
  blk = FluxSingleTransformerBlock(512, 4, 2048).to(torch.bfloat16).cuda()
  holder = torch.nn.ModuleList([blk])
  for name, lin in list(blk.named_modules()):
    if isinstance(lin, torch.nn.Linear):
      cache_dit.nn.convert_linear_(lin, "float8_per_row")
  g = torch.Generator(device="cuda").manual_seed(1)
  hid = torch.randn(1, 96, 512, device="cuda", generator=g).to(torch.bfloat16)
  enc = torch.randn(1, 32, 512, device="cuda", generator=g).to(torch.bfloat16)
  temb = torch.randn(1, 512, device="cuda", generator=g).to(torch.bfloat16)
  with torch.no_grad():
    e0, h0 = blk(hid, enc, temb)
    pf.apply_stage_patch(holder)
    assert blk.forward.__func__ is pf._flux_single_forward_two_streams
    with _Launches() as staged:
      e1, h1 = blk(hid, enc, temb)
    assert torch.equal(e1, e0) and torch.equal(h1, h0) and staged.n["batched"] == 1

  model, inputs = _flux()
  with torch.no_grad():
    y0 = model(**inputs)
    cache_dit.apply_stage_patch(model, fuse_norm_quant=True, materialize=False)
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
    for src in (other, inputs, other):
      want = model(**src)
      torch.cuda.synchronize()
      for k in static:
        static[k].copy_(src[k])
      graph.replay()
      torch.cuda.synchronize()
      assert torch.equal(ys, want)
    assert cosine(model(**inputs), y0) >= 0.9999
  with torch.inference_mode():  # nothing is batched or handed over; still the plain result
    cache_dit.apply_stage_patch(model)
    assert torch.equal(model(**inputs), y0)


def test_precompute_stage_wrong_guesses_cost_time_not_correctness():
  import cache_dit_amd as cache_dit
  from cache_dit_amd import nn as cnn
  torch.manual_seed(0)
  lins = [torch.nn.Linear(256, n, dtype=torch.bfloat16).cuda() for n in (128, 64, 192)]
  for lin in lins:
    cnn.convert_linear_(lin, "float8_per_row")
  g = torch.Generator(device="cuda").manual_seed(2)
  x = torch.randn(40, 256, device="cuda", generator=g).to(torch.bfloat16)
  z = torch.randn(24, 256, device="cuda", generator=g).to(torch.bfloat16)
  want = [lins[0](x), lins[1](x), lins[2](z)]
  assert cache_dit.precompute_stage([(x, lins[:2]), (z, lins[2:])])
  # another activation: computed afresh, the stash is gone afterwards
  y = lins[0](z)
  assert y.shape == (24, 128) and torch.equal(y, lins[0](z.clone()))
  assert lins[0]._precomputed is None
  assert torch.equal(lins[1](x), want[1])          # the right guess: handed out once
  assert lins[1]._precomputed is None and torch.equal(lins[1](x), want[1])
  x2 = x.clone()
  assert cache_dit.precompute_stage([(x2, lins[:2])])
  x2.add_(1)                                        # modified since: the stash must not be used
  assert torch.equal(lins[0](x2), lins[0](x2.clone()))
  assert torch.equal(lins[2](z), want[2])          # dropped by the later precompute_stage
  # refused: the same Linear twice, mixed types, inference tensors
  assert not cache_dit.precompute_stage([(x, [lins[0], lins[0]])])
  with torch.inference_mode():
    assert not cache_dit.precompute_stage([(x.clone(), lins[:2])])
  assert torch.equal(lins[0](x), want[0])


def test_patched_blocks_traced_by_torch_compile_keep_the_stages():
  """The patched blocks under torch.compile(fullgraph=True): every stage the wrappers and
  rebound forwards put together is ONE batch op in the traced graph (counted with a backend
  that only inspects the graph and runs it as it is), all blocks of a class share one
  compiled graph, and the output equals the eager forward's."""
  import cache_dit_amd as cache_dit
  try:
    import torch._dynamo as dynamo
  except Exception as e:
    pytest.skip(f"no graph tracer: {str(e)[:80]}")
  model, inputs = _flux(n_double=3, n_single=3)
  seen = []

  def inspect_only(gm, example_inputs):
    ops_in_graph = [str(n.target) for n in gm.graph.nodes if n.op == "call_function"]
    seen.append({"batch": sum("linear_w8a8_batch" in t for t in ops_in_graph),
                 "single": sum(t.startswith("cdit.linear_w8a8.") or t == "cdit.linear_w8a8" or
                               "cdit.linear_w8a8.default" in t for t in ops_in_graph),
                 "cat2": sum("linear_w8a8_cat2" in t for t in ops_in_graph)})
    return gm.forward

  with torch.no_grad():
    y0 = model(**inputs)
    cache_dit.apply_stage_patch(model)
    assert torch.equal(model(**inputs), y0)
    dynamo.reset()
    for blocks in (model.transformer_blocks, model.single_transformer_blocks):
      for i in range(len(blocks)):
        blocks[i] = torch.compile(blocks[i], backend=inspect_only, fullgraph=True)
    y1 = model(**inputs)
  # one graph per block class (the blocks of a class share it); double block: q/k/v of both
  # streams, the two ff.net.0.proj, the two ff.net.2 as batch ops, its two output projections
  # and two M = 1 Linears single; single block: proj_mlp + q/k/v one batch op, proj_out
  # reading its two sources, the M = 1 Linear
  assert len(seen) == 2, seen
  assert seen[0] == {"batch": 3, "single": 4, "cat2": 0}, seen
  assert seen[1] == {"batch": 1, "single": 1, "cat2": 1}, seen
  assert torch.equal(y1, y0)
  assert all(m._precomputed is None for m in model.modules() if hasattr(m, "_precomputed"))


def test_patched_qwen_image_and_wan_blocks_trace_without_graph_breaks():
  """The other two block families under torch.compile(fullgraph=True) with the stage patch:
  one graph per block class, the stages as batch ops, the eager forward's bits."""
  import cache_dit_amd as cache_dit
  from cache_dit_amd.testing import dit_shapes as ds
  try:
    import torch._dynamo as dynamo
  except Exception as e:
    pytest.skip(f"no graph tracer: {str(e)[:80]}")
  torch.manual_seed(0)
  qwen = ds.QwenImageLikeTransformer(dim=256, heads=2, mlp=512, n_layers=3, in_channels=64,
                                     text_dim=128).to(torch.bfloat16).cuda()
  cache_dit.quantize(qwen, cache_dit.QuantizeConfig())
  ds.fuse_gelu_epilogues(qwen)
  qin = ds.qwen_image_like_inputs("cuda", n_img=200, n_txt=24, in_channels=64, text_dim=128)
  wan = ds.WanLikeTransformer(dim=256, heads=2, ffn=512, n_layers=3, in_channels=64,
                              text_dim=128).to(torch.bfloat16).cuda()
  cache_dit.quantize(wan, cache_dit.QuantizeConfig())
  win = ds.wan_like_inputs("cuda", n_tokens=200, n_txt=48, in_channels=64, text_dim=128)
  for model, inputs, batch_ops in ((qwen, qin, 3), (wan, win, 2)):
    seen = []

    def inspect_only(gm, example_inputs, seen=seen):
      seen.append(sum("linear_w8a8_batch" in str(n.target) for n in gm.graph.nodes
                      if n.op == "call_function"))
      return gm.forward

    blocks = next(m for m in model.children() if isinstance(m, torch.nn.ModuleList))
    with torch.no_grad():
      y0 = model(**inputs)
      cache_dit.apply_stage_patch(model)
      dynamo.reset()
      for i in range(len(blocks)):
        blocks[i] = torch.compile(blocks[i], backend=inspect_only, fullgraph=True)
      y1 = model(**inputs)
    # Qwen-Image: q/k/v of both streams and the two pairs of MLP Linears (its joint output
    # projections rest on storage addresses and stay two ops in a traced graph); Wan: q/k/v of
    # the self-attention, the query next to k / v of the cross-attention
    assert seen == [batch_ops], seen
    assert torch.equal(y1, y0)
