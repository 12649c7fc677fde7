"""Layer-selection policy of quantize(): table-driven checks on module trees with
diffusers-style names, run on CPU with a recording converter. Known answers are
the reference's documented summary tables (docs/user_guide/QUANTIZATION.md:193-226,
263-274: FLUX.2-klein 88/56/144 and 96/32/8/8) and the per-model Linear counts."""
import logging

import pytest
import torch
from torch import nn

from cache_dit_amd import QuantizeConfig
from cache_dit_amd.quantization.policy import QuantizeContext, quantize_ao
from cache_dit_amd.testing import dit_shapes as ds

logging.getLogger("CACHE_DIT_AMD").setLevel(logging.WARNING)


def lin(i=32, o=32, dtype=torch.bfloat16, bias=True):
  return nn.Linear(i, o, bias=bias, dtype=dtype)


class _Attn(nn.Module):

  def __init__(self, double):
    super().__init__()
    if double:
      self.to_q, self.to_k, self.to_v = lin(), lin(), lin()
      self.to_out = nn.ModuleList([lin(), nn.Dropout(0.0)])
      self.add_q_proj, self.add_k_proj, self.add_v_proj, self.to_add_out = lin(), lin(), lin(), lin()
    else:
      self.to_qkv_mlp_proj, self.to_out = lin(), lin()


class _FF(nn.Module):

  def __init__(self):
    super().__init__()
    self.linear_in, self.linear_out = lin(), lin()


class Flux2TransformerBlock(nn.Module):

  def __init__(self):
    super().__init__()
    self.attn, self.ff, self.ff_context = _Attn(True), _FF(), _FF()


class Flux2SingleTransformerBlock(nn.Module):

  def __init__(self):
    super().__init__()
    self.attn = _Attn(False)


class Flux2KleinLike(nn.Module):
  """8 double + 24 single blocks = 144 Linears inside the repeated blocks."""
  _repeated_blocks = ["Flux2TransformerBlock", "Flux2SingleTransformerBlock"]

  def __init__(self):
    super().__init__()
    self.x_embedder = lin()
    self.transformer_blocks = nn.ModuleList([Flux2TransformerBlock() for _ in range(8)])
    self.single_transformer_blocks = nn.ModuleList([Flux2SingleTransformerBlock() for _ in range(24)])


ROWWISE = ["attn.to_out.0", "attn.to_add_out", "ff.linear_out", "ff_context.linear_out", "attn.to_out"]


def run(module, config):
  calls = []
  quantize_ao(module, config, _convert_fn=lambda l, qt: calls.append(qt))
  return module._quantize_context, calls


def test_flux2_klein_tp_without_fallback_88_of_144():
  m = Flux2KleinLike()
  m._rowwise_layers = ROWWISE
  ctx, calls = run(m, QuantizeConfig(per_tensor_fallback=False, verbose=True))
  assert ctx.quantized_map["float8_per_row"] == 88 and len(calls) == 88
  assert len(ctx.skipped_map["float8_per_row"]) == 56 and ctx.num_linear_layers == 144
  rows = ctx.summary_lines()
  assert rows[0] == "Quantized        Region: ['Flux2TransformerBlock', 'Flux2SingleTransformerBlock']"
  assert rows[1] == "Quantized Linear Layers: 88    float8_per_row     56 (skipped)"
  assert rows[2:5] == ["Quantized Linear Layers: 88    (total)", "Skipped   Linear Layers: 56    (total)",
                       "Linear           Layers: 144   (total)"]
  reasons = ctx.skipped_reason_lines()
  assert reasons == [
      "float8_per_row, skip: attn.to_out.0        : pattern<RowwiseParallel>: 8    layers",
      "float8_per_row, skip: attn.to_add_out      : pattern<RowwiseParallel>: 8    layers",
      "float8_per_row, skip: ff.linear_out        : pattern<RowwiseParallel>: 8    layers",
      "float8_per_row, skip: ff_context.linear_out: pattern<RowwiseParallel>: 8    layers",
      "float8_per_row, skip: attn.to_out          : pattern<RowwiseParallel>: 24   layers",
  ]


def test_flux2_klein_tp_with_fallback_144_of_144():
  m = Flux2KleinLike()
  m._rowwise_layers = ROWWISE
  ctx, calls = run(m, QuantizeConfig(per_tensor_fallback=True))
  assert ctx.quantized_map["float8_per_row"] == 88 and ctx.quantized_map["float8_per_tensor"] == 56
  assert calls.count("float8_per_tensor") == 56 and sum(len(v) for v in ctx.skipped_map.values()) == 0
  assert ctx.summary_lines() == [
      "Quantized        Region: ['Flux2TransformerBlock', 'Flux2SingleTransformerBlock']",
      "Quantized Linear Layers: 88    float8_per_row     0 (skipped)",
      "Quantized Linear Layers: 56    float8_per_tensor  0 (skipped)",
      "Quantized Linear Layers: 144   (total)",
      "Skipped   Linear Layers: 0     (total)",
      "Linear           Layers: 144   (total)",
  ]


def test_flux2_klein_precision_plan_96_32_8_8():
  m = Flux2KleinLike()
  plan = {"attn.to_q": "float8_per_tensor", "attn.to_k": "float8_weight_only",
          "attn.to_v": "float8_per_block", "attn.to_out": "float8_per_row"}
  for mod in m.modules():  # per-block needs 128-multiples
    if isinstance(mod, nn.Linear):
      mod.weight = nn.Parameter(torch.zeros(128, 128, dtype=torch.bfloat16))
  ctx, calls = run(m, QuantizeConfig(precision_plan=plan))
  got = {k: v for k, v in ctx.quantized_map.items() if v}
  assert got == {"float8_per_row": 96, "float8_per_tensor": 32, "float8_per_block": 8,
                 "float8_weight_only": 8}
  assert ctx.num_linear_layers == 144 and sum(len(v) for v in ctx.skipped_map.values()) == 0


def test_env_flag_disables_the_rowwise_handling(monkeypatch):
  monkeypatch.setenv("CACHE_DIT_DISABLE_EXCLUDE_FOR_QUANTIZE_AFTER_TP", "1")
  m = Flux2KleinLike()
  m._rowwise_layers = ROWWISE
  ctx, _ = run(m, QuantizeConfig(per_tensor_fallback=False))
  assert ctx.quantized_map["float8_per_row"] == 144


@pytest.mark.parametrize("cls,quantized,skipped,linears", [
    (ds.FluxLikeTransformer, 494, 0, 494),
    (ds.QwenImageLikeTransformer, 720, 120, 840),
    (ds.WanLikeTransformer, 400, 0, 400),
])
def test_baseline_models_linear_inventory(cls, quantized, skipped, linears):
  with torch.device("meta"):
    m = cls().to(torch.bfloat16)
  ctx, calls = run(m, QuantizeConfig())
  assert len(calls) == quantized == ctx.quantized_map["float8_per_row"]
  assert sum(len(v) for v in ctx.skipped_map.values()) == skipped and ctx.num_linear_layers == linears
  if skipped:
    assert set(ctx.skipped_map["float8_per_row"]) == {"skip: img_mod.1 -> pattern<mod>",
                                                      "skip: txt_mod.1 -> pattern<mod>"}
  assert m._is_quantized and m._quantize_type == "float8_per_row"
  assert m._exclude_layers == ["embedder", "embed", "modulation", "mod"]


def test_whole_module_mode_sees_root_relative_names():
  with torch.device("meta"):
    m = ds.FluxLikeTransformer(dim=64, heads=2, mlp=128, n_double=1, n_single=1, in_channels=16,
                               text_dim=32, pooled_dim=16).to(torch.bfloat16)
  ctx, _ = run(m, QuantizeConfig(regional_quantize=False))
  skipped = {r.split(" -> ")[0].removeprefix("skip: ") for r in ctx.skipped_map["float8_per_row"]}
  assert {"x_embedder", "context_embedder", "time_text_embed.timestep_embedder.0"} <= skipped
  assert ctx.quantized_map["float8_per_row"] == 14 + 6 + 2  # blocks + norm_out.linear + proj_out
  assert ctx.quantized_region == "FluxLikeTransformer"


def test_no_repeated_blocks_attribute_falls_back_to_whole_module():
  m = nn.Sequential(lin(), nn.ReLU(), lin())
  ctx, calls = run(m, QuantizeConfig(exclude_layers=[]))
  assert not ctx.regional_quantize and len(calls) == 2


def test_repeated_blocks_from_config_and_missing_region():
  m = nn.Sequential(Flux2SingleTransformerBlock(), lin())
  ctx, calls = run(m, QuantizeConfig(repeated_blocks=["Flux2SingleTransformerBlock"]))
  assert len(calls) == 2
  with pytest.raises(ValueError, match="Regional quantization failed"):
    run(nn.Sequential(lin()), QuantizeConfig(repeated_blocks=["NoSuchBlock"]))


def test_dtype_rules():
  m = nn.Sequential(lin(dtype=torch.float32))
  with pytest.raises(AssertionError, match="weight dtype of bfloat16"):
    run(m, QuantizeConfig(exclude_layers=[]))
  # weight-only and per-tensor have no dtype assertion: a layer the kernels cannot take
  # is left unquantized with a reason (torchao leaves such a layer alone without raising)
  for qt in ("float8_weight_only", "float8_per_tensor"):
    ctx, calls = run(nn.Sequential(lin(dtype=torch.float32)),
                     QuantizeConfig(quant_type=qt, exclude_layers=[]))
    assert calls == [] and ctx.quantized_map[qt] == 0
    assert ctx.skipped_map[qt] == ["skip: 0 -> pattern<dtype(torch.float32)!=bfloat16>"]


def test_dimensions_not_multiple_of_16_are_skipped():
  m = nn.Sequential(lin(30, 32), lin(32, 32))
  ctx, calls = run(m, QuantizeConfig(exclude_layers=[]))
  assert len(calls) == 1
  assert ctx.skipped_map["float8_per_row"] == ["skip: 0 -> pattern<weight_shape(32, 30)%16!=0>"]


def test_per_tensor_plan_and_fallback_skip_what_the_kernels_cannot_take():
  """A 100x64 Linear under a float8_per_tensor plan entry, and one reached by the
  per-tensor fallback pass, are skipped with a reason instead of raising in the
  middle of the walk."""

  class Blk(nn.Module):

    def __init__(self):
      super().__init__()
      self.odd, self.even, self.row_parallel = lin(64, 100), lin(64, 64), lin(100, 64)

  class Net(nn.Module):
    _repeated_blocks = ["Blk"]

    def __init__(self):
      super().__init__()
      self.blocks = nn.ModuleList([Blk(), Blk()])

  ctx, calls = run(Net(), QuantizeConfig(precision_plan={"odd": "float8_per_tensor"},
                                         per_tensor_fallback=False))
  assert calls == ["float8_per_row"] * 2  # `even`; `row_parallel` has K = 100
  assert ctx.quantized_map["float8_per_tensor"] == 0
  assert ctx.skipped_map["float8_per_tensor"] == ["skip: odd -> pattern<weight_shape(100, 64)%16!=0>"] * 2
  # the default pass meets `odd` again (still unquantized) and skips it once more
  assert ctx.skipped_map["float8_per_row"] == [
      "skip: odd -> pattern<weight_shape(100, 64)%16!=0>",
      "skip: row_parallel -> pattern<weight_shape(64, 100)%16!=0>"] * 2
  net = Net()
  net._rowwise_layers = ["row_parallel"]
  ctx, calls = run(net, QuantizeConfig())
  assert calls == ["float8_per_row"] * 2 and ctx.quantized_map["float8_per_tensor"] == 0
  assert "fallback: row_parallel -> pattern<weight_shape(64, 100)%16!=0>" in ctx.skipped_map[
      "float8_per_tensor"]
  for blk in net.blocks:
    assert not getattr(blk.row_parallel, "_is_inner_quantized", False)
    assert not getattr(blk.odd, "_is_inner_quantized", False)


def test_failed_conversion_rolls_the_bookkeeping_back():
  m = nn.Sequential(lin(), lin())
  seen = []

  def convert(linear, qt):
    seen.append(linear)
    if len(seen) == 2:
      raise RuntimeError("boom")

  with pytest.raises(RuntimeError, match="boom"):
    quantize_ao(m, QuantizeConfig(exclude_layers=[]), _convert_fn=convert)
  assert getattr(m[0], "_is_inner_quantized", False) and not getattr(m[1], "_is_inner_quantized", False)
  assert not getattr(m, "_is_quantized", False)


def test_dtype_overrides_other_than_e4m3fn_are_refused():
  """The reference forwards weight_dtype / activation_dtype to torchao
  (quantize_ao.py:548-555); only e4m3fn is built here."""
  for key in ("weight_dtype", "activation_dtype"):
    with pytest.raises(NotImplementedError, match=key):
      quantize_ao(nn.Sequential(lin()), QuantizeConfig(exclude_layers=[]),
                  _convert_fn=lambda l, qt: None, **{key: torch.float8_e5m2})
  calls = []
  quantize_ao(nn.Sequential(lin()), QuantizeConfig(exclude_layers=[]),
              _convert_fn=lambda l, qt: calls.append(qt), weight_dtype=torch.float8_e4m3fn)
  assert calls == ["float8_per_row"]


def test_bad_quant_types():
  with pytest.raises(AssertionError, match="not supported"):
    QuantizeContext(quant_type="float7")
  with pytest.raises(AssertionError, match="precision_plan"):
    run(Flux2KleinLike(), QuantizeConfig(precision_plan={"attn": "float7"}))
  # a type the reference routes to torchao but that has no kernel here fails loudly
  with pytest.raises((NotImplementedError, AssertionError, ImportError)):
    quantize_ao(nn.Sequential(lin()), QuantizeConfig(quant_type="int8_per_row", exclude_layers=[]))


def test_already_quantized_module_is_left_alone():
  m = Flux2KleinLike()
  _, calls = run(m, QuantizeConfig())
  n = len(calls)
  calls2 = []
  quantize_ao(m, QuantizeConfig(), _convert_fn=lambda l, qt: calls2.append(qt))
  assert n == 144 and calls2 == []
