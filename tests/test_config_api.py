"""QuantizeConfig, quantize() argument handling, YAML loading, enable_cache
plumbing and the bookkeeping attributes -- the Python API boundary."""
import logging
import os

import pytest
import torch
from torch import nn

import cache_dit_amd as cache_dit
from cache_dit_amd import QuantizeBackend, QuantizeConfig
from cache_dit_amd.quantization import policy

GOLD = os.path.join(os.path.dirname(__file__), "golden", "configs")
logging.getLogger("CACHE_DIT_AMD").setLevel(logging.ERROR)


def test_defaults_and_normalisation():
  c = QuantizeConfig()
  assert c.quant_type == "float8_per_row" and c.backend == QuantizeBackend.TORCHAO
  assert c.exclude_layers == ["embedder", "embed", "modulation", "mod"]
  assert c.regional_quantize and c.repeated_blocks == [] and c.per_tensor_fallback
  assert c.components_to_quantize is None and c.precision_plan is None and not c.verbose
  assert QuantizeConfig(quant_type="FLOAT8_Weight_Only").quant_type == "float8_weight_only"
  assert QuantizeConfig(backend="ao").backend == QuantizeBackend.TORCHAO
  assert QuantizeConfig(backend="TorchAO").backend == QuantizeBackend.TORCHAO
  with pytest.raises(ValueError):
    QuantizeConfig(backend="tensorrt")
  with pytest.raises(ValueError):
    QuantizeBackend.is_supported(QuantizeBackend.NONE)
  with pytest.raises(NotImplementedError, match="not built"):
    QuantizeConfig(quant_type="svdq_int4_r32")
  a, b = QuantizeConfig(), QuantizeConfig()
  a.exclude_layers.append("x")
  assert "x" not in b.exclude_layers  # default list is not shared


def test_from_kwargs_update_strify_components():
  c = QuantizeConfig.from_kwargs(quant_type="float8_weight_only", exclude_layers=["a"], bogus=1,
                                 config=QuantizeConfig(quant_type="int8_per_row"))
  assert c.quant_type == "float8_weight_only" and c.exclude_layers == ["a"]
  # the `config=` keyword is not a field: dropped, defaults apply (a reference quirk)
  assert QuantizeConfig.from_kwargs(config=QuantizeConfig(quant_type="int8_per_row")).quant_type == \
      "float8_per_row"
  c.update(quant_type="FLOAT8_PER_ROW", verbose=None)
  assert c.quant_type == "float8_per_row" and c.verbose is False
  assert c.strify() == "float8_per_row"
  multi = QuantizeConfig(components_to_quantize={"transformer": {"quant_type": "float8_per_row"},
                                                 "text_encoder": {"quant_type": "float8_weight_only",
                                                                  "exclude_layers": ["shared"]}})
  assert multi.strify() == "<transformer:float8_per_row><text_encoder:float8_weight_only>"
  assert multi.component_quant_types() == {"transformer": "float8_per_row",
                                           "text_encoder": "float8_weight_only"}
  parts = QuantizeConfig.expand_configs(multi)
  assert [p.components_to_quantize for p in parts] == [["transformer"], ["text_encoder"]]
  assert parts[1].quant_type == "float8_weight_only" and parts[1].exclude_layers == ["shared"]
  lst = QuantizeConfig(components_to_quantize=["transformer", "vae"])
  assert lst.component_quant_types() == {"transformer": "float8_per_row", "vae": "float8_per_row"}
  assert len(QuantizeConfig.expand_configs(lst)) == 2 and QuantizeConfig.expand_configs(c) == [c]


def test_yaml_fixtures_of_the_reference():
  c = cache_dit.load_quantize_config(os.path.join(GOLD, "quantize.yaml"))
  assert c.quant_type == "float8_per_row" and c.exclude_layers == ["embedder", "embed"] and not c.verbose
  c = cache_dit.load_quantize_config(os.path.join(GOLD, "combined.yaml"))
  assert c.quant_type == "float8_per_row" and c.exclude_layers == ["embedder", "embed"]
  c = cache_dit.load_quantize_config(os.path.join(GOLD, "quantize_extra.yaml"))
  assert set(c.components_to_quantize) == {"transformer", "text_encoder_2"}
  assert c.component_quant_types()["text_encoder_2"] == "float8_weight_only"
  c = cache_dit.load_quantize_config(os.path.join(GOLD, "quantize_plan.yaml"))
  t = QuantizeConfig.expand_configs(c)[0]
  assert t.precision_plan["attn.to_k"] == "float8_weight_only" and t.regional_quantize
  assert t.exclude_layers == ["embedder", "embed", "mod", "modulation"]
  c = cache_dit.load_quantize_config(os.path.join(GOLD, "quantize_plan_tp.yaml"))
  assert QuantizeConfig.expand_configs(c)[0].per_tensor_fallback is True
  assert cache_dit.load_quantize_config({"cache_config": {}}) is None
  c = cache_dit.load_quantize_config({"quantize_config": {"quant_type": "float8_weight_only",
                                                          "unknown_key": 3, "verbose": None}})
  assert c.quant_type == "float8_weight_only" and c.verbose is False
  with pytest.raises(FileNotFoundError):
    cache_dit.load_quantize_config("/nonexistent.yaml")
  with pytest.raises(ValueError):
    cache_dit.load_quantize_config(42)


class _Blk(nn.Module):

  def __init__(self):
    super().__init__()
    self.to_q = nn.Linear(32, 32, dtype=torch.bfloat16)


class _Net(nn.Module):
  _repeated_blocks = ["_Blk"]

  def __init__(self):
    super().__init__()
    self.blocks = nn.ModuleList([_Blk(), _Blk()])


@pytest.fixture
def recording_convert(monkeypatch):
  """Routes quantize() through the real dispatch but records instead of converting,
  so the API can be exercised without a GPU."""
  calls = []
  real = policy.quantize_ao

  def fake(module, quantize_config, **kw):
    kw.pop("_convert_fn", None)
    return real(module, quantize_config, _convert_fn=lambda l, qt: calls.append(qt), **kw)

  monkeypatch.setattr(policy, "quantize_ao", fake)
  return calls


def test_quantize_call_forms(recording_convert):
  m = _Net()
  assert cache_dit.quantize(m, QuantizeConfig()) is m  # positional, in place
  assert recording_convert == ["float8_per_row"] * 2
  assert cache_dit.check_quantized(m) and m._quantize_type == "float8_per_row"
  assert isinstance(m._quantize_config, QuantizeConfig) and m.blocks[0].to_q._is_inner_quantized
  m2 = _Net()
  cache_dit.quantize(m2, quantize_config=QuantizeConfig(quant_type="float8_weight_only"))
  assert recording_convert[-1] == "float8_weight_only"
  m3 = _Net()  # legacy keyword form
  cache_dit.quantize(m3, quant_type="float8_weight_only", exclude_layers=[])
  assert m3._quantize_type == "float8_weight_only"
  m4 = _Net()  # `config=` is not a parameter: silently ignored, defaults apply
  cache_dit.quantize(m4, config=QuantizeConfig(quant_type="float8_weight_only"))
  assert m4._quantize_type == "float8_per_row"
  with pytest.raises(ValueError, match="quantize_config should be specified"):
    cache_dit.quantize(_Net())
  n = len(recording_convert)
  cache_dit.quantize(m, QuantizeConfig())  # already quantized: warning, nothing happens
  assert len(recording_convert) == n
  cache_dit.remove_quantization_stats(m)
  assert not cache_dit.check_quantized(m) and not hasattr(m, "_quantize_config")


def test_enable_cache_quantize_plumbing(recording_convert):

  class Pipe:
    pass

  p = Pipe()
  p.transformer, p.transformer_2, p.text_encoder = _Net(), _Net(), _Net()
  assert cache_dit.enable_cache(p, quantize_config=QuantizeConfig()) is p
  assert cache_dit.check_quantized(p.transformer) and cache_dit.check_quantized(p.transformer_2)
  assert not cache_dit.check_quantized(p.text_encoder) and cache_dit.check_quantized(p)
  p2 = Pipe()
  p2.transformer, p2.text_encoder = _Net(), _Net()
  cfg = QuantizeConfig(components_to_quantize={"transformer": {"quant_type": "float8_per_row"},
                                               "text_encoder": {"quant_type": "float8_weight_only"}})
  cache_dit.enable_cache(p2, quantize_config=cfg)
  assert p2.transformer._quantize_type == "float8_per_row"
  assert p2.text_encoder._quantize_type == "float8_weight_only"
  with pytest.raises(AssertionError, match="not found in"):
    cache_dit.enable_cache(p2, quantize_config=QuantizeConfig(components_to_quantize=["vae"]))
  bare = _Net()
  assert cache_dit.enable_cache(bare, quantize_config=QuantizeConfig()) is bare and bare._is_quantized
  with pytest.raises(AssertionError):
    cache_dit.enable_cache(_Net(), quantize_config={"quant_type": "float8_per_row"})
  with pytest.raises(NotImplementedError, match="caching"):
    cache_dit.enable_cache(p, cache_config=object())
  assert cache_dit.enable_cache(p) is p  # nothing to do


def test_no_silent_cpu_path():
  """Without a GPU the real conversion must refuse, not fall back."""
  if torch.cuda.is_available():
    pytest.skip("GPU present")
  with pytest.raises(AssertionError, match="only supported on GPU"):
    cache_dit.quantize(_Net(), QuantizeConfig())
  from cache_dit_amd import nn as cnn, ops
  with pytest.raises(RuntimeError, match="no CPU path"):
    cnn.convert_linear_(nn.Linear(32, 32, dtype=torch.bfloat16), "float8_per_row")
  with pytest.raises(RuntimeError, match="no CPU path"):
    ops.fp8_rowwise_quant(torch.zeros(2, 16, dtype=torch.bfloat16))
  with pytest.raises(NotImplementedError):
    torch.ops.cdit.fp8_rowwise_quant(torch.zeros(2, 16, dtype=torch.bfloat16), 0)
  with pytest.raises(NotImplementedError, match="not built"):
    cnn.convert_linear_(nn.Linear(32, 32, dtype=torch.bfloat16), "int8_per_row")
