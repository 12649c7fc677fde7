"""The quantizer fused into its producer (LayerNorm + AdaLN modulation + per-row FP8
quantization in one kernel): codes and scales bit-exact against the oracle's quantizer
on the kernel's own bf16 output; that output against the eager bf16 op sequence (a
floating-point kernel: fp32 statistics summed in another order, so a bf16 result may
land on the other side of a rounding boundary: on at most 0.1 % of the elements, and
there by no more than an ulp of the intermediate product); and the hand-over of the codes to the consuming Linears."""
import logging

import numpy as np
import pytest
import torch

from helpers import bits_u8, bits_u32, cosine
from oracle import torch_oracle as to

pytestmark = pytest.mark.gpu
logging.getLogger("CACHE_DIT_AMD").setLevel(logging.WARNING)


def _inputs(shape, nb, seed):
  g = torch.Generator().manual_seed(seed)
  K = shape[-1]
  x = (torch.randn(*shape, generator=g) * 2 + 0.3)
  x.view(-1, K)[:, torch.randperm(K, generator=g)[:max(1, K // 1000)]] *= 20
  mod_shape = (K,) if nb == 1 else (nb, 1, K)
  shift = torch.randn(*mod_shape, generator=g) * 0.5
  scale = torch.randn(*mod_shape, generator=g) * 0.3
  return x.to(torch.bfloat16), shift.to(torch.bfloat16), scale.to(torch.bfloat16)


def _check_y(y, y_ref, shift):
  a, b = y.float().cpu().numpy(), y_ref.float().numpy()
  differ = a != b
  assert differ.mean() <= 1e-3, differ.mean()
  # where they differ, the normalised value landed one bf16 ulp apart: that moves
  # u = n * (1 + scale) by an ulp of u (|u| <= |y| + |shift|), and u and y round once more
  sh = np.broadcast_to(shift.float().numpy(), b.shape)
  tol = (np.abs(b) + np.abs(sh)) * 2.0**-6 + 1e-30
  assert (np.abs(a - b) <= tol).all()


@pytest.mark.parametrize("mode", ["bf16div", "fp32div"])
@pytest.mark.parametrize("shape,nb", [((2, 77, 3072), 2), ((1, 4608, 3072), 1), ((3, 40, 5120), 3),
                                      ((5, 64), 1), ((2, 9, 100), 2), ((4, 3, 8200), 1),
                                      ((1, 7, 24576), 1)])
def test_fused_producer_quantizer_parity(shape, nb, mode):
  from cache_dit_amd import _native
  import cache_dit_amd.ops  # noqa: F401
  x, shift, scale = _inputs(shape, nb, seed=sum(shape))
  mode_id = _native.SCALE_MODE_IDS[mode]
  y, q, s = torch.ops.cdit.ln_modulate_quant(x.cuda(), shift.cuda(), scale.cuda(), 1e-6, mode_id, True)
  torch.cuda.synchronize()
  assert y.shape == x.shape and q.shape == x.shape and s.shape == (*shape[:-1], 1)
  _check_y(y, to.ln_modulate(x, shift, scale, 1e-6), shift)
  q_ref, s_ref = to.quantize_rowwise(y.cpu(), mode)
  assert (bits_u8(q) == bits_u8(q_ref)).all()
  assert (bits_u32(s) == bits_u32(s_ref)).all()
  # without the bf16 write: same codes and scales
  _, q2, s2 = torch.ops.cdit.ln_modulate_quant(x.cuda(), shift.cuda(), scale.cuda(), 1e-6, mode_id, False)
  assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2, s)


def test_strided_rows_zero_variance_and_errors():
  import cache_dit_amd.ops  # noqa: F401
  x, shift, scale = _inputs((6, 20, 640), 1, seed=1)
  xg = x.cuda()[:, :, :512]
  y, q, s = torch.ops.cdit.ln_modulate_quant(xg, shift[:512].cuda(), scale[:512].cuda())
  _check_y(y, to.ln_modulate(x[:, :, :512], shift[:512], scale[:512]), shift[:512])
  q_ref, s_ref = to.quantize_rowwise(y.cpu())
  assert (bits_u8(q) == bits_u8(q_ref)).all() and (bits_u32(s) == bits_u32(s_ref)).all()
  # constant rows: variance 0, normalised row 0, y = shift; zero shift too: scale 1, codes 0
  const = torch.full((3, 256), 7.0, dtype=torch.bfloat16, device="cuda")
  zero = torch.zeros(256, dtype=torch.bfloat16, device="cuda")
  y, q, s = torch.ops.cdit.ln_modulate_quant(const, zero, zero)
  assert (y == 0).all() and (bits_u8(q) & 0x7f == 0).all() and (s == 1).all()
  with pytest.raises(ValueError, match="bfloat16"):
    torch.ops.cdit.ln_modulate_quant(const.float(), zero, zero)
  with pytest.raises(ValueError, match="modulation vectors"):
    torch.ops.cdit.ln_modulate_quant(const.view(3, 1, 256), zero.repeat(2, 1), zero.repeat(2, 1))


@pytest.mark.parametrize("K", [512, 3072, 8200])
def test_rows_with_a_large_offset(K):
  """Rows whose mean is far larger than their spread (mean^2 > 4 var): E[x^2] - mean^2 would
  cancel, so the kernel recomputes the variance around the mean from its registers. Mixed
  with ordinary rows in one launch so that both paths run inside the same workgroups."""
  import cache_dit_amd.ops  # noqa: F401
  g = torch.Generator().manual_seed(K)
  x = torch.randn(96, K, generator=g)
  x[0::3] = x[0::3] + 3.0
  x[1::3] = x[1::3] * 3.0 - 11.0
  x[4] = torch.where(torch.arange(K) % 2 == 0, 128.0, 129.0)  # two adjacent bf16 values
  shift = (torch.randn(K, generator=g) * 0.5).to(torch.bfloat16)
  scale = (torch.randn(K, generator=g) * 0.3).to(torch.bfloat16)
  x = x.to(torch.bfloat16)
  y, q, s = torch.ops.cdit.ln_modulate_quant(x.cuda(), shift.cuda(), scale.cuda())
  torch.cuda.synchronize()
  _check_y(y, to.ln_modulate(x, shift, scale, 1e-6), shift)
  q_ref, s_ref = to.quantize_rowwise(y.cpu())
  assert (bits_u8(q) == bits_u8(q_ref)).all() and (bits_u32(s) == bits_u32(s_ref)).all()


def test_codes_are_handed_to_the_consuming_linears():
  """A FLUX-shaped model with the fused producer: the Linears fed by a modulated norm
  launch no quantizer of their own, the output stays within the cosine bar of the
  unfused model, and dropping the bf16 write changes nothing."""
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
  cache_dit.share_activation_quant_(model)
  with torch.no_grad():
    ops.quant_launches = 0
    y0 = model(**inputs)
    plain = ops.quant_launches
    assert ds.fuse_norm_quant(model) == 2 * 3 + 3 * 1  # per double block: norm1, norm1_context, the block
    ops.quant_launches = 0
    y1 = model(**inputs)
    fused = ops.quant_launches
    ds.fuse_norm_quant(model, materialize=False)
    y2 = model(**inputs)
  # per double block 4 modulated activations (attention and MLP inputs of both streams),
  # per single block 1: their consumers no longer quantize
  assert plain - fused == 2 * 4 + 3 * 1, (plain, fused)
  assert torch.isfinite(y1.float()).all() and cosine(y1, y0) >= 0.9999, cosine(y1, y0)
  assert torch.equal(y2, y1)
  with torch.inference_mode():  # no version counters: nothing handed over, still correct
    y3 = model(**inputs)
  assert cosine(y3, y0) >= 0.9999
  ds.fuse_norm_quant(model, False)
  cache_dit.share_activation_quant_(model, False)


def _codes_only_activation(M=64, K=512, seed=3):
  """y = ln_modulate_quant(..., materialize=False): its bf16 values are never written."""
  from cache_dit_amd import ops
  x, shift, scale = _inputs((1, M, K), 1, seed=seed)
  xg, sh, sc = x.cuda(), shift.cuda(), scale.cuda()
  y = ops.ln_modulate_quant(xg, sh, sc, materialize=False)
  want = ops.ln_modulate_quant(xg.clone(), sh, sc, materialize=True)
  return y, want


def _linear(quant_type, K=512, N=256, share=False):
  import cache_dit_amd as cache_dit
  from cache_dit_amd import nn as cnn
  torch.manual_seed(0)
  lin = torch.nn.Linear(K, N, dtype=torch.bfloat16).cuda()
  cnn.convert_linear_(lin, quant_type)
  if share:
    lin.share_input_quant = True
  return lin


def test_codes_only_activation_reaches_its_consumer_or_raises():
  """The tensor ln_modulate_quant(materialize=False) returns holds no values. A consumer
  that finds the delivered codes uses them; every consumer that would read the bf16
  values instead must raise, never quantize uninitialised memory."""
  from cache_dit_amd import ops
  assert torch.cuda.is_available()
  # the happy path: a sharing float8_per_row Linear, also through a reshaped view
  y, want = _codes_only_activation()
  assert ops.is_codes_only(y) and ops.is_codes_only(y.view(-1, y.shape[-1])[8:])
  lin = _linear("float8_per_row", share=True)
  assert torch.equal(lin(y), lin(want))
  assert torch.equal(lin(y.view(-1, y.shape[-1])), lin(want.view(-1, want.shape[-1])))
  # a Linear that does not share its input quantization
  y, _ = _codes_only_activation(seed=4)
  with pytest.raises(RuntimeError, match="materialize=True"):
    _linear("float8_per_row", share=False)(y)
  # weight-only and per-tensor Linears read the bf16 values
  with pytest.raises(RuntimeError, match="materialize=True"):
    _linear("float8_weight_only")(y)
  with pytest.raises(RuntimeError, match="materialize=True"):
    _linear("float8_per_tensor")(y)
  # a slice is another activation (other shape): not in the lookup, and it aliases the buffer
  with pytest.raises(RuntimeError, match="materialize=True"):
    _linear("float8_per_row", share=True)(y[:, :32])
  # the entry evicted by other quantizations on the stream
  y, _ = _codes_only_activation(seed=5)
  lin = _linear("float8_per_row", share=True)
  for i in range(ops._SHARED_QUANT_ENTRIES + 1):
    lin(torch.randn(8, 512, device="cuda").to(torch.bfloat16))
  with pytest.raises(RuntimeError, match="materialize=True"):
    lin(y)
  # a consumer on another stream
  y, _ = _codes_only_activation(seed=6)
  side = torch.cuda.Stream()
  side.wait_stream(torch.cuda.current_stream())
  with torch.cuda.stream(side), pytest.raises(RuntimeError, match="materialize=True"):
    lin(y)
  torch.cuda.current_stream().wait_stream(side)
  # written through PyTorch afterwards: an ordinary activation again
  y, _ = _codes_only_activation(seed=7)
  y.copy_(torch.ones_like(y))
  assert not ops.is_codes_only(y)
  out = _linear("float8_weight_only")(y)
  assert torch.isfinite(out.float()).all()
  # sibling groups: per-row members find the codes, weight-only members raise
  from cache_dit_amd import nn as cnn
  y, want = _codes_only_activation(seed=8)
  a, b = _linear("float8_per_row"), _linear("float8_per_row")
  g = cnn.SiblingGroup([a, b])
  a.sibling_group = b.sibling_group = g
  ya, yb = a(y), b(y)
  a.sibling_group = b.sibling_group = None
  a.share_input_quant = b.share_input_quant = True
  assert torch.equal(ya, a(want)) and torch.equal(yb, b(want))
  y, _ = _codes_only_activation(seed=9)
  a, b = _linear("float8_weight_only"), _linear("float8_weight_only")
  a.sibling_group = b.sibling_group = cnn.SiblingGroup([a, b])
  with pytest.raises(RuntimeError, match="materialize=True"):
    a(y)


def test_codes_only_is_never_produced_under_compile_or_inference_mode():
  """Where nothing can be handed over the bf16 values are written whatever the caller asked."""
  from cache_dit_amd import ops
  x, shift, scale = _inputs((1, 32, 512), 1, seed=11)
  xg, sh, sc = x.cuda(), shift.cuda(), scale.cuda()
  want = ops.ln_modulate_quant(xg, sh, sc, materialize=True)
  with torch.inference_mode():
    y = ops.ln_modulate_quant(xg, sh, sc, materialize=False)
  assert torch.equal(y, want) and not ops.is_codes_only(y)
  lin = _linear("float8_weight_only")

  def f(x):
    return lin(ops.ln_modulate_quant(x, sh, sc, materialize=False))

  try:
    got = torch.compile(f, fullgraph=False)(xg)
  except Exception as e:  # no Inductor back end on the box
    pytest.skip(f"torch.compile unavailable: {str(e)[:80]}")
  assert torch.equal(got, lin(want))


def test_rows_per_mod_beyond_the_row_count_means_one_vector():
  """The C entry point takes any count >= M for 'one modulation vector for every row'."""
  import ctypes
  from cache_dit_amd import _native
  x, shift, scale = _inputs((1, 40, 512), 1, seed=12)
  xg, sh, sc = x.cuda().view(40, 512), shift.cuda(), scale.cuda()
  L, stream = _native.load(), torch.cuda.current_stream().cuda_stream
  outs = []
  for rows_per_mod in (40, 1 << 32, (1 << 63) - 1):
    q = torch.empty(40, 512, dtype=torch.uint8, device="cuda")
    s = torch.empty(40, dtype=torch.float32, device="cuda")
    _native.check(L.cdit_fp8_ln_modulate_quant(xg.data_ptr(), 40, 512, 512, sh.data_ptr(), sc.data_ptr(),
                                               512, rows_per_mod, 1e-6, None, 512, q.data_ptr(), 512,
                                               s.data_ptr(), 0, stream))
    torch.cuda.synchronize()
    outs.append((q.cpu(), s.cpu()))
  for q, s in outs[1:]:
    assert torch.equal(q, outs[0][0]) and torch.equal(s, outs[0][1])
