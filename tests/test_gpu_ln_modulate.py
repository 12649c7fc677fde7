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
