"""Random-init transformers with the Linear shapes, layer names, token counts and
block dataflow of FLUX.1-dev, Qwen-Image and Wan2.1-14B, for benchmarks and
end-to-end tests (diffusers is not a dependency of this package, and no
checkpoint is loaded).

Layer names are the diffusers ones, because `exclude_layers` and the policy
match on them: e.g. `attn.to_q`, `ff.net.0.proj`, `proj_mlp`, `norm1.linear`
(reference: src/cache_dit/distributed/transformers/flux.py:93-147),
`img_mod.1` (qwen_image.py:119-134), `attn1.to_q`, `ffn.net.0.proj`
(wan.py:284-293). Each class sets `_repeated_blocks`, which regional
quantization keys off (src/cache_dit/quantization/torchao/quantize_ao.py:358-367).
Block dataflows follow src/cache_dit/caching/patch_functors/functor_flux.py:48-211,
functor_qwen_image_controlnet.py:43-217 and functor_wan_vace.py:40-246; RoPE
tables, timestep embedders and (un)patchify are simplified: only what feeds the
quantized Linears realistic, normalised inputs is kept.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F
from torch import nn

# ------------------------------------------------------------------------------- pieces


class RMSNorm(nn.Module):

  def __init__(self, dim: int, eps: float = 1e-6):
    super().__init__()
    self.eps = eps
    self.weight = nn.Parameter(torch.ones(dim))

  def forward(self, x):
    v = x.float()
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + self.eps)
    return (v * self.weight.float()).to(x.dtype)


class GELUProj(nn.Module):
  """diffusers' `GELU` activation block: a Linear named `proj` followed by
  GELU(tanh); sits at `net.0` of a FeedForward."""

  def __init__(self, dim_in: int, dim_out: int):
    super().__init__()
    self.proj = nn.Linear(dim_in, dim_out)
    self.act = nn.GELU(approximate="tanh")

  def forward(self, x):
    return self.act(self.proj(x))


class FeedForward(nn.Module):

  def __init__(self, dim: int, inner: int):
    super().__init__()
    self.net = nn.ModuleList([GELUProj(dim, inner), nn.Dropout(0.0), nn.Linear(inner, dim)])

  def forward(self, x):
    for m in self.net:
      x = m(x)
    return x


def rope_table(seq: int, head_dim: int, device=None) -> torch.Tensor:
  """[seq, head_dim] interleaved (cos, sin) angles; a 1-D stand-in for the models'
  multi-axis tables."""
  pos = torch.arange(seq, dtype=torch.float32, device=device)
  freq = torch.exp(-math.log(10000.0) * torch.arange(0, head_dim, 2, device=device).float() /
                   head_dim)
  ang = pos[:, None] * freq[None, :]
  return torch.stack([ang.cos(), ang.sin()], dim=-1).reshape(seq, head_dim)


def apply_rope(x: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
  """x [B, H, S, D]; rotates interleaved pairs."""
  cos, sin = table[..., 0::2], table[..., 1::2]
  xf = x.float()
  a, b = xf[..., 0::2], xf[..., 1::2]
  out = torch.stack([a * cos - b * sin, a * sin + b * cos], dim=-1).flatten(-2)
  return out.to(x.dtype)


def _heads(x, n):
  b, s, _ = x.shape
  return x.view(b, s, n, -1).transpose(1, 2)


def _merge(x):
  b, h, s, d = x.shape
  return x.transpose(1, 2).reshape(b, s, h * d)


def _ln(x, eps=1e-6):
  return F.layer_norm(x.float(), (x.shape[-1], ), eps=eps).to(x.dtype)


class _ModulatedNorm:
  """Mixin of the modules that compute `layer_norm(x) * (1 + scale) + shift` for quantized
  Linears. With `fused_norm_quant` set (see fuse_norm_quant) the expression runs as one
  HIP kernel that also delivers the FP8 codes to those Linears."""
  fused_norm_quant = False
  fused_norm_materialize = True

  def _modulated(self, x, shift, scale):
    if self.fused_norm_quant and x.is_cuda:
      from .. import ops
      return ops.ln_modulate_quant(x, shift, scale, eps=1e-6,
                                   materialize=self.fused_norm_materialize)
    return _ln(x) * (1 + scale) + shift


class TimeEmbed(nn.Module):
  """timestep (+ pooled text) -> conditioning vector; names contain `embed`, so the
  default exclude list leaves these Linears alone when quantizing the whole model."""

  def __init__(self, dim: int, pooled_dim: Optional[int] = None):
    super().__init__()
    self.timestep_embedder = nn.Sequential(nn.Linear(256, dim), nn.SiLU(), nn.Linear(dim, dim))
    self.text_embedder = (nn.Sequential(nn.Linear(pooled_dim, dim), nn.SiLU(), nn.Linear(dim, dim))
                          if pooled_dim else None)

  def forward(self, timestep, pooled=None):
    half = 128
    freqs = torch.exp(-math.log(10000.0) * torch.arange(half, device=timestep.device) / half)
    ang = timestep.float()[:, None] * 1000.0 * freqs[None, :]
    emb = torch.cat([ang.cos(), ang.sin()], dim=-1).to(self.timestep_embedder[0].weight.dtype)
    out = self.timestep_embedder(emb)
    if self.text_embedder is not None and pooled is not None:
      out = out + self.text_embedder(pooled)
    return out


# ------------------------------------------------------------------------------- FLUX


class AdaLayerNormZero(_ModulatedNorm, nn.Module):

  def __init__(self, dim: int, chunks: int):
    super().__init__()
    self.chunks = chunks
    self.linear = nn.Linear(dim, chunks * dim)

  def forward(self, x, temb):
    mods = self.linear(F.silu(temb)).unsqueeze(1).chunk(self.chunks, dim=-1)
    shift, scale = mods[0], mods[1]
    return self._modulated(x, shift, scale), mods[2:]


def _batch(pairs):
  from ..nn import linear_batch
  return linear_batch(pairs)


def _ff_pair(ff_a: "FeedForward", xa, ff_b: "FeedForward", xb):
  """Two FeedForwards on independent inputs, their Linears launched pairwise."""
  (ha, ), (hb, ) = _batch([(xa, [ff_a.net[0].proj]), (xb, [ff_b.net[0].proj])])
  ha, hb = ff_a.net[0].act(ha), ff_b.net[0].act(hb)  # identity once fused into the epilogue
  (ya, ), (yb, ) = _batch([(ha, [ff_a.net[2]]), (hb, [ff_b.net[2]])])
  return ya, yb


class FluxAttention(nn.Module):
  batch_streams = False  # see batch_streams(): image- and text-stream Linears in one launch

  def __init__(self, dim: int, heads: int, joint: bool):
    super().__init__()
    self.heads = heads
    hd = dim // heads
    self.to_q, self.to_k, self.to_v = nn.Linear(dim, dim), nn.Linear(dim, dim), nn.Linear(dim, dim)
    self.norm_q, self.norm_k = RMSNorm(hd), RMSNorm(hd)
    self.joint = joint
    if joint:
      self.to_out = nn.ModuleList([nn.Linear(dim, dim), nn.Dropout(0.0)])
      self.add_q_proj, self.add_k_proj, self.add_v_proj = (nn.Linear(dim, dim), nn.Linear(dim, dim),
                                                           nn.Linear(dim, dim))
      self.norm_added_q, self.norm_added_k = RMSNorm(hd), RMSNorm(hd)
      self.to_add_out = nn.Linear(dim, dim)

  def forward(self, hidden, encoder=None, rope=None, qkv=None):
    if qkv is not None:  # computed by the caller together with other Linears on `hidden`
      q, k, v = qkv
    elif self.joint and self.batch_streams:
      (q, k, v), (eq, ek, ev) = _batch([(hidden, [self.to_q, self.to_k, self.to_v]),
                                        (encoder, [self.add_q_proj, self.add_k_proj, self.add_v_proj])])
    else:
      q, k, v = self.to_q(hidden), self.to_k(hidden), self.to_v(hidden)
      if self.joint:
        eq, ek, ev = self.add_q_proj(encoder), self.add_k_proj(encoder), self.add_v_proj(encoder)
    q = self.norm_q(_heads(q, self.heads))
    k = self.norm_k(_heads(k, self.heads))
    v = _heads(v, self.heads)
    if self.joint:
      eq = self.norm_added_q(_heads(eq, self.heads))
      ek = self.norm_added_k(_heads(ek, self.heads))
      ev = _heads(ev, self.heads)
      q, k, v = torch.cat([eq, q], 2), torch.cat([ek, k], 2), torch.cat([ev, v], 2)
    if rope is not None:
      q, k = apply_rope(q, rope), apply_rope(k, rope)
    o = _merge(F.scaled_dot_product_attention(q, k, v))
    if not self.joint:
      return o
    n_txt = encoder.shape[1]
    if self.batch_streams:
      (a, ), (ca, ) = _batch([(o[:, n_txt:], [self.to_out[0]]), (o[:, :n_txt], [self.to_add_out])])
      return self.to_out[1](a), ca
    return self.to_out[1](self.to_out[0](o[:, n_txt:])), self.to_add_out(o[:, :n_txt])


class FluxTransformerBlock(_ModulatedNorm, nn.Module):
  """Double-stream block: 14 Linears (7 per stream)."""

  def __init__(self, dim: int, heads: int, mlp: int):
    super().__init__()
    self.norm1, self.norm1_context = AdaLayerNormZero(dim, 6), AdaLayerNormZero(dim, 6)
    self.attn = FluxAttention(dim, heads, joint=True)
    self.ff, self.ff_context = FeedForward(dim, mlp), FeedForward(dim, mlp)

  def forward(self, hidden, encoder, temb, rope):
    nh, (gate_msa, shift_mlp, scale_mlp, gate_mlp) = self.norm1(hidden, temb)
    ne, (c_gate_msa, c_shift_mlp, c_scale_mlp, c_gate_mlp) = self.norm1_context(encoder, temb)
    a, ca = self.attn(nh, ne, rope)
    hidden = hidden + gate_msa * a
    encoder = encoder + c_gate_msa * ca
    if self.attn.batch_streams:
      f, cf = _ff_pair(self.ff, self._modulated(hidden, shift_mlp, scale_mlp), self.ff_context,
                       self._modulated(encoder, c_shift_mlp, c_scale_mlp))
    else:
      f = self.ff(self._modulated(hidden, shift_mlp, scale_mlp))
      cf = self.ff_context(self._modulated(encoder, c_shift_mlp, c_scale_mlp))
    hidden = hidden + gate_mlp * f
    encoder = encoder + c_gate_mlp * cf
    return encoder, hidden


class FluxSingleTransformerBlock(nn.Module):
  """Single-stream block: 6 Linears; `proj_mlp` is followed by GELU(tanh)."""

  def __init__(self, dim: int, heads: int, mlp: int):
    super().__init__()
    self.norm = AdaLayerNormZero(dim, 3)
    self.proj_mlp = nn.Linear(dim, mlp)
    self.act_mlp = nn.GELU(approximate="tanh")
    self.attn = FluxAttention(dim, heads, joint=False)
    self.proj_out = nn.Linear(dim + mlp, dim)
    self.fuse_cat = False  # fuse_cat_quant: proj_out quantizes [attn | mlp] without the copy
    self.batch_siblings = False  # batch_streams(single_blocks=True): proj_mlp + q/k/v in one launch

  def forward(self, hidden, temb, rope):
    normed, (gate, ) = self.norm(hidden, temb)
    if self.batch_siblings:
      (mlp, q, k, v), = _batch([(normed, [self.proj_mlp, self.attn.to_q, self.attn.to_k,
                                          self.attn.to_v])])
      mlp = self.act_mlp(mlp)
      attn = self.attn(normed, rope=rope, qkv=(q, k, v))
    else:
      mlp = self.act_mlp(self.proj_mlp(normed))
      attn = self.attn(normed, rope=rope)
    if self.fuse_cat:
      from ..nn import linear_on_cat
      return hidden + gate * linear_on_cat(self.proj_out, [attn, mlp])
    return hidden + gate * self.proj_out(torch.cat([attn, mlp], dim=2))


class FluxLikeTransformer(nn.Module):
  _repeated_blocks = ["FluxTransformerBlock", "FluxSingleTransformerBlock"]

  def __init__(self, dim=3072, heads=24, mlp=12288, n_double=19, n_single=38, in_channels=64,
               text_dim=4096, pooled_dim=768):
    super().__init__()
    self.dim, self.heads = dim, heads
    self.x_embedder = nn.Linear(in_channels, dim)
    self.context_embedder = nn.Linear(text_dim, dim)
    self.time_text_embed = TimeEmbed(dim, pooled_dim)
    self.transformer_blocks = nn.ModuleList(
        [FluxTransformerBlock(dim, heads, mlp) for _ in range(n_double)])
    self.single_transformer_blocks = nn.ModuleList(
        [FluxSingleTransformerBlock(dim, heads, mlp) for _ in range(n_single)])
    self.norm_out = AdaLayerNormZero(dim, 2)
    self.proj_out = nn.Linear(dim, in_channels)

  def forward(self, hidden_states, encoder_hidden_states, pooled_projections, timestep):
    hidden = self.x_embedder(hidden_states)
    encoder = self.context_embedder(encoder_hidden_states)
    temb = self.time_text_embed(timestep, pooled_projections)
    n_txt, n_img = encoder.shape[1], hidden.shape[1]
    rope = rope_table(n_txt + n_img, self.dim // self.heads, hidden.device)
    for blk in self.transformer_blocks:
      encoder, hidden = blk(hidden, encoder, temb, rope)
    hidden = torch.cat([encoder, hidden], dim=1)
    for blk in self.single_transformer_blocks:
      hidden = blk(hidden, temb, rope)
    hidden = hidden[:, n_txt:]
    hidden, _ = self.norm_out(hidden, temb)
    return self.proj_out(hidden)


def flux_like_inputs(device, n_img=4096, n_txt=512, in_channels=64, text_dim=4096, pooled_dim=768,
                     seed=0, dtype=torch.bfloat16):
  g = torch.Generator().manual_seed(seed)
  return {
      "hidden_states": torch.randn(1, n_img, in_channels, generator=g).to(dtype).to(device),
      "encoder_hidden_states": torch.randn(1, n_txt, text_dim, generator=g).to(dtype).to(device),
      "pooled_projections": torch.randn(1, pooled_dim, generator=g).to(dtype).to(device),
      "timestep": torch.tensor([0.5], device=device),
  }


# ------------------------------------------------------------------------------- Qwen-Image


class QwenImageTransformerBlock(_ModulatedNorm, nn.Module):
  """12 quantized Linears + `img_mod.1` / `txt_mod.1`, which the default exclude
  pattern "mod" skips."""

  def __init__(self, dim: int, heads: int, mlp: int):
    super().__init__()
    self.img_mod = nn.Sequential(nn.SiLU(), nn.Linear(dim, 6 * dim))
    self.txt_mod = nn.Sequential(nn.SiLU(), nn.Linear(dim, 6 * dim))
    self.attn = FluxAttention(dim, heads, joint=True)
    self.img_mlp, self.txt_mlp = FeedForward(dim, mlp), FeedForward(dim, mlp)

  def _modulate(self, x, shift, scale):
    return self._modulated(x, shift, scale)

  def forward(self, hidden, encoder, temb, rope):
    i1, i2 = self.img_mod(temb).unsqueeze(1).chunk(2, dim=-1)
    t1, t2 = self.txt_mod(temb).unsqueeze(1).chunk(2, dim=-1)
    (si1, sc1, g1), (si2, sc2, g2) = i1.chunk(3, dim=-1), i2.chunk(3, dim=-1)
    (ti1, tc1, tg1), (ti2, tc2, tg2) = t1.chunk(3, dim=-1), t2.chunk(3, dim=-1)
    a, ca = self.attn(self._modulate(hidden, si1, sc1), self._modulate(encoder, ti1, tc1), rope)
    hidden = hidden + g1 * a
    encoder = encoder + tg1 * ca
    if self.attn.batch_streams:
      f, cf = _ff_pair(self.img_mlp, self._modulate(hidden, si2, sc2), self.txt_mlp,
                       self._modulate(encoder, ti2, tc2))
    else:
      f = self.img_mlp(self._modulate(hidden, si2, sc2))
      cf = self.txt_mlp(self._modulate(encoder, ti2, tc2))
    hidden = hidden + g2 * f
    encoder = encoder + tg2 * cf
    return encoder, hidden


class QwenImageLikeTransformer(nn.Module):
  _repeated_blocks = ["QwenImageTransformerBlock"]

  def __init__(self, dim=3072, heads=24, mlp=12288, n_layers=60, in_channels=64, text_dim=3584):
    super().__init__()
    self.dim, self.heads = dim, heads
    self.img_in = nn.Linear(in_channels, dim)
    self.txt_norm = RMSNorm(text_dim)
    self.txt_in = nn.Linear(text_dim, dim)
    self.time_text_embed = TimeEmbed(dim)
    self.transformer_blocks = nn.ModuleList(
        [QwenImageTransformerBlock(dim, heads, mlp) for _ in range(n_layers)])
    self.norm_out = AdaLayerNormZero(dim, 2)
    self.proj_out = nn.Linear(dim, in_channels)

  def forward(self, hidden_states, encoder_hidden_states, timestep):
    hidden = self.img_in(hidden_states)
    encoder = self.txt_in(self.txt_norm(encoder_hidden_states))
    temb = self.time_text_embed(timestep)
    rope = rope_table(encoder.shape[1] + hidden.shape[1], self.dim // self.heads, hidden.device)
    for blk in self.transformer_blocks:
      encoder, hidden = blk(hidden, encoder, temb, rope)
    hidden, _ = self.norm_out(hidden, temb)
    return self.proj_out(hidden)


def qwen_image_like_inputs(device, n_img=6889, n_txt=256, in_channels=64, text_dim=3584, seed=0,
                           dtype=torch.bfloat16):
  g = torch.Generator().manual_seed(seed)
  return {
      "hidden_states": torch.randn(1, n_img, in_channels, generator=g).to(dtype).to(device),
      "encoder_hidden_states": torch.randn(1, n_txt, text_dim, generator=g).to(dtype).to(device),
      "timestep": torch.tensor([0.5], device=device),
  }


# ------------------------------------------------------------------------------- Wan


class WanAttention(nn.Module):

  def __init__(self, dim: int, heads: int):
    super().__init__()
    self.heads = heads
    self.to_q, self.to_k, self.to_v = nn.Linear(dim, dim), nn.Linear(dim, dim), nn.Linear(dim, dim)
    self.to_out = nn.ModuleList([nn.Linear(dim, dim), nn.Dropout(0.0)])
    self.norm_q, self.norm_k = RMSNorm(dim), RMSNorm(dim)  # full width, before the head split

  def forward(self, hidden, context=None, rope=None):
    src = hidden if context is None else context
    q = _heads(self.norm_q(self.to_q(hidden)), self.heads)
    k = _heads(self.norm_k(self.to_k(src)), self.heads)
    v = _heads(self.to_v(src), self.heads)
    if rope is not None:
      q, k = apply_rope(q, rope), apply_rope(k, rope)
    o = _merge(F.scaled_dot_product_attention(q, k, v))
    return self.to_out[1](self.to_out[0](o))


class WanTransformerBlock(_ModulatedNorm, nn.Module):
  """10 Linears: self-attention, cross-attention to the text, GELU-tanh FFN."""

  def __init__(self, dim: int, heads: int, ffn: int):
    super().__init__()
    self.attn1, self.attn2 = WanAttention(dim, heads), WanAttention(dim, heads)
    self.norm2 = nn.LayerNorm(dim, eps=1e-6)
    self.ffn = FeedForward(dim, ffn)
    self.scale_shift_table = nn.Parameter(torch.randn(1, 6, dim) / dim**0.5)

  def forward(self, hidden, context, temb6, rope):
    sh1, sc1, g1, sh2, sc2, g2 = (self.scale_shift_table + temb6).chunk(6, dim=1)
    hidden = hidden + g1 * self.attn1(self._modulated(hidden, sh1, sc1), rope=rope)
    hidden = hidden + self.attn2(self.norm2(hidden), context)
    return hidden + g2 * self.ffn(self._modulated(hidden, sh2, sc2))


class WanLikeTransformer(nn.Module):
  _repeated_blocks = ["WanTransformerBlock"]

  def __init__(self, dim=5120, heads=40, ffn=13824, n_layers=40, in_channels=64, text_dim=4096):
    super().__init__()
    self.dim, self.heads = dim, heads
    self.patch_embedding = nn.Linear(in_channels, dim)  # stands in for the Conv3d patchifier
    self.condition_embedder = nn.ModuleDict({
        "time_embedder": TimeEmbed(dim),
        "time_proj": nn.Linear(dim, 6 * dim),
        "text_embedder": nn.Sequential(nn.Linear(text_dim, dim), nn.GELU(approximate="tanh"),
                                       nn.Linear(dim, dim)),
    })
    self.blocks = nn.ModuleList([WanTransformerBlock(dim, heads, ffn) for _ in range(n_layers)])
    self.proj_out = nn.Linear(dim, in_channels)

  def forward(self, hidden_states, encoder_hidden_states, timestep):
    hidden = self.patch_embedding(hidden_states)
    temb = self.condition_embedder["time_embedder"](timestep)
    temb6 = self.condition_embedder["time_proj"](F.silu(temb)).view(-1, 6, self.dim)
    context = self.condition_embedder["text_embedder"](encoder_hidden_states)
    rope = rope_table(hidden.shape[1], self.dim // self.heads, hidden.device)
    for blk in self.blocks:
      hidden = blk(hidden, context, temb6, rope)
    return self.proj_out(_ln(hidden))


def wan_like_inputs(device, n_tokens=32760, n_txt=512, in_channels=64, text_dim=4096, seed=0,
                    dtype=torch.bfloat16):
  g = torch.Generator().manual_seed(seed)
  return {
      "hidden_states": torch.randn(1, n_tokens, in_channels, generator=g).to(dtype).to(device),
      "encoder_hidden_states": torch.randn(1, n_txt, text_dim, generator=g).to(dtype).to(device),
      "timestep": torch.tensor([0.5], device=device),
  }


# ------------------------------------------------------------------------------- helpers


def fuse_gelu_epilogues(model: nn.Module) -> int:
  """Moves every GELU(tanh) that directly follows a quantized Linear (`GELUProj.act`
  after `proj`, `act_mlp` after `proj_mlp`) into that Linear's epilogue. Returns
  the number of fused pairs."""
  from ..nn import _Fp8LinearBase, fuse_gelu_tanh_

  n = 0
  for m in model.modules():
    pairs = []
    if isinstance(m, GELUProj):
      pairs.append((m.proj, m.act))
    if isinstance(m, FluxSingleTransformerBlock):
      pairs.append((m.proj_mlp, m.act_mlp))
    for lin, act in pairs:
      if isinstance(lin, _Fp8LinearBase) and not getattr(act, "_cdit_fused_into_linear", False):
        fuse_gelu_tanh_(lin, act)
        n += 1
  return n


def batch_streams(model: nn.Module, enable: bool = True, single_blocks: bool = False) -> int:
  """Switches the double-stream blocks of `model` (FLUX, Qwen-Image) to forwards that hand
  the image-stream and the text-stream Linears of a stage to linear_batch: one GEMM launch
  per stage instead of one per Linear, the small text-stream GEMMs riding along with the
  large image-stream ones. single_blocks=True does the same for proj_mlp + q/k/v of FLUX
  single blocks (in eager code group_sibling_linears_ finds those by itself; a compiled
  graph needs the explicit call). Outputs are bit-identical. Returns the number of
  double-stream attention modules switched."""
  n = 0
  for m in model.modules():
    if isinstance(m, FluxAttention) and m.joint:
      m.batch_streams = bool(enable)
      n += 1
    if isinstance(m, FluxSingleTransformerBlock):
      m.batch_siblings = bool(enable) and single_blocks
  return n


def fuse_cat_quant(model: nn.Module, enable: bool = True) -> int:
  """Switches the single-stream blocks of `model` to `linear_on_cat`: proj_out's quantizer
  reads the attention output and the MLP activation in place instead of their torch.cat
  copy. Outputs are bit-identical. Returns the number of blocks switched."""
  n = 0
  for m in model.modules():
    if isinstance(m, FluxSingleTransformerBlock):
      m.fuse_cat = bool(enable)
      n += 1
  return n


def fuse_norm_quant(model: nn.Module, enable: bool = True, materialize: bool = True) -> int:
  """Switches every modulated LayerNorm of `model` to the kernel that also quantizes
  (ops.ln_modulate_quant). Pair it with share_activation_quant_ on the Linears so that
  they pick the delivered codes up. materialize=False also drops the bf16 write of the
  modulated activation: valid here because only quantized Linears read it. Returns the
  number of modules switched."""
  n = 0
  blocks = getattr(model, "_repeated_blocks", [])
  for blk in model.modules():
    if type(blk).__name__ not in blocks:
      continue  # outside the repeated blocks (norm_out) the consumer is an unquantized Linear
    for m in blk.modules():
      if isinstance(m, _ModulatedNorm):
        m.fused_norm_quant = bool(enable)
        m.fused_norm_materialize = bool(materialize)
        n += 1
  return n


def count_linears(model: nn.Module):
  total = sum(isinstance(m, nn.Linear) for m in model.modules())
  quantized = sum(bool(getattr(m, "_is_inner_quantized", False)) for m in model.modules())
  return total, quantized
