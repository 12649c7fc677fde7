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
# Module attributes, forward signatures and return conventions are those of diffusers'
# FluxTransformer2DModel blocks (the block forwards the reference adapts in
# src/cache_dit/caching/patch_functors/functor_flux.py:48-80), so that code written against a
# diffusers block -- the stage patchers of cache_dit_amd.patch_functors -- runs on these.


class AdaLayerNormZero(nn.Module):
  """diffusers' AdaLayerNormZero as FLUX uses it: `forward(x, emb=temb)` returns the modulated
  norm and (gate_msa, shift_mlp, scale_mlp, gate_mlp)."""

  def __init__(self, dim: int):
    super().__init__()
    self.silu = nn.SiLU()
    self.linear = nn.Linear(dim, 6 * dim)
    self.norm = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)

  def forward(self, x, timestep=None, class_labels=None, hidden_dtype=None, emb=None):
    emb = self.linear(self.silu(emb))
    shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = emb.chunk(6, dim=1)
    x = self.norm(x) * (1 + scale_msa[:, None]) + shift_msa[:, None]
    return x, gate_msa, shift_mlp, scale_mlp, gate_mlp


class AdaLayerNormZeroSingle(nn.Module):
  """diffusers' AdaLayerNormZeroSingle: `forward(x, emb=temb)` -> (modulated norm, gate)."""

  def __init__(self, dim: int):
    super().__init__()
    self.silu = nn.SiLU()
    self.linear = nn.Linear(dim, 3 * dim)
    self.norm = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)

  def forward(self, x, emb=None):
    emb = self.linear(self.silu(emb))
    shift_msa, scale_msa, gate_msa = emb.chunk(3, dim=1)
    x = self.norm(x) * (1 + scale_msa[:, None]) + shift_msa[:, None]
    return x, gate_msa


class AdaLayerNormContinuous(nn.Module):
  """diffusers' AdaLayerNormContinuous (norm_out): scale first, then shift."""

  def __init__(self, dim: int):
    super().__init__()
    self.silu = nn.SiLU()
    self.linear = nn.Linear(dim, 2 * dim)
    self.norm = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)

  def forward(self, x, conditioning_embedding):
    emb = self.linear(self.silu(conditioning_embedding).to(x.dtype))
    scale, shift = emb.chunk(2, dim=1)
    return self.norm(x) * (1 + scale)[:, None, :] + shift[:, None, :]


class FluxAttention(nn.Module):
  """Joint (added_kv) or plain self-attention with per-head RMS norms of q and k; text
  tokens first. `forward(hidden_states, encoder_hidden_states=None, image_rotary_emb=None)`
  returns (image part, text part) for joint attention, one tensor otherwise."""

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

  def forward(self, hidden_states, encoder_hidden_states=None, image_rotary_emb=None, **kwargs):
    q, k, v = self.to_q(hidden_states), self.to_k(hidden_states), self.to_v(hidden_states)
    q = self.norm_q(_heads(q, self.heads))
    k = self.norm_k(_heads(k, self.heads))
    v = _heads(v, self.heads)
    if self.joint:
      eq = self.add_q_proj(encoder_hidden_states)
      ek = self.add_k_proj(encoder_hidden_states)
      ev = self.add_v_proj(encoder_hidden_states)
      eq = self.norm_added_q(_heads(eq, self.heads))
      ek = self.norm_added_k(_heads(ek, self.heads))
      ev = _heads(ev, self.heads)
      q, k, v = torch.cat([eq, q], 2), torch.cat([ek, k], 2), torch.cat([ev, v], 2)
    if image_rotary_emb is not None:
      q, k = apply_rope(q, image_rotary_emb), apply_rope(k, image_rotary_emb)
    o = _merge(F.scaled_dot_product_attention(q, k, v))
    if not self.joint:
      return o
    n_txt = encoder_hidden_states.shape[1]
    encoder_part, hidden_part = o.split_with_sizes([n_txt, o.shape[1] - n_txt], dim=1)
    hidden_part = self.to_out[1](self.to_out[0](hidden_part))
    return hidden_part, self.to_add_out(encoder_part)


class FluxTransformerBlock(nn.Module):
  """Double-stream block: 14 Linears (7 per stream)."""

  def __init__(self, dim: int, heads: int, mlp: int):
    super().__init__()
    self.norm1, self.norm1_context = AdaLayerNormZero(dim), AdaLayerNormZero(dim)
    self.attn = FluxAttention(dim, heads, joint=True)
    self.norm2 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
    self.ff = FeedForward(dim, mlp)
    self.norm2_context = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
    self.ff_context = FeedForward(dim, mlp)

  def forward(self, hidden_states, encoder_hidden_states, temb, image_rotary_emb=None,
              joint_attention_kwargs=None):
    norm_hidden_states, gate_msa, shift_mlp, scale_mlp, gate_mlp = self.norm1(hidden_states, emb=temb)
    norm_encoder_hidden_states, c_gate_msa, c_shift_mlp, c_scale_mlp, c_gate_mlp = self.norm1_context(
        encoder_hidden_states, emb=temb)
    attn_output, context_attn_output = self.attn(hidden_states=norm_hidden_states,
                                                 encoder_hidden_states=norm_encoder_hidden_states,
                                                 image_rotary_emb=image_rotary_emb,
                                                 **(joint_attention_kwargs or {}))
    hidden_states = hidden_states + gate_msa.unsqueeze(1) * attn_output
    norm_hidden_states = self.norm2(hidden_states)
    norm_hidden_states = norm_hidden_states * (1 + scale_mlp[:, None]) + shift_mlp[:, None]
    hidden_states = hidden_states + gate_mlp.unsqueeze(1) * self.ff(norm_hidden_states)
    encoder_hidden_states = encoder_hidden_states + c_gate_msa.unsqueeze(1) * context_attn_output
    norm_encoder_hidden_states = self.norm2_context(encoder_hidden_states)
    norm_encoder_hidden_states = norm_encoder_hidden_states * (1 + c_scale_mlp[:, None]) + c_shift_mlp[:, None]
    encoder_hidden_states = encoder_hidden_states + c_gate_mlp.unsqueeze(1) * self.ff_context(
        norm_encoder_hidden_states)
    return encoder_hidden_states, hidden_states


class FluxSingleTransformerBlock(nn.Module):
  """Single-stream block on the concatenated [text | image] tokens: 6 Linears; `proj_mlp` is
  followed by GELU(tanh)."""

  def __init__(self, dim: int, heads: int, mlp: int):
    super().__init__()
    self.norm = AdaLayerNormZeroSingle(dim)
    self.proj_mlp = nn.Linear(dim, mlp)
    self.act_mlp = nn.GELU(approximate="tanh")
    self.attn = FluxAttention(dim, heads, joint=False)
    self.proj_out = nn.Linear(dim + mlp, dim)

  def forward(self, hidden_states, temb, image_rotary_emb=None, joint_attention_kwargs=None):
    residual = hidden_states
    norm_hidden_states, gate = self.norm(hidden_states, emb=temb)
    mlp_hidden_states = self.act_mlp(self.proj_mlp(norm_hidden_states))
    attn_output = self.attn(hidden_states=norm_hidden_states, image_rotary_emb=image_rotary_emb,
                            **(joint_attention_kwargs or {}))
    hidden_states = torch.cat([attn_output, mlp_hidden_states], dim=2)
    return residual + gate.unsqueeze(1) * self.proj_out(hidden_states)


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
    self.norm_out = AdaLayerNormContinuous(dim)
    self.proj_out = nn.Linear(dim, in_channels)

  def forward(self, hidden_states, encoder_hidden_states, pooled_projections, timestep):
    hidden = self.x_embedder(hidden_states)
    encoder = self.context_embedder(encoder_hidden_states)
    temb = self.time_text_embed(timestep, pooled_projections)
    n_txt, n_img = encoder.shape[1], hidden.shape[1]
    rope = rope_table(n_txt + n_img, self.dim // self.heads, hidden.device)
    for blk in self.transformer_blocks:
      encoder, hidden = blk(hidden_states=hidden, encoder_hidden_states=encoder, temb=temb,
                            image_rotary_emb=rope)
    hidden = torch.cat([encoder, hidden], dim=1)
    for blk in self.single_transformer_blocks:
      hidden = blk(hidden_states=hidden, temb=temb, image_rotary_emb=rope)
    hidden = hidden[:, n_txt:]
    hidden = self.norm_out(hidden, temb)
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


class QwenImageTransformerBlock(nn.Module):
  """12 quantized Linears + `img_mod.1` / `txt_mod.1`, which the default exclude pattern
  "mod" skips. Attributes, `_modulate` and the forward signature follow diffusers'
  QwenImageTransformerBlock (the block the reference adapts in
  src/cache_dit/caching/patch_functors/functor_qwen_image_controlnet.py:43-117)."""

  def __init__(self, dim: int, heads: int, mlp: int):
    super().__init__()
    self.img_mod = nn.Sequential(nn.SiLU(), nn.Linear(dim, 6 * dim))
    self.img_norm1 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
    self.attn = FluxAttention(dim, heads, joint=True)
    self.img_norm2 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
    self.img_mlp = FeedForward(dim, mlp)
    self.txt_mod = nn.Sequential(nn.SiLU(), nn.Linear(dim, 6 * dim))
    self.txt_norm1 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
    self.txt_norm2 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
    self.txt_mlp = FeedForward(dim, mlp)

  def _modulate(self, x, mod_params):
    shift, scale, gate = mod_params.chunk(3, dim=-1)
    return x * (1 + scale.unsqueeze(1)) + shift.unsqueeze(1), gate.unsqueeze(1)

  def forward(self, hidden_states, encoder_hidden_states, encoder_hidden_states_mask=None, temb=None,
              image_rotary_emb=None, joint_attention_kwargs=None):
    img_mod1, img_mod2 = self.img_mod(temb).chunk(2, dim=-1)
    txt_mod1, txt_mod2 = self.txt_mod(temb).chunk(2, dim=-1)
    img_modulated, img_gate1 = self._modulate(self.img_norm1(hidden_states), img_mod1)
    txt_modulated, txt_gate1 = self._modulate(self.txt_norm1(encoder_hidden_states), txt_mod1)
    img_attn_output, txt_attn_output = self.attn(hidden_states=img_modulated,
                                                 encoder_hidden_states=txt_modulated,
                                                 image_rotary_emb=image_rotary_emb,
                                                 **(joint_attention_kwargs or {}))
    hidden_states = hidden_states + img_gate1 * img_attn_output
    encoder_hidden_states = encoder_hidden_states + txt_gate1 * txt_attn_output
    img_modulated2, img_gate2 = self._modulate(self.img_norm2(hidden_states), img_mod2)
    hidden_states = hidden_states + img_gate2 * self.img_mlp(img_modulated2)
    txt_modulated2, txt_gate2 = self._modulate(self.txt_norm2(encoder_hidden_states), txt_mod2)
    encoder_hidden_states = encoder_hidden_states + txt_gate2 * self.txt_mlp(txt_modulated2)
    return encoder_hidden_states, hidden_states


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
    self.norm_out = AdaLayerNormContinuous(dim)
    self.proj_out = nn.Linear(dim, in_channels)

  def forward(self, hidden_states, encoder_hidden_states, timestep):
    hidden = self.img_in(hidden_states)
    encoder = self.txt_in(self.txt_norm(encoder_hidden_states))
    temb = self.time_text_embed(timestep)
    rope = rope_table(encoder.shape[1] + hidden.shape[1], self.dim // self.heads, hidden.device)
    for blk in self.transformer_blocks:
      encoder, hidden = blk(hidden_states=hidden, encoder_hidden_states=encoder,
                            encoder_hidden_states_mask=None, temb=temb, image_rotary_emb=rope)
    hidden = self.norm_out(hidden, temb)
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
  """`forward(hidden_states, encoder_hidden_states=None, rotary_emb=None)`: self-attention,
  or cross-attention to the text when `encoder_hidden_states` is given (diffusers'
  WanAttention; reference: src/cache_dit/distributed/transformers/wan.py:69-160)."""

  def __init__(self, dim: int, heads: int):
    super().__init__()
    self.heads = heads
    self.to_q, self.to_k, self.to_v = nn.Linear(dim, dim), nn.Linear(dim, dim), nn.Linear(dim, dim)
    self.to_out = nn.ModuleList([nn.Linear(dim, dim), nn.Dropout(0.0)])
    self.norm_q, self.norm_k = RMSNorm(dim), RMSNorm(dim)  # full width, before the head split

  def forward(self, hidden_states, encoder_hidden_states=None, attention_mask=None, rotary_emb=None,
              **kwargs):
    src = hidden_states if encoder_hidden_states is None else encoder_hidden_states
    q = _heads(self.norm_q(self.to_q(hidden_states)), self.heads)
    k = _heads(self.norm_k(self.to_k(src)), self.heads)
    v = _heads(self.to_v(src), self.heads)
    if rotary_emb is not None:
      q, k = apply_rope(q, rotary_emb), apply_rope(k, rotary_emb)
    o = _merge(F.scaled_dot_product_attention(q, k, v))
    return self.to_out[1](self.to_out[0](o))


class WanTransformerBlock(nn.Module):
  """10 Linears: self-attention, cross-attention to the text, GELU-tanh FFN. Attributes and
  the forward signature follow diffusers' WanTransformerBlock (the block the reference adapts
  in src/cache_dit/caching/patch_functors/functor_wan_vace.py:40-90); the two modulations are
  done in bf16 tensor ops here (diffusers computes them in fp32 and rounds once)."""

  def __init__(self, dim: int, heads: int, ffn: int):
    super().__init__()
    self.norm1 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
    self.attn1 = WanAttention(dim, heads)
    self.attn2 = WanAttention(dim, heads)
    self.norm2 = nn.LayerNorm(dim, eps=1e-6)
    self.ffn = FeedForward(dim, ffn)
    self.norm3 = nn.LayerNorm(dim, elementwise_affine=False, eps=1e-6)
    self.scale_shift_table = nn.Parameter(torch.randn(1, 6, dim) / dim**0.5)

  def forward(self, hidden_states, encoder_hidden_states, temb, rotary_emb=None):
    shift_msa, scale_msa, gate_msa, c_shift_msa, c_scale_msa, c_gate_msa = (
        self.scale_shift_table + temb).chunk(6, dim=1)
    norm_hidden_states = self.norm1(hidden_states) * (1 + scale_msa) + shift_msa
    attn_output = self.attn1(hidden_states=norm_hidden_states, rotary_emb=rotary_emb)
    hidden_states = hidden_states + attn_output * gate_msa
    norm_hidden_states = self.norm2(hidden_states)
    hidden_states = hidden_states + self.attn2(hidden_states=norm_hidden_states,
                                               encoder_hidden_states=encoder_hidden_states)
    norm_hidden_states = self.norm3(hidden_states) * (1 + c_scale_msa) + c_shift_msa
    return hidden_states + self.ffn(norm_hidden_states) * c_gate_msa


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
      hidden = blk(hidden_states=hidden, encoder_hidden_states=context, temb=temb6, rotary_emb=rope)
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


def _restage(model: nn.Module, **changes) -> None:
  """(Re)applies the stage patch functor with the options accumulated on `model`."""
  from ..patch_functors import StagePatchFunctor
  opts = model.__dict__.setdefault("_stage_opts", {
      "batch_stages": False, "single_blocks": False, "fuse_cat": False, "fuse_norm_quant": False,
      "materialize": True})
  opts.update(changes)
  if any(opts[k] for k in ("batch_stages", "fuse_cat", "fuse_norm_quant")):
    StagePatchFunctor().apply(model, **opts)
  else:
    StagePatchFunctor().remove(model)


def batch_streams(model: nn.Module, enable: bool = True, single_blocks: bool = False) -> int:
  """Patches `model` (cache_dit_amd.patch_functors.StagePatchFunctor) so that the Linears of
  every stage of a block run as one launch: the image-stream and the text-stream Linears of
  a double-stream block (FLUX, Qwen-Image), the query next to key / value of a cross
  attention (Wan); single_blocks=True also proj_mlp + q/k/v of FLUX single blocks. The
  model's own forwards stay as they are. Outputs are bit-identical. Returns the number of
  double-stream attention modules."""
  _restage(model, batch_stages=bool(enable), single_blocks=bool(enable) and single_blocks)
  return sum(isinstance(m, FluxAttention) and m.joint for m in model.modules())


def fuse_cat_quant(model: nn.Module, enable: bool = True) -> int:
  """Single-stream blocks of `model`: proj_out's quantizer reads the attention output and the
  MLP activation in place instead of their torch.cat copy (`nn.linear_on_cat`, through the
  stage patch functor). Outputs are bit-identical. Returns the number of such blocks."""
  _restage(model, fuse_cat=bool(enable))
  return sum(isinstance(m, FluxSingleTransformerBlock) for m in model.modules())


def fuse_norm_quant(model: nn.Module, enable: bool = True, materialize: bool = True) -> int:
  """Every modulated LayerNorm inside the repeated blocks of `model` runs as the kernel that
  also quantizes (ops.ln_modulate_quant, through the stage patch functor), and the Linears of
  the blocks pick the delivered codes up. materialize=False also drops the bf16 write of the
  modulated activation: valid here because only quantized Linears read it. Returns the number
  of modules whose forward computes a modulated norm (FLUX double block: norm1, norm1_context
  and the block itself; single block: norm; Qwen-Image and Wan blocks: the block)."""
  _restage(model, fuse_norm_quant=bool(enable), materialize=bool(materialize))
  n = 0
  for m in model.modules():
    name = type(m).__name__
    n += {"FluxTransformerBlock": 3, "FluxSingleTransformerBlock": 1, "QwenImageTransformerBlock": 1,
          "WanTransformerBlock": 1}.get(name, 0)
  return n


def count_linears(model: nn.Module):
  total = sum(isinstance(m, nn.Linear) for m in model.modules())
  quantized = sum(bool(getattr(m, "_is_inner_quantized", False)) for m in model.modules())
  return total, quantized
