"""Stage patch functors: make an UNMODIFIED diffusers-style transformer run its quantized
Linears stage by stage -- one quantizer launch and one batched GEMM launch per stage of a
block instead of one of each per Linear -- without editing the model's code.

The reference changes a block's forward without touching diffusers through patch functors
(src/cache_dit/caching/patch_functors/functor_base.py:13-60: `PatchFunctor.apply(transformer)`;
functor_flux.py:23-80 rebinds `block.forward` to a function adapted from diffusers). The
functors here follow that shape and are written against the same things the reference's are:
diffusers' attribute names (`norm1`, `attn.to_q`, `attn.add_q_proj`, `attn.to_out[0]`,
`attn.to_add_out`, `ff.net[0].proj`, `ff.net[2]`, `proj_mlp`, `proj_out`, `img_mod`, `attn1` ...)
and block forward signatures. Three mechanisms, from least to most intrusive:

  * a wrapper bound as `forward` of the attention modules (an instance attribute; the class
    and its processor stay as they are). It sees `hidden_states` and `encoder_hidden_states`
    before the module's own code (diffusers: its attention processor) calls to_q / to_k /
    to_v and add_q_proj / add_k_proj / add_v_proj one after the other, computes all of them
    with `nn.precompute_stage` and leaves each output on its Linear, which returns it when
    called with that very activation. The attention code itself (norms, RoPE, SDPA, whatever
    processor is installed) is not touched. A second wrapper on `to_out[0]` does the same for
    the output projections of a joint attention, whose two inputs are the two parts of one
    split tensor. (Wrappers rather than forward hooks: a hook handle carries a process-wide
    serial number, which a graph tracer guards on, so that every block would be compiled
    separately.)
  * rebound block forwards, adapted from the diffusers block forwards, for what these
    wrappers cannot do: the two FeedForwards of a double-stream block run at different
    points of the original forward (the text stream's input does not exist yet when the
    image stream's runs), so the forward is reordered to put both modulated inputs side by
    side; a FLUX single block
    precomputes proj_mlp next to q/k/v and lets proj_out's quantizer read
    `[attn_output | mlp_hidden_states]` in place (`nn.linear_on_cat`).
  * optionally (`fuse_norm_quant=True`) the modulated LayerNorms
    `norm(x) * (1 + scale) + shift` run as the kernel that also delivers the FP8 codes
    (`ops.ln_modulate_quant`), in the rebound forwards and in AdaLayerNormZero(/Single).

Outputs are bit-identical to the unpatched model in the first two cases (the kernels give the
same bits batched or not; the reordering moves whole tensor ops, not arithmetic inside them).
Everything falls back to the plain behaviour where nothing can be batched: inference-mode
tensors, Linears that were not converted. Inside a traced graph (torch.compile of the patched
blocks) a stage is the one traceable batch op; the fused norms and the joint output
projections keep their plain form there.
"""
from __future__ import annotations

import inspect
import types
from typing import Optional

import torch
from torch import nn

from . import nn as cnn
from . import ops
from .logger import init_logger

logger = init_logger(__name__)

_QUANT = (cnn.Fp8DynamicLinear, cnn.Fp8WeightOnlyLinear)


def _opts(block) -> dict:
  return getattr(block, "_cdit_stage_opts", None) or {}


def _quantized(*mods) -> bool:
  return all(isinstance(m, _QUANT) for m in mods)


# ------------------------------------------------------------------ attention modules


def _attention_forward(self, *args, **kwargs):
  """Bound as `forward` of an attention module (diffusers' Attention / FluxAttention /
  WanAttention interface: `hidden_states`, `encoder_hidden_states` first, by position or
  keyword). Computes the projections of the stage ahead, leaves each output on its Linear
  and runs the module's own forward, whose code (processor, norms, RoPE, SDPA) then calls
  the Linears one by one and finds the outputs."""
  if not getattr(self, "_cdit_stage_batch", False):
    return self._cdit_orig_forward(*args, **kwargs)
  hidden = kwargs.get("hidden_states", args[0] if args else None)
  encoder = kwargs.get("encoder_hidden_states", args[1] if len(args) > 1 else None)
  q, k, v = self.to_q, self.to_k, self.to_v
  add_q = getattr(self, "add_q_proj", None)
  if not isinstance(hidden, torch.Tensor) or q._precomputed is not None:
    pass  # (the block's forward already put this stage together: proj_mlp + q/k/v)
  elif add_q is not None and isinstance(encoder, torch.Tensor):
    self._cdit_n_txt = encoder.shape[1]
    cnn.precompute_stage([(hidden, [q, k, v]), (encoder, [add_q, self.add_k_proj, self.add_v_proj])])
  elif isinstance(encoder, torch.Tensor):  # cross-attention: the query on one activation, k / v on the other
    cnn.precompute_stage([(hidden, [q]), (encoder, [k, v])])
  else:
    cnn.precompute_stage([(hidden, [q, k, v])])
  out = self._cdit_orig_forward(*args, **kwargs)
  # what the module's code did not collect (it was called with other tensors) is dropped here
  cnn.release_precomputed([q, k, v, add_q, getattr(self, "add_k_proj", None), getattr(self, "add_v_proj", None)])
  return out


def _joint_out_forward(self, x):
  """Bound as `forward` of `attn.to_out[0]` of a joint attention: its input is the image
  part of the attention output, split off one tensor whose first `n_txt` tokens go to
  `attn.to_add_out` next. Both projections are computed here; the text part is addressed as
  the rows in front of the image part in the same storage. Whatever to_add_out is then called
  with, it only takes the stashed output if that is exactly this memory, unmodified. (Eager
  code only: a traced graph has no storage to address, the two Linears stay two ops there.)"""
  attn = self._cdit_joint_attn[0]
  if not torch.compiler.is_compiling() and getattr(attn, "_cdit_stage_batch", False):
    n_txt = getattr(attn, "_cdit_n_txt", 0)
    # (one batch element: with more, the rows of a part are not contiguous and every Linear
    # call works on a copy of its own, which no stash can be keyed on)
    if (isinstance(x, torch.Tensor) and x.dim() == 3 and n_txt > 0 and x._base is not None
        and x.shape[0] == 1 and x.stride(2) == 1 and x.stride(1) == x.shape[2]
        and x.storage_offset() >= n_txt * x.stride(1)):
      front = x.as_strided((x.shape[0], n_txt, x.shape[2]), x.stride(),
                           x.storage_offset() - n_txt * x.stride(1))
      cnn.precompute_stage([(x, [self]), (front, [attn.to_add_out])])
  return self._cdit_orig_forward(x)


# ------------------------------------------------------------------ pieces of the block forwards


def _modulated_norm(block, norm: nn.Module, x, shift, scale):
  """`norm(x) * (1 + scale) + shift` for a LayerNorm without affine parameters: as bf16 tensor
  ops, or as the kernel that also hands the FP8 codes to the consuming Linears."""
  o = _opts(block)
  # (a traced graph keeps the tensor ops: its compiler fuses them, and nothing is handed over there)
  if (o.get("fuse_norm") and not torch.compiler.is_compiling() and x.is_cuda and x.dtype == torch.bfloat16
      and isinstance(norm, nn.LayerNorm) and norm.weight is None and norm.bias is None):
    return ops.ln_modulate_quant(x, shift, scale, eps=norm.eps, materialize=o.get("materialize", True))
  return norm(x) * (1 + scale) + shift


def _feed_forward_pair(block, ff_a: nn.Module, xa, ff_b: nn.Module, xb):
  """Two diffusers FeedForwards (`net = [activation block with .proj, Dropout, Linear, ...]`)
  on independent inputs, their Linears launched pairwise."""
  net_a, net_b = getattr(ff_a, "net", None), getattr(ff_b, "net", None)
  if (not _opts(block).get("batch") or net_a is None or net_b is None or len(net_a) != len(net_b)
      or not hasattr(net_a[0], "proj") or not hasattr(net_b[0], "proj")):
    return ff_a(xa), ff_b(xb)
  cnn.precompute_stage([(xa, [net_a[0].proj]), (xb, [net_b[0].proj])])
  ha, hb = net_a[0](xa), net_b[0](xb)
  for ma, mb in zip(list(net_a)[1:], list(net_b)[1:]):
    if _quantized(ma, mb):
      cnn.precompute_stage([(ha, [ma]), (hb, [mb])])
    ha, hb = ma(ha), mb(hb)
  return ha, hb


def _clip_fp16(x):
  return x.clip(-65504, 65504) if x.dtype == torch.float16 else x


# ------------------------------------------------------------------ FLUX
# Adapted from diffusers' FluxTransformerBlock.forward / FluxSingleTransformerBlock.forward
# (src/diffusers/models/transformers/transformer_flux.py), the forwards the reference adapts in
# src/cache_dit/caching/patch_functors/functor_flux.py:48-80.


def _flux_double_forward(self, hidden_states, encoder_hidden_states, temb, image_rotary_emb=None,
                         joint_attention_kwargs=None):
  norm_hidden_states, gate_msa, shift_mlp, scale_mlp, gate_mlp = self.norm1(hidden_states, emb=temb)
  norm_encoder_hidden_states, c_gate_msa, c_shift_mlp, c_scale_mlp, c_gate_mlp = self.norm1_context(
      encoder_hidden_states, emb=temb)
  attention_outputs = self.attn(hidden_states=norm_hidden_states,
                                encoder_hidden_states=norm_encoder_hidden_states,
                                image_rotary_emb=image_rotary_emb, **(joint_attention_kwargs or {}))
  if len(attention_outputs) != 2:
    raise NotImplementedError("stage-patched FLUX block: attention returned "
                              f"{len(attention_outputs)} outputs (IP-adapter); remove the stage patch")
  attn_output, context_attn_output = attention_outputs
  hidden_states = hidden_states + gate_msa.unsqueeze(1) * attn_output
  encoder_hidden_states = encoder_hidden_states + c_gate_msa.unsqueeze(1) * context_attn_output
  # both streams' MLP inputs side by side (the original forward finishes the image stream first)
  norm_hidden_states = _modulated_norm(self, self.norm2, hidden_states, shift_mlp[:, None], scale_mlp[:, None])
  norm_encoder_hidden_states = _modulated_norm(self, self.norm2_context, encoder_hidden_states,
                                               c_shift_mlp[:, None], c_scale_mlp[:, None])
  ff_output, context_ff_output = _feed_forward_pair(self, self.ff, norm_hidden_states, self.ff_context,
                                                    norm_encoder_hidden_states)
  hidden_states = hidden_states + gate_mlp.unsqueeze(1) * ff_output
  encoder_hidden_states = encoder_hidden_states + c_gate_mlp.unsqueeze(1) * context_ff_output
  return _clip_fp16(encoder_hidden_states), hidden_states


def _flux_single_core(self, hidden_states, temb, image_rotary_emb, joint_attention_kwargs):
  o = _opts(self)
  residual = hidden_states
  norm_hidden_states, gate = self.norm(hidden_states, emb=temb)
  if o.get("batch") and _quantized(self.proj_mlp, self.attn.to_q, self.attn.to_k, self.attn.to_v):
    cnn.precompute_stage([(norm_hidden_states,
                           [self.proj_mlp, self.attn.to_q, self.attn.to_k, self.attn.to_v])])
  mlp_hidden_states = self.act_mlp(self.proj_mlp(norm_hidden_states))
  attn_output = self.attn(hidden_states=norm_hidden_states, image_rotary_emb=image_rotary_emb,
                          **(joint_attention_kwargs or {}))
  if o.get("fuse_cat"):
    projected = cnn.linear_on_cat(self.proj_out, [attn_output, mlp_hidden_states])
  else:
    projected = self.proj_out(torch.cat([attn_output, mlp_hidden_states], dim=2))
  return _clip_fp16(residual + gate.unsqueeze(1) * projected)


def _flux_single_forward(self, hidden_states, temb, image_rotary_emb=None, joint_attention_kwargs=None):
  """Single block of diffusers up to 0.34: the transformer concatenates the streams once."""
  return _flux_single_core(self, hidden_states, temb, image_rotary_emb, joint_attention_kwargs)


def _flux_single_forward_two_streams(self, hidden_states, encoder_hidden_states, temb,
                                     image_rotary_emb=None, joint_attention_kwargs=None):
  """Single block of newer diffusers: takes and returns the two streams."""
  text_seq_len = encoder_hidden_states.shape[1]
  hidden_states = torch.cat([encoder_hidden_states, hidden_states], dim=1)
  hidden_states = _flux_single_core(self, hidden_states, temb, image_rotary_emb, joint_attention_kwargs)
  return hidden_states[:, :text_seq_len], hidden_states[:, text_seq_len:]


def _adaln_zero_forward(self, x, timestep=None, class_labels=None, hidden_dtype=None, emb=None):
  """AdaLayerNormZero.forward with the modulated norm as one kernel (FLUX calls it with `emb`)."""
  if emb is None or getattr(self, "emb", None) is not None:
    return self._cdit_orig_forward(x, timestep=timestep, class_labels=class_labels,
                                   hidden_dtype=hidden_dtype, emb=emb)
  emb = self.linear(self.silu(emb))
  shift_msa, scale_msa, gate_msa, shift_mlp, scale_mlp, gate_mlp = emb.chunk(6, dim=1)
  x = _modulated_norm(self, self.norm, x, shift_msa[:, None], scale_msa[:, None])
  return x, gate_msa, shift_mlp, scale_mlp, gate_mlp


def _adaln_zero_single_forward(self, x, emb=None):
  emb = self.linear(self.silu(emb))
  shift_msa, scale_msa, gate_msa = emb.chunk(3, dim=1)
  x = _modulated_norm(self, self.norm, x, shift_msa[:, None], scale_msa[:, None])
  return x, gate_msa


# ------------------------------------------------------------------ Qwen-Image
# Adapted from diffusers' QwenImageTransformerBlock.forward
# (src/diffusers/models/transformers/transformer_qwenimage.py), the forward the reference adapts
# in src/cache_dit/caching/patch_functors/functor_qwen_image_controlnet.py:43-117.


def _qwen_modulated(block, norm, x, mod_params):
  shift, scale, gate = mod_params.chunk(3, dim=-1)
  return _modulated_norm(block, norm, x, shift.unsqueeze(1), scale.unsqueeze(1)), gate.unsqueeze(1)


def _qwen_image_forward(self, hidden_states, encoder_hidden_states, encoder_hidden_states_mask=None,
                        temb=None, image_rotary_emb=None, joint_attention_kwargs=None):
  img_mod1, img_mod2 = self.img_mod(temb).chunk(2, dim=-1)
  txt_mod1, txt_mod2 = self.txt_mod(temb).chunk(2, dim=-1)
  img_modulated, img_gate1 = _qwen_modulated(self, self.img_norm1, hidden_states, img_mod1)
  txt_modulated, txt_gate1 = _qwen_modulated(self, self.txt_norm1, encoder_hidden_states, txt_mod1)
  kwargs = dict(joint_attention_kwargs or {})
  if _opts(self).get("attn_takes_mask"):
    kwargs["encoder_hidden_states_mask"] = encoder_hidden_states_mask
  img_attn_output, txt_attn_output = self.attn(hidden_states=img_modulated,
                                               encoder_hidden_states=txt_modulated,
                                               image_rotary_emb=image_rotary_emb, **kwargs)
  hidden_states = hidden_states + img_gate1 * img_attn_output
  encoder_hidden_states = encoder_hidden_states + txt_gate1 * txt_attn_output
  img_modulated2, img_gate2 = _qwen_modulated(self, self.img_norm2, hidden_states, img_mod2)
  txt_modulated2, txt_gate2 = _qwen_modulated(self, self.txt_norm2, encoder_hidden_states, txt_mod2)
  img_mlp_output, txt_mlp_output = _feed_forward_pair(self, self.img_mlp, img_modulated2, self.txt_mlp,
                                                      txt_modulated2)
  hidden_states = hidden_states + img_gate2 * img_mlp_output
  encoder_hidden_states = encoder_hidden_states + txt_gate2 * txt_mlp_output
  return _clip_fp16(encoder_hidden_states), _clip_fp16(hidden_states)


# ------------------------------------------------------------------ Wan
# Adapted from diffusers' WanTransformerBlock.forward
# (src/diffusers/models/transformers/transformer_wan.py), the forward the reference adapts in
# src/cache_dit/caching/patch_functors/functor_wan_vace.py:40-90. One stream: the stages are the
# attention modules' own (their wrappers); the block forward is only rebound for the fused modulated
# norms, which are computed as bf16 tensor ops (diffusers does these two in fp32 and rounds
# once, so this rebinding is offered for models that accept the bf16 form).


def _wan_forward(self, hidden_states, encoder_hidden_states, temb, rotary_emb=None):
  shift_msa, scale_msa, gate_msa, c_shift_msa, c_scale_msa, c_gate_msa = (
      self.scale_shift_table + temb).chunk(6, dim=1)
  norm_hidden_states = _modulated_norm(self, self.norm1, hidden_states, shift_msa, scale_msa)
  attn_output = self.attn1(hidden_states=norm_hidden_states, rotary_emb=rotary_emb)
  hidden_states = hidden_states + attn_output * gate_msa
  norm_hidden_states = self.norm2(hidden_states)
  hidden_states = hidden_states + self.attn2(hidden_states=norm_hidden_states,
                                             encoder_hidden_states=encoder_hidden_states)
  norm_hidden_states = _modulated_norm(self, self.norm3, hidden_states, c_shift_msa, c_scale_msa)
  return hidden_states + self.ffn(norm_hidden_states) * c_gate_msa


# ------------------------------------------------------------------ the functors


class StagePatchFunctor:
  """`apply(transformer, ...)` patches every block of the families it knows in place and
  returns the transformer (the shape of the reference's PatchFunctor.apply,
  src/cache_dit/caching/patch_functors/functor_base.py:20-50); `remove(transformer)` undoes
  it. Blocks are recognised by class name, attention modules by their `to_q / to_k / to_v`.

  batch_stages     one quantizer + one GEMM launch per stage (rebound forwards)
  single_blocks    also precompute proj_mlp + q/k/v of FLUX single blocks as one stage (eager
                   code can leave this to nn.group_sibling_linears_; a rebound forward does
                   not need the discovery run)
  fuse_cat         FLUX single blocks: proj_out reads [attn | mlp] in place
  fuse_norm_quant  modulated LayerNorms as the kernel that also quantizes; switches
                   `share_input_quant` on for the Linears that pick the codes up
  materialize      with fuse_norm_quant: write the bf16 activation too (False: codes only; a
                   consumer that then reads the values raises)
  """

  #: block class name -> rebound forward (chosen by the original forward's parameters for
  #: the FLUX single block)
  BLOCK_FORWARDS = {
      "FluxTransformerBlock": _flux_double_forward,
      "FluxSingleTransformerBlock": _flux_single_forward,
      "QwenImageTransformerBlock": _qwen_image_forward,
      "WanTransformerBlock": _wan_forward,
  }
  NORM_FORWARDS = {
      "AdaLayerNormZero": _adaln_zero_forward,
      "AdaLayerNormZeroSingle": _adaln_zero_single_forward,
  }
  #: blocks whose rebound forward is only needed for the fused norms
  NORM_ONLY_BLOCKS = ("WanTransformerBlock", )

  def apply(self, transformer: nn.Module, batch_stages: bool = True, single_blocks: bool = True,
            fuse_cat: bool = True, fuse_norm_quant: bool = False, materialize: bool = True) -> nn.Module:
    if batch_stages and any(isinstance(m, _QUANT) and m.sibling_group is not None
                            for m in transformer.modules()):
      logger.warning("stage patch: sibling groups are removed (a stage is computed by the rebound "
                     "forwards instead)")
      cnn.group_sibling_linears_(transformer, enable=False)
    n_blocks = n_attn = 0
    batch_of = {}  # attention module -> whether its owning block batches stages
    for block in transformer.modules():
      name = type(block).__name__
      if name in self.BLOCK_FORWARDS:
        double = name != "FluxSingleTransformerBlock"
        opts = {
            "batch": bool(batch_stages) and (double or bool(single_blocks)),
            "fuse_cat": bool(fuse_cat),
            "fuse_norm": bool(fuse_norm_quant),
            "materialize": bool(materialize),
            # (looked up here: the rebound forwards may run inside a traced graph)
            "attn_takes_mask": (hasattr(block, "attn") and "encoder_hidden_states_mask" in inspect.signature(
                block.attn.__dict__.get("_cdit_orig_forward") or block.attn.forward).parameters),
        }
        block._cdit_stage_opts = opts
        rebind = (opts["fuse_norm"] if name in self.NORM_ONLY_BLOCKS else
                  opts["batch"] or opts["fuse_norm"] or (not double and opts["fuse_cat"]))
        self._rebind(block, self._block_forward(block) if rebind else None)
        n_blocks += 1
        for norm in block.children():
          if type(norm).__name__ in self.NORM_FORWARDS:
            norm._cdit_stage_opts = opts
            self._rebind(norm, self.NORM_FORWARDS[type(norm).__name__] if fuse_norm_quant else None)
        if fuse_norm_quant:
          for lin in self._norm_consumers(block):
            lin.share_input_quant = True  # they look the delivered codes up
        for sub in block.modules():
          batch_of.setdefault(id(sub), opts["batch"])
    for attn in transformer.modules():
      if all(isinstance(getattr(attn, a, None), _QUANT) for a in ("to_q", "to_k", "to_v")):
        attn._cdit_stage_batch = batch_of.get(id(attn), bool(batch_stages))
        self._rebind(attn, _attention_forward)
        to_out = getattr(attn, "to_out", None)
        if (getattr(attn, "to_add_out", None) is not None and to_out is not None
            and _quantized(to_out[0], attn.to_add_out)):
          to_out[0].__dict__["_cdit_joint_attn"] = (attn, )  # (a tuple: not registered as a submodule)
          self._rebind(to_out[0], _joint_out_forward)
        n_attn += 1
    transformer._cdit_stage_patched = True
    logger.info(f"stage patch: {n_blocks} blocks, {n_attn} attention modules of "
                f"{type(transformer).__name__}")
    return transformer

  def remove(self, transformer: nn.Module) -> nn.Module:
    for m in transformer.modules():
      self._rebind(m, None)
      m.__dict__.pop("_cdit_stage_opts", None)
      m.__dict__.pop("_cdit_stage_batch", None)
      m.__dict__.pop("_cdit_joint_attn", None)
    transformer.__dict__.pop("_cdit_stage_patched", None)
    return transformer

  @staticmethod
  def _norm_consumers(block: nn.Module):
    """The float8_per_row Linears of `block` that read a modulated norm: the attention input
    projections, the first Linear of every FeedForward, proj_mlp."""
    found = []
    for m in block.modules():
      for a in ("to_q", "to_k", "to_v", "add_q_proj", "add_k_proj", "add_v_proj", "proj_mlp"):
        found.append(getattr(m, a, None))
      net = getattr(m, "net", None)
      if isinstance(net, nn.ModuleList) and len(net) and hasattr(net[0], "proj"):
        found.append(net[0].proj)
    return [lin for lin in found if isinstance(lin, cnn.Fp8DynamicLinear)]

  def _block_forward(self, block: nn.Module):
    fn = self.BLOCK_FORWARDS[type(block).__name__]
    if fn is _flux_single_forward:
      orig = block.__dict__.get("_cdit_orig_forward") or block.forward
      if "encoder_hidden_states" in inspect.signature(orig).parameters:
        return _flux_single_forward_two_streams
    return fn

  @staticmethod
  def _rebind(module: nn.Module, fn) -> None:
    """Binds `fn` as module.forward (None: restores the original)."""
    d = module.__dict__
    if fn is None:
      if "_cdit_orig_forward" in d:
        if d["_cdit_orig_forward_was_instance_attr"]:
          d["forward"] = d["_cdit_orig_forward"]
        else:
          d.pop("forward", None)
        d.pop("_cdit_orig_forward", None)
        d.pop("_cdit_orig_forward_was_instance_attr", None)
      return
    if "_cdit_orig_forward" not in d:
      d["_cdit_orig_forward_was_instance_attr"] = "forward" in d
      d["_cdit_orig_forward"] = module.forward
    d["forward"] = types.MethodType(fn, module)


def apply_stage_patch(transformer: nn.Module, **kwargs) -> nn.Module:
  """StagePatchFunctor().apply(transformer, **kwargs)."""
  return StagePatchFunctor().apply(transformer, **kwargs)


def remove_stage_patch(transformer: nn.Module) -> nn.Module:
  return StagePatchFunctor().remove(transformer)
