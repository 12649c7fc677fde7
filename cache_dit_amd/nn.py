"""Quantized nn.Linear modules: the counterpart of torchao's Float8Tensor
`aten.linear` override that cache-dit installs with `quantize_`
(src/cache_dit/quantization/torchao/quantize_ao.py:166-179).

Conversion is in place: the nn.Linear object keeps its identity (parents, hooks
and block adapters that hold a reference keep working, and
`isinstance(m, nn.Linear)` stays true, which the reference's filter relies on);
its class is switched to a subclass whose forward calls the HIP kernels, its
`weight` becomes the e4m3 codes [N,K] and a `weight_scale` buffer [N,1] holds
the per-output-channel fp32 scales.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import nn

from . import _native, ops
from .logger import init_logger

logger = init_logger(__name__)

FP8 = torch.float8_e4m3fn

_warned_inference_bypass = False


def _note_inference_bypass(what: str) -> None:
  """Sharing, grouping and stage batching key their state on the activation's version
  counter, which inference-mode tensors do not have: under torch.inference_mode() every
  Linear runs on its own. Said once per process, since the slower path is otherwise silent."""
  global _warned_inference_bypass
  if not _warned_inference_bypass:
    _warned_inference_bypass = True
    logger.warning(
        f"{what}: the input is an inference-mode tensor (no version counter), so shared "
        "activation quantization, sibling groups and stage batching are bypassed and every "
        "Linear launches its own quantizer and GEMM. Run under torch.no_grad() instead of "
        "torch.inference_mode() to keep them.")

#: scale rounding used for activations and weights (see ops.fp8_rowwise_quant)
DEFAULT_SCALE_MODE = "bf16div"


def _quantize_weight(weight: torch.Tensor, scale_mode: str, per_tensor: bool = False):
  """W bf16 [N,K] -> (codes e4m3 [N,K], scale fp32 [N,1]) with the HIP quantizer.

  The reference quantizes the weight wherever it lives, and its CLI flow does so
  before `pipe.to(device)` (src/cache_dit/_utils/utils.py:2419,2459). There is no
  CPU kernel here, so a CPU weight makes a round trip through the GPU.
  """
  if weight.dtype != torch.bfloat16:
    raise ValueError(f"weight must be bfloat16 to be quantized to FP8, got {weight.dtype}")
  src = weight.detach()
  if not src.is_cuda:
    if not torch.cuda.is_available():
      raise RuntimeError("quantizing a CPU weight needs a GPU to run the quantizer kernel on; "
                         "there is no CPU path")
    src = src.to("cuda")
  quant = ops.fp8_tensorwise_quant if per_tensor else ops.fp8_rowwise_quant
  q, s = quant(src.contiguous(), scale_mode)
  return q.to(weight.device), s.to(weight.device)


class _Fp8LinearBase(nn.Linear):
  """Common state of the two quantized Linears. Never constructed directly:
  `convert_linear_` re-classes an existing nn.Linear."""

  weight_scale: torch.Tensor
  share_input_quant: bool = False
  #: (input key, output, stream, capture id) left by precompute_stage, or None
  _precomputed = None
  epilogue: int
  scale_mode: str
  quant_type: str

  def extra_repr(self) -> str:
    return (f"in_features={self.in_features}, out_features={self.out_features}, "
            f"bias={self.bias is not None}, quant_type={self.quant_type}, "
            f"epilogue={'gelu_tanh' if self.epilogue & _native.EPI_GELU_TANH else 'none'}")

  def _check_input(self, x: torch.Tensor) -> None:
    if x.dtype != torch.bfloat16:
      raise ValueError(f"{type(self).__name__} takes bfloat16 activations, got {x.dtype}")
    if not x.is_cuda:
      raise RuntimeError(f"{type(self).__name__}: input is on {x.device}; there is no CPU path")


class _InputKey:
  """Identity of an activation buffer: storage, offset, shape, strides and version
  counter; keeps the tensor alive so that its address cannot be handed out again."""
  __slots__ = ("x", "version")

  def __init__(self, x2: torch.Tensor):
    self.x, self.version = x2, x2._version

  def matches(self, x2: torch.Tensor) -> bool:
    x = self.x
    return (self.version == x2._version and x.data_ptr() == x2.data_ptr() and x.shape == x2.shape
            and x.stride() == x2.stride()
            and x.untyped_storage().data_ptr() == x2.untyped_storage().data_ptr())


class SiblingGroup:
  """Two to eight `float8_per_row` Linears (or `float8_weight_only` ones, which skip the
  quantization) that are handed the very same activation one
  after the other (attn.to_q / to_k / to_v; proj_mlp + q/k/v in FLUX single blocks;
  reference dataflow src/cache_dit/caching/patch_functors/functor_flux.py:60-67). The
  first member called with an activation quantizes it once and computes every member's
  output in ONE grouped GEMM launch; the others, called with the same unmodified buffer,
  return theirs. Outputs are bit-identical to the ungrouped Linears. A member called with
  anything else simply computes the group afresh, so a wrong guess costs time, not
  correctness."""

  def __init__(self, members):
    members = list(members)
    if not 2 <= len(members) <= _native.MAX_GROUP:
      raise ValueError(f"a sibling group holds 2 to {_native.MAX_GROUP} Linears, got {len(members)}")
    first = members[0]
    if type(first) not in (Fp8DynamicLinear, Fp8WeightOnlyLinear):
      raise TypeError("sibling groups are built from float8_per_row or float8_weight_only Linears")
    for m in members:
      if type(m) is not type(first):
        raise TypeError("the members of a sibling group must be of one quant type")
      if m.in_features != first.in_features or m._scale_mode_id != first._scale_mode_id:
        raise ValueError("the members of a sibling group must share in_features and scale mode")
    self.weight_only = type(first) is Fp8WeightOnlyLinear
    self.members = members
    self.index = {id(m): i for i, m in enumerate(members)}
    self.key = None  # _InputKey of the activation the pending outputs were computed from
    self.outs = None
    self.capture_id = 0
    self.stream = None  # (device index, raw stream) the pending outputs were launched on

  def drop_pending(self) -> None:
    """Forgets the outputs no sibling has collected (and the activation they came from)."""
    self.key = self.outs = None

  def forward_member(self, lin: "Fp8DynamicLinear", x: torch.Tensor) -> torch.Tensor:
    """Not thread-safe: a group's state belongs to the thread that runs the model."""
    global _pending_group
    x2 = ops._as_rows(x)
    i = self.index[id(lin)]
    capture_id = (_native.stream_capture_id(ops._stream_ptr(x2))
                  if torch.cuda.is_current_stream_capturing() else 0)
    stream = (x2.device.index, ops._stream_ptr(x2))
    # pending outputs are only handed out on the stream they were launched on (another
    # stream would read them without any ordering) and inside the capture they belong to
    if (self.key is not None and self.capture_id == capture_id and self.stream == stream
        and self.outs[i] is not None and self.key.matches(x2)):
      out, self.outs[i] = self.outs[i], None
      if all(o is None for o in self.outs):
        self.drop_pending()
        if _pending_group is self:
          _pending_group = None
      return out.view(*x.shape[:-1], lin.out_features)
    # A group that computes afresh while another still holds uncollected outputs: that
    # forward left its siblings early (an exception, a skipped branch); its leftovers (up to
    # M x sum(N) bf16) are released here rather than kept until its next call.
    if _pending_group is not None and _pending_group is not self:
      _pending_group.drop_pending()
    _pending_group = self
    M = x2.shape[0]
    members = self.members
    outs = [torch.empty((M, m.out_features), dtype=torch.bfloat16, device=x2.device) for m in members]
    if M > 0 and self.weight_only:
      ops.w8a16_batched_into([(x2, [m.weight for m in members], [m.weight_scale for m in members],
                               [m.bias for m in members], outs, [m.epilogue for m in members])])
    elif M > 0:
      q, s = ops.shared_activation_quant(x2, lin._scale_mode_id)
      ops.gemm_rowwise_grouped_into(q, s, [m.weight for m in members],
                                    [m.weight_scale for m in members], [m.bias for m in members],
                                    outs, [m.epilogue for m in members])
    out, outs[i] = outs[i], None
    self.key, self.outs, self.capture_id, self.stream = _InputKey(x2), outs, capture_id, stream
    return out.view(*x.shape[:-1], lin.out_features)


#: the sibling group whose outputs are waiting to be collected, if any (one at a time: the
#: siblings of a group are called back to back)
_pending_group: Optional[SiblingGroup] = None


def release_pending_outputs() -> None:
  """Drops the outputs a sibling group computed ahead for members that were never called
  (a forward that raised or returned between two siblings). Happens by itself at the next
  grouped call; for a caller that wants the memory back right away."""
  global _pending_group
  if _pending_group is not None:
    _pending_group.drop_pending()
    _pending_group = None


class _SiblingRecorder:
  """Notes, during one forward, which Linears are called back to back with the same
  activation buffer."""

  def __init__(self):
    self.runs, self.key = [], None

  def note(self, lin, x):
    x2 = ops._as_rows(x)
    if self.key is not None and self.key.matches(x2) and all(lin is not m for m in self.runs[-1]):
      self.runs[-1].append(lin)
    else:
      self.runs.append([lin])
      self.key = _InputKey(x2)


_recorder: Optional[_SiblingRecorder] = None


class Fp8DynamicLinear(_Fp8LinearBase):
  """`float8_per_row` (w8a8 dynamic): per-token e4m3 activation quantization,
  e4m3 x e4m3 GEMM with fp32 accumulate, per-token x per-channel scales, bias,
  optional fused GELU-tanh, bf16 out.

  Every forward is one `torch.ops.cdit.*` call, so Dynamo and Inductor see a single
  opaque node with a fake implementation, the way the reference keeps this path
  traceable (src/cache_dit/quantization/torchao/_scaled_mm.py:94-137, :338-357)."""

  sibling_group: Optional[SiblingGroup] = None

  def forward(self, x: torch.Tensor) -> torch.Tensor:
    self._check_input(x)
    # sharing and grouping keep state between calls (the last activation's codes, the
    # siblings' outputs); a compiled graph gets the stateless form (its front end owns the
    # memory its graphs are captured into), and so do inference-mode tensors, which carry
    # no version counter to tell a modified buffer by
    stateless = torch.compiler.is_compiling()
    if stateless:
      if self._precomputed is not None:
        out = _take_precomputed_traced(self, x)
        if out is not None:
          return out
    else:
      if x.is_inference():
        if self.sibling_group is not None or self.share_input_quant:
          _note_inference_bypass(type(self).__name__)
      else:
        if self._precomputed is not None:
          out = _take_precomputed(self, x)
          if out is not None:
            return out
        if _recorder is not None:
          _recorder.note(self, x)
        if self.sibling_group is not None:
          return self.sibling_group.forward_member(self, x)
    share = self.share_input_quant and not stateless
    return torch.ops.cdit.linear_w8a8(x, self.weight, self.weight_scale, self.bias,
                                      self._scale_mode_id, self.epilogue,
                                      ops.GRANULARITY_PER_ROW, share)


class Fp8DynamicLinearPerTensor(_Fp8LinearBase):
  """`float8_per_tensor` (w8a8 dynamic, one scale per tensor): the activation is
  quantized with a single scale computed from its global amax, the weight likewise
  at conversion time; `weight_scale` [N,1] then holds N copies of the weight's scale
  and the GEMM is the per-row one fed with constant scales."""

  def forward(self, x: torch.Tensor) -> torch.Tensor:
    self._check_input(x)
    return torch.ops.cdit.linear_w8a8(x, self.weight, self.weight_scale, self.bias,
                                      self._scale_mode_id, self.epilogue,
                                      ops.GRANULARITY_PER_TENSOR, False)


class Fp8WeightOnlyLinear(_Fp8LinearBase):
  """`float8_weight_only` (w8a16): bf16 activations, e4m3 weights dequantized in
  the GEMM mainloop, per-channel scale in the epilogue."""

  sibling_group: Optional[SiblingGroup] = None

  def forward(self, x: torch.Tensor) -> torch.Tensor:
    self._check_input(x)
    if torch.compiler.is_compiling():  # as in Fp8DynamicLinear
      if self._precomputed is not None:
        out = _take_precomputed_traced(self, x)
        if out is not None:
          return out
    else:
      if x.is_inference():
        if self.sibling_group is not None:
          _note_inference_bypass(type(self).__name__)
      else:
        if self._precomputed is not None:
          out = _take_precomputed(self, x)
          if out is not None:
            return out
        if _recorder is not None:
          _recorder.note(self, x)
        if self.sibling_group is not None:
          return self.sibling_group.forward_member(self, x)
    return torch.ops.cdit.w8a16_mm(x, self.weight.t(), self.weight_scale, self.bias,
                                   _native.DT_BF16, self.epilogue)


_CLASS_OF = {
    "float8_per_row": Fp8DynamicLinear,
    "float8_per_tensor": Fp8DynamicLinearPerTensor,
    "float8_weight_only": Fp8WeightOnlyLinear,
}


def convert_linear_(linear: nn.Linear,
                    quant_type: str,
                    scale_mode: str = DEFAULT_SCALE_MODE,
                    gelu_tanh: bool = False) -> nn.Linear:
  """Quantizes `linear` in place and returns it (same object)."""
  cls = _CLASS_OF.get(quant_type)
  if cls is None:
    raise NotImplementedError(
        f"quant_type {quant_type!r} is not built in this MI355X implementation; built: "
        f"{sorted(_CLASS_OF)}")
  if isinstance(linear, _Fp8LinearBase):
    return linear
  if type(linear) is not nn.Linear and type(linear).forward is not nn.Linear.forward:
    raise TypeError(f"cannot convert {type(linear).__name__}: it overrides nn.Linear.forward")
  if linear.in_features % 16 != 0 or linear.out_features % 16 != 0:
    raise ValueError(f"FP8 matmul needs in/out features that are multiples of 16, got "
                     f"{linear.in_features}x{linear.out_features}")
  q, s = _quantize_weight(linear.weight, scale_mode, per_tensor=quant_type == "float8_per_tensor")
  bias = linear.bias
  del linear.weight
  linear.weight = nn.Parameter(q, requires_grad=False)
  linear.register_buffer("weight_scale", s.reshape(-1, 1).contiguous())
  if bias is not None:
    if bias.dtype != torch.bfloat16:
      raise ValueError(f"bias must be bfloat16, got {bias.dtype}")
    linear.bias = nn.Parameter(bias.detach().contiguous(), requires_grad=False)
  linear.epilogue = _native.EPI_GELU_TANH if gelu_tanh else _native.EPI_NONE
  linear.scale_mode = scale_mode
  linear._scale_mode_id = _native.SCALE_MODE_IDS[scale_mode]
  linear.quant_type = quant_type
  linear.__class__ = cls
  return linear


def fuse_gelu_tanh_(linear: nn.Linear, act: nn.Module) -> None:
  """Moves a following nn.GELU(approximate="tanh") into `linear`'s epilogue and
  turns `act` into an identity, the way the reference wires its fused GELU MLP
  (src/cache_dit/quantization/svdquant/passes.py:489-511). The fused result
  applies GELU to the fp32 accumulator, one bf16 rounding less than the unfused
  pair."""
  if not isinstance(linear, _Fp8LinearBase):
    raise TypeError("fuse_gelu_tanh_ expects an already quantized Linear")
  if not (isinstance(act, nn.GELU) and act.approximate == "tanh"):
    raise TypeError("fuse_gelu_tanh_ expects nn.GELU(approximate='tanh')")
  linear.epilogue |= _native.EPI_GELU_TANH
  act.forward = lambda x: x  # type: ignore[method-assign]
  act._cdit_fused_into_linear = True  # type: ignore[attr-defined]


def share_activation_quant_(module: nn.Module, enable: bool = True) -> int:
  """Lets every `float8_per_row` Linear under `module` reuse the activation codes of
  the previous Linear on the stream when it is handed the very same, unmodified
  input buffer (q/k/v projections, FLUX `proj_mlp` + q/k/v): one quantizer launch
  per distinct input instead of one per Linear, with bit-identical outputs. Returns
  the number of Linears switched."""
  n = 0
  for m in module.modules():
    if isinstance(m, Fp8DynamicLinear):
      m.share_input_quant = bool(enable)
      n += 1
  if not enable:
    ops.clear_shared_activation_quant()
  return n


def group_sibling_linears_(module: nn.Module, run=None, enable: bool = True) -> int:
  """Finds the `float8_per_row` (or `float8_weight_only`) Linears under `module` that are
  called back to back with the very same activation and lets each such run (two to eight
  Linears of one quant type) compute its outputs in one grouped GEMM launch, for
  `float8_per_row` on one shared quantization (SiblingGroup). `run` is a
  callable that performs one forward of the model (e.g. `lambda: model(**inputs)`); it is
  executed once under torch.no_grad() to observe the calls. Returns the number of groups
  formed. enable=False removes every group under `module` (no `run` needed)."""
  global _recorder
  groupable = (Fp8DynamicLinear, Fp8WeightOnlyLinear)
  for m in module.modules():
    if type(m) in groupable:
      m.sibling_group = None
  if not enable:
    return 0
  if run is None:
    raise ValueError("group_sibling_linears_ needs `run`, a callable doing one forward")
  mine = {id(m) for m in module.modules() if type(m) in groupable}
  _recorder = rec = _SiblingRecorder()
  try:
    with torch.no_grad():
      run()
  finally:
    _recorder = None
  groups = 0
  for siblings in rec.runs:
    siblings = [m for m in siblings if id(m) in mine and type(m) in groupable
                and m.sibling_group is None]
    siblings = [m for m in siblings if type(m) is type(siblings[0])
                and m.in_features == siblings[0].in_features
                and m._scale_mode_id == siblings[0]._scale_mode_id]
    while len(siblings) >= 2:
      take, siblings = siblings[:_native.MAX_GROUP], siblings[_native.MAX_GROUP:]
      g = SiblingGroup(take)
      for m in take:
        m.sibling_group = g
      groups += 1
  return groups


def linear_batch(pairs):
  """Several quantized Linears of one stage in ONE GEMM launch. `pairs` is a list of
  (x, [linear, ...]): every Linear of an entry is applied to that entry's activation; the
  entries do not depend on each other (in a double-stream block: the image-stream and the
  text-stream projections of the same stage, e.g. [(hidden, [to_q, to_k, to_v]),
  (encoder, [add_q_proj, add_k_proj, add_v_proj])]). Returns the outputs in the same
  nesting, bit-identical to calling the Linears one by one. For block forwards that are
  written against this package; `float8_per_row` Linears (one quantizer launch for the
  stage as well) or `float8_weight_only` ones; other Linears, mixed types or inference-mode
  tensors simply run one by one. Inside a compiled graph the stage is one traceable op
  (`cdit::linear_w8a8_batch` / `cdit::w8a16_batch`) without the shared-quantization state."""
  flat = [lin for _, lins in pairs for lin in lins]
  first = flat[0]
  plain = (len(flat) > _native.MAX_GROUP
           or len(pairs) > _native.MAX_ACTS
           or type(first) not in (Fp8DynamicLinear, Fp8WeightOnlyLinear)
           or any(type(lin) is not type(first) or lin.in_features != first.in_features
                  or lin._scale_mode_id != first._scale_mode_id for lin in flat)
           or any(not x.is_cuda or x.dtype != torch.bfloat16 for x, _ in pairs))
  compiling = torch.compiler.is_compiling()
  if not plain and not compiling:  # (no version counters on inference tensors: nothing is shared)
    plain = any(x.is_inference() for x, _ in pairs)
    if plain:
      _note_inference_bypass("linear_batch")
  if plain:
    return [[lin(x) for lin in lins] for x, lins in pairs]
  if compiling:
    # a compiled graph gets the stateless form: one traceable op for the whole stage
    op = (torch.ops.cdit.w8a16_batch if type(first) is Fp8WeightOnlyLinear
          else torch.ops.cdit.linear_w8a8_batch)
    args = ([x for x, _ in pairs], [lin.weight for lin in flat],
            [lin.weight_scale.reshape(-1) for lin in flat], [lin.bias for lin in flat],
            [len(lins) for _, lins in pairs], [lin.epilogue for lin in flat])
    outs = op(*args) if type(first) is Fp8WeightOnlyLinear else op(*args, first._scale_mode_id)
    result, p = [], 0
    for _, lins in pairs:
      result.append(list(outs[p:p + len(lins)]))
      p += len(lins)
    return result
  acts, result, rows = [], [], []
  for x, lins in pairs:
    x2 = ops._as_rows(x)
    M = x2.shape[0]
    outs = [torch.empty((M, lin.out_features), dtype=torch.bfloat16, device=x2.device) for lin in lins]
    result.append([o.view(*x.shape[:-1], lin.out_features) for o, lin in zip(outs, lins)])
    if M == 0:
      continue
    rows.append(x2)
    acts.append([None, None, [lin.weight for lin in lins], [lin.weight_scale for lin in lins],
                 [lin.bias for lin in lins], outs, [lin.epilogue for lin in lins]])
  if acts and type(first) is Fp8WeightOnlyLinear:
    ops.w8a16_batched_into([(x2, *act[2:]) for x2, act in zip(rows, acts)])
  elif acts:
    # one quantizer launch for the activations the cache does not hold, one GEMM launch
    for act, (q, s) in zip(acts, ops.shared_activation_quant_many(rows, first._scale_mode_id)):
      act[0], act[1] = q, s
    ops.gemm_rowwise_batched_into(acts)
  return result


#: Linears that hold an output computed ahead by precompute_stage (dropped at the next stage)
_precomputed_holders: list = []


def _stream_state(x2: torch.Tensor):
  capture_id = (_native.stream_capture_id(ops._stream_ptr(x2))
                if torch.cuda.is_current_stream_capturing() else 0)
  return (x2.device.index, ops._stream_ptr(x2)), capture_id


def _take_precomputed(lin: "_Fp8LinearBase", x: torch.Tensor):
  """The output precompute_stage left on `lin`, if `x` is the very activation it was computed
  from (same buffer, unmodified, same stream and graph capture); None otherwise. Either way
  the stash is emptied: an output is handed out once."""
  key, out, stream, capture_id = lin._precomputed
  lin._precomputed = None
  x2 = ops._as_rows(x)
  if key.matches(x2) and (stream, capture_id) == _stream_state(x2):
    return out.view(*x.shape[:-1], lin.out_features)
  return None


def _take_precomputed_traced(lin: "_Fp8LinearBase", x: torch.Tensor):
  """Inside a traced graph a stash is (activation, output) and is taken when `x` is that very
  tensor object (the tracer follows objects, not storage); emptied either way."""
  stash = lin._precomputed
  lin._precomputed = None
  if len(stash) == 2 and stash[0] is x:
    return stash[1]
  return None


def _stage_batchable(pairs, flat, first, traced: bool) -> bool:
  if (type(first) not in (Fp8DynamicLinear, Fp8WeightOnlyLinear) or len(flat) > _native.MAX_GROUP
      or len(pairs) > _native.MAX_ACTS
      or any(flat[i] is flat[j] for i in range(len(flat)) for j in range(i))
      or any(type(lin) is not type(first) or lin.in_features != first.in_features
             or lin._scale_mode_id != first._scale_mode_id or lin.sibling_group is not None
             for lin in flat)):
    return False
  return not any(not x.is_cuda or x.dtype != torch.bfloat16 or x.shape[-1] != first.in_features
                 or (not traced and x.is_inference()) for x, _ in pairs)


def precompute_stage(pairs) -> bool:
  """Runs `linear_batch(pairs)` now and leaves every output on its Linear, to be returned
  when that Linear is next called with the very same activation. For code that knows which
  Linears an unmodified module is about to call on which tensors (a forward pre-hook on an
  attention module sees `hidden_states` and `encoder_hidden_states` before the module's own
  code calls to_q / to_k / to_v and add_q_proj / add_k_proj / add_v_proj one by one): the
  stage then costs one quantizer launch and one GEMM launch, and the module's code stays as
  it is. A Linear that is called with anything else computes as usual, so a wrong guess
  costs time, not correctness. Outputs nobody collects are dropped when the next stage is
  precomputed. Returns False (nothing done) where linear_batch would not batch:
  inference-mode tensors, Linears of other types or of mixed types. Inside a traced graph
  (torch.compile) the stage becomes the one traceable batch op and an output goes to the
  Linear call that receives the same tensor object; whoever stashes there also clears what
  is left (`release_precomputed`). Not thread-safe, like the sibling groups."""
  flat = [lin for _, lins in pairs for lin in lins]
  if not flat:
    return False
  first = flat[0]
  if torch.compiler.is_compiling():
    if not _stage_batchable(pairs, flat, first, True):
      return False
    outs = linear_batch(pairs)
    for (x, lins), ys in zip(pairs, outs):
      for lin, y in zip(lins, ys):
        lin._precomputed = (x, y)
    return True
  for lin in _precomputed_holders:
    lin._precomputed = None
  _precomputed_holders.clear()
  if not _stage_batchable(pairs, flat, first, False):
    return False
  outs = linear_batch(pairs)
  for (x, lins), ys in zip(pairs, outs):
    x2 = ops._as_rows(x)
    stream, capture_id = _stream_state(x2)
    key = _InputKey(x2)
    for lin, y in zip(lins, ys):
      lin._precomputed = (key, y.view(-1, lin.out_features), stream, capture_id)
      _precomputed_holders.append(lin)
  return True


def release_precomputed(linears) -> None:
  """Drops what precompute_stage left on `linears` and nobody collected."""
  for lin in linears:
    if lin is not None and lin._precomputed is not None:
      lin._precomputed = None


def linear_on_cat(linear: nn.Module, xs) -> torch.Tensor:
  """`linear(torch.cat(xs, dim=-1))` for two sources without the concatenated tensor when
  `linear` is a `float8_per_row` Linear: the per-token quantizer reads the sources in place
  (FLUX single blocks: `proj_out(torch.cat([attn_output, mlp_hidden_states], dim=2))`,
  reference dataflow src/cache_dit/caching/patch_functors/functor_flux.py:68-80).
  Bit-identical to the plain expression, which is what runs for any other module, number of
  sources or dtype."""
  xs = list(xs)
  if (type(linear) is Fp8DynamicLinear and len(xs) == 2 and linear.sibling_group is None
      and all(x.is_cuda and x.dtype == torch.bfloat16 for x in xs)):
    return torch.ops.cdit.linear_w8a8_cat2(xs[0], xs[1], linear.weight, linear.weight_scale,
                                           linear.bias, linear._scale_mode_id, linear.epilogue)
  return linear(torch.cat(xs, dim=-1))


def dequantize_weight(linear: _Fp8LinearBase) -> torch.Tensor:
  """bf16 view of the quantized weight (for inspection and tests)."""
  return (linear.weight.to(torch.float32) * linear.weight_scale).to(torch.bfloat16)
