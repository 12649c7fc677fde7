"""Operator boundary: `torch.ops.cdit.*`, backed by libcdit_hip.so.

Mirrors the reference's own op for this path,
`cache_dit_torchao_ops::float8_inference_scaled_mm`
(src/cache_dit/quantization/torchao/_scaled_mm.py:94-137): same argument
order and meaning (a_data [M,K] e4m3 row-major, a_scale [M,1], b_data [K,N] =
`qweight.t()` column-major, b_scale [1,N], optional bias, out dtype id 0/1/2 =
fp16/bf16/fp32, use_fast_accum), same fake-impl shape rule, same error types.
On top of it the quantizer (torchao's per-row `Float8Tensor.from_hp`) and the
weight-only matmul are ops of their own.

Ownership and stream conventions follow the reference's native extension
(src/cache_dit/kernels/cuda/_ops_registery.py:35-59): this wrapper allocates
every output with torch.empty and launches on the current torch stream.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _native

_DTYPE_TO_ID = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}
_ID_TO_DTYPE = {v: k for k, v in _DTYPE_TO_ID.items()}
FP8 = torch.float8_e4m3fn


def encode_output_dtype(output_dtype: torch.dtype) -> int:
  dtype_id = _DTYPE_TO_ID.get(output_dtype)
  if dtype_id is None:
    raise ValueError(f"Unsupported float8 inference output dtype: {output_dtype}")
  return dtype_id


def decode_output_dtype(dtype_id: int) -> torch.dtype:
  output_dtype = _ID_TO_DTYPE.get(dtype_id)
  if output_dtype is None:
    raise ValueError(f"Unsupported float8 inference output dtype id: {dtype_id}")
  return output_dtype


def _stream_ptr(t: torch.Tensor) -> int:
  return torch._C._cuda_getCurrentRawStream(t.device.index)


class _DeviceOf:
  """Makes `t`'s device current for the launch when it is not already (the kernels
  run on the current HIP device); free when it is."""
  __slots__ = ("guard", )

  def __init__(self, t: torch.Tensor):
    self.guard = None if t.device.index == torch.cuda.current_device() else torch.cuda.device(
        t.device)

  def __enter__(self):
    if self.guard is not None:
      self.guard.__enter__()

  def __exit__(self, *exc):
    if self.guard is not None:
      self.guard.__exit__(*exc)


def activation_workspace(M: int, K: int, device: torch.device):
  """(codes [M,K] e4m3, scales [M] fp32) scratch for one Linear forward, fresh from
  PyTorch's caching allocator: a block freed on a stream is handed out again on that
  stream, so consecutive Linears reuse the same memory without this module keeping any
  buffer alive (a module-level buffer created while a graph-capturing front end warms up
  inside its private pool would be an allocation that pool never sees released)."""
  return (torch.empty((M, K), dtype=FP8, device=device),
          torch.empty((M, ), dtype=torch.float32, device=device))


def amax_workspace(device: torch.device) -> torch.Tensor:
  """4 bytes of device scratch for the per-tensor quantizer."""
  return torch.empty((1,), dtype=torch.int32, device=device)


def _require_cuda(name: str, *tensors: Optional[torch.Tensor]) -> None:
  for t in tensors:
    if t is not None and not t.is_cuda:
      raise RuntimeError(f"{name}: expected tensors on the GPU, got a {t.device} tensor "
                         "(there is no CPU path)")


# --------------------------------------------------------------------------- raw launchers
# These take already-validated 2-D tensors and write into caller-provided outputs.


#: Buffers whose bf16 values were never written: ln_modulate_quant(materialize=False) returns
#: such a tensor, and only its FP8 codes (handed over through the shared-quantization lookup)
#: mean anything. storage address -> (weak reference to the storage, version counter at
#: hand-over). The storage object lives as long as any view of the buffer does, so the entry
#: covers every reshape and slice of it and disappears with the last of them.
_codes_only: dict = {}


def _mark_codes_only(y: torch.Tensor) -> None:
  import weakref
  st = y.untyped_storage()
  key = st.data_ptr()
  _codes_only[key] = (weakref.ref(st, lambda _r, k=key: _codes_only.pop(k, None)), y._version)


def is_codes_only(x: torch.Tensor) -> bool:
  """Whether x aliases a buffer that ln_modulate_quant(materialize=False) left unwritten
  (and nobody has written through PyTorch since)."""
  if not _codes_only or x.is_inference():
    return False
  st = x.untyped_storage()
  entry = _codes_only.get(st.data_ptr())
  return entry is not None and entry[0]() is st and entry[1] == x._version


def _reject_codes_only(what: str, *xs: torch.Tensor) -> None:
  """Every path that reads an activation's bf16 values calls this first: reading a
  codes-only buffer would quantize (or multiply) uninitialised memory without any error."""
  if not _codes_only:
    return
  for x in xs:
    if is_codes_only(x):
      raise RuntimeError(
          f"{what}: this activation comes from ln_modulate_quant(materialize=False), which "
          "writes FP8 codes only, and its codes were not found by the consumer (they are handed "
          "over per device and stream to float8_per_row Linears with share_activation_quant_ "
          "switched on, a few activations deep). Call ln_modulate_quant with materialize=True "
          "for this consumer.")


def quant_tensorwise_into(x2: torch.Tensor, q: torch.Tensor, scale: torch.Tensor,
                          amax_ws: torch.Tensor, scale_mode_id: int) -> None:
  """Per-tensor quantizer: one scale for all of x2, written to every scale[m].
  amax_ws: 4 bytes of device scratch (an int32 tensor of one element)."""
  _reject_codes_only("quant_tensorwise_into", x2)
  M, K = x2.shape
  with _DeviceOf(x2):
    _native.check(_native.load().cdit_fp8_quant_tensorwise(x2.data_ptr(), M, K, x2.stride(0),
                                                           q.data_ptr(), q.stride(0),
                                                           scale.data_ptr(), amax_ws.data_ptr(),
                                                           scale_mode_id, _stream_ptr(x2)))


def quant_rowwise_into(x2: torch.Tensor, q: torch.Tensor, scale: torch.Tensor,
                       scale_mode_id: int, gemm_follows: bool = False) -> None:
  """gemm_follows: the codes are read by a GEMM launched next on this stream (a cache
  hint for the quantizer; the results are the same)."""
  _reject_codes_only("quant_rowwise_into", x2)
  M, K = x2.shape
  mode = scale_mode_id | (_native.QUANT_GEMM_FOLLOWS if gemm_follows else 0)
  with _DeviceOf(x2):
    _native.check(_native.load().cdit_fp8_quant_rowwise(x2.data_ptr(), M, K, x2.stride(0),
                                                        q.data_ptr(), q.stride(0),
                                                        scale.data_ptr(), mode,
                                                        _stream_ptr(x2)))


def quant_rowwise_batched_into(items, scale_mode_id: int) -> None:
  """quant_rowwise_into for several activations of one K in a single launch. `items` is a
  list of (x2 [M,K] bf16, q [M,K] e4m3, scale [M] fp32), at most _native.MAX_ACTS of them on
  one device; the codes are taken to be read by a GEMM launched next. Bit-identical to one
  quant_rowwise_into per item."""
  _reject_codes_only("quant_rowwise_batched_into", *[x for x, _, _ in items])
  import ctypes
  n = len(items)
  x0 = items[0][0]
  K = x0.shape[1]
  if any(x.shape[1] != K or x.device != x0.device for x, _, _ in items):
    raise ValueError("quant_rowwise_batched_into: the activations must share K and the device")
  vp, i64 = ctypes.c_void_p, ctypes.c_int64
  with _DeviceOf(x0):
    _native.check(_native.load().cdit_fp8_quant_rowwise_batched(
        n, (vp * n)(*[x.data_ptr() for x, _, _ in items]), (i64 * n)(*[x.shape[0] for x, _, _ in items]),
        K, (i64 * n)(*[x.stride(0) for x, _, _ in items]), (vp * n)(*[q.data_ptr() for _, q, _ in items]),
        (i64 * n)(*[q.stride(0) for _, q, _ in items]), (vp * n)(*[s.data_ptr() for _, _, s in items]),
        scale_mode_id, _stream_ptr(x0)))


def quant_rowwise_cat2_into(x1: torch.Tensor, x2: torch.Tensor, q: torch.Tensor, scale: torch.Tensor,
                            scale_mode_id: int) -> None:
  """Quantizes the rows [x1 | x2] (bf16 [M,K1] and [M,K2]) into q [M,K1+K2] / scale [M] without
  the concatenated tensor; the results are those of quant_rowwise_into on torch.cat."""
  _reject_codes_only("quant_rowwise_cat2_into", x1, x2)
  with _DeviceOf(x1):
    _native.check(_native.load().cdit_fp8_quant_rowwise_cat2(
        x1.data_ptr(), x1.shape[1], x1.stride(0), x2.data_ptr(), x2.shape[1], x2.stride(0),
        x1.shape[0], q.data_ptr(), q.stride(0), scale.data_ptr(), scale_mode_id, _stream_ptr(x1)))


def cat2_quant_ok(x1: torch.Tensor, x2: torch.Tensor) -> bool:
  """Whether quant_rowwise_cat2_into takes these two row blocks (else: concatenate)."""
  return (x1.shape[0] == x2.shape[0] and x1.shape[1] % 8 == 0 and x2.shape[1] % 8 == 0
          and x1.shape[1] + x2.shape[1] <= 16384 and x1.stride(0) % 8 == 0 and x2.stride(0) % 8 == 0
          and x1.data_ptr() % 16 == 0 and x2.data_ptr() % 16 == 0)


def gemm_rowwise_into(a: torch.Tensor, a_scale: torch.Tensor, w: torch.Tensor,
                      w_scale: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                      epilogue: int) -> None:
  """a [M,K] e4m3, w [N,K] e4m3 (row-major), scales fp32 contiguous, out [M,N] fp16,
  bf16 or fp32; bias in the output's dtype (none for an fp32 output)."""
  M, K = a.shape
  N = w.shape[0]
  with _DeviceOf(a):
    _native.check(_native.load().cdit_fp8_gemm_rowwise(
        a.data_ptr(), a_scale.data_ptr(), w.data_ptr(), w_scale.data_ptr(),
        bias.data_ptr() if bias is not None else None, out.data_ptr(), M, N, K, a.stride(0),
        w.stride(0), out.stride(0), epilogue, encode_output_dtype(out.dtype), _stream_ptr(a)))


def gemm_rowwise_grouped_into(a: torch.Tensor, a_scale: torch.Tensor, weights, w_scales, biases,
                              outs, epilogues) -> None:
  """Sibling GEMMs on one activation (a [M,K] e4m3 with scales [M]) as one launch: member
  p is weights[p] [N_p,K] e4m3 with the same row stride, w_scales[p] fp32, biases[p] bf16
  or None, outs[p] [M,N_p] bf16, epilogues[p]. Bit-identical to one gemm_rowwise_into per
  member."""
  import ctypes
  n = len(weights)
  M, K = a.shape
  vp, i64 = ctypes.c_void_p, ctypes.c_int64
  ldb = weights[0].stride(0)
  if any(w.stride(0) != ldb or w.shape[1] != K for w in weights):
    raise ValueError("gemm_rowwise_grouped_into: the weights must share K and the row stride")
  with _DeviceOf(a):
    _native.check(_native.load().cdit_fp8_gemm_rowwise_grouped(
        a.data_ptr(), a_scale.data_ptr(), M, K, a.stride(0), n,
        (vp * n)(*[w.data_ptr() for w in weights]), (vp * n)(*[s.data_ptr() for s in w_scales]),
        (vp * n)(*[b.data_ptr() if b is not None else None for b in biases]),
        (vp * n)(*[o.data_ptr() for o in outs]), (i64 * n)(*[w.shape[0] for w in weights]), ldb,
        (i64 * n)(*[o.stride(0) for o in outs]), (ctypes.c_int * n)(*[int(e) for e in epilogues]),
        _stream_ptr(a)))


def gemm_rowwise_batched_into(acts) -> None:
  """Independent GEMMs of one stage as one launch. `acts` is a list of
  (a [M,K] e4m3, a_scale [M], weights, w_scales, biases, outs, epilogues): one entry per
  activation, its members listed as for gemm_rowwise_grouped_into; all activations and
  weights share K and their row strides. Bit-identical to one gemm_rowwise_into per
  member."""
  import ctypes
  vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
  a0 = acts[0][0]
  K, lda, ldb = a0.shape[1], a0.stride(0), acts[0][2][0].stride(0)
  ws, wss, bs, outs, epis, per_act = [], [], [], [], [], []
  for a, a_s, weights, w_scales, biases, o, e in acts:
    if a.shape[1] != K or a.stride(0) != lda or a.device != a0.device:
      raise ValueError("gemm_rowwise_batched_into: the activations must share K, the row stride "
                       "and the device")
    if any(w.stride(0) != ldb or w.shape[1] != K for w in weights):
      raise ValueError("gemm_rowwise_batched_into: the weights must share K and the row stride")
    ws += weights
    wss += w_scales
    bs += biases
    outs += o
    epis += e
    per_act.append(len(weights))
  n, na = len(ws), len(acts)
  with _DeviceOf(a0):
    _native.check(_native.load().cdit_fp8_gemm_rowwise_batched(
        na, (vp * na)(*[t[0].data_ptr() for t in acts]), (vp * na)(*[t[1].data_ptr() for t in acts]),
        (i64 * na)(*[t[0].shape[0] for t in acts]), K, lda, (ci * na)(*per_act),
        (vp * n)(*[w.data_ptr() for w in ws]), (vp * n)(*[s.data_ptr() for s in wss]),
        (vp * n)(*[b.data_ptr() if b is not None else None for b in bs]),
        (vp * n)(*[o.data_ptr() for o in outs]), (i64 * n)(*[w.shape[0] for w in ws]), ldb,
        (i64 * n)(*[o.stride(0) for o in outs]), (ci * n)(*[int(e) for e in epis]), _stream_ptr(a0)))


def w8a16_batched_into(acts) -> None:
  """Independent weight-only GEMMs of one stage as one launch. `acts` is a list of
  (x2 [M,K] bf16, weights, w_scales, biases, outs, epilogues): one entry per activation, its
  members e4m3 [N_p,K] weights with a common row stride, fp32 scales, bf16 biases or None,
  bf16 outputs [M,N_p] and epilogue flags. Activations whose row strides differ are
  launched apart. Bit-identical to one w8a16_into per member."""
  _reject_codes_only("w8a16_batched_into", *[t[0] for t in acts])
  import ctypes
  vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
  x0 = acts[0][0]
  if any(t[0].stride(0) != x0.stride(0) for t in acts[1:]):
    for t in acts:
      w8a16_batched_into([t])
    return
  K, lda, ldb = x0.shape[1], x0.stride(0), acts[0][1][0].stride(0)
  ws, wss, bs, outs, epis, per_act = [], [], [], [], [], []
  for x, weights, w_scales, biases, o, e in acts:
    if x.shape[1] != K or x.device != x0.device or x.dtype != torch.bfloat16 or x.stride(1) != 1:
      raise ValueError("w8a16_batched_into: the activations must be bf16 rows of one K on one device")
    if any(w.stride(0) != ldb or w.shape[1] != K for w in weights):
      raise ValueError("w8a16_batched_into: the weights must share K and the row stride")
    ws += weights
    wss += w_scales
    bs += biases
    outs += o
    epis += e
    per_act.append(len(weights))
  n, na = len(ws), len(acts)
  with _DeviceOf(x0):
    _native.check(_native.load().cdit_w8a16_gemm_batched(
        na, (vp * na)(*[t[0].data_ptr() for t in acts]), (i64 * na)(*[t[0].shape[0] for t in acts]),
        K, lda, (ci * na)(*per_act), (vp * n)(*[w.data_ptr() for w in ws]),
        (vp * n)(*[s.data_ptr() for s in wss]),
        (vp * n)(*[b.data_ptr() if b is not None else None for b in bs]),
        (vp * n)(*[o.data_ptr() for o in outs]), (i64 * n)(*[w.shape[0] for w in ws]), ldb,
        (i64 * n)(*[o.stride(0) for o in outs]), (ci * n)(*[int(e) for e in epis]), _stream_ptr(x0)))


def w8a16_into(x2: torch.Tensor, w: torch.Tensor, w_scale: torch.Tensor,
               bias: Optional[torch.Tensor], out: torch.Tensor, epilogue: int) -> None:
  _reject_codes_only("w8a16_into", x2)
  M, K = x2.shape
  N = w.shape[0]
  with _DeviceOf(x2):
    _native.check(_native.load().cdit_w8a16_gemm(
        x2.data_ptr(), w.data_ptr(), w_scale.data_ptr(),
        bias.data_ptr() if bias is not None else None, out.data_ptr(), M, N, K, x2.stride(0),
        w.stride(0), out.stride(0), epilogue, _native.DT_BF16, _stream_ptr(x2)))


class _SharedQuant:
  """An activation quantized on a (device, stream): the input view (kept alive, so its
  storage cannot be freed and handed out again), its version counter, the codes / scales
  computed from it, and the id of the graph capture it was made in (0: none)."""
  __slots__ = ("x", "version", "mode", "q", "s", "capture_id")

  def matches(self, x2: torch.Tensor, scale_mode_id: int) -> bool:
    return (self.mode == scale_mode_id and self.version == x2._version
            and self.x.data_ptr() == x2.data_ptr() and self.x.shape == x2.shape
            and self.x.stride() == x2.stride()
            and self.x.untyped_storage().data_ptr() == x2.untyped_storage().data_ptr())


#: (device, stream) -> most recent entries first. A DiT block keeps at most a few
#: quantized activations in use at a time (image and text stream normed inputs, then the
#: MLP input), so a handful of entries is enough.
_shared_quant: dict = {}
_SHARED_QUANT_ENTRIES = 4
quant_launches = 0  # quantizer launches issued through shared_activation_quant (for tests)


def _shared_entries(x2: torch.Tensor):
  """The live entries of x2's (device, stream), and the current capture id. Entries made
  inside a graph capture belong to that capture alone (their codes live in that graph's
  pool and are only valid inside its replays): a list made under another capture id, or
  on the other side of a capture boundary, is dropped."""
  dev = x2.device
  capture_id = (_native.stream_capture_id(_stream_ptr(x2))
                if torch.cuda.is_current_stream_capturing() else 0)
  key = (dev.index, torch._C._cuda_getCurrentRawStream(dev.index))
  entries = _shared_quant.get(key)
  if entries is None or (entries and entries[0].capture_id != capture_id):
    entries = _shared_quant[key] = []
  return entries, capture_id


def _remember_quant(entries, capture_id, x2, scale_mode_id, q, s) -> None:
  e = _SharedQuant()
  e.x, e.version, e.mode, e.q, e.s, e.capture_id = x2, x2._version, scale_mode_id, q, s, capture_id
  entries.insert(0, e)
  del entries[_SHARED_QUANT_ENTRIES:]


def shared_activation_quant(x2: torch.Tensor, scale_mode_id: int):
  """Codes and scales of `x2` [M,K], reusing an earlier result when the same buffer
  (storage, offset, shape, strides), unmodified since (same `_version`), is quantized
  again on the same stream -- sibling Linears such as to_q / to_k / to_v (and proj_mlp
  in FLUX single blocks) all read one normalized activation (reference dataflow:
  src/cache_dit/caching/patch_functors/functor_flux.py:60-67) -- or when its producer
  already delivered them (ln_modulate_quant). The results are bit-identical to
  quantizing again. In-place changes made through PyTorch bump `_version` and miss;
  writes by foreign kernels into a live input between two sibling calls would not be
  seen, which is why sharing is opt-in."""
  global quant_launches
  dev = x2.device
  M, K = x2.shape
  if x2.is_inference():
    # inference-mode tensors carry no version counter: an in-place change could not be
    # told from an unchanged buffer, so nothing is shared (torch.no_grad() keeps it)
    q = torch.empty((M, K), dtype=FP8, device=dev)
    s = torch.empty((M, ), dtype=torch.float32, device=dev)
    quant_rowwise_into(x2, q, s, scale_mode_id, gemm_follows=True)
    quant_launches += 1
    return q, s
  entries, capture_id = _shared_entries(x2)
  for e in entries:
    if e.matches(x2, scale_mode_id):
      return e.q, e.s
  q = torch.empty((M, K), dtype=FP8, device=dev)
  s = torch.empty((M, ), dtype=torch.float32, device=dev)
  quant_rowwise_into(x2, q, s, scale_mode_id, gemm_follows=True)
  quant_launches += 1
  _remember_quant(entries, capture_id, x2, scale_mode_id, q, s)
  return q, s


def shared_activation_quant_many(x2s, scale_mode_id: int):
  """shared_activation_quant for the activations of one stage: what the cache does not hold
  is quantized in ONE launch (cdit_fp8_quant_rowwise_batched) when the activations share K
  and the device. Returns [(codes, scales), ...] in the order of `x2s`."""
  global quant_launches
  x0 = x2s[0]
  if (len(x2s) < 2 or len(x2s) > _native.MAX_ACTS
      or any(x.is_inference() or x.shape[1] != x0.shape[1] or x.device != x0.device for x in x2s)):
    return [shared_activation_quant(x, scale_mode_id) for x in x2s]
  entries, capture_id = _shared_entries(x0)
  result, missing = [None] * len(x2s), []
  for i, x in enumerate(x2s):
    for e in entries:
      if e.matches(x, scale_mode_id):
        result[i] = (e.q, e.s)
        break
    else:
      if any(x is x2s[j] for j in missing):  # the same tensor twice in one stage
        continue
      missing.append(i)
  if len(missing) == 1:
    result[missing[0]] = shared_activation_quant(x2s[missing[0]], scale_mode_id)
  elif missing:
    items = []
    for i in missing:
      x = x2s[i]
      q = torch.empty(x.shape, dtype=FP8, device=x.device)
      s = torch.empty((x.shape[0], ), dtype=torch.float32, device=x.device)
      items.append((x, q, s))
    quant_rowwise_batched_into(items, scale_mode_id)
    quant_launches += 1
    for i, (x, q, s) in zip(missing, items):
      _remember_quant(entries, capture_id, x, scale_mode_id, q, s)
      result[i] = (q, s)
  for i, x in enumerate(x2s):  # repeats of a tensor that was quantized just now
    if result[i] is None:
      result[i] = shared_activation_quant(x, scale_mode_id)
  return result


def clear_shared_activation_quant() -> None:
  _shared_quant.clear()


def linear_w8a8_into(x2: torch.Tensor, w: torch.Tensor, w_scale: torch.Tensor,
                     bias: Optional[torch.Tensor], out: torch.Tensor, q_ws: torch.Tensor,
                     s_ws: torch.Tensor, scale_mode_id: int, epilogue: int) -> None:
  """Quantizer + GEMM of one Linear forward in a single library call."""
  _reject_codes_only("linear_w8a8_into", x2)
  M, K = x2.shape
  N = w.shape[0]
  with _DeviceOf(x2):
    rc = _native.load().cdit_fp8_linear_w8a8(
        x2.data_ptr(), w.data_ptr(), w_scale.data_ptr(),
        bias.data_ptr() if bias is not None else None, out.data_ptr(), q_ws.data_ptr(),
        s_ws.data_ptr(), M, N, K, x2.stride(0), w.stride(0), out.stride(0), scale_mode_id,
        epilogue, _native.DT_BF16, _stream_ptr(x2))
  if rc:
    _native.check(rc)


# --------------------------------------------------------------------------- op definitions

torch.library.define(
    "cdit::fp8_rowwise_quant",
    "(Tensor x, int scale_mode=0) -> (Tensor, Tensor)",
)
torch.library.define(
    "cdit::float8_inference_scaled_mm",
    "(Tensor a_data, Tensor a_scale, Tensor b_data, Tensor b_scale, Tensor? bias, "
    "int out_dtype_id, bool use_fast_accum, int epilogue=0) -> Tensor",
)
torch.library.define(
    "cdit::linear_w8a8",
    "(Tensor x, Tensor weight, Tensor weight_scale, Tensor? bias, int scale_mode=0, "
    "int epilogue=0, int granularity=0, bool share_input_quant=False) -> Tensor",
)
torch.library.define(
    "cdit::linear_w8a8_cat2",
    "(Tensor x1, Tensor x2, Tensor weight, Tensor weight_scale, Tensor? bias, int scale_mode=0, "
    "int epilogue=0) -> Tensor",
)
torch.library.define(
    "cdit::linear_w8a8_batch",
    "(Tensor[] xs, Tensor[] weights, Tensor[] weight_scales, Tensor?[] biases, "
    "int[] members_per_act, int[] epilogues, int scale_mode=0) -> Tensor[]",
)
torch.library.define(
    "cdit::w8a16_batch",
    "(Tensor[] xs, Tensor[] weights, Tensor[] weight_scales, Tensor?[] biases, "
    "int[] members_per_act, int[] epilogues) -> Tensor[]",
)
torch.library.define(
    "cdit::w8a16_mm",
    "(Tensor x, Tensor b_data, Tensor b_scale, Tensor? bias, int out_dtype_id, "
    "int epilogue=0) -> Tensor",
)


def _as_rows(x: torch.Tensor) -> torch.Tensor:
  x2 = x.reshape(-1, x.shape[-1])
  if x2.stride(-1) != 1:
    x2 = x2.contiguous()
  return x2


@torch.library.impl("cdit::fp8_rowwise_quant", "CUDA")
def _fp8_rowwise_quant(x: torch.Tensor, scale_mode: int = 0) -> Tuple[torch.Tensor, torch.Tensor]:
  if x.dtype != torch.bfloat16:
    raise ValueError(f"cdit::fp8_rowwise_quant: x must be bfloat16, got {x.dtype}")
  if x.dim() < 1:
    raise ValueError("cdit::fp8_rowwise_quant: x must have at least one dimension")
  if scale_mode not in (0, 1):
    raise ValueError(f"cdit::fp8_rowwise_quant: scale_mode must be 0 or 1, got {scale_mode}")
  x2 = _as_rows(x)
  q = torch.empty(x2.shape, dtype=FP8, device=x.device)
  scale = torch.empty((x2.shape[0], ), dtype=torch.float32, device=x.device)
  if x2.numel() > 0 or x2.shape[0] > 0:
    quant_rowwise_into(x2, q, scale, scale_mode)
  return q.reshape(x.shape), scale.reshape(*x.shape[:-1], 1)


@torch.library.register_fake("cdit::fp8_rowwise_quant")
def _fake_fp8_rowwise_quant(x, scale_mode=0):
  return (x.new_empty(x.shape, dtype=FP8), x.new_empty((*x.shape[:-1], 1), dtype=torch.float32))


def _weight_rows(b_data: torch.Tensor, name: str) -> torch.Tensor:
  """b_data is [K,N]; the kernels want the [N,K] row-major weight it is the
  transpose of (the reference passes `qweight.t()`, stride (1, K))."""
  if b_data.dim() != 2:
    raise ValueError(f"{name}: b_data must be 2-D [K,N], got shape {tuple(b_data.shape)}")
  w = b_data.t()
  if w.stride(-1) != 1:
    # a row-major [K,N] operand: materialise the K-contiguous layout once.
    w = w.contiguous()
  return w


def _aligned16(t: torch.Tensor) -> torch.Tensor:
  """The tuned kernels fetch scales and bias in 16-byte pieces; a slice that starts
  elsewhere is copied once rather than sent to the element-wise kernel."""
  return t if t.data_ptr() % 16 == 0 else t.clone()


def _scale_vector(scale: torch.Tensor, n: int) -> torch.Tensor:
  s = scale.reshape(-1).to(torch.float32)
  if s.numel() == 1 and n != 1:
    s = s.expand(n)
  return _aligned16(s.contiguous())


@torch.library.impl("cdit::float8_inference_scaled_mm", "CUDA")
def _float8_inference_scaled_mm(a_data, a_scale, b_data, b_scale, bias, out_dtype_id,
                                use_fast_accum, epilogue=0):
  del use_fast_accum  # a cuBLASLt hint; fp32 accumulation is the only mode here
  name = "cdit::float8_inference_scaled_mm"
  out_dtype = decode_output_dtype(out_dtype_id)
  if a_data.dtype != FP8 or b_data.dtype != FP8:
    raise ValueError(f"{name}: a_data/b_data must be float8_e4m3fn, got {a_data.dtype}/"
                     f"{b_data.dtype}")
  w = _weight_rows(b_data, name)
  a2 = _as_rows(a_data)
  M, K = a2.shape
  N = w.shape[0]
  if w.shape[1] != K:
    raise ValueError(f"{name}: shape mismatch a {tuple(a_data.shape)} x b {tuple(b_data.shape)}")
  if a_scale.numel() not in (1, M) or b_scale.numel() not in (1, N):
    raise ValueError(f"{name}: expected a_scale with {M} (or 1) and b_scale with {N} (or 1) "
                     f"elements, got {a_scale.numel()} and {b_scale.numel()}")
  # a scalar scale is a tensor-wise one (how float8_per_tensor reaches the reference's op,
  # which hands it to torch._scaled_mm as is): the kernel takes it as a constant vector
  a_s = _scale_vector(a_scale, M)
  b_s = _scale_vector(b_scale, N)
  if bias is not None and bias.numel() != N:
    raise ValueError(f"{name}: bias must have {N} elements")
  out = torch.empty((M, N), dtype=out_dtype, device=a_data.device)
  if out_dtype == torch.float32 and bias is not None:
    # the reference adds the bias after the matmul for an fp32 output
    # (_scaled_mm.py:71-81); with a fused activation it has to go in before that
    if int(epilogue) != 0:
      raise ValueError(f"{name}: an fp32 output with bias cannot fuse an activation")
    gemm_rowwise_into(a2, a_s, w, b_s, None, out, 0)
    out = out + bias.reshape(-1)
  else:
    if bias is not None:
      bias = _aligned16(bias.reshape(-1).to(out_dtype).contiguous())
    gemm_rowwise_into(a2, a_s, w, b_s, bias, out, int(epilogue))
  return out.reshape(*a_data.shape[:-1], N)


@torch.library.register_fake("cdit::float8_inference_scaled_mm")
def _fake_float8_inference_scaled_mm(a_data, a_scale, b_data, b_scale, bias, out_dtype_id,
                                     use_fast_accum, epilogue=0):
  return a_data.new_empty((*a_data.shape[:-1], b_data.shape[-1]),
                          dtype=decode_output_dtype(out_dtype_id))


torch.library.define(
    "cdit::ln_modulate_quant",
    "(Tensor x, Tensor shift, Tensor scale, float eps=1e-6, int scale_mode=0, "
    "bool write_y=True) -> (Tensor, Tensor, Tensor)",
)


@torch.library.impl("cdit::ln_modulate_quant", "CUDA")
def _ln_modulate_quant(x, shift, scale, eps=1e-6, scale_mode=0, write_y=True):
  """LayerNorm (no affine) over the last dimension, `* (1 + scale) + shift`, and the
  per-row FP8 quantization of the result, in one kernel. x bf16 [..., K]; shift, scale
  bf16 with K elements per modulation vector, either one vector for everything or one per
  leading index of x (AdaLN: [B, 1, K] for x [B, S, K]). Returns (y bf16 like x -- left
  unwritten when write_y is False --, codes e4m3 like x, scales fp32 [..., 1])."""
  name = "cdit::ln_modulate_quant"
  if x.dtype != torch.bfloat16 or shift.dtype != torch.bfloat16 or scale.dtype != torch.bfloat16:
    raise ValueError(f"{name}: x, shift and scale must be bfloat16, got {x.dtype}, {shift.dtype}, "
                     f"{scale.dtype}")
  if x.dim() < 1 or x.shape[-1] == 0:
    raise ValueError(f"{name}: x needs a non-empty last dimension")
  if scale_mode not in (0, 1):
    raise ValueError(f"{name}: scale_mode must be 0 or 1, got {scale_mode}")
  K = x.shape[-1]
  x2 = _as_rows(x)
  M = x2.shape[0]
  if shift.shape != scale.shape or shift.shape[-1] != K or shift.numel() % K != 0:
    raise ValueError(f"{name}: shift {tuple(shift.shape)} / scale {tuple(scale.shape)} do not "
                     f"hold vectors of K={K} elements")
  nb = shift.numel() // K
  if nb != 1 and not (x.dim() >= 2 and nb == x.shape[0] and M % nb == 0):
    raise ValueError(f"{name}: {nb} modulation vectors for x of shape {tuple(x.shape)}: expected "
                     "one, or one per index of x's first dimension")
  sh2, sc2 = shift.reshape(nb, K).contiguous(), scale.reshape(nb, K).contiguous()
  y = torch.empty((M, K), dtype=torch.bfloat16, device=x.device)
  q = torch.empty((M, K), dtype=FP8, device=x.device)
  s = torch.empty((M, ), dtype=torch.float32, device=x.device)
  if M > 0:
    with _DeviceOf(x2):
      _native.check(_native.load().cdit_fp8_ln_modulate_quant(
          x2.data_ptr(), M, K, x2.stride(0), sh2.data_ptr(), sc2.data_ptr(), K,
          M if nb == 1 else M // nb, float(eps), y.data_ptr() if write_y else None, K,
          q.data_ptr(), K, s.data_ptr(), int(scale_mode), _stream_ptr(x2)))
  return y.view(x.shape), q.view(x.shape), s.view(*x.shape[:-1], 1)


@torch.library.register_fake("cdit::ln_modulate_quant")
def _fake_ln_modulate_quant(x, shift, scale, eps=1e-6, scale_mode=0, write_y=True):
  return (x.new_empty(x.shape), x.new_empty(x.shape, dtype=FP8),
          x.new_empty((*x.shape[:-1], 1), dtype=torch.float32))


def ln_modulate_quant(x: torch.Tensor, shift: torch.Tensor, scale: torch.Tensor, eps: float = 1e-6,
                      scale_mode: str = "bf16div", materialize: bool = True) -> torch.Tensor:
  """`layer_norm(x) * (1 + scale) + shift` whose FP8 codes are produced in the same pass
  and handed to the quantized Linears that consume the result: they find them under the
  returned tensor's identity (the lookup `share_activation_quant_` switches on) and skip
  their own quantizer launch. The returned tensor is a drop-in for the unfused
  expression. With materialize=False its bf16 values are NOT written (the kernel then
  only writes codes and scales): only for a caller that knows every consumer is such a
  Linear. Inside torch.inference_mode() tensors carry no version counter to key the
  lookup on; the bf16 tensor is then always written and nothing is handed over."""
  _require_cuda("ln_modulate_quant", x, shift, scale)
  mode_id = _native.SCALE_MODE_IDS[scale_mode]
  # no hand-over (the bf16 tensor is then always written): inference-mode tensors carry no
  # version counter, and a graph being traced by torch.compile never shares codes (its
  # Linears run with sharing off)
  no_handover = (x.is_inference() or torch.is_inference_mode_enabled()
                 or torch.compiler.is_compiling())
  write_y = bool(materialize or no_handover)
  y, q, s = torch.ops.cdit.ln_modulate_quant(x, shift, scale, float(eps), mode_id, write_y)
  if not no_handover and y.numel() > 0:
    y2 = y.view(-1, y.shape[-1])
    entries, capture_id = _shared_entries(y2)
    _remember_quant(entries, capture_id, y2, mode_id, q.view(y2.shape), s.view(-1))
    if not write_y:
      _mark_codes_only(y)  # a consumer that does not find the codes raises
  return y


GRANULARITY_PER_ROW, GRANULARITY_PER_TENSOR = 0, 1


@torch.library.impl("cdit::linear_w8a8", "CUDA")
def _linear_w8a8(x, weight, weight_scale, bias, scale_mode=0, epilogue=0, granularity=0,
                 share_input_quant=False):
  """One quantized nn.Linear forward in the w8a8 dynamic modes as a single opaque op, what
  the reference gets by keeping torchao's Float8Tensor `aten.linear` behind one
  `torch.library` op (src/cache_dit/quantization/torchao/_scaled_mm.py:94-137, patched in
  at :338-357): x bf16 [..., K], weight e4m3 [N, K] (the nn.Linear layout), weight_scale
  fp32 with N elements, bias bf16 [N] or None -> bf16 [..., N]. granularity 0: per-token
  activation scales, 1: one scale for the whole activation. Workspaces are taken inside
  the op, so a traced graph only sees tensors in and a tensor out."""
  name = "cdit::linear_w8a8"
  if x.dtype != torch.bfloat16:
    raise ValueError(f"{name}: x must be bfloat16, got {x.dtype}")
  if weight.dtype != FP8 or weight.dim() != 2:
    raise ValueError(f"{name}: weight must be float8_e4m3fn [N,K], got {weight.dtype} "
                     f"{tuple(weight.shape)}")
  N, K = weight.shape
  if x.shape[-1] != K:
    raise ValueError(f"{name}: shape mismatch x {tuple(x.shape)} x weight {tuple(weight.shape)}")
  if scale_mode not in (0, 1) or granularity not in (0, 1):
    raise ValueError(f"{name}: scale_mode and granularity must be 0 or 1")
  if weight_scale.numel() != N or weight_scale.dtype != torch.float32:
    raise ValueError(f"{name}: weight_scale must hold {N} float32 values")
  if bias is not None and (bias.numel() != N or bias.dtype != torch.bfloat16):
    raise ValueError(f"{name}: bias must hold {N} bfloat16 values")
  x2 = _as_rows(x)
  w = weight if weight.stride(-1) == 1 else weight.contiguous()
  w_s = weight_scale if weight_scale.is_contiguous() else weight_scale.contiguous()
  if bias is not None and not bias.is_contiguous():
    bias = bias.contiguous()
  M = x2.shape[0]
  out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
  if M > 0:
    if granularity == GRANULARITY_PER_TENSOR:
      q, s = activation_workspace(M, K, x2.device)
      quant_tensorwise_into(x2, q, s, amax_workspace(x2.device), int(scale_mode))
      gemm_rowwise_into(q, s, w, w_s, bias, out, int(epilogue))
    elif share_input_quant:
      q, s = shared_activation_quant(x2, int(scale_mode))
      gemm_rowwise_into(q, s, w, w_s, bias, out, int(epilogue))
    else:
      q, s = activation_workspace(M, K, x2.device)
      linear_w8a8_into(x2, w, w_s, bias, out, q, s, int(scale_mode), int(epilogue))
  return out.view(*x.shape[:-1], N)


@torch.library.impl("cdit::linear_w8a8_cat2", "CUDA")
def _linear_w8a8_cat2(x1, x2, weight, weight_scale, bias, scale_mode=0, epilogue=0):
  """cdit::linear_w8a8 (per-token scales) on torch.cat([x1, x2], dim=-1) without that tensor:
  the two sources are quantized as one row (cdit_fp8_quant_rowwise_cat2). FLUX single blocks
  feed proj_out this way (reference dataflow
  src/cache_dit/caching/patch_functors/functor_flux.py:68-80). Bit-identical to the op on the
  concatenation; sources the kernel does not take are concatenated."""
  name = "cdit::linear_w8a8_cat2"
  if x1.dtype != torch.bfloat16 or x2.dtype != torch.bfloat16:
    raise ValueError(f"{name}: x1 and x2 must be bfloat16, got {x1.dtype} and {x2.dtype}")
  if x1.shape[:-1] != x2.shape[:-1]:
    raise ValueError(f"{name}: leading shapes differ: {tuple(x1.shape)} and {tuple(x2.shape)}")
  N, K = weight.shape
  if x1.shape[-1] + x2.shape[-1] != K:
    raise ValueError(f"{name}: shape mismatch [{x1.shape[-1]} | {x2.shape[-1]}] x weight "
                     f"{tuple(weight.shape)}")
  a, b = _as_rows(x1), _as_rows(x2)
  if not cat2_quant_ok(a, b) or a.shape[0] <= 16 or scale_mode not in (0, 1):
    return torch.ops.cdit.linear_w8a8(torch.cat([x1, x2], dim=-1), weight, weight_scale, bias,
                                      scale_mode, epilogue, GRANULARITY_PER_ROW, False)
  if weight.dtype != FP8 or weight_scale.numel() != N or weight_scale.dtype != torch.float32:
    raise ValueError(f"{name}: weight must be float8_e4m3fn [N,K] with {N} float32 scales")
  if bias is not None and (bias.numel() != N or bias.dtype != torch.bfloat16):
    raise ValueError(f"{name}: bias must hold {N} bfloat16 values")
  w = weight if weight.stride(-1) == 1 else weight.contiguous()
  w_s = weight_scale if weight_scale.is_contiguous() else weight_scale.contiguous()
  if bias is not None and not bias.is_contiguous():
    bias = bias.contiguous()
  M = a.shape[0]
  out = torch.empty((M, N), dtype=torch.bfloat16, device=x1.device)
  q, s = activation_workspace(M, K, a.device)
  quant_rowwise_cat2_into(a, b, q, s, int(scale_mode))
  gemm_rowwise_into(q, s, w, w_s, bias, out, int(epilogue))
  return out.view(*x1.shape[:-1], N)


@torch.library.register_fake("cdit::linear_w8a8_cat2")
def _fake_linear_w8a8_cat2(x1, x2, weight, weight_scale, bias, scale_mode=0, epilogue=0):
  return x1.new_empty((*x1.shape[:-1], weight.shape[0]), dtype=torch.bfloat16)


def _batch_check(name, xs, weights, weight_scales, biases, members_per_act, epilogues):
  n = len(weights)
  if (len(xs) != len(members_per_act) or sum(members_per_act) != n or len(weight_scales) != n
      or len(biases) != n or len(epilogues) != n or not 1 <= len(xs) <= _native.MAX_ACTS
      or n > _native.MAX_GROUP or any(c < 1 for c in members_per_act)):
    raise ValueError(f"{name}: 1 to {_native.MAX_ACTS} activations with 1 to {_native.MAX_GROUP} "
                     "members in all, listed activation by activation")
  K = xs[0].shape[-1]
  for x in xs:
    if x.dtype != torch.bfloat16 or x.shape[-1] != K:
      raise ValueError(f"{name}: activations must be bfloat16 [..., {K}]")
  for w, s, b in zip(weights, weight_scales, biases):
    if w.dtype != FP8 or w.dim() != 2 or w.shape[1] != K or w.stride(-1) != 1:
      raise ValueError(f"{name}: weights must be float8_e4m3fn [N, {K}] rows")
    if s.numel() != w.shape[0] or s.dtype != torch.float32 or not s.is_contiguous():
      raise ValueError(f"{name}: weight_scales must hold N contiguous float32 values")
    if b is not None and (b.numel() != w.shape[0] or b.dtype != torch.bfloat16 or not b.is_contiguous()):
      raise ValueError(f"{name}: biases must hold N contiguous bfloat16 values")


def _batch_outputs(xs, weights, members_per_act):
  rows, outs, shaped, p = [], [], [], 0
  for x, c in zip(xs, members_per_act):
    x2 = _as_rows(x)
    rows.append(x2)
    mine = [torch.empty((x2.shape[0], w.shape[0]), dtype=torch.bfloat16, device=x.device)
            for w in weights[p:p + c]]
    outs.append(mine)
    shaped += [o.view(*x.shape[:-1], o.shape[1]) for o in mine]
    p += c
  return rows, outs, shaped


@torch.library.impl("cdit::linear_w8a8_batch", "CUDA")
def _linear_w8a8_batch(xs, weights, weight_scales, biases, members_per_act, epilogues, scale_mode=0):
  """The float8_per_row Linears of one stage on up to four activations as one quantizer
  launch and one GEMM launch (cdit_fp8_quant_rowwise_batched + cdit_fp8_gemm_rowwise_batched)
  behind a single traceable op: xs[s] bf16 [..., K]; the members of activation s are the
  next members_per_act[s] entries of weights (e4m3 [N_p, K]), weight_scales, biases and
  epilogues. Returns one bf16 [..., N_p] per member, bit-identical to cdit::linear_w8a8 per
  member."""
  _batch_check("cdit::linear_w8a8_batch", xs, weights, weight_scales, biases, members_per_act,
               epilogues)
  rows, outs, shaped = _batch_outputs(xs, weights, members_per_act)
  live = [i for i, r in enumerate(rows) if r.shape[0] > 0]
  if not live:
    return shaped
  items = []
  for i in live:
    r = rows[i]
    items.append((r, torch.empty(r.shape, dtype=FP8, device=r.device),
                  torch.empty((r.shape[0], ), dtype=torch.float32, device=r.device)))
  if len(items) > 1:
    quant_rowwise_batched_into(items, int(scale_mode))
  else:
    quant_rowwise_into(items[0][0], items[0][1], items[0][2], int(scale_mode), gemm_follows=True)
  starts = [sum(members_per_act[:i]) for i in range(len(xs))]
  acts = []
  for (r, q, sc), i in zip(items, live):
    a, b = starts[i], starts[i] + members_per_act[i]
    acts.append((q, sc, list(weights[a:b]), list(weight_scales[a:b]), list(biases[a:b]), outs[i],
                 [int(e) for e in epilogues[a:b]]))
  if len(acts) == 1 and len(acts[0][2]) == 1:
    q, sc, w, ws, b, o, e = acts[0]
    gemm_rowwise_into(q, sc, w[0], ws[0], b[0], o[0], e[0])
  else:
    gemm_rowwise_batched_into(acts)
  return shaped


@torch.library.impl("cdit::w8a16_batch", "CUDA")
def _w8a16_batch(xs, weights, weight_scales, biases, members_per_act, epilogues):
  """The float8_weight_only counterpart of cdit::linear_w8a8_batch (cdit_w8a16_gemm_batched)."""
  _batch_check("cdit::w8a16_batch", xs, weights, weight_scales, biases, members_per_act, epilogues)
  rows, outs, shaped = _batch_outputs(xs, weights, members_per_act)
  starts = [sum(members_per_act[:i]) for i in range(len(xs))]
  acts = []
  for i, r in enumerate(rows):
    if r.shape[0] == 0:
      continue
    a, b = starts[i], starts[i] + members_per_act[i]
    acts.append((r, list(weights[a:b]), list(weight_scales[a:b]), list(biases[a:b]), outs[i],
                 [int(e) for e in epilogues[a:b]]))
  if acts:
    w8a16_batched_into(acts)
  return shaped


def _fake_batch(xs, weights, members_per_act):
  out, p = [], 0
  for x, c in zip(xs, members_per_act):
    out += [x.new_empty((*x.shape[:-1], w.shape[0]), dtype=torch.bfloat16) for w in weights[p:p + c]]
    p += c
  return out


@torch.library.register_fake("cdit::linear_w8a8_batch")
def _fake_linear_w8a8_batch(xs, weights, weight_scales, biases, members_per_act, epilogues,
                            scale_mode=0):
  return _fake_batch(xs, weights, members_per_act)


@torch.library.register_fake("cdit::w8a16_batch")
def _fake_w8a16_batch(xs, weights, weight_scales, biases, members_per_act, epilogues):
  return _fake_batch(xs, weights, members_per_act)


@torch.library.register_fake("cdit::linear_w8a8")
def _fake_linear_w8a8(x, weight, weight_scale, bias, scale_mode=0, epilogue=0, granularity=0,
                      share_input_quant=False):
  return x.new_empty((*x.shape[:-1], weight.shape[0]), dtype=torch.bfloat16)


@torch.library.impl("cdit::w8a16_mm", "CUDA")
def _w8a16_mm(x, b_data, b_scale, bias, out_dtype_id, epilogue=0):
  name = "cdit::w8a16_mm"
  out_dtype = decode_output_dtype(out_dtype_id)
  if out_dtype != torch.bfloat16 or x.dtype != torch.bfloat16:
    raise ValueError(f"{name}: only bfloat16 activations and output are built, got {x.dtype} -> "
                     f"{out_dtype}")
  if b_data.dtype != FP8:
    raise ValueError(f"{name}: b_data must be float8_e4m3fn, got {b_data.dtype}")
  w = _weight_rows(b_data, name)
  x2 = _as_rows(x)
  M, K = x2.shape
  N = w.shape[0]
  if w.shape[1] != K:
    raise ValueError(f"{name}: shape mismatch x {tuple(x.shape)} x b {tuple(b_data.shape)}")
  if b_scale.numel() != N:
    raise ValueError(f"{name}: b_scale must have {N} elements")
  b_s = b_scale.reshape(-1).to(torch.float32).contiguous()
  if bias is not None:
    bias = bias.reshape(-1).to(torch.bfloat16).contiguous()
  out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
  w8a16_into(x2, w, b_s, bias, out, int(epilogue))
  return out.reshape(*x.shape[:-1], N)


@torch.library.register_fake("cdit::w8a16_mm")
def _fake_w8a16_mm(x, b_data, b_scale, bias, out_dtype_id, epilogue=0):
  return x.new_empty((*x.shape[:-1], b_data.shape[-1]), dtype=decode_output_dtype(out_dtype_id))


# --------------------------------------------------------------------------- python-level API


def fp8_tensorwise_quant(x: torch.Tensor,
                         scale_mode: str = "bf16div") -> Tuple[torch.Tensor, torch.Tensor]:
  """Per-tensor dynamic e4m3 quantization of a bf16 tensor -> (codes, scale[M,1]
  with every entry equal to the tensor's scale)."""
  _require_cuda("fp8_tensorwise_quant", x)
  if x.dtype != torch.bfloat16:
    raise ValueError(f"fp8_tensorwise_quant: x must be bfloat16, got {x.dtype}")
  x2 = x.reshape(-1, x.shape[-1])
  if x2.stride(-1) != 1:
    x2 = x2.contiguous()
  M, K = x2.shape
  q = torch.empty((M, K), dtype=FP8, device=x.device)
  s = torch.empty((M,), dtype=torch.float32, device=x.device)
  ws = torch.empty((1,), dtype=torch.int32, device=x.device)
  if M > 0:
    quant_tensorwise_into(x2, q, s, ws, _native.SCALE_MODE_IDS[scale_mode])
  return q.view(x.shape), s.view(*x.shape[:-1], 1)


def fp8_rowwise_quant(x: torch.Tensor,
                      scale_mode: str = "bf16div") -> Tuple[torch.Tensor, torch.Tensor]:
  """Per-row dynamic e4m3 quantization of a bf16 tensor -> (codes, scale[...,1])."""
  _require_cuda("fp8_rowwise_quant", x)
  return torch.ops.cdit.fp8_rowwise_quant(x, _native.SCALE_MODE_IDS[scale_mode])


def float8_inference_scaled_mm(
    a_data: torch.Tensor,
    a_scale: torch.Tensor,
    b_data: torch.Tensor,
    b_scale: torch.Tensor,
    output_dtype: torch.dtype,
    output_scale: Optional[torch.Tensor] = None,
    bias: Optional[torch.Tensor] = None,
    use_fast_accum: bool = False,
    epilogue: int = 0,
) -> torch.Tensor:
  """Same signature as the reference's `_opaque_addmm_float8_unwrapped_inference`
  (src/cache_dit/quantization/torchao/_scaled_mm.py:140-162), incl. its refusal of
  `output_scale`."""
  if output_scale is not None:
    raise NotImplementedError("float8 scaled_mm wrapper does not support scale_result yet.")
  _require_cuda("float8_inference_scaled_mm", a_data, b_data)
  return torch.ops.cdit.float8_inference_scaled_mm(a_data, a_scale, b_data, b_scale, bias,
                                                   encode_output_dtype(output_dtype),
                                                   use_fast_accum, epilogue)


def w8a16_mm(x: torch.Tensor,
             b_data: torch.Tensor,
             b_scale: torch.Tensor,
             bias: Optional[torch.Tensor] = None,
             output_dtype: torch.dtype = torch.bfloat16,
             epilogue: int = 0) -> torch.Tensor:
  _require_cuda("w8a16_mm", x, b_data)
  return torch.ops.cdit.w8a16_mm(x, b_data, b_scale, bias, encode_output_dtype(output_dtype),
                                 epilogue)
