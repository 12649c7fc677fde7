#!/usr/bin/env python3
"""Benchmark of the FP8 quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the hot path over one batch: every quantized nn.Linear
of one denoising step of the FLUX.1-dev-shaped MMDiT (benchmark config 2: 19
double-stream + 38 single-stream blocks, 4096 image + 512 text tokens, hidden
3072, MLP 12288 with GELU-tanh) run back to back at its real shape with its own
weights -- per Linear: per-token e4m3 activation quantization, FP8 GEMM, fused
scale/bias/(GELU) epilogue, bf16 out. 494 Linears, 5.95e13 FLOP. Inputs are
synthetic (~N(0,1) bf16 activations, random e4m3 weights) and resident in HBM
before the timed region.

Prints ONE JSON line. `value` is the whole-step linear throughput in TFLOP/s
(sum of 2MKN / step time). Beside it: the headline-shape kernel figures
(`linear_headline`: GEMM and quantizer at M=4608 K=3072 N=12288), `roofline`
for the dominant kernel (the FP8 GEMM, timed with HIP events on the launch
stream), the full synthetic-transformer forward (`dit_step_ms`, attention and
glue included) and `cpu_baseline`: the CPU restatement of the reference path
(PyTorch CPU ops) timed on this box's host cores on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

FP8_PEAK_TFLOPS = 5000.0  # MI355X dense FP8 MFMA
BF16_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBPS = 8000.0
HEADLINE = (4608, 3072, 12288)  # M, K, N


def flux_step_linears():
  """(name, M, K, N, gelu, count) of every quantized Linear of one FLUX-shaped
  step; layer names as in diffusers' FluxTransformer2DModel."""
  img, txt, both, d, mlp = 4096, 512, 4608, 3072, 12288
  double = [
      ("attn.to_q", img, d, d, False), ("attn.to_k", img, d, d, False),
      ("attn.to_v", img, d, d, False), ("attn.to_out.0", img, d, d, False),
      ("ff.net.0.proj", img, d, mlp, True), ("ff.net.2", img, mlp, d, False),
      ("norm1.linear", 1, d, 6 * d, False),
      ("attn.add_q_proj", txt, d, d, False), ("attn.add_k_proj", txt, d, d, False),
      ("attn.add_v_proj", txt, d, d, False), ("attn.to_add_out", txt, d, d, False),
      ("ff_context.net.0.proj", txt, d, mlp, True), ("ff_context.net.2", txt, mlp, d, False),
      ("norm1_context.linear", 1, d, 6 * d, False),
  ]
  single = [
      ("norm.linear", 1, d, 3 * d, False), ("proj_mlp", both, d, mlp, True),
      ("attn.to_q", both, d, d, False), ("attn.to_k", both, d, d, False),
      ("attn.to_v", both, d, d, False), ("proj_out", both, d + mlp, d, False),
  ]
  out = []
  for i in range(19):
    out += [(f"transformer_blocks.{i}.{n}", M, K, N, g) for n, M, K, N, g in double]
  for i in range(38):
    out += [(f"single_transformer_blocks.{i}.{n}", M, K, N, g) for n, M, K, N, g in single]
  return out


def qwen_step_linears():
  """The 720 quantized Linears of one Qwen-Image-shaped step (benchmark config 4: 60
  blocks, 83 x 83 = 6889 image + 256 text tokens, hidden 3072, MLP 12288); layer names as
  in diffusers' QwenImageTransformer2DModel. `img_mod.1` / `txt_mod.1` stay bf16 (the
  default exclude pattern "mod")."""
  img, txt, d, mlp = 6889, 256, 3072, 12288
  block = [
      ("attn.to_q", img, d, d, False), ("attn.to_k", img, d, d, False),
      ("attn.to_v", img, d, d, False), ("attn.to_out.0", img, d, d, False),
      ("img_mlp.net.0.proj", img, d, mlp, True), ("img_mlp.net.2", img, mlp, d, False),
      ("attn.add_q_proj", txt, d, d, False), ("attn.add_k_proj", txt, d, d, False),
      ("attn.add_v_proj", txt, d, d, False), ("attn.to_add_out", txt, d, d, False),
      ("txt_mlp.net.0.proj", txt, d, mlp, True), ("txt_mlp.net.2", txt, mlp, d, False),
  ]
  return [(f"transformer_blocks.{i}.{n}", M, K, N, g) for i in range(60) for n, M, K, N, g in block]


def wan_step_linears():
  """The 400 quantized Linears of one Wan2.1-14B-shaped step (benchmark config 5: 40
  layers, 21 x 30 x 52 = 32760 video tokens, 512 text tokens, hidden 5120, FFN 13824);
  layer names as in diffusers' WanTransformer3DModel."""
  vid, txt, d, ffn = 32760, 512, 5120, 13824
  block = [
      ("attn1.to_q", vid, d, d, False), ("attn1.to_k", vid, d, d, False),
      ("attn1.to_v", vid, d, d, False), ("attn1.to_out.0", vid, d, d, False),
      ("attn2.to_q", vid, d, d, False), ("attn2.to_k", txt, d, d, False),
      ("attn2.to_v", txt, d, d, False), ("attn2.to_out.0", vid, d, d, False),
      ("ffn.net.0.proj", vid, d, ffn, True), ("ffn.net.2", vid, ffn, d, False),
  ]
  return [(f"blocks.{i}.{n}", M, K, N, g) for i in range(40) for n, M, K, N, g in block]


def _rand_fp8(shape, gen, device):
  import torch
  # random e4m3 codes with |value| <= 1.75 (exponent field <= 7): no NaN codes
  bits = torch.randint(0, 256, shape, dtype=torch.uint8, device=device, generator=gen)
  return (bits & 0xBF).view(torch.float8_e4m3fn)


class HotPath:
  """All quantized Linears of one step, each with its own weight."""

  def __init__(self, device, linears=None, mode="w8a8"):
    import torch
    from cache_dit_amd import _native
    self.torch = torch
    self.native = _native
    self.mode = mode
    self.linears = flux_step_linears() if linears is None else linears
    g = torch.Generator(device=device).manual_seed(0)
    self.layers = []
    self.flop = 0
    max_mk, max_mn = {}, 0
    for name, M, K, N, gelu in self.linears:
      w = _rand_fp8((N, K), g, device)
      ws = torch.rand(N, device=device, generator=g) * 1e-3 + 1e-4
      b = (torch.randn(N, device=device, generator=g) * 0.01).to(torch.bfloat16)
      self.layers.append((M, K, N, w, ws, b, 1 if gelu else 0))
      self.flop += 2 * M * K * N
      max_mk[(M, K)] = None
      max_mn = max(max_mn, M * N)
    # activations: one bf16 input per distinct (M, K); scratch for codes/scales/output
    self.x = {mk: torch.randn(mk, device=device, generator=g).to(torch.bfloat16) for mk in max_mk}
    self.q = {mk: torch.empty(mk, dtype=torch.float8_e4m3fn, device=device) for mk in max_mk}
    self.s = {mk: torch.empty(mk[0], dtype=torch.float32, device=device) for mk in max_mk}
    self.out = torch.empty(max_mn, dtype=torch.bfloat16, device=device)
    # a run of siblings writes its outputs side by side
    run_mn = max(sum(self.layers[i][0] * self.layers[i][2] for run in stage for i in run)
                 for stage in self.stages())
    self.out2 = torch.empty(run_mn, dtype=torch.bfloat16, device=device)

  def step(self):
    """One pass: for every Linear the same library call its module forward makes
    (quantizer + GEMM enqueued by cdit_fp8_linear_w8a8)."""
    from cache_dit_amd import ops
    if self.mode == "w8a16":  # weight-only: bf16 activations straight into the GEMM
      for M, K, N, w, ws, b, epi in self.layers:
        ops.w8a16_into(self.x[(M, K)], w, ws, b, self.out[:M * N].view(M, N), epi)
      return
    for M, K, N, w, ws, b, epi in self.layers:
      out = self.out[:M * N].view(M, N)
      ops.linear_w8a8_into(self.x[(M, K)], w, ws, b, out, self.q[(M, K)], self.s[(M, K)], 0, epi)

  def sibling_runs(self):
    """The Linears as runs of siblings: consecutive Linears that read the same activation in
    the model (q/k/v of a stream; proj_mlp + q/k/v in FLUX single blocks; Wan's cross
    attention k/v), each run a list of indices into self.layers."""
    runs = []
    for i, (name, *_) in enumerate(self.linears):
      leaf = name.split(".", 2)[2]
      same_input = leaf in ("attn.to_k", "attn.to_v", "attn.add_k_proj", "attn.add_v_proj",
                            "attn1.to_k", "attn1.to_v", "attn2.to_v") or (
                                name.startswith("single") and leaf == "attn.to_q")  # after proj_mlp
      if same_input and runs:
        runs[-1].append(i)
      else:
        runs.append([i])
    return runs

  def stages(self):
    """The sibling runs arranged in stages: runs of one stage are independent of each other
    in the model (image-stream and text-stream Linears of a double-stream block at the same
    point of the block; Wan's cross-attention query next to its key / value) and share K, so
    that a block forward written against linear_batch launches each stage as one GEMM."""
    partner = {"attn.add_q_proj": "attn.to_q", "attn.to_add_out": "attn.to_out.0",
               "ff_context.net.0.proj": "ff.net.0.proj", "ff_context.net.2": "ff.net.2",
               "txt_mlp.net.0.proj": "img_mlp.net.0.proj", "txt_mlp.net.2": "img_mlp.net.2",
               "attn2.to_k": "attn2.to_q"}
    stages, at = [], {}
    for run in self.sibling_runs():
      name = self.linears[run[0]][0]
      block, leaf = name.rsplit(".", name.count(".") - 1)[0], name.split(".", 2)[2]
      M, K = self.layers[run[0]][:2]
      want = partner.get(leaf)
      if want is not None and (block, want) in at and M > 16:
        stages[at[(block, want)]].append(run)
        continue
      if M > 16 and not name.startswith("single"):
        at[(block, leaf)] = len(stages)
      stages.append([run])
    return stages

  def step_batched(self):
    """The pass as block forwards written against linear_batch run it: ONE quantizer launch
    (cdit_fp8_quant_rowwise_batched) and ONE GEMM launch (cdit_fp8_gemm_rowwise_batched) per
    stage. Outputs are bit-identical to step()."""
    from cache_dit_amd import ops
    for stage in self.stages():
      if self.mode == "w8a16":  # weight-only: no quantizer, one GEMM launch per stage
        acts, at = [], 0
        for run in stage:
          M, K = self.layers[run[0]][:2]
          members = [self.layers[i] for i in run]
          outs = []
          for _, _, N, *_ in members:
            outs.append(self.out2[at:at + M * N].view(M, N))
            at += M * N
          acts.append((self.x[(M, K)], [m[3] for m in members], [m[4] for m in members],
                       [m[5] for m in members], outs, [m[6] for m in members]))
        ops.w8a16_batched_into(acts)
        continue
      if len(stage) == 1 and len(stage[0]) == 1:
        M, K, N, w, ws, b, epi = self.layers[stage[0][0]]
        ops.linear_w8a8_into(self.x[(M, K)], w, ws, b, self.out[:M * N].view(M, N), self.q[(M, K)],
                             self.s[(M, K)], 0, epi)
        continue
      acts, at = [], 0
      inputs = [self.layers[run[0]][:2] for run in stage]
      if len(inputs) > 1:  # one quantizer launch for the activations of the stage
        ops.quant_rowwise_batched_into([(self.x[mk], self.q[mk], self.s[mk]) for mk in inputs], 0)
      else:
        ops.quant_rowwise_into(self.x[inputs[0]], self.q[inputs[0]], self.s[inputs[0]], 0, gemm_follows=True)
      for run in stage:
        M, K = self.layers[run[0]][:2]
        members = [self.layers[i] for i in run]
        outs = []
        for _, _, N, *_ in members:
          outs.append(self.out2[at:at + M * N].view(M, N))
          at += M * N
        acts.append((self.q[(M, K)], self.s[(M, K)], [m[3] for m in members], [m[4] for m in members],
                     [m[5] for m in members], outs, [m[6] for m in members]))
      ops.gemm_rowwise_batched_into(acts)

  def step_shared_quant(self):
    """The same pass with one quantizer launch per distinct input: q/k/v (and
    proj_mlp in single blocks) read one activation, as share_activation_quant_
    arranges in a real model. Outputs are bit-identical to step()."""
    from cache_dit_amd import ops
    for run in self.sibling_runs():
      M, K = self.layers[run[0]][:2]
      ops.quant_rowwise_into(self.x[(M, K)], self.q[(M, K)], self.s[(M, K)], 0, gemm_follows=True)
      for i in run:
        _, _, N, w, ws, b, epi = self.layers[i]
        ops.gemm_rowwise_into(self.q[(M, K)], self.s[(M, K)], w, ws, b, self.out[:M * N].view(M, N), epi)

  def step_grouped(self):
    """The pass as a model runs it with group_sibling_linears_: every run of siblings is one
    quantizer launch and ONE grouped GEMM launch (cdit_fp8_gemm_rowwise_grouped); a Linear
    without siblings is the fused quantizer + GEMM call of step(). Outputs are bit-identical
    to step(); siblings write to disjoint parts of the output scratch."""
    from cache_dit_amd import ops
    for run in self.sibling_runs():
      M, K = self.layers[run[0]][:2]
      if len(run) == 1:
        _, _, N, w, ws, b, epi = self.layers[run[0]]
        ops.linear_w8a8_into(self.x[(M, K)], w, ws, b, self.out[:M * N].view(M, N), self.q[(M, K)],
                             self.s[(M, K)], 0, epi)
        continue
      ops.quant_rowwise_into(self.x[(M, K)], self.q[(M, K)], self.s[(M, K)], 0, gemm_follows=True)
      members = [self.layers[i] for i in run]
      outs, at = [], 0
      for _, _, N, *_ in members:
        outs.append(self.out2[at:at + M * N].view(M, N))
        at += M * N
      ops.gemm_rowwise_grouped_into(self.q[(M, K)], self.s[(M, K)], [m[3] for m in members],
                                    [m[4] for m in members], [m[5] for m in members], outs,
                                    [m[6] for m in members])


def step_leg(device, linears, mode, steps, warmup):
  """A step of another benchmark configuration (every quantized Linear of the model at
  its real shape with its own weights; stages batched as in the headline step),
  captured into a hipGraph and replayed like the headline step. Returns ms per step,
  TFLOP/s and the Linear count."""
  import torch
  hot = HotPath(device, linears, mode)

  def replay_ms(step):
    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
      step()
    for _ in range(warmup):
      graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
      graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3

  ms = replay_ms(hot.step_batched)
  res = {"ms_per_step": ms, "tflops": hot.flop / ms / 1e9, "linears": len(hot.layers),
         "linear_flop_per_step": hot.flop}
  if mode == "w8a16":  # every Linear on its own, beside the batched stages
    res["ungrouped_ms_per_step"] = replay_ms(hot.step)
  del hot
  torch.cuda.empty_cache()
  return res


def pmc_sequence(device):
  """Launch sequence for counter collection: run under `rocprofv3 --pmc FETCH_SIZE`, then
  under `--pmc WRITE_SIZE`, each in a run of its own. Four times over, each kernel behind a
  512 MiB fill (to push earlier data out of the caches): a plain device copy of the bf16
  activation (known size: the scale of the counters), the quantizer on that activation, the
  FP8 GEMM on the codes, the fused LayerNorm + modulate + quantizer, the weight-only GEMM
  and the grouped GEMM of a FLUX single block; all at the headline shape."""
  import torch
  from cache_dit_amd import ops
  M, K, N = HEADLINE
  g = torch.Generator(device=device).manual_seed(0)
  x = [torch.randn(M, K, device=device, generator=g).to(torch.bfloat16) for _ in range(4)]
  q = [torch.empty(M, K, dtype=torch.float8_e4m3fn, device=device) for _ in range(4)]
  s = torch.empty(M, dtype=torch.float32, device=device)
  w = [_rand_fp8((N, K), g, device) for _ in range(4)]
  ws = torch.rand(N, device=device, generator=g) * 1e-3
  b = torch.randn(N, device=device, generator=g).to(torch.bfloat16)
  out = torch.empty(M, N, dtype=torch.bfloat16, device=device)
  y = torch.empty(M, K, dtype=torch.bfloat16, device=device)
  flush = torch.empty(1 << 29, dtype=torch.uint8, device=device)
  # further kernels of the path, for their own counter summaries: the fused LayerNorm +
  # modulate + quantizer, the weight-only GEMM, and the grouped GEMM of a FLUX single block
  # (proj_mlp + q/k/v on one activation: 12288 + 3 x 3072 columns on 256 x 256 tiles)
  from cache_dit_amd import _native
  L, stream = _native.load(), torch.cuda.current_stream().cuda_stream
  shift = torch.randn(K, device=device, generator=g).to(torch.bfloat16)
  scale_mod = (torch.randn(K, device=device, generator=g) * 0.3).to(torch.bfloat16)
  sib_n = (N, K, K, K)
  sib_w = [_rand_fp8((n, K), g, device) for n in sib_n]
  sib_s = [torch.rand(n, device=device, generator=g) * 1e-3 for n in sib_n]
  sib_b = [torch.randn(n, device=device, generator=g).to(torch.bfloat16) for n in sib_n]
  sib_out = [torch.empty(M, n, dtype=torch.bfloat16, device=device) for n in sib_n]
  for i in range(4):
    flush.zero_()
    y.copy_(x[i])  # plain copy: reads 2MK, writes 2MK bytes
    flush.zero_()
    ops.quant_rowwise_into(x[i], q[i], s, 0)
    flush.zero_()
    ops.gemm_rowwise_into(q[i], s, w[i], ws, b, out, 0)
    flush.zero_()
    _native.check(L.cdit_fp8_ln_modulate_quant(x[i].data_ptr(), M, K, K, shift.data_ptr(),
                                               scale_mod.data_ptr(), K, M, 1e-6, None, K,
                                               q[i].data_ptr(), K, s.data_ptr(), 0, stream))
    flush.zero_()
    ops.w8a16_into(x[i], w[i], ws, b, out, 0)
    flush.zero_()
    ops.quant_rowwise_into(x[i], q[i], s, 0)
    ops.gemm_rowwise_grouped_into(q[i], s, sib_w, sib_s, sib_b, sib_out, [1, 0, 0, 0])
  torch.cuda.synchronize()


def measured_traffic(kernel_key):
  """HBM-side bytes per launch of a headline kernel from the committed counter summary
  (profiles/traffic.json): FETCH_SIZE and WRITE_SIZE in KiB per dispatch, each scaled by
  the factor that makes the same counter read the known size for a plain copy. None when
  the file or the entry is missing."""
  try:
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
      t = json.load(f)
    k, c, known = t[kernel_key], t["copy"], float(t["copy_known_kib"])
    return (k["fetch_kib"] * known / c["fetch_kib"] + k["write_kib"] * known / c["write_kib"]) * 1024.0
  except (OSError, KeyError, ValueError, ZeroDivisionError):
    return None


class _BoardPower:
  """Samples the board power the amdgpu driver reports for the GPU (hwmon power1_input or
  power1_average, microwatts; a reading the driver smooths over a few hundred ms) from a thread
  while a leg runs. `cap_w` is the power limit the driver enforces (power1_cap). Best effort:
  without the files every figure is None."""

  def __init__(self, device_index=0, period=0.02):
    import glob
    self.period, self.samples, self._stop, self._thread = period, [], False, None
    self.path = self.cap_w = None
    cards = sorted(glob.glob("/sys/class/drm/card[0-9]*/device/hwmon/hwmon*"))
    cards = [c for c in cards if any(os.path.exists(os.path.join(c, f)) for f in ("power1_input", "power1_average"))]
    if len(cards) > 1:  # several GPUs visible: the one whose PCI address is the torch device's
      try:
        import torch
        pr = torch.cuda.get_device_properties(device_index)
        addr = f"{pr.pci_domain_id:04x}:{pr.pci_bus_id:02x}:{pr.pci_device_id:02x}.0"
        cards = [c for c in cards if addr in os.path.realpath(c)] or cards[:0]
      except Exception:
        cards = cards[:0]
    if cards:
      for f in ("power1_input", "power1_average"):
        if os.path.exists(os.path.join(cards[0], f)):
          self.path = os.path.join(cards[0], f)
          break
      try:
        with open(os.path.join(cards[0], "power1_cap")) as fh:
          self.cap_w = int(fh.read()) / 1e6
      except (OSError, ValueError):
        pass

  def _run(self):
    while not self._stop:
      try:
        with open(self.path) as fh:
          self.samples.append((time.perf_counter(), int(fh.read()) / 1e6))
      except (OSError, ValueError):
        pass
      time.sleep(self.period)

  def __enter__(self):
    if self.path:
      import threading
      self._thread = threading.Thread(target=self._run, daemon=True)
      self._thread.start()
    return self

  def __exit__(self, *exc):
    self._stop = True
    if self._thread:
      self._thread.join()

  def settled_w(self, since=None):
    """Mean of the last quarter of the samples taken (after `since`): the smoothed reading
    needs about half a second of steady load to arrive."""
    w = [v for t, v in self.samples if since is None or t >= since]
    if not w:
      return None
    tail = w[-max(1, len(w) // 4):]
    return sum(tail) / len(tail)


def _time_events(fn, iters, warmup):
  """Average duration in ms of fn() over `iters` calls, HIP events on the current
  stream (the stream the kernels are launched on)."""
  import torch
  for _ in range(warmup):
    fn()
  torch.cuda.synchronize()
  e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  e0.record()
  for _ in range(iters):
    fn()
  e1.record()
  torch.cuda.synchronize()
  return e0.elapsed_time(e1) / iters


def headline_kernels(device):
  """GEMM and quantizer alone at the headline shape, rotating over enough distinct
  buffers that the 256 MiB last-level cache cannot serve repeats."""
  import torch
  from cache_dit_amd import ops
  M, K, N = HEADLINE
  g = torch.Generator(device=device).manual_seed(1)
  nbuf = 8
  xs = [torch.randn(M, K, device=device, generator=g).to(torch.bfloat16) for _ in range(nbuf)]
  qs = [torch.empty(M, K, dtype=torch.float8_e4m3fn, device=device) for _ in range(nbuf)]
  ss = [torch.empty(M, dtype=torch.float32, device=device) for _ in range(nbuf)]
  ws = [_rand_fp8((N, K), g, device) for _ in range(nbuf)]
  wsc = torch.rand(N, device=device, generator=g) * 1e-3 + 1e-4
  b = (torch.randn(N, device=device, generator=g) * 0.01).to(torch.bfloat16)
  outs = [torch.empty(M, N, dtype=torch.bfloat16, device=device) for _ in range(2)]
  for i in range(nbuf):
    ops.quant_rowwise_into(xs[i], qs[i], ss[i], 0)
  it = {"i": 0}

  def gemm():  # scales + bias epilogue: what quantize() installs by default
    i = it["i"] = (it["i"] + 1) % nbuf
    ops.gemm_rowwise_into(qs[i], ss[i], ws[i], wsc, b, outs[i & 1], 0)

  def gemm_gelu():  # with the optional GELU-tanh folded in (fuse_gelu_tanh_)
    i = it["i"] = (it["i"] + 1) % nbuf
    ops.gemm_rowwise_into(qs[i], ss[i], ws[i], wsc, b, outs[i & 1], 1)

  def quant():
    i = it["i"] = (it["i"] + 1) % nbuf
    ops.quant_rowwise_into(xs[i], qs[i], ss[i], 0)

  # Bring the clocks to their steady state first: under the power limit the shader clock
  # of this part keeps rising over the first second or two of a run of GEMMs (10 % between
  # the first hundred launches and the settled value). Blocks of 100 launches until two
  # consecutive blocks agree within 0.5 %, for at least 1.5 and at most 4 seconds.
  # The quantizer is timed twice, as the median of five blocks of 100 launches each: before
  # the GEMM legs (cooler part, higher clocks) and after them (the state it runs in inside a
  # step). Both are reported; roofline_quant quotes the later one.
  def quant_median_ms():
    blocks = sorted(_time_events(quant, 100, 20 if k == 0 else 0) for k in range(5))
    return blocks[2], blocks[0], blocks[-1]

  quant_before = quant_median_ms()
  power = _BoardPower(torch.device(device).index or 0)
  idle_w = None
  if power.path:
    time.sleep(0.3)
    try:
      with open(power.path) as fh:
        idle_w = int(fh.read()) / 1e6  # (between legs: not a cold idle)
    except (OSError, ValueError):
      pass
  with power:
    t_start, prev = time.perf_counter(), _time_events(gemm, 100, 100)
    while time.perf_counter() - t_start < 4.0:
      cur = _time_events(gemm, 100, 0)
      settled = abs(cur - prev) <= 0.005 * prev
      prev = cur
      if settled and time.perf_counter() - t_start > 1.5:
        break
    gemm_ms = _time_events(gemm, 100, 10)
    gemm_w = power.settled_w()
    gemm_max_w = max((v for _, v in power.samples), default=None)
    gemm_gelu_ms = _time_events(gemm_gelu, 100, 10)
  quant_after = quant_median_ms()
  quant_ms = quant_after[0]
  res = {
      "shape": {"M": M, "K": K, "N": N},
      "gemm_ms": gemm_ms,
      "gemm_tflops": 2.0 * M * K * N / gemm_ms / 1e9,
      "gemm_gelu_ms": gemm_gelu_ms,
      "gemm_gelu_tflops": 2.0 * M * K * N / gemm_gelu_ms / 1e9,
      "quant_ms": quant_ms,
      "quant_gbps": (3.0 * M * K + 4.0 * M) / quant_ms / 1e6,
      # median, fastest and slowest of five blocks of 100 back-to-back launches (ms)
      "quant_ms_before_gemm_legs": list(quant_before),
      "quant_ms_after_gemm_legs": list(quant_after),
      # board power as the amdgpu driver reports it (hwmon), sampled every 20 ms while the
      # GEMM legs ran: the settled reading against the limit the driver enforces
      "board_power": {"cap_w": power.cap_w, "gemm_w": gemm_w, "gemm_max_w": gemm_max_w,
                      "before_gemm_legs_w": idle_w,
                      "source": power.path},
  }
  # Where the workgroups of such a launch finish, by XCD (the measurement instance of the same
  # kernel: cdit_debug_gemm_stamps): the clocks of the eight XCDs differ under the power
  # limit, the launch ends with the slowest; whether handing tiles out dynamically could
  # help is a matter of that spread against one tile's time.
  from cache_dit_amd import _native
  L, stream = _native.load(), torch.cuda.current_stream().cuda_stream
  try:
    import ctypes
    stamps = torch.zeros(4 * 256, dtype=torch.int64, device=device)
    n_wg = ctypes.c_int(0)
    per_xcd, last_xcd, tile_us, launch_us = {}, {}, [], []
    for rep in range(12):
      for _ in range(25):  # keeps the part in the power-limited state the timed legs run in
        gemm()
      i = it["i"] = (it["i"] + 1) % nbuf
      _native.check(L.cdit_debug_gemm_stamps(qs[i].data_ptr(), ss[i].data_ptr(), ws[i].data_ptr(),
                                              wsc.data_ptr(), b.data_ptr(), outs[i & 1].data_ptr(),
                                              M, N, K, K, K, N, stamps.data_ptr(), ctypes.byref(n_wg),
                                              stream))
      torch.cuda.synchronize()
      if rep < 2:
        continue  # (warm-up)
      st = stamps.view(-1, 4)[:n_wg.value].cpu()
      t0 = int(st[:, 0].min())
      end_us = (st[:, 1] - t0).double() / 100.0  # 100 MHz ticks
      launch_us.append(float(end_us.max()))
      tile_us.append(float(((st[:, 1] - st[:, 0]).double() / st[:, 3].double()).mean() / 100.0))
      for x in sorted(set(st[:, 2].tolist())):
        per_xcd.setdefault(int(x), []).append(float(end_us[st[:, 2] == x].mean()))
        last_xcd.setdefault(int(x), []).append(float(end_us[st[:, 2] == x].max()))
    xcd_last = {x: sum(v) / len(v) for x, v in last_xcd.items()}
    xcd_mean = {x: sum(v) / len(v) for x, v in per_xcd.items()}
    t_tile = sum(tile_us) / len(tile_us)
    finish = {
        "mean_finish_us_by_xcd": [round(xcd_mean[x], 2) for x in sorted(xcd_mean)],
        "last_finish_us_by_xcd": [round(xcd_last[x], 2) for x in sorted(xcd_last)],
        "launch_us": round(sum(launch_us) / len(launch_us), 2),
        "tile_us": round(t_tile, 2),
        "tiles_per_workgroup": float(st[:, 3].double().mean()),
        "spread_fastest_to_slowest_xcd_in_tiles": round((max(xcd_mean.values()) - min(xcd_mean.values())) / t_tile, 3),
        "note": "10 launches of the 288x192 kernel with per-workgroup time stamps, each behind 25 "
                "ordinary launches; finish = end of a workgroup after the first start, averaged per "
                "XCD; a tile = a workgroup's time / its tiles",
    }
  except Exception as e:
    finish = {"note": f"unavailable: {str(e)[:120]}"}
  res["xcd_finish_times"] = finish
  # What bounds the quantizer at this size: the fixed cost of a launch of M one-wavefront
  # workgroups. The same kernel with K = 0 (4608 workgroups that only write their scale)
  # and on a single row, next to the 42 MB case; rocprofv3 --kernel-trace of this command
  # gives the matching device-side durations (profiles/).

  def quant_raw(rows, cols):
    def fn():
      i = it["i"] = (it["i"] + 1) % nbuf
      _native.check(L.cdit_fp8_quant_rowwise(xs[i].data_ptr(), rows, cols, K, qs[i].data_ptr(), K,
                                             ss[i].data_ptr(), 0, stream))
    return fn

  res["quant_floor"] = {
      "empty_4608_workgroups_us": _time_events(quant_raw(M, 0), 200, 20) * 1e3,
      "one_row_us": _time_events(quant_raw(1, K), 200, 20) * 1e3,
      "headline_us": quant_ms * 1e3,
      "note": "HIP-event averages over back-to-back launches: K=0 (every workgroup only writes "
              "its scale), one row of K=3072, and the 4608 x 3072 activation",
  }
  # the quantizer fused into its producer (LayerNorm + AdaLN modulation + quantization in one
  # pass, bf16 output not written): same algorithmic bytes as the quantizer alone, 3MK + 4M
  shift = torch.randn(K, device=device, generator=g).to(torch.bfloat16)
  scale_mod = (torch.randn(K, device=device, generator=g) * 0.3).to(torch.bfloat16)

  def ln_quant():
    i = it["i"] = (it["i"] + 1) % nbuf
    _native.check(L.cdit_fp8_ln_modulate_quant(xs[i].data_ptr(), M, K, K, shift.data_ptr(),
                                               scale_mod.data_ptr(), K, M, 1e-6, None, K,
                                               qs[i].data_ptr(), K, ss[i].data_ptr(), 0, stream))

  lnq_ms = sorted(_time_events(ln_quant, 100, 20 if k == 0 else 0) for k in range(5))[2]
  res["ln_modulate_quant_ms"] = lnq_ms
  res["ln_modulate_quant_gbps"] = (3.0 * M * K + 4.0 * M) / lnq_ms / 1e6
  for i in range(nbuf):  # the codes the later legs read are those of xs again
    ops.quant_rowwise_into(xs[i], qs[i], ss[i], 0)
  res["gemm_frac_fp8_peak"] = res["gemm_tflops"] / FP8_PEAK_TFLOPS
  res["quant_frac_hbm_peak"] = res["quant_gbps"] / HBM_PEAK_GBPS
  res["linear_tflops"] = 2.0 * M * K * N / (gemm_ms + quant_ms) / 1e9
  # the vendor library on the same codes, as a comparator (not a baseline)
  try:
    a_s = ss[0].reshape(M, 1)
    w_s = wsc.reshape(1, N)

    def vendor():
      torch._scaled_mm(qs[0], ws[0].t(), scale_a=a_s, scale_b=w_s, bias=b,
                       out_dtype=torch.bfloat16)

    v_ms = _time_events(vendor, 20, 5)
    res["hipblaslt_scaled_mm_tflops"] = 2.0 * M * K * N / v_ms / 1e9
  except Exception as e:  # not every build has row-wise _scaled_mm
    res["hipblaslt_scaled_mm_tflops"] = None
    res["hipblaslt_note"] = str(e)[:120]
  # weight-only mode at the same shape
  try:
    def w8a16():
      i = it["i"] = (it["i"] + 1) % nbuf
      ops.w8a16_into(xs[i], ws[i], wsc, b, outs[i & 1], 0)

    # (settled clocks as for the FP8 GEMM: blocks of 50 launches until two in a row agree to
    # 0.5 %, at most 2 s, then the median of three blocks)
    t_start, prev = time.perf_counter(), _time_events(w8a16, 50, 20)
    while time.perf_counter() - t_start < 2.0:
      cur = _time_events(w8a16, 50, 0)
      settled = abs(cur - prev) <= 0.005 * prev
      prev = cur
      if settled and time.perf_counter() - t_start > 0.5:
        break
    w_ms = sorted(_time_events(w8a16, 50, 0) for _ in range(3))[1]
    res["w8a16_ms"] = w_ms
    res["w8a16_tflops"] = 2.0 * M * K * N / w_ms / 1e9
    res["w8a16_frac_bf16_peak"] = res["w8a16_tflops"] / BF16_PEAK_TFLOPS
    # comparators on the same box: the vendor library's plain bf16 GEMM on a bf16 copy of the
    # weights, and the form the weight-only mode replaces (dequantize with tensor ops, then
    # that GEMM)
    wb = [ws[i].to(torch.bfloat16) for i in range(2)]

    def blas_bf16():
      i = it["i"] = (it["i"] + 1) % nbuf
      torch.nn.functional.linear(xs[i], wb[i & 1], b)

    def dequant_then_gemm():
      i = it["i"] = (it["i"] + 1) % nbuf
      w = (ws[i].to(torch.float32) * wsc[:, None]).to(torch.bfloat16)
      torch.nn.functional.linear(xs[i], w, b)

    res["hipblaslt_bf16_tflops"] = 2.0 * M * K * N / _time_events(blas_bf16, 30, 10) / 1e9
    res["w8a16_dequant_then_gemm_ms"] = _time_events(dequant_then_gemm, 20, 5)
    del wb
  except Exception as e:
    res["w8a16_note"] = str(e)[:120]
  # the per-tensor quantizer (float8_per_tensor and the policy's fallback pass): three launches
  # (zero the amax word, amax over the tensor, cast), the tensor read twice: 5MK + 4M bytes
  try:
    amax_ws = torch.zeros(1, dtype=torch.int32, device=device)

    def pt_tensor():
      i = it["i"] = (it["i"] + 1) % nbuf
      ops.quant_tensorwise_into(xs[i], qs[i], ss[i], amax_ws, 0)

    pt_ms = sorted(_time_events(pt_tensor, 100, 20 if k == 0 else 0) for k in range(3))[1]
    res["per_tensor_quant_ms"] = pt_ms
    res["per_tensor_quant_gbps"] = (5.0 * K + 4) * M / pt_ms / 1e6
  except Exception as e:
    res["per_tensor_quant_note"] = str(e)[:120]
  # the FP8 comm quantizers (scale packed behind each row) on an activation of the headline
  # size and on its q/k/v as [B, S, 3, heads, head_dim]; GB/s over their algorithmic bytes
  try:
    heads, hd = 24, 128
    yq = [torch.empty(M, K + 2, dtype=torch.uint8, device=device) for _ in range(nbuf)]
    back = torch.empty(M, K, dtype=torch.bfloat16, device=device)
    qkv = [torch.randn(1, M, 3, heads, hd, device=device, generator=g).to(torch.bfloat16)
           for _ in range(3)]
    pq = [torch.empty(3, M, 1, heads, hd + 4, dtype=torch.uint8, device=device) for _ in range(3)]
    pback = torch.empty(1, M, heads, hd, dtype=torch.bfloat16, device=device)

    def pt_quant():
      i = it["i"] = (it["i"] + 1) % nbuf
      _native.check(L.cdit_fp8_comm_per_token_quant(xs[i].data_ptr(), M, K, yq[i].data_ptr(), stream))

    def pt_dequant():
      i = it["i"] = (it["i"] + 1) % nbuf
      _native.check(L.cdit_fp8_comm_per_token_dequant(yq[i].data_ptr(), M, K, back.data_ptr(), stream))

    def qkv_quant():
      i = it["i"] = (it["i"] + 1) % 3
      x = qkv[i]
      _native.check(L.cdit_fp8_comm_qkv_permute_quant(
          x.data_ptr(), 1, M, 3, heads, hd, x.stride(0), x.stride(1), x.stride(2),
          pq[i].data_ptr(), stream))

    def qkv_dequant():
      i = it["i"] = (it["i"] + 1) % 3
      one = pq[i][0]  # [S, B, N, D + 4] bytes: strides are byte strides
      _native.check(L.cdit_fp8_comm_qkv_permute_dequant(one.data_ptr(), M, 1, heads, hd, one.stride(0),
                                                        one.stride(1), one.stride(2),
                                                        pback.data_ptr(), stream))

    rows = 3 * M * heads
    res["comm_quant"] = {
        "per_token_quant_gbps": (3.0 * K + 2) * M / _time_events(pt_quant, 200, 20) / 1e6,
        "per_token_dequant_gbps": (3.0 * K + 2) * M / _time_events(pt_dequant, 200, 20) / 1e6,
        "qkv_permute_quant_gbps": (3.0 * hd + 4) * rows / _time_events(qkv_quant, 100, 10) / 1e6,
        "qkv_permute_dequant_gbps": (3.0 * hd + 4) * (rows / 3) / _time_events(qkv_dequant, 100, 10) / 1e6,
        "note": "per token: 4608 x 3072 bf16 <-> codes + bf16 scale; qkv: [1, 4608, 3, 24, 128] "
                "-> [3, 4608, 1, 24, 132], dequant of one of the three slices",
    }
  except Exception as e:
    res["comm_quant_note"] = str(e)[:160]
  return res


def mfma_only_ceiling(device):
  """What the matrix cores of this part sustain on the GEMM's own instruction
  (v_mfma_f32_16x16x128_f8f6f4) with nothing else going on: 256 workgroups of four
  wavefronts, register operands, no memory traffic (cdit_debug_mfma_only). With all-ones
  operands the part holds its rated clock; with random e4m3 operands (the benchmark's data)
  the power limit lowers it. The random-operand figure is the ceiling of any FP8 kernel on
  this data before a byte is moved. Each case: two warm-up launches, then the median of
  three launches of about 15 ms."""
  import ctypes
  import torch
  from cache_dit_amd import _native
  L, stream = _native.load(), torch.cuda.current_stream().cuda_stream
  blocks, iters = 256, 60000
  out = torch.empty(blocks * 256, dtype=torch.float32, device=device)
  res = {}
  for key, rnd in (("constant_operands_tflops", 0), ("random_operands_tflops", 1)):
    flop = ctypes.c_double(0.0)

    def fn():
      _native.check(L.cdit_debug_mfma_only(out.data_ptr(), blocks, iters, rnd, ctypes.byref(flop), stream))

    times = sorted(_time_events(fn, 1, 2 if k == 0 else 0) for k in range(3))
    res[key] = flop.value / times[1] / 1e9
    # the same loop held for 0.6 s (40 launches) with the board power sampled: the smoothed
    # reading needs that long; the rate of the last 10 launches next to it
    with _BoardPower(torch.device(device).index or 0) as power:
      _time_events(fn, 30, 0)
      sustained_ms = _time_events(fn, 10, 0)
    res[key.replace("_tflops", "_sustained_tflops")] = flop.value / sustained_ms / 1e9
    res[key.replace("_tflops", "_board_w")] = power.settled_w()
    res["board_cap_w"] = power.cap_w
  res["note"] = ("loop of v_mfma_f32_16x16x128_f8f6f4 on register operands, 256 workgroups x 4 "
                 "wavefronts, 16 independent accumulators, no memory traffic; HIP events")
  return res


def quant_large_shapes(device):
  """The per-row quantizer on the largest activation of each benchmark configuration
  (FLUX proj_out input 4608 x 15360, Qwen-Image MLP hidden 6889 x 12288, Wan hidden
  32760 x 5120 and FFN hidden 32760 x 13824): algorithmic bytes 3MK + 4M over the median of
  five blocks of launches, rotating over two buffer sets (each beyond the 256 MiB last-level
  cache together with its codes)."""
  import torch
  from cache_dit_amd import ops
  out = []
  g = torch.Generator(device=device).manual_seed(2)
  for name, M, K in (("flux proj_out input", 4608, 15360), ("qwen img_mlp.net.2 input", 6889, 12288),
                     ("wan hidden", 32760, 5120), ("wan ffn.net.2 input", 32760, 13824)):
    xs = [torch.randn(M, K, device=device, generator=g).to(torch.bfloat16) for _ in range(2)]
    qs = [torch.empty(M, K, dtype=torch.float8_e4m3fn, device=device) for _ in range(2)]
    sc = [torch.empty(M, dtype=torch.float32, device=device) for _ in range(2)]
    it = {"i": 0}

    def quant():
      i = it["i"] = it["i"] ^ 1
      ops.quant_rowwise_into(xs[i], qs[i], sc[i], 0)

    n = max(10, min(100, int(2.0e10 / (3.0 * M * K))))  # about 3 ms per block at 6 TB/s
    blocks = sorted(_time_events(quant, n, 4 if k == 0 else 0) for k in range(5))
    nbytes = 3.0 * M * K + 4.0 * M
    gbps = nbytes / blocks[2] / 1e6
    out.append({"kernel": f"per-row quantizer, {name} (M={M} K={K})", "bound": "hbm",
                "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS,
                "traffic": None, "algorithmic_bytes": nbytes, "us": blocks[2] * 1e3,
                "us_fastest_block": blocks[0] * 1e3, "us_slowest_block": blocks[-1] * 1e3})
    del xs, qs, sc
    torch.cuda.empty_cache()
  return out


def cpu_baseline():
  """The CPU restatement of the reference path (oracle.torch_oracle: eager PyTorch
  CPU ops) on benchmark config 1 (M=4608, K=3072, N=3072): activation quantization +
  scaled matmul + bias, weights pre-quantized. One warm-up, then timed runs for about
  10 s of CPU work; the median is reported."""
  import torch
  from oracle import torch_oracle as to
  cores = os.cpu_count() or 1
  try:  # a shared host exports its CPU share this way
    cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
  except ValueError:
    pass
  torch.set_num_threads(cores)
  # benchmark config 1, drawn exactly as the parity tests draw it (seed 0, CPU generator,
  # fp32 then bf16): x ~N(0,1) with max(1, floor(0.001 K)) = 3 channels picked by
  # randperm scaled by 20, W ~N(0,0.02), bias ~N(0,0.01)
  g = torch.Generator().manual_seed(0)
  M, K, N = 4608, 3072, 3072
  x = torch.randn(1, M, K, generator=g)
  x[..., torch.randperm(K, generator=g)[:max(1, int(0.001 * K))]] *= 20.0
  x = x.to(torch.bfloat16).reshape(M, K)
  w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
  b = (torch.randn(N, generator=g) * 0.01).to(torch.bfloat16)
  wq, ws = to.quantize_rowwise(w)
  times, qtimes = [], []
  budget_s, started = 10.0, None
  while started is None or len(times) < 3 or (
      time.perf_counter() - started < budget_s and len(times) < 1000):
    t0 = time.perf_counter()
    xq, xs = to.quantize_rowwise(x)
    t1 = time.perf_counter()
    to.scaled_mm_rowwise(xq, xs, wq, ws, b)
    t2 = time.perf_counter()
    if started is None:  # warm-up run
      started = t2
      continue
    times.append(t2 - t0)
    qtimes.append(t1 - t0)
  total_s = sum(times)
  times.sort()
  qtimes.sort()
  t, tq = times[len(times) // 2], qtimes[len(qtimes) // 2]
  return {
      "value": 2.0 * M * K * N / t / 1e12,
      "unit": "TFLOP/s",
      "cores": torch.get_num_threads(),
      "kind": "port",
      "sample": f"benchmark config 1 linear (M={M} K={K} N={N}, 3 outlier channels x20): per-token quant + scaled matmul "
                f"+ bias in eager PyTorch CPU ops, median of {len(times)} runs ({total_s:.0f} s of "
                f"CPU work), {t*1e3:.0f} ms/linear",
      "quant_gbps": (3.0 * M * K + 4.0 * M) / tq / 1e9,
      "ms_per_linear": t * 1e3,
  }


def dit_forward_ms(device, iters=5):
  """Full synthetic FLUX-shaped transformer forward (attention, norms, RoPE and residual
  glue included), quantized with float8_per_row and set up the way a serving loop would:
  GELU-tanh folded into the producing Linear, sibling Linears grouped, the quantizer fused
  into the modulated LayerNorms. Timed with eager launches and as one hipGraph replay.
  Returns (eager ms, graph ms or None, note)."""
  try:
    import torch
    import cache_dit_amd
    from cache_dit_amd.testing import dit_shapes
    from cache_dit_amd.testing.dit_shapes import FluxLikeTransformer, flux_like_inputs
  except Exception as e:
    return None, None, f"synthetic transformer unavailable: {e}"[:160]
  torch.manual_seed(0)
  with torch.device(device):
    model = FluxLikeTransformer().to(torch.bfloat16)
  cache_dit_amd.quantize(model, cache_dit_amd.QuantizeConfig(quant_type="float8_per_row"))
  dit_shapes.fuse_gelu_epilogues(model)
  inputs = flux_like_inputs(device)
  # the model's block and attention code stays as it is: the stage patch functor rebinds the
  # forwards of the blocks and of their attention modules (cache_dit_amd.patch_functors)
  cache_dit_amd.apply_stage_patch(model, batch_stages=True, single_blocks=True, fuse_cat=True,
                                  fuse_norm_quant=True, materialize=False)
  graph_ms = None
  with torch.no_grad():
    ms = _time_events(lambda: model(**inputs), iters, 2)
    try:
      side = torch.cuda.Stream()
      side.wait_stream(torch.cuda.current_stream())
      with torch.cuda.stream(side):
        model(**inputs)
      torch.cuda.current_stream().wait_stream(side)
      torch.cuda.synchronize()
      graph = torch.cuda.CUDAGraph()
      with torch.cuda.graph(graph):
        model(**inputs)
      graph_ms = _time_events(graph.replay, iters, 2)
      del graph
    except Exception as e:
      graph_ms = None
      note_err = f"; graph capture failed: {str(e)[:80]}"
    else:
      note_err = ""
  del model
  torch.cuda.empty_cache()
  return ms, graph_ms, ("float8_per_row on the unmodified synthetic model + apply_stage_patch: "
                        "GELU-tanh fused into the producing Linear, the Linears of a stage (image "
                        "and text stream, proj_mlp + q/k/v) one quantizer and one batched GEMM "
                        "launch, quantizer fused into the modulated LayerNorms and reading "
                        "proj_out's two sources in place; bf16 SDPA attention, RMS norms, RoPE "
                        "and residual glue in eager PyTorch ops" + note_err)


def dit_forward_compiled_ms(device, iters=5):
  """The same transformer, stage-patched, with its blocks compiled by torch.compile (regional
  compilation, fullgraph): every stage is one registered batch op, every other converted
  Linear one op, so Inductor fuses the element-wise glue around them. Returns (ms, seconds
  spent compiling, cosine against the eager forward) or (None, None, note)."""
  try:
    import torch
    import cache_dit_amd
    from cache_dit_amd.testing import dit_shapes
    torch.manual_seed(0)
    with torch.device(device):
      model = dit_shapes.FluxLikeTransformer().to(torch.bfloat16)
    cache_dit_amd.quantize(model, cache_dit_amd.QuantizeConfig(quant_type="float8_per_row"))
    dit_shapes.fuse_gelu_epilogues(model)
    inputs = dit_shapes.flux_like_inputs(device)
    with torch.no_grad():
      want = model(**inputs)
      # (inside the traced graph the rebound forwards emit one batch op per stage; the fused
      # norms stay tensor ops there, which Inductor fuses itself)
      cache_dit_amd.apply_stage_patch(model)
      t0 = time.perf_counter()
      for blk in list(model.transformer_blocks) + list(model.single_transformer_blocks):
        blk.compile(fullgraph=True)
      got = model(**inputs)
      torch.cuda.synchronize()
      compile_s = time.perf_counter() - t0
      ms = _time_events(lambda: model(**inputs), iters, 2)
    cos = torch.nn.functional.cosine_similarity(want.float().flatten(), got.float().flatten(),
                                                dim=0).item()
    del model
    torch.cuda.empty_cache()
    return ms, compile_s, cos
  except Exception as e:  # no Inductor back end on this box, or a compile failure
    return None, None, f"torch.compile leg failed: {str(e)[:160]}"


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=10)
  ap.add_argument("--warmup", type=int, default=3)
  ap.add_argument("--skip-cpu", action="store_true", help="skip the cpu_baseline leg")
  ap.add_argument("--skip-dit", action="store_true", help="skip the full-transformer forward")
  ap.add_argument("--skip-compiled", action="store_true",
                  help="skip the torch.compile leg of the full-transformer forward")
  ap.add_argument("--skip-other-configs", action="store_true",
                  help="skip the step legs of the other benchmark configurations (FLUX-shaped "
                       "w8a16, Qwen-Image-shaped and Wan-shaped w8a8)")
  ap.add_argument("--headline-only", action="store_true",
                  help="run only the headline-shape kernels (the roofline legs) and print their "
                       "figures: the command to put under rocprofv3 when per-kernel averages "
                       "must not mix shapes")
  ap.add_argument("--dit-only", action="store_true",
                  help="run only the full synthetic transformer forward (eager and as a hipGraph "
                       "replay): the command to put under rocprofv3 for the kernel mix of a whole "
                       "DiT step")
  ap.add_argument("--pmc-sequence", action="store_true",
                  help="run only the launch sequence for rocprofv3 --pmc counter collection "
                       "(fill, plain copy, quantizer, fill, GEMM at the headline shape, 4 times)")
  ap.add_argument("--step-only", action="store_true",
                  help="run only the hot-path step legs (eager, hipGraph replay, shared "
                       "quantization) and print their figures: the command to put under "
                       "rocprofv3 for the kernel mix of one step")
  ap.add_argument("--step-form", default="all",
                  choices=["all", "batched", "grouped", "shared", "ungrouped"],
                  help="with --step-only: time just this form of the step (default: all four "
                       "and the eager launches), so that a kernel trace covers one form")
  args = ap.parse_args()
  if args.gpus != 1:
    sys.exit("bench.py: this build runs on exactly one GPU (no collectives, no sharding); "
             "use --gpus 1")
  import torch
  if not torch.cuda.is_available():
    sys.exit("bench.py: no GPU visible; the hot path has no CPU fallback")
  from cache_dit_amd import _native
  device = torch.device("cuda", 0)
  torch.cuda.set_device(device)
  arch = _native.device_arch()

  if args.pmc_sequence:
    pmc_sequence(device)
    print(json.dumps({"pmc_sequence": "done", "device": arch}))
    return
  if args.dit_only:
    ms, gms, note = dit_forward_ms(device, iters=args.steps)
    out = {"dit_step_ms": ms, "dit_step_ms_graph": gms, "dit_step_note": note, "device": arch}
    if not args.skip_compiled:
      cms, cs, cos = dit_forward_compiled_ms(device, iters=args.steps)
      out.update({"dit_step_ms_compiled": cms, "dit_compile_seconds": cs, "dit_compiled_cosine": cos})
    print(json.dumps(out))
    return
  if args.headline_only:
    print(json.dumps({"linear_headline": headline_kernels(device),
                      "mfma_only": mfma_only_ceiling(device),
                      "roofline_quant_large": quant_large_shapes(device), "device": arch}))
    return

  hot = HotPath(device)
  one_form = args.step_form if args.step_only and args.step_form != "all" else None
  eager_ms = None
  if one_form is None:
    for _ in range(args.warmup):
      hot.step()
    torch.cuda.synchronize()
    # eager launches (988 kernel launches per step issued from Python)
    t0 = time.perf_counter()
    for _ in range(args.steps):
      hot.step()
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) / args.steps * 1e3
  # The same step captured once into a hipGraph and replayed: what a serving loop does
  # with a fixed-shape denoising step; removes the host launch cost. Four forms of the
  # step, all with bit-identical outputs: every Linear on its own (quantizer + GEMM each);
  # one quantizer launch per distinct activation (share_activation_quant_); sibling Linears
  # also as one grouped GEMM launch (group_sibling_linears_); and, the headline, every stage
  # of a block -- the siblings of the image stream together with those of the text stream --
  # as one batched GEMM launch (block forwards written against linear_batch).
  def replay_ms(step_fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
      step_fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
      step_fn()
    for _ in range(args.warmup):
      graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):  # exactly `steps` timed steps
      graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / args.steps * 1e3

  launch_mode = "hipGraph replay"
  if one_form is not None:
    form = {"batched": hot.step_batched, "grouped": hot.step_grouped,
            "shared": hot.step_shared_quant, "ungrouped": hot.step}[one_form]
    ms = replay_ms(form)
    print(json.dumps({"step_form": one_form, "ms_per_step": ms, "tflops": hot.flop / ms / 1e9,
                      "launch": launch_mode, "steps": args.steps, "warmup": args.warmup,
                      "device": arch}))
    return
  try:
    ungrouped_ms = replay_ms(hot.step)
    shared_ms = replay_ms(hot.step_shared_quant)
    grouped_ms = replay_ms(hot.step_grouped)
    ms_per_step = replay_ms(hot.step_batched)
  except Exception as e:  # capture unavailable: report the eager figure of the plain step
    launch_mode = f"eager (graph capture failed: {str(e)[:80]})"
    ungrouped_ms = shared_ms = grouped_ms = None
    ms_per_step = eager_ms
  value = hot.flop / ms_per_step / 1e9
  n_runs = len(hot.stages())
  n_layers = len(hot.layers)
  step_flop = hot.flop
  del hot
  torch.cuda.empty_cache()
  if args.step_only:
    print(json.dumps({"value": value, "unit": "TFLOP/s", "ms_per_step": ms_per_step,
                      "launch": launch_mode, "eager_ms_per_step": eager_ms,
                      "ungrouped_ms_per_step": ungrouped_ms,
                      "shared_quant_ms_per_step": shared_ms,
                      "grouped_ms_per_step": grouped_ms, "steps": args.steps,
                      "warmup": args.warmup, "device": arch}))
    return

  head = headline_kernels(device)
  ceiling = mfma_only_ceiling(device)
  quant_large = quant_large_shapes(device)
  M, K, N = HEADLINE
  roofline = {
      "kernel": "gemm_fp8_wide<288x192> (w8a8 GEMM + scale/bias epilogue) at M=4608 K=3072 "
                "N=12288",
      "bound": "mfma",
      "achieved": head["gemm_tflops"],
      "peak": FP8_PEAK_TFLOPS,
      "unit": "TFLOP/s",
      "frac": head["gemm_tflops"] / FP8_PEAK_TFLOPS,
      # HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a plain
      # copy of known size (read from profiles/traffic.json); algorithmic 165.2 MB
      "traffic": measured_traffic("gemm_fp8_wide_headline"),
      # the same instruction with nothing else going on, timed in this run (mfma_only): the
      # rate the power-limited part sustains on random e4m3 operands, and the GEMM against it
      "mfma_only_tflops": ceiling["random_operands_tflops"],
      "frac_of_mfma_only": head["gemm_tflops"] / ceiling["random_operands_tflops"],
      # board power the driver reports while this kernel runs back to back, and its limit
      "board_power_w": head["board_power"]["gemm_max_w"],
      "board_power_cap_w": head["board_power"]["cap_w"],
  }
  roofline_quant = {
      "kernel": "quant_rowwise_regs at M=4608 K=3072",
      "bound": "hbm",
      "achieved": head["quant_gbps"],
      "peak": HBM_PEAK_GBPS,
      "unit": "GB/s",
      "frac": head["quant_gbps"] / HBM_PEAK_GBPS,
      "traffic": measured_traffic("quant_rowwise_headline"),  # algorithmic 3MK + 4M = 42.49 MB
  }
  other = {}
  if not args.skip_other_configs:
    few = max(2, args.steps // 3)  # these steps are long; a few replays settle them
    other["w8a16_step"] = step_leg(device, flux_step_linears(), "w8a16", args.steps, args.warmup)
    other["w8a16_step"]["frac_bf16_peak"] = other["w8a16_step"]["tflops"] / BF16_PEAK_TFLOPS
    other["qwen_step"] = step_leg(device, qwen_step_linears(), "w8a8", few, 1)
    other["wan_step"] = step_leg(device, wan_step_linears(), "w8a8", few, 1)
    for k in ("qwen_step", "wan_step"):
      other[k]["frac_fp8_peak"] = other[k]["tflops"] / FP8_PEAK_TFLOPS
  dit_ms, dit_graph_ms, dit_note = (None, None, "skipped") if args.skip_dit else dit_forward_ms(device)
  dit_compiled = (None, None, "skipped")
  if not args.skip_dit and not args.skip_compiled:
    dit_compiled = dit_forward_compiled_ms(device)
  cpu = None if args.skip_cpu else cpu_baseline()

  line = {
      "metric": "fp8_w8a8_linear_tflops",
      "value": value,
      "unit": "TFLOP/s",
      "n_gpus": 1,
      "steps": args.steps,
      "warmup": args.warmup,
      "ms_per_step": ms_per_step,
      "higher_is_better": True,
      "scaling": "weak",
      "vs_baseline": None,
      "dtype": "fp8_e4m3 (fp32 accumulate, bf16 out)",
      "data": "synthetic",
      "config": {
          "workload": "flux1_dev_shaped_step: all quantized Linears of one denoising step "
                      "(19 double + 38 single blocks, 4096 img + 512 txt tokens): per-token "
                      "quant + FP8 GEMM + epilogue; Linears that read one activation (q/k/v, "
                      "proj_mlp + q/k/v) share its quantization, and the independent Linears of "
                      "one stage of a block (image stream + text stream) run as one quantizer "
                      "launch and one batched GEMM launch (two where the tile cost model splits "
                      "the stage), bit-identical to running each Linear on its own. This is the "
                      "launch pattern cache_dit_amd.apply_stage_patch gives an unmodified model "
                      "(rebound forwards of its attention modules and blocks); plain "
                      "quantize() alone gives ungrouped_*, group_sibling_linears_ grouped_*",
          "quant_type": "float8_per_row",
          "launch": launch_mode,
          "linears_per_step": n_layers,
          "stages_per_step": n_runs,
          "linear_flop_per_step": step_flop,
          "batch": 1,
      },
      "frac_fp8_peak": value / FP8_PEAK_TFLOPS,
      # the same step with every Linear on its own (eager launches, then replayed), and
      # with shared quantization but one GEMM launch per Linear
      "eager_ms_per_step": eager_ms,
      "ungrouped_ms_per_step": ungrouped_ms,
      "ungrouped_tflops": None if not ungrouped_ms else step_flop / ungrouped_ms / 1e9,
      "shared_quant_ms_per_step": shared_ms,
      # sibling Linears grouped per activation only (what group_sibling_linears_ gives a model
      # whose block forwards are untouched)
      "grouped_ms_per_step": grouped_ms,
      "grouped_tflops": None if not grouped_ms else step_flop / grouped_ms / 1e9,
      "linear_headline": head,
      # the other benchmark configurations as steps of their own (same construction as the
      # headline step): config 3 = FLUX-shaped w8a16, config 4 = Qwen-Image-shaped w8a8,
      # config 5 = Wan2.1-14B-shaped w8a8
      "w8a16_step_ms": other.get("w8a16_step", {}).get("ms_per_step"),
      "w8a16_step_tflops": other.get("w8a16_step", {}).get("tflops"),
      "w8a16_step_frac_bf16_peak": other.get("w8a16_step", {}).get("frac_bf16_peak"),
      "qwen_step_ms": other.get("qwen_step", {}).get("ms_per_step"),
      "qwen_step_tflops": other.get("qwen_step", {}).get("tflops"),
      "wan_step_ms": other.get("wan_step", {}).get("ms_per_step"),
      "wan_step_tflops": other.get("wan_step", {}).get("tflops"),
      "other_configs": other,
      "dit_step_ms": dit_ms,
      "dit_step_ms_graph": dit_graph_ms,
      "dit_step_note": dit_note,
      # the same forward with its blocks under torch.compile (Inductor fuses the glue around
      # the registered ops), seconds spent compiling, cosine against the eager forward
      "dit_step_ms_compiled": dit_compiled[0],
      "dit_compile_seconds": dit_compiled[1],
      "dit_compiled_cosine": dit_compiled[2],
      "roofline": roofline,
      "roofline_quant": roofline_quant,
      # the same kernel on the largest activation of each benchmark configuration
      "roofline_quant_large": quant_large,
      "roofline_ln_modulate_quant": {
          "kernel": "ln_modulate_quant (LayerNorm + AdaLN modulation + per-row quantizer in one "
                    "pass) at M=4608 K=3072",
          "bound": "hbm", "achieved": head["ln_modulate_quant_gbps"], "peak": HBM_PEAK_GBPS,
          "unit": "GB/s", "frac": head["ln_modulate_quant_gbps"] / HBM_PEAK_GBPS,
          "traffic": measured_traffic("ln_modulate_quant_headline"),
      },
      "mfma_only": ceiling,
      "cpu_baseline": cpu,
      "device": arch,
  }
  print(json.dumps(line))


if __name__ == "__main__":
  main()
