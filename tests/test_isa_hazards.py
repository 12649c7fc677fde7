"""The wide GEMM kernels (w8a8 and w8a16) issue their MFMAs through inline assembly
(the accumulators are tied to AGPR tuples), so the compiler's hazard recognizer
does not see them. This test compiles their sources to gfx950 assembly (no GPU
needed) and checks, in the code the compiler produced for every instance,
three situations in which the hardware needs software wait states, and two
things the compiler may add that the kernels must not have:

  1. no MFMA reads (as its C operand) an AGPR that a VALU instruction
     (v_accvgpr_write / v_accvgpr_mov) wrote: accumulators start from MFMAs with a
     zero C operand and are otherwise only written by MFMAs;
  2. no VALU instruction writes a VGPR in the 4 instructions before an MFMA that
     reads it as A or B operand (the w8a16 kernel converts its weights to bf16 one
     block ahead of their use; an operand converted right before the MFMA gave
     wrong results on hardware);
  3. at least 18 wait states lie between an MFMA and the first v_accvgpr_read of
     an accumulator (the epilogue);
  4. no `s_waitcnt vmcnt(0)` lies between the first and the last MFMA: the K loop
     waits for the LDS-DMA of the next step only. The compiler drains all of it
     before an LDS read that it thinks may alias an LDS-DMA write, which exposes
     the memory latency at every step; reads through a restrict-qualified pointer
     carry alias scope information and are exempt;
  5. no scratch (register spill) access anywhere: a scratch reload is a vector
     memory load, the wait for it (vmcnt) also waits for every output store in
     flight, which serialises the epilogue of a tile with the next tile's K loop;
  6. (w8a8 kernel) the waits of the first K steps of a tile count the output stores
     of the previous tile's epilogue, so every wave must issue all of them whatever
     part of the tile exists: the expected number of buffer stores, no global stores,
     none under a lane mask or inside a loop over descriptor values;
  7. (w8a8 kernel) the epilogue operands staged in LDS by DMA are read after a vmcnt wait
     that covers them: with a DMA stream more than 3 steps deep the waits of the K loop
     do not, and the first LDS read after the last MFMA of a tile needs one of its own.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "cache_dit_amd", "csrc")
SOURCES = {"gemm_fp8.hip": "gemm_fp8_wide", "gemm_w8a16.hip": "gemm_w8a16_wide"}


def _hipcc():
  for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
    if cand and os.path.exists(cand):
      return cand
  return None


labeled = {}  # the same kernels with their branch labels kept (for control-flow checks)


@pytest.fixture(scope="module", params=sorted(SOURCES))
def wide_kernels(request, tmp_path_factory):
  hipcc = _hipcc()
  if hipcc is None:
    pytest.skip("hipcc not found")
  src, kernel = request.param, SOURCES[request.param]
  out = tmp_path_factory.mktemp("isa") / (src + ".s")
  from cache_dit_amd.csrc import build
  cmd = [hipcc, *build.DEVICE_FLAGS, "-I", os.path.join(ROOT, "include"), "-I", CSRC,
         "--cuda-device-only", "-S", os.path.join(CSRC, src), "-o", str(out)]
  r = subprocess.run(cmd, capture_output=True, text=True)
  assert r.returncode == 0, r.stderr[-2000:]
  text = out.read_text()
  kernels = {}
  labeled.clear()
  for m in re.finditer(r"^(_ZN\S*" + kernel + r"\S*):[^\n]*\n(.*?)s_endpgm", text, re.S | re.M):
    body = [l.strip() for l in m.group(2).split("\n")]
    kernels[m.group(1)] = [l for l in body if l and not l.startswith(";") and not l.startswith(".")]
    labeled[m.group(1)] = [l.split(";")[0].strip() for l in body
                           if l and not l.startswith(";") and
                           (not l.startswith(".") or re.match(r"\.\w+:", l))]
  assert len(kernels) >= 3, "wide kernel instances not found in the assembly"
  return kernels


def _regs(tok):
  """v[8:15] -> ('v', {8..15}); a12 -> ('a', {12}); else None."""
  m = re.fullmatch(r"([va])\[(\d+):(\d+)\]", tok)
  if m:
    return m.group(1), set(range(int(m.group(2)), int(m.group(3)) + 1))
  m = re.fullmatch(r"([va])(\d+)", tok)
  if m:
    return m.group(1), {int(m.group(2))}
  return None


def _operands(line):
  parts = line.split(None, 1)
  if len(parts) < 2:
    return []
  return [t.strip() for t in parts[1].split(";")[0].split(",")]


def _wait_states(line):
  m = re.match(r"s_nop\s+(\d+)", line)
  return int(m.group(1)) + 1 if m else 1


def test_inline_asm_mfma_hazards(wide_kernels):
  for name, code in wide_kernels.items():
    mfma = [i for i, l in enumerate(code) if l.startswith("v_mfma")]
    assert mfma, name
    acc = set()
    for i in mfma:
      ops = _operands(code[i])
      kind, regs = _regs(ops[0])
      assert kind == "a", f"{name}: MFMA accumulator not in AGPRs: {code[i]}"
      acc |= regs
      assert ops[3] in (ops[0], "0"), f"{name}: accumulator not tied: {code[i]}"
    # 1. an MFMA never reads an accumulator that a VALU instruction wrote: after a
    # VALU write of such an AGPR (the compiler parks VGPRs in accumulators that are
    # dead between the epilogue and the next tile) the next MFMA on it must be one
    # with a zero C operand, which only writes it
    for i, l in enumerate(code):
      if l.startswith(("v_accvgpr_write", "v_accvgpr_mov")):
        kind, regs = _regs(_operands(l)[0])
        if not (kind == "a" and regs & acc):
          continue
        nxt = next((k for k in mfma if k > i and _regs(_operands(code[k])[0])[1] & regs), None)
        assert nxt is None or _operands(code[nxt])[3] == "0", \
            f"{name}: {code[nxt]!r} reads an accumulator written by {l!r}"
    # 2. no VALU write of an A/B operand in the 4 instructions before the MFMA
    for i in mfma:
      ops = _operands(code[i])
      src = _regs(ops[1])[1] | _regs(ops[2])[1]
      for l in code[max(0, i - 4):i]:
        if l.startswith("v_") and not l.startswith("v_mfma"):
          d = _regs(_operands(l)[0])
          assert not (d and d[0] == "v" and d[1] & src), \
              f"{name}: VALU write {l!r} right before {code[i]!r}"
    # 3. wait states between the last MFMA and an accumulator read
    for i, l in enumerate(code):
      if l.startswith("v_accvgpr_read"):
        ops = _operands(l)
        kind, regs = _regs(ops[1])
        if not (kind == "a" and regs & acc):
          continue
        states, j = 0, i - 1
        while j >= 0 and states < 18 and not code[j].startswith("v_mfma"):
          states += _wait_states(code[j])
          j -= 1
        assert states >= 18 or j < 0, f"{name}: accumulator read {states} wait states after an MFMA"
    # 5. no register spills
    for l in code:
      assert not l.startswith("scratch_"), f"{name}: register spill {l!r}"
    # 4. no complete drain of the DMA stream inside the K loop
    for l in code[mfma[0]:mfma[-1]]:
      assert not (l.startswith("s_waitcnt") and "vmcnt(0)" in l), \
          f"{name}: {l!r} between MFMAs"


def test_output_stores_are_unconditional(wide_kernels):
  """Rule 6. The epilogue exists twice (with and without GELU, chosen by a scalar
  branch); for 16-bit outputs the stores of the last row of blocks follow the join."""
  counted = 0
  for name, code in wide_kernels.items():
    m = re.search(r"gemm_fp8_wideINS0_7CfgWideILi(\d+)ELi(\d+)ELi\d+ELi\d+ELb[01]EEELi(\d)ELb[01]ELb([01])E", name)
    if not m:
      continue
    bm, bn, out = int(m.group(1)), int(m.group(2)), int(m.group(3))
    # (the measurement instance leaves its time stamps with two more 16-byte stores)
    stamp_stores = 2 if m.group(4) == "1" else 0
    per_row = bn // 64 * (2 if out == 2 else 1)
    expect = bm // 32 * per_row
    shared = 0 if out == 2 else per_row
    assert not any(l.startswith("global_store") for l in code), name
    code = labeled[name]
    stores = [i for i, l in enumerate(code) if l.startswith("buffer_store_dwordx4")]
    assert len(stores) == 2 * (expect - shared) + shared + stamp_stores, \
        f"{name}: {len(stores)} output stores, expected 2 * {expect - shared} + {shared} + {stamp_stores}"
    # no store under a lane mask (a store that may be skipped) or in a loop over the
    # values of a descriptor: none lies between an exec-conditional branch and its target
    label_at = {m.group(1): i for i, l in enumerate(code) for m in [re.match(r"(\.\w+):", l)] if m}
    for i, l in enumerate(code):
      if l.startswith(("s_cbranch_execz", "s_cbranch_execnz")):
        lo, hi = sorted((i, label_at[l.split()[-1]]))
        if any(c.startswith("v_mfma") for c in code[lo:hi]):
          continue  # the loop over the tiles
        assert not any(lo <= k <= hi for k in stores), f"{name}: output store under {l!r}"
    counted += 1
  if any("gemm_fp8_wide" in n for n in wide_kernels):
    assert counted >= 3


def test_staged_epilogue_operands_are_waited_for(wide_kernels):
  """Rule 7. Between the end of a K loop (the pair of s_nop 15 in front of the epilogue)
  and the first LDS read behind it, the instances whose DMA stream runs 4 or 5 steps ahead
  wait with vmcnt(2 ND): the staging DMA is older than the 2 ND panel instructions of the
  last two steps, nothing else may be in flight in front of the read."""
  checked = 0
  for name, code in wide_kernels.items():
    m = re.search(r"gemm_fp8_wideINS0_7CfgWideILi(\d+)ELi(\d+)ELi\d+ELi(\d+)ELb[01]EEELi(\d)E", name)
    if not m or int(m.group(3)) <= 3:
      continue
    bm, bn = int(m.group(1)), int(m.group(2))
    nd = bm // 32 + bn // 32
    ends = [i for i in range(len(code) - 1)
            if code[i].startswith("s_nop 15") and code[i + 1].startswith("s_nop 15")]
    assert ends, name
    for e in ends:
      first_read = next(i for i in range(e, len(code)) if code[i].startswith("ds_read"))
      waits = [re.search(r"vmcnt\((\d+)\)", l) for l in code[e:first_read] if l.startswith("s_waitcnt")]
      counts = [int(w.group(1)) for w in waits if w]
      assert counts and min(counts) <= 2 * nd, \
          f"{name}: LDS read {code[first_read]!r} after the K loop without a vmcnt wait <= {2 * nd}"
    checked += 1
  if any("gemm_fp8_wide" in n for n in wide_kernels):
    assert checked >= 2
