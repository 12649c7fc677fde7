"""The wide FP8 GEMM kernel issues its MFMAs through inline assembly (the
accumulators are tied to AGPR tuples), so the compiler's hazard recognizer does
not see them. This test compiles gemm_fp8.hip to gfx950 assembly (no GPU needed)
and checks, in the code the compiler produced for every instance of that kernel,
the three situations in which the hardware needs software wait states:

  1. no VALU instruction (v_accvgpr_write / v_accvgpr_mov) writes an AGPR that an
     MFMA uses as accumulator: accumulators are only ever written by MFMAs;
  2. no VALU instruction writes a VGPR within the 8 instructions before an MFMA
     that reads it as A or B operand (operands come from LDS reads, which
     s_waitcnt covers);
  3. at least 18 wait states lie between an MFMA and the first v_accvgpr_read of
     an accumulator (the epilogue).
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "cache_dit_amd", "csrc", "gemm_fp8.hip")


def _hipcc():
  for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
    if cand and os.path.exists(cand):
      return cand
  return None


@pytest.fixture(scope="module")
def wide_kernels(tmp_path_factory):
  hipcc = _hipcc()
  if hipcc is None:
    pytest.skip("hipcc not found")
  out = tmp_path_factory.mktemp("isa") / "gemm_fp8.s"
  from cache_dit_amd.csrc import build
  cmd = [hipcc, *build.DEVICE_FLAGS, "-I", os.path.join(ROOT, "include"), "-I",
         os.path.dirname(SRC), "--cuda-device-only", "-S", SRC, "-o", str(out)]
  r = subprocess.run(cmd, capture_output=True, text=True)
  assert r.returncode == 0, r.stderr[-2000:]
  text = out.read_text()
  kernels = {}
  for m in re.finditer(r"^(_ZN\S*gemm_fp8_wide\S*):[^\n]*\n(.*?)s_endpgm", text, re.S | re.M):
    body = [l.strip() for l in m.group(2).split("\n")]
    kernels[m.group(1)] = [l for l in body if l and not l.startswith(";") and not l.startswith(".")]
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
    # 1. accumulators written by MFMAs only
    for l in code:
      if l.startswith(("v_accvgpr_write", "v_accvgpr_mov")):
        kind, regs = _regs(_operands(l)[0])
        assert not (kind == "a" and regs & acc), f"{name}: VALU write of an accumulator: {l}"
    # 2. no VALU write of an A/B operand shortly before the MFMA that reads it
    for i in mfma:
      ops = _operands(code[i])
      src = _regs(ops[1])[1] | _regs(ops[2])[1]
      for l in code[max(0, i - 8):i]:
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
