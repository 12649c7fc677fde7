"""The quantizer kernel divides with a two-term reciprocal per row plus a multiply and an
FMA per element. tests/native/divcheck.c proves on the CPU, exhaustively over every bf16
amax and every bf16 x with |x| <= amax in both scale modes, that this yields the
same e4m3 code as the IEEE division of the oracle."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def test_divcheck_exhaustive(tmp_path):
  exe = str(tmp_path / "divcheck")
  src = [os.path.join(HERE, "native", "divcheck.c"), os.path.join(ROOT, "oracle", "cdit_oracle.c")]
  cc = subprocess.run(["gcc", "-O2", "-fopenmp", "-mfma", "-ffp-contract=off", "-o", exe, *src,
                       "-lm"], capture_output=True, text=True)
  if cc.returncode != 0 and "mfma" in cc.stderr:
    pytest.skip("host compiler lacks -mfma")
  assert cc.returncode == 0, cc.stderr
  env = dict(os.environ, OMP_NUM_THREADS=str(min(8, os.cpu_count() or 1)))
  r = subprocess.run([exe, "1"], capture_output=True, text=True, env=env, timeout=600)
  assert r.returncode == 0, r.stdout + r.stderr
  fields = dict(kv.split("=") for kv in r.stdout.split())
  assert int(fields["checked"]) > 1_500_000_000 and int(fields["code_mismatch"]) == 0


def test_kernel_source_uses_the_checked_window():
  """The exponent window in the kernel and in the checker must be the same."""
  k = open(os.path.join(ROOT, "cache_dit_amd", "csrc", "quant_device.h")).read()
  c = open(os.path.join(HERE, "native", "divcheck.c")).read()
  assert "e >= 27u && e <= 227u" in k and "e >= 27 && e <= 227" in c
