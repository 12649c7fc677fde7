"""Builds libcdit_hip.so (the HIP kernels + C ABI) for gfx950 with hipcc.

Usage: python -m cache_dit_amd.csrc.build   (or call build())
The library is written to cache_dit_amd/lib/libcdit_hip.so, in-tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB_DIR = os.path.join(os.path.dirname(HERE), "lib")
LIB_PATH = os.path.join(LIB_DIR, "libcdit_hip.so")
SOURCES = ["capi.hip", "quant_rowwise.hip", "comm_quant.hip", "gemm_fp8.hip", "gemm_w8a16.hip"]

# -ffp-contract=off: the quantizer's arithmetic is specified operation by
# operation (explicit FMAs only). The packed-fp32 feature is switched off on
# purpose for every device compile.
DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _hipcc() -> str:
  for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
    if cand and os.path.exists(cand):
      return cand
  raise RuntimeError("hipcc not found (set HIPCC or add /opt/rocm/bin to PATH)")


def build(verbose: bool = False) -> str:
  hipcc = _hipcc()
  os.makedirs(LIB_DIR, exist_ok=True)
  obj_dir = os.path.join(LIB_DIR, "obj")
  os.makedirs(obj_dir, exist_ok=True)
  inc = ["-I" + os.path.join(ROOT, "include"), "-I" + HERE]

  def compile_one(src: str) -> str:
    obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
    cmd = [hipcc, *DEVICE_FLAGS, *inc, "-c", os.path.join(HERE, src), "-o", obj]
    if verbose:
      print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
      raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    return obj

  with ThreadPoolExecutor(max_workers=4) as ex:
    objs = list(ex.map(compile_one, SOURCES))
  tmp = LIB_PATH + ".tmp"
  cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
  r = subprocess.run(cmd, capture_output=True, text=True)
  if r.returncode != 0:
    raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
  os.replace(tmp, LIB_PATH)
  return LIB_PATH


if __name__ == "__main__":
  print(build(verbose="-v" in sys.argv))
