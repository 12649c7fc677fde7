"""ctypes binding of oracle/libcdit_oracle.so (the plain-C restatement).
TEST INFRASTRUCTURE ONLY. Build with `make -C oracle`."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcdit_oracle.so")
_lib = None


def build(force: bool = False) -> str:
  src = os.path.join(_HERE, "cdit_oracle.c")
  if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
    subprocess.run(["make", "-C", _HERE, "-B", "libcdit_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
  return _LIB_PATH


def lib() -> ctypes.CDLL:
  global _lib
  if _lib is None:
    if not os.path.exists(_LIB_PATH):
      build()
    L = ctypes.CDLL(_LIB_PATH)
    L.oracle_e4m3_encode.restype = ctypes.c_uint8
    L.oracle_e4m3_encode.argtypes = [ctypes.c_float]
    L.oracle_e4m3_decode.restype = ctypes.c_float
    L.oracle_e4m3_decode.argtypes = [ctypes.c_uint8]
    L.oracle_row_scale.restype = ctypes.c_float
    L.oracle_row_scale.argtypes = [ctypes.c_uint16, ctypes.c_int]
    L.oracle_gelu_tanh.restype = ctypes.c_float
    L.oracle_gelu_tanh.argtypes = [ctypes.c_float]
    i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
    L.oracle_quant_rowwise.restype = None
    L.oracle_quant_rowwise.argtypes = [vp, i64, i64, i64, vp, i64, vp, ci]
    L.oracle_quant_tensorwise.restype = None
    L.oracle_quant_tensorwise.argtypes = [vp, i64, i64, i64, vp, i64, vp, ci]
    L.oracle_gemm_rowwise.restype = None
    L.oracle_gemm_rowwise.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci]
    L.oracle_w8a16.restype = None
    L.oracle_w8a16.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci]
    _lib = L
  return _lib


def _ptr(a):
  return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def quant_rowwise(x_bits: np.ndarray, mode: int):
  """x_bits uint16 [M,K] (bf16 bit patterns) -> (codes uint8 [M,K], scale f32 [M])."""
  x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
  M, K = x_bits.shape
  q = np.empty((M, K), dtype=np.uint8)
  s = np.empty((M,), dtype=np.float32)
  lib().oracle_quant_rowwise(_ptr(x_bits), M, K, K, _ptr(q), K, _ptr(s), mode)
  return q, s


def quant_tensorwise(x_bits: np.ndarray, mode: int):
  """Per-tensor variant: (codes uint8 [M,K], scale f32 [M], all entries equal)."""
  x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
  M, K = x_bits.shape
  q = np.empty((M, K), dtype=np.uint8)
  s = np.empty((M,), dtype=np.float32)
  lib().oracle_quant_tensorwise(_ptr(x_bits), M, K, K, _ptr(q), K, _ptr(s), mode)
  return q, s


def gemm_rowwise(a, a_scale, b, b_scale, bias_bits=None, gelu: int = 0):
  a = np.ascontiguousarray(a, dtype=np.uint8)
  b = np.ascontiguousarray(b, dtype=np.uint8)
  a_scale = np.ascontiguousarray(a_scale, dtype=np.float32).reshape(-1)
  b_scale = np.ascontiguousarray(b_scale, dtype=np.float32).reshape(-1)
  if bias_bits is not None:
    bias_bits = np.ascontiguousarray(bias_bits, dtype=np.uint16)
  M, K = a.shape
  N = b.shape[0]
  out = np.empty((M, N), dtype=np.uint16)
  lib().oracle_gemm_rowwise(_ptr(a), _ptr(a_scale), _ptr(b), _ptr(b_scale), _ptr(bias_bits),
                            _ptr(out), M, N, K, K, K, N, gelu)
  return out


def w8a16(x_bits, b, b_scale, bias_bits=None, gelu: int = 0, dequant_bf16: bool = True):
  x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
  b = np.ascontiguousarray(b, dtype=np.uint8)
  b_scale = np.ascontiguousarray(b_scale, dtype=np.float32).reshape(-1)
  if bias_bits is not None:
    bias_bits = np.ascontiguousarray(bias_bits, dtype=np.uint16)
  M, K = x_bits.shape
  N = b.shape[0]
  out = np.empty((M, N), dtype=np.uint16)
  lib().oracle_w8a16(_ptr(x_bits), _ptr(b), _ptr(b_scale), _ptr(bias_bits), _ptr(out), M, N, K, K,
                     K, N, gelu, int(dequant_bf16))
  return out


def e4m3_encode_table_check(values: np.ndarray) -> np.ndarray:
  L = lib()
  return np.array([L.oracle_e4m3_encode(float(v)) for v in values], dtype=np.uint8)
