"""ctypes binding of libcdit_hip.so (C ABI declared in include/cdit_hip.h).

The library is loaded lazily, on the first call that needs it, and only after
`torch` has been imported so that it binds to the HIP runtime PyTorch already
loaded (same SONAME). There is no fallback: if the library is missing or the
device is not a gfx950 every entry point raises.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch  # noqa: F401  (must be imported before the library is loaded)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libcdit_hip.so")
ABI_VERSION = 1

SCALE_MODE_IDS = {"bf16div": 0, "fp32div": 1}
QUANT_GEMM_FOLLOWS = 0x100  # cache hint, OR-ed into the scale mode of the per-row quantizer
EPI_NONE = 0
EPI_GELU_TANH = 1
DT_F16, DT_BF16, DT_F32 = 0, 1, 2
MAX_GROUP = 8  # members of cdit_fp8_gemm_rowwise_grouped / _batched
MAX_ACTS = 4  # activations of cdit_fp8_gemm_rowwise_batched
STATIC_WS_CODE_BYTES, STATIC_WS_ROWS = 96 << 20, 65536  # cdit_fp8_linear_w8a8_static

#: every symbol include/cdit_hip.h declares
EXPORTS = (
    "cdit_abi_version",
    "cdit_last_error",
    "cdit_device_arch",
    "cdit_fp8_quant_rowwise",
    "cdit_fp8_quant_rowwise_batched",
    "cdit_fp8_quant_rowwise_cat2",
    "cdit_fp8_quant_tensorwise",
    "cdit_fp8_ln_modulate_quant",
    "cdit_fp8_gemm_rowwise",
    "cdit_fp8_gemm_rowwise_grouped",
    "cdit_fp8_gemm_rowwise_batched",
    "cdit_w8a16_gemm",
    "cdit_w8a16_gemm_batched",
    "cdit_fp8_linear_w8a8",
    "cdit_fp8_linear_w8a8_static",
    "cdit_fp8_comm_per_token_quant",
    "cdit_fp8_comm_per_token_dequant",
    "cdit_fp8_comm_qkv_permute_quant",
    "cdit_fp8_comm_qkv_permute_dequant",
    "cdit_debug_set_gemm_variant",
    "cdit_debug_set_quant_hints",
    "cdit_debug_mfma_only",
    "cdit_debug_gemm_stamps",
    "cdit_stream_capture_id",
)

_lib = None
_lock = threading.Lock()


class CditNativeError(RuntimeError):
  """A libcdit_hip.so call returned a non-zero status."""


def _bind(L: ctypes.CDLL) -> None:
  i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
  L.cdit_abi_version.restype = ci
  L.cdit_abi_version.argtypes = []
  L.cdit_last_error.restype = ctypes.c_char_p
  L.cdit_last_error.argtypes = []
  L.cdit_device_arch.restype = ci
  L.cdit_device_arch.argtypes = [ctypes.c_char_p, ci]
  L.cdit_stream_capture_id.restype = ci
  L.cdit_stream_capture_id.argtypes = [vp, ctypes.POINTER(ctypes.c_uint64)]
  L.cdit_debug_set_gemm_variant.restype = ci
  L.cdit_debug_set_gemm_variant.argtypes = [ci]
  L.cdit_debug_set_quant_hints.restype = ci
  L.cdit_debug_set_quant_hints.argtypes = [ci]
  L.cdit_debug_mfma_only.restype = ci
  L.cdit_debug_mfma_only.argtypes = [vp, ci, ci, ci, ctypes.POINTER(ctypes.c_double), vp]
  L.cdit_debug_gemm_stamps.restype = ci
  L.cdit_debug_gemm_stamps.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, vp,
                                       ctypes.POINTER(ci), vp]
  L.cdit_fp8_quant_rowwise.restype = ci
  L.cdit_fp8_quant_rowwise.argtypes = [vp, i64, i64, i64, vp, i64, vp, ci, vp]
  L.cdit_fp8_quant_rowwise_cat2.restype = ci
  L.cdit_fp8_quant_rowwise_cat2.argtypes = [vp, i64, i64, vp, i64, i64, i64, vp, i64, vp, ci, vp]
  L.cdit_fp8_quant_rowwise_batched.restype = ci
  L.cdit_fp8_quant_rowwise_batched.argtypes = [ci, vp, vp, i64, vp, vp, vp, vp, ci, vp]
  L.cdit_fp8_ln_modulate_quant.restype = ci
  L.cdit_fp8_ln_modulate_quant.argtypes = [vp, i64, i64, i64, vp, vp, i64, i64, ctypes.c_float, vp,
                                           i64, vp, i64, vp, ci, vp]
  L.cdit_fp8_quant_tensorwise.restype = ci
  L.cdit_fp8_quant_tensorwise.argtypes = [vp, i64, i64, i64, vp, i64, vp, vp, ci, vp]
  L.cdit_fp8_gemm_rowwise.restype = ci
  L.cdit_fp8_gemm_rowwise.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci,
                                      vp]
  L.cdit_fp8_gemm_rowwise_grouped.restype = ci
  L.cdit_fp8_gemm_rowwise_grouped.argtypes = [vp, vp, i64, i64, i64, ci, ctypes.POINTER(vp),
                                              ctypes.POINTER(vp), ctypes.POINTER(vp),
                                              ctypes.POINTER(vp), ctypes.POINTER(i64), i64,
                                              ctypes.POINTER(i64), ctypes.POINTER(ci), vp]
  L.cdit_fp8_gemm_rowwise_batched.restype = ci
  L.cdit_fp8_gemm_rowwise_batched.argtypes = [ci, ctypes.POINTER(vp), ctypes.POINTER(vp),
                                              ctypes.POINTER(i64), i64, i64, ctypes.POINTER(ci),
                                              ctypes.POINTER(vp), ctypes.POINTER(vp),
                                              ctypes.POINTER(vp), ctypes.POINTER(vp),
                                              ctypes.POINTER(i64), i64, ctypes.POINTER(i64),
                                              ctypes.POINTER(ci), vp]
  L.cdit_fp8_linear_w8a8.restype = ci
  L.cdit_fp8_linear_w8a8.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci,
                                     ci, vp]
  L.cdit_fp8_linear_w8a8_static.restype = ci
  L.cdit_fp8_linear_w8a8_static.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci,
                                            ci, vp]
  L.cdit_fp8_comm_per_token_quant.restype = ci
  L.cdit_fp8_comm_per_token_quant.argtypes = [vp, i64, i64, vp, vp]
  L.cdit_fp8_comm_per_token_dequant.restype = ci
  L.cdit_fp8_comm_per_token_dequant.argtypes = [vp, i64, i64, vp, vp]
  L.cdit_fp8_comm_qkv_permute_quant.restype = ci
  L.cdit_fp8_comm_qkv_permute_quant.argtypes = [vp, i64, i64, i64, i64, i64, i64, i64, i64, vp, vp]
  L.cdit_fp8_comm_qkv_permute_dequant.restype = ci
  L.cdit_fp8_comm_qkv_permute_dequant.argtypes = [vp, i64, i64, i64, i64, i64, i64, i64, vp, vp]
  L.cdit_w8a16_gemm_batched.restype = ci
  L.cdit_w8a16_gemm_batched.argtypes = [ci, vp, vp, i64, i64, vp, vp, vp, vp, vp, vp, i64, vp, vp, vp]
  L.cdit_w8a16_gemm.restype = ci
  L.cdit_w8a16_gemm.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, ci, ci, vp]


def load(path: str | None = None) -> ctypes.CDLL:
  """Loads (once) and returns the library; raises if it is not built."""
  global _lib
  if _lib is not None:
    return _lib
  with _lock:
    if _lib is None:
      p = path or os.environ.get("CDIT_HIP_LIB", LIB_PATH)
      if not os.path.exists(p):
        raise CditNativeError(
            f"{p} not found: build it with `python -m cache_dit_amd.csrc.build` "
            "(needs hipcc). There is no fallback path.")
      L = ctypes.CDLL(p)
      for name in EXPORTS:
        if not hasattr(L, name):
          raise CditNativeError(f"{p} does not export {name}")
      _bind(L)
      if L.cdit_abi_version() != ABI_VERSION:
        raise CditNativeError(f"{p}: ABI version {L.cdit_abi_version()} != {ABI_VERSION}; rebuild")
      _lib = L
  return _lib


def is_built() -> bool:
  return os.path.exists(os.environ.get("CDIT_HIP_LIB", LIB_PATH))


def last_error() -> str:
  return load().cdit_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
  if rc != 0:
    raise CditNativeError(f"libcdit_hip status {rc}: {last_error()}")


def device_arch() -> str:
  """gcnArchName of the current device; raises unless it is a gfx950."""
  buf = ctypes.create_string_buffer(256)
  check(load().cdit_device_arch(buf, 256))
  return buf.value.decode()


def set_gemm_variant(variant: int) -> int:
  return load().cdit_debug_set_gemm_variant(int(variant))


def stream_capture_id(stream: int) -> int:
  """Id of the graph capture `stream` is recording into, 0 when it is not capturing."""
  out = ctypes.c_uint64(0)
  check(load().cdit_stream_capture_id(stream, ctypes.byref(out)))
  return int(out.value)
