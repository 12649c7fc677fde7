"""The C ABI library loads and exports every symbol include/cdit_hip.h declares;
argument validation that needs no GPU; fake (meta) implementations of the ops."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
  text = open(os.path.join(ROOT, "include", "cdit_hip.h")).read()
  text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
  return sorted(set(re.findall(r"\b(cdit_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
  from cache_dit_amd import _native
  if not _native.is_built():
    pytest.skip("libcdit_hip.so not built (run __graft_entry__.build())")
  names = _declared()
  assert sorted(_native.EXPORTS) == names
  L = ctypes.CDLL(_native.LIB_PATH)
  for n in names:
    assert hasattr(L, n), n
  assert _native.load().cdit_abi_version() == _native.ABI_VERSION == 1


def test_argument_validation_without_gpu():
  from cache_dit_amd import _native
  if not _native.is_built():
    pytest.skip("libcdit_hip.so not built")
  L = _native.load()
  assert L.cdit_fp8_quant_rowwise(None, -1, 8, 8, None, 8, None, 0, None) == 1
  assert b"bad shape" in L.cdit_last_error()
  assert L.cdit_fp8_quant_rowwise(None, 4, 8, 8, None, 8, None, 5, None) == 1
  assert b"scale_mode" in L.cdit_last_error()
  assert L.cdit_fp8_quant_rowwise(None, 0, 8, 8, None, 8, None, 0, None) == 0  # empty: no-op
  one = ctypes.c_void_p(16)
  assert L.cdit_fp8_gemm_rowwise(one, one, one, one, None, one, 4, 4, 24, 24, 24, 4, 0, 1, None) == 1
  assert b"multiple of 16" in L.cdit_last_error()
  assert L.cdit_fp8_gemm_rowwise(one, one, one, one, None, one, 4, 4, 32, 32, 32, 4, 0, 3, None) == 1
  assert b"out_dtype_id" in L.cdit_last_error()
  # an fp32 output takes no bias (the reference adds it after the matmul)
  assert L.cdit_fp8_gemm_rowwise(one, one, one, one, one, one, 4, 4, 32, 32, 32, 4, 0, 2, None) == 1
  assert b"no bias" in L.cdit_last_error()
  # the weight-only GEMM builds bf16 only
  assert L.cdit_w8a16_gemm(one, one, one, None, one, 4, 4, 32, 32, 32, 4, 0, 0, None) == 1
  assert b"not built" in L.cdit_last_error()
  assert L.cdit_fp8_gemm_rowwise(one, one, one, one, None, one, 4, 4, 32, 32, 32, 4, 8, 1, None) == 1
  assert L.cdit_fp8_gemm_rowwise(one, one, one, one, None, one, 4, 4, 32, 16, 32, 4, 0, 1, None) == 1
  assert b"leading dimension" in L.cdit_last_error()
  assert L.cdit_w8a16_gemm(one, one, None, None, one, 4, 4, 32, 32, 32, 4, 0, 1, None) == 1
  assert b"null pointer" in L.cdit_last_error()
  assert L.cdit_w8a16_gemm(one, one, one, None, one, 0, 4, 32, 32, 32, 4, 0, 1, None) == 0
  assert L.cdit_debug_set_gemm_variant(3) == -1 and L.cdit_debug_set_gemm_variant(-1) == 3


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
  from cache_dit_amd import _native
  monkeypatch.setattr(_native, "_lib", None)
  monkeypatch.setenv("CDIT_HIP_LIB", str(tmp_path / "nope.so"))
  with pytest.raises(_native.CditNativeError, match="no fallback"):
    _native.load()


def test_fake_impls_shapes_and_dtypes():
  import cache_dit_amd.ops  # noqa: F401  (registers torch.ops.cdit)
  from torch._subclasses.fake_tensor import FakeTensorMode
  FP8 = torch.float8_e4m3fn
  with FakeTensorMode():
    x = torch.empty(2, 77, 3072, dtype=torch.bfloat16, device="cuda")
    q, s = torch.ops.cdit.fp8_rowwise_quant(x, 0)
    assert q.shape == (2, 77, 3072) and q.dtype == FP8 and q.device.type == "cuda"
    assert s.shape == (2, 77, 1) and s.dtype == torch.float32
    a = torch.empty(154, 3072, dtype=FP8, device="cuda")
    b = torch.empty(12288, 3072, dtype=FP8, device="cuda").t()
    for dt_id, dt in ((0, torch.float16), (1, torch.bfloat16), (2, torch.float32)):
      y = torch.ops.cdit.float8_inference_scaled_mm(a, s.reshape(-1, 1), b,
                                                    torch.empty(1, 12288, device="cuda"), None,
                                                    dt_id, True)
      assert y.shape == (154, 12288) and y.dtype == dt
    y = torch.ops.cdit.w8a16_mm(x, b, torch.empty(12288, device="cuda"), None, 1, 1)
    assert y.shape == (2, 77, 12288) and y.dtype == torch.bfloat16
    w = torch.empty(12288, 3072, dtype=FP8, device="cuda")
    y = torch.ops.cdit.linear_w8a8(x, w, torch.empty(12288, 1, device="cuda"), None)
    assert y.shape == (2, 77, 12288) and y.dtype == torch.bfloat16 and y.device.type == "cuda"
    ys = torch.ops.cdit.linear_w8a8_batch(
        [x, torch.empty(5, 3072, dtype=torch.bfloat16, device="cuda")], [w, w, w],
        [torch.empty(12288, device="cuda")] * 3, [None, None, None], [2, 1], [0, 1, 0])
    assert [tuple(y.shape) for y in ys] == [(2, 77, 12288), (2, 77, 12288), (5, 12288)]
    ys = torch.ops.cdit.w8a16_batch([x], [w, w], [torch.empty(12288, device="cuda")] * 2, [None, None],
                                    [2], [0, 0])
    assert [tuple(y.shape) for y in ys] == [(2, 77, 12288)] * 2 and ys[0].dtype == torch.bfloat16
    w2 = torch.empty(3072, 3072 + 12288, dtype=FP8, device="cuda")
    y = torch.ops.cdit.linear_w8a8_cat2(x, torch.empty(2, 77, 12288, dtype=torch.bfloat16, device="cuda"),
                                        w2, torch.empty(3072, 1, device="cuda"), None)
    assert y.shape == (2, 77, 3072) and y.dtype == torch.bfloat16 and y.device.type == "cuda"


def _meta_quantized_linear(cls_name, in_f, out_f):
  """A quantized Linear as convert_linear_ leaves it, built without a GPU (fake
  tensors stand in for the codes)."""
  from cache_dit_amd import _native, nn as cnn
  lin = torch.nn.Linear(in_f, out_f, dtype=torch.bfloat16, device="cuda")
  lin.weight = torch.nn.Parameter(torch.empty(out_f, in_f, dtype=torch.float8_e4m3fn,
                                              device="cuda"), requires_grad=False)
  lin.register_buffer("weight_scale", torch.empty(out_f, 1, device="cuda"))
  lin.bias.requires_grad_(False)
  lin.epilogue, lin.scale_mode, lin._scale_mode_id = _native.EPI_NONE, "bf16div", 0
  lin.quant_type = "test"
  lin.__class__ = getattr(cnn, cls_name)
  return lin


@pytest.mark.parametrize("cls_name", ["Fp8DynamicLinear", "Fp8DynamicLinearPerTensor",
                                      "Fp8WeightOnlyLinear"])
def test_quantized_linear_forward_traces_to_one_opaque_op(cls_name):
  """The module forward is one torch.ops.cdit call: under FakeTensorMode (what Dynamo
  and Inductor trace with) it needs no data pointer, no ctypes call and no library, and
  make_fx records exactly one cdit node. Shapes of the reference's opaque-op test
  (tests/kernels/test_opaque_scaled_mm.py:46-94): W[32,64], x[4,64]."""
  import cache_dit_amd.ops  # noqa: F401
  from torch._subclasses.fake_tensor import FakeTensorMode
  from torch.fx.experimental.proxy_tensor import make_fx
  with FakeTensorMode(allow_non_fake_inputs=False) as mode:
    lin = _meta_quantized_linear(cls_name, 64, 32)
    x = torch.empty(4, 64, dtype=torch.bfloat16, device="cuda")
    y = lin(x)
    assert y.shape == (4, 32) and y.dtype == torch.bfloat16
    y3 = lin(torch.empty(2, 5, 64, dtype=torch.bfloat16, device="cuda"))
    assert y3.shape == (2, 5, 32)
    gm = make_fx(lambda t: lin(t), tracing_mode="fake")(x)
  targets = [str(n.target) for n in gm.graph.nodes if n.op == "call_function"]
  cdit = [t for t in targets if t.startswith("cdit.")]
  assert len(cdit) == 1, targets
  assert cdit[0] == ("cdit.w8a16_mm.default" if cls_name == "Fp8WeightOnlyLinear" else
                     "cdit.linear_w8a8.default")


def test_dtype_id_codec():
  from cache_dit_amd import ops
  assert [ops.encode_output_dtype(d) for d in (torch.float16, torch.bfloat16, torch.float32)] == [0, 1, 2]
  assert ops.decode_output_dtype(1) is torch.bfloat16
  with pytest.raises(ValueError, match="output dtype"):
    ops.encode_output_dtype(torch.float64)
  with pytest.raises(ValueError, match="dtype id"):
    ops.decode_output_dtype(9)
