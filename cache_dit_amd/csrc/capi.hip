// extern "C" layer of libcdit_hip.so: argument validation, device check,
// error reporting. Declarations and their reference citations: include/cdit_hip.h.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "cdit_internal.h"

namespace cdit {

namespace {
thread_local char g_err[512] = "";
int g_gemm_variant = -1;

// gfx950 check, cached per device ordinal (the answer cannot change).
int check_arch() {
  static int cached[64];  // 0 unknown, 1 ok, 2 wrong arch
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("hipGetDevice: %s", hipGetErrorString(e));
    return CDIT_EHIP;
  }
  if (dev >= 0 && dev < 64 && cached[dev] == 1) return CDIT_OK;
  hipDeviceProp_t p;
  e = hipGetDeviceProperties(&p, dev);
  if (e != hipSuccess) {
    set_error("hipGetDeviceProperties: %s", hipGetErrorString(e));
    return CDIT_EHIP;
  }
  const bool ok = strncmp(p.gcnArchName, "gfx950", 6) == 0;
  if (dev >= 0 && dev < 64) cached[dev] = ok ? 1 : 2;
  if (!ok) {
    set_error("device %d is %s; libcdit_hip.so is built for gfx950 only (its FP8 is OCP e4m3fn, "
              "older CDNA parts use e4m3fnuz)", dev, p.gcnArchName);
    return CDIT_EARCH;
  }
  return CDIT_OK;
}

int after_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return CDIT_EHIP;
  }
  return CDIT_OK;
}

int check_gemm(const char* fn, const void* a, const void* b, const float* b_scale,
               const void* bias, const void* out, int64_t M, int64_t N, int64_t K, int64_t lda,
               int64_t ldb, int64_t ldo, int epilogue, int out_dtype_id, bool bf16_only) {
  if (M < 0 || N < 0 || K < 0) {
    set_error("%s: negative dimension (M=%lld N=%lld K=%lld)", fn, (long long)M, (long long)N,
              (long long)K);
    return CDIT_EINVAL;
  }
  if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) {
    set_error("%s: dimension exceeds int32", fn);
    return CDIT_EINVAL;
  }
  if (out_dtype_id != CDIT_DT_F16 && out_dtype_id != CDIT_DT_BF16 && out_dtype_id != CDIT_DT_F32) {
    set_error("%s: unknown out_dtype_id %d (0 = fp16, 1 = bf16, 2 = fp32)", fn, out_dtype_id);
    return CDIT_EINVAL;
  }
  if (bf16_only && out_dtype_id != CDIT_DT_BF16) {
    set_error("%s: out_dtype_id %d not built (only 1 = bf16)", fn, out_dtype_id);
    return CDIT_EINVAL;
  }
  if (out_dtype_id == CDIT_DT_F32 && bias) {
    set_error("%s: an fp32 output takes no bias (add it afterwards, as the reference does around "
              "torch._scaled_mm)", fn);
    return CDIT_EINVAL;
  }
  if (epilogue & ~CDIT_EPI_GELU_TANH) {
    set_error("%s: unknown epilogue bits 0x%x", fn, epilogue);
    return CDIT_EINVAL;
  }
  if (K % 16 != 0) {
    set_error("%s: K=%lld is not a multiple of 16", fn, (long long)K);
    return CDIT_EINVAL;
  }
  if (lda < K || ldb < K || ldo < N) {
    set_error("%s: leading dimension smaller than the row (lda=%lld ldb=%lld ldo=%lld)", fn,
              (long long)lda, (long long)ldb, (long long)ldo);
    return CDIT_EINVAL;
  }
  if (M > 0 && N > 0 && (!out || !b_scale || (K > 0 && (!a || !b)))) {
    set_error("%s: null pointer argument", fn);
    return CDIT_EINVAL;
  }
  return CDIT_OK;
}

}  // namespace

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

}  // namespace cdit

using namespace cdit;

extern "C" {

int cdit_abi_version(void) { return CDIT_ABI_VERSION; }

const char* cdit_last_error(void) { return g_err; }

int cdit_device_arch(char* buf, int buf_len) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  hipDeviceProp_t p;
  if (e == hipSuccess) e = hipGetDeviceProperties(&p, dev);
  if (e != hipSuccess) {
    set_error("cdit_device_arch: %s", hipGetErrorString(e));
    return CDIT_EHIP;
  }
  if (buf && buf_len > 0) {
    strncpy(buf, p.gcnArchName, (size_t)buf_len - 1);
    buf[buf_len - 1] = '\0';
  }
  return check_arch();
}

int cdit_stream_capture_id(void* stream, uint64_t* id) {
  if (!id) {
    set_error("cdit_stream_capture_id: id is null");
    return CDIT_EINVAL;
  }
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long cid = 0;
  hipError_t e = hipStreamGetCaptureInfo(static_cast<hipStream_t>(stream), &status, &cid);
  if (e != hipSuccess) {
    set_error("hipStreamGetCaptureInfo: %s", hipGetErrorString(e));
    return CDIT_EHIP;
  }
  // ids start at 1 in the runtime; make sure an active capture never reads as "none"
  *id = status == hipStreamCaptureStatusActive ? (uint64_t)cid + 1 : 0;
  return CDIT_OK;
}

int cdit_debug_set_gemm_variant(int variant) {
  int prev = g_gemm_variant;
  g_gemm_variant = variant;
  return prev;
}

int cdit_debug_set_quant_hints(int hints) {
  int prev = cdit::g_quant_variant;
  cdit::g_quant_variant = hints >= 0 && hints <= 7 ? hints : -1;
  return prev;
}

int cdit_debug_mfma_only(void* out_f32, int blocks, int iters, int random_operands, double* flop,
                         void* stream) {
  const char* fn = "cdit_debug_mfma_only";
  if (!out_f32 || blocks < 1 || blocks > 65536 || iters < 1) {
    set_error("%s: out is null, or blocks=%d / iters=%d out of range", fn, blocks, iters);
    return CDIT_EINVAL;
  }
  int rc = check_arch();
  if (rc) return rc;
  rc = launch_mfma_only(static_cast<float*>(out_f32), blocks, iters, random_operands != 0, flop,
                        static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

int cdit_debug_gemm_stamps(const void* a_q, const float* a_scale, const void* b_q, const float* b_scale,
                           const void* bias, void* out, int64_t M, int64_t N, int64_t K, int64_t lda,
                           int64_t ldb, int64_t ldo, void* stamps_u64, int* workgroups, void* stream) {
  const char* fn = "cdit_debug_gemm_stamps";
  int rc = check_gemm(fn, a_q, b_q, b_scale, bias, out, M, N, K, lda, ldb, ldo, 0, CDIT_DT_BF16, false);
  if (rc) return rc;
  if (!a_scale || !stamps_u64 || M == 0 || N == 0) {
    set_error("%s: a_scale or stamps is null, or an empty problem", fn);
    return CDIT_EINVAL;
  }
  rc = check_arch();
  if (rc) return rc;
  GemmArgs g;
  g.a = a_q;
  g.a_scale = a_scale;
  g.b = static_cast<const uint8_t*>(b_q);
  g.b_scale = b_scale;
  g.bias = static_cast<const uint16_t*>(bias);
  g.out = static_cast<uint16_t*>(out);
  g.M = (int)M;
  g.N = (int)N;
  g.K = (int)K;
  g.lda = lda;
  g.ldb = ldb;
  g.ldo = ldo;
  g.epilogue = 0;
  g.out_dtype = CDIT_DT_BF16;
  rc = launch_gemm_fp8_stamps(g, static_cast<unsigned long long*>(stamps_u64), workgroups,
                              static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

// consumer_follows: the codes are read by a GEMM launched right behind (the fused
// Linear entry point): the quantizer then keeps its loads and stores cacheable.
static int quant_rowwise_impl(const char* fn, const void* x_bf16, int64_t M, int64_t K,
                             int64_t ld_x, void* q_e4m3, int64_t ld_q, float* scale,
                             int scale_mode, void* stream, bool consumer_follows) {
  if (scale_mode >= 0 && (scale_mode & CDIT_QUANT_GEMM_FOLLOWS)) {
    consumer_follows = true;
    scale_mode &= ~CDIT_QUANT_GEMM_FOLLOWS;
  }
  if (M < 0 || K < 0 || M > INT32_MAX || K > INT32_MAX) {
    set_error("%s: bad shape M=%lld K=%lld", fn, (long long)M, (long long)K);
    return CDIT_EINVAL;
  }
  if (scale_mode != CDIT_SCALE_BF16DIV && scale_mode != CDIT_SCALE_FP32DIV) {
    set_error("%s: unknown scale_mode %d", fn, scale_mode);
    return CDIT_EINVAL;
  }
  if (M == 0) return CDIT_OK;
  if (ld_x < K || ld_q < K) {
    set_error("%s: leading dimension smaller than K (ld_x=%lld ld_q=%lld K=%lld)", fn,
              (long long)ld_x, (long long)ld_q, (long long)K);
    return CDIT_EINVAL;
  }
  if (!scale || (K > 0 && (!x_bf16 || !q_e4m3))) {
    set_error("%s: null pointer argument", fn);
    return CDIT_EINVAL;
  }
  int rc = check_arch();
  if (rc) return rc;
  rc = launch_quant_rowwise(x_bf16, M, K, ld_x, q_e4m3, ld_q, scale, scale_mode,
                            consumer_follows, static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

int cdit_fp8_quant_rowwise(const void* x_bf16, int64_t M, int64_t K, int64_t ld_x, void* q_e4m3,
                           int64_t ld_q, float* scale, int scale_mode, void* stream) {
  return quant_rowwise_impl("cdit_fp8_quant_rowwise", x_bf16, M, K, ld_x, q_e4m3, ld_q, scale,
                           scale_mode, stream, false);
}

int cdit_fp8_quant_rowwise_cat2(const void* x1_bf16, int64_t K1, int64_t ld_x1,
                                const void* x2_bf16, int64_t K2, int64_t ld_x2, int64_t M,
                                void* q_e4m3, int64_t ld_q, float* scale, int scale_mode,
                                void* stream) {
  const char* fn = "cdit_fp8_quant_rowwise_cat2";
  const int mode = scale_mode >= 0 ? scale_mode & ~CDIT_QUANT_GEMM_FOLLOWS : scale_mode;
  if (M < 0 || K1 <= 0 || K2 <= 0 || M > INT32_MAX || K1 + K2 > INT32_MAX) {
    set_error("%s: bad shape M=%lld K1=%lld K2=%lld", fn, (long long)M, (long long)K1, (long long)K2);
    return CDIT_EINVAL;
  }
  if (mode != CDIT_SCALE_BF16DIV && mode != CDIT_SCALE_FP32DIV) {
    set_error("%s: unknown scale_mode %d", fn, scale_mode);
    return CDIT_EINVAL;
  }
  if (M == 0) return CDIT_OK;
  if (ld_x1 < K1 || ld_x2 < K2 || ld_q < K1 + K2) {
    set_error("%s: leading dimension smaller than the row (ld_x1=%lld ld_x2=%lld ld_q=%lld)", fn,
              (long long)ld_x1, (long long)ld_x2, (long long)ld_q);
    return CDIT_EINVAL;
  }
  if (!x1_bf16 || !x2_bf16 || !q_e4m3 || !scale) {
    set_error("%s: null pointer argument", fn);
    return CDIT_EINVAL;
  }
  int rc = check_arch();
  if (rc) return rc;
  if (cdit::launch_quant_rowwise_cat2(x1_bf16, K1, ld_x1, x2_bf16, K2, ld_x2, M, q_e4m3, ld_q, scale,
                                      mode, static_cast<hipStream_t>(stream)) != 0) {
    set_error("%s: K1 and K2 must be multiples of 8 with K1 + K2 <= 16384, rows 16-byte aligned "
              "(K1=%lld K2=%lld ld_x1=%lld ld_x2=%lld ld_q=%lld): concatenate and call "
              "cdit_fp8_quant_rowwise instead", fn, (long long)K1, (long long)K2, (long long)ld_x1,
              (long long)ld_x2, (long long)ld_q);
    return CDIT_EINVAL;
  }
  return after_launch(fn);
}

int cdit_fp8_quant_rowwise_batched(int n_act, const void* const* x_bf16, const int64_t* M,
                                   int64_t K, const int64_t* ld_x, void* const* q_e4m3,
                                   const int64_t* ld_q, float* const* scale, int scale_mode,
                                   void* stream) {
  const char* fn = "cdit_fp8_quant_rowwise_batched";
  if (n_act < 1 || n_act > cdit::kMaxQuantActs || !x_bf16 || !M || !ld_x || !q_e4m3 || !ld_q || !scale) {
    set_error("%s: 1 to %d activations and non-null argument arrays, got n_act=%d", fn,
              cdit::kMaxQuantActs, n_act);
    return CDIT_EINVAL;
  }
  const int mode = scale_mode >= 0 ? scale_mode & ~CDIT_QUANT_GEMM_FOLLOWS : scale_mode;
  if (mode != CDIT_SCALE_BF16DIV && mode != CDIT_SCALE_FP32DIV) {
    set_error("%s: unknown scale_mode %d", fn, scale_mode);
    return CDIT_EINVAL;
  }
  cdit::QuantBatch batch = {};
  int64_t rows = 0;
  bool one_launch = K > 0 && K <= INT32_MAX;
  for (int s = 0; s < n_act; ++s) {
    if (M[s] < 0 || M[s] > INT32_MAX || K < 0 || K > INT32_MAX) {
      set_error("%s: bad shape M[%d]=%lld K=%lld", fn, s, (long long)M[s], (long long)K);
      return CDIT_EINVAL;
    }
    if (M[s] == 0) continue;
    if (ld_x[s] < K || ld_q[s] < K) {
      set_error("%s: leading dimension smaller than K (activation %d: ld_x=%lld ld_q=%lld K=%lld)",
                fn, s, (long long)ld_x[s], (long long)ld_q[s], (long long)K);
      return CDIT_EINVAL;
    }
    if (!scale[s] || (K > 0 && (!x_bf16[s] || !q_e4m3[s]))) {
      set_error("%s: null pointer argument (activation %d)", fn, s);
      return CDIT_EINVAL;
    }
    const int at = batch.acts++;
    batch.row_begin[at] = (int)rows;
    batch.x[at] = static_cast<const uint16_t*>(x_bf16[s]);
    batch.ld_x[at] = ld_x[s];
    batch.q[at] = static_cast<uint8_t*>(q_e4m3[s]);
    batch.ld_q[at] = ld_q[s];
    batch.scale[at] = scale[s];
    rows += M[s];
  }
  if (batch.acts == 0) return CDIT_OK;
  one_launch = one_launch && rows <= INT32_MAX && batch.acts > 1;
  for (int s = batch.acts; s <= cdit::kMaxQuantActs; ++s) batch.row_begin[s] = (int)(one_launch ? rows : 0);
  int rc = check_arch();
  if (rc) return rc;
  if (one_launch &&
      cdit::launch_quant_rowwise_batched(batch, K, mode, static_cast<hipStream_t>(stream)) == 0)
    return after_launch(fn);
  // a single activation, or a batch the one-launch kernel does not take: one by one
  for (int s = 0; s < n_act; ++s) {
    if (M[s] == 0) continue;
    rc = quant_rowwise_impl(fn, x_bf16[s], M[s], K, ld_x[s], q_e4m3[s], ld_q[s], scale[s], mode,
                            stream, true);
    if (rc) return rc;
  }
  return CDIT_OK;
}

int cdit_fp8_ln_modulate_quant(const void* x_bf16, int64_t M, int64_t K, int64_t ld_x,
                               const void* shift_bf16, const void* scale_bf16, int64_t ld_mod,
                               int64_t rows_per_mod, float eps, void* y_bf16, int64_t ld_y,
                               void* q_e4m3, int64_t ld_q, float* scale, int scale_mode,
                               void* stream) {
  const char* fn = "cdit_fp8_ln_modulate_quant";
  if (M < 0 || K < 0 || M > INT32_MAX || K > INT32_MAX) {
    set_error("%s: bad shape M=%lld K=%lld", fn, (long long)M, (long long)K);
    return CDIT_EINVAL;
  }
  if (scale_mode != CDIT_SCALE_BF16DIV && scale_mode != CDIT_SCALE_FP32DIV) {
    set_error("%s: unknown scale_mode %d", fn, scale_mode);
    return CDIT_EINVAL;
  }
  if (M == 0) return CDIT_OK;
  if (K == 0) {
    set_error("%s: K = 0 has no mean to normalise by", fn);
    return CDIT_EINVAL;
  }
  if (ld_x < K || ld_q < K || (y_bf16 && ld_y < K) || rows_per_mod < 1 ||
      (ld_mod < K && rows_per_mod < M)) {
    set_error("%s: bad leading dimension or rows_per_mod (ld_x=%lld ld_q=%lld ld_y=%lld "
              "ld_mod=%lld rows_per_mod=%lld K=%lld)", fn, (long long)ld_x, (long long)ld_q,
              (long long)ld_y, (long long)ld_mod, (long long)rows_per_mod, (long long)K);
    return CDIT_EINVAL;
  }
  if (!(eps >= 0.0f)) {
    set_error("%s: eps must be >= 0", fn);
    return CDIT_EINVAL;
  }
  if (!x_bf16 || !shift_bf16 || !scale_bf16 || !q_e4m3 || !scale) {
    set_error("%s: null pointer argument", fn);
    return CDIT_EINVAL;
  }
  // one modulation vector for all rows may be spelled with any large count
  if (rows_per_mod > M) rows_per_mod = M;
  int rc = check_arch();
  if (rc) return rc;
  rc = launch_ln_modulate_quant(x_bf16, M, K, ld_x, shift_bf16, scale_bf16, ld_mod, rows_per_mod,
                                eps, y_bf16, ld_y, q_e4m3, ld_q, scale, scale_mode,
                                static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

int cdit_fp8_quant_tensorwise(const void* x_bf16, int64_t M, int64_t K, int64_t ld_x,
                              void* q_e4m3, int64_t ld_q, float* scale, void* amax_ws,
                              int scale_mode, void* stream) {
  const char* fn = "cdit_fp8_quant_tensorwise";
  if (M < 0 || K < 0 || M > INT32_MAX || K > INT32_MAX) {
    set_error("%s: bad shape M=%lld K=%lld", fn, (long long)M, (long long)K);
    return CDIT_EINVAL;
  }
  if (scale_mode != CDIT_SCALE_BF16DIV && scale_mode != CDIT_SCALE_FP32DIV) {
    set_error("%s: unknown scale_mode %d", fn, scale_mode);
    return CDIT_EINVAL;
  }
  if (M == 0) return CDIT_OK;
  if (ld_x < K || ld_q < K) {
    set_error("%s: leading dimension smaller than K (ld_x=%lld ld_q=%lld K=%lld)", fn,
              (long long)ld_x, (long long)ld_q, (long long)K);
    return CDIT_EINVAL;
  }
  if (!scale || !amax_ws || (K > 0 && (!x_bf16 || !q_e4m3))) {
    set_error("%s: null pointer argument", fn);
    return CDIT_EINVAL;
  }
  if (reinterpret_cast<uintptr_t>(amax_ws) % 4 != 0) {
    set_error("%s: amax_ws must be 4-byte aligned", fn);
    return CDIT_EINVAL;
  }
  int rc = check_arch();
  if (rc) return rc;
  rc = launch_quant_tensorwise(x_bf16, M, K, ld_x, q_e4m3, ld_q, scale,
                               static_cast<uint32_t*>(amax_ws), scale_mode,
                               static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

int cdit_fp8_gemm_rowwise(const void* a_q, const float* a_scale, const void* b_q,
                          const float* b_scale, const void* bias, void* out, int64_t M,
                          int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldo,
                          int epilogue, int out_dtype_id, void* stream) {
  const char* fn = "cdit_fp8_gemm_rowwise";
  int rc = check_gemm(fn, a_q, b_q, b_scale, bias, out, M, N, K, lda, ldb, ldo, epilogue,
                      out_dtype_id, false);
  if (rc) return rc;
  if (M == 0 || N == 0) return CDIT_OK;
  if (!a_scale) {
    set_error("%s: a_scale is null", fn);
    return CDIT_EINVAL;
  }
  rc = check_arch();
  if (rc) return rc;
  GemmArgs g;
  g.a = a_q;
  g.a_scale = a_scale;
  g.b = static_cast<const uint8_t*>(b_q);
  g.b_scale = b_scale;
  g.bias = static_cast<const uint16_t*>(bias);
  g.out = static_cast<uint16_t*>(out);
  g.M = (int)M;
  g.N = (int)N;
  g.K = (int)K;
  g.lda = lda;
  g.ldb = ldb;
  g.ldo = ldo;
  g.epilogue = epilogue;
  g.out_dtype = out_dtype_id;
  rc = launch_gemm_fp8(g, g_gemm_variant, static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

// n_act activations, activation s with members_per_act[s] members (flattened in order).
// weight_only: the w8a16 form (a_q holds bf16 activations, a_scale is null)
static int gemm_batched_impl(const char* fn, bool weight_only, int n_act, const void* const* a_q,
                             const float* const* a_scale, const int64_t* M, int64_t K, int64_t lda,
                             const int* members_per_act, const void* const* b_q,
                             const float* const* b_scale, const void* const* bias,
                             void* const* out, const int64_t* N, int64_t ldb, const int64_t* ldo,
                             const int* epilogue, void* stream) {
  if (n_act < 1 || n_act > kMaxActs || !a_q || (!a_scale && !weight_only) || !M || !members_per_act) {
    set_error("%s: 1 to %d activations with their arrays, got n_act=%d", fn, kMaxActs, n_act);
    return CDIT_EINVAL;
  }
  int count = 0;
  for (int s = 0; s < n_act; ++s) {
    if (members_per_act[s] < 1) {
      set_error("%s: activation %d has no member", fn, s);
      return CDIT_EINVAL;
    }
    count += members_per_act[s];
  }
  if (count > kMaxGroup) {
    set_error("%s: count=%d, a batch holds 1 to %d GEMMs", fn, count, kMaxGroup);
    return CDIT_EINVAL;
  }
  if (!b_q || !b_scale || !out || !N || !ldo) {
    set_error("%s: null array argument", fn);
    return CDIT_EINVAL;
  }
  GemmGroup grp = {};
  grp.count = count;
  grp.acts = n_act;
  bool any_empty = false;
  for (int s = 0, p = 0; s < n_act; ++s) {
    grp.first_member[s] = p;
    for (int j = 0; j < members_per_act[s]; ++j, ++p) {
      int rc = check_gemm(fn, a_q[s], b_q[p], b_scale[p], bias ? bias[p] : nullptr, out[p], M[s], N[p],
                          K, lda, ldb, ldo[p], epilogue ? epilogue[p] : 0, CDIT_DT_BF16, weight_only);
      if (rc) return rc;
      if (!weight_only && M[s] > 0 && N[p] > 0 && !a_scale[s]) {
        set_error("%s: a_scale is null", fn);
        return CDIT_EINVAL;
      }
      grp.b[p] = static_cast<const uint8_t*>(b_q[p]);
      grp.b_scale[p] = b_scale[p];
      grp.bias[p] = static_cast<const uint16_t*>(bias ? bias[p] : nullptr);
      grp.out[p] = static_cast<uint16_t*>(out[p]);
      grp.N[p] = (int)N[p];
      grp.ldo[p] = ldo[p];
      grp.epilogue[p] = epilogue ? epilogue[p] : 0;
      any_empty |= N[p] == 0;
    }
    grp.a[s] = a_q[s];
    grp.a_scale[s] = weight_only ? nullptr : a_scale[s];
    grp.M[s] = (int)M[s];
    any_empty |= M[s] == 0;
  }
  for (int s = n_act; s <= kMaxActs; ++s) grp.first_member[s] = count;
  int rc = check_arch();
  if (rc) return rc;
  if (!any_empty) {
    GemmArgs common = {};
    common.K = (int)K;
    common.lda = lda;
    common.ldb = ldb;
    common.out_dtype = CDIT_DT_BF16;
    rc = weight_only
             ? launch_gemm_w8a16_grouped(common, grp, g_gemm_variant, static_cast<hipStream_t>(stream))
             : launch_gemm_fp8_grouped(common, grp, g_gemm_variant, static_cast<hipStream_t>(stream));
    if (rc == 0) return after_launch(fn);
    if (rc > 0) return rc;
  }
  // not taken as a batch (a single member, an M <= 16 problem, an alignment only the
  // element-wise kernel takes): the members one after the other, same results
  for (int s = 0, p = 0; s < n_act; ++s)
    for (int j = 0; j < members_per_act[s]; ++j, ++p) {
      rc = weight_only
               ? cdit_w8a16_gemm(a_q[s], b_q[p], b_scale[p], bias ? bias[p] : nullptr, out[p], M[s],
                                 N[p], K, lda, ldb, ldo[p], epilogue ? epilogue[p] : 0, CDIT_DT_BF16,
                                 stream)
               : cdit_fp8_gemm_rowwise(a_q[s], a_scale[s], b_q[p], b_scale[p],
                                       bias ? bias[p] : nullptr, out[p], M[s], N[p], K, lda, ldb,
                                       ldo[p], epilogue ? epilogue[p] : 0, CDIT_DT_BF16, stream);
      if (rc) return rc;
    }
  return CDIT_OK;
}

int cdit_fp8_gemm_rowwise_grouped(const void* a_q, const float* a_scale, int64_t M, int64_t K,
                                  int64_t lda, int count, const void* const* b_q,
                                  const float* const* b_scale, const void* const* bias,
                                  void* const* out, const int64_t* N, int64_t ldb,
                                  const int64_t* ldo, const int* epilogue, void* stream) {
  return gemm_batched_impl("cdit_fp8_gemm_rowwise_grouped", false, 1, &a_q, &a_scale, &M, K, lda, &count,
                           b_q, b_scale, bias, out, N, ldb, ldo, epilogue, stream);
}

int cdit_fp8_gemm_rowwise_batched(int n_act, const void* const* a_q, const float* const* a_scale,
                                  const int64_t* M, int64_t K, int64_t lda,
                                  const int* members_per_act, const void* const* b_q,
                                  const float* const* b_scale, const void* const* bias,
                                  void* const* out, const int64_t* N, int64_t ldb,
                                  const int64_t* ldo, const int* epilogue, void* stream) {
  return gemm_batched_impl("cdit_fp8_gemm_rowwise_batched", false, n_act, a_q, a_scale, M, K, lda,
                           members_per_act, b_q, b_scale, bias, out, N, ldb, ldo, epilogue, stream);
}

int cdit_w8a16_gemm_batched(int n_act, const void* const* x_bf16, const int64_t* M, int64_t K,
                            int64_t lda, const int* members_per_act, const void* const* b_q,
                            const float* const* b_scale, const void* const* bias,
                            void* const* out, const int64_t* N, int64_t ldb, const int64_t* ldo,
                            const int* epilogue, void* stream) {
  return gemm_batched_impl("cdit_w8a16_gemm_batched", true, n_act, x_bf16, nullptr, M, K, lda,
                           members_per_act, b_q, b_scale, bias, out, N, ldb, ldo, epilogue, stream);
}

int cdit_fp8_linear_w8a8(const void* x_bf16, const void* w_q, const float* w_scale,
                         const void* bias, void* out, void* q_ws, float* scale_ws, int64_t M,
                         int64_t N, int64_t K, int64_t ld_x, int64_t ldw, int64_t ldo,
                         int scale_mode, int epilogue, int out_dtype_id, void* stream) {
  // M <= 16 (the M = 1 modulation Linears): one kernel that quantizes the rows itself,
  // when every argument passes the checks of the two entry points it stands for
  if (M >= 1 && M <= 16 && N > 0 && K > 0 && K <= INT32_MAX && N <= INT32_MAX && x_bf16 && q_ws &&
      scale_ws && w_scale && ld_x >= K &&
      (scale_mode == CDIT_SCALE_BF16DIV || scale_mode == CDIT_SCALE_FP32DIV) &&
      check_gemm("cdit_fp8_linear_w8a8", q_ws, w_q, w_scale, bias, out, M, N, K, K, ldw, ldo,
                 epilogue, out_dtype_id, false) == CDIT_OK &&
      check_arch() == CDIT_OK) {
    GemmArgs g;
    g.a = x_bf16;
    g.a_scale = nullptr;
    g.b = static_cast<const uint8_t*>(w_q);
    g.b_scale = w_scale;
    g.bias = static_cast<const uint16_t*>(bias);
    g.out = static_cast<uint16_t*>(out);
    g.M = (int)M;
    g.N = (int)N;
    g.K = (int)K;
    g.lda = ld_x;
    g.ldb = ldw;
    g.ldo = ldo;
    g.epilogue = epilogue;
    g.out_dtype = out_dtype_id;
    if (launch_linear_fp8_skinny_fused(g, q_ws, scale_ws, scale_mode, g_gemm_variant,
                                       static_cast<hipStream_t>(stream)) == 0)
      return after_launch("cdit_fp8_linear_w8a8");
  }
  int rc = quant_rowwise_impl("cdit_fp8_linear_w8a8", x_bf16, M, K, ld_x, q_ws, K, scale_ws,
                              scale_mode, stream, true);
  if (rc) return rc;
  return cdit_fp8_gemm_rowwise(q_ws, scale_ws, w_q, w_scale, bias, out, M, N, K, K, ldw, ldo,
                               epilogue, out_dtype_id, stream);
}

// ---- FP8 quantizers with packed trailing scales (activations that cross GPUs)
static int check_comm(const char* fn, const void* in, const void* out, int64_t rows, int64_t width,
                      int64_t min_width) {
  if (rows < 0 || width < min_width || rows > INT32_MAX * (int64_t)64 || width > INT32_MAX) {
    set_error("%s: bad shape rows=%lld width=%lld", fn, (long long)rows, (long long)width);
    return CDIT_EINVAL;
  }
  if (rows > 0 && (!in || !out)) {
    set_error("%s: null pointer argument", fn);
    return CDIT_EINVAL;
  }
  return CDIT_OK;
}

int cdit_fp8_comm_per_token_quant(const void* x_bf16, int64_t M, int64_t H, void* y_e4m3,
                                  void* stream) {
  const char* fn = "cdit_fp8_comm_per_token_quant";
  int rc = check_comm(fn, x_bf16, y_e4m3, M, H, 0);
  if (rc || M == 0) return rc;
  if ((rc = check_arch())) return rc;
  rc = launch_comm_per_token_quant(x_bf16, M, H, y_e4m3, static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

int cdit_fp8_comm_per_token_dequant(const void* x_e4m3, int64_t M, int64_t H, void* y_bf16,
                                    void* stream) {
  const char* fn = "cdit_fp8_comm_per_token_dequant";
  int rc = check_comm(fn, x_e4m3, y_bf16, M, H, 0);
  if (rc || M == 0) return rc;
  if ((rc = check_arch())) return rc;
  rc = launch_comm_per_token_dequant(x_e4m3, M, H, y_bf16, static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

int cdit_fp8_comm_qkv_permute_quant(const void* x_bf16, int64_t B, int64_t S, int64_t P, int64_t N,
                                    int64_t D, int64_t stride_b, int64_t stride_s, int64_t stride_p,
                                    void* quant_x, void* stream) {
  const char* fn = "cdit_fp8_comm_qkv_permute_quant";
  if (B < 0 || S < 0 || P < 0 || N < 0 || D < 0 || B > INT32_MAX || S > INT32_MAX || P > INT32_MAX ||
      N > INT32_MAX || D > INT32_MAX) {
    set_error("%s: bad shape B=%lld S=%lld P=%lld N=%lld D=%lld", fn, (long long)B, (long long)S,
              (long long)P, (long long)N, (long long)D);
    return CDIT_EINVAL;
  }
  if (D % 4 != 0) {  // the fp32 scale sits at byte D of a row that starts on a 4-byte boundary
    set_error("%s: D=%lld is not a multiple of 4", fn, (long long)D);
    return CDIT_EINVAL;
  }
  if (B * S * P * N == 0) return CDIT_OK;
  if (!x_bf16 || !quant_x) {
    set_error("%s: null pointer argument", fn);
    return CDIT_EINVAL;
  }
  int rc = check_arch();
  if (rc) return rc;
  rc = launch_comm_qkv_permute_quant(x_bf16, (int)B, (int)S, (int)P, (int)N, (int)D, stride_b,
                                     stride_s, stride_p, quant_x, static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

int cdit_fp8_comm_qkv_permute_dequant(const void* quant_x, int64_t S, int64_t B, int64_t N, int64_t D,
                                      int64_t stride_s, int64_t stride_b, int64_t stride_n,
                                      void* x_bf16, void* stream) {
  const char* fn = "cdit_fp8_comm_qkv_permute_dequant";
  if (B < 0 || S < 0 || N < 0 || D < 0 || B > INT32_MAX || S > INT32_MAX || N > INT32_MAX ||
      D > INT32_MAX) {
    set_error("%s: bad shape S=%lld B=%lld N=%lld D=%lld", fn, (long long)S, (long long)B,
              (long long)N, (long long)D);
    return CDIT_EINVAL;
  }
  if (D % 4 != 0) {
    set_error("%s: D=%lld is not a multiple of 4", fn, (long long)D);
    return CDIT_EINVAL;
  }
  if (B * S * N == 0) return CDIT_OK;
  if (!x_bf16 || !quant_x) {
    set_error("%s: null pointer argument", fn);
    return CDIT_EINVAL;
  }
  if (stride_n < D + 4) {
    set_error("%s: stride_n=%lld is smaller than a row of D + 4 bytes", fn, (long long)stride_n);
    return CDIT_EINVAL;
  }
  int rc = check_arch();
  if (rc) return rc;
  rc = launch_comm_qkv_permute_dequant(quant_x, (int)S, (int)B, (int)N, (int)D, stride_s, stride_b,
                                       stride_n, x_bf16, static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

// ---- allocation-free Linear: activation codes and scales in a library-owned array
// One copy of the array lives on every GPU the library runs on, for the life of the
// process. Host code never uses the array's name as an address (it is a host-side
// stand-in): the device address is looked up once per device and kept.
static __device__ __align__(256) uint8_t scratch[CDIT_STATIC_WS_CODE_BYTES +
                                                 CDIT_STATIC_WS_ROWS * sizeof(float)];

// Device address of `scratch` on the current device (looked up on the first call on that
// device, with the device current), or nullptr with the error set.
static uint8_t* static_scratch_of_current_device() {
  static std::mutex mu;
  static uint8_t* ptr[64];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("hipGetDevice: %s", hipGetErrorString(e));
    return nullptr;
  }
  if (dev < 0 || dev >= 64) {
    set_error("device ordinal %d out of range", dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      set_error("hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    ptr[dev] = static_cast<uint8_t*>(p);
  }
  return ptr[dev];
}

int cdit_fp8_linear_w8a8_static(const void* x_bf16, const void* w_q, const float* w_scale,
                                const void* bias, void* out, int64_t M, int64_t N, int64_t K,
                                int64_t ld_x, int64_t ldw, int64_t ldo, int scale_mode,
                                int epilogue, int out_dtype_id, void* stream) {
  const char* fn = "cdit_fp8_linear_w8a8_static";
  if (M < 0 || K < 0 || N < 0) {
    set_error("%s: negative dimension (M=%lld N=%lld K=%lld)", fn, (long long)M, (long long)N,
              (long long)K);
    return CDIT_EINVAL;
  }
  if (M > CDIT_STATIC_WS_ROWS || (K > 0 && M > CDIT_STATIC_WS_CODE_BYTES / K)) {
    set_error("%s: M=%lld K=%lld exceeds the built-in workspace (M*K <= %lld bytes of codes, M <= "
              "%lld rows); use cdit_fp8_linear_w8a8 with workspaces of your own",
              fn, (long long)M, (long long)K, (long long)CDIT_STATIC_WS_CODE_BYTES,
              (long long)CDIT_STATIC_WS_ROWS);
    return CDIT_EINVAL;
  }
  if (M == 0 || N == 0) {
    // nothing to compute; the arguments still get the checks of the full entry point
    return check_gemm(fn, x_bf16, w_q, w_scale, bias, out, M, N, K, K, ldw, ldo, epilogue,
                      out_dtype_id, false);
  }
  int rc = check_arch();
  if (rc) return rc;
  uint8_t* ws = static_scratch_of_current_device();
  if (!ws) return CDIT_EHIP;
  // codes first (contiguous rows of K bytes), scales behind them at a fixed, aligned offset
  return cdit_fp8_linear_w8a8(x_bf16, w_q, w_scale, bias, out, ws,
                              reinterpret_cast<float*>(ws + CDIT_STATIC_WS_CODE_BYTES), M, N, K,
                              ld_x, ldw, ldo, scale_mode, epilogue, out_dtype_id, stream);
}

int cdit_w8a16_gemm(const void* x_bf16, const void* b_q, const float* b_scale,
                    const void* bias_bf16, void* out, int64_t M, int64_t N, int64_t K,
                    int64_t lda, int64_t ldb, int64_t ldo, int epilogue, int out_dtype_id,
                    void* stream) {
  const char* fn = "cdit_w8a16_gemm";
  int rc = check_gemm(fn, x_bf16, b_q, b_scale, bias_bf16, out, M, N, K, lda, ldb, ldo, epilogue,
                      out_dtype_id, true);
  if (rc) return rc;
  if (M == 0 || N == 0) return CDIT_OK;
  rc = check_arch();
  if (rc) return rc;
  GemmArgs g;
  g.a = x_bf16;
  g.a_scale = nullptr;
  g.b = static_cast<const uint8_t*>(b_q);
  g.b_scale = b_scale;
  g.bias = static_cast<const uint16_t*>(bias_bf16);
  g.out = static_cast<uint16_t*>(out);
  g.M = (int)M;
  g.N = (int)N;
  g.K = (int)K;
  g.lda = lda;
  g.ldb = ldb;
  g.ldo = ldo;
  g.epilogue = epilogue;
  rc = launch_gemm_w8a16(g, g_gemm_variant, static_cast<hipStream_t>(stream));
  return rc ? rc : after_launch(fn);
}

}  // extern "C"
