/*
 * cdit_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement, in plain C, of the arithmetic on cache-dit's FP8
 * quantized-linear path. It exists only so that tests/, the smoke check and
 * the benchmark's cpu_baseline leg can check or time the algorithm; nothing in
 * the shipped package may link or call it.
 *
 * The arithmetic itself lives in torchao (>= 0.17, un-pinned and un-vendored:
 * /root/reference/pyproject.toml:30-34) and in torch._scaled_mm; the reference
 * holds only the call sites, so each function below cites the call site it
 * serves and restates the published torchao / PyTorch behaviour:
 *   - scale:    torchao _choose_scale_float8 with cache-dit's zero-scale patch,
 *               src/cache_dit/quantization/torchao/quantize_ao.py:43-71
 *   - cast:     torchao _quantize_affine_float8 (clamp to +-448, then
 *               .to(float8_e4m3fn)), reached through Float8Tensor.from_hp at
 *               tests/kernels/test_opaque_scaled_mm.py:68-73
 *   - GEMM:     torch._scaled_mm row-wise, fp32 accumulate, bias, bf16 out,
 *               src/cache_dit/quantization/torchao/_scaled_mm.py:62-91
 *   - w8a16:    F.linear(x, W.dequantize(), b), Float8WeightOnlyConfig,
 *               src/cache_dit/quantization/torchao/quantize_ao.py:604-610
 *   - GELU:     diffusers nn.GELU(approximate="tanh") after proj_mlp,
 *               src/cache_dit/caching/patch_functors/functor_flux.py:48-80
 *
 * PARITY STATUS. The reference's own tests hold no golden vector for this path
 * (tests/kernels/test_opaque_scaled_mm.py:91-94 only bounds eager-vs-compiled
 * by 0.5), and torchao cannot be imported here, so:
 *   - e4m3 encode/decode, clamp, RNE, amax, GEMM, GELU are pinned against
 *     PyTorch's own CPU float8_e4m3fn cast / matmul / gelu and closed forms
 *     (tests/test_oracle_*.py);
 *   - whether torchao rounds amax/448 to bf16 before widening
 *     (CDIT_SCALE_BF16DIV) or divides in fp32 (CDIT_SCALE_FP32DIV) is
 *     "parity unpinned": both modes are implemented and selectable.
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp -ffp-contract=off)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define FP8_MAX 448.0f

static inline float u2f(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t f2u(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

float oracle_bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }

/* fp32 -> bf16, round to nearest even (c10::BFloat16 rule; NaN -> 0x7FC0). */
uint16_t oracle_f32_to_bf16(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/*
 * fp32 -> OCP e4m3fn byte, round to nearest even, written from the format's
 * definition (S.EEEE.MMM, bias 7, subnormal step 2^-9, max finite 448 = 0x7E,
 * 0x7F/0xFF = NaN, no infinity). Values that round beyond 448 become NaN, as
 * torch's cast does (464 -> 448 by the tie rule, 465 -> NaN).
 */
uint8_t oracle_e4m3_encode(float f) {
  uint32_t u = f2u(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  float a = fabsf(f);
  if (a != a) return (uint8_t)(sign | 0x7f);
  if (a >= 480.0f) return (uint8_t)(sign | 0x7f); /* inf and overflow */
  int e;
  /* quantum = spacing of e4m3 values around a */
  if (a < 0.015625f) { /* below 2^-6: subnormal range, spacing 2^-9 */
    e = -6;
  } else {
    (void)frexpf(a, &e); /* a = m * 2^e, m in [0.5,1) */
    e -= 1;              /* a = 1.x * 2^e */
  }
  float quantum = ldexpf(1.0f, e - 3);
  /* a / quantum is exact (power of two) and < 2^24: nearbyintf rounds half-even */
  float n = nearbyintf(a / quantum);
  float r = n * quantum; /* rounded magnitude, exact */
  if (r > 448.0f) return (uint8_t)(sign | 0x7f);
  if (r == 0.0f) return sign;
  if (r < 0.015625f) return (uint8_t)(sign | (uint8_t)n); /* subnormal: mantissa = n */
  int e2;
  float m = frexpf(r, &e2); /* r = m*2^e2, m in [0.5,1) -> 1.x * 2^(e2-1) */
  int expo = e2 - 1 + 7;
  int mant = (int)((m * 2.0f - 1.0f) * 8.0f);
  return (uint8_t)(sign | (expo << 3) | mant);
}

float oracle_e4m3_decode(uint8_t b) {
  int expo = (b >> 3) & 0xf, mant = b & 7;
  float v;
  if (expo == 0xf && mant == 7) return u2f(0x7fc00000u | ((uint32_t)(b & 0x80) << 24));
  if (expo == 0)
    v = ldexpf((float)mant, -9);
  else
    v = ldexpf(1.0f + (float)mant / 8.0f, expo - 7);
  return (b & 0x80) ? -v : v;
}

/* scale of one row from its bf16 amax; mode 0 = BF16DIV, 1 = FP32DIV. */
float oracle_row_scale(uint16_t amax_bf16, int mode) {
  float s = oracle_bf16_to_f32(amax_bf16) / FP8_MAX;
  if (mode == 0) s = oracle_bf16_to_f32(oracle_f32_to_bf16(s));
  if (s == 0.0f) s = 1.0f; /* quantize_ao.py:65-67 */
  return s;
}

uint8_t oracle_quant_one(uint16_t x_bf16, float s) {
  float y = oracle_bf16_to_f32(x_bf16) / s; /* true division */
  if (y == y) {                             /* torch.clamp propagates NaN */
    if (y < -FP8_MAX) y = -FP8_MAX;
    if (y > FP8_MAX) y = FP8_MAX;
  }
  return oracle_e4m3_encode(y);
}

/* x bf16 [M,K] (ld_x) -> q e4m3 [M,K] (ld_q), scale fp32 [M]. */
void oracle_quant_rowwise(const uint16_t* x, int64_t M, int64_t K, int64_t ld_x, uint8_t* q,
                          int64_t ld_q, float* scale, int mode) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    const uint16_t* xr = x + m * ld_x;
    uint16_t amax = 0;
    int has_nan = 0;
    for (int64_t k = 0; k < K; ++k) {
      uint16_t a = xr[k] & 0x7fff;
      if (a > 0x7f80) has_nan = 1;
      if (a > amax) amax = a;
    }
    if (has_nan) amax = 0x7fc0; /* torch.amax propagates NaN */
    float s = oracle_row_scale(amax, mode);
    scale[m] = s;
    for (int64_t k = 0; k < K; ++k) q[m * ld_q + k] = oracle_quant_one(xr[k], s);
  }
}

/* Per-tensor: one amax over the whole tensor, scale[m] = that scale for every m. */
void oracle_quant_tensorwise(const uint16_t* x, int64_t M, int64_t K, int64_t ld_x, uint8_t* q,
                             int64_t ld_q, float* scale, int mode) {
  uint16_t amax = 0;
  int has_nan = 0;
  for (int64_t m = 0; m < M; ++m)
    for (int64_t k = 0; k < K; ++k) {
      uint16_t a = x[m * ld_x + k] & 0x7fff;
      if (a > 0x7f80) has_nan = 1;
      if (a > amax) amax = a;
    }
  if (has_nan) amax = 0x7fc0;
  const float s = oracle_row_scale(amax, mode);
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    scale[m] = s;
    for (int64_t k = 0; k < K; ++k) q[m * ld_q + k] = oracle_quant_one(x[m * ld_x + k], s);
  }
}

float oracle_gelu_tanh(float v) {
  const float kAlpha = 0.7978845608028654f, kBeta = 0.044715f;
  return 0.5f * v * (1.0f + tanhf(kAlpha * (v + kBeta * v * v * v)));
}

/*
 * out[m,n] = bf16( epi( (sum_k a[m,k] b[n,k]) * a_scale[m] * b_scale[n] + bias[n] ) )
 * Products of two e4m3 values are exact in fp32; the sum is taken in double
 * and rounded once, so it is the correctly rounded value any fp32
 * accumulation order approximates. gelu: 0 none, 1 fused (on the fp32 value),
 * 2 unfused (on the bf16-rounded linear output, as the separate nn.GELU does).
 */
void oracle_gemm_rowwise(const uint8_t* a, const float* a_scale, const uint8_t* b,
                         const float* b_scale, const uint16_t* bias, uint16_t* out, int64_t M,
                         int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldo, int gelu) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = oracle_e4m3_decode((uint8_t)i);
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k)
        acc += (double)(lut[a[m * lda + k]] * lut[b[n * ldb + k]]);
      float v = (float)acc * a_scale[m] * b_scale[n];
      if (bias) v += oracle_bf16_to_f32(bias[n]);
      if (gelu == 1) v = oracle_gelu_tanh(v);
      uint16_t o = oracle_f32_to_bf16(v);
      if (gelu == 2) o = oracle_f32_to_bf16(oracle_gelu_tanh(oracle_bf16_to_f32(o)));
      out[m * ldo + n] = o;
    }
  }
}

/*
 * Weight-only linear. dequant_bf16 = 1 restates the reference (weight
 * dequantized to bf16 first: Wd = bf16(float(q) * s), then a bf16 GEMM with
 * fp32 accumulate); 0 is the fused form (scale applied to the accumulator).
 */
void oracle_w8a16(const uint16_t* x, const uint8_t* b, const float* b_scale, const uint16_t* bias,
                  uint16_t* out, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb,
                  int64_t ldo, int gelu, int dequant_bf16) {
  float lut[256];
  for (int i = 0; i < 256; ++i) lut[i] = oracle_e4m3_decode((uint8_t)i);
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k) {
        float w = lut[b[n * ldb + k]];
        if (dequant_bf16) w = oracle_bf16_to_f32(oracle_f32_to_bf16(w * b_scale[n]));
        acc += (double)oracle_bf16_to_f32(x[m * lda + k]) * (double)w;
      }
      float v = dequant_bf16 ? (float)acc : (float)acc * b_scale[n];
      if (bias) v += oracle_bf16_to_f32(bias[n]);
      if (gelu == 1) v = oracle_gelu_tanh(v);
      uint16_t o = oracle_f32_to_bf16(v);
      if (gelu == 2) o = oracle_f32_to_bf16(oracle_gelu_tanh(oracle_bf16_to_f32(o)));
      out[m * ldo + n] = o;
    }
  }
}
