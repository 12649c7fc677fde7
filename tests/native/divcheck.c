/*
 * divcheck.c -- exhaustive CPU proof that the quantizer kernel's division
 * (per row the reciprocal of the scale as an unevaluated sum hi + lo of two
 * fp32 values, per element one multiply and one FMA: x hi + x lo) yields the
 * same e4m3 code as the IEEE division the oracle uses, for EVERY input the
 * kernel can see on its fast path: every bf16 amax whose scale lies in the
 * fast path's exponent window, both scale modes, and every bf16 x with
 * |x| <= amax, both signs (a negative zero keeps its sign).
 *
 * Usage: divcheck [stride]   (stride > 1 subsamples the amax values)
 * Prints the number of (x, amax) pairs checked, how many of the fp32 values
 * differ from the fp32 quotient of the division (allowed: a double rounding
 * of the small term) and how many e4m3 codes differ; exit 1 on any code
 * mismatch.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

float oracle_bf16_to_f32(uint16_t b);
float oracle_row_scale(uint16_t amax_bf16, int mode);
uint8_t oracle_e4m3_encode(float f);

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* the kernel's fast-path window (must match quant_rowwise.hip) */
static int scale_in_fast_window(float s) {
  uint32_t e = (f2u(s) >> 23) & 0xff;
  return e >= 27 && e <= 227; /* 2^-100 <= s < 2^101 */
}

int main(int argc, char** argv) {
  int stride = argc > 1 ? atoi(argv[1]) : 1;
  if (stride < 1) stride = 1;
  long long checked = 0, bad_q = 0, bad_code = 0;
#pragma omp parallel for schedule(dynamic, 16) reduction(+ : checked, bad_q, bad_code)
  for (int am = 1; am < 0x7f80; am += stride) { /* finite, non-zero amax */
    for (int mode = 0; mode < 2; ++mode) {
      const float s = oracle_row_scale((uint16_t)am, mode);
      if (!scale_in_fast_window(s)) continue;
      /* the kernel's make_recip: hi at or just below 1 / s, lo >= 0 the remainder */
      const float r = 1.0f / s;
      float r_hi = r;
      if (fmaf(-s, r, 1.0f) < 0.0f) {
        const uint32_t u = f2u(r) - 1u;
        memcpy(&r_hi, &u, 4);
      }
      const float r_lo = fmaf(-s, r_hi, 1.0f) * r;
      for (int xb = 0; xb <= am; ++xb) { /* |x| <= amax; sign symmetric, check both */
        for (int sg = 0; sg < 2; ++sg) {
          const float x = oracle_bf16_to_f32((uint16_t)(xb | (sg << 15)));
          const float ref = x / s;
          /* the kernel's form (-ffp-contract=off: the product is rounded on its own) */
          const float t = x * r_lo;
          const float q1 = fmaf(x, r_hi, t);
          ++checked;
          /* the kernel's fast path does not clamp: the raw quotient must encode like
           * the oracle's clamped one (it stays below the tie at 464) */
          {
            float rc = ref;
            if (rc < -448.f) rc = -448.f;
            if (rc > 448.f) rc = 448.f;
            if (!(fabsf(q1) < 464.0f) || oracle_e4m3_encode(q1) != oracle_e4m3_encode(rc)) ++bad_code;
          }
          if (f2u(q1) != f2u(ref)) ++bad_q;
        }
      }
    }
  }
  printf("checked=%lld quotient_mismatch=%lld code_mismatch=%lld\n", checked, bad_q, bad_code);
  return bad_code != 0;
}
