/*
 * divcheck.c -- exhaustive CPU proof that the quantizer kernel's division
 * (one correctly rounded reciprocal per row, then multiply + two FMAs per
 * element) yields the same fp32 quotient, hence the same e4m3 code, as the
 * IEEE division the oracle uses, for EVERY input the kernel can see on its
 * fast path: every bf16 amax whose scale lies in the fast path's exponent
 * window, both scale modes, and every bf16 x with |x| <= amax.
 *
 * Usage: divcheck [stride]   (stride > 1 subsamples the amax values)
 * Prints the number of (x, amax) pairs checked and of mismatches; exit 1 on
 * any mismatch.
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
      const float r = 1.0f / s;
      for (int xb = 0; xb <= am; ++xb) { /* |x| <= amax; sign symmetric, check both */
        for (int sg = 0; sg < 2; ++sg) {
          const float x = oracle_bf16_to_f32((uint16_t)(xb | (sg << 15)));
          const float ref = x / s;
          const float q0 = x * r;
          /* the kernel's form: the residual negated, no copysign (keeps the sign of -0).
           * The empty asm hides where d comes from: gcc -O1 and above otherwise rewrites
           * -fma(a, b, c) as fma(-a, b, -c), which is not the same operation for a zero
           * result (it turns this form back into the usual one and -0 into +0). */
          float d = fmaf(q0, s, -x);
          __asm__ volatile("" : "+x"(d));
          const float q1 = fmaf(-d, r, q0);
          ++checked;
          /* the kernel's fast path does not clamp: the raw quotient must encode like
           * the oracle's clamped one (it stays below the tie at 464) */
          {
            float rc = ref;
            if (rc < -448.f) rc = -448.f;
            if (rc > 448.f) rc = 448.f;
            if (!(fabsf(q1) < 464.0f) || oracle_e4m3_encode(q1) != oracle_e4m3_encode(rc)) ++bad_code;
          }
          if (f2u(q1) != f2u(ref)) {
            ++bad_q;
            float a = ref, b = q1;
            if (a < -448.f) a = -448.f; if (a > 448.f) a = 448.f;
            if (b < -448.f) b = -448.f; if (b > 448.f) b = 448.f;
            (void)a;
            (void)b;
          }
        }
      }
    }
  }
  printf("checked=%lld quotient_mismatch=%lld code_mismatch=%lld\n", checked, bad_q, bad_code);
  return bad_code != 0;
}
