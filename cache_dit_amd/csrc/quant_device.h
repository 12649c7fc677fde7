// Device-side arithmetic of the per-row FP8 quantizer, shared by the quantizer kernels
// and by the GEMM kernel that quantizes its own activation rows (M <= 16).
#ifndef CDIT_QUANT_DEVICE_H_
#define CDIT_QUANT_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cdit_internal.h"

namespace cdit {
namespace {

constexpr float kFp8Max = 448.0f;

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// fp32 -> nearest-even bf16, returned widened back to fp32 (c10::BFloat16 rule).
__device__ __forceinline__ float round_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return __uint_as_float(0x7fc00000u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return __uint_as_float(u & 0xffff0000u);
}

// two fp32 -> packed bf16 pair, round to nearest even (v_cvt_pk_bf16_f32: one
// instruction for what round_to_bf16 spells out in five integer operations per value;
// a NaN keeps its sign and payload bits here, round_to_bf16 returns the canonical one)
__device__ __forceinline__ uint32_t pk_bf16(float lo, float hi) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
  const v2f v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, v2bf));
}

// max over the wavefront of an unsigned value (order independent, exact). Four
// DPP steps reduce each row of 16 lanes (xor 1, xor 2, half mirror, mirror), then
// the four row results are read into scalars.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  auto step = [](uint32_t a, int ctrl_id) {
    uint32_t o;
    switch (ctrl_id) {
      case 0: o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)a, 0xB1, 0xf, 0xf, false); break;
      case 1: o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)a, 0x4E, 0xf, 0xf, false); break;
      case 2: o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)a, 0x141, 0xf, 0xf, false); break;
      default: o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)a, 0x140, 0xf, 0xf, false); break;
    }
    return a > o ? a : o;
  };
  v = step(v, 0);  // quad_perm [1,0,3,2]
  v = step(v, 1);  // quad_perm [2,3,0,1]
  v = step(v, 2);  // row_half_mirror
  v = step(v, 3);  // row_mirror
  const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0);
  const uint32_t b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
  const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32);
  const uint32_t d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
  const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
  return ab > cd ? ab : cd;
}

// Sum over the wavefront, the same in every lane: four DPP steps inside each row of 16
// lanes (the pattern of wave_max_u32: no LDS crossbar, no waits), then the four row sums
// through scalars. The order of the additions is fixed, so the result does not depend on
// where the wavefront runs.
__device__ __forceinline__ float wave_sum_f32(float v) {
  auto step = [](float a, int ctrl_id) {
    int o;
    const int ai = __float_as_int(a);
    switch (ctrl_id) {
      case 0: o = __builtin_amdgcn_update_dpp(0, ai, 0xB1, 0xf, 0xf, false); break;   // quad_perm [1,0,3,2]
      case 1: o = __builtin_amdgcn_update_dpp(0, ai, 0x4E, 0xf, 0xf, false); break;   // quad_perm [2,3,0,1]
      case 2: o = __builtin_amdgcn_update_dpp(0, ai, 0x141, 0xf, 0xf, false); break;  // row_half_mirror
      default: o = __builtin_amdgcn_update_dpp(0, ai, 0x140, 0xf, 0xf, false); break;  // row_mirror
    }
    return a + __int_as_float(o);
  };
  v = step(v, 0);
  v = step(v, 1);
  v = step(v, 2);
  v = step(v, 3);
  const float a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  const float b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  const float c = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  const float d = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return (a + b) + (c + d);
}

__device__ __forceinline__ float row_scale(uint32_t amax_bits, int scale_mode) {
  // amax_bits: bf16 bit pattern of max |x| (sign cleared).
  float amax = __uint_as_float(amax_bits << 16);
  float s = amax / kFp8Max;
  if (scale_mode == CDIT_SCALE_BF16DIV) s = round_to_bf16(s);
  return s == 0.0f ? 1.0f : s;
}

// torch.clamp keeps NaN (fminf / fmaxf would drop it): a NaN quotient -- Inf / Inf in a
// row that holds an infinity, anything in a row that holds a NaN -- must reach the
// converter as NaN. Only the cold paths clamp.
__device__ __forceinline__ float clamp448(float y) {
  return y != y ? y : fminf(fmaxf(y, -kFp8Max), kFp8Max);
}

// 1 / s of the fast path as an unevaluated sum hi + lo of two fp32 values: hi is the fp32
// value at or just below 1 / s (the correctly rounded reciprocal, stepped down by one unit in
// the last place when it lies above), lo >= 0 the remainder (1 - s hi) / s to fp32 accuracy.
// Worked out once per row.
struct Recip {
  float hi, lo;
};
__device__ __forceinline__ Recip make_recip(float s) {
  const float r = 1.0f / s;
  const float hi = __fmaf_rn(-s, r, 1.0f) < 0.0f ? __uint_as_float(__float_as_uint(r) - 1u) : r;
  return Recip{hi, __fmaf_rn(-s, hi, 1.0f) * r};
}

// x / s with s > 0 finite. FAST (s inside the window, r = make_recip(s)): x hi + x lo in a
// multiply and an FMA. The sum hi + lo carries 1 / s to about 48 bits, so the result is
// x / s rounded once, up to a double rounding of the small term: not always the fp32
// quotient of the division, but always a value that converts to the same e4m3 code -- the
// roundings of that conversion lie 2^20 times further apart than those of fp32, and an exact
// tie of the conversion is reproduced exactly (tests/native/divcheck.c checks every input
// pair). With lo >= 0 both terms carry the sign of x, so x = -0 gives -0.
template <bool FAST>
__device__ __forceinline__ float div_scale(float x, float s, Recip r) {
  if constexpr (FAST) {
    return __fmaf_rn(x, r.hi, x * r.lo);
  } else {
    return x / s;
  }
}

// 2^-100 <= s < 2^101: the window the fast division is proven on.
__device__ __forceinline__ bool scale_in_fast_window(float s) {
  const uint32_t e = (__float_as_uint(s) >> 23) & 0xffu;
  return e >= 27u && e <= 227u;
}

// two bf16 pairs (4 elements) -> 4 e4m3 bytes. On the fast path the clamp is
// implicit: |x| <= amax and scale >= amax/448 * (1 - 2^-9), so |x/scale| < 450,
// below the tie at 464 where the e4m3 conversion would stop rounding to 448
// (tests/native/divcheck.c checks the unclamped quotient of every input pair).
template <bool FAST>
__device__ __forceinline__ uint32_t quant4(uint32_t w0, uint32_t w1, float s, Recip r) {
  float a = div_scale<FAST>(bf16_lo(w0), s, r);
  float b = div_scale<FAST>(bf16_hi(w0), s, r);
  float c = div_scale<FAST>(bf16_lo(w1), s, r);
  float d = div_scale<FAST>(bf16_hi(w1), s, r);
  if constexpr (!FAST) {
    a = clamp448(a);
    b = clamp448(b);
    c = clamp448(c);
    d = clamp448(d);
  }
  uint32_t p = 0;
  p = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, p, false);
  p = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, p, true);
  return p;
}

// Running max of packed |bf16| pairs, both halves at once: m and the result hold
// two independent 16-bit maxima (v_pk_max_u16), compared as unsigned integers
// (monotone in magnitude; a NaN pattern wins, as in torch.amax). fold2 merges the
// halves at the end.
__device__ __forceinline__ uint32_t absmax2(uint32_t m, uint32_t w) {
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  const u16x2 a = __builtin_bit_cast(u16x2, w & 0x7fff7fffu);
  const u16x2 r = __builtin_elementwise_max(__builtin_bit_cast(u16x2, m), a);
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint32_t fold2(uint32_t m) {
  const uint32_t lo = m & 0xffffu, hi = m >> 16;
  return lo > hi ? lo : hi;
}

}  // namespace
}  // namespace cdit
#endif
