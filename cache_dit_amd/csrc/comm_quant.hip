// FP8 (OCP e4m3fn) quantizers for activations that cross GPUs, with the scale packed
// behind the codes of each row so that one buffer travels. Counterparts of the
// reference's Triton kernels, src/cache_dit/kernels/triton/_float8_comm.py:
//   per-token quant / dequant  (:5-40, :43-62; wrappers _ops_registery.py:52-112)
//     row of H bf16 -> H codes + the scale as bf16 in 2 trailing bytes (pitch H + 2);
//     amax floored at 1e-4, codes = cast(clamp(x * (1 / (amax / 448)), +-448)); the
//     scale that travels is amax / 448 rounded to bf16, dequant multiplies by it.
//   qkv permute quant / dequant (:66-113, :116-148; wrappers :115-185)
//     x [B,S,P,N,D] -> [P,S,B,N,D+4]: per head row of D values the codes followed by the
//     fp32 scale max(amax / 448, 1e-6) in 4 trailing bytes; codes = cast(clamp(x / scale,
//     +-448)) with a true division; dequant [S,B,N,D+4] -> [B,S,N,D] bf16.
// This arithmetic differs from the GEMM path's quantizer (reciprocal multiply, eps
// floors, where the scale is rounded) and shares none of its contract.
//
// All four are pure HBM streaming: one 64-lane wavefront per row, the row read once
// and kept in registers between the amax and the cast. Rows with a pitch of H + 2 (or
// D + 4) bytes start on 2- (4-) byte boundaries, so code rows are moved in the widest
// pieces their alignment allows.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cdit_internal.h"
#include "quant_device.h"

namespace cdit {
namespace {

constexpr int kMaxChunks = 32;  // 16-byte chunks of bf16 per lane: rows of up to 16384 values

__device__ __forceinline__ float wave_max_f32_nonneg(float v) {
  // non-negative floats order like their bit patterns
  return __uint_as_float(wave_max_u32(__float_as_uint(v)));
}

// fp32 -> bf16 bits, round to nearest even; NaN stays NaN.
__device__ __forceinline__ uint32_t f32_to_bf16_bits_rne(float f) {
  return __float_as_uint(round_to_bf16(f)) >> 16;
}

__device__ __forceinline__ uint32_t cvt4_fp8(float a, float b, float c, float d) {
  uint32_t p = 0;
  p = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, p, false);
  p = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, p, true);
  return p;
}

// 8 code bytes to dst, which is 2-byte aligned at least (wave-uniform alignment).
__device__ __forceinline__ void store8(uint8_t* dst, uint32_t lo, uint32_t hi, int align) {
  if (align >= 8) {
    *reinterpret_cast<uint2*>(dst) = uint2{lo, hi};
  } else if (align >= 4) {
    reinterpret_cast<uint32_t*>(dst)[0] = lo;
    reinterpret_cast<uint32_t*>(dst)[1] = hi;
  } else {
    uint16_t* d = reinterpret_cast<uint16_t*>(dst);
    d[0] = (uint16_t)lo;
    d[1] = (uint16_t)(lo >> 16);
    d[2] = (uint16_t)hi;
    d[3] = (uint16_t)(hi >> 16);
  }
}

__device__ __forceinline__ uint2 load8(const uint8_t* src, int align) {
  if (align >= 8) return *reinterpret_cast<const uint2*>(src);
  if (align >= 4) {
    return uint2{reinterpret_cast<const uint32_t*>(src)[0], reinterpret_cast<const uint32_t*>(src)[1]};
  }
  const uint16_t* s = reinterpret_cast<const uint16_t*>(src);
  return uint2{(uint32_t)s[0] | ((uint32_t)s[1] << 16), (uint32_t)s[2] | ((uint32_t)s[3] << 16)};
}

// Division of a row index by a launch constant (N, B, S of the permuted layouts): the
// compiler's 64-bit division costs more instructions than the row's arithmetic. For
// n < 2^31 and 2^(s-1) < d <= 2^s: n / d = (n * mul) >> (31 + s) with mul = floor(2^(31+s) / d)
// + 1 (mul * d exceeds 2^(31+s) by at most d, so the error term n * d / 2^(31+s) stays below
// one), which is one v_mul_hi_u32 and a shift. d = 1 is passed as mul = 0.
struct FastDiv {
  uint32_t d, mul, shift;
};
FastDiv make_fastdiv(uint32_t d) {
  if (d <= 1) return FastDiv{1u, 0u, 0u};
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  return FastDiv{d, (uint32_t)((1ull << (31 + s)) / d + 1ull), s - 1};
}
__device__ __forceinline__ uint32_t fd_div(uint32_t n, FastDiv f) {
  return f.mul ? __umulhi(n, f.mul) >> f.shift : n;
}

// max over each group of G adjacent lanes (G = 8, 16, 32), the same in every lane of the
// group: DPP inside rows of 16 lanes, one crossbar step for G = 32.
template <int G>
__device__ __forceinline__ uint32_t group_max_u32(uint32_t v) {
  auto mx = [](uint32_t a, uint32_t b) { return a > b ? a : b; };
  v = mx(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  v = mx(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  v = mx(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, false));  // row_half_mirror
  if constexpr (G >= 16) v = mx(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xf, 0xf, false));  // row_mirror
  if constexpr (G >= 32) v = mx(v, (uint32_t)__shfl_xor((int)v, 16, 64));
  return v;
}

__device__ __forceinline__ int align_of(const void* p) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p);
  return (a & 7) == 0 ? 8 : (a & 3) == 0 ? 4 : (a & 1) == 0 ? 2 : 1;
}

// SCALE: 0 = per-token form (bf16 scale, eps on amax, reciprocal multiply),
//        1 = qkv form (fp32 scale, eps on the scale, true division).
// Row r of `rows` rows: source x + src_off(r) (H bf16, 16-byte aligned when VEC), codes at
// y + r * (H + tail) followed by the scale.
// CH: 16-byte chunks per lane the row is held in (H <= 512 CH when vec): the register
// budget, and with it the number of rows in flight per CU, follows the row length.
template <int SCALE, int CH>
__device__ __forceinline__ void quant_row(const uint16_t* __restrict__ xr, uint8_t* __restrict__ yr,
                                          int H, bool vec, int lane) {
  const int nchunks = H >> 3;
  uint4 v[CH];
  float amax = 0.0f;
  if (vec) {
    const uint4* xv = reinterpret_cast<const uint4*>(xr);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = c * 64 + lane;
      if (c * 64 < nchunks) {  // wave-uniform: whole groups of 64 chunks
        v[c] = idx < nchunks ? xv[idx] : make_uint4(0, 0, 0, 0);
        uint32_t m = 0;
        m = absmax2(m, v[c].x);
        m = absmax2(m, v[c].y);
        m = absmax2(m, v[c].z);
        m = absmax2(m, v[c].w);
        amax = fmaxf(amax, __uint_as_float(fold2(m) << 16));
      }
    }
  } else {
    for (int k = lane; k < H; k += 64) amax = fmaxf(amax, __uint_as_float((uint32_t)(xr[k] & 0x7fffu) << 16));
  }
  amax = wave_max_f32_nonneg(amax);
  // (a NaN in the row has the largest bit pattern and arrives here as the amax)
  const bool finite_row = (__float_as_uint(amax) & 0x7fffffffu) < 0x7f800000u;
  float scale, inv = 0.0f;
  bool plain;  // wave-uniform: the clamp is a no-op and, for SCALE 1, the fast division is exact
  if constexpr (SCALE == 0) {
    amax = fmaxf(amax, 1e-4f);
    scale = amax / kFp8Max;
    inv = 1.0f / scale;
    // |x| <= amax: |x * inv| <= 448 (1 + 2^-22) < 464, where the conversion still rounds to 448
    plain = finite_row;
  } else {
    const float raw = amax / kFp8Max;
    scale = fmaxf(raw, 1e-6f);
    inv = 1.0f / scale;
    // scale = fl(amax / 448) inside the window: the case the fast division is proven on
    // (tests/native/divcheck.c, fp32 scales); a floored scale takes the compiler's division
    plain = finite_row && scale == raw && scale_in_fast_window(scale);
  }
  auto q = [&](float x) {
    if (plain) return SCALE == 0 ? x * inv : div_scale<true>(x, scale, inv);
    const float y = SCALE == 0 ? x * inv : x / scale;
    return y != y ? y : fminf(fmaxf(y, -kFp8Max), kFp8Max);
  };
  const int sh = (int)(reinterpret_cast<uintptr_t>(yr) & 7);  // wave-uniform
  if (vec && (sh == 2 || sh == 4 || sh == 6)) {
    // The row starts sh bytes behind an 8-byte boundary (the pitch H + 2 or D + 4 is not a
    // multiple of 8): piece by piece 2- or 4-byte stores would quadruple the store count.
    // The byte stream is shifted instead: the aligned 8-byte word k of the row holds the
    // last sh bytes of piece k-1 and the first 8 - sh of piece k; a lane gets its left
    // neighbour's piece with a wavefront shift (DPP), lane 0 the last piece of the previous
    // group of 64 through a scalar. Only the first 8 - sh bytes of the row and its last sh
    // bytes go out in 2-byte stores.
    uint8_t* const base = yr - sh;
    uint32_t carry_lo = 0, carry_hi = 0;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = c * 64 + lane;
      if (c * 64 < nchunks) {
        uint32_t lo = 0, hi = 0;
        if (idx < nchunks) {
          lo = cvt4_fp8(q(bf16_lo(v[c].x)), q(bf16_hi(v[c].x)), q(bf16_lo(v[c].y)), q(bf16_hi(v[c].y)));
          hi = cvt4_fp8(q(bf16_lo(v[c].z)), q(bf16_hi(v[c].z)), q(bf16_lo(v[c].w)), q(bf16_hi(v[c].w)));
        }
        // wave_shr:1 -- lane l takes lane l-1, lane 0 keeps the first operand
        const uint32_t plo = (uint32_t)__builtin_amdgcn_update_dpp((int)carry_lo, (int)lo, 0x138, 0xf, 0xf, false);
        const uint32_t phi = (uint32_t)__builtin_amdgcn_update_dpp((int)carry_hi, (int)hi, 0x138, 0xf, 0xf, false);
        uint32_t wlo, whi;
        if (sh == 2) {
          wlo = __builtin_amdgcn_alignbyte(lo, phi, 2);
          whi = __builtin_amdgcn_alignbyte(hi, lo, 2);
        } else if (sh == 4) {
          wlo = phi;
          whi = lo;
        } else {
          wlo = __builtin_amdgcn_alignbyte(phi, plo, 2);
          whi = __builtin_amdgcn_alignbyte(lo, phi, 2);
        }
        if (idx > 0 && idx < nchunks) *reinterpret_cast<uint2*>(base + 8 * (int64_t)idx) = uint2{wlo, whi};
        const uint16_t hw[4] = {(uint16_t)lo, (uint16_t)(lo >> 16), (uint16_t)hi, (uint16_t)(hi >> 16)};
        if (idx == 0) {  // head of the row: its first 8 - sh bytes
#pragma unroll
          for (int j = 0; j < 3; ++j)
            if (2 * j < 8 - sh) reinterpret_cast<uint16_t*>(yr)[j] = hw[j];
        }
        if (idx == nchunks - 1) {  // tail: the last sh bytes of the last piece
          uint16_t* t = reinterpret_cast<uint16_t*>(base + 8 * (int64_t)nchunks);
#pragma unroll
          for (int j = 1; j < 4; ++j)
            if (2 * j >= 8 - sh) t[j - (8 - sh) / 2] = hw[j];
        }
        carry_lo = (uint32_t)__builtin_amdgcn_readlane((int)lo, 63);
        carry_hi = (uint32_t)__builtin_amdgcn_readlane((int)hi, 63);
      }
    }
  } else if (vec) {
    const int al = align_of(yr);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = c * 64 + lane;
      if (c * 64 < nchunks && idx < nchunks) {
        const uint32_t lo = cvt4_fp8(q(bf16_lo(v[c].x)), q(bf16_hi(v[c].x)), q(bf16_lo(v[c].y)),
                                     q(bf16_hi(v[c].y)));
        const uint32_t hi = cvt4_fp8(q(bf16_lo(v[c].z)), q(bf16_hi(v[c].z)), q(bf16_lo(v[c].w)),
                                     q(bf16_hi(v[c].w)));
        store8(yr + 8 * idx, lo, hi, al);
      }
    }
  } else {
    for (int k = lane; k < H; k += 64) {
      const float y = q(__uint_as_float((uint32_t)xr[k] << 16));
      yr[k] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(y, y, 0u, false) & 0xffu);
    }
  }
  if (lane == 0) {
    if constexpr (SCALE == 0) {
      const uint16_t s16 = (uint16_t)(__float_as_uint(round_to_bf16(scale)) >> 16);
      yr[H] = (uint8_t)s16;  // byte stores: the row end is only 1-byte aligned for odd H
      yr[H + 1] = (uint8_t)(s16 >> 8);
    } else {
      const uint32_t s32 = __float_as_uint(scale);
#pragma unroll
      for (int b = 0; b < 4; ++b) yr[H + b] = (uint8_t)(s32 >> (8 * b));
    }
  }
}

// codes (+ trailing scale) -> bf16 row. SCALE as above (only the scale's format differs).
template <int SCALE>
__device__ __forceinline__ void dequant_row(const uint8_t* __restrict__ xr, uint16_t* __restrict__ yr,
                                            int H, bool vec, int lane) {
  float scale;
  if constexpr (SCALE == 0) {
    scale = __uint_as_float(((uint32_t)xr[H] | ((uint32_t)xr[H + 1] << 8)) << 16);
  } else {
    scale = __uint_as_float((uint32_t)xr[H] | ((uint32_t)xr[H + 1] << 8) | ((uint32_t)xr[H + 2] << 16) |
                            ((uint32_t)xr[H + 3] << 24));
  }
  auto de = [&](uint32_t w, int byte) {  // one code -> scaled fp32
    float f;
    switch (byte) {
      case 0: f = __builtin_amdgcn_cvt_f32_fp8((int)w, 0); break;
      case 1: f = __builtin_amdgcn_cvt_f32_fp8((int)w, 1); break;
      case 2: f = __builtin_amdgcn_cvt_f32_fp8((int)w, 2); break;
      default: f = __builtin_amdgcn_cvt_f32_fp8((int)w, 3); break;
    }
    return f * scale;
  };
  if (vec) {
    const int al = align_of(xr);
    uint4* yv = reinterpret_cast<uint4*>(yr);
    for (int idx = lane; idx < (H >> 3); idx += 64) {
      const uint2 w = load8(xr + 8 * idx, al);
      uint4 o;
      o.x = (f32_to_bf16_bits_rne(de(w.x, 0))) | (f32_to_bf16_bits_rne(de(w.x, 1)) << 16);
      o.y = (f32_to_bf16_bits_rne(de(w.x, 2))) | (f32_to_bf16_bits_rne(de(w.x, 3)) << 16);
      o.z = (f32_to_bf16_bits_rne(de(w.y, 0))) | (f32_to_bf16_bits_rne(de(w.y, 1)) << 16);
      o.w = (f32_to_bf16_bits_rne(de(w.y, 2))) | (f32_to_bf16_bits_rne(de(w.y, 3)) << 16);
      yv[idx] = o;
    }
  } else {
    for (int k = lane; k < H; k += 64) {
      const float f = __builtin_amdgcn_cvt_f32_fp8((int)xr[k], 0) * scale;
      yr[k] = (uint16_t)f32_to_bf16_bits_rne(f);
    }
  }
}

template <int CH>
__global__ __launch_bounds__(64) void comm_per_token_quant(const uint16_t* __restrict__ x,
                                                           uint8_t* __restrict__ y, int64_t M, int H,
                                                           bool vec) {
  const int lane = threadIdx.x;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x)
    quant_row<0, CH>(x + row * H, y + row * (H + 2), H, vec, lane);
}

__global__ __launch_bounds__(64) void comm_per_token_dequant(const uint8_t* __restrict__ x,
                                                             uint16_t* __restrict__ y, int64_t M,
                                                             int H, bool vec) {
  const int lane = threadIdx.x;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x)
    dequant_row<0>(x + row * (H + 2), y + row * H, H, vec, lane);
}

// One wavefront per head row. Output row index r = ((p * S + s) * B + b) * N + n of
// [P,S,B,N,D+4]; the source row is x[b,s,p,n,:] (element strides for b, s, p; heads and
// channels contiguous, as the reference kernel assumes).
template <int CH>
__global__ __launch_bounds__(64) void comm_qkv_permute_quant(
    const uint16_t* __restrict__ x, uint8_t* __restrict__ y, uint32_t rows, FastDiv dN, FastDiv dB,
    FastDiv dS, int D, int64_t sb, int64_t ss, int64_t sp, bool vec) {
  const int lane = threadIdx.x;
  for (uint32_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const uint32_t t = fd_div(r, dN), n = r - t * dN.d;
    const uint32_t u = fd_div(t, dB), b = t - u * dB.d;
    const uint32_t p = fd_div(u, dS), s = u - p * dS.d;
    quant_row<1, CH>(x + b * sb + s * ss + p * sp + (int64_t)n * D, y + (int64_t)r * (D + 4), D, vec, lane);
  }
}

// quant_x [S,B,N,D+4] (byte strides for s, b, n) -> x [B,S,N,D] contiguous bf16.
__global__ __launch_bounds__(64) void comm_qkv_permute_dequant(
    const uint8_t* __restrict__ qx, uint16_t* __restrict__ x, uint32_t rows, FastDiv dN, FastDiv dS,
    int D, int64_t qs, int64_t qb, int64_t qn, bool vec) {
  const int lane = threadIdx.x;
  for (uint32_t r = blockIdx.x; r < rows; r += gridDim.x) {  // r = (b * S + s) * N + n
    const uint32_t t = fd_div(r, dN), n = r - t * dN.d;
    const uint32_t b = fd_div(t, dS), s = t - b * dS.d;
    dequant_row<1>(qx + s * qs + b * qb + n * qn, x + (int64_t)r * D, D, vec, lane);
  }
}

// Head rows are short (D = 64 .. 256): with one lane per 16-byte chunk a row only needs
// G = D / 8 lanes (rounded up to a power of two), so a wavefront takes 64 / G rows at a
// time and the amax is reduced inside each group of G lanes.
template <int G>
__global__ __launch_bounds__(64) void comm_qkv_permute_quant_grouped(
    const uint16_t* __restrict__ x, uint8_t* __restrict__ y, uint32_t rows, FastDiv dN, FastDiv dB,
    FastDiv dS, int D, int64_t sb, int64_t ss, int64_t sp) {
  constexpr int RPW = 64 / G;  // rows per wavefront
  const int lane = threadIdx.x, j = lane % G, sub = lane / G;
  const int nchunks = D >> 3;
  for (uint32_t r0 = blockIdx.x * RPW; r0 < rows; r0 += gridDim.x * RPW) {
    const uint32_t r = r0 + sub;
    const bool row_ok = r < rows, active = row_ok && j < nchunks;
    const uint32_t rc = row_ok ? r : rows - 1;
    const uint32_t t = fd_div(rc, dN), n = rc - t * dN.d;
    const uint32_t u = fd_div(t, dB), b = t - u * dB.d;
    const uint32_t p = fd_div(u, dS), s = u - p * dS.d;
    const uint16_t* xr = x + b * sb + s * ss + p * sp + (int64_t)n * D;
    const uint4 v = active ? reinterpret_cast<const uint4*>(xr)[j] : make_uint4(0, 0, 0, 0);
    uint32_t m = 0;
    m = absmax2(m, v.x);
    m = absmax2(m, v.y);
    m = absmax2(m, v.z);
    m = absmax2(m, v.w);
    const uint32_t mbits = group_max_u32<G>(fold2(m));  // bf16 pattern of the row's max |x|
    const float raw = __uint_as_float(mbits << 16) / kFp8Max;
    const float scale = fmaxf(raw, 1e-6f);
    const float inv = 1.0f / scale;
    // The proven fast division where every row of the wavefront has a finite amax and an
    // unfloored scale inside the window (scale = fl(amax / 448); tests/native/divcheck.c),
    // the compiler's division and the clamp for the whole wavefront otherwise.
    const bool plain = mbits < 0x7f80u && scale == raw && scale_in_fast_window(scale);
    uint32_t lo, hi;
    if (__builtin_amdgcn_ballot_w64(!plain) == 0) {
      auto q = [&](float f) { return div_scale<true>(f, scale, inv); };
      lo = cvt4_fp8(q(bf16_lo(v.x)), q(bf16_hi(v.x)), q(bf16_lo(v.y)), q(bf16_hi(v.y)));
      hi = cvt4_fp8(q(bf16_lo(v.z)), q(bf16_hi(v.z)), q(bf16_lo(v.w)), q(bf16_hi(v.w)));
    } else {
      auto q = [&](float f) {
        const float yv = f / scale;
        return yv != yv ? yv : fminf(fmaxf(yv, -kFp8Max), kFp8Max);
      };
      lo = cvt4_fp8(q(bf16_lo(v.x)), q(bf16_hi(v.x)), q(bf16_lo(v.y)), q(bf16_hi(v.y)));
      hi = cvt4_fp8(q(bf16_lo(v.z)), q(bf16_hi(v.z)), q(bf16_lo(v.w)), q(bf16_hi(v.w)));
    }
    if (active) {
      uint8_t* yr = y + (int64_t)rc * (D + 4);  // 4-byte aligned: D % 8 == 0 and y is
      reinterpret_cast<uint32_t*>(yr + 8 * j)[0] = lo;
      reinterpret_cast<uint32_t*>(yr + 8 * j)[1] = hi;
      if (j == 0) *reinterpret_cast<float*>(yr + D) = scale;
    }
  }
}

template <int G>
__global__ __launch_bounds__(64) void comm_qkv_permute_dequant_grouped(
    const uint8_t* __restrict__ qx, uint16_t* __restrict__ x, uint32_t rows, FastDiv dN, FastDiv dS,
    int D, int64_t qs, int64_t qb, int64_t qn) {
  constexpr int RPW = 64 / G;
  const int lane = threadIdx.x, j = lane % G, sub = lane / G;
  const int nchunks = D >> 3;
  for (uint32_t r0 = blockIdx.x * RPW; r0 < rows; r0 += gridDim.x * RPW) {
    const uint32_t r = r0 + sub;  // (b * S + s) * N + n
    if (r >= rows || j >= nchunks) continue;
    const uint32_t t = fd_div(r, dN), n = r - t * dN.d;
    const uint32_t b = fd_div(t, dS), s = t - b * dS.d;
    const uint8_t* xr = qx + s * qs + b * qb + n * qn;
    const float scale = *reinterpret_cast<const float*>(xr + D);
    const uint32_t w0 = reinterpret_cast<const uint32_t*>(xr + 8 * j)[0];
    const uint32_t w1 = reinterpret_cast<const uint32_t*>(xr + 8 * j)[1];
    auto pair = [&](float a, float c) {
      return f32_to_bf16_bits_rne(a * scale) | (f32_to_bf16_bits_rne(c * scale) << 16);
    };
    uint4 o;
    o.x = pair(__builtin_amdgcn_cvt_f32_fp8((int)w0, 0), __builtin_amdgcn_cvt_f32_fp8((int)w0, 1));
    o.y = pair(__builtin_amdgcn_cvt_f32_fp8((int)w0, 2), __builtin_amdgcn_cvt_f32_fp8((int)w0, 3));
    o.z = pair(__builtin_amdgcn_cvt_f32_fp8((int)w1, 0), __builtin_amdgcn_cvt_f32_fp8((int)w1, 1));
    o.w = pair(__builtin_amdgcn_cvt_f32_fp8((int)w1, 2), __builtin_amdgcn_cvt_f32_fp8((int)w1, 3));
    reinterpret_cast<uint4*>(x + (int64_t)r * D)[j] = o;
  }
}

unsigned grid_for(int64_t rows) {
  const int64_t cap = 256 * 256;  // the grid-stride loops take the rest
  return (unsigned)(rows < cap ? rows : cap);
}

}  // namespace

int launch_comm_per_token_quant(const void* x, int64_t M, int64_t H, void* y, hipStream_t stream) {
  const bool vec = H % 8 == 0 && H <= kMaxChunks * 512 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(y) % 2 == 0;
  const int need = vec ? (int)((H + 511) / 512) : 1;
#define CDIT_PT_Q(CH)                                                                          \
  if (need <= CH) {                                                                            \
    hipLaunchKernelGGL(comm_per_token_quant<CH>, dim3(grid_for(M)), dim3(64), 0, stream,        \
                       static_cast<const uint16_t*>(x), static_cast<uint8_t*>(y), M, (int)H, vec); \
    return 0;                                                                                  \
  }
  CDIT_PT_Q(1) CDIT_PT_Q(2) CDIT_PT_Q(4) CDIT_PT_Q(6) CDIT_PT_Q(8) CDIT_PT_Q(12) CDIT_PT_Q(16)
  CDIT_PT_Q(24) CDIT_PT_Q(32)
#undef CDIT_PT_Q
  return 0;
}

int launch_comm_per_token_dequant(const void* x, int64_t M, int64_t H, void* y, hipStream_t stream) {
  const bool vec = H % 8 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(x) % 2 == 0;
  hipLaunchKernelGGL(comm_per_token_dequant, dim3(grid_for(M)), dim3(64), 0, stream,
                     static_cast<const uint8_t*>(x), static_cast<uint16_t*>(y), M, (int)H, vec);
  return 0;
}

int launch_comm_qkv_permute_quant(const void* x, int B, int S, int P, int N, int D, int64_t sb,
                                  int64_t ss, int64_t sp, void* y, hipStream_t stream) {
  const bool vec = D % 8 == 0 && D <= kMaxChunks * 512 && sb % 8 == 0 && ss % 8 == 0 && sp % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 4 == 0;
  const int64_t rows = (int64_t)P * S * B * N;
  if (rows >= (int64_t)1 << 31) {
    set_error("cdit_fp8_comm_qkv_permute_quant: %lld head rows, at most 2^31 - 1", (long long)rows);
    return CDIT_EINVAL;
  }
  const FastDiv dN = make_fastdiv((uint32_t)N), dB = make_fastdiv((uint32_t)B), dS = make_fastdiv((uint32_t)S);
  if (vec && D <= 256) {
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    uint8_t* yp = static_cast<uint8_t*>(y);
#define CDIT_QKV_Q(G)                                                                            \
  hipLaunchKernelGGL(comm_qkv_permute_quant_grouped<G>, dim3(grid_for((rows + 64 / G - 1) / (64 / G))), \
                     dim3(64), 0, stream, xp, yp, (uint32_t)rows, dN, dB, dS, D, sb, ss, sp)
    if (D <= 64) CDIT_QKV_Q(8);
    else if (D <= 128) CDIT_QKV_Q(16);
    else CDIT_QKV_Q(32);
#undef CDIT_QKV_Q
    return 0;
  }
  const int need = vec ? (D + 511) / 512 : 1;
#define CDIT_QKV_ROW(CH)                                                                          \
  if (need <= CH) {                                                                               \
    hipLaunchKernelGGL(comm_qkv_permute_quant<CH>, dim3(grid_for(rows)), dim3(64), 0, stream,      \
                       static_cast<const uint16_t*>(x), static_cast<uint8_t*>(y), (uint32_t)rows,  \
                       dN, dB, dS, D, sb, ss, sp, vec);                                           \
    return 0;                                                                                     \
  }
  CDIT_QKV_ROW(1) CDIT_QKV_ROW(4) CDIT_QKV_ROW(32)
#undef CDIT_QKV_ROW
  return 0;
}

int launch_comm_qkv_permute_dequant(const void* qx, int S, int B, int N, int D, int64_t qs, int64_t qb,
                                    int64_t qn, void* x, hipStream_t stream) {
  const bool vec = D % 8 == 0 && qs % 4 == 0 && qb % 4 == 0 && qn % 4 == 0 &&
                   reinterpret_cast<uintptr_t>(qx) % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0;
  const int64_t rows = (int64_t)B * S * N;
  if (rows >= (int64_t)1 << 31) {
    set_error("cdit_fp8_comm_qkv_permute_dequant: %lld head rows, at most 2^31 - 1", (long long)rows);
    return CDIT_EINVAL;
  }
  const FastDiv dN = make_fastdiv((uint32_t)N), dS = make_fastdiv((uint32_t)S);
  if (vec && D <= 256) {
    const uint8_t* qp = static_cast<const uint8_t*>(qx);
    uint16_t* xp = static_cast<uint16_t*>(x);
#define CDIT_QKV_D(G)                                                                              \
  hipLaunchKernelGGL(comm_qkv_permute_dequant_grouped<G>, dim3(grid_for((rows + 64 / G - 1) / (64 / G))), \
                     dim3(64), 0, stream, qp, xp, (uint32_t)rows, dN, dS, D, qs, qb, qn)
    if (D <= 64) CDIT_QKV_D(8);
    else if (D <= 128) CDIT_QKV_D(16);
    else CDIT_QKV_D(32);
#undef CDIT_QKV_D
    return 0;
  }
  hipLaunchKernelGGL(comm_qkv_permute_dequant, dim3(grid_for(rows)), dim3(64), 0, stream,
                     static_cast<const uint8_t*>(qx), static_cast<uint16_t*>(x), (uint32_t)rows, dN, dS, D,
                     qs, qb, qn, vec);
  return 0;
}

}  // namespace cdit
