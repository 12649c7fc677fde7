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
// floors, where the scale is rounded) and shares none of its contract; where a row's scale
// is amax / 448 unfloored, the qkv form's true division is the GEMM path's proven exact
// fast division (quant_device.h), and the clamp, which cannot act on |x| <= amax, is left
// out; rows with a floored scale, a NaN or an infinity take the literal form.
//
// All four are pure HBM streaming: one 64-lane wavefront per row (several head rows per
// wavefront for D <= 256), the row read once and kept in registers between the amax and
// the cast. Rows with a pitch of H + 2 (or D + 4) bytes start on 2- (4-) byte boundaries:
// the row kernels move them as aligned 8-byte words of a byte stream shifted through the
// neighbouring lane, with buffer accesses whose descriptor drops what lies beyond the row
// (no branch per lane). Row indices of the permuted layouts are split with multiply-high
// by launch constants instead of 64-bit divisions.
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
typedef unsigned int u4v __attribute__((ext_vector_type(4)));
typedef unsigned int u2v __attribute__((ext_vector_type(2)));
constexpr uint32_t kBeyond = 0x80000000u;  // a lane offset beyond any descriptor: nothing moves
constexpr int kWrittenOnce = 2;            // non-temporal stores: the codes are read by another engine

__device__ __forceinline__ __amdgpu_buffer_rsrc_t bytes_buf(const void* base, int bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}

// The codes of a row whose clamp cannot act (`plain` in quant_row), written without a branch
// per lane: buffer stores whose descriptor covers the row, lanes without a piece get an
// offset beyond it. SH = the row's start modulo 8 (0, 2, 4, 6). For SH > 0 the byte stream is
// shifted: the aligned 8-byte word k of the row holds the last SH bytes of piece k-1 and the
// first 8 - SH of piece k; a lane gets its left neighbour's piece with a wavefront shift (DPP),
// lane 0 the last piece of the previous group of 64 through a scalar. Only the first 8 - SH
// bytes of the row and its last SH bytes go out in 2- and 4-byte stores.
template <int SCALE, int CH, int SH>
__device__ __forceinline__ void store_codes_plain(const uint4 (&v)[CH], uint8_t* __restrict__ yr, int H,
                                                  float scale, float inv, Recip rc, int lane) {
  const int nchunks = H >> 3;
  const __amdgpu_buffer_rsrc_t rb = bytes_buf(yr - SH, SH + H);
  auto q = [&](float x) { return SCALE == 0 ? x * inv : div_scale<true>(x, scale, rc); };
  uint32_t carry_lo = 0, carry_hi = 0;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    if (c * 64 < nchunks) {  // wave-uniform: whole groups of 64 chunks
      const int idx = c * 64 + lane;
      const uint32_t lo = cvt4_fp8(q(bf16_lo(v[c].x)), q(bf16_hi(v[c].x)), q(bf16_lo(v[c].y)), q(bf16_hi(v[c].y)));
      const uint32_t hi = cvt4_fp8(q(bf16_lo(v[c].z)), q(bf16_hi(v[c].z)), q(bf16_lo(v[c].w)), q(bf16_hi(v[c].w)));
      if constexpr (SH == 0) {
        __builtin_amdgcn_raw_buffer_store_b64(u2v{lo, hi}, rb, idx < nchunks ? 8 * idx : kBeyond, 0, kWrittenOnce);
      } else {
        // wave_shr:1 -- lane l takes lane l-1, lane 0 keeps the first operand
        const uint32_t plo = (uint32_t)__builtin_amdgcn_update_dpp((int)carry_lo, (int)lo, 0x138, 0xf, 0xf, false);
        const uint32_t phi = (uint32_t)__builtin_amdgcn_update_dpp((int)carry_hi, (int)hi, 0x138, 0xf, 0xf, false);
        uint32_t wlo, whi;
        if constexpr (SH == 2) {
          wlo = __builtin_amdgcn_alignbyte(lo, phi, 2);
          whi = __builtin_amdgcn_alignbyte(hi, lo, 2);
        } else if constexpr (SH == 4) {
          wlo = phi;
          whi = lo;
        } else {
          wlo = __builtin_amdgcn_alignbyte(phi, plo, 2);
          whi = __builtin_amdgcn_alignbyte(lo, phi, 2);
        }
        __builtin_amdgcn_raw_buffer_store_b64(u2v{wlo, whi}, rb, idx > 0 && idx < nchunks ? 8 * idx : kBeyond, 0,
                                              kWrittenOnce);
        if (c == 0) {  // head of the row: the first 8 - SH bytes of piece 0, from lane 0
          const uint32_t mid = __builtin_amdgcn_alignbyte(hi, lo, 2);  // bytes 2..5 of the piece
          if constexpr (SH == 2) {
            __builtin_amdgcn_raw_buffer_store_b16((uint16_t)lo, rb, lane == 0 ? 2 : kBeyond, 0, 0);
            __builtin_amdgcn_raw_buffer_store_b32(mid, rb, lane == 0 ? 4 : kBeyond, 0, 0);
          } else if constexpr (SH == 4) {
            __builtin_amdgcn_raw_buffer_store_b32(lo, rb, lane == 0 ? 4 : kBeyond, 0, 0);
          } else {
            __builtin_amdgcn_raw_buffer_store_b16((uint16_t)lo, rb, lane == 0 ? 6 : kBeyond, 0, 0);
          }
        }
        if (c == (nchunks - 1) >> 6) {  // wave-uniform: the group with the last piece; its last SH bytes
          const uint32_t off = idx == nchunks - 1 ? 8 * nchunks : kBeyond;
          if constexpr (SH == 2) {
            __builtin_amdgcn_raw_buffer_store_b16((uint16_t)(hi >> 16), rb, off, 0, 0);
          } else if constexpr (SH == 4) {
            __builtin_amdgcn_raw_buffer_store_b32(hi, rb, off, 0, 0);
          } else {
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_amdgcn_alignbyte(hi, lo, 2), rb, off, 0, 0);
            __builtin_amdgcn_raw_buffer_store_b16((uint16_t)(hi >> 16), rb, off + 4, 0, 0);
          }
        }
        carry_lo = (uint32_t)__builtin_amdgcn_readlane((int)lo, 63);
        carry_hi = (uint32_t)__builtin_amdgcn_readlane((int)hi, 63);
      }
    }
  }
}

template <int SCALE, int CH>
__device__ __forceinline__ void quant_row(const uint16_t* __restrict__ xr, uint8_t* __restrict__ yr,
                                          int H, bool vec, int lane) {
  const int nchunks = H >> 3;
  uint4 v[CH];
  float amax = 0.0f;
  if (vec) {
    const __amdgpu_buffer_rsrc_t xb = bytes_buf(xr, H * 2);  // beyond the row: zeros
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = c * 64 + lane;
      v[c] = make_uint4(0, 0, 0, 0);
      if (c * 64 < nchunks) {  // wave-uniform: whole groups of 64 chunks
        const u4v t = __builtin_amdgcn_raw_buffer_load_b128(xb, 16 * idx, 0, 0);
        v[c] = make_uint4(t[0], t[1], t[2], t[3]);
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
  Recip rc{};
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
    rc = make_recip(scale);
    // scale = fl(amax / 448) inside the window: the case the fast division is proven on
    // (tests/native/divcheck.c, fp32 scales); a floored scale takes the compiler's division
    plain = finite_row && scale == raw && scale_in_fast_window(scale);
  }
  auto q = [&](float x) {
    if (plain) return SCALE == 0 ? x * inv : div_scale<true>(x, scale, rc);
    const float y = SCALE == 0 ? x * inv : x / scale;
    return y != y ? y : fminf(fmaxf(y, -kFp8Max), kFp8Max);
  };
  const int sh = (int)(reinterpret_cast<uintptr_t>(yr) & 7);  // wave-uniform
  if (vec && plain && (sh & 1) == 0) {
    switch (sh) {
      case 0: store_codes_plain<SCALE, CH, 0>(v, yr, H, scale, inv, rc, lane); break;
      case 2: store_codes_plain<SCALE, CH, 2>(v, yr, H, scale, inv, rc, lane); break;
      case 4: store_codes_plain<SCALE, CH, 4>(v, yr, H, scale, inv, rc, lane); break;
      default: store_codes_plain<SCALE, CH, 6>(v, yr, H, scale, inv, rc, lane); break;
    }
    // the scale behind the codes, from lane 0 (H is even here: 2- resp. 4-byte aligned)
    const __amdgpu_buffer_rsrc_t sb = bytes_buf(yr + H, 4);
    if constexpr (SCALE == 0) {
      __builtin_amdgcn_raw_buffer_store_b16((uint16_t)(__float_as_uint(round_to_bf16(scale)) >> 16), sb,
                                            lane == 0 ? 0 : kBeyond, 0, 0);
    } else {
      if ((reinterpret_cast<uintptr_t>(yr + H) & 3) == 0) {
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(scale), sb, lane == 0 ? 0 : kBeyond, 0, 0);
      } else {
        __builtin_amdgcn_raw_buffer_store_b16((uint16_t)__float_as_uint(scale), sb, lane == 0 ? 0 : kBeyond, 0, 0);
        __builtin_amdgcn_raw_buffer_store_b16((uint16_t)(__float_as_uint(scale) >> 16), sb,
                                              lane == 0 ? 2 : kBeyond, 0, 0);
      }
    }
    return;
  }
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

// 8 codes -> 8 bf16 (four packed words), value = code * scale rounded to nearest even by the
// packed hardware conversion. A NaN code (0x7f, 0xff) gives a bf16 NaN; which NaN is not
// specified (the reference's Triton kernel and PyTorch's CPU conversion differ there too).
__device__ __forceinline__ u4v dequant8(uint32_t w0, uint32_t w1, float scale) {
  const float f[8] = {__builtin_amdgcn_cvt_f32_fp8((int)w0, 0) * scale, __builtin_amdgcn_cvt_f32_fp8((int)w0, 1) * scale,
                      __builtin_amdgcn_cvt_f32_fp8((int)w0, 2) * scale, __builtin_amdgcn_cvt_f32_fp8((int)w0, 3) * scale,
                      __builtin_amdgcn_cvt_f32_fp8((int)w1, 0) * scale, __builtin_amdgcn_cvt_f32_fp8((int)w1, 1) * scale,
                      __builtin_amdgcn_cvt_f32_fp8((int)w1, 2) * scale, __builtin_amdgcn_cvt_f32_fp8((int)w1, 3) * scale};
  u4v o;
#pragma unroll
  for (int k = 0; k < 4; ++k) o[k] = pk_bf16(f[2 * k], f[2 * k + 1]);
  return o;
}

// Row of H codes (H % 8 == 0) that starts SH bytes behind an 8-byte boundary, scale behind it,
// to a 16-byte aligned bf16 row, without a branch per lane: aligned 8-byte buffer loads of
// the row's words (zeros beyond the row), each lane takes its right neighbour's word with a
// wavefront shift (DPP; lane 63 the first word of the next group through a scalar) and cuts
// its piece out of the two; 16-byte buffer stores, lanes beyond the row dropped. CH groups of
// 64 pieces (H <= 512 CH).
template <int SCALE, int CH, int SH>
__device__ __forceinline__ void dequant_row_aligned(const uint8_t* __restrict__ xr, uint16_t* __restrict__ yr,
                                                    int H, float scale, int lane) {
  const int nchunks = H >> 3;
  // (the descriptor reaches over the scale behind the codes, so that the word with the row's
  // last SH bytes is inside it whole)
  const __amdgpu_buffer_rsrc_t xb = bytes_buf(xr - SH, SH + H + (SCALE == 0 ? 2 : 4));
  const __amdgpu_buffer_rsrc_t yb = bytes_buf(yr, H * 2);
  u2v w[CH + 1];
#pragma unroll
  for (int c = 0; c <= CH; ++c) {
    w[c] = u2v{0u, 0u};
    if (c * 64 <= nchunks)  // wave-uniform (the group after the last piece holds its last SH bytes)
      w[c] = __builtin_amdgcn_raw_buffer_load_b64(xb, 8 * (c * 64 + lane), 0, 0);
  }
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    if (c * 64 < nchunks) {
      uint32_t lo = w[c][0], hi = w[c][1];
      if constexpr (SH != 0) {
        // wave_shl:1 -- lane l takes lane l+1, lane 63 keeps the first operand
        const int first_lo = __builtin_amdgcn_readlane((int)w[c + 1][0], 0);
        const int first_hi = __builtin_amdgcn_readlane((int)w[c + 1][1], 0);
        const uint32_t nlo = (uint32_t)__builtin_amdgcn_update_dpp(first_lo, (int)w[c][0], 0x130, 0xf, 0xf, false);
        const uint32_t nhi = (uint32_t)__builtin_amdgcn_update_dpp(first_hi, (int)w[c][1], 0x130, 0xf, 0xf, false);
        if constexpr (SH == 2) {
          lo = __builtin_amdgcn_alignbyte(w[c][1], w[c][0], 2);
          hi = __builtin_amdgcn_alignbyte(nlo, w[c][1], 2);
        } else if constexpr (SH == 4) {
          lo = w[c][1];
          hi = nlo;
        } else {
          lo = __builtin_amdgcn_alignbyte(nlo, w[c][1], 2);
          hi = __builtin_amdgcn_alignbyte(nhi, nlo, 2);
        }
      }
      const u4v o = dequant8(lo, hi, scale);
      const int idx = c * 64 + lane;
      __builtin_amdgcn_raw_buffer_store_b128(o, yb, idx < nchunks ? 16 * idx : kBeyond, 0, 0);
    }
  }
}

// codes (+ trailing scale) -> bf16 row. SCALE as above (only the scale's format differs).
// CH > 0: rows of up to 512 CH codes take the branch-free form when `vec`.
template <int SCALE, int CH = 0>
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
  if constexpr (CH > 0) {
    const int sh = (int)(reinterpret_cast<uintptr_t>(xr) & 7);  // wave-uniform
    if (vec && (sh & 1) == 0 && H <= 512 * CH) {
      switch (sh) {
        case 0: dequant_row_aligned<SCALE, CH, 0>(xr, yr, H, scale, lane); break;
        case 2: dequant_row_aligned<SCALE, CH, 2>(xr, yr, H, scale, lane); break;
        case 4: dequant_row_aligned<SCALE, CH, 4>(xr, yr, H, scale, lane); break;
        default: dequant_row_aligned<SCALE, CH, 6>(xr, yr, H, scale, lane); break;
      }
      return;
    }
  }
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

template <int CH>
__global__ __launch_bounds__(64) void comm_per_token_dequant(const uint8_t* __restrict__ x,
                                                             uint16_t* __restrict__ y, int64_t M,
                                                             int H, bool vec) {
  const int lane = threadIdx.x;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x)
    dequant_row<0, CH>(x + row * (H + 2), y + row * H, H, vec, lane);
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
constexpr int kGroupedWaves = 4;   // wavefronts per workgroup of the grouped kernels
constexpr int kGroupedUnroll = 4;  // groups of 64 / G rows a wavefront of the grouped kernels takes per pass

template <int G>
__global__ __launch_bounds__(64 * kGroupedWaves) void comm_qkv_permute_quant_grouped(
    const uint16_t* __restrict__ x, uint8_t* __restrict__ y, uint32_t rows, FastDiv dN, FastDiv dB,
    FastDiv dS, int D, int64_t sb, int64_t ss, int64_t sp) {
  constexpr int RPW = 64 / G;  // rows per wavefront
  const int lane = threadIdx.x & 63, j = lane % G, sub = lane / G;
  const int nchunks = D >> 3;
  const uint32_t wave = blockIdx.x * kGroupedWaves + (threadIdx.x >> 6), nwaves = gridDim.x * kGroupedWaves;
  // kGroupedUnroll groups of RPW rows per pass, all their loads in flight before the first is used
  for (uint32_t r0 = wave * (RPW * kGroupedUnroll); r0 < rows; r0 += nwaves * (RPW * kGroupedUnroll)) {
    uint4 v[kGroupedUnroll];
#pragma unroll
    for (int u = 0; u < kGroupedUnroll; ++u) {
      const uint32_t r = r0 + u * RPW + sub;
      const uint32_t rc = r < rows ? r : rows - 1;
      const uint32_t t = fd_div(rc, dN), n = rc - t * dN.d;
      const uint32_t w = fd_div(t, dB), b = t - w * dB.d;
      const uint32_t p = fd_div(w, dS), s = w - p * dS.d;
      const uint16_t* xr = x + b * sb + s * ss + p * sp + (int64_t)n * D;
      v[u] = r < rows && j < nchunks ? reinterpret_cast<const uint4*>(xr)[j] : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int u = 0; u < kGroupedUnroll; ++u) {
      const uint32_t r = r0 + u * RPW + sub;
      uint32_t m = 0;
      m = absmax2(m, v[u].x);
      m = absmax2(m, v[u].y);
      m = absmax2(m, v[u].z);
      m = absmax2(m, v[u].w);
      const uint32_t mbits = group_max_u32<G>(fold2(m));  // bf16 pattern of the row's max |x|
      const float raw = __uint_as_float(mbits << 16) / kFp8Max;
      const float scale = fmaxf(raw, 1e-6f);
      const Recip rc = make_recip(scale);
      // The proven fast division where every row of the wavefront has a finite amax and an
      // unfloored scale inside the window (scale = fl(amax / 448); tests/native/divcheck.c),
      // the compiler's division and the clamp for the whole wavefront otherwise.
      const bool plain = mbits < 0x7f80u && scale == raw && scale_in_fast_window(scale);
      uint32_t lo, hi;
      if (__builtin_amdgcn_ballot_w64(!plain) == 0) {
        auto q = [&](float f) { return div_scale<true>(f, scale, rc); };
        lo = cvt4_fp8(q(bf16_lo(v[u].x)), q(bf16_hi(v[u].x)), q(bf16_lo(v[u].y)), q(bf16_hi(v[u].y)));
        hi = cvt4_fp8(q(bf16_lo(v[u].z)), q(bf16_hi(v[u].z)), q(bf16_lo(v[u].w)), q(bf16_hi(v[u].w)));
      } else {
        auto q = [&](float f) {
          const float yv = f / scale;
          return yv != yv ? yv : fminf(fmaxf(yv, -kFp8Max), kFp8Max);
        };
        lo = cvt4_fp8(q(bf16_lo(v[u].x)), q(bf16_hi(v[u].x)), q(bf16_lo(v[u].y)), q(bf16_hi(v[u].y)));
        hi = cvt4_fp8(q(bf16_lo(v[u].z)), q(bf16_hi(v[u].z)), q(bf16_lo(v[u].w)), q(bf16_hi(v[u].w)));
      }
      if (r < rows && j < nchunks) {
        uint8_t* yr = y + (int64_t)r * (D + 4);  // 4-byte aligned: D % 8 == 0 and y is
        reinterpret_cast<uint32_t*>(yr + 8 * j)[0] = lo;
        reinterpret_cast<uint32_t*>(yr + 8 * j)[1] = hi;
        if (j == 0) *reinterpret_cast<float*>(yr + D) = scale;
      }
    }
  }
}

template <int G>
__global__ __launch_bounds__(64 * kGroupedWaves) void comm_qkv_permute_dequant_grouped(
    const uint8_t* __restrict__ qx, uint16_t* __restrict__ x, uint32_t rows, FastDiv dN, FastDiv dS,
    int D, int64_t qs, int64_t qb, int64_t qn) {
  constexpr int RPW = 64 / G;
  const int lane = threadIdx.x & 63, j = lane % G, sub = lane / G;
  const int nchunks = D >> 3;
  const uint32_t wave = blockIdx.x * kGroupedWaves + (threadIdx.x >> 6), nwaves = gridDim.x * kGroupedWaves;
  // kGroupedUnroll groups of RPW rows per pass, all their loads in flight before the first is used
  for (uint32_t r0 = wave * (RPW * kGroupedUnroll); r0 < rows; r0 += nwaves * (RPW * kGroupedUnroll)) {
    uint32_t w0[kGroupedUnroll], w1[kGroupedUnroll];
    float scale[kGroupedUnroll];
    bool active[kGroupedUnroll];
#pragma unroll
    for (int u = 0; u < kGroupedUnroll; ++u) {
      const uint32_t r = r0 + u * RPW + sub;  // (b * S + s) * N + n
      active[u] = r < rows && j < nchunks;
      const uint32_t rc = r < rows ? r : rows - 1;
      const uint32_t t = fd_div(rc, dN), n = rc - t * dN.d;
      const uint32_t b = fd_div(t, dS), s = t - b * dS.d;
      const uint8_t* xr = qx + s * qs + b * qb + n * qn;
      const int jc = j < nchunks ? j : 0;
      scale[u] = *reinterpret_cast<const float*>(xr + D);
      w0[u] = reinterpret_cast<const uint32_t*>(xr + 8 * jc)[0];
      w1[u] = reinterpret_cast<const uint32_t*>(xr + 8 * jc)[1];
    }
#pragma unroll
    for (int u = 0; u < kGroupedUnroll; ++u) {
      const u4v t = dequant8(w0[u], w1[u], scale[u]);
      if (active[u])
        reinterpret_cast<uint4*>(x + (int64_t)(r0 + u * RPW + sub) * D)[j] = make_uint4(t[0], t[1], t[2], t[3]);
    }
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
  const int need = vec && H <= kMaxChunks * 512 ? (int)((H + 511) / 512) : 0;
#define CDIT_PT_D(CH)                                                                            \
  if (need <= CH) {                                                                              \
    hipLaunchKernelGGL(comm_per_token_dequant<CH>, dim3(grid_for(M)), dim3(64), 0, stream,        \
                       static_cast<const uint8_t*>(x), static_cast<uint16_t*>(y), M, (int)H, vec); \
    return 0;                                                                                    \
  }
  CDIT_PT_D(0) CDIT_PT_D(1) CDIT_PT_D(2) CDIT_PT_D(4) CDIT_PT_D(6) CDIT_PT_D(8) CDIT_PT_D(12) CDIT_PT_D(16)
  CDIT_PT_D(24) CDIT_PT_D(32)
#undef CDIT_PT_D
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
  hipLaunchKernelGGL(comm_qkv_permute_quant_grouped<G>,                                          \
                     dim3(grid_for((rows + kGroupedWaves * kGroupedUnroll * (64 / G) - 1) /        \
                                   (kGroupedWaves * kGroupedUnroll * (64 / G)))),                  \
                     dim3(64 * kGroupedWaves), 0, stream, xp, yp, (uint32_t)rows, dN, dB, dS, D, sb, ss, sp)
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
  hipLaunchKernelGGL(comm_qkv_permute_dequant_grouped<G>,                                        \
                     dim3(grid_for((rows + kGroupedWaves * kGroupedUnroll * (64 / G) - 1) /        \
                                   (kGroupedWaves * kGroupedUnroll * (64 / G)))),                  \
                     dim3(64 * kGroupedWaves), 0, stream, qp, xp, (uint32_t)rows, dN, dS, D, qs, qb, qn)
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
