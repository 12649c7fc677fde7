// Pieces shared by the two tiled MFMA GEMM kernels (w8a8 and w8a16).
#ifndef CDIT_GEMM_COMMON_H_
#define CDIT_GEMM_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cdit_internal.h"

namespace cdit {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned int v4u __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

// fp32 -> bf16 bits, round to nearest even (finite inputs; NaN stays NaN).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

// two fp32 -> packed bf16 with the hardware converter (v_cvt_pk_bf16_f32, RNE).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  const v2f v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, v2bf));
}

// two fp32 -> packed fp16 (round to nearest even, overflow to infinity).
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  typedef float v2f __attribute__((ext_vector_type(2)));
  typedef _Float16 v2h __attribute__((ext_vector_type(2)));
  const v2f v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, v2h));
}

// 16 bits of a bias vector -> fp32; the bias has the output's dtype (fp16 or bf16).
template <int OUT>
__device__ __forceinline__ float bias_to_f32(uint32_t bits16) {
  if constexpr (OUT == CDIT_DT_F16) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
  } else {
    return __uint_as_float(bits16 << 16);
  }
}

// Element-wise forms for the kernels that are not tuned per output dtype.
__device__ __forceinline__ float bias_at(const GemmArgs& g, int n) {
  const uint32_t b = g.bias[n];
  return g.out_dtype == CDIT_DT_F16 ? bias_to_f32<CDIT_DT_F16>(b) : bias_to_f32<CDIT_DT_BF16>(b);
}
__device__ __forceinline__ void store_out(const GemmArgs& g, int64_t idx, float v) {
  if (g.out_dtype == CDIT_DT_F32) {
    reinterpret_cast<float*>(g.out)[idx] = v;
  } else if (g.out_dtype == CDIT_DT_F16) {
    g.out[idx] = __builtin_bit_cast(uint16_t, (_Float16)v);
  } else {
    g.out[idx] = (uint16_t)f32_to_bf16_bits(v);
  }
}

// tanh-approximated GELU, the formula of torch.nn.functional.gelu(approximate="tanh"):
// 0.5 v (1 + tanh(u)), u = sqrt(2/pi) (v + 0.044715 v^3). Since
// 0.5 (1 + tanh(u)) = 1 / (1 + exp(-2u)), it is evaluated as v * rcp(1 + exp2(c u))
// with the hardware exp2 and reciprocal (about 1 ulp each; the result is rounded
// to the output dtype afterwards), and c u = v (c0 + c1 v^2) with the constants
// folded: 3 multiplies, 1 FMA, 1 add and the two transcendental instructions per
// element. exp2 overflow gives v * 0 = -0 for very negative v and exp2 underflow
// gives v * 1 for very positive v, the correct limits.
__device__ __forceinline__ float gelu_tanh(float v) {
  const float kC0 = -2.302208198f;    // -2 log2(e) sqrt(2/pi)
  const float kC1 = -0.10294323958f;  // kC0 * 0.044715
  const float e = __builtin_amdgcn_exp2f(v * __fmaf_rn(v * v, kC1, kC0));
  return v * __builtin_amdgcn_rcpf(1.0f + e);
}

// s_waitcnt vmcnt(N) lgkmcnt(0) followed by a bare workgroup barrier. The memory
// clobber keeps the compiler from moving LDS accesses across it.
// The s_waitcnt is emitted through the builtin so that the compiler's own wait
// insertion sees it (it would otherwise re-wait for LDS reads with lgkmcnt(0)).
template <int VM>
__device__ __forceinline__ void wait_and_barrier() {
  asm volatile("" ::: "memory");
  // simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14
  __builtin_amdgcn_s_waitcnt((VM & 0xf) | (7 << 4) | (0 << 8) | ((VM >> 4) << 14));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
template <int VM>
__device__ __forceinline__ void wait_vm() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt((VM & 0xf) | (7 << 4) | (0xf << 8) | ((VM >> 4) << 14));
  asm volatile("" ::: "memory");
}
// Waits until at most `later` steps (of D DMA instructions each) are in flight,
// `later` in [0, MAXL]; the count has to be an immediate, hence the switch.
template <int D, int MAXL, bool BARRIER>
__device__ __forceinline__ void wait_steps(int later) {
#define CDIT_WAIT_CASE(L)                                 \
  case L:                                                 \
    if constexpr (L <= MAXL) {                            \
      if constexpr (BARRIER) {                            \
        wait_and_barrier<(L * D > 63 ? 63 : L * D)>();    \
      } else {                                            \
        wait_vm<(L * D > 63 ? 63 : L * D)>();             \
      }                                                   \
    }                                                     \
    break;
  switch (later) {
    CDIT_WAIT_CASE(0)
    CDIT_WAIT_CASE(1)
    CDIT_WAIT_CASE(2)
    CDIT_WAIT_CASE(3)
    CDIT_WAIT_CASE(4)
    CDIT_WAIT_CASE(5)
    CDIT_WAIT_CASE(6)
    default:
      if constexpr (BARRIER) {
        wait_and_barrier<0>();
      } else {
        wait_vm<0>();
      }
  }
#undef CDIT_WAIT_CASE
}

// Raises a kernel's dynamic LDS limit to `bytes`, once per device: the attribute belongs
// to the function on the current device. done: one flag per device ordinal, owned by the
// caller (a static array per kernel instance; setting the attribute twice is harmless).
inline int allow_dynamic_lds(const void* kernel, int bytes, bool* done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
  if (dev >= 0 && done[dev]) return 0;
  hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) {
    set_error("hipFuncSetAttribute(%d bytes LDS): %s", bytes, hipGetErrorString(e));
    return CDIT_EHIP;
  }
  if (dev >= 0) done[dev] = true;
  return 0;
}

// Number of CUs of the current device (cached per device ordinal); 0 on error.
inline int cu_count() {
  static int cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64 && cached[dev] > 0) return cached[dev];
  int n = 0;
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (dev >= 0 && dev < 64) cached[dev] = n;
  return n;
}

// Workgroup id -> output tile. Workgroups are handed to the 8 XCDs round-robin
// and each XCD has its own L2, so ids that land on one XCD are first made
// consecutive, then walked in column-major order inside groups of GROUP_M tile
// rows: the 32 workgroups resident on an XCD then share a handful of A and B
// panels.
// Linear tile id -> (tile row, tile column): column-major inside groups of GROUP_M
// tile rows.
template <int GROUP_M>
__device__ __forceinline__ void tile_of_linear(int id, int tiles_m, int tiles_n, int* tm,
                                               int* tn) {
  const int per_group = GROUP_M * tiles_n;
  const int group = id / per_group;
  const int first_m = group * GROUP_M;
  const int gsize = min(tiles_m - first_m, GROUP_M);
  const int in_group = id - group * per_group;
  *tm = first_m + in_group % gsize;
  *tn = in_group / gsize;
}

template <int GROUP_M>
__device__ __forceinline__ void tile_of_block(int bid, int nblocks, int tiles_m, int tiles_n,
                                              int* tm, int* tn) {
  constexpr int kXcd = 8;
  int id = bid;
  if (nblocks % kXcd == 0) id = (bid % kXcd) * (nblocks / kXcd) + bid / kXcd;
  tile_of_linear<GROUP_M>(id, tiles_m, tiles_n, tm, tn);
}

// Epilogue shared by the tiled kernels. The MFMAs were issued with the
// operands swapped, so acc[i][j][4*gq+e] is out[m][n] with
//   m = m0 + wm*WM + 32i + (lane&31),  n = n0 + wn*WN + 32j + 8*gq + 4*(lane>>5) + e:
// four consecutive columns per lane. Per element: one multiply by a_scale[m], one
// FMA with b_scale[n] and bias[n], optional GELU, hardware bf16 pack. With
// EPI_LDS each 32-row block of the wave tile is transposed through a wave-private
// LDS tile (32 rows x EPI_PITCH bytes at `et`; no workgroup barrier needed) so that
// every lane stores 16 bytes along a row; otherwise lanes store their 8 bytes
// directly. a_scale may be null (weight-only mode): then it is 1.
// Whether the wave-private epilogue tile has unpadded rows (EPI_PITCH == 2*WN).
template <class C>
__device__ __forceinline__ constexpr bool epi_rotated() {
  return C::EPI_PITCH == C::WN * 2;
}

template <class C>
__device__ __forceinline__ void tile_epilogue(v16f (&acc)[C::TM][C::TN], const GemmArgs& g,
                                              uint8_t* et, int m0, int n0, int wm, int wn,
                                              int lane) {
  const int h = lane >> 5, r = lane & 31;
  const bool gelu = (g.epilogue & CDIT_EPI_GELU_TANH) != 0;
  const int nw = n0 + wn * C::WN;  // first column of the wave tile
  const int mw = m0 + wm * C::WM;
  // b_scale / bias of this lane's 4-column groups, loaded once (the operand
  // registers of the main loop are free by now). Reloading them per 32-row block
  // would save registers but measured 10 % slower on 96-wide wave tiles.
  constexpr bool kPreload = true;
  auto load_cols = [&](int j, int gq, v4f& s4, v4f& b4) {
    const int n = nw + 32 * j + 8 * gq + 4 * h;  // N % 8 == 0: a group of 4 is all in or out
    s4 = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    b4 = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    if (n < g.N) {
      s4 = *reinterpret_cast<const v4f*>(g.b_scale + n);
      if (g.bias) {
        const uint2 bb = *reinterpret_cast<const uint2*>(g.bias + n);
        b4[0] = __uint_as_float(bb.x << 16);
        b4[1] = __uint_as_float(bb.x & 0xffff0000u);
        b4[2] = __uint_as_float(bb.y << 16);
        b4[3] = __uint_as_float(bb.y & 0xffff0000u);
      }
    }
  };
  v4f bs[kPreload ? C::TN : 1][4], bi[kPreload ? C::TN : 1][4];
  if constexpr (kPreload) {
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) load_cols(j, gq, bs[j][gq], bi[j][gq]);
  }
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    const int m = mw + 32 * i + r;
    const float as = g.a_scale ? (m < g.M ? g.a_scale[m] : 0.0f) : 1.0f;
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int gq = 0; gq < 4; ++gq) {
        v4f s4, b4;
        if constexpr (kPreload) {
          s4 = bs[j][gq];
          b4 = bi[j][gq];
        } else {
          load_cols(j, gq, s4, b4);
        }
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = __fmaf_rn(acc[i][j][4 * gq + e] * as, s4[e], b4[e]);
          if (gelu) v[e] = gelu_tanh(v[e]);
        }
        uint2 pk;
        pk.x = pack_bf16x2(v[0], v[1]);
        pk.y = pack_bf16x2(v[2], v[3]);
        const int nl = 32 * j + 8 * gq + 4 * h;  // column inside the wave tile
        if constexpr (C::EPI_LDS) {
          if constexpr (epi_rotated<C>()) {
            // unpadded rows: rotate the 16-byte chunks by the row index instead
            const int chunk = ((nl >> 3) + r) % (C::WN / 8);
            *reinterpret_cast<uint2*>(et + r * C::EPI_PITCH + chunk * 16 + (nl & 7) * 2) = pk;
          } else {
            *reinterpret_cast<uint2*>(et + r * C::EPI_PITCH + nl * 2) = pk;
          }
        } else {
          if (m < g.M && nw + nl < g.N)
            *reinterpret_cast<uint2*>(g.out + (int64_t)m * g.ldo + nw + nl) = pk;
        }
      }
    if constexpr (C::EPI_LDS) {
      // read the 32 x WN block back row-wise, 16 bytes (8 columns) per lane
      constexpr int CPR = C::WN / 8;         // 16-byte chunks per row
      constexpr int PER_LANE = 32 * CPR / 64;  // chunks per lane
      static_assert((32 * CPR) % 64 == 0, "wave tile width must be a multiple of 16");
#pragma unroll
      for (int t = 0; t < PER_LANE; ++t) {
        const int q = t * 64 + lane;
        const int row = q / CPR, cc = q % CPR;
        const int pc = epi_rotated<C>() ? (cc + row) % CPR : cc;
        const uint4 d = *reinterpret_cast<const uint4*>(et + row * C::EPI_PITCH + pc * 16);
        const int mm = mw + 32 * i + row, nn = nw + cc * 8;
        if (mm < g.M && nn < g.N) *reinterpret_cast<uint4*>(g.out + (int64_t)mm * g.ldo + nn) = d;
      }
    }
  }
}

}  // namespace cdit
#endif
