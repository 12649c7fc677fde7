// Pieces shared by the two tiled MFMA GEMM kernels (w8a8 and w8a16).
#ifndef CDIT_GEMM_COMMON_H_
#define CDIT_GEMM_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cdit_internal.h"

namespace cdit {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
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

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return f32_to_bf16_bits(lo) | (f32_to_bf16_bits(hi) << 16);
}

// tanh-approximated GELU, the formula of torch.nn.functional.gelu(approximate="tanh"):
// 0.5 v (1 + tanh(u)), u = sqrt(2/pi) (v + 0.044715 v^3). Since
// 0.5 (1 + tanh(u)) = 1 / (1 + exp(-2u)), it is evaluated as v * rcp(1 + exp2(c u))
// with the hardware exp2 and reciprocal (about 1 ulp each; the result is rounded
// to bf16 afterwards). exp2 overflow gives v * 0 = -0 for very negative v and
// exp2 underflow gives v * 1 for very positive v, the correct limits.
__device__ __forceinline__ float gelu_tanh(float v) {
  const float kAlpha = 0.7978845608028654f;  // sqrt(2/pi)
  const float kBeta = 0.044715f;
  const float kM2Log2e = -2.8853900817779268f;  // -2 * log2(e)
  const float u = kAlpha * (v + kBeta * v * v * v);
  const float e = __builtin_amdgcn_exp2f(kM2Log2e * u);
  return v * __builtin_amdgcn_rcpf(1.0f + e);
}

// Workgroup id -> output tile. Workgroups are handed to the 8 XCDs round-robin
// and each XCD has its own L2, so ids that land on one XCD are first made
// consecutive, then walked in column-major order inside groups of GROUP_M tile
// rows: the 32 workgroups resident on an XCD then share a handful of A and B
// panels.
template <int GROUP_M>
__device__ __forceinline__ void tile_of_block(int bid, int nblocks, int tiles_m, int tiles_n,
                                              int* tm, int* tn) {
  constexpr int kXcd = 8;
  int id = bid;
  if (nblocks % kXcd == 0) id = (bid % kXcd) * (nblocks / kXcd) + bid / kXcd;
  const int per_group = GROUP_M * tiles_n;
  const int group = id / per_group;
  const int first_m = group * GROUP_M;
  const int gsize = min(tiles_m - first_m, GROUP_M);
  const int in_group = id - group * per_group;
  *tm = first_m + in_group % gsize;
  *tn = in_group / gsize;
}


// Epilogue shared by the tiled kernels. The MFMAs were issued with the
// operands swapped, so acc[i][j][4*gq+e] is out[m][n] with
//   m = m0 + wm*WM + 32i + (lane&31),  n = n0 + wn*WN + 32j + 8*gq + 4*(lane>>5) + e:
// four consecutive columns per lane. They are scaled, biased, optionally
// GELU'd, packed to bf16 and stored 8 bytes at a time, or (EPI_LDS) transposed
// through a per-wave LDS tile and stored 16 bytes per lane along rows.
// a_scale may be null (weight-only mode): then it is 1.
template <class C>
__device__ __forceinline__ void tile_epilogue(v16f (&acc)[C::TM][C::TN], const GemmArgs& g,
                                              uint8_t* smem, int m0, int n0, int wm, int wn,
                                              int lane, int wave) {
  const int h = lane >> 5;
  const bool gelu = (g.epilogue & CDIT_EPI_GELU_TANH) != 0;
  float as[C::TM];
#pragma unroll
  for (int i = 0; i < C::TM; ++i) {
    const int m = m0 + wm * C::WM + 32 * i + (lane & 31);
    as[i] = (g.a_scale && m < g.M) ? g.a_scale[m] : 1.0f;
  }
  if constexpr (C::EPI_LDS) __syncthreads();  // all waves are done with the stage buffers
  uint8_t* et = smem + wave * (C::WM * C::EPI_PITCH);
#pragma unroll
  for (int j = 0; j < C::TN; ++j) {
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const int nl = 32 * j + 8 * gq + 4 * h;  // column inside the wave tile
      const int n = n0 + wn * C::WN + nl;
      float bs[4], bi[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const bool ok = n + e < g.N;
        bs[e] = ok ? g.b_scale[n + e] : 0.0f;
        bi[e] = (ok && g.bias) ? __uint_as_float((uint32_t)g.bias[n + e] << 16) : 0.0f;
      }
#pragma unroll
      for (int i = 0; i < C::TM; ++i) {
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v[e] = acc[i][j][4 * gq + e] * as[i] * bs[e] + bi[e];
          if (gelu) v[e] = gelu_tanh(v[e]);
        }
        uint2 pk;
        pk.x = pack_bf16x2(v[0], v[1]);
        pk.y = pack_bf16x2(v[2], v[3]);
        const int ml = 32 * i + (lane & 31);  // row inside the wave tile
        if constexpr (C::EPI_LDS) {
          *reinterpret_cast<uint2*>(et + ml * C::EPI_PITCH + nl * 2) = pk;
        } else {
          const int m = m0 + wm * C::WM + ml;
          if (m < g.M && n < g.N)  // N % 8 == 0, so a group of 4 is all in or all out
            *reinterpret_cast<uint2*>(g.out + (int64_t)m * g.ldo + n) = pk;
        }
      }
    }
  }
  if constexpr (C::EPI_LDS) {
    // Each wave re-reads its own tile row-wise: 16 bytes (8 columns) per lane.
    constexpr int LANES_PER_ROW = C::WN / 8;
    constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
    const int cl = (lane % LANES_PER_ROW) * 8;
    const int n = n0 + wn * C::WN + cl;
#pragma unroll
    for (int r0 = 0; r0 < C::WM; r0 += ROWS_PER_PASS) {
      const int ml = r0 + lane / LANES_PER_ROW;
      const int m = m0 + wm * C::WM + ml;
      const uint4 v = *reinterpret_cast<const uint4*>(et + ml * C::EPI_PITCH + cl * 2);
      if (m < g.M && n < g.N) *reinterpret_cast<uint4*>(g.out + (int64_t)m * g.ldo + n) = v;
    }
  }
}

}  // namespace cdit
#endif
