// Per-row dynamic FP8 (OCP e4m3fn) quantizer for gfx950.
//
// One 64-lane wavefront owns one row: it reads the row once from HBM with
// 128-bit loads and keeps it in VGPRs, reduces |x| to the row amax with a
// cross-lane max, derives the scale, then divides, converts with the hardware
// e4m3 converter (v_cvt_pk_fp8_f32, RNE) and writes 64-bit packs. The stores
// carry the nontemporal hint.
// Algorithmic traffic is 2 B read + 1 B written per element + 4 B per row.
//
// Arithmetic follows torchao's _choose_scale_float8 / _quantize_affine_float8
// as cache-dit calls them (src/cache_dit/quantization/torchao/quantize_ao.py:54-70):
// amax in bf16, scale = amax/448 (optionally rounded to bf16), zero scale -> 1,
// q = cast(clamp(float(x)/scale, +-448)). The codes must be those of the IEEE
// division: a bare reciprocal multiply flips about 1e-4 of them. Per row the
// kernel therefore works out 1/scale as an unevaluated sum hi + lo of two fp32
// values (make_recip) and per element
//   q = fma(x, hi, x * lo)
// which is x/scale rounded once up to a double rounding of the small term, and
// keeps the sign of x = -0. That this
// reproduces x/scale down to the e4m3 code has been verified exhaustively on
// the CPU for every (x, amax) pair of bf16 values with |x| <= amax, in both
// scale modes, whenever 2^-100 <= scale < 2^101 (tests/native/divcheck.c);
// rows whose scale falls outside that window take the plain `/`.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <type_traits>

#include "cdit_internal.h"
#include "quant_device.h"

namespace cdit {
namespace {

// Row resident in registers: CH 16-byte chunks per lane (K <= CH*512).
struct NoBatch {};

// BATCHED: the rows of several activations in one launch (QuantBatch); x, q, scale and
// their leading dimensions then come from the activation the row belongs to and M is the
// total row count. The instances without it are unchanged by its existence.
template <int CH, bool NT_LOAD = false, bool NT_STORE = false, bool BATCHED = false>
__global__ __launch_bounds__(64) void quant_rowwise_regs(
    const uint16_t* __restrict__ x, int64_t ld_x, uint8_t* __restrict__ q, int64_t ld_q,
    float* __restrict__ scale, int M, int K, int scale_mode,
    std::conditional_t<BATCHED, QuantBatch, NoBatch> batch = {}) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves_per_block = blockDim.x >> 6;
  const int nchunks = K >> 3;
  for (int64_t row = (int64_t)blockIdx.x * waves_per_block + wave; row < M;
       row += (int64_t)gridDim.x * waves_per_block) {
    const uint16_t* x_row = x + row * ld_x;
    uint8_t* q_row = q + row * ld_q;
    float* s_row = scale + row;
    if constexpr (BATCHED) {
      // wave-uniform: one row per wavefront (row_begin beyond the last activation holds M)
      const int r = __builtin_amdgcn_readfirstlane((int)row);
      int s = 0;
#pragma unroll
      for (int i = 1; i < kMaxQuantActs; ++i) s += r >= batch.row_begin[i];
      const int64_t local = r - batch.row_begin[s];
      x_row = batch.x[s] + local * batch.ld_x[s];
      q_row = batch.q[s] + local * batch.ld_q[s];
      s_row = batch.scale[s] + local;
    }
    const uint4* xr = reinterpret_cast<const uint4*>(x_row);
    uint4 v[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = c * 64 + lane;
      if (idx < nchunks) {
        if constexpr (NT_LOAD) {
          typedef unsigned int u4v __attribute__((ext_vector_type(4)));
          const u4v t = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(xr + idx));
          v[c] = make_uint4(t[0], t[1], t[2], t[3]);
        } else {
          v[c] = xr[idx];
        }
      } else {
        v[c] = make_uint4(0, 0, 0, 0);
      }
    }
    uint32_t m = 0;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      m = absmax2(m, v[c].x);
      m = absmax2(m, v[c].y);
      m = absmax2(m, v[c].z);
      m = absmax2(m, v[c].w);
    }
    m = wave_max_u32(fold2(m));
    const float s = row_scale(m, scale_mode);
    if (lane == 0) *s_row = s;
    uint2* qr = reinterpret_cast<uint2*>(q_row);
    if (scale_in_fast_window(s)) {  // wave-uniform
      const Recip r = make_recip(s);
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int idx = c * 64 + lane;
        if (idx < nchunks) {
          uint2 o;
          o.x = quant4<true>(v[c].x, v[c].y, s, r);
          o.y = quant4<true>(v[c].z, v[c].w, s, r);
          if constexpr (NT_STORE) {
            typedef unsigned int u2v __attribute__((ext_vector_type(2)));
            const u2v t = {o.x, o.y};
            __builtin_nontemporal_store(t, reinterpret_cast<u2v*>(qr + idx));
          } else {
            qr[idx] = o;
          }
        }
      }
    } else {
      // cold path, kept small: re-reads the row (an L2 hit) in a rolled loop
#pragma unroll 1
      for (int idx = lane; idx < nchunks; idx += 64) {
        const uint4 w = xr[idx];
        uint2 o;
        o.x = quant4<false>(w.x, w.y, s, Recip{});
        o.y = quant4<false>(w.z, w.w, s, Recip{});
        qr[idx] = o;
      }
    }
  }
}

// WAVES (two or four) wavefronts share a row, each keeps its part of it in registers: fewer
// registers per wavefront, more wavefronts in flight, and a row's loads, arithmetic and
// stores overlap between its parts; the partial maxima meet in LDS. Measured against one
// wavefront per row (codes read by a GEMM next; us): 4608 x 15360 40.0 -> 36.2, 4096 x 12288
// 27.5 -> 25.9, 4608 x 3072 9.0 -> 8.5, 32760 x 5120 87.1 -> 85.4. BATCHED as in
// quant_rowwise_regs.
template <int CH, bool NT_LOAD, bool NT_STORE, bool BATCHED = false, int WAVES = 2>
__global__ __launch_bounds__(64 * WAVES) void quant_rowwise_split2(
    const uint16_t* __restrict__ x, int64_t ld_x, uint8_t* __restrict__ q, int64_t ld_q,
    float* __restrict__ scale, int M, int K, int scale_mode,
    std::conditional_t<BATCHED, QuantBatch, NoBatch> batch = {}) {
  __shared__ uint32_t part[WAVES];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nchunks = K >> 3;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const uint16_t* x_row = x + row * ld_x;
    uint8_t* q_row = q + row * ld_q;
    float* s_row = scale + row;
    if constexpr (BATCHED) {
      const int r = __builtin_amdgcn_readfirstlane((int)row);
      int s = 0;
#pragma unroll
      for (int i = 1; i < kMaxQuantActs; ++i) s += r >= batch.row_begin[i];
      const int64_t local = r - batch.row_begin[s];
      x_row = batch.x[s] + local * batch.ld_x[s];
      q_row = batch.q[s] + local * batch.ld_q[s];
      s_row = batch.scale[s] + local;
    }
    const uint4* xr = reinterpret_cast<const uint4*>(x_row);
    uint4 v[CH];
    uint32_t m = 0;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = (WAVES * c + wave) * 64 + lane;
      if (idx < nchunks) {
        if constexpr (NT_LOAD) {
          typedef unsigned int u4v __attribute__((ext_vector_type(4)));
          const u4v t = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(xr + idx));
          v[c] = make_uint4(t[0], t[1], t[2], t[3]);
        } else {
          v[c] = xr[idx];
        }
      } else {
        v[c] = make_uint4(0, 0, 0, 0);
      }
      m = absmax2(absmax2(absmax2(absmax2(m, v[c].x), v[c].y), v[c].z), v[c].w);
    }
    m = wave_max_u32(fold2(m));
    if (lane == 0) part[wave] = m;
    __syncthreads();
    m = part[0];
#pragma unroll
    for (int i = 1; i < WAVES; ++i) m = max(m, part[i]);
    __syncthreads();  // part is free for the next row
    const float s = row_scale(m, scale_mode);
    if (threadIdx.x == 0) *s_row = s;
    uint2* qr = reinterpret_cast<uint2*>(q_row);
    if (scale_in_fast_window(s)) {  // uniform
      const Recip r = make_recip(s);
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int idx = (WAVES * c + wave) * 64 + lane;
        if (idx < nchunks) {
          const uint2 o = {quant4<true>(v[c].x, v[c].y, s, r), quant4<true>(v[c].z, v[c].w, s, r)};
          if constexpr (NT_STORE) {
            typedef unsigned int u2v __attribute__((ext_vector_type(2)));
            const u2v t = {o.x, o.y};
            __builtin_nontemporal_store(t, reinterpret_cast<u2v*>(qr + idx));
          } else {
            qr[idx] = o;
          }
        }
      }
    } else {  // cold path: re-reads the row
#pragma unroll 1
      for (int idx = threadIdx.x; idx < nchunks; idx += 64 * WAVES) {
        const uint4 w = xr[idx];
        qr[idx] = uint2{quant4<false>(w.x, w.y, s, Recip{}), quant4<false>(w.z, w.w, s, Recip{})};
      }
    }
  }
}

// The regs kernel on a row that is the concatenation of two source rows, [x1 | x2]: the
// input of FLUX single blocks' proj_out is torch.cat([attn_output, mlp_hidden_states], dim=2)
// (reference dataflow src/cache_dit/caching/patch_functors/functor_flux.py:68-80), read by
// that quantized Linear only -- quantizing the two sources in place of their copy saves the
// copy's write and the quantizer's read of it. n1 = chunks (8 elements) of x1 per row; the
// codes go to one [M, K1 + K2] buffer and are those of the quantizer on the concatenation.
template <int CH, bool NT_LOAD, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void quant_rowwise_cat_regs(
    const uint16_t* __restrict__ x1, int64_t ld_x1, int n1, const uint16_t* __restrict__ x2,
    int64_t ld_x2, uint8_t* __restrict__ q, int64_t ld_q, float* __restrict__ scale, int M, int K,
    int scale_mode) {
  __shared__ uint32_t part[WAVES];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nchunks = K >> 3;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const uint4* r1 = reinterpret_cast<const uint4*>(x1 + row * ld_x1);
    const uint4* r2 = reinterpret_cast<const uint4*>(x2 + row * ld_x2) - n1;
    auto load = [&](int idx) -> uint4 {
      const uint4* src = (idx < n1 ? r1 : r2) + idx;
      if constexpr (NT_LOAD) {
        typedef unsigned int u4v __attribute__((ext_vector_type(4)));
        const u4v t = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(src));
        return make_uint4(t[0], t[1], t[2], t[3]);
      } else {
        return *src;
      }
    };
    uint4 v[CH];
    uint32_t m = 0;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int idx = (WAVES * c + wave) * 64 + lane;
      v[c] = idx < nchunks ? load(idx) : make_uint4(0, 0, 0, 0);
      m = absmax2(absmax2(absmax2(absmax2(m, v[c].x), v[c].y), v[c].z), v[c].w);
    }
    m = wave_max_u32(fold2(m));
    if constexpr (WAVES > 1) {  // the wavefronts of a row meet in LDS, as in quant_rowwise_split2
      if (lane == 0) part[wave] = m;
      __syncthreads();
      m = part[0];
#pragma unroll
      for (int i = 1; i < WAVES; ++i) m = max(m, part[i]);
      __syncthreads();
    }
    const float s = row_scale(m, scale_mode);
    if (threadIdx.x == 0) scale[row] = s;
    uint2* qr = reinterpret_cast<uint2*>(q + row * ld_q);
    if (scale_in_fast_window(s)) {  // uniform
      const Recip r = make_recip(s);
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int idx = (WAVES * c + wave) * 64 + lane;
        if (idx < nchunks)
          qr[idx] = uint2{quant4<true>(v[c].x, v[c].y, s, r), quant4<true>(v[c].z, v[c].w, s, r)};
      }
    } else {  // cold path: re-reads the row
#pragma unroll 1
      for (int idx = threadIdx.x; idx < nchunks; idx += 64 * WAVES) {
        const uint4 w = load(idx);
        qr[idx] = uint2{quant4<false>(w.x, w.y, s, Recip{}), quant4<false>(w.z, w.w, s, Recip{})};
      }
    }
  }
}

// Any K, any alignment: one wavefront per row, two passes over the row with
// element-wise loads (the second pass hits L2). Slow path for odd shapes.
__global__ __launch_bounds__(64) void quant_rowwise_generic(
    const uint16_t* __restrict__ x, int64_t ld_x, uint8_t* __restrict__ q, int64_t ld_q,
    float* __restrict__ scale, int M, int K, int scale_mode) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves_per_block = blockDim.x >> 6;
  for (int64_t row = (int64_t)blockIdx.x * waves_per_block + wave; row < M;
       row += (int64_t)gridDim.x * waves_per_block) {
    const uint16_t* xr = x + row * ld_x;
    uint32_t m = 0;
    for (int k = lane; k < K; k += 64) {
      uint32_t a = xr[k] & 0x7fffu;
      m = m > a ? m : a;
    }
    m = wave_max_u32(m);
    const float s = row_scale(m, scale_mode);
    if (lane == 0) scale[row] = s;
    uint8_t* qr = q + row * ld_q;
    for (int k = lane; k < K; k += 64) {
      float y = clamp448(__uint_as_float((uint32_t)xr[k] << 16) / s);
      uint32_t p = __builtin_amdgcn_cvt_pk_fp8_f32(y, y, 0u, false);
      qr[k] = (uint8_t)(p & 0xffu);
    }
  }
}

// ---------------------------------------------------------------------------
// Per-tensor variant (one scale for the whole [M,K] tensor): three launches.
//   zero_amax:           *amax_ws = 0 (a kernel, not a memset, so that the sequence
//                        can be recorded into a hipGraph)
//   tensor_amax:         amax over all elements, one wavefront per row at a time,
//                        integer atomic max into *amax_ws (exact, order free)
//   quant_tensorwise_*:  scale from *amax_ws, written to scale[m] for every row (the
//                        GEMM takes per-row scales), and the same cast as above
__global__ void zero_amax(uint32_t* amax_ws) { *amax_ws = 0u; }

__global__ __launch_bounds__(64) void tensor_amax(const uint16_t* __restrict__ x, int64_t ld_x,
                                                  int M, int K, bool vec,
                                                  uint32_t* __restrict__ amax_ws) {
  const int lane = threadIdx.x & 63;
  uint32_t m = 0;
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const uint16_t* xr = x + row * ld_x;
    if (vec) {
      const uint4* xv = reinterpret_cast<const uint4*>(xr);
      for (int idx = lane; idx < (K >> 3); idx += 64) {
        const uint4 w = xv[idx];
        m = absmax2(m, w.x);
        m = absmax2(m, w.y);
        m = absmax2(m, w.z);
        m = absmax2(m, w.w);
      }
    } else {
      for (int k = lane; k < K; k += 64) {
        const uint32_t a = xr[k] & 0x7fffu;
        m = m > a ? m : a;
      }
    }
  }
  m = wave_max_u32(fold2(m));
  if (lane == 0 && m > __hip_atomic_load(amax_ws, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
    atomicMax(amax_ws, m);
}

// vec: 16-byte aligned rows with K % 8 == 0
__global__ __launch_bounds__(64) void quant_tensorwise_cast(
    const uint16_t* __restrict__ x, int64_t ld_x, uint8_t* __restrict__ q, int64_t ld_q,
    float* __restrict__ scale, int M, int K, int scale_mode, bool vec,
    const uint32_t* __restrict__ amax_ws) {
  const int lane = threadIdx.x & 63;
  const float s = row_scale(*amax_ws, scale_mode);
  const bool fast = scale_in_fast_window(s);
  const Recip r = make_recip(s);
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    if (lane == 0) scale[row] = s;
    const uint16_t* xr = x + row * ld_x;
    uint8_t* qr = q + row * ld_q;
    if (vec) {
      const uint4* xv = reinterpret_cast<const uint4*>(xr);
      uint2* qv = reinterpret_cast<uint2*>(qr);
      if (fast) {
        for (int idx = lane; idx < (K >> 3); idx += 64) {
          const uint4 w = xv[idx];
          uint2 o;
          o.x = quant4<true>(w.x, w.y, s, r);
          o.y = quant4<true>(w.z, w.w, s, r);
          qv[idx] = o;
        }
      } else {
#pragma unroll 1
        for (int idx = lane; idx < (K >> 3); idx += 64) {
          const uint4 w = xv[idx];
          uint2 o;
          o.x = quant4<false>(w.x, w.y, s, Recip{});
          o.y = quant4<false>(w.z, w.w, s, Recip{});
          qv[idx] = o;
        }
      }
    } else {
      for (int k = lane; k < K; k += 64) {
        const float y = clamp448(__uint_as_float((uint32_t)xr[k] << 16) / s);
        const uint32_t p = __builtin_amdgcn_cvt_pk_fp8_f32(y, y, 0u, false);
        qr[k] = (uint8_t)(p & 0xffu);
      }
    }
  }
}

// The same two kernels for 16-byte aligned rows of up to 512 CH elements: all loads of a row
// in flight at once (the row loop above issues them one by one), buffer accesses whose
// descriptor drops what lies beyond the row, non-temporal stores of the codes. Atomics on one
// address are served one after the other (measured: 15 ns each, 69 us for one per row of a
// 4608-row activation), so the amax kernel runs on at most one workgroup of eight wavefronts
// per CU, each wavefront with several rows, the eight maxima meet in LDS, and the workgroup
// skips its atomic where the word already holds at least its maximum (a relaxed read at
// device scope suffices: the word only grows).
constexpr int kAmaxWaves = 8;  // wavefronts per workgroup of tensor_amax_rows

template <int CH>
__global__ __launch_bounds__(64 * kAmaxWaves) void tensor_amax_rows(const uint16_t* __restrict__ x,
                                                                     int64_t ld_x, int M, int K,
                                                                     uint32_t* __restrict__ amax_ws) {
  typedef unsigned int u4v __attribute__((ext_vector_type(4)));
  __shared__ uint32_t part[kAmaxWaves];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t m = 0;
  for (int64_t row = (int64_t)blockIdx.x * kAmaxWaves + wave; row < M; row += (int64_t)gridDim.x * kAmaxWaves) {
    const __amdgpu_buffer_rsrc_t xb = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(x + row * ld_x), 0, K * 2, 0x00020000);
    u4v w[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) w[c] = __builtin_amdgcn_raw_buffer_load_b128(xb, 16 * (c * 64 + lane), 0, 0);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      m = absmax2(m, w[c][0]);
      m = absmax2(m, w[c][1]);
      m = absmax2(m, w[c][2]);
      m = absmax2(m, w[c][3]);
    }
  }
  m = wave_max_u32(fold2(m));
  if (lane == 0) part[wave] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < kAmaxWaves; ++w) m = m > part[w] ? m : part[w];
    // (read at device scope: a plain load may be served by this CU's own cache with the value
    // an earlier workgroup saw)
    if (m > __hip_atomic_load(amax_ws, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(amax_ws, m);
  }
}

template <int CH>
__global__ __launch_bounds__(64) void quant_tensorwise_cast_rows(
    const uint16_t* __restrict__ x, int64_t ld_x, uint8_t* __restrict__ q, int64_t ld_q,
    float* __restrict__ scale, int M, int K, int scale_mode, const uint32_t* __restrict__ amax_ws) {
  typedef unsigned int u4v __attribute__((ext_vector_type(4)));
  typedef unsigned int u2v __attribute__((ext_vector_type(2)));
  const int lane = threadIdx.x & 63;
  const float s = row_scale(*amax_ws, scale_mode);
  const bool fast = scale_in_fast_window(s);
  const Recip r = make_recip(s);
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    if (lane == 0) scale[row] = s;
    const __amdgpu_buffer_rsrc_t xb = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(x + row * ld_x), 0, K * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t qb = __builtin_amdgcn_make_buffer_rsrc(q + row * ld_q, 0, K, 0x00020000);
    u4v w[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) w[c] = __builtin_amdgcn_raw_buffer_load_b128(xb, 16 * (c * 64 + lane), 0, 0);
    if (fast) {
#pragma unroll
      for (int c = 0; c < CH; ++c)
        __builtin_amdgcn_raw_buffer_store_b64(
            u2v{quant4<true>(w[c][0], w[c][1], s, r), quant4<true>(w[c][2], w[c][3], s, r)}, qb,
            8 * (c * 64 + lane), 0, 2);
    } else {
#pragma unroll 1
      for (int c = 0; c < CH; ++c)
        __builtin_amdgcn_raw_buffer_store_b64(
            u2v{quant4<false>(w[c][0], w[c][1], s, Recip{}), quant4<false>(w[c][2], w[c][3], s, Recip{})}, qb,
            8 * (c * 64 + lane), 0, 2);
    }
  }
}

// ---------------------------------------------------------------------------
// Producer-fused quantizer: LayerNorm (no affine) + AdaLN modulation + per-row FP8
// quantization of one activation row in one pass over it. The modulated activation
// of a DiT block, `norm(x) * (1 + scale) + shift`, is read by quantized Linears only
// (q/k/v, proj_mlp, ff.net.0.proj; reference dataflow
// src/cache_dit/caching/patch_functors/functor_flux.py:48-80), so the codes can be
// produced where the activation is: 2 B read + 1 B written per element instead of the
// producer's bf16 write and the quantizer's read of it on top. y is written as well on
// request (WRITE_Y), for consumers that read the bf16 tensor.
//
// Arithmetic, element k of a row (every step rounds to bf16 where the unfused sequence of
// bf16 tensor ops does, so that the codes are those the stand-alone quantizer gives on y):
//   mean = sum(x) / K,  var = sum((x - mean)^2) / K,  rstd = 1 / sqrt(var + eps)   (fp32)
//   n = bf16((x - mean) * rstd);  t = bf16(1 + scale[k]);  u = bf16(n * t);
//   y = bf16(u + shift[k]);  then amax / scale / e4m3 cast of y as in quant_rowwise_regs.
// shift and scale are bf16 [*, K]; row m uses their row m / rows_per_mod (one modulation
// vector per batch element, broadcast over its tokens).
__device__ __forceinline__ uint32_t bf16_bits(float f) {
  return __float_as_uint(round_to_bf16(f)) >> 16;
}

// y bits of one element: x, scale, shift as fp32 (exact widenings of bf16 values)
__device__ __forceinline__ uint32_t modulate1(float x, float mean, float rstd, float sc, float sh) {
  const float n = round_to_bf16((x - mean) * rstd);
  const float t = round_to_bf16(1.0f + sc);
  const float u = round_to_bf16(n * t);
  return bf16_bits(u + sh);
}

// Wave-wide reductions that leave the result in lane 63: four butterfly steps inside each
// row of 16 lanes (DPP quad_perm / row_half_mirror / row_mirror), then the row results travel
// up with row_bcast:15 into rows 1 and 3 and row_bcast:31 into rows 2 and 3. Six DPP
// instructions, a fixed order of operations.
template <class Op>
__device__ __forceinline__ uint32_t wave_reduce_to_lane63(uint32_t v, Op op) {
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xf, 0xf, false));  // row_half_mirror
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xf, 0xf, false));  // row_mirror
  // rows 1 and 3 take in lane 15 of the row below them; the other rows keep their value
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp((int)Op::identity(), (int)v, 0x142, 0xa, 0xf, false));
  // rows 2 and 3 take in lane 31
  v = op(v, (uint32_t)__builtin_amdgcn_update_dpp((int)Op::identity(), (int)v, 0x143, 0xc, 0xf, false));
  return v;
}
struct AddF32 {
  static __device__ __forceinline__ uint32_t identity() { return 0u; }  // +0.0f
  __device__ __forceinline__ uint32_t operator()(uint32_t a, uint32_t b) const {
    return __float_as_uint(__uint_as_float(a) + __uint_as_float(b));
  }
};
struct MaxU32 {
  static __device__ __forceinline__ uint32_t identity() { return 0u; }
  __device__ __forceinline__ uint32_t operator()(uint32_t a, uint32_t b) const { return a > b ? a : b; }
};

// x.lo * y.lo + x.hi * y.hi + acc of two packed bf16 pairs in one instruction
// (v_dot2c_f32_bf16). The products are exact in fp32; how the three-term sum is rounded
// inside is the instruction's own business, which row statistics tolerate.
__device__ __forceinline__ float dot_pair(uint32_t a, uint32_t b, float acc) {
  typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(v2bf, a), __builtin_bit_cast(v2bf, b), acc,
                                         false);
}

// fp32 -> nearest-even bf16, widened back to fp32, in one instruction: v_cvt_pk_bf16_f32 with
// a zero in the low half leaves the rounded value's bits where an fp32 has them.
__device__ __forceinline__ float round_bf16_wide(float f) { return __uint_as_float(pk_bf16(0.0f, f)); }

// two widened bf16 values -> packed pair (their high halves), one byte permute
__device__ __forceinline__ uint32_t pack_wide(float lo, float hi) {
  return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

// A workgroup of WAVES wavefronts owns `rows_per_wg` consecutive rows; chunk (WAVES c + wave)
// * 64 + lane of a row belongs to this thread, CH chunks of 8 elements per thread.
//  * What is the same for every row of a modulation vector stays in registers from row to row,
//    widened to fp32: t = bf16(1 + scale[k]) (0 beyond K) and shift[k].
//  * The next row is fetched while the current one is worked on (two register sets, taken in
//    turn). Every load and store of the row loop is a buffer access without a branch around
//    it (beyond the row: zeros read, nothing written; the scale leaves through a lane offset
//    beyond its descriptor for every thread but one), so that the compiler can count the
//    accesses in flight: with a store under a lane mask it waits for everything (vmcnt(0))
//    where it needs the prefetched row, which puts the latency of the previous row's stores
//    into every row.
//  * Statistics in one pass over the packed row: sum and sum of squares with one
//    v_dot2c_f32_bf16 each per pair, var = E[x^2] - mean^2; when that difference has lost more
//    than two bits to cancellation (mean^2 > 4 var, a zero or negative result, non-finite
//    input) the deviations are summed in a second pass as the unfused LayerNorm does. One
//    workgroup reduction for both sums, one for the amax: lane 63 of every wavefront
//    leaves its partial result in an LDS slot (slots alternate with the row parity, so one
//    barrier each).
//  * Per element: widen, one FMA for (x - mean) rstd (as x rstd - mean rstd), then every step
//    that the unfused bf16 op sequence rounds is one v_cvt_pk_bf16_f32 that rounds and
//    widens at once; amax as integer maxima of the raw bits, positive and negative values
//    apart (a NaN pattern is the largest of either kind, as in torch.amax); the e4m3 cast
//    as in the stand-alone quantizer. About 14 VALU instructions per element.
template <int CH, bool WRITE_Y, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void ln_modulate_quant_rows(
    const uint16_t* __restrict__ x, int64_t ld_x, const uint16_t* __restrict__ shift,
    const uint16_t* __restrict__ scale_mod, int64_t ld_mod, int rows_per_mod, float eps,
    uint16_t* __restrict__ y, int64_t ld_y, uint8_t* __restrict__ q, int64_t ld_q,
    float* __restrict__ scale, int M, int K, int scale_mode, int rows_per_wg) {
  constexpr int kCached = 0;
  typedef unsigned int u4v __attribute__((ext_vector_type(4)));
  typedef unsigned int u2v __attribute__((ext_vector_type(2)));
  __shared__ float red_f[2][8][2];
  __shared__ uint32_t red_m[2][8];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int nchunks = K >> 3;
  const float inv_k = 1.0f / (float)K;
  const int row0 = blockIdx.x * rows_per_wg;
  const int row_end = min(M, row0 + rows_per_wg);
  if (row0 >= row_end) return;
  int idx[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) idx[c] = (WAVES * c + wave) * 64 + lane;
  auto row_buf = [&](const void* base, int64_t byte0, int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint8_t*>(static_cast<const uint8_t*>(base)) + byte0, 0, bytes, 0x00020000);
  };

  float t_f[CH][8], sh_f[CH][8];  // modulation vectors of the current modulation row
  int cur_mod = -1;
  auto widen_mod = [&](int c, const u4v& sh, const u4v& sc) {
    const bool valid = idx[c] < nchunks;  // beyond K: t = 0, so that y = 0 there
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      t_f[c][2 * e] = valid ? round_bf16_wide(1.0f + bf16_lo(sc[e])) : 0.0f;
      t_f[c][2 * e + 1] = valid ? round_bf16_wide(1.0f + bf16_hi(sc[e])) : 0.0f;
      sh_f[c][2 * e] = bf16_lo(sh[e]);
      sh_f[c][2 * e + 1] = bf16_hi(sh[e]);
    }
  };
  auto load_mod = [&](int mod) {
    const __amdgpu_buffer_rsrc_t shb = row_buf(shift, (int64_t)mod * ld_mod * 2, K * 2);
    const __amdgpu_buffer_rsrc_t scb = row_buf(scale_mod, (int64_t)mod * ld_mod * 2, K * 2);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const u4v sh = __builtin_amdgcn_raw_buffer_load_b128(shb, idx[c] * 16, 0, kCached);
      const u4v sc = __builtin_amdgcn_raw_buffer_load_b128(scb, idx[c] * 16, 0, kCached);
      widen_mod(c, sh, sc);
    }
    cur_mod = mod;
  };
  auto load_row = [&](int row, u4v (&dst)[CH]) {
    const __amdgpu_buffer_rsrc_t xb = row_buf(x, (int64_t)row * ld_x * 2, K * 2);
#pragma unroll
    for (int c = 0; c < CH; ++c) dst[c] = __builtin_amdgcn_raw_buffer_load_b128(xb, idx[c] * 16, 0, kCached);
  };
  // sum of (a, b) over the workgroup, the same in every thread
  auto block_sum2 = [&](float& a, float& b, float (*slot)[2]) {
    a = __uint_as_float(wave_reduce_to_lane63(__float_as_uint(a), AddF32{}));
    b = __uint_as_float(wave_reduce_to_lane63(__float_as_uint(b), AddF32{}));
    if constexpr (WAVES == 1) {
      a = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(a), 63));
      b = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(b), 63));
    } else {
      if (lane == 63) {
        slot[wave][0] = a;
        slot[wave][1] = b;
      }
      __syncthreads();
      a = slot[0][0] + slot[1][0];
      b = slot[0][1] + slot[1][1];
#pragma unroll
      for (int w = 2; w < WAVES; w += 2) {  // a fixed order of additions
        a += slot[w][0] + slot[w + 1][0];
        b += slot[w][1] + slot[w + 1][1];
      }
    }
  };
  auto block_max = [&](uint32_t m, uint32_t* slot) -> uint32_t {
    m = wave_reduce_to_lane63(m, MaxU32{});
    if constexpr (WAVES == 1) return (uint32_t)__builtin_amdgcn_readlane((int)m, 63);
    if (lane == 63) slot[wave] = m;
    __syncthreads();
    uint32_t r = max(slot[0], slot[1]);
#pragma unroll
    for (int w = 2; w < WAVES; w += 2) r = max(r, max(slot[w], slot[w + 1]));
    return r;
  };

  // One row: `cur` holds it, `nxt` receives the row after it (the last row once more where
  // there is none: a load that is never used, so that the count of accesses stays fixed).
  auto one_row = [&](int row, u4v (&cur)[CH], u4v (&nxt)[CH]) {
    const int par = row & 1;
    const int mod = row / rows_per_mod;
    if (mod != cur_mod) load_mod(mod);  // uniform, rare
    load_row(min(row + 1, row_end - 1), nxt);

    float sum = 0.0f, sq = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        sum = dot_pair(cur[c][e], 0x3f803f80u, sum);
        sq = dot_pair(cur[c][e], cur[c][e], sq);
      }
    block_sum2(sum, sq, red_f[par]);
    const float mean = sum * inv_k;
    float var = sq * inv_k - mean * mean;
    if (!(mean * mean <= 4.0f * var)) {  // uniform; also taken by var <= 0 and by NaN
      float ss = 0.0f, unused = 0.0f;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const bool valid = idx[c] < nchunks;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          uint32_t w = cur[c][e];
          asm volatile("" : "+v"(w));  // keeps this path's widening inside the (cold) branch
          const float a = valid ? bf16_lo(w) - mean : 0.0f;
          const float b = valid ? bf16_hi(w) - mean : 0.0f;
          ss = __fmaf_rn(a, a, ss);
          ss = __fmaf_rn(b, b, ss);
        }
      }
      __syncthreads();  // the slots of this parity are read by everyone before they are reused
      block_sum2(ss, unused, red_f[par]);
      var = ss * inv_k;
    }
    // (v_rsq_f32, about an ulp: the statistics are fp32 sums in an order of their own anyway)
    const float rstd = __builtin_amdgcn_rsqf(var + eps);
    const float off = -mean * rstd;

    uint32_t mpos = 0, mneg = 0;  // signed and unsigned maxima of the raw bits
    float yv[CH][8];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float n0 = round_bf16_wide(__fmaf_rn(bf16_lo(cur[c][e]), rstd, off));
        const float n1 = round_bf16_wide(__fmaf_rn(bf16_hi(cur[c][e]), rstd, off));
        const float u0 = round_bf16_wide(n0 * t_f[c][2 * e]);
        const float u1 = round_bf16_wide(n1 * t_f[c][2 * e + 1]);
        const float y0 = round_bf16_wide(u0 + sh_f[c][2 * e]);
        const float y1 = round_bf16_wide(u1 + sh_f[c][2 * e + 1]);
        yv[c][2 * e] = y0;
        yv[c][2 * e + 1] = y1;
        const int b0 = __float_as_int(y0), b1 = __float_as_int(y1);
        mpos = (uint32_t)max(max((int)mpos, b0), b1);          // v_max3_i32: the largest positive pattern
        mneg = max(max(mneg, (uint32_t)b0), (uint32_t)b1);     // v_max3_u32: the largest negative one
      }
      if constexpr (WRITE_Y) {
        const __amdgpu_buffer_rsrc_t yb = row_buf(y, (int64_t)row * ld_y * 2, K * 2);
        const u4v packed = {pack_wide(yv[c][0], yv[c][1]), pack_wide(yv[c][2], yv[c][3]),
                            pack_wide(yv[c][4], yv[c][5]), pack_wide(yv[c][6], yv[c][7])};
        __builtin_amdgcn_raw_buffer_store_b128(packed, yb, idx[c] * 16, 0, kCached);
      }
    }
    // magnitude bits of the larger of the two (mneg only counts when it is a negative pattern)
    const uint32_t mag_neg = (mneg & 0x80000000u) ? (mneg & 0x7fffffffu) : 0u;
    uint32_t m = max(mpos, mag_neg) >> 16;  // bf16 bit pattern of max |y|
    m = block_max(m, red_m[par]);
    const float s = row_scale(m, scale_mode);
    // thread 0 writes the scale; everyone else's offset lies beyond the 4-byte descriptor
    __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(s), row_buf(scale, (int64_t)row * 4, 4),
                                          threadIdx.x == 0 ? 0 : 4, 0, kCached);
    u2v o[CH];
    if (scale_in_fast_window(s)) {  // uniform
      const Recip r = make_recip(s);
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        uint32_t p[2] = {0u, 0u};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float a = div_scale<true>(yv[c][2 * e], s, r), b = div_scale<true>(yv[c][2 * e + 1], s, r);
          p[e >> 1] = (e & 1) ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, p[e >> 1], true)
                              : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, p[e >> 1], false);
        }
        o[c] = u2v{p[0], p[1]};
      }
    } else {
#pragma unroll 1
      for (int c = 0; c < CH; ++c) {
        uint32_t p[2] = {0u, 0u};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float a = clamp448(yv[c][2 * e] / s), b = clamp448(yv[c][2 * e + 1] / s);
          p[e >> 1] = (e & 1) ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, p[e >> 1], true)
                              : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, p[e >> 1], false);
        }
        o[c] = u2v{p[0], p[1]};
      }
    }
    const __amdgpu_buffer_rsrc_t qb = row_buf(q, (int64_t)row * ld_q, K);
#pragma unroll
    for (int c = 0; c < CH; ++c) __builtin_amdgcn_raw_buffer_store_b64(o[c], qb, idx[c] * 8, 0, kCached);
  };

  u4v va[CH], vb[CH];
  // The modulation vectors first: they come from the L2 (every workgroup reads the same two)
  // and are widened while the first row is still on its way from memory.
  {
    const __amdgpu_buffer_rsrc_t xb = row_buf(x, (int64_t)row0 * ld_x * 2, K * 2);
    const int mod = row0 / rows_per_mod;
    const __amdgpu_buffer_rsrc_t shb = row_buf(shift, (int64_t)mod * ld_mod * 2, K * 2);
    const __amdgpu_buffer_rsrc_t scb = row_buf(scale_mod, (int64_t)mod * ld_mod * 2, K * 2);
    u4v sh[CH], sc[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      sh[c] = __builtin_amdgcn_raw_buffer_load_b128(shb, idx[c] * 16, 0, kCached);
      sc[c] = __builtin_amdgcn_raw_buffer_load_b128(scb, idx[c] * 16, 0, kCached);
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) va[c] = __builtin_amdgcn_raw_buffer_load_b128(xb, idx[c] * 16, 0, kCached);
#pragma unroll
    for (int c = 0; c < CH; ++c) widen_mod(c, sh[c], sc[c]);
    cur_mod = mod;
  }
  {
    // As many stores as a row issues, every lane beyond its descriptor (nothing is written):
    // the first row then meets the same sequence of accesses in flight as every later one,
    // and the wait for its data is the same count (the compiler takes the smaller of the two
    // otherwise, which makes every other row wait for stores of the row before it).
    const __amdgpu_buffer_rsrc_t none = row_buf(scale, 0, 0);
    if constexpr (WRITE_Y) {
#pragma unroll
      for (int c = 0; c < CH; ++c) __builtin_amdgcn_raw_buffer_store_b128(va[0], none, 0, 0, kCached);
    }
    __builtin_amdgcn_raw_buffer_store_b32(0u, none, 0, 0, kCached);
#pragma unroll
    for (int c = 0; c < CH; ++c) __builtin_amdgcn_raw_buffer_store_b64(u2v{0u, 0u}, none, 0, 0, kCached);
  }
  for (int row = row0;;) {
    one_row(row, va, vb);
    if (++row >= row_end) break;
    one_row(row, vb, va);
    if (++row >= row_end) break;
  }
}

// Any K and alignment: the same arithmetic element by element; y is recomputed in the
// cast pass (the row is an L2 hit by then).
__global__ __launch_bounds__(64) void ln_modulate_quant_generic(
    const uint16_t* __restrict__ x, int64_t ld_x, const uint16_t* __restrict__ shift,
    const uint16_t* __restrict__ scale_mod, int64_t ld_mod, int rows_per_mod, float eps,
    uint16_t* __restrict__ y, int64_t ld_y, uint8_t* __restrict__ q, int64_t ld_q,
    float* __restrict__ scale, int M, int K, int scale_mode) {
  const int lane = threadIdx.x & 63;
  const float inv_k = 1.0f / (float)K;
  auto f = [](uint16_t b) { return __uint_as_float((uint32_t)b << 16); };
  for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
    const uint16_t* xr = x + row * ld_x;
    const uint16_t* shr = shift + (row / rows_per_mod) * ld_mod;
    const uint16_t* scr = scale_mod + (row / rows_per_mod) * ld_mod;
    float sum = 0.0f;
    for (int k = lane; k < K; k += 64) sum += f(xr[k]);
    const float mean = wave_sum_f32(sum) * inv_k;
    float ss = 0.0f;
    for (int k = lane; k < K; k += 64) {
      const float a = f(xr[k]) - mean;
      ss = __fmaf_rn(a, a, ss);
    }
    const float rstd = 1.0f / sqrtf(wave_sum_f32(ss) * inv_k + eps);
    uint32_t m = 0;
    for (int k = lane; k < K; k += 64) {
      const uint32_t yb = modulate1(f(xr[k]), mean, rstd, f(scr[k]), f(shr[k]));
      if (y) y[row * ld_y + k] = (uint16_t)yb;
      const uint32_t a = yb & 0x7fffu;
      m = m > a ? m : a;
    }
    m = wave_max_u32(m);
    const float s = row_scale(m, scale_mode);
    if (lane == 0) scale[row] = s;
    for (int k = lane; k < K; k += 64) {
      const uint32_t yb = modulate1(f(xr[k]), mean, rstd, f(scr[k]), f(shr[k]));
      const float v = clamp448(__uint_as_float(yb << 16) / s);
      q[row * ld_q + k] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(v, v, 0u, false) & 0xffu);
    }
  }
}

}  // namespace

// Cache hints of the row-in-registers kernel. 0: non-temporal loads and stores; 1: both plain;
// 2: non-temporal loads only; 3: non-temporal stores only; -1 (default): when the GEMM that
// reads the codes follows in the same call (the fused Linear entry point) 1 for activations
// of up to 64 MB and 2 above, else 3 up to 64 MB and 0 above. Measured on activations that
// come from HBM: 4608 x 3072 (28 MB) 9.2 / 10.9 / 9.8 / 8.4 us for 0 / 1 / 2 / 3, 4608 x
// 15360 (142 MB) 40.8 / 47.6 / 40.5 / 43.3, 32760 x 5120 (335 MB) 81 / 92 / 88 / 87; inside
// a step of 494 fused Linears with one hint for all of them 1 is the fastest, 3 is 1.1 % and
// 0 2.3 % behind; quantizer + GEMM of one Linear, 0 / 1 / 2 / 3: 4608 x 15360 x 3072 186.9 /
// 187.0 / 183.8 / 190.6 us, K = 12288 150.9 / 150.7 / 148.1 / 154.1, 4608 x 3072 x 12288
// 144.4 / 143.4 / 144.9 / 145.5, N = 3072 47.1 / 46.1 / 48.2 / 45.8.
int g_quant_variant = -1;

int launch_quant_rowwise(const void* x, int64_t M, int64_t K, int64_t ld_x, void* q,
                         int64_t ld_q, float* scale, int scale_mode, bool consumer_follows,
                         hipStream_t stream) {
  const uint16_t* xp = static_cast<const uint16_t*>(x);
  uint8_t* qp = static_cast<uint8_t*>(q);
  const bool aligned = (K % 8 == 0) && (ld_x % 8 == 0) && (ld_q % 8 == 0) &&
                       (reinterpret_cast<uintptr_t>(x) % 16 == 0) &&
                       (reinterpret_cast<uintptr_t>(q) % 8 == 0);
  // one wavefront per workgroup: rows spread evenly over the CUs whatever M is
  constexpr int kThreads = 64, kWaves = kThreads / 64;
  int64_t blocks = (M + kWaves - 1) / kWaves;
  // enough blocks to cover the chip many times over; rows beyond that are
  // picked up by the grid-stride loop.
  const int64_t kMaxBlocks = 256 * 256;
  if (blocks > kMaxBlocks) blocks = kMaxBlocks;
  dim3 grid((unsigned)blocks), block(kThreads);
  const int Mi = (int)M, Ki = (int)K;
  const int need = (int)((K + 511) / 512);  // 16-byte chunks per lane
  // Cache hints (0: loads and stores non-temporal, 1: neither, 2: loads, 3: stores) and,
  // from 4 on, the same hints with two wavefronts per row. Codes that a GEMM reads next
  // keep their stores cacheable; activations beyond 64 MB are loaded non-temporally; two
  // wavefronts per row wherever a GEMM follows, and for a stand-alone call on long rows or
  // large activations (one wavefront per row is the faster at 4608 x 3072 on its own:
  // 8.0 against 8.2 us).
  const bool large = M * K * 2 > ((int64_t)64 << 20);
  const int hints = g_quant_variant >= 0 ? g_quant_variant
                    : consumer_follows   ? (large ? 6 : 5)
                    : large              ? 4
                    : K >= 8192          ? 7
                                         : 3;
  if (aligned && hints >= 4 && need >= 2 && need <= 32) {
    // several wavefronts per row: two up to 3584 elements, four beyond (measured: four gain
    // another 2-4 % from K = 5120 on and lose 3-8 % at K = 3072)
    const int h = hints & 3;
#define CDIT_SPLIT_LAUNCH(W, CH, NL, NS)                                                        \
  hipLaunchKernelGGL((quant_rowwise_split2<CH, NL, NS, false, W>), grid, dim3(64 * W), 0, stream, \
                     xp, ld_x, qp, ld_q, scale, Mi, Ki, scale_mode)
#define CDIT_SPLIT_CASE(W, CH)                                                                  \
  if (need <= W * CH) {                                                                         \
    switch (h) {                                                                                \
      case 0: CDIT_SPLIT_LAUNCH(W, CH, true, true); break;                                      \
      case 2: CDIT_SPLIT_LAUNCH(W, CH, true, false); break;                                     \
      case 3: CDIT_SPLIT_LAUNCH(W, CH, false, true); break;                                     \
      default: CDIT_SPLIT_LAUNCH(W, CH, false, false); break;                                   \
    }                                                                                           \
    return 0;                                                                                   \
  }
    if (need < 8) {
      CDIT_SPLIT_CASE(2, 1) CDIT_SPLIT_CASE(2, 2) CDIT_SPLIT_CASE(2, 3) CDIT_SPLIT_CASE(2, 4)
    } else {
      CDIT_SPLIT_CASE(4, 2) CDIT_SPLIT_CASE(4, 3) CDIT_SPLIT_CASE(4, 4) CDIT_SPLIT_CASE(4, 5)
      CDIT_SPLIT_CASE(4, 6) CDIT_SPLIT_CASE(4, 7) CDIT_SPLIT_CASE(4, 8)
    }
#undef CDIT_SPLIT_CASE
#undef CDIT_SPLIT_LAUNCH
  }
#define CDIT_QUANT_LAUNCH(CH, NL, NS)                                                        \
  hipLaunchKernelGGL((quant_rowwise_regs<CH, NL, NS>), grid, block, 0, stream, xp, ld_x, qp,   \
                     ld_q, scale, Mi, Ki, scale_mode)
#define CDIT_QUANT_CASE(CH)                                                                  \
  if (aligned && need <= CH) {                                                               \
    switch (hints & 3) {                                                                         \
      case 0: CDIT_QUANT_LAUNCH(CH, true, true); break;                                      \
      case 2: CDIT_QUANT_LAUNCH(CH, true, false); break;                                     \
      case 3: CDIT_QUANT_LAUNCH(CH, false, true); break;                                     \
      default: CDIT_QUANT_LAUNCH(CH, false, false); break;                                   \
    }                                                                                        \
    return 0;                                                                                \
  }
  CDIT_QUANT_CASE(1)
  CDIT_QUANT_CASE(2)
  CDIT_QUANT_CASE(4)
  CDIT_QUANT_CASE(6)
  CDIT_QUANT_CASE(8)
  CDIT_QUANT_CASE(10)
  CDIT_QUANT_CASE(12)
  CDIT_QUANT_CASE(16)
  CDIT_QUANT_CASE(20)
  CDIT_QUANT_CASE(24)
  CDIT_QUANT_CASE(27)
  CDIT_QUANT_CASE(30)
  CDIT_QUANT_CASE(32)
#undef CDIT_QUANT_CASE
#undef CDIT_QUANT_LAUNCH
  hipLaunchKernelGGL(quant_rowwise_generic, grid, block, 0, stream, xp, ld_x, qp, ld_q, scale, Mi,
                     Ki, scale_mode);
  return 0;
}

// 0: launched; 1: not taken (K1 or K2 not a multiple of 8, rows not 16-byte aligned,
// K1 + K2 beyond the register-resident kernel).
int launch_quant_rowwise_cat2(const void* x1, int64_t K1, int64_t ld_x1, const void* x2, int64_t K2,
                              int64_t ld_x2, int64_t M, void* q, int64_t ld_q, float* scale,
                              int scale_mode, hipStream_t stream) {
  const int64_t K = K1 + K2;
  const bool aligned = K1 % 8 == 0 && K2 % 8 == 0 && K <= 32 * 512 && ld_x1 % 8 == 0 && ld_x2 % 8 == 0 &&
                       ld_q % 8 == 0 && reinterpret_cast<uintptr_t>(x1) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(x2) % 16 == 0 &&
                       reinterpret_cast<uintptr_t>(q) % 8 == 0;
  if (!aligned || M <= 0) return 1;
  dim3 grid((unsigned)(M < 256 * 256 ? M : 256 * 256));
  const int need = (int)((K + 511) / 512);
  // the codes are read by the GEMM that follows: plain stores; loads of a large activation
  // carry the non-temporal hint (as launch_quant_rowwise chooses)
  const bool nt_load = M * K * 2 > ((int64_t)64 << 20);
  const uint16_t* p1 = static_cast<const uint16_t*>(x1);
  const uint16_t* p2 = static_cast<const uint16_t*>(x2);
#define CDIT_QUANT_CASE(W, CH)                                                                      \
  if (need <= W * CH) {                                                                             \
    if (nt_load) {                                                                                  \
      hipLaunchKernelGGL((quant_rowwise_cat_regs<CH, true, W>), grid, dim3(64 * W), 0, stream, p1,  \
                         ld_x1, (int)(K1 / 8), p2, ld_x2, static_cast<uint8_t*>(q), ld_q, scale,   \
                         (int)M, (int)K, scale_mode);                                               \
    } else {                                                                                        \
      hipLaunchKernelGGL((quant_rowwise_cat_regs<CH, false, W>), grid, dim3(64 * W), 0, stream, p1, \
                         ld_x1, (int)(K1 / 8), p2, ld_x2, static_cast<uint8_t*>(q), ld_q, scale,   \
                         (int)M, (int)K, scale_mode);                                               \
    }                                                                                               \
    return 0;                                                                                       \
  }
  if (need < 2) {  // wavefronts per row as in launch_quant_rowwise
    CDIT_QUANT_CASE(1, 1)
  } else if (need < 8) {
    CDIT_QUANT_CASE(2, 1) CDIT_QUANT_CASE(2, 2) CDIT_QUANT_CASE(2, 3) CDIT_QUANT_CASE(2, 4)
  } else {
    CDIT_QUANT_CASE(4, 2) CDIT_QUANT_CASE(4, 3) CDIT_QUANT_CASE(4, 4) CDIT_QUANT_CASE(4, 5)
    CDIT_QUANT_CASE(4, 6) CDIT_QUANT_CASE(4, 7) CDIT_QUANT_CASE(4, 8)
  }
#undef CDIT_QUANT_CASE
  return 1;
}

int launch_quant_rowwise_batched(const QuantBatch& batch, int64_t K, int scale_mode,
                                 hipStream_t stream) {
  const int64_t M = batch.row_begin[batch.acts];
  bool aligned = K % 8 == 0 && K > 0 && K <= 32 * 512;
  for (int s = 0; s < batch.acts; ++s)
    aligned = aligned && batch.ld_x[s] % 8 == 0 && batch.ld_q[s] % 8 == 0 &&
              reinterpret_cast<uintptr_t>(batch.x[s]) % 16 == 0 &&
              reinterpret_cast<uintptr_t>(batch.q[s]) % 8 == 0;
  if (!aligned || M <= 0) return 1;
  int64_t blocks = M < 256 * 256 ? M : 256 * 256;
  dim3 grid((unsigned)blocks), block(64);
  const int Mi = (int)M, Ki = (int)K;
  const int need = (int)((K + 511) / 512);
  // the codes are read by the GEMM that follows: cacheable stores; loads of a large batch
  // carry the non-temporal hint (as launch_quant_rowwise chooses for one activation)
  const bool nt_load = g_quant_variant >= 0 ? ((g_quant_variant & 3) == 0 || (g_quant_variant & 3) == 2)
                                            : M * K * 2 > ((int64_t)64 << 20);
#define CDIT_QUANT_CASE(W, CH)                                                                   \
  if (need <= W * CH) {                                                                          \
    if (nt_load) {                                                                               \
      hipLaunchKernelGGL((quant_rowwise_split2<CH, true, false, true, W>), grid, dim3(64 * W), 0, \
                         stream, nullptr, 0, nullptr, 0, nullptr, Mi, Ki, scale_mode, batch);    \
    } else {                                                                                     \
      hipLaunchKernelGGL((quant_rowwise_split2<CH, false, false, true, W>), grid, dim3(64 * W), 0, \
                         stream, nullptr, 0, nullptr, 0, nullptr, Mi, Ki, scale_mode, batch);    \
    }                                                                                            \
    return 0;                                                                                    \
  }
  if (need >= 2 && need < 8) {  // wavefronts per row as in launch_quant_rowwise
    CDIT_QUANT_CASE(2, 1) CDIT_QUANT_CASE(2, 2) CDIT_QUANT_CASE(2, 3) CDIT_QUANT_CASE(2, 4)
  } else if (need >= 8) {
    CDIT_QUANT_CASE(4, 2) CDIT_QUANT_CASE(4, 3) CDIT_QUANT_CASE(4, 4) CDIT_QUANT_CASE(4, 5)
    CDIT_QUANT_CASE(4, 6) CDIT_QUANT_CASE(4, 7) CDIT_QUANT_CASE(4, 8)
  }
#undef CDIT_QUANT_CASE
  if (need == 1) {  // rows of up to 512 elements: one wavefront each
    if (nt_load) {
      hipLaunchKernelGGL((quant_rowwise_regs<1, true, false, true>), grid, block, 0, stream, nullptr, 0,
                         nullptr, 0, nullptr, Mi, Ki, scale_mode, batch);
    } else {
      hipLaunchKernelGGL((quant_rowwise_regs<1, false, false, true>), grid, block, 0, stream, nullptr,
                         0, nullptr, 0, nullptr, Mi, Ki, scale_mode, batch);
    }
    return 0;
  }
  return 1;
}

// CUs of the current device, `fallback` when the query fails
static int64_t cu_count_or(int64_t fallback) {
  static int cached[64];  // per device ordinal; the answer cannot change
  int dev = 0, n = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fallback;
  if (dev >= 0 && dev < 64 && cached[dev] > 0) return cached[dev];
  if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
    return fallback;
  if (dev >= 0 && dev < 64) cached[dev] = n;
  return n;
}

int launch_ln_modulate_quant(const void* x, int64_t M, int64_t K, int64_t ld_x, const void* shift,
                             const void* scale_mod, int64_t ld_mod, int64_t rows_per_mod, float eps,
                             void* y, int64_t ld_y, void* q, int64_t ld_q, float* scale,
                             int scale_mode, hipStream_t stream) {
  const uint16_t* xp = static_cast<const uint16_t*>(x);
  const uint16_t* shp = static_cast<const uint16_t*>(shift);
  const uint16_t* scp = static_cast<const uint16_t*>(scale_mod);
  uint16_t* yp = static_cast<uint16_t*>(y);
  uint8_t* qp = static_cast<uint8_t*>(q);
  auto a16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool aligned = K % 8 == 0 && ld_x % 8 == 0 && ld_q % 8 == 0 && ld_mod % 8 == 0 &&
                       (!y || (ld_y % 8 == 0 && a16(y))) && a16(x) && a16(shift) &&
                       a16(scale_mod) && reinterpret_cast<uintptr_t>(q) % 8 == 0;
  int64_t blocks = M;
  const int64_t kMaxBlocks = 256 * 256;
  if (blocks > kMaxBlocks) blocks = kMaxBlocks;
  dim3 grid((unsigned)blocks), block(64);
  const int need = (int)((K + 511) / 512);
  // Wavefronts per row: the fewest of 1, 2, 4, 8 that leave a thread at most three chunks of 8
  // elements (the row, the prefetched next row and the two modulation vectors live in
  // registers: 153 at three chunks, three wavefronts per SIMD); rows beyond 12288 elements
  // take four chunks at eight wavefronts (K <= 16384). Workgroups: about six wavefronts'
  // worth per SIMD (twice what is resident at once), each with the same number of
  // consecutive rows.
  if (aligned && need <= 32) {
    int waves = 8;
    for (int w = 1; w <= 8; w *= 2)
      if ((need + w - 1) / w <= 3) {
        waves = w;
        break;
      }
    const int ch = (need + waves - 1) / waves;
    const int64_t cus = cu_count_or(256);
    // (measured at 4608 x 3072: 16.1 us with 16 wavefronts' worth of workgroups per CU, 15.2
    // with 20 or 24; four wavefronts of two chunks per row instead of two of three: 17.4-17.7)
    // (32760 x 5120: 104.7 us with 48 wavefronts' worth per CU, 11 rows each, against 107.8
    // with 24; with fewer than eight rows per workgroup the smaller number wins)
    int64_t target = cus * 48 / waves;
    if (M < 8 * target) target = cus * 24 / waves;
    const int rows_per_wg = (int)((M + target - 1) / target);
    const dim3 rgrid((unsigned)((M + rows_per_wg - 1) / rows_per_wg));
#define CDIT_LNQ_LAUNCH(W, CH, WY)                                                              \
  hipLaunchKernelGGL((ln_modulate_quant_rows<CH, WY, W>), rgrid, dim3(64 * W), 0, stream, xp,   \
                     ld_x, shp, scp, ld_mod, (int)rows_per_mod, eps, yp, ld_y, qp, ld_q, scale, \
                     (int)M, (int)K, scale_mode, rows_per_wg)
#define CDIT_LNQ_CASE(W, CH)                  \
  if (waves == W && ch <= CH) {               \
    if (y)                                    \
      CDIT_LNQ_LAUNCH(W, CH, true);           \
    else                                      \
      CDIT_LNQ_LAUNCH(W, CH, false);          \
    return 0;                                 \
  }
    CDIT_LNQ_CASE(1, 1) CDIT_LNQ_CASE(1, 2) CDIT_LNQ_CASE(1, 3)
    CDIT_LNQ_CASE(2, 2) CDIT_LNQ_CASE(2, 3)
    CDIT_LNQ_CASE(4, 2) CDIT_LNQ_CASE(4, 3)
    CDIT_LNQ_CASE(8, 2) CDIT_LNQ_CASE(8, 3) CDIT_LNQ_CASE(8, 4)
#undef CDIT_LNQ_CASE
#undef CDIT_LNQ_LAUNCH
  }
  hipLaunchKernelGGL(ln_modulate_quant_generic, grid, block, 0, stream, xp, ld_x, shp, scp, ld_mod,
                     (int)rows_per_mod, eps, yp, ld_y, qp, ld_q, scale, (int)M, (int)K, scale_mode);
  return 0;
}

int launch_quant_tensorwise(const void* x, int64_t M, int64_t K, int64_t ld_x, void* q,
                            int64_t ld_q, float* scale, uint32_t* amax_ws, int scale_mode,
                            hipStream_t stream) {
  const uint16_t* xp = static_cast<const uint16_t*>(x);
  uint8_t* qp = static_cast<uint8_t*>(q);
  const bool vec = (K % 8 == 0) && (ld_x % 8 == 0) && (ld_q % 8 == 0) &&
                   (reinterpret_cast<uintptr_t>(x) % 16 == 0) &&
                   (reinterpret_cast<uintptr_t>(q) % 8 == 0);
  int64_t blocks = M;
  const int64_t kMaxBlocks = 256 * 64;  // the rest is picked up by the grid-stride loops
  if (blocks > kMaxBlocks) blocks = kMaxBlocks;
  hipLaunchKernelGGL(zero_amax, dim3(1), dim3(1), 0, stream, amax_ws);
  if (vec && K <= 32 * 512) {
    const int need = (int)((K + 511) / 512);
#define CDIT_PT_CASE(CH)                                                                           \
  if (need <= CH) {                                                                                \
    hipLaunchKernelGGL(tensor_amax_rows<CH>,                                                       \
                       dim3((unsigned)std::min<int64_t>((M + kAmaxWaves - 1) / kAmaxWaves, cu_count_or(256))), \
                       dim3(64 * kAmaxWaves), 0, stream, xp, ld_x, (int)M, (int)K, amax_ws);        \
    hipLaunchKernelGGL(quant_tensorwise_cast_rows<CH>, dim3((unsigned)blocks), dim3(64), 0, stream,  \
                       xp, ld_x, qp, ld_q, scale, (int)M, (int)K, scale_mode, amax_ws);            \
    return 0;                                                                                      \
  }
    CDIT_PT_CASE(1) CDIT_PT_CASE(2) CDIT_PT_CASE(3) CDIT_PT_CASE(4) CDIT_PT_CASE(6) CDIT_PT_CASE(8)
    CDIT_PT_CASE(12) CDIT_PT_CASE(16) CDIT_PT_CASE(24) CDIT_PT_CASE(32)
#undef CDIT_PT_CASE
  }
  hipLaunchKernelGGL(tensor_amax, dim3((unsigned)blocks), dim3(64), 0, stream, xp, ld_x, (int)M,
                     (int)K, vec, amax_ws);
  hipLaunchKernelGGL(quant_tensorwise_cast, dim3((unsigned)blocks), dim3(64), 0, stream, xp, ld_x,
                     qp, ld_q, scale, (int)M, (int)K, scale_mode, vec, amax_ws);
  return 0;
}

}  // namespace cdit
