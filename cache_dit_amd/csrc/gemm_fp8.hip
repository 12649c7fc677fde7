// Row-wise scaled FP8 (e4m3 x e4m3 -> fp32) GEMM for gfx950 with the scale /
// bias / GELU-tanh / bf16 epilogue fused in.
//
//   out[m,n] = epi((sum_k a[m,k] b[n,k]) * a_scale[m] * b_scale[n] + bias[n])
//
// Both operands are K-contiguous ("NT" GEMM), which is what the MFMA operand
// registers want: v_mfma_f32_32x32x64_f8f6f4 takes, per lane, 32 consecutive
// K bytes of one row (lane&31) in K-half (lane>>5).
//
// Tiled kernel: a workgroup of WGM x WGN wavefronts owns a BM x BN output
// tile and walks K in steps of BK = 128 bytes. A and B panels are staged in
// LDS, double buffered; rows are 128 B = 8 chunks of 16 B and chunk c of row r
// is stored at chunk position c ^ (r & 7), which makes both the 16-byte
// staging writes and the 16-byte operand reads bank-conflict free.
// Panels reach LDS either through registers (global_load_dwordx4 +
// ds_write_b128) or directly (global_load_lds_dwordx4, gfx950's 128-bit
// LDS-DMA, 1 KiB of LDS per wavefront instruction).
//
// The MFMA is issued with the operands swapped (B rows first), so that every
// lane ends up with 4 consecutive output columns per accumulator group: the
// epilogue packs them to bf16 and either stores 8 bytes directly or goes
// through a per-wave LDS transpose to store 16 bytes per lane along rows.
//
// Replaces torch._scaled_mm as called at
// src/cache_dit/quantization/torchao/_scaled_mm.py:62-91.
#include "gemm_common.h"

namespace cdit {
namespace {

constexpr int BK = 128;  // bytes of K per pipeline step (two 64-wide MFMA steps)

template <int BM_, int BN_, int WGM_, int WGN_, bool DIRECT_, bool EPI_LDS_, int GROUP_M_>
struct Cfg {
  static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
  static constexpr bool DIRECT = DIRECT_, EPI_LDS = EPI_LDS_;
  static constexpr int GROUP_M = GROUP_M_;
  static constexpr int WAVES = WGM * WGN;
  static constexpr int THREADS = WAVES * 64;
  static constexpr int WM = BM / WGM, WN = BN / WGN;  // wave tile
  static constexpr int TM = WM / 32, TN = WN / 32;    // 32x32 MFMA tiles per wave
  static constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int EPI_PITCH = WN * 2 + 16;  // bytes per row of the per-wave transpose tile
  static constexpr int EPI_BYTES = EPI_LDS ? WAVES * WM * EPI_PITCH : 0;
  static constexpr int LDS_BYTES = (2 * STAGE_BYTES > EPI_BYTES) ? 2 * STAGE_BYTES : EPI_BYTES;
  // staging: 16-byte chunks per thread and per wave instruction
  static constexpr int A_CHUNKS = BM * 8 / THREADS, B_CHUNKS = BN * 8 / THREADS;
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
  static_assert((BM * 8) % THREADS == 0 && (BN * 8) % THREADS == 0, "panel/threads mismatch");
  static_assert(BM % (8 * WAVES) == 0 && BN % (8 * WAVES) == 0, "panel/waves mismatch");
};

typedef __attribute__((address_space(3))) uint8_t lds_u8;

template <class C>
__global__ __launch_bounds__(C::THREADS) void gemm_fp8_tiled(GemmArgs g, int tiles_m,
                                                             int tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / C::WGN, wn = wave % C::WGN;

  int tm, tn;
  tile_of_block<C::GROUP_M>(blockIdx.x, gridDim.x, tiles_m, tiles_n, &tm, &tn);
  const int m0 = tm * C::BM, n0 = tn * C::BN;
  const uint8_t* __restrict__ A = static_cast<const uint8_t*>(g.a) + (int64_t)m0 * g.lda;
  const uint8_t* __restrict__ B = g.b + (int64_t)n0 * g.ldb;
  const int rows_a = g.M - m0;  // valid rows of this tile (may exceed BM)
  const int rows_b = g.N - n0;

  // ---- staging maps -------------------------------------------------------
  // Through registers: thread t owns chunk (row = t/8 + p*THREADS/8, c = t%8).
  // Direct: wave instruction i of wave w fills LDS rows [8*(w*n_i + i), +8);
  // lane l lands on row l/8, chunk position l%8, so it must fetch logical
  // chunk (l%8) ^ (l/8).
  uint32_t a_off[C::A_CHUNKS], b_off[C::B_CHUNKS];  // global byte offsets (without k0)
  uint32_t a_lds[C::A_CHUNKS], b_lds[C::B_CHUNKS];  // LDS byte offsets inside a stage
  if constexpr (!C::DIRECT) {
    const int c = tid & 7;
#pragma unroll
    for (int p = 0; p < C::A_CHUNKS; ++p) {
      const int row = (tid >> 3) + p * (C::THREADS / 8);
      a_off[p] = (uint32_t)min(row, rows_a - 1) * (uint32_t)g.lda + c * 16;
      a_lds[p] = row * BK + ((c ^ (row & 7)) << 4);
    }
#pragma unroll
    for (int p = 0; p < C::B_CHUNKS; ++p) {
      const int row = (tid >> 3) + p * (C::THREADS / 8);
      b_off[p] = (uint32_t)min(row, rows_b - 1) * (uint32_t)g.ldb + c * 16;
      b_lds[p] = C::A_BYTES + row * BK + ((c ^ (row & 7)) << 4);
    }
  } else {
    const int lrow = lane >> 3;
    const int c = (lane & 7) ^ lrow;
#pragma unroll
    for (int p = 0; p < C::A_CHUNKS; ++p) {
      const int rg = wave * C::A_CHUNKS + p;  // 8-row group
      const int row = rg * 8 + lrow;
      a_off[p] = (uint32_t)min(row, rows_a - 1) * (uint32_t)g.lda + c * 16;
      a_lds[p] = rg * 1024;  // wave-uniform base; the DMA adds lane*16
    }
#pragma unroll
    for (int p = 0; p < C::B_CHUNKS; ++p) {
      const int rg = wave * C::B_CHUNKS + p;
      const int row = rg * 8 + lrow;
      b_off[p] = (uint32_t)min(row, rows_b - 1) * (uint32_t)g.ldb + c * 16;
      b_lds[p] = C::A_BYTES + rg * 1024;
    }
  }

  // ---- operand read map ---------------------------------------------------
  // lane reads row (lane&31) of a 32-row MFMA block, K-half h = lane>>5 of the
  // 64-byte MFMA step s: logical chunks 4s+2h and 4s+2h+1.
  const int h = lane >> 5;
  uint32_t rd_a[2][2], rd_b[2][2];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int chunk = ((4 * s + 2 * h + e) ^ (lane & 7)) << 4;
      rd_a[s][e] = (wm * C::WM + (lane & 31)) * BK + chunk;
      rd_b[s][e] = C::A_BYTES + (wn * C::WN + (lane & 31)) * BK + chunk;
    }

  v16f acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int KT = g.K / BK;
  uint4 ra[C::A_CHUNKS], rb[C::B_CHUNKS];  // register staging (unused when DIRECT)

  auto fetch = [&](int kt, int stage) {
    const uint8_t* Ak = A + (int64_t)kt * BK;
    const uint8_t* Bk = B + (int64_t)kt * BK;
    if constexpr (C::DIRECT) {
      uint8_t* st = smem + stage * C::STAGE_BYTES;
#pragma unroll
      for (int p = 0; p < C::A_CHUNKS; ++p)
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(Ak + a_off[p]),
            (__attribute__((address_space(3))) void*)(st + a_lds[p]), 16, 0, 0);
#pragma unroll
      for (int p = 0; p < C::B_CHUNKS; ++p)
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(Bk + b_off[p]),
            (__attribute__((address_space(3))) void*)(st + b_lds[p]), 16, 0, 0);
    } else {
#pragma unroll
      for (int p = 0; p < C::A_CHUNKS; ++p)
        ra[p] = *reinterpret_cast<const uint4*>(Ak + a_off[p]);
#pragma unroll
      for (int p = 0; p < C::B_CHUNKS; ++p)
        rb[p] = *reinterpret_cast<const uint4*>(Bk + b_off[p]);
    }
  };
  auto commit = [&](int stage) {  // registers -> LDS (register staging only)
    if constexpr (!C::DIRECT) {
      uint8_t* st = smem + stage * C::STAGE_BYTES;
#pragma unroll
      for (int p = 0; p < C::A_CHUNKS; ++p) *reinterpret_cast<uint4*>(st + a_lds[p]) = ra[p];
#pragma unroll
      for (int p = 0; p < C::B_CHUNKS; ++p) *reinterpret_cast<uint4*>(st + b_lds[p]) = rb[p];
    }
  };
  auto compute = [&](int stage) {
    const uint8_t* st = smem + stage * C::STAGE_BYTES;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      v8i af[C::TM], bf[C::TN];
#pragma unroll
      for (int i = 0; i < C::TM; ++i) {
        const v4i lo = *reinterpret_cast<const v4i*>(st + rd_a[s][0] + i * 32 * BK);
        const v4i hi = *reinterpret_cast<const v4i*>(st + rd_a[s][1] + i * 32 * BK);
        af[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
#pragma unroll
      for (int j = 0; j < C::TN; ++j) {
        const v4i lo = *reinterpret_cast<const v4i*>(st + rd_b[s][0] + j * 32 * BK);
        const v4i hi = *reinterpret_cast<const v4i*>(st + rd_b[s][1] + j * 32 * BK);
        bf[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
#pragma unroll
      for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
          // operands swapped: result rows follow B (n), result columns follow A (m)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bf[j], af[i], acc[i][j], 0,
                                                                      0, 0, 0, 0, 0);
    }
  };

  // ---- main loop ----------------------------------------------------------
  if constexpr (C::DIRECT) {
    fetch(0, 0);
    for (int kt = 0; kt < KT; ++kt) {
      // tile kt has landed (this wave's part), then everyone's part; all waves
      // have also left compute(kt-1), so stage (kt+1)&1 may be overwritten.
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      __syncthreads();
      if (kt + 1 < KT) fetch(kt + 1, (kt + 1) & 1);
      compute(kt & 1);
    }
  } else {
    fetch(0, 0);
    commit(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      if (kt + 1 < KT) fetch(kt + 1, 0);
      compute(kt & 1);
      if (kt + 1 < KT) commit((kt + 1) & 1);
      __syncthreads();
    }
  }

  tile_epilogue<C>(acc, g, smem, m0, n0, wm, wn, lane, wave);
}

// Any shape, any alignment: a 16x16 output tile per workgroup, one output
// element per thread, scalar decode + FMA. Only for shapes the tiled kernel
// cannot take (K not a multiple of 128, N not a multiple of 8, odd strides).
__global__ __launch_bounds__(256) void gemm_fp8_generic(GemmArgs g) {
  const int n = blockIdx.x * 16 + (threadIdx.x & 15);
  const int m = blockIdx.y * 16 + (threadIdx.x >> 4);
  if (m >= g.M || n >= g.N) return;
  const uint8_t* a = static_cast<const uint8_t*>(g.a) + (int64_t)m * g.lda;
  const uint8_t* b = g.b + (int64_t)n * g.ldb;
  float acc = 0.0f;
  for (int k = 0; k < g.K; ++k) {
    const float x = __builtin_amdgcn_cvt_f32_fp8((int)a[k], 0);
    const float w = __builtin_amdgcn_cvt_f32_fp8((int)b[k], 0);
    acc = fmaf(x, w, acc);
  }
  float v = acc * g.a_scale[m] * g.b_scale[n];
  if (g.bias) v += __uint_as_float((uint32_t)g.bias[n] << 16);
  if (g.epilogue & CDIT_EPI_GELU_TANH) v = gelu_tanh(v);
  g.out[(int64_t)m * g.ldo + n] = (uint16_t)f32_to_bf16_bits(v);
}

template <class C>
int launch_tiled(const GemmArgs& g, hipStream_t stream) {
  static bool attr_set = false;  // benign race: setting it twice is harmless
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_fp8_tiled<C>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES);
    if (e != hipSuccess) {
      set_error("hipFuncSetAttribute(%d bytes LDS): %s", C::LDS_BYTES, hipGetErrorString(e));
      return CDIT_EHIP;
    }
    attr_set = true;
  }
  const int tiles_m = (g.M + C::BM - 1) / C::BM, tiles_n = (g.N + C::BN - 1) / C::BN;
  hipLaunchKernelGGL(gemm_fp8_tiled<C>, dim3(tiles_m * tiles_n), dim3(C::THREADS), C::LDS_BYTES,
                     stream, g, tiles_m, tiles_n);
  return 0;
}

bool tiled_ok(const GemmArgs& g) {
  return g.K >= BK && g.K % BK == 0 && g.N % 8 == 0 && g.lda % 16 == 0 && g.ldb % 16 == 0 && g.ldo % 8 == 0 &&
         reinterpret_cast<uintptr_t>(g.a) % 16 == 0 && reinterpret_cast<uintptr_t>(g.b) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(g.out) % 16 == 0 &&
         // 32-bit in-tile byte offsets
         (int64_t)512 * g.lda < (int64_t)1 << 31 && (int64_t)512 * g.ldb < (int64_t)1 << 31;
}

}  // namespace

//                 BM   BN  WGM WGN direct epiLDS groupM
typedef Cfg<256, 256, 2, 2, false, false, 8> V0;  // register staging, direct stores
typedef Cfg<256, 256, 2, 2, true, true, 8> V1;    // LDS-DMA staging, LDS-transposed stores
typedef Cfg<256, 256, 2, 2, false, true, 8> V2;
typedef Cfg<256, 256, 2, 2, true, false, 8> V3;
typedef Cfg<256, 128, 2, 2, true, true, 8> V4;
typedef Cfg<128, 256, 2, 2, true, true, 8> V5;
typedef Cfg<128, 128, 2, 2, true, true, 8> V6;
typedef Cfg<256, 256, 2, 4, true, true, 8> V7;  // 8 waves, 128x64 wave tiles

int launch_gemm_fp8(const GemmArgs& g, int variant, hipStream_t stream) {
  if (!tiled_ok(g) || variant == 100) {
    dim3 grid((g.N + 15) / 16, (g.M + 15) / 16);
    hipLaunchKernelGGL(gemm_fp8_generic, grid, dim3(256), 0, stream, g);
    return 0;
  }
  if (variant < 0) {
    // enough 256x256 tiles to cover the 256 CUs: the 8-wave kernel; else smaller tiles
    const int64_t big_tiles = (int64_t)((g.M + 255) / 256) * ((g.N + 255) / 256);
    variant = big_tiles >= 200 ? 7 : 6;
  }
  switch (variant) {
    case 0: return launch_tiled<V0>(g, stream);
    case 1: return launch_tiled<V1>(g, stream);
    case 2: return launch_tiled<V2>(g, stream);
    case 3: return launch_tiled<V3>(g, stream);
    case 4: return launch_tiled<V4>(g, stream);
    case 5: return launch_tiled<V5>(g, stream);
    case 6: return launch_tiled<V6>(g, stream);
    case 7: return launch_tiled<V7>(g, stream);
    default:
      set_error("cdit_fp8_gemm_rowwise: unknown kernel variant %d", variant);
      return CDIT_EINVAL;
  }
}

}  // namespace cdit
