// Row-wise scaled FP8 (e4m3 x e4m3 -> fp32) GEMM for gfx950 with the scale /
// bias / GELU-tanh / bf16 epilogue fused in.
//
//   out[m,n] = epi((sum_k a[m,k] b[n,k]) * a_scale[m] * b_scale[n] + bias[n])
//
// Both operands are K-contiguous ("NT" GEMM), which is what the MFMA operand
// registers want: per lane, 32 consecutive K bytes of one row. The production kernel
// (gemm_fp8_wide) issues v_mfma_f32_16x16x128_f8f6f4: row lane&15, 32-byte K group
// lane>>4 of a 128-byte K step; the older tiled kernel v_mfma_f32_32x32x64_f8f6f4: row
// lane&31, K half lane>>5 of a 64-byte step.
//
// Kernels in this file: gemm_fp8_wide (persistent, one wave per SIMD, the one every
// large or medium problem runs; described in front of CfgWide), gemm_fp8_tiled (the
// older kernel described next, kept for very short K), gemm_fp8_skinny and
// linear_fp8_skinny_fused (M <= 16), linear_fp8_row1 (M = 1, K <= 4096),
// gemm_fp8_generic (any shape and alignment).
//
// Tiled kernel: a workgroup of WGM x WGN wavefronts owns a BM x BN output
// tile and walks K in steps of BK = 128 bytes. A and B panels are staged in
// LDS, double buffered; rows are 128 B = 8 chunks of 16 B and chunk c of row r
// is stored at chunk position c ^ ((r >> 1) & 7). gfx950's LDS has 64 banks of
// 4 B (two panel rows per bank row) and serves a 16-byte access 16 lanes at a
// time (lanes of one half-wave whose bits 2..4 have equal parity), so this
// makes the operand reads bank-conflict free (measured: 190 B/clk/CU against
// 125 with c ^ (r & 7)).
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
#include <type_traits>

#include "gemm_common.h"
#include "quant_device.h"

namespace cdit {
namespace {

constexpr int BK = 128;  // bytes of K per pipeline step (two 64-wide MFMA steps)

template <int BM_, int BN_, int WGM_, int WGN_, bool DIRECT_, bool EPI_LDS_, int GROUP_M_,
          int STAGES_ = 2>
struct Cfg {
  static constexpr int STAGES = STAGES_;  // LDS buffers; more than 2 needs DIRECT staging
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
  static constexpr int EPI_BYTES = EPI_LDS ? WAVES * 32 * EPI_PITCH : 0;
  static constexpr int LDS_BYTES =
      (STAGES * STAGE_BYTES > EPI_BYTES) ? STAGES * STAGE_BYTES : EPI_BYTES;
  static_assert(STAGES == 2 || DIRECT, "multi-stage needs LDS-DMA staging");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
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
  // lane l lands on row l/8, chunk position l%8, so it must fetch the logical
  // chunk that the swizzle stores there.
  uint32_t a_off[C::A_CHUNKS], b_off[C::B_CHUNKS];  // global byte offsets (without k0)
  uint32_t a_lds[C::A_CHUNKS], b_lds[C::B_CHUNKS];  // LDS byte offsets inside a stage
  if constexpr (!C::DIRECT) {
    const int c = tid & 7;
#pragma unroll
    for (int p = 0; p < C::A_CHUNKS; ++p) {
      const int row = (tid >> 3) + p * (C::THREADS / 8);
      a_off[p] = (uint32_t)min(row, rows_a - 1) * (uint32_t)g.lda + c * 16;
      a_lds[p] = row * BK + ((c ^ ((row >> 1) & 7)) << 4);
    }
#pragma unroll
    for (int p = 0; p < C::B_CHUNKS; ++p) {
      const int row = (tid >> 3) + p * (C::THREADS / 8);
      b_off[p] = (uint32_t)min(row, rows_b - 1) * (uint32_t)g.ldb + c * 16;
      b_lds[p] = C::A_BYTES + row * BK + ((c ^ ((row >> 1) & 7)) << 4);
    }
  } else {
    const int lrow = lane >> 3;
#pragma unroll
    for (int p = 0; p < C::A_CHUNKS; ++p) {
      const int rg = wave * C::A_CHUNKS + p;  // 8-row group
      const int row = rg * 8 + lrow;
      const int c = (lane & 7) ^ ((row >> 1) & 7);
      a_off[p] = (uint32_t)min(row, rows_a - 1) * (uint32_t)g.lda + c * 16;
      a_lds[p] = rg * 1024;  // wave-uniform base; the DMA adds lane*16
    }
#pragma unroll
    for (int p = 0; p < C::B_CHUNKS; ++p) {
      const int rg = wave * C::B_CHUNKS + p;
      const int row = rg * 8 + lrow;
      const int c = (lane & 7) ^ ((row >> 1) & 7);
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
      const int chunk = ((4 * s + 2 * h + e) ^ ((lane >> 1) & 7)) << 4;
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
  if constexpr (C::DIRECT && C::STAGES > 2) {
    // STAGES-1 steps in flight; bare barriers with explicit vmcnt so that the
    // younger DMA keeps flying across them.
    constexpr int PD = C::STAGES - 1, D = C::A_CHUNKS + C::B_CHUNKS;
#pragma unroll
    for (int s = 0; s < PD; ++s)
      if (s < KT) fetch(s, s);
    wait_steps<D, PD - 1, true>(min(PD, KT) - 1);
    for (int kt = 0; kt < KT; ++kt) {
      // stage (kt+PD)%STAGES was read in iteration kt-1; the barrier that ended it
      // makes it free
      if (kt + PD < KT) fetch(kt + PD, (kt + PD) % C::STAGES);
      compute(kt % C::STAGES);
      wait_steps<D, PD - 1, true>(max(min(kt + PD, KT - 1) - (kt + 1), 0));
    }
  } else if constexpr (C::DIRECT) {
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

  if constexpr (C::EPI_LDS) __syncthreads();  // all waves are done with the stage buffers
  tile_epilogue<C>(acc, g, smem + wave * (32 * C::EPI_PITCH), m0, n0, wm, wn, lane);
}

// ---------------------------------------------------------------------------
// Wide kernel: a BM x BN tile (256x256 and relatives) per workgroup of 4 waves, one
// wave per SIMD with up to 512 registers, each owning a (BM/2) x (BN/2) wave tile as
// TM x TN blocks of v_mfma_f32_16x16x128_f8f6f4 (8 passes; one wave alone keeps the
// matrix core busy with it, which the 16-pass 32x32x64 does not). K advances in
// 128-byte steps through LDS stages filled by LDS-DMA, D = DEPTH steps ahead. A wave
// holds all TM + TN operand fragments of a step in registers (A_i: rows 16i..16i+15
// of its half of the A panel, B_j likewise), so every panel byte is read from LDS
// once per wave: 32 KiB per wave and step for 64 MFMAs with the 128x128 wave tile.
//
// The A panel has D+1 LDS stages and the B panel D. Step kt:
//   rows 0..H-1, i-major:  MFMA(i, 0..TN-1); meanwhile read the remaining A
//                          fragments of step kt, and issue the A-panel DMA of step
//                          kt+D (into the stage that step kt-1 read)
//   wait (own LDS reads; own DMA of step kt+1, not the younger ones),
//   workgroup barrier: the B stage of step kt is now free, step kt+1 is in LDS
//   rows H..TM-1, j-major: MFMA(H..TM-1, j), then B_j is dead: read B_j of step
//                          kt+1; A_0 of step kt+1 likewise; the B-panel DMA of step
//                          kt+D is issued in between
// One barrier per step, in the middle of the MFMA stream. Which read or DMA
// instruction goes in front of which MFMA is fixed at compile time (CfgWide::slot1
// and relatives): a CU's vector memory path moves 64 B per clock (16 clocks per
// DMA instruction), a step needs (BM + BN) * 128 B through it against TM * TN * 32
// clocks of MFMA per wave, and a wave that is held at a DMA instruction or a pair
// of LDS reads for longer than the MFMA in flight lasts leaves the matrix core idle.
//
// Panel rows are 128 B = 8 chunks of 16 B. An operand read takes row (lane & 15),
// chunks 2*(lane >> 4) + {0, 1}; the LDS serves 16 lanes per pass (lane bit 5 and
// the parity of lane bits 2..4 select the pass), and chunk c of row r stored at
// c ^ swz(r) with swz = (bit 1 of r) | 6 * (bit 3 of r) makes every pass hit 16
// distinct 16-byte bank groups. The B fragments take their 16 rows in a permuted
// order, fragment j = 4t + q, operand row p:
//     n = 64 t + 32 (q >> 1) + 8 (p >> 2) + 4 (q & 1) + (p & 3)
// so that a lane ends with 8 consecutive output columns per pair of fragments (16
// bytes of a 16-bit output; 4 lanes cover 64 contiguous bytes of a row); for those
// rows lane bit 3 is row bit 4, hence swz_b. Before they are stored the packed words
// change lanes once more (ds_bpermute_b32) so that adjacent lanes hold adjacent
// bytes: the memory pipeline only merges those into one request (see the epilogue).
template <int BM_, int BN_, int GROUP_M_, int DEPTH_ = 2, bool FULL_LINE_ = true>
struct CfgWide {
  static constexpr int BM = BM_, BN = BN_, GROUP_M = GROUP_M_;
  // K steps the DMA stream runs ahead of the MFMAs. 2 for the large tiles (their
  // stages fill the LDS); small tiles have short steps and need more of them in
  // flight to cover the memory latency.
  static constexpr int DEPTH = DEPTH_;
  static constexpr int WAVES = 4, THREADS = 256;
  static constexpr int WM = BM / 2, WN = BN / 2;      // wave tile (2 x 2 waves)
  static constexpr int TM = WM / 16, TN = WN / 16;    // 16x16 MFMA blocks per wave
  static constexpr int H = TM / 2;                    // rows of the first (i-major) half
  static constexpr int BKW = 128;
  static constexpr int A_BYTES = BM * BKW, B_BYTES = BN * BKW;
  // A panel: DEPTH + 1 LDS stages (its DMA goes out in the first half of a step,
  // into the stage read one step earlier); B panel: DEPTH stages (DMA in the
  // second half, into the stage just read)
  static constexpr int A_STAGES = DEPTH + 1, B_STAGES = DEPTH;
  static constexpr int B_BASE = A_STAGES * A_BYTES;
  static constexpr int PANEL_BYTES = A_STAGES * A_BYTES + B_STAGES * B_BYTES;
  // Epilogue operands of a tile (b_scale and bias of its BN columns, a_scale of its BM
  // rows) are staged after the panels when 4 KiB are left: LDS-DMA instructions of
  // 1 KiB each, b_scale | a_scale (two) | bias.
  static constexpr bool STAGE_EPI = PANEL_BYTES + 4096 <= 160 * 1024 && BN * 4 <= 1024 && BM * 4 <= 2048;
  static constexpr int EPI_BS = PANEL_BYTES, EPI_AS = PANEL_BYTES + 1024, EPI_BI = PANEL_BYTES + 3072;
  static constexpr int LDS_BYTES = PANEL_BYTES + (STAGE_EPI ? 4096 : 0);
  // DMA instructions (1 KiB = 8 panel rows) per wave and step
  static constexpr int NDA = BM / 8 / WAVES, NDB = BN / 8 / WAVES, ND = NDA + NDB;
  static_assert(WM % 16 == 0 && WN % 32 == 0, "wave tile: 16-row A fragments, B fragments in pairs");
  static_assert(BM % 32 == 0 && BN % 32 == 0, "panels are dealt 8 rows x 4 waves at a time");
  static_assert(TM * TN <= 64, "accumulators: at most 256 registers");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
  static_assert(DEPTH >= 2 && (DEPTH - 2) * ND + NDA < 63, "DMA instructions in flight: vmcnt has 6 bits");

  // Which columns of the tile a wave owns. A pair of B fragments gives a lane 8 consecutive
  // output columns and the four lanes of a row 32 columns = 64 bytes of a 16-bit output: half
  // a 128-byte memory line. FULL_LINE: two neighbouring pairs are stored together, 8 lanes on
  // the 128 contiguous bytes of a row, so that every store instruction writes whole lines
  // (with 16 rows x 64 bytes per instruction a line leaves the L2 in two halves under the
  // write-once hint). A wave tile is then LP line-wide column blocks of 64 plus, where WN is
  // an odd multiple of 32, one half-line block; the line-wide blocks of wave column wn start
  // at 64 LP wn, the half-line blocks follow behind all of them at 128 LP + 32 wn, so that
  // every line-wide block starts on a line boundary of the tile (WN = 96: wave column 0 owns
  // columns 0..63 and 128..159, wave column 1 owns 64..127 and 160..191).
  static constexpr bool FULL_LINE = FULL_LINE_;
  static constexpr int NPAIR = TN / 2;               // fragment pairs per row of blocks
  static constexpr int LP = FULL_LINE ? WN / 64 : 0;  // pairs of pairs stored as whole lines
  static constexpr int NHALF = NPAIR - 2 * LP;        // pairs stored as half lines
  static constexpr bool SPLIT_COLS = FULL_LINE && WN % 64 != 0;
  // first column (inside the tile) of fragment pair u in wave column wn
  __host__ __device__ static constexpr int colbase(int u, int wn) {
    if (!SPLIT_COLS) return wn * WN + 32 * u;
    return u < 2 * LP ? wn * 64 * LP + 32 * u : 128 * LP + 32 * wn + 32 * (u - 2 * LP);
  }

  // Issue schedule of a K step: which LDS reads and DMA instructions go in front of
  // which MFMA. An LDS read pair or a DMA instruction holds the wave's instruction
  // issue for a dozen clocks or more, an MFMA gives it 32: one such item between two
  // MFMAs is free, a cluster of them leaves the matrix core idle.
  // First half: S1 MFMAs (slot s = i*TN + j). Items: the TM-1 fragment reads A_1 ..
  // A_{TM-1} of this step (in that order) and the NDA DMA instructions of the A panel,
  // merged evenly, a read first, and spread evenly over the slots.
  static constexpr int S1 = H * TN, NR1 = TM - 1, T1 = NR1 + NDA;
  static constexpr int item_of_read1(int q) { return q * T1 / NR1; }  // a read leads
  static constexpr bool is_read1(int t) {
    for (int q = 0; q < NR1; ++q)
      if (item_of_read1(q) == t) return true;
    return false;
  }
  static constexpr int read1_index(int t) {  // reads before item t
    int n = 0;
    for (int q = 0; q < NR1; ++q) n += item_of_read1(q) < t;
    return n;
  }
  static constexpr int dma1_index(int t) { return t - read1_index(t); }  // DMAs before item t
  static constexpr int slot1(int t) { return t * S1 / T1; }
  // A_{i} (i < H) is used from slot i*TN on: its read must be a few MFMAs earlier
  static constexpr bool first_half_reads_in_time() {
    for (int t = 0; t < T1; ++t)
      if (is_read1(t) && read1_index(t) + 1 < H && slot1(t) + 3 > (read1_index(t) + 1) * TN)
        return false;
    return true;
  }
  static_assert(first_half_reads_in_time(), "A fragment read too late for its first use");
  // Second half: S2 MFMAs, column-major (slot s = j*R + i-H). B_j of the next step is
  // read one MFMA after the last use of B_j (slot (j+1)*R + 1, at most S2 = after the
  // last MFMA), A_0 of the next step in front of slot 1, the NDB DMA instructions of
  // the B panel in the middle of their share of the slots.
  static constexpr int R = TM - H, S2 = R * TN;
  static constexpr int slot_b(int j) { return (j + 1) * R + 1 < S2 ? (j + 1) * R + 1 : S2; }
  static constexpr int slot_a0 = S2 > 1 ? 1 : 0;
  static constexpr int slot_dma2(int p) { return (2 * p + 1) * S2 / (2 * NDB); }
};

__device__ __forceinline__ int swz_a(int row) { return ((row >> 1) & 1) | (((row >> 3) & 1) * 6); }
__device__ __forceinline__ int swz_b(int row) { return ((row >> 1) & 1) | (((row >> 4) & 1) * 6); }

// acc += B-fragment x A-fragment. Inline assembly with the accumulator tied to an
// AGPR tuple: with the builtin the register allocator now and then gives source and
// destination accumulators different registers and copies them through VGPRs
// inside the loop (all 256 AGPRs hold accumulators, there is no room to shuffle).
// The compiler does not know this is an MFMA, so the code that reads the
// accumulators afterwards (the epilogue) waits for the matrix core itself.
// FIRST: the first K step of a tile, acc = product (C operand 0). The accumulators
// are never initialised by other instructions: a VALU write of an AGPR right before
// an MFMA that reads it needs wait states which the compiler cannot insert here.
template <bool FIRST>
__device__ __forceinline__ void mfma_16x16x128_fp8(v4f& acc, const v8i& b, const v8i& a) {
  if constexpr (FIRST) {
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, 0" : "=a"(acc) : "v"(b), "v"(a));
  } else {
    asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc) : "v"(b), "v"(a));
  }
}

// A batch of GEMMs as one launch (GemmGroup, declared with the launchers): sibling Linears
// that read one activation -- to_q / to_k / to_v, and proj_mlp next to them in FLUX single
// blocks (reference dataflow: src/cache_dit/caching/patch_functors/functor_flux.py:60-67) --
// are members of that activation and are walked as if their weights were stacked along N;
// independent Linears of the same stage on other activations (the text stream next to the
// image stream of a double block) follow in the same tile stream. Every member has its own
// weight, scale, bias, output and epilogue flag; K, lda and ldb are common.
struct NoGroup {};

// OUT: dtype of the output and of the bias (CDIT_DT_*), a template parameter so that
// the bf16 instances carry no trace of the others. GROUPED: the launch walks the tiles
// of a GemmGroup (the B-side fields of `g` are then unused); the instances without it
// are unchanged by its existence.
// STAMPS (a measurement instance, never launched by the operator entry points): every
// workgroup leaves four 64-bit words at stamps + 4 * blockIdx.x -- the constant-rate wall
// clock (100 MHz) at its start and after its last store has been issued and its DMA has
// drained, the id of the XCD it ran on and the number of tiles it took -- so that the spread
// of the finish times over the XCDs can be read off a real launch.
struct StampArgs {
  unsigned long long* stamps;
};
template <class C, int OUT = CDIT_DT_BF16, bool GROUPED = false, bool STAMPS = false>
__global__ __launch_bounds__(C::THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) void
gemm_fp8_wide(GemmArgs g, int tiles_m, int tiles_n,
              std::conditional_t<GROUPED, GemmGroup, std::conditional_t<STAMPS, StampArgs, NoGroup>> grp) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x;
  unsigned long long stamp_start = 0;
  int stamp_tiles = 0;
  if constexpr (STAMPS) stamp_start = wall_clock64();
  const int lane = tid & 63;
  // wave-uniform on purpose: LDS-DMA destinations (M0) then come from scalar code
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int BKW = C::BKW, TM = C::TM, TN = C::TN, H = C::H;
  constexpr int D = C::DEPTH;
  // output stores per wave and tile (16 bytes per lane each); every wave issues all of them
  constexpr int NST = TM * (TN / 2) * (OUT == CDIT_DT_F32 ? 2 : 1);
  static_assert((D - 2) * C::ND + C::NDA + NST <= 63, "vmcnt is a 6-bit counter");
  const int KT = g.K / BKW;  // >= D (checked by the launcher)
  int ntiles = tiles_m * tiles_n;
  if constexpr (GROUPED) ntiles = grp.tile_begin[grp.acts];

  // The workgroup is persistent: it takes tiles blockIdx.x, blockIdx.x + gridDim.x,
  // ... and runs their K loops as one stream: the DMA of the last D steps of a
  // tile already fetches the first D steps of the next one, and the fragments read at
  // the end of the last step are the next tile's first. The epilogue of a tile
  // then runs with the next tile's panels landing in LDS, and its stores drain
  // while the next K loop is under way.
  // Where a tile lives: for a batch, activation and member are looked up from the linear
  // tile id (the table sits in the kernel arguments: scalar loads with uniform indices).
  struct Where {
    int act, member, m0, n0;
  };
  auto locate = [&](int t) -> Where {
    Where w;
    if constexpr (GROUPED) {
      constexpr int kXcd = 8;
      int id = t;  // ids that run on one XCD are made consecutive, as tile_of_block does
      if (ntiles % kXcd == 0) id = (t % kXcd) * (ntiles / kXcd) + t / kXcd;
      int s = 0;
#pragma unroll
      for (int i = 1; i < kMaxActs; ++i)
        if (i < grp.acts && id >= grp.tile_begin[i]) s = i;
      int tm, tn;
      tile_of_linear<C::GROUP_M>(id - grp.tile_begin[s], grp.tiles_m[s], grp.tiles_n[s], &tm, &tn);
      int p = grp.first_member[s];
      const int p_end = grp.first_member[s + 1];
#pragma unroll
      for (int i = 1; i < kMaxGroup; ++i)
        if (i > p && i < p_end && tn >= grp.col_begin[i]) p = i;
      w.act = s;
      w.member = p;
      w.m0 = tm * C::BM;
      w.n0 = (tn - grp.col_begin[p]) * C::BN;
    } else {
      int tm, tn;
      tile_of_block<C::GROUP_M>(t, ntiles, tiles_m, tiles_n, &tm, &tn);
      w.act = 0;
      w.member = 0;
      w.m0 = tm * C::BM;
      w.n0 = tn * C::BN;
    }
    return w;
  };
  auto a_of = [&](int s) -> const uint8_t* {
    if constexpr (GROUPED) return static_cast<const uint8_t*>(grp.a[s]);
    return static_cast<const uint8_t*>(g.a);
  };
  auto a_scale_of = [&](int s) -> const float* {
    if constexpr (GROUPED) return grp.a_scale[s];
    return g.a_scale;
  };
  auto m_of = [&](int s) -> int {
    if constexpr (GROUPED) return grp.M[s];
    return g.M;
  };
  auto b_of = [&](int p) -> const uint8_t* {
    if constexpr (GROUPED) return grp.b[p];
    return g.b;
  };
  auto n_of = [&](int p) -> int {
    if constexpr (GROUPED) return grp.N[p];
    return g.N;
  };
  auto grp_b_scale = [&](int p) -> const float* {
    if constexpr (GROUPED) return grp.b_scale[p];
    return g.b_scale;
  };
  auto grp_bias = [&](int p) -> const uint16_t* {
    if constexpr (GROUPED) return grp.bias[p];
    return g.bias;
  };
  int m0, n0;          // tile being computed
  int cur = 0;         // member it belongs to
  int cur_act = 0;     // and its activation
  {
    const Where w = locate(blockIdx.x);
    cur = w.member;
    cur_act = w.act;
    m0 = w.m0;
    n0 = w.n0;
  }

  // DMA source: tile whose panels the DMA stream currently fetches. Instruction p
  // of this wave fills 8 panel rows (1 KiB): rows 8 (wave + 4p) of the A panel for
  // p < NDA, of the B panel after that. Lane l lands on row l/8, position l%8 and
  // fetches the logical chunk that the swizzle stores there.
  const uint8_t* A;
  const uint8_t* B;
  uint32_t off[C::ND];
  int nrec = 0x7fffffff;  // 0: the stream has run past the last tile, fetch nothing
  // The lane offsets only depend on the tile through the clamps at the last rows of A
  // and B: between two tiles without partial panels they are not recomputed (some 130
  // VALU instructions in the middle of the MFMA stream otherwise).
  bool off_clamped = true;  // the first call computes them
  auto set_source = [&](int sm0, int sn0, int member, int act) {
    A = a_of(act) + (int64_t)sm0 * g.lda;
    B = b_of(member) + (int64_t)sn0 * g.ldb;
    const int rows_a = m_of(act) - sm0, rows_b = n_of(member) - sn0;
    const bool clamped = rows_a < C::BM || rows_b < C::BN;
    if (!clamped && !off_clamped) return;
    off_clamped = clamped;
    // recomputed from the lane id at every call: opaque to the optimizer, which
    // would otherwise keep all the row indices in registers across the K loop
    int lrow = lane >> 3;
    asm volatile("" : "+v"(lrow));
#pragma unroll
    for (int p = 0; p < C::ND; ++p) {
      const bool is_a = p < C::NDA;
      const int row = (wave + 4 * (is_a ? p : p - C::NDA)) * 8 + lrow;
      const int c = (lane & 7) ^ (is_a ? swz_a(row) : swz_b(row));
      off[p] = is_a ? (uint32_t)min(row, rows_a - 1) * (uint32_t)g.lda + c * 16
                    : (uint32_t)min(row, rows_b - 1) * (uint32_t)g.ldb + c * 16;
    }
  };
  set_source(m0, n0, cur, cur_act);
  // buffer_load ... lds (MUBUF form: the compiler tracks it with vmcnt only, while
  // the global_load form makes it wait for all LDS reads at every use). With a
  // descriptor of zero records every lane is out of range: nothing is fetched and
  // zeros land in the (free) stage, so the loop body has no special cases.
  auto dma_a = [&](int kt, int a_lds, int p) {
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(A), 0, nrec, 0x00020000);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        rsrc, (__attribute__((address_space(3))) void*)(smem + a_lds + (wave + 4 * p) * 1024), 16,
        (int)off[p], kt * BKW, 0, 0);
  };
  auto dma_b = [&](int kt, int b_lds, int p) {
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(B), 0, nrec, 0x00020000);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        rsrc, (__attribute__((address_space(3))) void*)(smem + b_lds + (wave + 4 * p) * 1024), 16,
        (int)off[C::NDA + p], kt * BKW, 0, 0);
  };

  // operand read map
  const int r16 = lane & 15, kg = lane >> 4;
  const int brow = 8 * (r16 >> 2) + (r16 & 3);
  // B fragments: pair u of this wave reads panel rows colbase(u, wn) + brow (+ 4 for the
  // second fragment of the pair). The pairs stored as whole lines are contiguous from
  // colbase(0, wn) on; the half-line pair (SPLIT_COLS) has a base of its own, rd_bh. All
  // bases are multiples of 32, which leaves swz_b (row bits 1 and 4) to brow alone.
  uint32_t rd_a[2], rd_b[2], rd_bh[2];
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    rd_a[e] = (wm * C::WM + r16) * BKW + (((2 * kg + e) ^ swz_a(wm * C::WM + r16)) << 4);
    const uint32_t chunk = ((2 * kg + e) ^ swz_b(brow)) << 4;
    rd_b[e] = (C::colbase(0, wn) + brow) * BKW + chunk;
    rd_bh[e] = (C::colbase(C::NPAIR - 1, wn) + brow) * BKW + chunk;
  }
  // __restrict__: loads through a restrict-qualified pointer carry alias scope
  // information. Without it the compiler assumes that an LDS read may alias any
  // LDS-DMA write in flight and puts s_waitcnt vmcnt(0) in front of the read, which
  // drains the DMA stream at every step. The stages read in a step are never the
  // ones its DMA fills; the explicit waits before the barriers order the two.
  auto read_a = [&](const uint8_t* __restrict__ st, int i) -> v8i {
    const v4i lo = *reinterpret_cast<const v4i*>(st + rd_a[0] + i * 16 * BKW);
    const v4i hi = *reinterpret_cast<const v4i*>(st + rd_a[1] + i * 16 * BKW);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto read_b = [&](const uint8_t* __restrict__ st, int j) -> v8i {
    const bool half = C::SPLIT_COLS && (j >> 1) >= 2 * C::LP;
    const int ro = (half ? 0 : 32 * (j >> 1)) + 4 * (j & 1);
    const v4i lo = *reinterpret_cast<const v4i*>(st + (half ? rd_bh[0] : rd_b[0]) + ro * BKW);
    const v4i hi = *reinterpret_cast<const v4i*>(st + (half ? rd_bh[1] : rd_b[1]) + ro * BKW);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  v4f acc[TM][TN];
  v8i af[TM], bf[TN];

  // LDS offsets of the stages of steps kt-1 / kt / kt+1 (A) and kt / kt+1 (B);
  // step s lives in A stage s mod (D+1) and B stage s mod D
  int a_prev = D * C::A_BYTES, a_cur = 0, a_next = C::A_BYTES;
  int b_cur = C::B_BASE, b_next = C::B_BASE + C::B_BYTES;
  // prologue: steps 0 .. D-1 in flight, step 0 landed
#pragma unroll
  for (int s = 0; s < D; ++s) {
#pragma unroll
    for (int p = 0; p < C::NDA; ++p) dma_a(s, s * C::A_BYTES, p);
#pragma unroll
    for (int p = 0; p < C::NDB; ++p) dma_b(s, C::B_BASE + s * C::B_BYTES, p);
  }
  wait_and_barrier<(D - 1) * C::ND>();

  for (int tile = blockIdx.x;; tile += gridDim.x) {
    const int next_tile = tile + gridDim.x;
    int nm0 = 0, nn0 = 0, next_member = 0, next_act = 0;
    // fragments of step 0 (in LDS since the prologue, or since the barrier of the
    // previous tile's last step). The last step of a tile reads them too, like
    // every step does for its successor, but keeping them across the epilogue
    // would cost 72 registers there.
#pragma unroll
    for (int j = 0; j < TN; ++j) bf[j] = read_b(smem + b_cur, j);
    af[0] = read_a(smem + a_cur, 0);
    // epilogue operands of this tile, fetched two steps before they are needed:
    // acc[i][4t+q][e] is out[m][n] with
    //   m = m0 + wm*WM + 16i + (lane&15),
    //   n = n0 + colbase(2t + (q>>1), wn) + 8(lane>>4) + 4(q&1) + e
    const int mw = m0 + wm * C::WM + r16;
    v4f bs[TN];
    uint2 bi[TN];  // bias stays packed (bf16 pairs) until used: registers are scarce
    float as[TM];

    // One K step; FIRST: step 0 of the tile (the accumulators start from zero).
    // EVENTS: the step may be one of the last max(D, 2) of the tile, where the DMA stream
    // moves on to the next tile and the epilogue operands are fetched. The steps before
    // them run in a loop of their own without these tests: what stands between the last
    // MFMA of a step and the first of the next (tests, taken branches, stage arithmetic)
    // is time the matrix core waits.
    auto step = [&](int kt, auto first_tag, auto events_tag) {
      constexpr bool FIRST = decltype(first_tag)::value;
      constexpr bool EVENTS = decltype(events_tag)::value;
      if (EVENTS && kt == KT - D) {
        // every DMA of this tile has been issued: the stream moves on
        if (next_tile < ntiles) {
          const Where w = locate(next_tile);
          next_member = w.member;
          next_act = w.act;
          nm0 = w.m0;
          nn0 = w.n0;
          set_source(nm0, nn0, next_member, next_act);
        } else {
          nrec = 0;
        }
      }
      if (EVENTS && kt == KT - 2) {
        // buffer accesses: what lies beyond N (M) reads as zero, no bounds branches; a
        // null bias becomes an empty buffer
        const float* const cur_b_scale = GROUPED ? grp_b_scale(cur) : g.b_scale;
        const uint16_t* const cur_bias = GROUPED ? grp_bias(cur) : g.bias;
        const int cur_n = n_of(cur);
        const __amdgpu_buffer_rsrc_t bs_buf = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(cur_b_scale), 0, cur_n * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t bi_buf = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t*>(cur_bias), 0, cur_bias ? cur_n * 2 : 0, 0x00020000);
        const __amdgpu_buffer_rsrc_t as_buf = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(a_scale_of(cur_act)), 0, m_of(cur_act) * 4, 0x00020000);
        if constexpr (C::STAGE_EPI) {
          // Four LDS-DMA instructions (every wave issues all four: the same bytes land
          // four times, and the waves' instruction counts stay equal) instead of TM +
          // 2 TN loads per lane, whose issue alone held the MFMAs up for 700 cycles.
          // They are older than this step's panel DMA, so the waits of the next two
          // steps cover them.
          auto stage = [&](__amdgpu_buffer_rsrc_t buf, int byte0, int lds) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                buf, (__attribute__((address_space(3))) void*)(smem + lds), 16, byte0 + 16 * lane, 0,
                0, 0);
          };
          stage(bs_buf, n0 * 4, C::EPI_BS);
          stage(as_buf, m0 * 4, C::EPI_AS);
          stage(as_buf, m0 * 4 + 1024, C::EPI_AS + 1024);
          stage(bi_buf, n0 * 2, C::EPI_BI);
        } else {
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            const int n = n0 + C::colbase(j >> 1, wn) + 8 * kg + 4 * (j & 1);
            bs[j] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(bs_buf, n * 4, 0, 0));
            bi[j] = __builtin_bit_cast(uint2, __builtin_amdgcn_raw_buffer_load_b64(bi_buf, n * 2, 0, 0));
          }
#pragma unroll
          for (int i = 0; i < TM; ++i)
            as[i] = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(as_buf, (mw + 16 * i) * 4, 0, 0));
        }
      }
      // step (of its tile) to fetch
      const int kd = !EVENTS || kt + D < KT ? kt + D : kt + D - KT;
      const uint8_t* st = smem + a_cur;
      // first half: rows 0..H-1, row-major; meanwhile the other A fragments of this
      // step are read and the A panel D steps ahead goes into the stage that step
      // kt-1 read (schedule: CfgWide::slot1)
#pragma unroll
      for (int sl = 0; sl < C::S1; ++sl) {
#pragma unroll
        for (int t = 0; t < C::T1; ++t) {
          if (C::slot1(t) != sl) continue;
          if (C::is_read1(t)) {
            af[C::read1_index(t) + 1] = read_a(st, C::read1_index(t) + 1);
          } else {
            dma_a(kd, a_prev, C::dma1_index(t));
          }
        }
        mfma_16x16x128_fp8<FIRST>(acc[sl / TN][sl % TN], bf[sl % TN], af[sl / TN]);
        __builtin_amdgcn_sched_barrier(0);
      }
      // own LDS reads of this step done, own DMA of the next step landed (the
      // steps after it and the A panel issued above may still fly); then
      // everyone's. In the first D-1 steps of a later tile the NST output stores of
      // the previous epilogue were issued after the DMA in question (the counter
      // retires in issue order) and may keep flying as well.
      if ((FIRST || D > 2) && kt <= D - 2 && tile != (int)blockIdx.x) {
        wait_and_barrier<(D - 2) * C::ND + C::NDA + NST>();
      } else {
        wait_and_barrier<(D - 2) * C::ND + C::NDA>();
      }
      // second half: rows H..TM-1, column-major; B_j of the next step replaces B_j
      // after its last use, the B panel D steps ahead goes into the B stage of this
      // step (after the very last step the reads fetch zeros that are never used)
      auto second_half_items = [&](int sl) {
        if (sl == C::slot_a0) af[0] = read_a(smem + a_next, 0);
#pragma unroll
        for (int j = 0; j < TN; ++j)
          if (C::slot_b(j) == sl) bf[j] = read_b(smem + b_next, j);
#pragma unroll
        for (int p = 0; p < C::NDB; ++p)
          if (C::slot_dma2(p) == sl) dma_b(kd, b_cur, p);
      };
      int a_after = 0, b_after = 0;  // stages of the step after the next
#pragma unroll
      for (int sl = 0; sl < C::S2; ++sl) {
        second_half_items(sl);
        if (sl == C::S2 - 1) {
          // worked out in front of the last MFMA, not behind it
          a_after = a_next + C::A_BYTES == C::A_STAGES * C::A_BYTES ? 0 : a_next + C::A_BYTES;
          b_after = b_next + C::B_BYTES == C::B_BASE + C::B_STAGES * C::B_BYTES
                        ? C::B_BASE
                        : b_next + C::B_BYTES;
        }
        mfma_16x16x128_fp8<FIRST>(acc[H + sl % C::R][sl / C::R], bf[sl / C::R], af[H + sl % C::R]);
        __builtin_amdgcn_sched_barrier(0);
      }
      second_half_items(C::S2);
      __builtin_amdgcn_sched_barrier(0);
      // rotate the stages
      a_prev = a_cur;
      a_cur = a_next;
      a_next = a_after;
      b_cur = b_next;
      b_next = b_after;
    };
    step(0, std::true_type{}, std::true_type{});
    {
      const int events_from = KT - (D > 2 ? D : 2);  // first step that may have an event
      int kt = 1;
      for (; kt < events_from; ++kt) step(kt, std::false_type{}, std::false_type{});
      for (; kt < KT; ++kt) step(kt, std::false_type{}, std::true_type{});
    }
    // the last MFMAs (8 passes each) must have written their accumulators
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    // ---- epilogue
    // Nothing is drained here: the next tile's step 0 landed before the barrier of
    // the last step, its later steps keep flying under the epilogue.
    // The accumulators are read with inline assembly, one row of blocks at a time:
    // left to itself the compiler copies all of them to VGPRs first, parks everything
    // else that is live (DMA offsets, scales) in spare AGPRs and scratch, and a scratch
    // reload waits for every output store in flight (vmcnt). The GELU decision is
    // taken once per tile, not once per element.
    // Stores are buffer stores that every wave always issues, NST per tile, so that
    // the waits of the next K loop can count them: the descriptor of a row of blocks
    // covers the rows of it that exist (the hardware drops lanes beyond), lanes whose
    // columns do not exist get an offset beyond any descriptor. Per lane a 32-bit
    // byte offset (the launcher bounds 512 * ldo), per row of blocks a scalar base.
    if constexpr (C::STAGE_EPI) {
      // Staged at the start of step KT-2. The wait of the last step lets (D-2) ND + NDA
      // instructions fly, and ND + NDA were issued behind the staging by then: up to
      // D = 3 that wait covers it, a deeper stream needs one of its own here (the two
      // steps' 2 ND panel instructions are younger and may keep flying). Without it the
      // first of these reads could run ahead of its DMA when that was slow (a cold TLB,
      // the first launch of a process) and pick up what an earlier tile or kernel left.
      // (The compiler puts a wait for all DMA in front of the later reads: it cannot tell
      // them from the panels in flight. Measured: no cost, the next tile's first steps
      // are in the LDS by then.)
      if constexpr (D > 3) wait_vm<2 * C::ND>();
      auto read_staged = [&](const uint8_t* __restrict__ ep) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int c = C::colbase(j >> 1, wn) + 8 * kg + 4 * (j & 1);
          bs[j] = *reinterpret_cast<const v4f*>(ep + C::EPI_BS + c * 4);
          bi[j] = *reinterpret_cast<const uint2*>(ep + C::EPI_BI + c * 2);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
          as[i] = *reinterpret_cast<const float*>(ep + C::EPI_AS + (wm * C::WM + r16 + 16 * i) * 4);
      };
      read_staged(smem);
    }
    constexpr int OB = OUT == CDIT_DT_F32 ? 4 : 2;  // bytes per output element
    constexpr uint32_t kNoColumn = 0x80000000u;
    constexpr int kStoreOnce = 2;  // cache policy of the output stores: non-temporal (written once)
    // Where a wave tile has whole-line pairs and a half-line pair (96 columns), the half lines
    // are stored with the plain policy unless the epilogue is the long one (GELU): the other
    // half of such a line comes from the other wave of the row, and a non-temporal half can
    // leave the L2 before it arrives. Measured at 4608 x 3072 x 12288, alternating builds:
    // 2 % faster than all stores non-temporal (which in turn beats all stores plain) without
    // GELU, 2-3 % slower with it, where the two waves' stores lie further apart in time.
    uint16_t* cur_out = g.out;
    int64_t cur_ldo = g.ldo;
    int cur_epilogue = g.epilogue;
    if constexpr (GROUPED) {
      cur_out = grp.out[cur];
      cur_ldo = grp.ldo[cur];
      cur_epilogue = grp.epilogue[cur];
    }
    const int cur_N = n_of(cur);
    uint8_t* const out_wave =
        reinterpret_cast<uint8_t*>(cur_out) + ((int64_t)(m0 + wm * C::WM) * cur_ldo + n0) * OB;
    const int rows_wave = m_of(cur_act) - (m0 + wm * C::WM);  // rows of the wave tile that exist
    // The memory pipeline merges the lanes of a store into one request only when
    // adjacent lanes write adjacent bytes: with lane = 16 kg + r16 holding row r16,
    // 16-byte piece kg, every lane is a request of its own (measured: 294 clocks per
    // store instruction with four waves storing, against 77 when lanes 4r .. 4r+3 hold
    // the 64 contiguous bytes of row r). 16-bit outputs are therefore moved with
    // ds_bpermute_b32 (the LDS crossbar, no LDS memory) before they are stored.
    // Half-line pairs: lane L takes the packed words of lane 16 (L & 3) + (L >> 2) and
    // holds piece L & 3 of row L >> 2 (16 rows x 64 bytes per store instruction).
    // Whole lines (pairs 2v and 2v+1 together, 64 columns): first the two halves of a row
    // of 16 lanes trade words (DPP row_ror:8 under a bank mask), P = {rows 0-7: pair 2v |
    // rows 8-15: pair 2v+1 of the row 8 above}, Q = {rows 0-7: pair 2v of the row 8 below |
    // rows 8-15: pair 2v+1}; then lane L = 8 row + piece takes P (store A, block rows 0-7)
    // and Q (store B, block rows 8-15) from lane 16 (piece & 3) + 8 (piece >> 2) + row: 8
    // lanes on the 128 contiguous bytes of a row, 8 rows per store instruction.
    constexpr bool PERMUTE = OUT != CDIT_DT_F32;
    constexpr int LP = PERMUTE ? C::LP : 0, NP = TN / 2, NH = NP - 2 * LP;
    const int st_row = PERMUTE ? lane >> 2 : r16, st_piece = PERMUTE ? lane & 3 : kg;
    const int bp_addr = 4 * (16 * (lane & 3) + (lane >> 2));
    const int bp_line = 4 * (16 * (lane & 3) + 8 * ((lane >> 2) & 1) + (lane >> 3));
    const uint32_t out_lane = ((uint32_t)st_row * (uint32_t)cur_ldo + 8u * st_piece) * OB;
    const uint32_t out_lane_line = ((uint32_t)(lane >> 3) * (uint32_t)cur_ldo + 8u * (lane & 7)) * OB;
    const uint32_t rows8 = 8u * (uint32_t)cur_ldo * OB;  // block rows 8-15 of a whole-line store
    uint32_t out_off[NH > 0 ? NH : 1], out_off_line[LP > 0 ? LP : 1];
#pragma unroll
    for (int h = 0; h < NH; ++h) {
      const int col = C::colbase(2 * LP + h, wn);
      out_off[h] = n0 + col + 8 * st_piece < cur_N ? out_lane + col * OB : kNoColumn;
    }
#pragma unroll
    for (int v = 0; v < LP; ++v) {
      const int col = C::colbase(2 * v, wn);
      out_off_line[v] = n0 + col + 8 * (lane & 7) < cur_N ? out_lane_line + col * OB : kNoColumn;
    }
    auto out_row_of = [&](int i) {
      // (made a scalar explicitly: a descriptor the compiler takes for divergent is
      // applied in a loop over its distinct values)
      const int rows = __builtin_amdgcn_readfirstlane(min(max(rows_wave - 16 * i, 0), 16));
      return __builtin_amdgcn_make_buffer_rsrc(out_wave + (int64_t)(16 * i) * cur_ldo * OB, 0,
                                               rows * cur_ldo * OB, 0x00020000);
    };
    // 16-bit outputs: the permuted words of a row of blocks are stored while the next
    // row is being computed, so the latency of the permutation is not waited for; the
    // last row's after the two copies of the epilogue have joined
    uint32_t moved[NH > 0 ? NH : 1][4], moved_a[LP > 0 ? LP : 1][4], moved_b[LP > 0 ? LP : 1][4];
    auto store_moved = [&](int i, auto half_policy_tag) {
      constexpr int kHalfPolicy = decltype(half_policy_tag)::value;
      const __amdgpu_buffer_rsrc_t row = out_row_of(i);
#pragma unroll
      for (int v = 0; v < LP; ++v) {
        __builtin_amdgcn_raw_buffer_store_b128(
            v4u{moved_a[v][0], moved_a[v][1], moved_a[v][2], moved_a[v][3]}, row,
            (int)out_off_line[v], 0, kStoreOnce);
        __builtin_amdgcn_raw_buffer_store_b128(
            v4u{moved_b[v][0], moved_b[v][1], moved_b[v][2], moved_b[v][3]}, row,
            (int)(out_off_line[v] + rows8), 0, kStoreOnce);
      }
#pragma unroll
      for (int h = 0; h < NH; ++h)
        __builtin_amdgcn_raw_buffer_store_b128(
            v4u{moved[h][0], moved[h][1], moved[h][2], moved[h][3]}, row, (int)out_off[h], 0, kHalfPolicy);
    };
    auto epilogue = [&](auto gelu_tag) {
      constexpr bool GELU = decltype(gelu_tag)::value;
      constexpr std::integral_constant<int, (LP > 0 && !GELU) ? 0 : kStoreOnce> half_policy{};
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const __amdgpu_buffer_rsrc_t out_row = out_row_of(i);
        uint32_t pk[TN / 2][4];
#pragma unroll
        for (int u = 0; u < TN / 2; ++u) {  // pair of fragments 2u, 2u+1: 8 consecutive columns
          float v[8];
#pragma unroll
          for (int d = 0; d < 2; ++d) {
            const int j = 2 * u + d;
            const float b4[4] = {bias_to_f32<OUT>(bi[j].x & 0xffffu), bias_to_f32<OUT>(bi[j].x >> 16),
                                 bias_to_f32<OUT>(bi[j].y & 0xffffu), bias_to_f32<OUT>(bi[j].y >> 16)};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              float a;
              asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(a) : "a"(acc[i][j][e]));
              float t = __fmaf_rn(a * as[i], bs[j][e], b4[e]);
              if constexpr (GELU) t = gelu_tanh(t);
              v[4 * d + e] = t;
            }
          }
          if constexpr (OUT == CDIT_DT_F32) {
            __builtin_amdgcn_raw_buffer_store_b128(
                v4u{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]),
                    __float_as_uint(v[3])},
                out_row, (int)out_off[u], 0, kStoreOnce);
            __builtin_amdgcn_raw_buffer_store_b128(
                v4u{__float_as_uint(v[4]), __float_as_uint(v[5]), __float_as_uint(v[6]),
                    __float_as_uint(v[7])},
                out_row, (int)(out_off[u] + 16u), 0, kStoreOnce);  // (fp32: every pair is a half-line pair)
          } else {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              if constexpr (OUT == CDIT_DT_F16) {
                pk[u][k] = pack_f16x2(v[2 * k], v[2 * k + 1]);
              } else {
                pk[u][k] = pack_bf16x2(v[2 * k], v[2 * k + 1]);
              }
            }
          }
        }
        if constexpr (PERMUTE) {
          // the previous row's words have had this row's arithmetic to arrive
          __builtin_amdgcn_sched_barrier(0);
          if (i > 0) store_moved(i - 1, half_policy);
#pragma unroll
          for (int v = 0; v < LP; ++v)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const int w0 = (int)pk[2 * v][k], w1 = (int)pk[2 * v + 1][k];
              // row_ror:8 = 0x128; bank mask 0xc: lanes 8-15 of a row take the other half's
              // word, lanes 0-7 keep `old`; 0x3 the other way round
              const int p = __builtin_amdgcn_update_dpp(w0, w1, 0x128, 0xf, 0xc, false);
              const int q = __builtin_amdgcn_update_dpp(w1, w0, 0x128, 0xf, 0x3, false);
              moved_a[v][k] = (uint32_t)__builtin_amdgcn_ds_bpermute(bp_line, p);
              moved_b[v][k] = (uint32_t)__builtin_amdgcn_ds_bpermute(bp_line, q);
            }
#pragma unroll
          for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int k = 0; k < 4; ++k)
              moved[h][k] = (uint32_t)__builtin_amdgcn_ds_bpermute(bp_addr, (int)pk[2 * LP + h][k]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    if (cur_epilogue & CDIT_EPI_GELU_TANH) {
      epilogue(std::true_type{});
    } else {
      epilogue(std::false_type{});
    }
    // (one copy of the last row's stores for both epilogues, all non-temporal)
    if constexpr (PERMUTE) store_moved(TM - 1, std::integral_constant<int, kStoreOnce>{});
    if constexpr (STAMPS) ++stamp_tiles;
    if (next_tile >= ntiles) break;
    m0 = nm0;
    n0 = nn0;
    cur = next_member;
    cur_act = next_act;
  }
  // the zero-record DMA of the last D steps must not outlive the workgroup
  wait_vm<0>();
  if constexpr (STAMPS) {
    typedef unsigned int u2v __attribute__((ext_vector_type(2)));
    const unsigned long long stamp_end = wall_clock64();
    // HW_REG_XCC_ID (register 20), bits 3:0
    const unsigned xcc = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11));
    const __amdgpu_buffer_rsrc_t sb = __builtin_amdgcn_make_buffer_rsrc(grp.stamps + 4 * blockIdx.x, 0, 32, 0x00020000);
    // (thread 0 writes; every other thread's offset lies beyond the 32 bytes. 8-byte stores:
    // the 16-byte buffer stores of this kernel are the output's, and are counted)
    const int off = tid == 0 ? 0 : 64;
    __builtin_amdgcn_raw_buffer_store_b64(u2v{(unsigned)stamp_start, (unsigned)(stamp_start >> 32)}, sb, off, 0, 0);
    __builtin_amdgcn_raw_buffer_store_b64(u2v{(unsigned)stamp_end, (unsigned)(stamp_end >> 32)}, sb, off + 8, 0, 0);
    __builtin_amdgcn_raw_buffer_store_b64(u2v{xcc, 0u}, sb, off + 16, 0, 0);
    __builtin_amdgcn_raw_buffer_store_b64(u2v{(unsigned)stamp_tiles, 0u}, sb, off + 24, 0, 0);
  }
}

template <class C, int OUT = CDIT_DT_BF16>
int launch_wide(const GemmArgs& g, hipStream_t stream) {
  static bool lds_allowed[64];
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_fp8_wide<C, OUT>), C::LDS_BYTES,
                                 lds_allowed))
    return rc;
  const int cus = cu_count();
  if (cus <= 0) {
    set_error("cannot query the CU count of the current device");
    return CDIT_EHIP;
  }
  const int tiles_m = (g.M + C::BM - 1) / C::BM, tiles_n = (g.N + C::BN - 1) / C::BN;
  const int ntiles = tiles_m * tiles_n;
  // one persistent workgroup per CU (its LDS and registers fill the CU)
  hipLaunchKernelGGL((gemm_fp8_wide<C, OUT>), dim3(ntiles < cus ? ntiles : cus), dim3(C::THREADS),
                     C::LDS_BYTES, stream, g, tiles_m, tiles_n, NoGroup{});
  return 0;
}

// The measurement instance of the same kernel (StampArgs above).
template <class C>
int launch_wide_stamps(const GemmArgs& g, unsigned long long* stamps, int* workgroups, hipStream_t stream) {
  static bool lds_allowed[64];
  if (int rc = allow_dynamic_lds(
          reinterpret_cast<const void*>(&gemm_fp8_wide<C, CDIT_DT_BF16, false, true>), C::LDS_BYTES,
          lds_allowed))
    return rc;
  const int cus = cu_count();
  if (cus <= 0) {
    set_error("cannot query the CU count of the current device");
    return CDIT_EHIP;
  }
  const int tiles_m = (g.M + C::BM - 1) / C::BM, tiles_n = (g.N + C::BN - 1) / C::BN;
  // (the caller's buffer holds the stamps of 256 workgroups)
  const int ntiles = tiles_m * tiles_n, wgs = std::min(ntiles, std::min(cus, 256));
  if (workgroups) *workgroups = wgs;
  hipLaunchKernelGGL((gemm_fp8_wide<C, CDIT_DT_BF16, false, true>), dim3(wgs), dim3(C::THREADS),
                     C::LDS_BYTES, stream, g, tiles_m, tiles_n, StampArgs{stamps});
  return 0;
}

// The batch as one launch: fills the tile tables of `grp` for this tile shape.
template <class C>
int launch_wide_grouped(const GemmArgs& g, GemmGroup grp, hipStream_t stream) {
  static bool lds_allowed[64];
  if (int rc = allow_dynamic_lds(
          reinterpret_cast<const void*>(&gemm_fp8_wide<C, CDIT_DT_BF16, true>), C::LDS_BYTES,
          lds_allowed))
    return rc;
  const int cus = cu_count();
  if (cus <= 0) {
    set_error("cannot query the CU count of the current device");
    return CDIT_EHIP;
  }
  int ntiles = 0;
  for (int s = 0; s < grp.acts; ++s) {
    int cols = 0;
    for (int p = grp.first_member[s]; p < grp.first_member[s + 1]; ++p) {
      grp.col_begin[p] = cols;
      cols += (grp.N[p] + C::BN - 1) / C::BN;
    }
    grp.tiles_m[s] = (grp.M[s] + C::BM - 1) / C::BM;
    grp.tiles_n[s] = cols;
    grp.tile_begin[s] = ntiles;
    ntiles += grp.tiles_m[s] * cols;
  }
  for (int s = grp.acts; s <= kMaxActs; ++s) grp.tile_begin[s] = ntiles;
  for (int p = grp.count; p <= kMaxGroup; ++p) grp.col_begin[p] = 0x7fffffff;
  hipLaunchKernelGGL((gemm_fp8_wide<C, CDIT_DT_BF16, true>), dim3(ntiles < cus ? ntiles : cus),
                     dim3(C::THREADS), C::LDS_BYTES, stream, g, 0, 0, grp);
  return 0;
}

// ---------------------------------------------------------------------------
// Skinny kernel for M <= 16 (the M = 1 modulation Linears `norm1.linear`,
// `norm.linear` of every block): pure weight streaming. A workgroup of 4 waves
// owns 16 output channels; each wave takes a quarter of K and reads its weight
// rows straight from HBM into MFMA operand registers (lane = row l&15, 32-byte K
// group l>>4; 16 x 128-byte segments per pair of loads), multiplies by the (zero
// padded) activation rows with v_mfma_f32_16x16x128_f8f6f4, and the four partial
// 16x16 tiles are summed through LDS before the epilogue. No LDS staging of the
// weights: every weight byte is used exactly once. The weight loads carry no
// non-temporal hint: with this access pattern (16 rows x 64 bytes per instruction)
// the hinted loads measured 17 % slower in a read-only loop and 10 % in the kernel.
__global__ __launch_bounds__(256) void gemm_fp8_skinny(GemmArgs g) {
  __shared__ float part[4][16][17];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kg = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int nrow = min(n0 + r, g.N - 1);
  const int KT = g.K / 128;           // 128-byte steps in total
  const int per = (KT + 3) / 4;       // steps per wave
  const int k_begin = wave * per, k_end = min(KT, k_begin + per);
  const uint8_t* __restrict__ wp = g.b + (int64_t)nrow * g.ldb + kg * 32;
  const uint8_t* __restrict__ ap =
      static_cast<const uint8_t*>(g.a) + (int64_t)min(r, g.M - 1) * g.lda + kg * 32;
  const bool a_valid = r < g.M;
  v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
  constexpr int U = 6;  // steps in flight
  for (int k0 = k_begin; k0 < k_end; k0 += U) {
    v4i w[U][2], a[U][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kt = min(k0 + u, k_end - 1);  // clamped duplicates are not accumulated
      const v4i* wq = reinterpret_cast<const v4i*>(wp + (int64_t)kt * 128);
      w[u][0] = wq[0];
      w[u][1] = wq[1];
      const v4i* aq = reinterpret_cast<const v4i*>(ap + (int64_t)kt * 128);
      a[u][0] = aq[0];
      a[u][1] = aq[1];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (k0 + u < k_end) {
        v8i wf = __builtin_shufflevector(w[u][0], w[u][1], 0, 1, 2, 3, 4, 5, 6, 7);
        v8i af = __builtin_shufflevector(a[u][0], a[u][1], 0, 1, 2, 3, 4, 5, 6, 7);
        if (!a_valid) af = v8i{0, 0, 0, 0, 0, 0, 0, 0};
        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, acc, 0, 0, 0, 0, 0, 0);
      }
    }
  }
  // acc[e] = partial out[m = lane&15][n0 + 4*(lane>>4) + e]
#pragma unroll
  for (int e = 0; e < 4; ++e) part[wave][r][4 * kg + e] = acc[e];
  __syncthreads();
  if (wave == 0) {
    const int m = r, nl = 4 * kg;
    if (m < g.M && n0 + nl < g.N) {
      const float as = g.a_scale[m];
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float sum = (part[0][m][nl + e] + part[1][m][nl + e]) +
                          (part[2][m][nl + e] + part[3][m][nl + e]);
        const int n = n0 + nl + e;
        float t = sum * as * g.b_scale[n];
        if (g.bias) t += bias_at(g, n);
        if (g.epilogue & CDIT_EPI_GELU_TANH) t = gelu_tanh(t);
        v[e] = t;
      }
      if (g.out_dtype == CDIT_DT_BF16) {
        uint2 pk;
        pk.x = pack_bf16x2(v[0], v[1]);
        pk.y = pack_bf16x2(v[2], v[3]);
        *reinterpret_cast<uint2*>(g.out + (int64_t)m * g.ldo + n0 + nl) = pk;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) store_out(g, (int64_t)m * g.ldo + n0 + nl + e, v[e]);
      }
    }
  }
}

// The skinny kernel with the per-token quantizer inside, for one whole Linear forward at
// M <= 16 (the M = 1 modulation Linears): a separate quantizer launch for a single row
// costs as much as this GEMM's weight stream. Every workgroup quantizes the M activation
// rows itself (a few KiB, an L2 hit for all but the first) into LDS with the quantizer's
// own arithmetic (quant_device.h), so the codes and scales are those of
// cdit_fp8_quant_rowwise bit for bit; workgroup 0 also writes them to the caller's
// workspaces. The first batch of weight loads is issued before that, so the HBM latency
// of the weights covers it. g.a is the bf16 activation here, g.lda its leading dimension.
constexpr int kFusedPad = 16;  // LDS row pitch K + 16 bytes: rows start 4 banks apart
__global__ __launch_bounds__(256) void linear_fp8_skinny_fused(GemmArgs g, uint8_t* q_ws,
                                                               float* scale_ws, int scale_mode) {
  extern __shared__ __attribute__((aligned(16))) uint8_t codes[];  // [M][K + kFusedPad]
  __shared__ float part[4][16][17];
  __shared__ uint32_t wave_amax[4];
  __shared__ float row_s[16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kg = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int nrow = min(n0 + r, g.N - 1);
  const int KT = g.K / 128;
  const int per = (KT + 3) / 4;
  const int k_begin = wave * per, k_end = min(KT, k_begin + per);
  const int pitch = g.K + kFusedPad;
  const uint8_t* __restrict__ wp = g.b + (int64_t)nrow * g.ldb + kg * 32;
  constexpr int U = 6;  // steps in flight
  v4i w[U][2];
  auto load_w = [&](int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kt = min(k0 + u, max(k_end, 1) - 1);  // clamped duplicates are not accumulated
      const v4i* wq = reinterpret_cast<const v4i*>(wp + (int64_t)kt * 128);
      w[u][0] = wq[0];
      w[u][1] = wq[1];
    }
  };
  load_w(k_begin);

  // ---- quantize the activation rows into LDS
  const uint16_t* x = static_cast<const uint16_t*>(g.a);
  const int nchunks = g.K >> 3;  // 16-byte chunks of 8 bf16
  for (int m = 0; m < g.M; ++m) {
    const uint4* xr = reinterpret_cast<const uint4*>(x + (int64_t)m * g.lda);
    uint32_t am = 0;
    for (int c = threadIdx.x; c < nchunks; c += 256) {
      const uint4 v = xr[c];
      am = absmax2(absmax2(absmax2(absmax2(am, v.x), v.y), v.z), v.w);
    }
    am = wave_max_u32(fold2(am));
    if (lane == 0) wave_amax[wave] = am;
    __syncthreads();
    const uint32_t a01 = max(wave_amax[0], wave_amax[1]), a23 = max(wave_amax[2], wave_amax[3]);
    const float s = row_scale(max(a01, a23), scale_mode);
    if (threadIdx.x == 0) row_s[m] = s;
    uint2* dst = reinterpret_cast<uint2*>(codes + m * pitch);
    if (scale_in_fast_window(s)) {  // uniform
      const Recip rcp = make_recip(s);
      for (int c = threadIdx.x; c < nchunks; c += 256) {
        const uint4 v = xr[c];
        dst[c] = uint2{quant4<true>(v.x, v.y, s, rcp), quant4<true>(v.z, v.w, s, rcp)};
      }
    } else {
      for (int c = threadIdx.x; c < nchunks; c += 256) {
        const uint4 v = xr[c];
        dst[c] = uint2{quant4<false>(v.x, v.y, s, Recip{}), quant4<false>(v.z, v.w, s, Recip{})};
      }
    }
    __syncthreads();  // codes of row m complete; wave_amax free for the next row
  }
  if (blockIdx.x == 0) {  // the caller's workspaces get what cdit_fp8_quant_rowwise would write
    for (int m = 0; m < g.M; ++m) {
      const uint2* src = reinterpret_cast<const uint2*>(codes + m * pitch);
      uint2* dst = reinterpret_cast<uint2*>(q_ws + (int64_t)m * g.K);
      for (int c = threadIdx.x; c < nchunks; c += 256) dst[c] = src[c];
    }
    if ((int)threadIdx.x < g.M) scale_ws[threadIdx.x] = row_s[threadIdx.x];
  }

  // ---- the skinny GEMM, activation fragments from LDS
  const bool a_valid = r < g.M;
  const uint8_t* ap = codes + min(r, g.M - 1) * pitch + kg * 32;
  v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int k0 = k_begin; k0 < k_end; k0 += U) {
    if (k0 != k_begin) load_w(k0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (k0 + u < k_end) {
        const v4i* aq = reinterpret_cast<const v4i*>(ap + (k0 + u) * 128);
        v8i af = __builtin_shufflevector(aq[0], aq[1], 0, 1, 2, 3, 4, 5, 6, 7);
        if (!a_valid) af = v8i{0, 0, 0, 0, 0, 0, 0, 0};
        const v8i wf = __builtin_shufflevector(w[u][0], w[u][1], 0, 1, 2, 3, 4, 5, 6, 7);
        acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, acc, 0, 0, 0, 0, 0, 0);
      }
    }
  }
  // acc[e] = partial out[m = lane&15][n0 + 4*(lane>>4) + e]
#pragma unroll
  for (int e = 0; e < 4; ++e) part[wave][r][4 * kg + e] = acc[e];
  __syncthreads();
  if (wave == 0) {
    const int m = r, nl = 4 * kg;
    if (m < g.M && n0 + nl < g.N) {
      const float as = row_s[m];
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float sum = (part[0][m][nl + e] + part[1][m][nl + e]) +
                          (part[2][m][nl + e] + part[3][m][nl + e]);
        const int n = n0 + nl + e;
        float t = sum * as * g.b_scale[n];
        if (g.bias) t += bias_at(g, n);
        if (g.epilogue & CDIT_EPI_GELU_TANH) t = gelu_tanh(t);
        v[e] = t;
      }
      if (g.out_dtype == CDIT_DT_BF16) {
        uint2 pk;
        pk.x = pack_bf16x2(v[0], v[1]);
        pk.y = pack_bf16x2(v[2], v[3]);
        *reinterpret_cast<uint2*>(g.out + (int64_t)m * g.ldo + n0 + nl) = pk;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) store_out(g, (int64_t)m * g.ldo + n0 + nl + e, v[e]);
      }
    }
  }
}

// One activation row (M = 1: the modulation Linears of every block), K <= 4096. The
// 16-row arrangement above makes every lane of a weight load a memory request of its own
// (adjacent lanes read different rows); here a load instruction of the wavefront reads
// 1 KiB of one weight row, lane l bytes 16 l .. 16 l + 15. A dot product does not care in
// which order K is walked, so the MFMA's 16 "rows" are 16 interleaved K subsets of the
// same weight row: with the activation codes fetched at the same positions, lane for lane,
// D[i][i] is the partial dot product over subset i, the diagonal sums to the whole one and
// the other 240 entries are never read (the matrix core has 17 times the rate this
// stream needs). One MFMA takes two such 1 KiB pieces of a row. A wavefront owns R whole
// rows, all of their loads in flight at once, and no partial sums cross wavefronts.
// Measured at K = 3072 with a different weight matrix per launch, against the 16-row
// kernel: 7.4 us instead of 10.1 at N = 9216 and 11.2 instead of 15.1 at N = 18432
// (three rows per wavefront and four wavefronts were the best of 1-4 rows and 2-8
// wavefronts; with this access pattern the non-temporal hint on the weight loads gains
// 6-8 %, where it cost 10 % with the 16-row pattern).
// FUSED: the row is quantized by every workgroup itself, as in linear_fp8_skinny_fused
// (same codes, same scale, workgroup 0 writes them to the caller's workspaces); else
// g.a holds the codes and g.a_scale the scale.
constexpr int kRow1Rows = 3, kRow1Waves = 4;
template <int CHK, bool FUSED>
__global__ __launch_bounds__(64 * kRow1Waves) void linear_fp8_row1(GemmArgs g, uint8_t* q_ws,
                                                                   float* scale_ws, int scale_mode) {
  constexpr int R = kRow1Rows, WAVES = kRow1Waves, THREADS = 64 * WAVES;
  constexpr int PP = (CHK * 128 + THREADS - 1) / THREADS;  // 8-element pieces of x per thread
  __shared__ __attribute__((aligned(16))) uint8_t codes[FUSED ? CHK * 1024 : 16];
  __shared__ uint32_t wave_amax[WAVES];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row0 = (blockIdx.x * WAVES + wave) * R;
  const v4i zero4 = {0, 0, 0, 0};
  v4i w[R][CHK];
#pragma unroll
  for (int q = 0; q < R; ++q) {
    const uint8_t* __restrict__ wp = g.b + (int64_t)min(row0 + q, g.N - 1) * g.ldb + lane * 16;
#pragma unroll
    for (int c = 0; c < CHK; ++c) {
      const v4i* src = reinterpret_cast<const v4i*>(wp + c * 1024);
      if (c * 1024 + lane * 16 < g.K) {
        w[q][c] = __builtin_nontemporal_load(src);
      } else {
        w[q][c] = zero4;
      }
    }
  }
  v4i xa[CHK];
  float as;
  if constexpr (FUSED) {
    // thread t quantizes the 8-element pieces t, t + THREADS, ...; pieces beyond K become
    // zero codes (their weights are zeros too, but 0 x NaN is NaN)
    const uint4* xr = static_cast<const uint4*>(g.a);
    const int nchunks = g.K >> 3, t = threadIdx.x;
    uint4 v[PP];
    uint32_t am = 0u;
#pragma unroll
    for (int p = 0; p < PP; ++p) {
      v[p] = t + p * THREADS < nchunks ? xr[t + p * THREADS] : uint4{0u, 0u, 0u, 0u};
      am = absmax2(absmax2(absmax2(absmax2(am, v[p].x), v[p].y), v[p].z), v[p].w);
    }
    am = wave_max_u32(fold2(am));
    if (lane == 0) wave_amax[wave] = am;
    __syncthreads();
    uint32_t amax = wave_amax[0];
#pragma unroll
    for (int i = 1; i < WAVES; ++i) amax = max(amax, wave_amax[i]);
    as = row_scale(amax, scale_mode);
    const bool fast = scale_in_fast_window(as);  // uniform
    const Recip rcp = make_recip(as);
    uint2* dst = reinterpret_cast<uint2*>(codes);
#pragma unroll
    for (int p = 0; p < PP; ++p) {
      const int c = t + p * THREADS;
      uint2 code;
      if (fast) {
        code = uint2{quant4<true>(v[p].x, v[p].y, as, rcp), quant4<true>(v[p].z, v[p].w, as, rcp)};
      } else {
        code = uint2{quant4<false>(v[p].x, v[p].y, as, Recip{}), quant4<false>(v[p].z, v[p].w, as, Recip{})};
      }
      if (c >= nchunks) code = uint2{0u, 0u};
      if (c < CHK * 128) dst[c] = code;
      if (blockIdx.x == 0 && c < nchunks) reinterpret_cast<uint2*>(q_ws)[c] = code;
    }
    if (blockIdx.x == 0 && t == 0) scale_ws[0] = as;
    __syncthreads();
#pragma unroll
    for (int c = 0; c < CHK; ++c) xa[c] = *reinterpret_cast<const v4i*>(codes + c * 1024 + lane * 16);
  } else {
    const uint8_t* __restrict__ ap = static_cast<const uint8_t*>(g.a) + lane * 16;
#pragma unroll
    for (int c = 0; c < CHK; ++c)
      xa[c] = c * 1024 + lane * 16 < g.K ? *reinterpret_cast<const v4i*>(ap + c * 1024) : zero4;
    as = g.a_scale[0];
  }
  // lane l holds D[4 (l >> 4) + e][l & 15]: the diagonal entry of lanes 0-3, 20-23, 40-43, 60-63
  const int diag = (lane & 15) - 4 * (lane >> 4);
  float mine = 0.0f;  // lane q keeps the dot product of row row0 + q
#pragma unroll
  for (int q = 0; q < R; ++q) {
    v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int c = 0; c < CHK; c += 2) {
      const v4i w1 = c + 1 < CHK ? w[q][c + 1] : zero4, x1 = c + 1 < CHK ? xa[c + 1] : zero4;
      const v8i wf = __builtin_shufflevector(w[q][c], w1, 0, 1, 2, 3, 4, 5, 6, 7);
      const v8i af = __builtin_shufflevector(xa[c], x1, 0, 1, 2, 3, 4, 5, 6, 7);
      acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, acc, 0, 0, 0, 0, 0, 0);
    }
    float d = 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) d = diag == e ? acc[e] : d;
    const float sum = wave_sum_f32(d);
    mine = lane == q ? sum : mine;
  }
  const int n = row0 + lane;
  if (lane < R && n < g.N) {
    float t = mine * as * g.b_scale[n];
    if (g.bias) t += bias_at(g, n);
    if (g.epilogue & CDIT_EPI_GELU_TANH) t = gelu_tanh(t);
    store_out(g, n, t);
  }
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
  if (g.bias) v += bias_at(g, n);
  if (g.epilogue & CDIT_EPI_GELU_TANH) v = gelu_tanh(v);
  store_out(g, (int64_t)m * g.ldo + n, v);
}

template <class C>
int launch_tiled(const GemmArgs& g, hipStream_t stream) {
  static bool lds_allowed[64];
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_fp8_tiled<C>), C::LDS_BYTES,
                                 lds_allowed))
    return rc;
  const int tiles_m = (g.M + C::BM - 1) / C::BM, tiles_n = (g.N + C::BN - 1) / C::BN;
  hipLaunchKernelGGL(gemm_fp8_tiled<C>, dim3(tiles_m * tiles_n), dim3(C::THREADS), C::LDS_BYTES,
                     stream, g, tiles_m, tiles_n);
  return 0;
}

bool tiled_ok(const GemmArgs& g) {
  return g.K >= BK && g.K % BK == 0 && g.N % 8 == 0 && g.lda % 16 == 0 && g.ldb % 16 == 0 && g.ldo % 8 == 0 &&
         reinterpret_cast<uintptr_t>(g.a) % 16 == 0 && reinterpret_cast<uintptr_t>(g.b) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(g.out) % 16 == 0 &&
         // the epilogues fetch scales and bias in 16-byte pieces
         reinterpret_cast<uintptr_t>(g.a_scale) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(g.b_scale) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(g.bias) % 16 == 0 &&
         // 32-bit byte offsets inside a tile
         (int64_t)512 * g.lda < (int64_t)1 << 31 && (int64_t)512 * g.ldb < (int64_t)1 << 31 &&
         (int64_t)512 * g.ldo < (int64_t)1 << 29;
}

}  // namespace

// Kernel variants. The entry point picks one by shape; tests and the tuning hook
// (cdit_debug_set_gemm_variant) can force any of them.
//          BM   BN  WGM WGN direct epiLDS groupM stages
typedef Cfg<256, 256, 2, 2, false, false, 8> V0;      // register staging, direct stores
typedef Cfg<256, 256, 2, 2, true, true, 8> V1;        // LDS-DMA, 2 stages, 4 waves
typedef Cfg<128, 128, 2, 2, true, true, 8> V6;        // two workgroups per CU
typedef Cfg<256, 256, 2, 4, true, true, 8> V7;        // 8 waves in phase, 2 stages
typedef Cfg<128, 64, 2, 2, true, true, 8, 4> V20;     // small tiles, 4 stages of 128 B
typedef Cfg<64, 128, 2, 2, true, true, 8, 4> V21;
typedef CfgWide<256, 256, 4> V12;                     // 4 waves, 128x128 wave tiles, 16x16x128 MFMA
typedef CfgWide<288, 192, 4> V14;                     // ... 144x96 wave tiles
typedef CfgWide<256, 192, 4> V15;                     // ... 128x96 wave tiles
typedef CfgWide<128, 192, 4, 3> V16;                  // ... 64x96 wave tiles, DMA 3 steps ahead
typedef CfgWide<64, 128, 8, 5> V17;                   // ... 32x64 wave tiles, DMA 5 steps ahead
typedef CfgWide<128, 128, 4, 4> V18;                  // ... 64x64 wave tiles, DMA 4 steps ahead
// the two large tiles with contiguous wave columns and half-line output stores (16 rows x 64
// bytes per store instruction), kept to measure the whole-line stores against: variants 112, 114
typedef CfgWide<256, 256, 4, 2, false> V12H;
typedef CfgWide<288, 192, 4, 2, false> V14H;

// The M = 1 kernel when the shape fits it (variant 51 forces it, 50 the 16-row kernel);
// returns 1 when it is not taken.
template <bool FUSED>
int launch_row1(const GemmArgs& g, uint8_t* q_ws, float* scale_ws, int scale_mode, int variant,
                hipStream_t stream) {
  const bool ok = g.M == 1 && g.K >= 128 && g.K % 128 == 0 && g.K <= 4096 && g.ldb % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(g.a) % 16 == 0 && reinterpret_cast<uintptr_t>(g.b) % 16 == 0 &&
                  (!FUSED || reinterpret_cast<uintptr_t>(q_ws) % 8 == 0) &&
                  (variant < 0 || variant == 51);
  if (!ok) return 1;
  constexpr int rows_wg = kRow1Rows * kRow1Waves;
  auto go = [&](auto chk_tag) {
    hipLaunchKernelGGL((linear_fp8_row1<decltype(chk_tag)::value, FUSED>),
                       dim3((g.N + rows_wg - 1) / rows_wg), dim3(64 * kRow1Waves), 0, stream, g, q_ws,
                       scale_ws, scale_mode);
  };
  switch ((g.K + 1023) / 1024) {
    case 1: go(std::integral_constant<int, 1>{}); break;
    case 2: go(std::integral_constant<int, 2>{}); break;
    case 3: go(std::integral_constant<int, 3>{}); break;
    default: go(std::integral_constant<int, 4>{}); break;
  }
  return 0;
}

int launch_linear_fp8_skinny_fused(const GemmArgs& g, void* q_ws, float* scale_ws, int scale_mode,
                                   int variant, hipStream_t stream) {
  // Bit-identical to the quantizer followed by cdit_fp8_gemm_rowwise only where that call
  // would run the same M <= 16 kernels: arguments it would hand to the any-alignment kernel
  // (N not a multiple of 8, misaligned scales, ...) take the two calls here as well.
  GemmArgs two_step = g;
  two_step.a = q_ws;
  two_step.a_scale = scale_ws;
  two_step.lda = g.K;
  if (!tiled_ok(two_step)) return 1;
  if (launch_row1<true>(g, static_cast<uint8_t*>(q_ws), scale_ws, scale_mode, variant, stream) == 0) return 0;
  const int64_t lds = (int64_t)g.M * (g.K + kFusedPad);
  const bool ok = g.M >= 1 && g.M <= 16 && (variant < 0 || variant == 50) && g.K >= 128 &&
                  g.K % 128 == 0 && g.N % 8 == 0 && lds <= 48 * 1024 && g.lda % 8 == 0 &&
                  g.ldb % 16 == 0 && g.ldo % 8 == 0 &&
                  reinterpret_cast<uintptr_t>(g.a) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(g.b) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(g.out) % 16 == 0 &&
                  reinterpret_cast<uintptr_t>(q_ws) % 8 == 0;
  if (!ok) return 1;
  hipLaunchKernelGGL(linear_fp8_skinny_fused, dim3((g.N + 15) / 16), dim3(256), (size_t)lds, stream,
                     g, static_cast<uint8_t*>(q_ws), scale_ws, scale_mode);
  return 0;
}

struct TileChoice {
  int variant;
  int64_t cost;  // 1000 x CUs x tile area per full round over the CUs (K left out)
};
template <class Tiles, class WideOk>
TileChoice choose_bf16_variant(Tiles tiles, WideOk wide_ok);
template <class WideOk>
int launch_bf16_variant(const GemmArgs& g, int variant, WideOk wide_ok, hipStream_t stream);

int launch_gemm_fp8_stamps(const GemmArgs& g, unsigned long long* stamps, int* workgroups,
                           hipStream_t stream) {
  if (!tiled_ok(g) || g.out_dtype != CDIT_DT_BF16 || g.K < 128 * 3 || g.M <= 16) {
    set_error("cdit_debug_gemm_stamps: the 288 x 192 kernel takes bf16 outputs, aligned operands, "
              "K >= 384 and M > 16");
    return CDIT_EINVAL;
  }
  return launch_wide_stamps<V14>(g, stamps, workgroups, stream);
}

int launch_gemm_fp8(const GemmArgs& g, int variant, hipStream_t stream) {
  if (!tiled_ok(g) || variant == 100) {
    dim3 grid((g.N + 15) / 16, (g.M + 15) / 16);
    hipLaunchKernelGGL(gemm_fp8_generic, grid, dim3(256), 0, stream, g);
    return 0;
  }
  if ((variant < 0 || variant == 51) &&
      launch_row1<false>(g, nullptr, nullptr, 0, variant, stream) == 0)
    return 0;
  if ((variant < 0 && g.M <= 16) || variant == 50) {
    if (g.M > 16) {
      set_error("cdit_fp8_gemm_rowwise: the skinny kernel takes M <= 16, got %d", g.M);
      return CDIT_EINVAL;
    }
    hipLaunchKernelGGL(gemm_fp8_skinny, dim3((g.N + 15) / 16), dim3(256), 0, stream, g);
    return 0;
  }
  // the wide kernels stream K two or more steps ahead: shorter K runs the 128x128 kernel
  // at least `depth` K steps to prefetch, and at least 3: the epilogue operands of a tile are
  // staged in LDS two steps before its end, which must be behind the first barrier of the
  // tile (before it, slower waves may still be reading the previous tile's)
  auto wide_ok = [&](int depth) { return g.K >= 128 * (depth > 3 ? depth : 3); };
  if (g.out_dtype != CDIT_DT_BF16) {
    // fp16 / fp32 outputs (the op's other two out_dtype ids): one large and one small
    // wide tile are built for them, chosen like the small-problem case below; what
    // those cannot take runs the generic kernel.
    const int64_t t_large = (int64_t)((g.M + 255) / 256) * ((g.N + 191) / 192);
    const int64_t t_small = (int64_t)((g.M + 63) / 64) * ((g.N + 127) / 128);
    const int64_t ncu = cu_count() > 0 ? cu_count() : 256;
    const bool large = variant == 15 ||
                       (variant != 17 && (!wide_ok(V17::DEPTH) ||
                                          (t_large + ncu - 1) / ncu * 256 * 192 * 1000 <=
                                              (t_small + ncu - 1) / ncu * 64 * 128 * 1493));
    if (large && wide_ok(V15::DEPTH)) {
      return g.out_dtype == CDIT_DT_F16 ? launch_wide<V15, CDIT_DT_F16>(g, stream)
                                        : launch_wide<V15, CDIT_DT_F32>(g, stream);
    }
    if (!large && wide_ok(V17::DEPTH)) {
      return g.out_dtype == CDIT_DT_F16 ? launch_wide<V17, CDIT_DT_F16>(g, stream)
                                        : launch_wide<V17, CDIT_DT_F32>(g, stream);
    }
    dim3 grid((g.N + 15) / 16, (g.M + 15) / 16);
    hipLaunchKernelGGL(gemm_fp8_generic, grid, dim3(256), 0, stream, g);
    return 0;
  }
  if (variant < 0) {
    variant = choose_bf16_variant(
        [&](int bm, int bn) { return (int64_t)((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn); },
        wide_ok).variant;
  }
  return launch_bf16_variant(g, variant, wide_ok, stream);
}

// Tile choice for a bf16-output problem whose tile count for a bm x bn tile is tiles(bm, bn)
// (a single GEMM, or a batch of GEMMs walked as one tile stream), with the modelled cost of
// that choice; both branches count in the same unit.
template <class Tiles, class WideOk>
TileChoice choose_bf16_variant(Tiles tiles, WideOk wide_ok) {
  // workgroups a round holds: one per CU (what launch_wide starts)
  const int64_t cus = cu_count() > 0 ? cu_count() : 256;
  TileChoice best;
  if (tiles(256, 256) * 256 >= 160 * cus) {
    // Large problems take one of the large-tile wide kernels. Cost model, fitted to
    // measured times: tile area times the number of rounds over the CUs, where a
    // last, partial round of r tiles counts 0.4 + 0.6 r/CUs (the chip is power
    // limited: with fewer CUs busy the clocks rise); ties go to the larger tile.
    auto cost = [&](int bm, int bn, int pen) {
      const int64_t t = tiles(bm, bn), full = t / cus, rem = t % cus;
      return (full * 10 * cus + (rem ? 4 * cus + 6 * rem : 0)) * bm * bn * pen;
    };
    best = {12, cost(256, 256, 100)};
    const struct { int v, bm, bn, pen; } cand[] = {
        {14, 288, 192, 101}, {15, 256, 192, 102}};
    for (const auto& c : cand) {
      const int64_t t = cost(c.bm, c.bn, c.pen);
      if (t < best.cost) best = {c.v, t};
    }
  } else {
    // Smaller problems (the text-stream Linears, M of a few hundred to a few
    // thousand): whole rounds over the CUs times tile area, the small tiles
    // penalised by their measured lower MFMA rate (per mille); ties go to the
    // larger tile. Tiles whose prefetch depth K cannot feed are left out.
    const struct { int v, bm, bn, pen, depth; } cand[] = {
        {12, 256, 256, 1000, 2}, {14, 288, 192, 1000, 2}, {15, 256, 192, 1000, 2},
        {16, 128, 192, 1124, 3}, {18, 128, 128, 1000, 4}, {17, 64, 128, 1493, 5}};
    // K < 256: the kernels without a K stream across tiles (cost not modelled)
    best = {tiles(128, 128) >= cus ? 6 : 21, INT64_MAX / 8};
    for (const auto& c : cand) {
      if (!wide_ok(c.depth)) continue;
      const int64_t t = (tiles(c.bm, c.bn) + cus - 1) / cus * cus * c.bm * c.bn * c.pen;
      if (t < best.cost) best = {c.v, t};
    }
  }
  return best;
}

template <class WideOk>
int launch_bf16_variant(const GemmArgs& g, int variant, WideOk wide_ok, hipStream_t stream) {
  switch (variant) {
    case 0: return launch_tiled<V0>(g, stream);
    case 1: return launch_tiled<V1>(g, stream);
    case 6: return launch_tiled<V6>(g, stream);
    case 7: return launch_tiled<V7>(g, stream);
    case 20: return launch_tiled<V20>(g, stream);
    case 21: return launch_tiled<V21>(g, stream);
    case 12: return wide_ok(V12::DEPTH) ? launch_wide<V12>(g, stream) : launch_tiled<V6>(g, stream);
    case 14: return wide_ok(V14::DEPTH) ? launch_wide<V14>(g, stream) : launch_tiled<V6>(g, stream);
    case 15: return wide_ok(V15::DEPTH) ? launch_wide<V15>(g, stream) : launch_tiled<V6>(g, stream);
    case 16: return wide_ok(V16::DEPTH) ? launch_wide<V16>(g, stream) : launch_tiled<V6>(g, stream);
    case 17: return wide_ok(V17::DEPTH) ? launch_wide<V17>(g, stream) : launch_tiled<V6>(g, stream);
    case 18: return wide_ok(V18::DEPTH) ? launch_wide<V18>(g, stream) : launch_tiled<V6>(g, stream);
    case 112: return wide_ok(V12H::DEPTH) ? launch_wide<V12H>(g, stream) : launch_tiled<V6>(g, stream);
    case 114: return wide_ok(V14H::DEPTH) ? launch_wide<V14H>(g, stream) : launch_tiled<V6>(g, stream);
    default:
      set_error("cdit_fp8_gemm_rowwise: unknown kernel variant %d", variant);
      return CDIT_EINVAL;
  }
}

// The batch as one launch. Returns 0 when launched, -1 when the batch is not taken (the
// caller then runs the members one by one), a CDIT_E* code on error.
int launch_gemm_fp8_grouped(const GemmArgs& common, const GemmGroup& grp, int variant,
                            hipStream_t stream) {
  if (grp.count < 2 || grp.count > kMaxGroup || grp.acts < 1 || grp.acts > kMaxActs ||
      common.out_dtype != CDIT_DT_BF16)
    return -1;
  for (int s = 0; s < grp.acts; ++s) {
    if (grp.M[s] <= 16 || grp.first_member[s + 1] <= grp.first_member[s]) return -1;
    for (int p = grp.first_member[s]; p < grp.first_member[s + 1]; ++p) {
      GemmArgs g = common;
      g.a = grp.a[s];
      g.a_scale = grp.a_scale[s];
      g.M = grp.M[s];
      g.b = grp.b[p];
      g.b_scale = grp.b_scale[p];
      g.bias = grp.bias[p];
      g.out = grp.out[p];
      g.N = grp.N[p];
      g.ldo = grp.ldo[p];
      if (!tiled_ok(g) || g.N <= 0) return -1;
    }
  }
  auto wide_ok = [&](int depth) { return common.K >= 128 * (depth > 3 ? depth : 3); };
  auto tiles = [&](int bm, int bn) {
    int64_t t = 0;
    for (int s = 0; s < grp.acts; ++s) {
      int64_t cols = 0;
      for (int p = grp.first_member[s]; p < grp.first_member[s + 1]; ++p) cols += (grp.N[p] + bn - 1) / bn;
      t += (int64_t)((grp.M[s] + bm - 1) / bm) * cols;
    }
    return t;
  };
  if (variant < 0) {
    const TileChoice whole = choose_bf16_variant(tiles, wide_ok);
    variant = whole.variant;
    if (grp.acts > 1) {
      // One tile stream is not always the cheaper form: the tiles of a small activation
      // can push a batch that filled whole rounds of large tiles into one more round
      // (FLUX ff.net.0.proj: 4096 rows fill three rounds of 256 x 256 tiles exactly, the
      // 512 text rows add a fourth, nearly empty one; on its own the text GEMM is one round
      // of small tiles: measured 148 us as two launches, 173 as one). Compare with one
      // launch per activation, each with the tile it would choose, plus what a further
      // launch costs (about 3 us, in the unit of the model: a CU does about 4900 K-steps of
      // one output element per us).
      const int64_t cus = cu_count() > 0 ? cu_count() : 256;
      int64_t apart = (grp.acts - 1) * (3 * 1000 * cus * 4900 / (common.K > 0 ? common.K : 1));
      for (int s = 0; s < grp.acts; ++s) {
        auto tiles_s = [&](int bm, int bn) {
          int64_t cols = 0;
          for (int p = grp.first_member[s]; p < grp.first_member[s + 1]; ++p) cols += (grp.N[p] + bn - 1) / bn;
          return (int64_t)((grp.M[s] + bm - 1) / bm) * cols;
        };
        apart += choose_bf16_variant(tiles_s, wide_ok).cost;
      }
      // (the model is good to a few per cent: within 3 % the single stream is kept, which
      // measured faster in every such case)
      if (apart * 100 < whole.cost * 97) {
        for (int s = 0; s < grp.acts; ++s) {
          GemmGroup one = {};
          one.acts = 1;
          one.count = grp.first_member[s + 1] - grp.first_member[s];
          one.a[0] = grp.a[s];
          one.a_scale[0] = grp.a_scale[s];
          one.M[0] = grp.M[s];
          one.first_member[0] = 0;
          one.first_member[1] = one.count;
          for (int p = 0; p < one.count; ++p) {
            const int src = grp.first_member[s] + p;
            one.b[p] = grp.b[src];
            one.b_scale[p] = grp.b_scale[src];
            one.bias[p] = grp.bias[src];
            one.out[p] = grp.out[src];
            one.N[p] = grp.N[src];
            one.ldo[p] = grp.ldo[src];
            one.epilogue[p] = grp.epilogue[src];
          }
          int rc = one.count >= 2 ? launch_gemm_fp8_grouped(common, one, -1, stream) : -1;
          if (rc > 0) return rc;
          if (rc == 0) continue;
          for (int p = 0; p < one.count; ++p) {  // a single member, or a group that is not taken
            GemmArgs g = common;
            g.a = one.a[0];
            g.a_scale = one.a_scale[0];
            g.M = one.M[0];
            g.b = one.b[p];
            g.b_scale = one.b_scale[p];
            g.bias = one.bias[p];
            g.out = one.out[p];
            g.N = one.N[p];
            g.ldo = one.ldo[p];
            g.epilogue = one.epilogue[p];
            if ((rc = launch_gemm_fp8(g, -1, stream))) return rc;
          }
        }
        return 0;
      }
    }
  }
  switch (variant) {
    case 12: return wide_ok(V12::DEPTH) ? launch_wide_grouped<V12>(common, grp, stream) : -1;
    case 14: return wide_ok(V14::DEPTH) ? launch_wide_grouped<V14>(common, grp, stream) : -1;
    case 15: return wide_ok(V15::DEPTH) ? launch_wide_grouped<V15>(common, grp, stream) : -1;
    case 16: return wide_ok(V16::DEPTH) ? launch_wide_grouped<V16>(common, grp, stream) : -1;
    case 17: return wide_ok(V17::DEPTH) ? launch_wide_grouped<V17>(common, grp, stream) : -1;
    case 18: return wide_ok(V18::DEPTH) ? launch_wide_grouped<V18>(common, grp, stream) : -1;
    default: return -1;  // the kernels without a tile stream have no grouped form
  }
}

// ---------------------------------------------------------------------------
// Measurement aid: a loop of nothing but the wide kernel's MFMA instruction on register
// operands (one wave per SIMD, four per workgroup, 16 independent accumulators), so that the
// rate the matrix cores sustain before a byte is moved can be timed on the part at hand.
// RANDOM: operands are pseudo-random e4m3 codes with |value| <= 1.75 (what the benchmark's
// weights are drawn from); otherwise every code is 1.0. The clock a power-limited part
// settles at depends on the operand bits, and with it the ceiling of any FP8 kernel.
namespace {
template <bool RANDOM>
__global__ __launch_bounds__(256) void mfma_only_loop(float* out, int iters) {
  constexpr int NACC = 16, NOP = 4;
  v8i a[NOP], b[NOP];
  uint32_t h = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
  for (int o = 0; o < NOP; ++o)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      h = h * 1664525u + 1013904223u;
      a[o][i] = RANDOM ? (int)((h ^ (h >> 13)) & 0xBFBFBFBFu) : 0x38383838;
      h = h * 1664525u + 1013904223u;
      b[o][i] = RANDOM ? (int)((h ^ (h >> 11)) & 0xBFBFBFBFu) : 0x38383838;
    }
  v4f acc[NACC];
#pragma unroll
  for (int j = 0; j < NACC; ++j) acc[j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < NACC; ++j)
      acc[j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[j % NOP], b[(j / NOP) % NOP], acc[j],
                                                                0, 0, 0, 0, 0, 0);
  }
  float sum = 0.0f;
#pragma unroll
  for (int j = 0; j < NACC; ++j) sum += (acc[j][0] + acc[j][1]) + (acc[j][2] + acc[j][3]);
  out[blockIdx.x * 256 + threadIdx.x] = sum;
}
}  // namespace

int launch_mfma_only(float* out, int blocks, int iters, bool random_operands, double* flop,
                     hipStream_t stream) {
  if (random_operands) {
    hipLaunchKernelGGL(mfma_only_loop<true>, dim3(blocks), dim3(256), 0, stream, out, iters);
  } else {
    hipLaunchKernelGGL(mfma_only_loop<false>, dim3(blocks), dim3(256), 0, stream, out, iters);
  }
  if (flop) *flop = (double)blocks * 4.0 * iters * 16.0 * (2.0 * 16 * 16 * 128);
  return 0;
}

}  // namespace cdit
