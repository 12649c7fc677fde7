// Weight-only FP8 GEMM (w8a16) for gfx950: bf16 activations x e4m3 weights,
// the weights dequantized to bf16 inside the mainloop, fp32 accumulate,
// per-output-channel scale + bias + optional GELU-tanh + bf16 in the epilogue.
//
//   out[m,n] = epi((sum_k x[m,k] float(b[n,k])) * b_scale[n] + bias[n])
//
// Every e4m3 value is exactly representable in bf16, so the in-loop conversion
// (v_cvt_scalef32_pk_bf16_fp8 with scale 1) is lossless and the weight never
// exists in HBM at 16 bits: B costs 1 byte per element of traffic instead of
// the 1 (read) + 2 (write) + 2 (read) of dequantize-then-GEMM.
//
// MFMA: v_mfma_f32_32x32x16_bf16; per lane 8 consecutive K elements of row
// (lane&31), K-group h = lane>>5. The K order inside a 32-element block is
// free as long as A and B agree, so lane group h takes elements [16h, 16h+16)
// of the block: one 16-byte read of B (two MFMA steps of 8 bytes) and one
// 32-byte read of A.
//
// Tile: BM x BN outputs, BK = 64 elements per pipeline step: A panel rows are
// 128 bytes (8 chunks, chunk c of row r at position c ^ ((r>>1)&7)), B panel
// rows are 64 bytes (4 chunks, chunk c of row r at position c ^ ((r>>2)&3)):
// with 64 LDS banks of 4 B and 16 lanes served per pass, both are conflict free
// for the 16-byte operand reads. Panels
// are staged with 128-bit LDS-DMA loads, double buffered.
//
// Replaces F.linear(x, W.dequantize(), bias) of the reference's
// float8_weight_only mode (src/cache_dit/quantization/torchao/quantize_ao.py:604-610).
#include <type_traits>

#include "gemm_common.h"
#include "quant_device.h"

namespace cdit {
namespace {

constexpr int BKE = 64;  // K elements per pipeline step

template <int BM_, int BN_, int WGM_, int WGN_, bool EPI_LDS_, int GROUP_M_>
struct CfgW {
  static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
  static constexpr bool EPI_LDS = EPI_LDS_;
  static constexpr int GROUP_M = GROUP_M_;
  static constexpr int WAVES = WGM * WGN;
  static constexpr int THREADS = WAVES * 64;
  static constexpr int WM = BM / WGM, WN = BN / WGN;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int A_ROW = BKE * 2, B_ROW = BKE;  // bytes per panel row
  static constexpr int A_BYTES = BM * A_ROW, B_BYTES = BN * B_ROW;
  static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
  static constexpr int EPI_PITCH = WN * 2 + 16;
  static constexpr int EPI_BYTES = EPI_LDS ? WAVES * 32 * EPI_PITCH : 0;
  static constexpr int LDS_BYTES = (2 * STAGE_BYTES > EPI_BYTES) ? 2 * STAGE_BYTES : EPI_BYTES;
  // LDS-DMA instructions per wave and stage (1 KiB each)
  static constexpr int A_DMA = A_BYTES / 1024 / WAVES, B_DMA = B_BYTES / 1024 / WAVES;
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
  static_assert(A_BYTES % (1024 * WAVES) == 0 && B_BYTES % (1024 * WAVES) == 0,
                "panel/waves mismatch");
};

template <class C>
__global__ __launch_bounds__(C::THREADS) void gemm_w8a16_tiled(GemmArgs g, int tiles_m,
                                                               int tiles_n) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / C::WGN, wn = wave % C::WGN;

  int tm, tn;
  tile_of_block<C::GROUP_M>(blockIdx.x, gridDim.x, tiles_m, tiles_n, &tm, &tn);
  const int m0 = tm * C::BM, n0 = tn * C::BN;
  const uint8_t* __restrict__ A =
      static_cast<const uint8_t*>(g.a) + (int64_t)m0 * g.lda * 2;  // bf16: 2 bytes/element
  const uint8_t* __restrict__ B = g.b + (int64_t)n0 * g.ldb;
  const int rows_a = g.M - m0, rows_b = g.N - n0;

  // ---- LDS-DMA maps: a wave instruction fills 1 KiB = 8 A rows or 16 B rows;
  // lane l lands on (row l/8, position l%8) resp. (row l/4, position l%4) and
  // fetches the logical chunk that the swizzle puts there.
  uint32_t a_off[C::A_DMA], b_off[C::B_DMA];
#pragma unroll
  for (int p = 0; p < C::A_DMA; ++p) {
    const int row = (wave * C::A_DMA + p) * 8 + (lane >> 3);
    const int c = (lane & 7) ^ ((row >> 1) & 7);
    a_off[p] = (uint32_t)min(row, rows_a - 1) * (uint32_t)(g.lda * 2) + c * 16;
  }
#pragma unroll
  for (int p = 0; p < C::B_DMA; ++p) {
    const int row = (wave * C::B_DMA + p) * 16 + (lane >> 2);
    const int c = (lane & 3) ^ ((row >> 2) & 3);
    b_off[p] = (uint32_t)min(row, rows_b - 1) * (uint32_t)g.ldb + c * 16;
  }

  // ---- operand read maps; kb = 32-element K block inside the step (0..1)
  const int h = lane >> 5;
  uint32_t rd_a[2][2], rd_b[2];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    const int ra_row = wm * C::WM + (lane & 31);
#pragma unroll
    for (int e = 0; e < 2; ++e)
      rd_a[kb][e] = ra_row * C::A_ROW + (((4 * kb + 2 * h + e) ^ ((lane >> 1) & 7)) << 4);
    const int rb_row = wn * C::WN + (lane & 31);
    rd_b[kb] = C::A_BYTES + rb_row * C::B_ROW + (((2 * kb + h) ^ ((lane >> 2) & 3)) << 4);
  }

  v16f acc[C::TM][C::TN];
#pragma unroll
  for (int i = 0; i < C::TM; ++i)
#pragma unroll
    for (int j = 0; j < C::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int KT = g.K / BKE;

  auto fetch = [&](int kt, int stage) {
    const uint8_t* Ak = A + (int64_t)kt * C::A_ROW;
    const uint8_t* Bk = B + (int64_t)kt * C::B_ROW;
    uint8_t* st = smem + stage * C::STAGE_BYTES;
#pragma unroll
    for (int p = 0; p < C::A_DMA; ++p)
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(Ak + a_off[p]),
          (__attribute__((address_space(3))) void*)(st + (wave * C::A_DMA + p) * 1024), 16, 0, 0);
#pragma unroll
    for (int p = 0; p < C::B_DMA; ++p)
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(Bk + b_off[p]),
          (__attribute__((address_space(3))) void*)(st + C::A_BYTES +
                                                    (wave * C::B_DMA + p) * 1024),
          16, 0, 0);
  };

  auto compute = [&](int stage) {
    const uint8_t* st = smem + stage * C::STAGE_BYTES;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      v8bf a_lo[C::TM], a_hi[C::TM];  // MFMA steps 0 and 1 of this block
#pragma unroll
      for (int i = 0; i < C::TM; ++i) {
        a_lo[i] = *reinterpret_cast<const v8bf*>(st + rd_a[kb][0] + i * 32 * C::A_ROW);
        a_hi[i] = *reinterpret_cast<const v8bf*>(st + rd_a[kb][1] + i * 32 * C::A_ROW);
      }
#pragma unroll
      for (int j = 0; j < C::TN; ++j) {
        const uint4 w = *reinterpret_cast<const uint4*>(st + rd_b[kb] + j * 32 * C::B_ROW);
        // 16 e4m3 bytes -> 16 bf16 (exact), two at a time
        v2bf c0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.x, 1.0f, false);
        v2bf c1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.x, 1.0f, true);
        v2bf c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.y, 1.0f, false);
        v2bf c3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.y, 1.0f, true);
        v2bf c4 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.z, 1.0f, false);
        v2bf c5 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.z, 1.0f, true);
        v2bf c6 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.w, 1.0f, false);
        v2bf c7 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w.w, 1.0f, true);
        const v8bf b_lo = {c0[0], c0[1], c1[0], c1[1], c2[0], c2[1], c3[0], c3[1]};
        const v8bf b_hi = {c4[0], c4[1], c5[0], c5[1], c6[0], c6[1], c7[0], c7[1]};
#pragma unroll
        for (int i = 0; i < C::TM; ++i) {
          // operands swapped: result rows follow B (n), result columns follow A (m)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b_lo, a_lo[i], acc[i][j], 0, 0, 0);
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b_hi, a_hi[i], acc[i][j], 0, 0, 0);
        }
      }
    }
  };

  fetch(0, 0);
  for (int kt = 0; kt < KT; ++kt) {
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of step kt is in LDS
    __syncthreads();                     // ... and everyone's; stage (kt+1)&1 is free again
    if (kt + 1 < KT) fetch(kt + 1, (kt + 1) & 1);
    compute(kt & 1);
  }

  if constexpr (C::EPI_LDS) __syncthreads();  // all waves are done with the stage buffers
  tile_epilogue<C>(acc, g, smem + wave * (32 * C::EPI_PITCH), m0, n0, wm, wn, lane);
}

// ---------------------------------------------------------------------------
// Wide kernel: the schedule of the wide w8a8 kernel (one persistent workgroup of 4
// waves per CU, one wave per SIMD with all 256 AGPRs as accumulators, LDS-DMA by
// buffer loads spread over the MFMA stream DEPTH steps ahead, A panel in DEPTH + 1 LDS
// stages and B panel in DEPTH, one barrier per K step, the DMA stream running across
// tiles) with bf16 MFMAs:
// v_mfma_f32_32x32x16_bf16 (8 passes), K steps of 64 elements, wave tile
// (BM/2) x (BN/2) as TM x TN blocks of 32x32, four MFMAs per block and step.
//
// Panels: A rows 128 B (bf16), chunk c of row r at c ^ ((r>>1)&7); B rows 64 B
// (e4m3), chunk c at c ^ ((r>>2)&3). A lane reads, per 32-row block, the four A
// chunks 4t+2h+s (h = lane>>5) and the two B chunks 2t+h: the 16 B bytes of one
// chunk are the weights of MFMA steps 2t and 2t+1 (K order permuted identically on
// both sides). The weights are converted to bf16 once per step, two conversion
// instructions (half an operand) at a time on a compile-time schedule that ends two
// MFMAs ahead of the first use, and kept for all row blocks.
//
// The B fragments take their 32 rows in a permuted order, operand row p reads
// panel row 16 ((p>>2)&1) + 4 (p>>3) + (p&3) of its block: with the operands
// swapped (weights first) a lane then ends with 16 consecutive output columns per
// block, n = 32j + 16h + r for accumulator register r, and stores them with two
// 16-byte stores, no transpose.
template <int BM_, int BN_, int GROUP_M_, int DEPTH_ = 2>
struct CfgWW {
  static constexpr int BM = BM_, BN = BN_, GROUP_M = GROUP_M_;
  // K steps the DMA stream runs ahead of the MFMAs (A panel in DEPTH + 1 LDS stages,
  // B panel in DEPTH): 2 for the large tiles, more for small tiles with short steps
  static constexpr int DEPTH = DEPTH_;
  static constexpr int WAVES = 4, THREADS = 256;
  static constexpr int WM = BM / 2, WN = BN / 2;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int H = TM / 2;
  static constexpr int A_ROW = BKE * 2, B_ROW = BKE;
  static constexpr int A_BYTES = BM * A_ROW, B_BYTES = BN * B_ROW;
  static constexpr int A_STAGES = DEPTH + 1, B_STAGES = DEPTH;
  static constexpr int B_BASE = A_STAGES * A_BYTES;
  static constexpr int PANEL_BYTES = A_STAGES * A_BYTES + B_STAGES * B_BYTES;
  // b_scale and bias of a tile's BN columns are staged behind the panels (1 KiB each)
  static constexpr int EPI_BS = PANEL_BYTES, EPI_BI = PANEL_BYTES + 1024;
  static constexpr int LDS_BYTES = PANEL_BYTES + 2048;
  static_assert(BN * 4 <= 1024, "one LDS-DMA instruction per staged operand");
  // DMA instructions (1 KiB: 8 A rows or 16 B rows) per wave and step
  static constexpr int NDA = BM / 8 / WAVES, NDB = BN / 16 / WAVES, ND = NDA + NDB;
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
  static_assert(BM % 32 == 0 && BN % 64 == 0, "panels are dealt 1 KiB x 4 waves at a time");
  static_assert(TM * TN <= 16, "accumulators: at most 256 registers");
  static_assert(TM >= 2, "two halves per step");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
  static_assert(DEPTH >= 2 && (DEPTH - 2) * ND + NDA < 63, "DMA instructions in flight: vmcnt has 6 bits");

  // Issue schedule of a K step. Between two MFMAs (8 passes, 32 cycles) the wave issues
  // in order; one LDS read or DMA instruction and two conversions (8 cycles each) fit,
  // more delays the next MFMA, and the matrix core never makes that up. So everything is
  // spread: all slot numbers below are compile-time constants.
  //
  // First half: S1 MFMAs over the rows 0..H-1, MFMA step q of all their blocks before step
  // q+1: slot s = (q*H + i)*TN + j. A new weight operand (j, q) is then needed every
  // H slots only, which leaves room to convert it in pieces (below). Items: the
  // 4 (TM-1) single LDS reads of the fragments A_1 .. A_{TM-1} in the order of their first
  // use, and the NDA DMA instructions of the A panel, merged evenly, a read first, and
  // spread evenly over the slots.
  static constexpr int S1 = H * 4 * TN, NR1 = 4 * (TM - 1), T1 = NR1 + NDA;
  static constexpr int R = TM - H, S2 = R * 4 * TN, NR2 = 4 + 2 * TN;
  static constexpr int i_of_slot1(int s) { return s / TN % H; }
  static constexpr int q_of_slot1(int s) { return s / (H * TN); }
  // first use of A_i, MFMA step q, counted in slots from the start of the step
  static constexpr int use_a(int i, int q) {
    return i < H ? (q * H + i) * TN : S1 + (q * R + i - H) * TN;
  }
  static constexpr int H1 = H > 1 ? H - 1 : 1;
  static constexpr int read1_row(int r) {  // read r of the first half: fragment A_i ...
    return r < 4 * (H - 1) ? 1 + r % H1 : H + (r - 4 * (H - 1)) % R;
  }
  static constexpr int read1_step(int r) {  // ... MFMA step q
    return r < 4 * (H - 1) ? r / H1 : (r - 4 * (H - 1)) / R;
  }
  static constexpr int item_of_read1(int r) { return r * T1 / NR1; }
  static constexpr bool is_read1(int t) {
    for (int r = 0; r < NR1; ++r)
      if (item_of_read1(r) == t) return true;
    return false;
  }
  static constexpr int read1_index(int t) {  // reads before item t
    int n = 0;
    for (int r = 0; r < NR1; ++r) n += item_of_read1(r) < t;
    return n;
  }
  static constexpr int dma1_index(int t) { return t - read1_index(t); }
  static constexpr int slot1(int t) { return t * S1 / T1; }
  static constexpr bool first_half_reads_in_time() {
    for (int r = 0; r < NR1; ++r)
      if (slot1(item_of_read1(r)) + 3 > use_a(read1_row(r), read1_step(r))) return false;
    return true;
  }
  static_assert(first_half_reads_in_time(), "A fragment read too late for its first use");
  // Second half: S2 MFMAs over the rows H..TM-1 in the same order, slot s =
  // (q*R + i-H)*TN + j. The LDS reads of the next step (its raw weights, 2 per column, and
  // A_0, 4) are spread evenly over the slots from 1 on: first halves of the weights, A_0 of
  // MFMA step 0, second halves, rest of A_0. The NDB DMA instructions of the B panel go in
  // the middle of their share of the slots.
  static constexpr int key_w(int j, int t) { return t == 0 ? j : TN + 1 + j; }
  static constexpr int key_a0(int q) { return q == 0 ? TN : 2 * TN + 1 + q; }
  static constexpr int rank2(int key) {  // reads of the second half with a smaller key
    int n = 0;
    for (int j = 0; j < TN; ++j)
      for (int t = 0; t < 2; ++t) n += key_w(j, t) < key;
    for (int q = 0; q < 4; ++q) n += key_a0(q) < key;
    return n;
  }
  static constexpr int slot2(int key) { return 1 + rank2(key) * (S2 - 1) / NR2; }
  static constexpr int slot_w(int j, int t) { return slot2(key_w(j, t)); }  // read t (0/1) of column j
  static constexpr int slot_a0(int q) { return slot2(key_a0(q)); }
  // Conversions. Weight operand (j, q) (8 e4m3 bytes -> 8 bf16, four conversion
  // instructions) is converted as two half operands. Time t counts first-half slots of the
  // step the operand belongs to; t < 0 is second-half slot S2 + t of the step before (the
  // raw weights of a step are read during the step before it). A half operand must be
  // converted in front of slot use - CONVERT_AHEAD at the latest (an MFMA operand written
  // by a VALU instruction just before the inline-assembly MFMA reads stale data), and not
  // before the registers it goes to have been read for the last time (plus one MFMA) and
  // the LDS read it comes from has had three slots to land. Operands are placed latest
  // deadline first, each half in the latest slot with room for it; the smallest number of
  // half operands per slot that works is taken. Tiles too small for any of that convert
  // each operand whole in front of slot use - CONVERT_AHEAD, the first ones at the top of
  // the step (kConvTop).
  static constexpr int CONVERT_AHEAD = 2;
  static constexpr int kConvTop = -1000;
  static constexpr bool PIN_CONVERT = TM * TN >= 12;  // see convert_half() in the kernel
  static constexpr int last_use2(int j, int q) { return (q * R + R - 1) * TN + j; }
  static constexpr int conv_deadline(int j, int q) { return q * H * TN + j - CONVERT_AHEAD; }
  static constexpr int conv_release(int j, int q) {
    const int a = last_use2(j, q) + 2, b = slot_w(j, q >> 1) + 3;
    return (a > b ? a : b) - S2;
  }
  struct ConvSched {
    int t[TN][4][2];
    bool ok;
  };
  static constexpr ConvSched conv_sched_with(int cap) {
    ConvSched c{};
    c.ok = true;
    int load[S1 + S2] = {};  // half operands in slot t, at index t + S2
    for (int o = 4 * TN - 1; o >= 0; --o) {
      const int q = o / TN, j = o % TN;
      for (int h = 1; h >= 0; --h) {
        int t = conv_deadline(j, q);
        while (t >= conv_release(j, q) && load[t + S2] >= cap) --t;
        if (t < conv_release(j, q)) {
          c.ok = false;
          return c;
        }
        ++load[t + S2];
        c.t[j][q][h] = t;
      }
    }
    return c;
  }
  static constexpr ConvSched conv_sched() {
    for (int cap = 1; cap <= 2; ++cap) {
      const ConvSched c = conv_sched_with(cap);
      if (c.ok) return c;
    }
    ConvSched c{};
    c.ok = true;
    for (int j = 0; j < TN; ++j)
      for (int q = 0; q < 4; ++q)
        for (int h = 0; h < 2; ++h)
          c.t[j][q][h] = conv_deadline(j, q) < 0 ? kConvTop : conv_deadline(j, q);
    return c;
  }
  static constexpr ConvSched CONV = conv_sched();
  static constexpr int slot_dma2(int p) { return (2 * p + 1) * S2 / (2 * NDB); }
};

struct AFrag {
  v8bf k[4];  // operands of MFMA steps 0..3 of a K step (one 32-row block)
};
struct WRaw {
  uint4 t[2];  // weights as read from LDS: 2 x 16 e4m3 bytes
};

// acc (+)= W-fragment x A-fragment, accumulator tied to an AGPR tuple (see the wide
// w8a8 kernel for why this is inline assembly and what that obliges the code to do).
template <bool FIRST>
__device__ __forceinline__ void mfma_32x32x16_bf16(v16f& acc, const v8bf& w, const v8bf& a) {
  if constexpr (FIRST) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=a"(acc) : "v"(w), "v"(a));
  } else {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(w), "v"(a));
  }
}

struct NoGroup {};

// GROUPED: the launch walks the tiles of a GemmGroup as one tile stream, as the w8a8
// kernel's grouped form does (gemm_fp8.hip): sibling Linears on one activation are members
// stacked along N, the Linears of the same stage on other activations follow; every member
// has its own weight, scale, bias, output and epilogue flag, K and the row strides are
// common (the B-side fields of `g` and grp.a_scale are unused). The instances without it are
// unchanged by its existence.
template <class C, bool GROUPED = false>
__global__ __launch_bounds__(C::THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) void
gemm_w8a16_wide(GemmArgs g, int tiles_m, int tiles_n,
                std::conditional_t<GROUPED, GemmGroup, NoGroup> grp) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: M0 from scalar code
  const int wm = wave >> 1, wn = wave & 1;
  // local copies: a template-dependent expression as a builtin argument inside a
  // lambda makes the host pass drop the kernel stub without a diagnostic
  constexpr int TM = C::TM, TN = C::TN, H = C::H, A_ROW = C::A_ROW, B_ROW = C::B_ROW;
  constexpr int D = C::DEPTH;
  const int KT = g.K / BKE;  // >= D (checked by the launcher)
  int ntiles = tiles_m * tiles_n;
  if constexpr (GROUPED) ntiles = grp.tile_begin[grp.acts];

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
  int m0, n0;       // tile being computed
  int cur = 0;      // member it belongs to
  int cur_act = 0;  // and its activation
  {
    const Where w = locate(blockIdx.x);
    cur = w.member;
    cur_act = w.act;
    m0 = w.m0;
    n0 = w.n0;
  }

  // DMA source: the tile whose panels the DMA stream currently fetches
  const uint8_t* A;
  const uint8_t* B;
  uint32_t off[C::ND];
  int nrec = 0x7fffffff;  // 0: the stream has run past the last tile, fetch nothing
  // The lane offsets only depend on the tile through the clamps at the last rows of A
  // and B: between two tiles without partial panels they are not recomputed.
  bool off_clamped = true;  // the first call computes them
  auto set_source = [&](int sm0, int sn0, int member, int act) {
    A = a_of(act) + (int64_t)sm0 * g.lda * 2;
    B = b_of(member) + (int64_t)sn0 * g.ldb;
    const int rows_a = m_of(act) - sm0, rows_b = n_of(member) - sn0;
    const bool clamped = rows_a < C::BM || rows_b < C::BN;
    if (!clamped && !off_clamped) return;
    off_clamped = clamped;
    int l = lane;  // opaque: keeps the row indices out of registers across the K loop
    asm volatile("" : "+v"(l));
#pragma unroll
    for (int p = 0; p < C::NDA; ++p) {  // 8 rows of 128 B per instruction
      const int row = (wave + 4 * p) * 8 + (l >> 3);
      const int c = (l & 7) ^ ((row >> 1) & 7);
      off[p] = (uint32_t)min(row, rows_a - 1) * (uint32_t)(g.lda * 2) + c * 16;
    }
#pragma unroll
    for (int p = 0; p < C::NDB; ++p) {  // 16 rows of 64 B per instruction
      const int row = (wave + 4 * p) * 16 + (l >> 2);
      const int c = (l & 3) ^ ((row >> 2) & 3);
      off[C::NDA + p] = (uint32_t)min(row, rows_b - 1) * (uint32_t)g.ldb + c * 16;
    }
  };
  set_source(m0, n0, cur, cur_act);
  auto dma_a = [&](int kt, int a_lds, int p) {
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(A), 0, nrec, 0x00020000);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        rsrc, (__attribute__((address_space(3))) void*)(smem + a_lds + (wave + 4 * p) * 1024), 16,
        (int)off[p], kt * A_ROW, 0, 0);
  };
  auto dma_b = [&](int kt, int b_lds, int p) {
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(B), 0, nrec, 0x00020000);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        rsrc, (__attribute__((address_space(3))) void*)(smem + b_lds + (wave + 4 * p) * 1024), 16,
        (int)off[C::NDA + p], kt * B_ROW, 0, 0);
  };

  // operand read map: A row lane&31 of its block, chunks 4t+2h+s; W operand row
  // p = lane&31 reads panel row 16((p>>2)&1) + 4(p>>3) + (p&3), chunks 2t+h
  const int h = lane >> 5, r32 = lane & 31;
  const int wrow = 16 * ((r32 >> 2) & 1) + 4 * (r32 >> 3) + (r32 & 3);
  uint32_t rd_a[4], rd_b[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int e = 0; e < 2; ++e)
      rd_a[2 * t + e] =
          (wm * C::WM + r32) * C::A_ROW + (((4 * t + 2 * h + e) ^ ((r32 >> 1) & 7)) << 4);
    rd_b[t] = (wn * C::WN + wrow) * C::B_ROW + (((2 * t + h) ^ ((wrow >> 2) & 3)) << 4);
  }
  // __restrict__: loads through a restrict-qualified pointer carry alias scope
  // information. Without it the compiler assumes that an LDS read may alias any
  // LDS-DMA write in flight and puts s_waitcnt vmcnt(0) in front of the read, which
  // drains the DMA stream at every step. The stages read in a step are never the
  // ones its DMA fills; the explicit waits before the barriers order the two.
  auto read_a = [&](const uint8_t* __restrict__ st, int i) -> AFrag {
    AFrag f;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      f.k[q] = *reinterpret_cast<const v8bf*>(st + rd_a[q] + i * 32 * C::A_ROW);
    return f;
  };
  auto read_a1 = [&](const uint8_t* __restrict__ st, int i, int q) -> v8bf {
    return *reinterpret_cast<const v8bf*>(st + rd_a[q] + i * 32 * C::A_ROW);
  };
  auto read_w1 = [&](const uint8_t* __restrict__ st, int j, int t) -> uint4 {
    return *reinterpret_cast<const uint4*>(st + rd_b[t] + j * 32 * C::B_ROW);
  };
  auto read_w = [&](const uint8_t* __restrict__ st, int j) -> WRaw {
    WRaw f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
      f.t[t] = *reinterpret_cast<const uint4*>(st + rd_b[t] + j * 32 * C::B_ROW);
    return f;
  };

  v16f acc[TM][TN];
  AFrag af[TM];
  AFrag wf[TN];  // converted weights
  WRaw wr[TN];   // weights as read from LDS (next step's, until converted)

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
    // previous tile's last step)
#pragma unroll
    for (int j = 0; j < TN; ++j) wr[j] = read_w(smem + b_cur, j);
    af[0] = read_a(smem + a_cur, 0);

    // One K step; FIRST: step 0 of the tile (the accumulators start from zero).
    // EVENTS: the step may be one of the last max(D, 2) of the tile, where the DMA stream
    // moves on to the next tile and the epilogue operands are staged. The steps before
    // them run in a loop of their own without these tests: what stands between the last
    // MFMA of a step and the first of the next (tests, taken branches) is time the matrix
    // core waits.
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
        // b_scale and bias of this tile's columns go to the LDS with two DMA instructions
        // (every wave issues both: equal instruction counts; the same bytes land four
        // times) instead of 6 TN loads per lane at the start of the epilogue. What lies
        // beyond N reads as zero, a null bias is an empty buffer.
        const float* cur_b_scale = g.b_scale;
        const uint16_t* cur_bias = g.bias;
        if constexpr (GROUPED) {
          cur_b_scale = grp.b_scale[cur];
          cur_bias = grp.bias[cur];
        }
        const int cur_n = n_of(cur);
        const __amdgpu_buffer_rsrc_t bs_buf = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(cur_b_scale), 0, cur_n * 4, 0x00020000);
        const __amdgpu_buffer_rsrc_t bi_buf = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint16_t*>(cur_bias), 0, cur_bias ? cur_n * 2 : 0, 0x00020000);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            bs_buf, (__attribute__((address_space(3))) void*)(smem + C::EPI_BS), 16,
            n0 * 4 + 16 * lane, 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            bi_buf, (__attribute__((address_space(3))) void*)(smem + C::EPI_BI), 16,
            n0 * 2 + 16 * lane, 0, 0, 0);
      }
      // step (of its tile) to fetch
      const int kd = !EVENTS || kt + D < KT ? kt + D : kt + D - KT;
      const uint8_t* st = smem + a_cur;
      // half h of the weight operand of column j, MFMA step q: 4 e4m3 bytes -> 4 bf16
      auto convert_half = [&](int j, int q, int h) {
        const uint4& w = wr[j].t[q >> 1];
        const uint32_t src = (q & 1) ? (h ? w.w : w.z) : (h ? w.y : w.x);
        uint4 o = __builtin_bit_cast(uint4, wf[j].k[q]);
        uint32_t c0, c1;
        if constexpr (C::PIN_CONVERT) {
          // Inline assembly (volatile): the conversions stay in the MFMA slot they are
          // written in. As builtins they are pure functions of loaded values, and with the
          // large wave tiles the compiler gathered most of a step's conversions at the top
          // of the loop, where the matrix core then waited for them (with the small wave
          // tiles its own placement is the better one).
          asm volatile("v_cvt_scalef32_pk_bf16_fp8 %0, %1, 1.0" : "=v"(c0) : "v"(src));
          asm volatile("v_cvt_scalef32_pk_bf16_fp8 %0, %1, 1.0 op_sel:[1,0,0]" : "=v"(c1) : "v"(src));
        } else {
          c0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(src, 1.0f, false));
          c1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(src, 1.0f, true));
        }
        if (h) {
          o.z = c0;
          o.w = c1;
        } else {
          o.x = c0;
          o.y = c1;
        }
        wf[j].k[q] = __builtin_bit_cast(v8bf, o);
      };
      // the half operands the schedule puts at time t (CfgWW::CONV)
      auto conversions_at = [&](int t) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h)
              if (C::CONV.t[j][q][h] == t) convert_half(j, q, h);
      };
      auto mfma = [&](int i, int j, int q) {
        if (FIRST && q == 0) {
          mfma_32x32x16_bf16<true>(acc[i][j], wf[j].k[q], af[i].k[q]);
        } else {
          mfma_32x32x16_bf16<false>(acc[i][j], wf[j].k[q], af[i].k[q]);
        }
      };
      // The weights of this step were read from LDS during the previous step, which has
      // also converted the operands the schedule puts there; step 0 of a tile converts
      // those itself.
      if constexpr (FIRST) {
#pragma unroll
        for (int t = -C::S2; t < 0; ++t) conversions_at(t);
      }
      conversions_at(C::kConvTop);
      __builtin_amdgcn_sched_barrier(0);
      // first half: rows 0..H-1, MFMA step q of all their blocks before step q+1
      // (schedule: CfgWW::slot1 ...)
#pragma unroll
      for (int sl = 0; sl < C::S1; ++sl) {
        const int i = C::i_of_slot1(sl), q = C::q_of_slot1(sl), j = sl % TN;
        conversions_at(sl);
#pragma unroll
        for (int t = 0; t < C::T1; ++t) {
          if (C::slot1(t) != sl) continue;
          if (C::is_read1(t)) {
            const int r = C::read1_index(t);
            af[C::read1_row(r)].k[C::read1_step(r)] = read_a1(st, C::read1_row(r), C::read1_step(r));
          } else {
            dma_a(kd, a_prev, C::dma1_index(t));
          }
        }
        mfma(i, j, q);
        __builtin_amdgcn_sched_barrier(0);
      }
      // own LDS reads of this step done, own DMA of the next step landed (the steps
      // after it and the A panel issued above may still fly); then everyone's. In the
      // first D-1 steps of a later tile that DMA was waited for before the previous
      // epilogue's stores.
      if ((FIRST || D > 2) && kt <= D - 2 && tile != (int)blockIdx.x) {
        wait_and_barrier<63>();
      } else {
        wait_and_barrier<(D - 2) * C::ND + C::NDA>();
      }
      // second half: rows H..TM-1 in the same order; the next step's raw weights and A_0
      // are read, its first operands converted (in the last step of a tile: of no use,
      // step 0 of the next tile reads and converts its own) and the B panel D steps ahead
      // goes into the B stage of this step (schedule: CfgWW::slot_w ...)
#pragma unroll
      for (int sl = 0; sl < C::S2; ++sl) {
        const int q = sl / (C::R * TN), i = H + sl / TN % C::R, j = sl % TN;
#pragma unroll
        for (int qq = 0; qq < 4; ++qq)
          if (C::slot_a0(qq) == sl) af[0].k[qq] = read_a1(smem + a_next, 0, qq);
#pragma unroll
        for (int jj = 0; jj < TN; ++jj)
#pragma unroll
          for (int t = 0; t < 2; ++t)
            if (C::slot_w(jj, t) == sl) wr[jj].t[t] = read_w1(smem + b_next, jj, t);
#pragma unroll
        for (int p = 0; p < C::NDB; ++p)
          if (C::slot_dma2(p) == sl) dma_b(kd, b_cur, p);
        conversions_at(sl - C::S2);
        if (sl == C::S2 - 1) {
          // the stages move on in front of the last MFMA, not behind it
          a_prev = a_cur;
          a_cur = a_next;
          a_next = a_next + C::A_BYTES == C::A_STAGES * C::A_BYTES ? 0 : a_next + C::A_BYTES;
          b_cur = b_next;
          b_next = b_next + C::B_BYTES == C::B_BASE + C::B_STAGES * C::B_BYTES
                       ? C::B_BASE
                       : b_next + C::B_BYTES;
        }
        mfma(i, j, q);
        __builtin_amdgcn_sched_barrier(0);
      }
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

    // ---- epilogue: acc[i][j][r] is out[m][n] with
    //   m = m0 + wm*WM + 32i + (lane&31),  n = n0 + wn*WN + 32j + 16h + r
    const int nw = n0 + wn * C::WN + 16 * h;
    const int mw = m0 + wm * C::WM + r32;
    // epilogue operands of all column blocks (the fragment registers are free now):
    // staged in LDS two steps ago, read after the wait below
    v4f bs[TN][4];
    uint4 bi[TN][2];
    // every DMA issued so far (the next tile's first D steps) must have landed
    // before the stores go out: step 0 of the next tile then waits for nothing
    wait_vm<0>();
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int c = wn * C::WN + 16 * h + 32 * j;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        bs[j][q] = *reinterpret_cast<const v4f*>(smem + C::EPI_BS + (c + 4 * q) * 4);
      bi[j][0] = *reinterpret_cast<const uint4*>(smem + C::EPI_BI + c * 2);
      bi[j][1] = *reinterpret_cast<const uint4*>(smem + C::EPI_BI + c * 2 + 16);
    }
    // Accumulators are read with inline assembly, one block at a time (left to itself
    // the compiler copies all of them to VGPRs first and spills what else is live);
    // the GELU decision is taken once per tile, not once per element.
    // Stores: the memory pipeline merges the lanes of a store into one request only
    // when adjacent lanes write adjacent bytes; with lane = 32 h + r32 holding 32 bytes
    // of row r32 every lane is a request of its own, which costs four times the issue
    // time. So the packed words of a block are rearranged first: v_permlane16_swap
    // leaves lane r32 < 16 with the first 16 bytes of rows r32 and r32 + 16 and lane
    // r32 + 16 with their second 16 bytes, then ds_bpermute_b32 (the LDS crossbar, no
    // LDS memory) hands lane L the piece L & 3 of row L >> 2: two stores of 16 rows x
    // 64 contiguous bytes, lanes 4r .. 4r+3 on row r. They are issued while the next
    // block is computed, the last block's after the two copies of the epilogue join.
    const int bp_addr = 4 * (16 * (lane & 3) + (lane >> 2));
    // Buffer stores: the descriptor of a block covers the rows of it that exist (the
    // hardware drops lanes beyond), lanes whose columns do not exist get an offset
    // beyond any descriptor -- no bounds branches, no 64-bit address arithmetic per store.
    constexpr uint32_t kNoColumn = 0x80000000u;
    uint16_t* cur_out = g.out;
    int64_t cur_ldo = g.ldo;
    int cur_epilogue = g.epilogue;
    if constexpr (GROUPED) {
      cur_out = grp.out[cur];
      cur_ldo = grp.ldo[cur];
      cur_epilogue = grp.epilogue[cur];
    }
    const int cur_N = n_of(cur);
    uint8_t* const out_wave = reinterpret_cast<uint8_t*>(cur_out) +
                              ((int64_t)(m0 + wm * C::WM) * cur_ldo + (n0 + wn * C::WN)) * 2;
    const int rows_wave = m_of(cur_act) - (m0 + wm * C::WM);
    const uint32_t out_lane = ((uint32_t)(lane >> 2) * (uint32_t)cur_ldo + 8u * (lane & 3)) * 2;
    const uint32_t half_block = 16u * (uint32_t)cur_ldo * 2;
    uint32_t out_off[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
      out_off[j] = n0 + wn * C::WN + 32 * j + 8 * (lane & 3) < cur_N ? out_lane + 64 * j : kNoColumn;
    uint32_t moved[8];
    auto store_moved = [&](int i, int j) {
      const int rows = __builtin_amdgcn_readfirstlane(min(max(rows_wave - 32 * i, 0), 32));
      const __amdgpu_buffer_rsrc_t block = __builtin_amdgcn_make_buffer_rsrc(
          out_wave + (int64_t)(32 * i) * cur_ldo * 2, 0, rows * cur_ldo * 2, 0x00020000);
      __builtin_amdgcn_raw_buffer_store_b128(v4u{moved[0], moved[1], moved[2], moved[3]}, block,
                                             (int)out_off[j], 0, 2);
      __builtin_amdgcn_raw_buffer_store_b128(v4u{moved[4], moved[5], moved[6], moved[7]}, block,
                                             (int)(out_off[j] + half_block), 0, 2);
    };
    auto epilogue = [&](auto gelu_tag) {
      constexpr bool GELU = decltype(gelu_tag)::value;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const uint32_t bw[8] = {bi[j][0].x, bi[j][0].y, bi[j][0].z, bi[j][0].w,
                                bi[j][1].x, bi[j][1].y, bi[j][1].z, bi[j][1].w};
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          uint32_t pk[8];
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            const float b0 = __uint_as_float(bw[r >> 1] << 16);
            const float b1 = __uint_as_float(bw[r >> 1] & 0xffff0000u);
            float a0, a1;
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(a0) : "a"(acc[i][j][r]));
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(a1) : "a"(acc[i][j][r + 1]));
            float v0 = __fmaf_rn(a0, bs[j][r >> 2][r & 3], b0);
            float v1 = __fmaf_rn(a1, bs[j][r >> 2][(r + 1) & 3], b1);
            if constexpr (GELU) {
              v0 = gelu_tanh(v0);
              v1 = gelu_tanh(v1);
            }
            pk[r >> 1] = pack_bf16x2(v0, v1);
          }
          // the previous block's words have had this block's arithmetic to arrive
          __builtin_amdgcn_sched_barrier(0);
          if (i > 0) {
            store_moved(i - 1, j);
          } else if (j > 0) {
            store_moved(TM - 1, j - 1);
          }
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const auto sw = __builtin_amdgcn_permlane16_swap(pk[k], pk[4 + k], false, false);
            moved[k] = (uint32_t)__builtin_amdgcn_ds_bpermute(bp_addr, (int)sw[0]);
            moved[4 + k] = (uint32_t)__builtin_amdgcn_ds_bpermute(bp_addr, (int)sw[1]);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    };
    if (cur_epilogue & CDIT_EPI_GELU_TANH) {
      epilogue(std::true_type{});
    } else {
      epilogue(std::false_type{});
    }
    store_moved(TM - 1, TN - 1);
    if (next_tile >= ntiles) break;
    m0 = nm0;
    n0 = nn0;
    cur = next_member;
    cur_act = next_act;
  }
  // the zero-record DMA of the last D steps must not outlive the workgroup
  wait_vm<0>();
}

template <class C>
int launch_wide(const GemmArgs& g, hipStream_t stream) {
  static bool lds_allowed[64];
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_w8a16_wide<C>), C::LDS_BYTES,
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
  hipLaunchKernelGGL(gemm_w8a16_wide<C>, dim3(ntiles < cus ? ntiles : cus), dim3(C::THREADS),
                     C::LDS_BYTES, stream, g, tiles_m, tiles_n, NoGroup{});
  return 0;
}

// A GemmGroup as one launch: the launcher fills the tile tables of the group for this tile
// shape (grp is a copy).
template <class C>
int launch_wide_grouped(const GemmArgs& g, GemmGroup grp, hipStream_t stream) {
  static bool lds_allowed[64];
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_w8a16_wide<C, true>),
                                 C::LDS_BYTES, lds_allowed))
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
  hipLaunchKernelGGL((gemm_w8a16_wide<C, true>), dim3(ntiles < cus ? ntiles : cus), dim3(C::THREADS),
                     C::LDS_BYTES, stream, g, 0, 0, grp);
  return 0;
}

// ---------------------------------------------------------------------------
// Skinny kernel for M <= 16 (M = 1 modulation Linears): weight streaming. A
// workgroup of 4 waves owns 16 output channels, each wave a quarter of K. Per
// 128-element chunk a lane (weight row l&15, K group l>>4) loads 32 e4m3 bytes
// straight from HBM and the matching 32 bf16 activations (zero for rows >= M),
// converts the weights to bf16 and issues four v_mfma_f32_16x16x32_bf16; the four
// partial tiles are summed through LDS.
__global__ __launch_bounds__(256) void gemm_w8a16_skinny(GemmArgs g) {
  __shared__ float part[4][16][17];
  typedef float v4f_ __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, kg = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int nrow = min(n0 + r, g.N - 1);
  const int KT = g.K / 128;
  const int per = (KT + 3) / 4;
  const int k_begin = wave * per, k_end = min(KT, k_begin + per);
  const uint8_t* __restrict__ wp = g.b + (int64_t)nrow * g.ldb + kg * 32;
  const uint16_t* __restrict__ ap =
      static_cast<const uint16_t*>(g.a) + (int64_t)min(r, g.M - 1) * g.lda + kg * 32;
  const bool a_valid = r < g.M;
  v4f_ acc = {0.0f, 0.0f, 0.0f, 0.0f};
  constexpr int U = 3;  // chunks in flight
  for (int k0 = k_begin; k0 < k_end; k0 += U) {
    uint4 w[U][2];
    v8bf a[U][4];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kt = min(k0 + u, k_end - 1);
      const uint4* wq = reinterpret_cast<const uint4*>(wp + (int64_t)kt * 128);
      w[u][0] = wq[0];
      w[u][1] = wq[1];
      const v8bf* aq = reinterpret_cast<const v8bf*>(ap + (int64_t)kt * 128);
#pragma unroll
      for (int t = 0; t < 4; ++t) a[u][t] = aq[t];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (k0 + u < k_end) {
        const uint32_t words[8] = {w[u][0].x, w[u][0].y, w[u][0].z, w[u][0].w,
                                   w[u][1].x, w[u][1].y, w[u][1].z, w[u][1].w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const v2bf c0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(words[2 * t], 1.0f, false);
          const v2bf c1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(words[2 * t], 1.0f, true);
          const v2bf c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(words[2 * t + 1], 1.0f, false);
          const v2bf c3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(words[2 * t + 1], 1.0f, true);
          const v8bf wf = {c0[0], c0[1], c1[0], c1[1], c2[0], c2[1], c3[0], c3[1]};
          v8bf af = a[u][t];
          if (!a_valid) af = v8bf{0, 0, 0, 0, 0, 0, 0, 0};
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, af, acc, 0, 0, 0);
        }
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
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float sum = (part[0][m][nl + e] + part[1][m][nl + e]) +
                          (part[2][m][nl + e] + part[3][m][nl + e]);
        const int n = n0 + nl + e;
        float t = sum * g.b_scale[n];
        if (g.bias) t += __uint_as_float((uint32_t)g.bias[n] << 16);
        if (g.epilogue & CDIT_EPI_GELU_TANH) t = gelu_tanh(t);
        v[e] = t;
      }
      uint2 pk;
      pk.x = pack_bf16x2(v[0], v[1]);
      pk.y = pack_bf16x2(v[2], v[3]);
      *reinterpret_cast<uint2*>(g.out + (int64_t)m * g.ldo + n0 + nl) = pk;
    }
  }
}

// One activation row (M = 1: the modulation Linears), K <= 4096, with the access pattern of
// the w8a8 path's linear_fp8_row1: a load instruction of the wavefront reads 1 KiB of one
// weight row (lane l bytes 16 l .. 16 l + 15) where the 16-row arrangement above makes every
// lane a memory request of its own; the MFMA's 16 "rows" are 16 interleaved K subsets of that
// row, the activation is fetched at the same positions lane for lane (32 bytes of bf16 per
// 16 weight bytes), D[i][i] is the partial dot product over subset i and the diagonal sums
// to the whole one. A wavefront owns three whole rows, all of their loads in flight at once.
constexpr int kRow1Rows = 3, kRow1Waves = 4;
template <int CHK>
__global__ __launch_bounds__(64 * kRow1Waves) void gemm_w8a16_row1(GemmArgs g) {
  constexpr int R = kRow1Rows;
  typedef float v4f_ __attribute__((ext_vector_type(4)));
  typedef unsigned int u4v __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int row0 = (blockIdx.x * kRow1Waves + wave) * R;
  const u4v zero4 = {0u, 0u, 0u, 0u};
  u4v w[R][CHK];
#pragma unroll
  for (int q = 0; q < R; ++q) {
    const uint8_t* __restrict__ wp = g.b + (int64_t)min(row0 + q, g.N - 1) * g.ldb + lane * 16;
#pragma unroll
    for (int c = 0; c < CHK; ++c) {
      if (c * 1024 + lane * 16 < g.K) {
        w[q][c] = __builtin_nontemporal_load(reinterpret_cast<const u4v*>(wp + c * 1024));
      } else {
        w[q][c] = zero4;
      }
    }
  }
  const uint16_t* __restrict__ ap = static_cast<const uint16_t*>(g.a) + lane * 16;
  const v8bf zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  v8bf xa[CHK][2];
#pragma unroll
  for (int c = 0; c < CHK; ++c) {
    const bool in = c * 1024 + lane * 16 < g.K;
    const v8bf* src = reinterpret_cast<const v8bf*>(ap + c * 1024);
    xa[c][0] = in ? src[0] : zero8;
    xa[c][1] = in ? src[1] : zero8;
  }
  // lane l holds D[4 (l >> 4) + e][l & 15]: the diagonal entry of lanes 0-3, 20-23, 40-43, 60-63
  const int diag = (lane & 15) - 4 * (lane >> 4);
  float mine = 0.0f;  // lane q keeps the dot product of row row0 + q
#pragma unroll
  for (int q = 0; q < R; ++q) {
    v4f_ acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int c = 0; c < CHK; ++c) {
      const uint32_t words[4] = {w[q][c][0], w[q][c][1], w[q][c][2], w[q][c][3]};
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const v2bf c0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(words[2 * t], 1.0f, false);
        const v2bf c1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(words[2 * t], 1.0f, true);
        const v2bf c2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(words[2 * t + 1], 1.0f, false);
        const v2bf c3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(words[2 * t + 1], 1.0f, true);
        const v8bf wf = {c0[0], c0[1], c1[0], c1[1], c2[0], c2[1], c3[0], c3[1]};
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xa[c][t], acc, 0, 0, 0);
      }
    }
    float d = 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) d = diag == e ? acc[e] : d;
    const float sum = wave_sum_f32(d);
    mine = lane == q ? sum : mine;
  }
  const int n = row0 + lane;
  if (lane < R && n < g.N) {
    float t = mine * g.b_scale[n];
    if (g.bias) t += __uint_as_float((uint32_t)g.bias[n] << 16);
    if (g.epilogue & CDIT_EPI_GELU_TANH) t = gelu_tanh(t);
    g.out[n] = (uint16_t)(pack_bf16x2(t, 0.0f) & 0xffffu);
  }
}

// Any shape: one output element per thread, scalar decode + FMA.
__global__ __launch_bounds__(256) void gemm_w8a16_generic(GemmArgs g) {
  const int n = blockIdx.x * 16 + (threadIdx.x & 15);
  const int m = blockIdx.y * 16 + (threadIdx.x >> 4);
  if (m >= g.M || n >= g.N) return;
  const uint16_t* a = static_cast<const uint16_t*>(g.a) + (int64_t)m * g.lda;
  const uint8_t* b = g.b + (int64_t)n * g.ldb;
  float acc = 0.0f;
  for (int k = 0; k < g.K; ++k) {
    const float x = __uint_as_float((uint32_t)a[k] << 16);
    const float w = __builtin_amdgcn_cvt_f32_fp8((int)b[k], 0);
    acc = fmaf(x, w, acc);
  }
  float v = acc * g.b_scale[n];
  if (g.bias) v += __uint_as_float((uint32_t)g.bias[n] << 16);
  if (g.epilogue & CDIT_EPI_GELU_TANH) v = gelu_tanh(v);
  g.out[(int64_t)m * g.ldo + n] = (uint16_t)f32_to_bf16_bits(v);
}

template <class C>
int launch_tiled(const GemmArgs& g, hipStream_t stream) {
  static bool lds_allowed[64];
  if (int rc = allow_dynamic_lds(reinterpret_cast<const void*>(&gemm_w8a16_tiled<C>), C::LDS_BYTES,
                                 lds_allowed))
    return rc;
  const int tiles_m = (g.M + C::BM - 1) / C::BM, tiles_n = (g.N + C::BN - 1) / C::BN;
  hipLaunchKernelGGL(gemm_w8a16_tiled<C>, dim3(tiles_m * tiles_n), dim3(C::THREADS), C::LDS_BYTES,
                     stream, g, tiles_m, tiles_n);
  return 0;
}

bool tiled_ok(const GemmArgs& g) {
  return g.K >= BKE && g.K % BKE == 0 && g.N % 8 == 0 && g.lda % 8 == 0 && g.ldb % 16 == 0 &&
         g.ldo % 8 == 0 && reinterpret_cast<uintptr_t>(g.a) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(g.b) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(g.out) % 16 == 0 &&
         // the epilogues load scales as float4 and bias as 8-byte packs
         reinterpret_cast<uintptr_t>(g.b_scale) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(g.bias) % 16 == 0 &&
         (int64_t)1024 * g.lda < (int64_t)1 << 31 && (int64_t)512 * g.ldb < (int64_t)1 << 31 &&
         (int64_t)512 * g.ldo < (int64_t)1 << 29;  // 32-bit byte offsets within a block of rows
}

}  // namespace

typedef CfgW<256, 256, 2, 2, true, 8> W0;   // 4 waves, 2 stages
typedef CfgW<128, 128, 2, 2, true, 8> W3;   // small tiles, two workgroups per CU
typedef CfgWW<256, 256, 4> W7;              // wide: 4 waves, 128x128 wave tiles
typedef CfgWW<256, 192, 4> W8;              // wide: 128x96 wave tiles
typedef CfgWW<192, 256, 4> W9;              // wide: 96x128 wave tiles
typedef CfgWW<128, 192, 4, 4> W10;          // wide: 64x96 wave tiles, DMA 4 steps ahead
typedef CfgWW<128, 128, 4, 5> W11;          // wide: 64x64 wave tiles, DMA 5 steps ahead
typedef CfgWW<128, 64, 4, 6> W12;           // wide: 64x32 wave tiles, DMA 6 steps ahead

namespace {
struct TileChoice {
  int variant;
  int64_t cost;  // 1000 x CUs x tile area per full round over the CUs (K left out)
};

// Tile choice for a problem whose tile count for a bm x bn tile is tiles(bm, bn) (one GEMM,
// or a batch walked as one tile stream). Same cost model as the w8a8 entry point: tile area
// times rounds over the CUs (one persistent workgroup each), a last partial round of r tiles
// counting 0.4 + 0.6 r/CUs; both branches count in the same unit.
template <class Tiles, class WideOk>
TileChoice choose_variant(Tiles tiles, WideOk wide_ok) {
  const int64_t cus = cu_count() > 0 ? cu_count() : 256;
  if (tiles(256, 256) * 256 >= 160 * cus && wide_ok(2)) {
    auto cost = [&](int bm, int bn, int pen) {
      const int64_t t = tiles(bm, bn), full = t / cus, rem = t % cus;
      return (full * 10 * cus + (rem ? 4 * cus + 6 * rem : 0)) * bm * bn * pen;
    };
    // (256 x 192 against 256 x 256, measured: 0.98 at 4608 x 3072 x 12288, 0.955 at N = 15360,
    // 1.03 at 4096 x 3072 x 12288, 1.05 at N = 9216; a penalty of 2 % puts all four on the right side)
    const int64_t c8 = cost(256, 192, 102), c7 = cost(256, 256, 100);
    return c8 < c7 ? TileChoice{8, c8} : TileChoice{7, c7};
  }
  // Smaller problems: whole rounds over the CUs times tile area, the small tiles
  // penalised by their measured lower MFMA rate (per mille); ties go to the larger
  // tile. Tiles whose prefetch depth K cannot feed are left out; without any wide
  // tile (N not a multiple of 16, very short K) the 128x128 kernel runs.
  const struct { int v, bm, bn, pen, depth; } cand[] = {
      {7, 256, 256, 1000, 2}, {8, 256, 192, 1000, 2}, {10, 128, 192, 1300, 4},
      {11, 128, 128, 1400, 5}, {12, 128, 64, 1700, 6}};
  TileChoice best = {3, INT64_MAX / 8};  // the 128x128 kernel takes what no wide tile can
  for (const auto& c : cand) {
    if (!wide_ok(c.depth)) continue;
    const int64_t t = (tiles(c.bm, c.bn) + cus - 1) / cus * cus * c.bm * c.bn * c.pen;
    if (t < best.cost) best = {c.v, t};
  }
  return best;
}
}  // namespace

int launch_gemm_w8a16(const GemmArgs& g, int variant, hipStream_t stream) {
  if (!tiled_ok(g) || variant == 100) {
    dim3 grid((g.N + 15) / 16, (g.M + 15) / 16);
    hipLaunchKernelGGL(gemm_w8a16_generic, grid, dim3(256), 0, stream, g);
    return 0;
  }
  if ((variant < 0 || variant == 51) && g.M == 1 && g.K % 128 == 0 && g.K <= 4096) {
    // (tiled_ok has checked the alignment of the operands and of ldb)
    constexpr int rows_wg = kRow1Rows * kRow1Waves;
    const dim3 grid((g.N + rows_wg - 1) / rows_wg), block(64 * kRow1Waves);
    switch ((g.K + 1023) / 1024) {
      case 1: hipLaunchKernelGGL(gemm_w8a16_row1<1>, grid, block, 0, stream, g); break;
      case 2: hipLaunchKernelGGL(gemm_w8a16_row1<2>, grid, block, 0, stream, g); break;
      case 3: hipLaunchKernelGGL(gemm_w8a16_row1<3>, grid, block, 0, stream, g); break;
      default: hipLaunchKernelGGL(gemm_w8a16_row1<4>, grid, block, 0, stream, g); break;
    }
    return 0;
  }
  if ((variant < 0 && g.M <= 16 && g.K % 128 == 0) || variant == 50) {
    if (g.M > 16 || g.K % 128 != 0) {
      set_error("cdit_w8a16_gemm: the skinny kernel takes M <= 16 and K %% 128 == 0");
      return CDIT_EINVAL;
    }
    hipLaunchKernelGGL(gemm_w8a16_skinny, dim3((g.N + 15) / 16), dim3(256), 0, stream, g);
    return 0;
  }
  // the wide kernels stream K two or more steps ahead and store 16 columns per lane
  // at least `depth` K steps to prefetch, and at least 3: the epilogue operands of a tile are
  // staged in LDS two steps before its end, which must be behind the first barrier of the
  // tile (before it, slower waves may still be reading the previous tile's)
  auto wide_ok = [&](int depth) { return g.K >= (depth > 3 ? depth : 3) * BKE && g.N % 16 == 0; };
  if (variant < 0) {
    variant = choose_variant(
        [&](int bm, int bn) { return (int64_t)((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn); },
        wide_ok).variant;
  }
  switch (variant) {
    case 0: return launch_tiled<W0>(g, stream);
    case 3: return launch_tiled<W3>(g, stream);
    case 7: return wide_ok(W7::DEPTH) ? launch_wide<W7>(g, stream) : launch_tiled<W3>(g, stream);
    case 8: return wide_ok(W8::DEPTH) ? launch_wide<W8>(g, stream) : launch_tiled<W3>(g, stream);
    case 9: return wide_ok(W9::DEPTH) ? launch_wide<W9>(g, stream) : launch_tiled<W3>(g, stream);
    case 10: return wide_ok(W10::DEPTH) ? launch_wide<W10>(g, stream) : launch_tiled<W3>(g, stream);
    case 11: return wide_ok(W11::DEPTH) ? launch_wide<W11>(g, stream) : launch_tiled<W3>(g, stream);
    case 12: return wide_ok(W12::DEPTH) ? launch_wide<W12>(g, stream) : launch_tiled<W3>(g, stream);
    default:
      set_error("cdit_w8a16_gemm: unknown kernel variant %d", variant);
      return CDIT_EINVAL;
  }
}

// The batch as one launch (or, where the cost model says so, one launch per activation).
// Returns 0 when launched, -1 when the batch is not taken (the caller then runs the members
// one by one), a CDIT_E* code on error.
int launch_gemm_w8a16_grouped(const GemmArgs& common, const GemmGroup& grp, int variant,
                              hipStream_t stream) {
  if (grp.count < 2 || grp.count > kMaxGroup || grp.acts < 1 || grp.acts > kMaxActs ||
      common.out_dtype != CDIT_DT_BF16)
    return -1;
  bool n16 = true;
  for (int s = 0; s < grp.acts; ++s) {
    if (grp.M[s] <= 16 || grp.first_member[s + 1] <= grp.first_member[s]) return -1;
    for (int p = grp.first_member[s]; p < grp.first_member[s + 1]; ++p) {
      GemmArgs g = common;
      g.a = grp.a[s];
      g.M = grp.M[s];
      g.b = grp.b[p];
      g.b_scale = grp.b_scale[p];
      g.bias = grp.bias[p];
      g.out = grp.out[p];
      g.N = grp.N[p];
      g.ldo = grp.ldo[p];
      if (!tiled_ok(g) || g.N <= 0) return -1;
      n16 = n16 && g.N % 16 == 0;
    }
  }
  auto wide_ok = [&](int depth) { return common.K >= (depth > 3 ? depth : 3) * BKE && n16; };
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
    const TileChoice whole = choose_variant(tiles, wide_ok);
    variant = whole.variant;
    if (grp.acts > 1) {
      // one tile stream against one launch per activation, as in the w8a8 launcher: a small
      // activation can push a batch that filled whole rounds into one more, nearly empty one
      // (a further launch costs about 3 us; a CU does about 2450 K elements of one output
      // element per us at the bf16 rate)
      const int64_t cus = cu_count() > 0 ? cu_count() : 256;
      int64_t apart = (grp.acts - 1) * (3 * 1000 * cus * 2450 / (common.K > 0 ? common.K : 1));
      for (int s = 0; s < grp.acts; ++s) {
        auto tiles_s = [&](int bm, int bn) {
          int64_t cols = 0;
          for (int p = grp.first_member[s]; p < grp.first_member[s + 1]; ++p) cols += (grp.N[p] + bn - 1) / bn;
          return (int64_t)((grp.M[s] + bm - 1) / bm) * cols;
        };
        apart += choose_variant(tiles_s, wide_ok).cost;
      }
      if (apart * 100 < whole.cost * 97) {
        for (int s = 0; s < grp.acts; ++s) {
          GemmGroup one = {};
          one.acts = 1;
          one.count = grp.first_member[s + 1] - grp.first_member[s];
          one.a[0] = grp.a[s];
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
          int rc = one.count >= 2 ? launch_gemm_w8a16_grouped(common, one, -1, stream) : -1;
          if (rc > 0) return rc;
          if (rc == 0) continue;
          for (int p = 0; p < one.count; ++p) {  // a single member, or a group that is not taken
            GemmArgs g = common;
            g.a = one.a[0];
            g.M = one.M[0];
            g.b = one.b[p];
            g.b_scale = one.b_scale[p];
            g.bias = one.bias[p];
            g.out = one.out[p];
            g.N = one.N[p];
            g.ldo = one.ldo[p];
            g.epilogue = one.epilogue[p];
            if ((rc = launch_gemm_w8a16(g, -1, stream))) return rc;
          }
        }
        return 0;
      }
    }
  }
  switch (variant) {
    case 7: return wide_ok(W7::DEPTH) ? launch_wide_grouped<W7>(common, grp, stream) : -1;
    case 8: return wide_ok(W8::DEPTH) ? launch_wide_grouped<W8>(common, grp, stream) : -1;
    case 9: return wide_ok(W9::DEPTH) ? launch_wide_grouped<W9>(common, grp, stream) : -1;
    case 10: return wide_ok(W10::DEPTH) ? launch_wide_grouped<W10>(common, grp, stream) : -1;
    case 11: return wide_ok(W11::DEPTH) ? launch_wide_grouped<W11>(common, grp, stream) : -1;
    case 12: return wide_ok(W12::DEPTH) ? launch_wide_grouped<W12>(common, grp, stream) : -1;
    default: return -1;  // the kernels without a tile stream have no grouped form
  }
}

}  // namespace cdit
