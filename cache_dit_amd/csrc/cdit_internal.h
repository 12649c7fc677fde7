// Internal declarations shared by the kernel files and the C-ABI layer.
#ifndef CDIT_INTERNAL_H_
#define CDIT_INTERNAL_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "cdit_hip.h"

namespace cdit {

// Each launcher validates nothing: capi.hip checks shapes, strides, alignment
// and the device before calling. They return 0 or a CDIT_E* code.
int launch_quant_rowwise(const void* x, int64_t M, int64_t K, int64_t ld_x, void* q,
                         int64_t ld_q, float* scale, int scale_mode, bool consumer_follows,
                         hipStream_t stream);

// Up to kMaxQuantActs activations of one K quantized row-wise in one launch (the image- and
// text-stream inputs of one stage of a double-stream block): global row r belongs to
// activation s with row_begin[s] <= r < row_begin[s + 1].
constexpr int kMaxQuantActs = 4;
struct QuantBatch {
  int acts;
  int row_begin[kMaxQuantActs + 1];
  const uint16_t* x[kMaxQuantActs];
  int64_t ld_x[kMaxQuantActs];
  uint8_t* q[kMaxQuantActs];
  int64_t ld_q[kMaxQuantActs];
  float* scale[kMaxQuantActs];
};
// 0: launched; 1: not taken (alignment, K beyond the register-resident kernel): the caller
// launches the activations one by one.
int launch_quant_rowwise_batched(const QuantBatch& batch, int64_t K, int scale_mode,
                                 hipStream_t stream);
// Rows that are the concatenation [x1 | x2] of two sources quantized as one row. 0: launched;
// 1: not taken (alignment, K1 + K2 beyond the register-resident kernel).
int launch_quant_rowwise_cat2(const void* x1, int64_t K1, int64_t ld_x1, const void* x2, int64_t K2,
                              int64_t ld_x2, int64_t M, void* q, int64_t ld_q, float* scale,
                              int scale_mode, hipStream_t stream);

int launch_quant_tensorwise(const void* x, int64_t M, int64_t K, int64_t ld_x, void* q,
                            int64_t ld_q, float* scale, uint32_t* amax_ws, int scale_mode,
                            hipStream_t stream);

// LayerNorm (no affine) + `* (1 + scale) + shift` + per-row quantization in one pass; y may be
// null (then only codes and scales are written).
int launch_ln_modulate_quant(const void* x, int64_t M, int64_t K, int64_t ld_x, const void* shift,
                             const void* scale_mod, int64_t ld_mod, int64_t rows_per_mod, float eps,
                             void* y, int64_t ld_y, void* q, int64_t ld_q, float* scale,
                             int scale_mode, hipStream_t stream);

extern int g_quant_variant;

struct GemmArgs {
  const void* a;         // fp8 [M,K] (w8a8) or bf16 [M,K] (w8a16)
  const float* a_scale;  // [M] (w8a8) or nullptr (w8a16)
  const uint8_t* b;      // fp8 [N,K]
  const float* b_scale;  // [N]
  const uint16_t* bias;  // [N] in the output's dtype (fp16 or bf16) or nullptr; fp32 output: nullptr
  uint16_t* out;         // [M,N] of out_dtype (fp32 output: really a float*, ldo in elements)
  int M, N, K;
  int64_t lda, ldb, ldo;
  int epilogue;
  int out_dtype = CDIT_DT_BF16;  // CDIT_DT_*; the w8a16 kernels only build bf16
};

// A batch of GEMMs run as one launch of the wide kernel. The batch holds up to kMaxActs
// activations (A operands: codes, per-row scales, M); each activation has one or more
// members (B side: weight, per-channel scale, bias, output, epilogue flag), up to kMaxGroup
// members in all. K, lda and ldb are common. Members of one activation are walked as if their
// weights were stacked along N (tile columns [col_begin[p], col_begin[p + 1]) of that
// activation), activations one after the other. The fields marked (launcher) are filled by
// launch_gemm_fp8_grouped for the tile shape it picks.
constexpr int kMaxGroup = 8;
constexpr int kMaxActs = 4;
struct GemmGroup {
  int count;  // members
  int acts;   // activations
  // per activation
  const void* a[kMaxActs];
  const float* a_scale[kMaxActs];
  int M[kMaxActs];
  int first_member[kMaxActs + 1];  // members of activation s: [first_member[s], first_member[s + 1])
  int tile_begin[kMaxActs + 1];    // (launcher) first linear tile id of activation s
  int tiles_m[kMaxActs];           // (launcher) tile rows of activation s
  int tiles_n[kMaxActs];           // (launcher) tile columns of activation s, all its members
  // per member
  int col_begin[kMaxGroup + 1];    // (launcher) first tile column of member p inside its activation
  const uint8_t* b[kMaxGroup];
  const float* b_scale[kMaxGroup];
  const uint16_t* bias[kMaxGroup];
  uint16_t* out[kMaxGroup];
  int N[kMaxGroup];
  int64_t ldo[kMaxGroup];
  int epilogue[kMaxGroup];
};

// variant < 0: choose by shape.
int launch_gemm_fp8(const GemmArgs& g, int variant, hipStream_t stream);
// the 288 x 192 kernel with per-workgroup time stamps (measurement only; gemm_fp8.hip)
int launch_gemm_fp8_stamps(const GemmArgs& g, unsigned long long* stamps, int* workgroups,
                           hipStream_t stream);
// All members of `grp` in one launch (K, lda, ldb and the output dtype from `common`; its other
// fields are ignored). 0: launched; -1: not taken (shape, alignment or variant without a
// grouped form); else a CDIT_E* code.
int launch_gemm_fp8_grouped(const GemmArgs& common, const GemmGroup& grp, int variant,
                            hipStream_t stream);
int launch_gemm_w8a16(const GemmArgs& g, int variant, hipStream_t stream);
// The same for the weight-only GEMM (grp.a: bf16 activations; grp.a_scale unused).
int launch_gemm_w8a16_grouped(const GemmArgs& common, const GemmGroup& grp, int variant,
                              hipStream_t stream);
// One w8a8 Linear forward at M <= 16 in a single kernel (per-token quantizer + GEMM);
// g.a is the bf16 activation, g.lda its leading dimension in elements. Returns 0 when
// launched, 1 when the shape or alignment is not taken (the caller then runs the
// quantizer and the GEMM one after the other).
int launch_linear_fp8_skinny_fused(const GemmArgs& g, void* q_ws, float* scale_ws, int scale_mode,
                                   int variant, hipStream_t stream);

// FP8 quantizers with the scale packed behind each row (comm_quant.hip).
int launch_comm_per_token_quant(const void* x, int64_t M, int64_t H, void* y, hipStream_t stream);
int launch_comm_per_token_dequant(const void* x, int64_t M, int64_t H, void* y, hipStream_t stream);
int launch_comm_qkv_permute_quant(const void* x, int B, int S, int P, int N, int D, int64_t sb,
                                  int64_t ss, int64_t sp, void* y, hipStream_t stream);
int launch_comm_qkv_permute_dequant(const void* qx, int S, int B, int N, int D, int64_t qs, int64_t qb,
                                    int64_t qn, void* x, hipStream_t stream);

// Measurement aid: `blocks` workgroups of four wavefronts run `iters` rounds of 16 MFMAs
// (v_mfma_f32_16x16x128_f8f6f4) on register operands; out: blocks * 256 floats. *flop gets the
// floating-point operations of the launch.
int launch_mfma_only(float* out, int blocks, int iters, bool random_operands, double* flop,
                     hipStream_t stream);

void set_error(const char* fmt, ...);

}  // namespace cdit
#endif
