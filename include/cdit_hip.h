/*
 * cdit_hip.h -- C ABI of libcdit_hip.so: MI355X (gfx950 / CDNA4) kernels for
 * the FP8 quantized-linear hot path of cache-dit's `float8_per_row`
 * (w8a8, dynamic per-token activation scales) and `float8_weight_only`
 * (w8a16) quantize modes.
 *
 * Conventions (they follow the native-op conventions of the reference's own
 * extension, csrc/kernels/svdq/torch.h:9-24 and
 * src/cache_dit/kernels/cuda/_ops_registery.py:35-59):
 *   - the caller owns every buffer; nothing here allocates or frees device
 *     memory and no pointer is retained after the call returns;
 *   - all pointers are device pointers on the current HIP device;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); work
 *     is enqueued on it and the call returns without synchronising;
 *   - every function returns 0 on success and a non-zero CDIT_E* code on
 *     failure; cdit_last_error() then returns a thread-local message;
 *   - FP8 means OCP e4m3fn (bias 7, max 448, NaN 0x7F/0xFF, no inf), the
 *     format torch.float8_e4m3fn names; bf16 buffers are raw uint16 bits;
 *   - matrices are row-major with a leading dimension in ELEMENTS.
 *
 * Only plain C types cross this boundary: a maintainer binds it with ctypes,
 * cffi, pybind or a torch extension as they prefer.
 */
#ifndef CDIT_HIP_H_
#define CDIT_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CDIT_ABI_VERSION 1

enum cdit_status {
  CDIT_OK = 0,
  CDIT_EINVAL = 1,  /* bad shape, stride, alignment, mode or null pointer */
  CDIT_EARCH = 2,   /* current device is not gfx950                       */
  CDIT_EHIP = 3     /* a HIP runtime call failed (message has the reason) */
};

/* How the per-row scale amax/448 is rounded (the reference leaves this to
 * torchao's _choose_scale_float8, call site
 * src/cache_dit/quantization/torchao/quantize_ao.py:54-70):
 *   BF16DIV: fp32 true divide, round-to-nearest-even to bf16, widen to fp32
 *            (what an un-upcast bf16 `amax / 448.0` does in eager PyTorch);
 *   FP32DIV: fp32 true divide, kept in fp32. */
enum cdit_scale_mode { CDIT_SCALE_BF16DIV = 0, CDIT_SCALE_FP32DIV = 1 };
/* May be OR-ed into the scale_mode of cdit_fp8_quant_rowwise: the codes are read by a GEMM
 * launched next on the same stream. A cache hint only (the quantizer then keeps its stores
 * cacheable, as the fused cdit_fp8_linear_w8a8 does); results do not depend on it. */
#define CDIT_QUANT_GEMM_FOLLOWS 0x100

/* Epilogue flags of the GEMM entry points (bit mask). */
enum cdit_epilogue {
  CDIT_EPI_NONE = 0,
  CDIT_EPI_GELU_TANH = 1 /* 0.5 v (1 + tanh(0.79788456 (v + 0.044715 v^3))),
                            the diffusers nn.GELU(approximate="tanh") that follows
                            proj_mlp / ff.net.0.proj (reference dataflow:
                            src/cache_dit/caching/patch_functors/functor_flux.py:48-80;
                            formula precedent csrc/kernels/svdq/gemm_utils.cuh:363-378) */
};

/* Output element type ids, the reference's numbering
 * (src/cache_dit/quantization/torchao/_scaled_mm.py:38-43). */
enum cdit_dtype_id { CDIT_DT_F16 = 0, CDIT_DT_BF16 = 1, CDIT_DT_F32 = 2 };

/* ABI version of the loaded library (== CDIT_ABI_VERSION it was built with). */
int cdit_abi_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char* cdit_last_error(void);

/* Writes the gcnArchName of the current device (e.g. "gfx950:sramecc+:xnack-")
 * into buf. Returns CDIT_OK, or CDIT_EARCH when it is not a gfx950. */
int cdit_device_arch(char* buf, int buf_len);

/*
 * Per-row (per-token / per-output-channel) dynamic FP8 quantizer.
 * Replaces torchao's _choose_scale_float8 + _quantize_affine_float8 as called
 * through Float8Tensor.from_hp(x, PerRow()) -- reference call sites
 * src/cache_dit/quantization/torchao/quantize_ao.py:54-70 (scale, with the
 * zero-scale patch :65-67) and tests/kernels/test_opaque_scaled_mm.py:68-73.
 *
 *   amax[m]  = max_k |x[m,k]|                      (bf16, exact)
 *   scale[m] = amax/448 rounded per scale_mode; 0 -> 1
 *   q[m,k]   = e4m3fn_rne(clamp(float(x[m,k]) / scale[m], -448, 448))
 *
 * x: bf16 [M,K], leading dimension ld_x; q: e4m3 bytes [M,K], leading
 * dimension ld_q; scale: fp32 [M]. The codes are those of the IEEE division.
 * M == 0 or K == 0 is a no-op that returns CDIT_OK. NaN/Inf inputs are outside
 * the bit-exact contract.
 */
int cdit_fp8_quant_rowwise(const void* x_bf16, int64_t M, int64_t K, int64_t ld_x,
                           void* q_e4m3, int64_t ld_q, float* scale,
                           int scale_mode, void* stream);

/*
 * cdit_fp8_quant_rowwise on up to 4 activations of one K in a single launch: the inputs of
 * the Linears of one stage that run as one batched GEMM (cdit_fp8_gemm_rowwise_batched), e.g.
 * the image-stream and the text-stream activation of a double-stream block (reference
 * dataflow: src/cache_dit/caching/patch_functors/functor_flux.py:48-80 patches the block
 * forwards these Linears are called from). Activation s is x_bf16[s] [M[s], K] (ld_x[s]) ->
 * q_e4m3[s] (ld_q[s]), scale[s] [M[s]]; codes and scales are those of one
 * cdit_fp8_quant_rowwise call per activation, bit for bit (activations with M[s] == 0 are
 * skipped; a batch the one-launch kernel does not take -- K not a multiple of 8, K > 16384,
 * misaligned pointers -- runs as those calls). The codes are taken to be read by a GEMM
 * launched next (CDIT_QUANT_GEMM_FOLLOWS is implied).
 */
int cdit_fp8_quant_rowwise_batched(int n_act, const void* const* x_bf16, const int64_t* M,
                                   int64_t K, const int64_t* ld_x, void* const* q_e4m3,
                                   const int64_t* ld_q, float* const* scale, int scale_mode,
                                   void* stream);

/*
 * cdit_fp8_quant_rowwise on rows that are the concatenation [x1 | x2] of two sources, without
 * the concatenated tensor: FLUX single blocks feed proj_out with
 * torch.cat([attn_output, mlp_hidden_states], dim=2) (reference dataflow
 * src/cache_dit/caching/patch_functors/functor_flux.py:68-80), which only that quantized Linear
 * reads. x1 bf16 [M,K1] (ld_x1), x2 bf16 [M,K2] (ld_x2) -> q e4m3 [M,K1+K2] (ld_q), scale [M]:
 * the codes and scales of cdit_fp8_quant_rowwise on the concatenation, bit for bit. K1 and K2
 * must be multiples of 8, K1 + K2 <= 16384, rows 16-byte aligned (CDIT_EINVAL otherwise:
 * concatenate and use cdit_fp8_quant_rowwise). The codes are taken to be read by a GEMM
 * launched next.
 */
int cdit_fp8_quant_rowwise_cat2(const void* x1_bf16, int64_t K1, int64_t ld_x1,
                                const void* x2_bf16, int64_t K2, int64_t ld_x2, int64_t M,
                                void* q_e4m3, int64_t ld_q, float* scale, int scale_mode,
                                void* stream);

/*
 * Per-tensor dynamic FP8 quantization: one scale for the whole tensor. Replaces
 * torchao's Float8Tensor.from_hp(x, PerTensor()) as selected for the
 * "float8_per_tensor" quant type and the per-tensor fallback pass,
 * src/cache_dit/quantization/torchao/quantize_ao.py:559-575 and :139-148.
 *
 *   amax     = max_{m,k} |x[m,k]|
 *   s        = amax/448 rounded per scale_mode; 0 -> 1
 *   q[m,k]   = e4m3fn_rne(clamp(float(x[m,k]) / s, -448, 448))
 *   scale[m] = s for every m (the GEMM entry point takes per-row scales)
 *
 * amax_ws: 4 bytes of device memory owned by the caller, used as scratch (the
 * bf16 bit pattern of amax is left in it). Three kernels are enqueued; nothing is
 * allocated or synchronised.
 */
int cdit_fp8_quant_tensorwise(const void* x_bf16, int64_t M, int64_t K, int64_t ld_x,
                              void* q_e4m3, int64_t ld_q, float* scale, void* amax_ws,
                              int scale_mode, void* stream);

/*
 * The per-row quantizer fused into its producer: LayerNorm without affine parameters,
 * AdaLN modulation and per-row FP8 quantization in one pass over the activation. In a DiT
 * block the modulated activation `norm(x) * (1 + scale) + shift` is read by quantized
 * Linears only (reference dataflow src/cache_dit/caching/patch_functors/functor_flux.py:48-80:
 * `self.norm(...)` feeds proj_mlp and attn.to_q/k/v), so the codes are produced where the
 * activation is. Per row m, with mod = m / rows_per_mod (one modulation vector per batch
 * element, broadcast over its tokens):
 *
 *   mean = sum_k x / K;  var = sum_k (x - mean)^2 / K;  rstd = 1 / sqrt(var + eps)   (fp32)
 *   y[m,k] = bf16(bf16(bf16((x - mean) * rstd) * bf16(1 + scale[mod,k])) + shift[mod,k])
 *   (q[m,:], out_scale[m]) = the per-row quantization of y[m,:], exactly as
 *                            cdit_fp8_quant_rowwise computes it
 *
 * Every step rounds to bf16 where the unfused sequence of bf16 tensor ops does. x bf16
 * [M,K] (ld_x); shift, scale bf16 [ceil(M / rows_per_mod), K] (ld_mod); y bf16 [M,K]
 * (ld_y) or NULL when no consumer reads the bf16 tensor; q e4m3 [M,K] (ld_q); out_scale
 * fp32 [M]. Algorithmic bytes per row: 3 K + 4 (5 K + 4 with y).
 */
int cdit_fp8_ln_modulate_quant(const void* x_bf16, int64_t M, int64_t K, int64_t ld_x,
                               const void* shift_bf16, const void* scale_bf16, int64_t ld_mod,
                               int64_t rows_per_mod, float eps, void* y_bf16, int64_t ld_y,
                               void* q_e4m3, int64_t ld_q, float* out_scale, int scale_mode,
                               void* stream);

/*
 * Row-wise scaled FP8 GEMM with fused epilogue. Replaces
 * torch._scaled_mm(a, b, scale_a, scale_b, bias, out_dtype) as called by
 * _run_float8_inference_scaled_mm, src/cache_dit/quantization/torchao/_scaled_mm.py:62-91
 * (op schema :94-98).
 *
 *   out[m,n] = epi( (sum_k a[m,k] * b[n,k]) * a_scale[m] * b_scale[n] + bias[n] )
 *
 * a_q: e4m3 [M,K] row-major (lda); b_q: e4m3 [N,K] row-major (ldb) -- the
 * quantized nn.Linear weight as stored, i.e. the reference's column-major
 * [K,N] `qweight.t()`; a_scale fp32 [M]; b_scale fp32 [N]; out [M,N] (ldo, in
 * elements) of out_dtype_id: CDIT_DT_F16, CDIT_DT_BF16 or CDIT_DT_F32, the
 * op's three out_dtype ids (_scaled_mm.py:38-59). bias [N] has the output's
 * dtype (fp16 or bf16) or is NULL; an fp32 output takes no bias: the reference
 * adds it after the matmul in that case (_scaled_mm.py:71-81) and so must the
 * caller. Accumulation is fp32. Requires K % 16 == 0 (as the reference's FP8
 * matmul does) and 16-byte aligned a_q/b_q rows. bf16 is the tuned path; the
 * other two dtypes have two tile shapes of the same kernel and a generic
 * fallback.
 */
int cdit_fp8_gemm_rowwise(const void* a_q, const float* a_scale,
                          const void* b_q, const float* b_scale,
                          const void* bias, void* out,
                          int64_t M, int64_t N, int64_t K,
                          int64_t lda, int64_t ldb, int64_t ldo,
                          int epilogue, int out_dtype_id, void* stream);

/*
 * `count` (1 to 8) row-wise scaled FP8 GEMMs that share the A operand -- the same
 * activation codes and scales, hence the same M, K and lda -- as ONE launch whose tile
 * stream runs over all their output tiles: sibling Linears that read one activation, such
 * as attn.to_q / to_k / to_v, and proj_mlp next to them in FLUX single blocks (reference
 * dataflow src/cache_dit/caching/patch_functors/functor_flux.py:60-67; each is a separate
 * torch._scaled_mm call there, _scaled_mm.py:62-91). Member p has its own weight b_q[p]
 * [N[p],K] (common ldb), b_scale[p] [N[p]], bias[p] (bf16 [N[p]] or NULL; `bias` itself may
 * be NULL), out[p] bf16 [M,N[p]] (ldo[p]) and epilogue[p] (`epilogue` may be NULL = none).
 * The arrays live on the host and are read before the call returns. Results are those of
 * `count` calls of cdit_fp8_gemm_rowwise with CDIT_DT_BF16, bit for bit; shapes the
 * grouped kernel does not take are run that way.
 */
int cdit_fp8_gemm_rowwise_grouped(const void* a_q, const float* a_scale,
                                  int64_t M, int64_t K, int64_t lda, int count,
                                  const void* const* b_q, const float* const* b_scale,
                                  const void* const* bias, void* const* out,
                                  const int64_t* N, int64_t ldb, const int64_t* ldo,
                                  const int* epilogue, void* stream);

/*
 * The general form of the call above: `n_act` (1 to 4) activations, activation s with
 * members_per_act[s] GEMMs on it; the member arrays list the members of activation 0,
 * then those of activation 1, ... (1 to 8 members in all). K, lda and ldb are common. For
 * Linears of one stage that do not depend on each other, on the same or on different
 * activations: in a FLUX double block attn.to_q/k/v on the image tokens and
 * attn.add_q/k/v_proj on the text tokens, then to_out.0 and to_add_out, ff.net.0.proj and
 * ff_context.net.0.proj, ... (dataflow src/cache_dit/caching/patch_functors/functor_flux.py:
 * 48-80 and the double-stream block it patches around); small text-stream GEMMs then ride in
 * the tile stream of the large image-stream ones instead of half filling the chip on their
 * own. Same results as one cdit_fp8_gemm_rowwise call per member, bit for bit.
 */
int cdit_fp8_gemm_rowwise_batched(int n_act, const void* const* a_q, const float* const* a_scale,
                                  const int64_t* M, int64_t K, int64_t lda,
                                  const int* members_per_act,
                                  const void* const* b_q, const float* const* b_scale,
                                  const void* const* bias, void* const* out,
                                  const int64_t* N, int64_t ldb, const int64_t* ldo,
                                  const int* epilogue, void* stream);

/*
 * Weight-only FP8 GEMM (w8a16): bf16 activations, e4m3 weights dequantized in
 * the mainloop, per-output-channel scale applied in the epilogue. Replaces
 * F.linear(x, W.dequantize(), bias) of torchao's Float8WeightOnlyConfig
 * (reference selection: src/cache_dit/quantization/torchao/quantize_ao.py:604-610).
 *
 *   out[m,n] = epi( (sum_k x[m,k] * float(b[n,k])) * b_scale[n] + bias[n] )
 *
 * x_bf16 [M,K] (lda); b_q e4m3 [N,K] (ldb); b_scale fp32 [N]; bias bf16 [N] or
 * NULL; out bf16 [M,N] (ldo). Requires K % 16 == 0.
 */
int cdit_w8a16_gemm(const void* x_bf16, const void* b_q, const float* b_scale,
                    const void* bias_bf16, void* out,
                    int64_t M, int64_t N, int64_t K,
                    int64_t lda, int64_t ldb, int64_t ldo,
                    int epilogue, int out_dtype_id, void* stream);

/*
 * cdit_w8a16_gemm for the Linears of one stage as one launch: up to 4 activations
 * (x_bf16[s] bf16 [M[s], K], common lda) with members_per_act[s] weight-only Linears each, up to
 * 8 members in all, listed activation by activation (member p: b_q[p] e4m3 [N[p], K] with the
 * common ldb, b_scale[p], bias[p] bf16 or NULL, out[p] bf16 [M, N[p]] with ldo[p], epilogue[p]).
 * The weight-only counterpart of cdit_fp8_gemm_rowwise_batched: sibling Linears that read one
 * activation (attn.to_q / to_k / to_v, proj_mlp next to them; reference dataflow
 * src/cache_dit/caching/patch_functors/functor_flux.py:60-67) and the same stage of the other
 * stream of a double-stream block, which the reference runs as one `F.linear` on a dequantized
 * weight each (Float8WeightOnlyConfig, src/cache_dit/quantization/torchao/quantize_ao.py:604-610).
 * Bit-identical to one cdit_w8a16_gemm call per member; what the tile stream does not take
 * (M <= 16, N not a multiple of 16, a single member) runs as those calls.
 */
int cdit_w8a16_gemm_batched(int n_act, const void* const* x_bf16, const int64_t* M, int64_t K,
                            int64_t lda, const int* members_per_act, const void* const* b_q,
                            const float* const* b_scale, const void* const* bias,
                            void* const* out, const int64_t* N, int64_t ldb, const int64_t* ldo,
                            const int* epilogue, void* stream);

/*
 * One quantized nn.Linear forward in the w8a8 dynamic mode: the two calls above
 * back to back on `stream` (per-token quantization of x into the caller's
 * workspace, then the scaled GEMM), saving one trip through the caller's FFI;
 * at M <= 16 a single kernel that quantizes the rows itself, with the same
 * results and the same workspace contents.
 * This is what torchao's Float8Tensor `aten.linear` override does for a Linear
 * that cache-dit converted with `quantize_(..., Float8DynamicActivation
 * Float8WeightConfig(granularity=(PerRow(), PerRow())))`
 * (src/cache_dit/quantization/torchao/quantize_ao.py:166-179, :540-558).
 *
 * x_bf16 [M,K] (ld_x); w_q e4m3 [N,K] (ldw); w_scale fp32 [N]; bias and out as
 * for cdit_fp8_gemm_rowwise (out_dtype_id; a Linear passes CDIT_DT_BF16, the dtype
 * of its input); q_ws: workspace of M*K bytes (receives the activation codes,
 * contiguous); scale_ws: workspace of M floats.
 */
int cdit_fp8_linear_w8a8(const void* x_bf16, const void* w_q, const float* w_scale,
                         const void* bias, void* out, void* q_ws, float* scale_ws,
                         int64_t M, int64_t N, int64_t K,
                         int64_t ld_x, int64_t ldw, int64_t ldo,
                         int scale_mode, int epilogue, int out_dtype_id, void* stream);

/*
 * FP8 quantizers for activations that cross GPUs: the scale is packed behind the codes
 * of each row, so that one buffer travels. They replace the reference's Triton kernels
 * src/cache_dit/kernels/triton/_float8_comm.py:5-148 (op wrappers
 * src/cache_dit/kernels/triton/_ops_registery.py:52-185). Their arithmetic is NOT the
 * GEMM path's quantizer: eps floors, a reciprocal multiply in the per-token form, and
 * their own scale formats. All buffers are contiguous unless a stride is passed.
 *
 * per_token_quant (_float8_comm.py:5-40): x bf16 [M,H] -> y e4m3 [M,H+2]
 *     amax = max(1e-4, max_h |x|);  s = amax / 448;  r = 1 / s           (fp32)
 *     y[m,:H] = e4m3fn_rne(clamp(x * r, -448, 448));  y[m,H:H+2] = bf16_rne(s)
 * per_token_dequant (:43-62): x e4m3 [M,H+2] -> y bf16 [M,H] = bf16_rne(float(code) * s)
 * qkv_permute_quant (:66-113): x bf16 [B,S,P,N,D] (element strides for B, S, P; the last
 *   two dimensions contiguous) -> quant_x e4m3 [P,S,B,N,D+4] contiguous; per head row
 *     s = max(max_d |x| / 448, 1e-6);  codes = e4m3fn_rne(clamp(x / s, -448, 448));
 *     the fp32 s in the 4 trailing bytes. D must be a multiple of 4.
 * qkv_permute_dequant (:116-148): quant_x e4m3 [S,B,N,D+4] (BYTE strides for S, B, N: a
 *   slice quant_x[p] of the above is not contiguous) -> x bf16 [B,S,N,D] contiguous.
 */
int cdit_fp8_comm_per_token_quant(const void* x_bf16, int64_t M, int64_t H, void* y_e4m3,
                                  void* stream);
int cdit_fp8_comm_per_token_dequant(const void* x_e4m3, int64_t M, int64_t H, void* y_bf16,
                                    void* stream);
int cdit_fp8_comm_qkv_permute_quant(const void* x_bf16, int64_t B, int64_t S, int64_t P, int64_t N,
                                    int64_t D, int64_t stride_b, int64_t stride_s, int64_t stride_p,
                                    void* quant_x, void* stream);
int cdit_fp8_comm_qkv_permute_dequant(const void* quant_x, int64_t S, int64_t B, int64_t N, int64_t D,
                                      int64_t stride_s, int64_t stride_b, int64_t stride_n,
                                      void* x_bf16, void* stream);

/*
 * cdit_fp8_linear_w8a8 without the two workspace arguments: the activation codes and
 * scales go to an array inside the library (device memory that every GPU the library
 * runs on holds from the first call on it until the process ends:
 * CDIT_STATIC_WS_CODE_BYTES + 4 * CDIT_STATIC_WS_ROWS bytes). The call allocates and
 * frees nothing, neither on the host nor on the device.
 * This entry point has no counterpart in the reference. It is for callers that cannot
 * allocate: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.
 * Limits: M * K <= CDIT_STATIC_WS_CODE_BYTES and M <= CDIT_STATIC_WS_ROWS, else
 * CDIT_EINVAL with a message and nothing is launched. All calls on one GPU share that
 * GPU's array: calls that overlap in time on one GPU (different streams, different
 * threads) race on it, so keep them on one stream or order them yourself. Nothing in
 * the array has to be cleared between calls: every call overwrites the M rows of codes
 * and the M scales it reads afterwards. Results are those of cdit_fp8_linear_w8a8, bit
 * for bit (the same kernels run).
 */
#define CDIT_STATIC_WS_CODE_BYTES ((int64_t)96 << 20) /* 96 MiB: 6889 x 12288 and smaller */
#define CDIT_STATIC_WS_ROWS ((int64_t)65536)
int cdit_fp8_linear_w8a8_static(const void* x_bf16, const void* w_q, const float* w_scale,
                                const void* bias, void* out,
                                int64_t M, int64_t N, int64_t K,
                                int64_t ld_x, int64_t ldw, int64_t ldo,
                                int scale_mode, int epilogue, int out_dtype_id, void* stream);

/*
 * Writes to *id the id of the graph capture that `stream` is recording into, 0 when it is
 * not capturing. For bindings that keep per-stream state between calls (the Python
 * binding reuses activation codes across sibling Linears): state made inside one capture
 * is only valid inside that capture. No counterpart in the reference, whose op holds no
 * state.
 */
int cdit_stream_capture_id(void* stream, uint64_t* id);

/*
 * Debug and measurement hooks, not part of the operator interface. Both set a
 * process-global value that every later call on any thread reads; they are not thread
 * safe and must not be called while another thread is inside the library. A production
 * caller never needs them (the default, -1, is the automatic choice).
 *
 * cdit_debug_set_gemm_variant: forces the kernel variant the GEMM entry points pick (-1 = by
 * shape). Returns the previous value. The tests use it to run every variant on one shape.
 * cdit_debug_set_quant_hints: forces the cache hints of the per-row quantizer (0: loads
 * and stores non-temporal, 1: neither, 2: loads, 3: stores; anything else = -1 = by
 * size). Returns the previous value. Results never depend on it.
 */
int cdit_debug_set_gemm_variant(int variant);
int cdit_debug_set_quant_hints(int hints);

/*
 * Measurement aid, not part of the operator interface (no counterpart in the reference):
 * launches `blocks` workgroups of four wavefronts that run `iters` rounds of 16 independent
 * v_mfma_f32_16x16x128_f8f6f4 instructions (the FP8 GEMM's instruction) on register
 * operands and nothing else, with pseudo-random e4m3 operands (random_operands != 0) or
 * all-ones operands. out_f32: blocks * 256 floats of device memory (written so that the loop
 * is not dead code). *flop (host memory, may be null) receives the floating-point operations
 * of the launch. Timing it gives the rate the matrix cores of the part at hand sustain before
 * a byte is moved: the ceiling bench.py reports next to the GEMM's rate.
 */
int cdit_debug_mfma_only(void* out_f32, int blocks, int iters, int random_operands, double* flop,
                         void* stream);

/*
 * Measurement aid, not part of the operator interface (no counterpart in the reference):
 * cdit_fp8_gemm_rowwise (bf16 output, no epilogue flags) on the 288 x 192 tile kernel, built
 * with time stamps: every workgroup (one per CU, at most one per tile; their number goes to
 * *workgroups, host memory, may be null) leaves four 64-bit words at stamps_u64 + 4 * its
 * index: the constant-rate wall clock (100 MHz ticks) at its start and at its end, the id
 * of the XCD it ran on, and the number of tiles it computed. stamps_u64: device memory for
 * 4 * 256 words at least. The output is the GEMM's. What bench.py derives from it: how far
 * the workgroups' finish times lie apart by XCD, in units of one tile's time, which is what
 * decides whether handing tiles out dynamically could shorten a launch.
 */
int cdit_debug_gemm_stamps(const void* a_q, const float* a_scale, const void* b_q, const float* b_scale,
                           const void* bias, void* out, int64_t M, int64_t N, int64_t K, int64_t lda,
                           int64_t ldb, int64_t ldo, void* stamps_u64, int* workgroups, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CDIT_HIP_H_ */
