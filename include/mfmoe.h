/*
 * mfmoe.h — C ABI of libmfmoe: the MoE expert hot path of Mference on MI355X
 * (gfx950), hand-written HIP behind plain pointers and sizes.
 *
 * The reference has no C/FFI interface; its operator surface is a set of Swift
 * classes under Sources/Mference/Kernels/ whose encode…() methods append
 * dispatches to a caller-owned MTLCommandBuffer.  Each entry point below names
 * the Swift method (file:line, relative to the Mference repository root) it
 * replaces.  Conventions of the mapping:
 *
 *   MetalContext                    -> mf_ctx*            (device + kernel state)
 *   MTLCommandBuffer                -> mf_stream          (a hipStream_t; work is
 *                                      ordered by the stream, nothing is synchronised)
 *   (MTLBuffer, byte offset)        -> device pointer, the caller adds the offset
 *   `throws` / precondition         -> negative mf_status, nothing is launched
 *   half activations                -> bf16 bit patterns (uint16_t); accumulation
 *                                      is fp32 and the reference's narrowing points
 *                                      are kept, narrowing to bf16 instead of fp16
 *
 * All pointers are DEVICE pointers unless a parameter says "host".  Activations
 * and scale/bias tables must be 2-byte aligned; packed weights may have any
 * alignment (16-byte aligned tensors take the fast 128-bit-load kernels).
 * A handle (mf_moe*) owns a small device workspace and is therefore serial:
 * do not use one handle from two streams at once (MapleMoE.swift:3-6).
 */
#ifndef MFMOE_H
#define MFMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MF_GROUP_SIZE 64 /* Quantization.groupSize, Quantization.swift:5 */
#define MF_MAX_TOKENS 8  /* kMultiXMaxT, dequant_int4.metal:356 */
#define MF_MAX_TOPK 8    /* kMaxStreamedExperts, moe.metal:5 */
#define MF_MAX_EXPERTS 512
/* rows (tokens) one batched call takes: row * top_k and the byte offsets derived from it stay inside
 * 32 bits; a larger t is refused (MF_ERR_INVALID_ARGUMENT, MF_ERR_QUERY_COUNT where the reference
 * names the query count) */
#define MF_MAX_ROWS (1u << 20)

typedef enum {
  MF_OK = 0,
  MF_ERR_INVALID_ARGUMENT = -1,   /* precondition failures (MoE.swift:165-167) */
  MF_ERR_DIMENSION_MISMATCH = -2, /* SharedExpertError.dimensionMismatch */
  MF_ERR_UNSUPPORTED_BITS = -3,   /* SharedExpertError.unsupportedWeightBits */
  MF_ERR_SCRATCH_TOO_SMALL = -4,  /* SharedExpertError.scratchTooSmall */
  MF_ERR_NO_DEVICE = -5,          /* MetalError.noDevice */
  MF_ERR_OUT_OF_MEMORY = -6,
  MF_ERR_LAUNCH = -7,             /* a HIP call failed; see mf_last_hip_error */
  /* PrefillMoEGroupingError, PrefillMoEGrouping.swift:52-88 */
  MF_ERR_QUERY_COUNT = -10,
  MF_ERR_TOPK = -11,
  MF_ERR_NUM_EXPERTS = -12,
  MF_ERR_TILE_EXPERT_COUNT = -13,
  MF_ERR_PAIR_COUNT = -14,
  MF_ERR_TOKEN_RANGE = -15,
  MF_ERR_RANK_RANGE = -16,
  MF_ERR_EXPERT_RANGE = -17,
  MF_ERR_DUPLICATE_TOKEN_RANK = -18,
  MF_ERR_SORT_KEY_COUNT = -19
} mf_status;

/* weight formats (bits per code) */
typedef enum {
  MF_BITS_TERNARY = 1, /* 2-bit codes {0,1,2}, bf16 scale per 64, bias = -scale */
  MF_BITS_2 = 2,       /* 2-bit affine: 16 codes per uint32, element j at bit 2*(j%16) */
  MF_BITS_4 = 4,       /* 4-bit affine: 8 codes per uint32, element j at bit 4*(j%8)   */
  MF_BITS_8 = 8        /* 8-bit affine, a byte per code (Metal/Quant/dequant_int8.metal:5-13): accepted by
                          mf_quantize_affine, mf_dequantize and mf_gemv, and as the format of the scalar
                          shared gate (mf_moe_layer_weights.w_sg_q8); the experts, the shared expert and
                          mf_qmm take the three formats above */
} mf_bits;

typedef enum {
  MF_ROUTER_TOPK_SOFTMAX = 0, /* select on logits, softmax over the selected
                                 (router_topk_select_k8, moe.metal:190-240) */
  MF_ROUTER_FULL_SOFTMAX = 1  /* softmax over all experts, k x argmax, renormalise
                                 (maple_router_top8_full_softmax, maple_moe.metal:62-119) */
} mf_router_mode;

typedef struct mf_ctx mf_ctx;
typedef struct mf_moe mf_moe;
typedef void* mf_stream; /* hipStream_t; NULL = the default stream */

/* MoEExpertOffsets, Kernels/MoE/MoE.swift:4-29: byte offsets of the nine
 * sub-tensors inside one expert blob. */
typedef struct {
  uint32_t gate_w, gate_s, gate_b;
  uint32_t up_w, up_s, up_b;
  uint32_t down_w, down_s, down_b;
} mf_expert_offsets;

/* One quantized projection: SharedExpertProjection (SharedExpertInt4.swift). */
typedef struct {
  const void* weights;    /* packed codes, rows x cols*bits/8 bytes */
  const uint16_t* scales; /* bf16 [rows, cols/64] */
  const uint16_t* biases; /* bf16 [rows, cols/64]; ignored for MF_BITS_TERNARY */
} mf_qtensor;

/* PrefillTokenExpertPair, Kernels/Prefill/MoE/PrefillRouter.swift:4-28
 * (16-byte POD).  weight_bits carries the fp32 bit pattern of the routing
 * weight (the reference carries fp16 bits in the same field). */
typedef struct {
  uint32_t token, expert, rank, weight_bits;
} mf_pair;

/* ---------------------------------------------------------------- context */

/* MetalContext.init, Infrastructure/Metal/MetalContext.swift:45-65 */
mf_status mf_ctx_create(int device, mf_ctx** out);
void mf_ctx_destroy(mf_ctx* ctx);
const char* mf_status_string(mf_status s);
/* text of the last failing HIP call on this context ("" if none) */
const char* mf_last_hip_error(const mf_ctx* ctx);
int mf_abi_version(void);

/* ----------------------------------------------------------------- format */

/* Quantization.quantizeInt4Affine (Infrastructure/ModelIO/Quantization.swift:50-102)
 * and Int4AffineEncoder.encodeTensor (MferenceRepack/Core/Quantization/
 * Int4AffineEncoder.swift:41-97), on device: w fp32 [rows, n] -> packed codes,
 * bf16 scales, bf16 biases.  bits = 4 or 2. */
mf_status mf_quantize_affine(mf_ctx* ctx, mf_stream stream, const float* w, size_t rows,
                             size_t n, mf_bits bits, void* packed, uint16_t* scales,
                             uint16_t* biases);
/* Quantization.dequantizeInt4Affine (Quantization.swift:104-119): out fp32
 * [rows, n] = float(q) * scale + bias, two roundings (the bit-exact target). */
mf_status mf_dequantize(mf_ctx* ctx, mf_stream stream, mf_qtensor q, size_t rows, size_t n,
                        mf_bits bits, float* out);

/* ------------------------------------------------------------------- GEMV */

/* DequantInt4GEMV.encode (Kernels/Quant/DequantInt4GEMV.swift:57-103) for t = 1,
 * DequantInt4GEMVMultiX.encode (Kernels/Quant/DequantInt4GEMVMultiX.swift:48-82)
 * for 1 < t <= 8, MapleTernaryGEMV.encode (Kernels/Quant/MapleTernaryGEMV.swift:
 * 29-45) for ternary.  x bf16 [t, n], y [t, m] bf16 or fp32 (out_f32 != 0,
 * the _f32out kernels).  Each weight row is read once for all t tokens.
 * Two storages of ternary weights exist in the reference.  Routed experts pack four 2-bit codes
 * per byte with a scale table only (RepackPlanner.swift:560-651): MF_BITS_TERNARY.  The resident
 * projections MapleTernaryGEMV reads keep the same codes widened to nibbles, with a scale (alpha)
 * and a bias (-alpha) table repeated over each source group of 128 (RepackPlanner.swift:414-470,
 * Metal/Quant/maple_ternary.metal:12-15, 59-69): that is a 4-bit affine tensor whose codes happen
 * to be 0, 1, 2 -- pass it as MF_BITS_4. */
mf_status mf_gemv(mf_ctx* ctx, mf_stream stream, mf_qtensor w, mf_bits bits, const uint16_t* x,
                  void* y, uint32_t m, uint32_t n, uint32_t t, int out_f32);

/* Elementwise.encode… (Kernels/Primitives/Elementwise.swift:60-87):
 * silu_mul (utility.metal:21-33), sigmoid_scalar_mul (:49-59), residual_add (:83-92).
 * gate in mf_sigmoid_scalar_mul is one bf16 value per row of `row` elements. */
mf_status mf_silu_mul(mf_ctx* ctx, mf_stream stream, const uint16_t* gate, const uint16_t* up,
                      uint16_t* out, uint32_t count);
mf_status mf_sigmoid_scalar_mul(mf_ctx* ctx, mf_stream stream, uint16_t* y,
                                const uint16_t* gate, uint32_t row, uint32_t rows);
mf_status mf_residual_add(mf_ctx* ctx, mf_stream stream, uint16_t* hidden,
                          const uint16_t* delta, uint32_t count);

/* The step in front of the MoE layer in RealForwardRunner.produceToken
 * (Runtime/Inference/RealForwardRunner.swift:2799-2808): Elementwise.encodeResidualAdd
 * (hidden += delta; utility.metal:83-92) followed by RMSNorm.encodeBF16W
 * (Kernels/Primitives/RMSNorm.swift:52-64; rmsnorm_bf16w, Metal/Primitives/rmsnorm.metal:68-92),
 * as one launch over t rows of d: hidden[t,d] = bf16(hidden + delta) when delta is not NULL, then
 * out[t,d] = bf16(hidden * rsqrt(mean(hidden^2) + eps) * weight[d]), the sum of squares in fp32.
 * out may not alias hidden. */
mf_status mf_residual_rmsnorm(mf_ctx* ctx, mf_stream stream, uint16_t* hidden, const uint16_t* delta,
                              const uint16_t* weight, uint16_t* out, uint32_t d, uint32_t t, float eps);

/* MPPPrefillInt4QMM.encode (Kernels/TensorCore/MPPPrefillInt4QMM.swift:34-78; kernel
 * mpp_prefill_affine_threadgroup_f16, Metal/TensorCore/tensorops.metal:13-105) and its scalar twin
 * PrefillInt4QMM (prefill_dequant_int4_qmm_f16_block, Metal/Prefill/prefill.metal:822-859): the
 * dense projection of many rows, y[m, n] = x[m, k] . deq(W[n, k])^T with fp32 accumulation, x bf16
 * [m, k], y bf16 [m, n] (fp32 when out_f32 != 0), k a multiple of 64, any m and n.  With n and k
 * multiples of 128, 16-byte aligned w.weights / x / y and a 16-byte aligned workspace of at least
 * mf_qmm_workspace_bytes(m, n, k) the call runs on the matrix cores (codes expanded to exact bf16 in
 * registers, one fp32 scale multiply per 64-wide K group -- the kernel of mf_moe_prefill_layer; a K
 * beyond 4096 is cut into windows whose fp32 results are added in order); every other shape,
 * alignment or workspace runs row by row through the kernels of mf_gemv, bit-identical to
 * mf_gemv.  Where the reference returns .unavailable (bad sizes or offsets) the call returns a
 * negative status and launches nothing.  Replaces the 4-bit, 2-bit and ternary projections alike. */
size_t mf_qmm_workspace_bytes(uint32_t m, uint32_t n, uint32_t k);
mf_status mf_qmm(mf_ctx* ctx, mf_stream stream, mf_qtensor w, mf_bits bits, const uint16_t* x, void* y, uint32_t m,
                 uint32_t n, uint32_t k, int out_f32, void* workspace, size_t workspace_bytes);
/* The `Path` MPPPrefillInt4QMM.encode returns (MPPPrefillInt4QMM.swift:5-8, 43-55): which kernel mf_qmm
 * takes for these arguments -- MF_QMM_PATH_MATRIX_CORE or MF_QMM_PATH_ROWS (row by row through the
 * kernels of mf_gemv) -- or the negative status with which mf_qmm would refuse them (the reference's
 * .unavailable).  Launches nothing and touches no device memory. */
#define MF_QMM_PATH_MATRIX_CORE 1
#define MF_QMM_PATH_ROWS 2
int mf_qmm_path(mf_qtensor w, mf_bits bits, const uint16_t* x, const void* y, uint32_t m, uint32_t n, uint32_t k,
                const void* workspace, size_t workspace_bytes);

/* SharedExpertInt4.encode (Kernels/MoE/SharedExpertInt4.swift:70-165) /
 * SharedExpertRuntime.encode (:193-202): y[t,d] = bf16(down . act),
 * act = bf16(silu(bf16(gate.x)) * bf16(up.x)).  Also the dense SwiGLU MLP of Qwen38ForwardRunner
 * (mlp.encode, :1094) and, for any t, PrefillSharedExpert.encodeBlock (Kernels/Prefill/MoE/
 * PrefillSharedExpert.swift:81-190) / encodeDenseMLPPrefill (Qwen38ForwardRunner.swift:862-913):
 * from 32 rows on the projections run on the matrix cores when d and f are multiples of 128,
 * d <= 7168, the operands are 16-byte aligned and scratch_act holds
 * mf_shared_expert_scratch_bytes(d, f, t) bytes; otherwise row by row, MF_MAX_TOKENS rows per pair
 * of launches, for which t*f bf16 of scratch suffice (all that t <= MF_MAX_TOKENS ever needs). */
size_t mf_shared_expert_scratch_bytes(uint32_t d, uint32_t f, uint32_t t);
mf_status mf_shared_expert(mf_ctx* ctx, mf_stream stream, const uint16_t* x, mf_qtensor gate,
                           mf_qtensor up, mf_qtensor down, mf_bits bits, uint32_t d, uint32_t f,
                           uint32_t t, uint16_t* y, uint16_t* scratch_act,
                           size_t scratch_act_bytes);

/* SharedExpertInt8.encode (Kernels/MoE/SharedExpertInt8.swift:78-181; SharedExpertInt4's bits == 8 case,
 * SharedExpertInt4.swift:187): the dense MLP on 8-bit affine tensors (MF_BITS_8: one code per byte, bf16
 * scale and bias per 64).  gate and up rows in one launch (shared_int8_gate_up_act_simd,
 * Metal/Quant/dequant_int8.metal:110-164): both narrowed to 16 bits, act[f] = narrow(a(gate) * up) with
 * a = the tanh form of GELU (int8_gelu_pytorch_tanh, :44-49) or, silu_activation != 0, SiLU
 * (FC_SHARED_INT8_ACT_SILU, :51-57); then y[d] = narrow(down . act) (dequant_int8_gemv_simd, :66-107).
 * Any t; scratch_act holds t*f bf16.  tanh is built on this library's exp (as every exp on this path). */
mf_status mf_shared_expert_int8(mf_ctx* ctx, mf_stream stream, const uint16_t* x, mf_qtensor gate,
                                mf_qtensor up, mf_qtensor down, uint32_t d, uint32_t f, uint32_t t,
                                int silu_activation, uint16_t* y, uint16_t* scratch_act,
                                size_t scratch_act_bytes);

/* mf_shared_expert for callers that cannot allocate device memory and bring no scratch buffer:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference, whose operators always take the caller's scratch buffer.
 * The activation vector act[t,f] lives in a device array that is
 * part of the library image (MF_STATIC_ACT_ELEMS bf16 = 512 KiB, held on every GPU the library
 * runs on until the process ends); the call launches the kernels of mf_shared_expert and calls no
 * hipMalloc / hipFree.  Same arguments, checks and results (bit for bit) as mf_shared_expert;
 * t * f > MF_STATIC_ACT_ELEMS returns MF_ERR_SCRATCH_TOO_SMALL and launches nothing.  All calls on
 * one GPU share the array: calls that overlap on one GPU (two streams, two threads) race. */
#define MF_STATIC_ACT_ELEMS (MF_MAX_TOKENS * 32768u)
mf_status mf_shared_expert_static(mf_ctx* ctx, mf_stream stream, const uint16_t* x, mf_qtensor gate,
                                  mf_qtensor up, mf_qtensor down, mf_bits bits, uint32_t d, uint32_t f,
                                  uint32_t t, uint16_t* y);

/* ---------------------------------------------------------- MoE operator */

/* Shape/activation specialisation of one operator instance: MoE.init
 * (Kernels/MoE/MoE.swift:65-151), MoEDeepseekV4.init (MoEDeepseekV4.swift:31-87),
 * MapleMoE.init (MapleMoE.swift). */
typedef struct {
  uint32_t d;            /* hidden size, multiple of 64 */
  uint32_t f;            /* routed expert intermediate, multiple of 64 */
  uint32_t num_experts;  /* <= MF_MAX_EXPERTS */
  uint32_t top_k;        /* 1..MF_MAX_TOPK */
  mf_bits bits;          /* routed expert format */
  mf_router_mode router_mode;
  float swiglu_limit;    /* FC_MOE_SWIGLU_LIMIT, moe.metal:27-34; <= 0: none */
  uint32_t shared_f;     /* shared expert intermediate; 0 = no shared expert */
  mf_bits shared_bits;
  uint32_t maple_rounding; /* 1: MapleMoE's rounding points -- gate and up narrowed to bf16 and
                            * clamped at 7 / +-7, the sigmoid built in bf16 steps
                            * (maple_swiglu, Metal/MoE/maple_moe.metal:153-164), each expert's
                            * down output narrowed to bf16 before its routing weight
                            * (maple_moe_phase2, maple_moe.metal:243-264); swiglu_limit is
                            * ignored.  0: the MoE / MoEDeepseekV4 rule (moe.metal:27-34, 528,
                            * 1262-1270) */
  uint32_t gate_group_size; /* quantization group of the routed GATE projection: 0 or 64 = like every other
                             * table; 32 = the DeepSeek-V4 conversion's gate_proj (two scale / bias entries
                             * per 64 weights: moe_int2_gate_up_rows_simd_dev_vec's gate_group_size,
                             * Metal/MoE/moe.metal:962-1060; MoEDeepseekV4.encodeRoutedPhase1(gateGroupSize:),
                             * MoEDeepseekV4.swift:199-263; Model.routedGateGroupSize,
                             * Runtime/Inference/ModelExpertIO.swift:118-135).  2-bit experts only.  Such a
                             * layer runs on the chain of launches (the fused launch and the matrix-core
                             * prefill take group 64); up and down stay at 64. */
} mf_moe_config;

/* The preconditions of MoE.init / MoEDeepseekV4.init / MapleMoE.init (MoE.swift:65-151, 165-167;
 * MoEDeepseekV4.swift:31-87) as a status instead of a trap: MF_OK when mf_moe_create would accept the
 * shape.  Host arithmetic only, no device.  Refused: sizes that are no multiples of 64, more than
 * MF_MAX_EXPERTS experts or MF_MAX_TOPK routes, an unknown format, the full-softmax router
 * (MF_ROUTER_FULL_SOFTMAX) with an expert count that is no multiple of 32, a gate group of 32 on
 * anything but 2-bit experts. */
mf_status mf_moe_config_check(const mf_moe_config* cfg);

/* MoE.init (Kernels/MoE/MoE.swift:65-151): one operator instance per shape; owns the
 * router-logit and activation workspace (MoE.swift:136-150). */
mf_status mf_moe_create(mf_ctx* ctx, const mf_moe_config* cfg, mf_moe** out);
void mf_moe_destroy(mf_moe* h);

/* Router: bf16 GEMV + top-k + routing weights.
 * MoEDeepseekV4.encodeRouterGemv + encodeRouterTopK (MoEDeepseekV4.swift:153-173,
 * 92-100), MoE.encodeRouterGemma4 (MoE.swift:153-203), MapleMoE.encodeRouterTop8
 * (MapleMoE.swift:81-131), PrefillRouter.encodeGemma4Block for t > 1
 * (Kernels/Prefill/MoE/PrefillRouter.swift:37-89).
 * router_w bf16 [num_experts, d]; x bf16, row t at x + t*x_stride elements;
 * out_idx uint32 [t, top_k]; out_w fp32 [t, top_k]; out_logits fp32
 * [t, num_experts] or NULL.  Any t >= 1.  From 16 tokens on the logits of a call are
 * computed by the batched kernels of the prefill layer (the same bits); without
 * out_logits the call works through the handle's own buffer 256 rows at a time. */
mf_status mf_moe_router(mf_moe* h, mf_stream stream, const uint16_t* router_w,
                        const uint16_t* x, uint32_t t, uint32_t x_stride, uint32_t* out_idx,
                        float* out_w, float* out_logits);

/* ---- family-specific routers.  Stand-alone (no operator handle): the logits go through the
 * caller's fp32 buffer `logits` [t, rows], which stands in for the operators' internal
 * routerLogits buffer (MoEDeepseekV4.swift:31-87, InklingKernels.swift:377-417).  All keep the
 * tie rule of mf_moe_router (equal score keeps the lower index) and write fp32 routing
 * weights where the reference narrows to fp16.  top_k <= MF_MAX_TOPK, experts <=
 * MF_MAX_EXPERTS, d a multiple of 8; x rows as in mf_moe_router.  Their outputs feed
 * mf_moe_phase1 / mf_moe_phase2 like mf_moe_router's. */

/* MoEDeepseekV4.encodeRouterTopK (Kernels/MoE/MoEDeepseekV4.swift:92-124): bf16 router GEMV
 * (router_gemv_bf16_r4, Metal/MoE/moe.metal:162-185), then
 * router_topk_select_sqrtsoftplus_k6(_par) (moe.metal:744-841): experts are picked on
 * sqrt(softplus(logit)) + correction_bias[e], weighed by the raw scores of the picked,
 * renormalised and times route_scale.  correction_bias fp32 [num_experts]. */
mf_status mf_router_sqrtsoftplus(mf_ctx* ctx, mf_stream stream, const uint16_t* router_w,
                                 const uint16_t* x, uint32_t t, uint32_t x_stride,
                                 uint32_t num_experts, uint32_t d, uint32_t top_k,
                                 const float* correction_bias, float route_scale, float* logits,
                                 uint32_t* out_idx, float* out_w);

/* MoEDeepseekV4.encodeRouterHashWeights (MoEDeepseekV4.swift:126-151),
 * router_hash_weights_k6(_par) (moe.metal:847-896): the experts of every token are given
 * (indices uint32 [t, top_k], repeats allowed); only their weights are computed.  An index
 * >= num_experts gets weight 0. */
mf_status mf_router_hash_weights(mf_ctx* ctx, mf_stream stream, const uint16_t* router_w,
                                 const uint16_t* x, uint32_t t, uint32_t x_stride,
                                 uint32_t num_experts, uint32_t d, uint32_t top_k,
                                 const uint32_t* indices, float route_scale, float* logits,
                                 float* out_w);

/* InklingKernels.encodeRouter / encodeRouterPrefill (Kernels/Inkling/InklingKernels.swift:
 * 377-476), inkling_router_select(_prefill) (Metal/Inkling/inkling.metal:503-626): router_w
 * bf16 [n_routed + n_shared, d], the shared-expert sink rows last.  Experts are picked on
 * sigmoid(logit) + gate_bias[e] (fp32 [n_routed]); weights are the softmax over logsigmoid of
 * the raw logits of the picked experts and the sinks, times route_scale * global_scale[0]
 * (device fp32).  out_gammas fp32 [t, n_shared] (may be NULL when n_shared == 0);
 * n_shared <= 8; out_idx / out_w are [t, top_k] (the reference's fixed stride is 8). */
mf_status mf_router_inkling(mf_ctx* ctx, mf_stream stream, const uint16_t* router_w,
                            const uint16_t* x, uint32_t t, uint32_t x_stride, uint32_t n_routed,
                            uint32_t n_shared, uint32_t d, uint32_t top_k, const float* gate_bias,
                            const float* global_scale, float route_scale, float* logits,
                            uint32_t* out_idx, float* out_w, float* out_gammas);

/* MoE.encodeRouterGemma4 (Kernels/MoE/MoE.swift:153-202): router_gemv_gemma4_r4
 * (moe.metal:102-157) over 8-bit affine router rows (codes uint8 [num_experts, d], bf16
 * scales and biases [num_experts, d/64]) with x scaled element-wise by effective_scale
 * (bf16 [d]), then router_topk_select_k8(_par) (moe.metal:190-345): softmax over the picked
 * experts times per_expert_scale[e] (bf16 [num_experts]).  d a multiple of 64. */
mf_status mf_router_gemma4(mf_ctx* ctx, mf_stream stream, const uint8_t* router_codes,
                           const uint16_t* router_scales, const uint16_t* router_biases,
                           const uint16_t* x, uint32_t t, uint32_t x_stride,
                           const uint16_t* effective_scale, const uint16_t* per_expert_scale,
                           uint32_t num_experts, uint32_t d, uint32_t top_k, float* logits,
                           uint32_t* out_idx, float* out_w);

/* Routed phase 1: acts[t,k,f] = bf16(act(gate.x) * up.x).
 * MoE.encodeRoutedPersistentPhase1U16Load (MoE.swift:220-253),
 * MoEDeepseekV4.encodeRoutedPhase1 (MoEDeepseekV4.swift:191-199),
 * MapleMoE.encodePhase1 (MapleMoE.swift:146-150).  Experts are resident:
 * blob of expert e at expert_base + e*expert_stride (the slab + slot-offset
 * addressing of MoE.encodeSlotMapGuardedFFN, MoE.swift:333-346), selected on
 * device by idx[t,k]; idx >= num_experts (router sentinel) gives zero acts. */
mf_status mf_moe_phase1(mf_moe* h, mf_stream stream, const void* expert_base,
                        size_t expert_stride, const mf_expert_offsets* offsets,
                        const uint32_t* idx, const uint16_t* x, uint32_t t, uint32_t x_stride,
                        uint16_t* acts);

/* The same for a subset of the routed slots: MoE.encodeRoutedPersistentPhase1SubsetU16Load
 * (MoE.swift:255-298), MoEDeepseekV4.encodeRoutedPhase1Subset (MoEDeepseekV4.swift:223-263),
 * moe_phase1_gate_up_act_subset_u16load (moe.metal:531-565) -- the reference splits phase 1
 * into cache hits and misses; with every expert resident nothing needs the split, but its
 * invariant holds: the subsets together write the same bits as the full call.
 * active_slots: device uint32 [active_count], entries token*top_k + slot; an entry past
 * t*top_k does nothing (moe.metal:551); active_count == 0 launches nothing. */
mf_status mf_moe_phase1_subset(mf_moe* h, mf_stream stream, const void* expert_base,
                               size_t expert_stride, const mf_expert_offsets* offsets,
                               const uint32_t* idx, const uint16_t* x, uint32_t t,
                               uint32_t x_stride, uint16_t* acts, const uint32_t* active_slots,
                               uint32_t active_count);

/* Routed phase 2: y[t,d] = bf16(residual[t,d] + sum_k w[t,k] * (down_k . acts[t,k]))
 * in rank order.  MoE.encodeRoutedPersistentPhase2Reduce (MoE.swift:400-440),
 * MoEDeepseekV4.encodeRoutedPhase2Reduce (MoEDeepseekV4.swift:265-274).
 * residual may be NULL (MapleMoE.encodePhase2, MapleMoE.swift:214-219). */
mf_status mf_moe_phase2(mf_moe* h, mf_stream stream, const void* expert_base,
                        size_t expert_stride, const mf_expert_offsets* offsets,
                        const uint32_t* idx, const float* w, const uint16_t* acts,
                        const uint16_t* residual, uint32_t t, uint16_t* y);

/* Byte offsets of the nine sub-tensors of one routed expert of hidden size d and intermediate
 * size f, laid out back to back in the order the reference's repacker writes them -- gate
 * {codes, scales, biases}, up {...}, down {...} (MferenceRepack/Core/Planning/RepackPlanner.swift:
 * 544-712; read back by Model.routedExpertOffsets, Runtime/Inference/ModelExpertIO.swift:20-35);
 * blob_bytes: size of one expert; stride: that size rounded up to `align` (the reference rounds to a
 * 16 KiB page).  Host arithmetic only; for callers that build a resident pool themselves (synthetic
 * weights, tests).
 * Ternary experts, mf_expert_blob_layout: a COMPACT form private to this library -- codes and scale tables
 * only, bias offsets 0 (the kernels take bias = -scale) -- which is NOT the byte layout of a Maple
 * packed_experts file.  mf_expert_blob_layout_repacked gives the layout the reference's repacker writes for
 * every format: ternary tensors carry their negated-scale bias tables there too (RepackPlanner.swift:619-640),
 * so offsets, blob size and stride equal those of a real file; for 4-bit and 2-bit experts the two calls
 * agree.  The ternary operators accept either layout (they read the scale tables only). */
mf_status mf_expert_blob_layout(uint32_t d, uint32_t f, mf_bits bits, uint32_t align, mf_expert_offsets* offsets,
                                size_t* blob_bytes, size_t* stride);
mf_status mf_expert_blob_layout_repacked(uint32_t d, uint32_t f, mf_bits bits, uint32_t align,
                                         mf_expert_offsets* offsets, size_t* blob_bytes, size_t* stride);

/* The routed phases over slots named directly, for a caller that holds its experts in slots of its
 * own (a streaming cache) instead of one pool indexed by expert id.  Slot s = token * top_k + rank
 * reads the blob at (uint8*)slab + slot_offsets[s]:
 *  - slab + per-slot byte offsets: MoE.encodeSlotMapGuardedFFN (Kernels/MoE/MoE.swift:333-407; kernels
 *    moe_phase1_gate_up_act_slotmap / moe_phase2_down_reduce_slotmap, Metal/MoE/moe.metal:619-708);
 *  - slab == NULL and the table holding device ADDRESSES: the routed argument buffer of K
 *    (buffer, offset) pairs, MoE.makeRoutedArgumentBuffer + encodeRoutedPersistentPhase1U16Load /
 *    encodeRoutedPersistentPhase2Reduce(routedArgBuffer:routedBlobs:) (MoE.swift:205-253, 409-440).
 * slot_offsets: device, uint64 [t * top_k] (the reference's are 32-bit: its slab is below 4 GiB); every
 * blob starts on a 16-byte boundary.  all_hit (nullable): a device word; the launches do nothing while it
 * reads 0 -- the guard of the reference's slot-map form, whose lookup kernel writes it.
 * mf_moe_slot_lookup is that kernel, router_slot_lookup_k8 (moe.metal:594-617): slot_of is the caller's
 * device table int16 [num_experts] (negative: not in a slot); out_slot_offsets[s] = slot * slot_stride,
 * out_all_hit = 1 when every routed expert of the call has a slot.
 * Limits: t <= MF_MAX_TOKENS in all three calls (one guard word covers one lookup; longer batches go in
 * chunks, each with its own lookup and guard word).  slot_stride has to be a multiple of 16 (anything else
 * is refused with MF_ERR_INVALID_ARGUMENT); a slab that is not 16-byte aligned is read through the byte-wise
 * kernels.  In the table-of-addresses form (slab == NULL) the host cannot see the addresses: the 16-byte
 * alignment of every blob is the caller's promise there, as the header of this comment states. */
mf_status mf_moe_slot_lookup(mf_moe* h, mf_stream stream, const uint32_t* idx, uint32_t t,
                             const int16_t* slot_of, uint64_t slot_stride, uint64_t* out_slot_offsets,
                             uint32_t* out_all_hit);
mf_status mf_moe_phase1_slots(mf_moe* h, mf_stream stream, const void* slab, const uint64_t* slot_offsets,
                              const uint32_t* all_hit, const mf_expert_offsets* offsets, const uint16_t* x,
                              uint32_t t, uint32_t x_stride, uint16_t* acts);
mf_status mf_moe_phase2_slots(mf_moe* h, mf_stream stream, const void* slab, const uint64_t* slot_offsets,
                              const uint32_t* all_hit, const mf_expert_offsets* offsets, const float* w,
                              const uint16_t* acts, const uint16_t* residual, uint32_t t, uint16_t* y);

/* Everything one layer reads. */
typedef struct {
  const uint16_t* router_w;   /* bf16 [num_experts, d]; NULL: the routing is the caller's -- the layer
                               * calls then READ out_idx / out_w (both required, e.g. written by a
                               * family router above; the reference's runners likewise route first and
                               * hand the result to the expert phases,
                               * RealForwardRunner+DSV4Prefill.swift:690-806) and run no router.  An
                               * index >= num_experts contributes nothing. */
  const void* expert_base;
  size_t expert_stride;
  mf_expert_offsets offsets;
  mf_qtensor shared_gate, shared_up, shared_down; /* used when shared_f > 0 */
  const uint16_t* w_sg;       /* bf16 [d] scalar shared gate, or NULL */
  mf_qtensor w_sg_q8;         /* the scalar shared gate as the reference's model files store it: 8-bit affine
                               * [1, d] with bf16 scale / bias per 64 (DequantInt8GEMV on sharedProj.scalarGate,
                               * Runtime/Inference/RealForwardRunner.swift:2925-2941; dequant_int8_gemv_simd,
                               * Metal/Quant/dequant_int8.metal:66-107).  Used when w_sg_q8.weights != NULL
                               * (w_sg is then ignored); all three pointers zero: w_sg decides.  The gate
                               * logit is the mf_gemv(MF_BITS_8) value of that row, narrowed to bf16. */
  const void* expert_tiled;   /* NULL, or a second copy of the expert pool in the prefill matmul's own order
                               * (mf_moe_tile_experts: same stride, same offsets).  mf_moe_prefill_layer reads the
                               * routed experts from it when it is given (and the configuration takes the
                               * matrix-core path); the decode calls never do.  Same results, bit for bit. */
} mf_moe_layer_weights;

/* The fused decode layer, one launch: router -> top-k -> routed gate/up/act ->
 * down + weighted sum, + gated shared expert.  Replaces the per-layer chain of
 * RealForwardRunner.produceToken (Runtime/Inference/RealForwardRunner.swift:
 * 2811-2820 router, :2910-2942 shared expert + sigmoid gate, :3181-3218 routed
 * phases) with no host readback between router and experts.
 * x, y bf16 [t, d], t <= MF_MAX_TOKENS; out_idx / out_w may be NULL.
 * If `hidden` is not NULL, hidden[t,d] = bf16(hidden + y) is applied in the same
 * launch (residual_add_fp16, utility.metal:83-92).
 *
 * What the caller owes the fused launch.  It is one workgroup per compute unit, and the workgroups
 * hand each other the router logits and the routed activations through device memory while they
 * run, so all of them must be on the device at the same time: while it runs, nothing else may
 * occupy compute units of this device -- no kernel on another stream, no other process on the
 * card.  Launches on ONE stream (or one captured graph) keep the contract by themselves.  A
 * workgroup that waits for a neighbour that never started gives up after a bounded spin (about
 * 0.1 s), writes NaN to every element of y it owns, leaves `hidden` untouched and records the
 * event; mf_moe_status then returns MF_ERR_LAUNCH.  So a y of NaN with a finite x means: check
 * mf_moe_status.  An engine that overlaps this layer with kernels on other streams (attention,
 * copies done by kernels) calls mf_moe_set_fused(h, 0) once and gets the chain of ordinary
 * launches, which have no such requirement and give the same bits.  Two handles used at the same
 * time on two streams of one device fall under the same rule. */
mf_status mf_moe_decode_layer(mf_moe* h, mf_stream stream, const mf_moe_layer_weights* wts,
                              const uint16_t* x, uint32_t t, uint16_t* y, uint16_t* hidden,
                              uint32_t* out_idx, float* out_w);

/* mf_moe_decode_layer with the step in front of it in the same launch (RealForwardRunner.produceToken,
 * Runtime/Inference/RealForwardRunner.swift:2799-2808: Elementwise.encodeResidualAdd, RMSNorm.encodeBF16W,
 * then the MoE layer and the residual add behind it): h' = bf16(hidden + delta) when delta is not NULL (else
 * hidden), x = bf16(h' * rsqrt(mean(h'^2) + eps) * norm_weight[d]) as mf_residual_rmsnorm makes it, y = the
 * layer on x, hidden[t,d] = bf16(h' + y).  One launch when the fused launch takes the layer (own routing,
 * d <= 4096, the normalised rows fit its LDS): every workgroup normalises the rows for itself and reads x
 * from LDS, the separate norm launch and the graph node between the two go away (Qwen shape, one token,
 * 40 layers from a graph: 13.2 us per layer against 19.7 us as two launches).  Otherwise mf_residual_rmsnorm into rows of the handle followed by mf_moe_decode_layer.
 * Both forms give the bits of those two calls.  When a bounded wait of the fused launch gives up
 * (mf_moe_status), hidden is left as it was, delta not added. */
mf_status mf_moe_decode_layer_normed(mf_moe* h, mf_stream stream, const mf_moe_layer_weights* wts,
                                     uint16_t* hidden, const uint16_t* delta, const uint16_t* norm_weight,
                                     float eps, uint32_t t, uint16_t* y, uint32_t* out_idx, float* out_w);

/* Chooses between the single fused launch (default) and the chain of separate
 * launches (router, top-k, shared expert, phase 1, phase 2) inside
 * mf_moe_decode_layer.  Both give bit-identical results; the chain is the
 * structure of the reference's decode step and handles operands that are not
 * 16-byte aligned.  enabled = 2: the fused launch, but through the kernel instance that reads every
 * dimension from its arguments even when the build holds an instance with this layer's shape as
 * literals (the reference specialises every shape through function constants, Kernels/MoE/MoE.swift:80-91;
 * here the build specialises the shapes listed in mference_amd/fused_shapes.json) -- same bits, for
 * measuring what the literals buy.  No counterpart in the reference. */
mf_status mf_moe_set_fused(mf_moe* h, int enabled);

/* Phase trace of the fused launch: when device_buffer is not NULL every
 * workgroup writes the 100 MHz wall clock at its stage boundaries (slots:
 * 0 start, 1 stage A done, 2 logits gathered, 3 top-k done, 4 stage B done,
 * 5 routed activations gathered, 6 end) to device_buffer[workgroup*8 + slot]; needs
 * mf_ctx_num_cu()*8*8 bytes.  mf_moe_prefill_layer writes, for as many work
 * items (tile x row slice) of its routed gate/up matmul as the buffer holds, the
 * stamps 0 start, 1 loads issued, 2 tables and bias terms done, 3 main loop done,
 * 4 end at device_buffer[item*8 + slot].  The counterpart of the reference's
 * MFERENCE_PHASES=1 phase counters (RealForwardRunner.swift:397-398). */
mf_status mf_moe_set_phase_trace(mf_moe* h, uint64_t* device_buffer, size_t bytes);
int mf_ctx_num_cu(const mf_ctx* ctx);

/* Synchronises `stream` and reports whether any fused launch of this handle
 * gave up waiting for data of another workgroup (MF_ERR_LAUNCH) since the handle was created
 * (the outputs of such a launch are NaN, see mf_moe_decode_layer; mf_last_hip_error names the
 * status word).  MF_OK means every fused launch so far ran to the end.
 * No counterpart in the reference (Metal reports this through
 * MTLCommandBuffer.error). */
mf_status mf_moe_status(mf_moe* h, mf_stream stream);

/* ------------------------------------------------------- ragged prefill */

/* PrefillRouter.makeTokenExpertPairs + PrefillMoEGrouping.groupTokenExpertPairs
 * (Kernels/Prefill/MoE/PrefillRouter.swift:91-111, PrefillMoEGrouping.swift:
 * 91-192) on device with no host readback: histogram, exclusive scan and stable
 * scatter.  idx [t, top_k] and w [t, top_k] as written by mf_moe_router.
 * Outputs: sorted pairs [t*top_k] ordered by (expert, token, rank);
 * expert_offsets [num_experts] (0xFFFFFFFF for an expert with no token);
 * expert_counts [num_experts].  Routes whose idx >= num_experts are invalid
 * and make the call's device-side status word non-zero (checked by
 * mf_moe_group_status). */
mf_status mf_moe_group(mf_moe* h, mf_stream stream, const uint32_t* idx, const float* w,
                       uint32_t t, mf_pair* sorted_pairs, uint32_t* expert_offsets,
                       uint32_t* expert_counts);
/* Synchronises the stream and maps the device status word of the last
 * mf_moe_group to MF_OK / MF_ERR_EXPERT_RANGE: the device-side form of
 * PrefillMoEGroupingError.expertOutOfRange (PrefillMoEGrouping.swift:60, 131),
 * which the reference throws from its host loop. */
mf_status mf_moe_group_status(mf_moe* h, mf_stream stream);

/* PrefillMoEGrouping.groupTokenExpertPairs (Kernels/Prefill/MoE/
 * PrefillMoEGrouping.swift:91-192) with the reference's full result and error
 * contract, on HOST pointers: pairs sorted by (sort key, expert, token, rank),
 * per-expert offsets (0xFFFFFFFF when empty) and counts, groups, and tiles of
 * <= tile_expert_count live experts.  groups/tiles need room for min(num_experts, n_pairs). */
typedef struct { uint32_t expert, pair_start, pair_count; } mf_group;
typedef struct { uint32_t group_start, group_count, pair_start, pair_count; } mf_tile;
mf_status mf_group_pairs_host(const mf_pair* pairs, size_t n_pairs, int query_count, int top_k,
                              int num_experts, int tile_expert_count,
                              const uint64_t* sort_keys, size_t n_sort_keys, mf_pair* sorted,
                              uint32_t* offsets, uint32_t* counts, mf_group* groups,
                              size_t* n_groups, mf_tile* tiles, size_t* n_tiles,
                              uint32_t err_detail[2]);

/* Ragged prefill layer: router -> device grouping -> per-expert gather-QMM
 * (4-bit codes expanded to exact bf16 in registers, bf16 MFMA, per-group fp32 scale) ->
 * SwiGLU -> down-proj -> weighted un-permute, + shared expert.  Replaces
 * PrefillGroupedRoutedMoE.encodeStreamedBatched (Kernels/Prefill/MoE/
 * PrefillGroupedRoutedMoE.swift:392-466) + PrefillMoE.encodeReduceTokenMajor
 * (PrefillMoE.swift:11-38) + PrefillSharedExpert.encodeBlock/encodeQwenScalarGate
 * (PrefillSharedExpert.swift:81-99, 27-36).  Result per token equals
 * mf_moe_decode_layer on that token within the layer tolerance.
 * Any t >= 1.  The matrix-core path takes 4-bit, 2-bit and ternary experts (with a 4-bit
 * shared expert, if any) with d, f, shared_f multiples of 128 and x, y and every weight
 * tensor 16-byte aligned; every other configuration (other widths, another shared-expert
 * format) runs the same rows through the decode launch, MF_MAX_TOKENS at a time, and needs
 * no workspace.  Covers MoEDeepseekV4's pair-major 2-bit prefill
 * (Metal/MoE/moe.metal:1293-1409) with the same call.
 * workspace: device scratch of at least mf_moe_prefill_workspace_bytes(h, t) (0 when the
 * configuration takes the decode launch; workspace may then be null). */
size_t mf_moe_prefill_workspace_bytes(const mf_moe* h, uint32_t t);
mf_status mf_moe_prefill_layer(mf_moe* h, mf_stream stream, const mf_moe_layer_weights* wts,
                               const uint16_t* x, uint32_t t, uint16_t* y, void* workspace,
                               size_t workspace_bytes, uint32_t* out_idx, float* out_w);

/* A copy of the expert pool for the prefill matmuls.  The reference repacks a model's experts once, offline,
 * into the layout its kernels read best (MferenceRepack, RepackPlanner.swift:414-651); the counterpart here
 * is done at load time on the device: `tiled` (expert_stride * num_experts bytes, 16-byte aligned, not
 * overlapping the source) receives every blob with its three code sub-tensors re-ordered so that a load
 * instruction of the matrix-core matmul reads consecutive bytes (inside a sub-tensor: blocks of 32 rows, K
 * group by K group, the 64 half-group pieces of a block and group side by side); tables, offsets and stride
 * are unchanged.  Costs a second pool in HBM (Qwen shape: 453 MB per layer) and buys 4..7 % of a prefill
 * layer.  Needs the matrix-core configuration (mf_moe_prefill_workspace_bytes(h, t) != 0), else
 * MF_ERR_DIMENSION_MISMATCH. */
mf_status mf_moe_tile_experts(mf_moe* h, mf_stream stream, const void* expert_base, size_t expert_stride,
                              const mf_expert_offsets* offsets, void* tiled);

/* How mf_moe_prefill_layer rounds a route's down-projection result before it meets its routing weight.
 * narrow = 0 (default): kept in fp32, as the decode step keeps it (moe.metal:1262-1270) -- prefill and
 * decode then agree to the last rounding of the sum.  narrow = 1: narrowed to a 16-bit number first, the
 * rule of the reference's prefill kernels (prefill_moe_int4_down_route_partials writes 16-bit
 * route_partials, prefill_moe_reduce_token_major reads them, Metal/Prefill/prefill.metal:817-819,
 * 644-651; 16-bit is bf16 here, as everywhere on this path): half the bytes between the down projection
 * and the reduce.  A handle with maple_rounding narrows either way (maple_moe.metal:258) and always
 * stores 16-bit results.  mf_moe_ragged_qmm's route_partials stay fp32. */
mf_status mf_moe_set_prefill_route_rounding(mf_moe* h, int narrow);


/* The two halves of the ragged layer on their own, for callers that hold a grouping already.
 *
 * mf_moe_ragged_qmm: PrefillGroupedRoutedMoE.encodeStreamedBatched (Kernels/Prefill/MoE/
 * PrefillGroupedRoutedMoE.swift:392-466): for every route of `sorted_pairs` (mf_moe_group's output:
 * the routes of expert 0, then expert 1, ..., expert_counts[e] of them each, starting at 0) the routed
 * expert's gate/up -> SwiGLU -> down result as fp32 in route_partials[(token * top_k + rank), d], the
 * row order the reference's down kernel writes (prefill.metal route_partials).  Rows of routes that are
 * not in the grouping are left untouched.  The reference walks the pairs in micro-batches of 32 rows
 * per dispatch pair; here one launch per projection covers every tile of every expert.  The counts
 * and pairs are checked on the device before they are trusted (sum of counts <= t * top_k, token < t,
 * rank < top_k): a grouping that fails computes nothing and mf_moe_group_status returns
 * MF_ERR_EXPERT_RANGE.  Needs the matrix-core configuration (mf_moe_prefill_workspace_bytes(h, t) != 0),
 * else MF_ERR_DIMENSION_MISMATCH; workspace as for mf_moe_prefill_layer.
 *
 * mf_moe_unpermute: PrefillMoE.encodeReduceTokenMajor (Kernels/Prefill/MoE/PrefillMoE.swift:11-38,
 * Metal/Prefill/prefill.metal:631-652): y[token, :] = sum over ranks of route_weights[token, rank] *
 * route_partials[token * top_k + rank, :], accumulated in fp32 in rank order, stored as bf16.
 * idx (nullable) [t, top_k]: routes whose expert index is >= num_experts are skipped, as the layer call
 * skips them; residual (nullable) [t, d] bf16 is the value the sum starts from (the shared expert's
 * output in the layer call). */
mf_status mf_moe_ragged_qmm(mf_moe* h, mf_stream stream, const void* expert_base, size_t expert_stride,
                            const mf_expert_offsets* offsets, const uint16_t* x,
                            const mf_pair* sorted_pairs, const uint32_t* expert_counts, uint32_t t,
                            float* route_partials, void* workspace, size_t workspace_bytes);
mf_status mf_moe_unpermute(mf_moe* h, mf_stream stream, const float* route_partials,
                           const float* route_weights, const uint32_t* idx, const uint16_t* residual,
                           uint32_t t, uint16_t* y);

#ifdef __cplusplus
}
#endif
#endif /* MFMOE_H */
