/*
 * mf_oracle — CPU restatement of Mference's MoE expert hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker for the HIP kernels:
 * only the test-suite, the smoke check and the benchmark's cpu_baseline leg may
 * load it.  The product library (libmfmoe) never links or calls it.
 *
 * Every function cites the reference file:line (relative to the Mference
 * repository root) whose semantics it restates.  Activations are bf16 bit
 * patterns (uint16_t); all accumulation is fp32 unless stated.
 *
 * Parity status of each function is listed in mf_oracle.c's header comment.
 */
#ifndef MF_ORACLE_H
#define MF_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* weight formats */
enum {
  MFO_BITS_TERNARY = 1, /* 2-bit codes {0,1,2}, scale only, bias = -scale */
  MFO_BITS_2 = 2,       /* 2-bit affine, 16 codes per uint32              */
  MFO_BITS_4 = 4,       /* 4-bit affine, 8 codes per uint32               */
  MFO_BITS_8 = 8        /* 8-bit affine (router / scalar gate in Gemma)    */
};

/* byte offsets of the nine sub-tensors inside one expert blob
 * (Sources/Mference/Kernels/MoE/MoE.swift:4-29, Metal/MoE/moe.metal:86-96) */
typedef struct {
  uint32_t gate_w, gate_s, gate_b;
  uint32_t up_w, up_s, up_b;
  uint32_t down_w, down_s, down_b;
} mfo_expert_offsets;

/* 16-byte route record (Kernels/Prefill/MoE/PrefillRouter.swift:4-28) */
typedef struct {
  uint32_t token, expert, rank, weight_bits;
} mfo_pair;

typedef struct { uint32_t expert, pair_start, pair_count; } mfo_group;
typedef struct { uint32_t group_start, group_count, pair_start, pair_count; } mfo_tile;

/* ---- bf16 -------------------------------------------------------------- */
uint16_t mfo_bf16_bits(float x);
float mfo_bf16_to_float(uint16_t bits);
void mfo_bf16_encode(const float* x, size_t n, uint16_t* out);
void mfo_bf16_decode(const uint16_t* x, size_t n, float* out);

/* ---- deterministic generators ------------------------------------------ */
typedef struct { uint64_t state; } mfo_rng;
mfo_rng mfo_rng_seed(uint64_t seed);
mfo_rng mfo_seed_tree_key(uint64_t root, const char* label);
uint64_t mfo_rng_next(mfo_rng* r);
float mfo_rng_uniform(mfo_rng* r, float lo, float hi);
/* Box-Muller over the uniform stream (this build's own; the reference has no
 * normal generator).  Fills n values of N(mean, sigma). */
void mfo_rng_normal(mfo_rng* r, float mean, float sigma, float* out, size_t n);
void mfo_rng_uniform_fill(mfo_rng* r, float lo, float hi, float* out, size_t n);

/* ---- quantization ------------------------------------------------------ */
size_t mfo_packed_row_bytes(int bits, size_t n);
/* rows x n fp32 -> packed codes + bf16 scale/bias per group of 64.
 * bits 4 / 8 follow the reference quantizer; bits 2 is this build's analogue
 * (parity unpinned for the 2-bit QUANTIZER, see mf_oracle.c). */
int mfo_quantize_affine(const float* w, size_t rows, size_t n, int bits,
                        uint8_t* packed, uint16_t* scales, uint16_t* biases);
/* ternary: codes[] in {0,1,2}; alpha per row-group given as fp32, rounded to bf16 */
int mfo_pack_codes(const uint8_t* codes, size_t rows, size_t n, int bits, uint8_t* packed);
int mfo_dequantize(const uint8_t* packed, const uint16_t* scales, const uint16_t* biases,
                   size_t rows, size_t n, int bits, float* out);

/* ---- router ------------------------------------------------------------ */
float mfo_exp(float x);
/* logits[e] = sum_i bf16(W[e,i]) * bf16(x[i]) in the fixed lane/tree order
 * documented in mf_oracle.c (bit-exact contract with the HIP kernel). */
void mfo_router_logits_bf16(const uint16_t* w, const uint16_t* x, size_t e, size_t d,
                            float* logits);
float mfo_dot_bf16_laneorder(const uint16_t* w, const uint16_t* x, size_t d);
/* serial insertion top-k + softmax over the selected (moe.metal:190-240) */
void mfo_topk_softmax(const float* logits, size_t e, size_t k, uint32_t* idx, float* w);
/* full softmax -> k x argmax -> renormalise (maple_moe.metal:62-119) */
void mfo_topk_full_softmax(const float* logits, size_t e, size_t k, uint32_t* idx, float* w);

/* ---- family routers (all share the tie rule of mfo_topk_softmax) -------- */
/* log(t) on [1,2] and sqrt(softplus(x)) (moe.metal:736-740), IEEE sequences shared with the kernels */
float mfo_log_1to2(float t);
float mfo_sqrtsoftplus(float x);
/* router_topk_select_sqrtsoftplus_k6 (moe.metal:744-786), k <= 8 */
void mfo_router_sqrtsoftplus(const float* logits, const float* correction_bias, size_t e, size_t k,
                             float route_scale, uint32_t* idx, float* w);
/* router_hash_weights_k6 (moe.metal:847-866), k <= 8 */
void mfo_router_hash_weights(const float* logits, const uint32_t* idx, size_t k, float route_scale,
                             float* w);
/* inkling_router_select (inkling.metal:503-566); logits [n_routed + n_shared] */
void mfo_router_inkling(const float* logits, const float* bias, float global_scale,
                        size_t n_routed, size_t n_shared, size_t k, float route_scale,
                        uint32_t* idx, float* w, float* gammas);
/* router_gemv_gemma4_body (moe.metal:102-139) in the build's fixed lane order */
float mfo_dot_int8_laneorder(const uint8_t* codes, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, const uint16_t* effective_scale, size_t d);
void mfo_router_logits_int8(const uint8_t* codes, const uint16_t* scales, const uint16_t* biases,
                            const uint16_t* x, const uint16_t* effective_scale, size_t e, size_t d,
                            float* logits);
/* router_topk_select_k8 incl. per_expert_scale (moe.metal:190-240) */
void mfo_topk_softmax_scaled(const float* logits, const uint16_t* per_expert_scale, size_t e, size_t k,
                             uint32_t* idx, float* w);

/* ---- GEMV / expert FFN ------------------------------------------------- */
/* y[m] = sum_n deq(W[m,n]) * x[n]; bulk dequant then sequential fp32 dot
 * (MferenceValidation/Support/Reference/Quant/DequantInt4Gemv.swift:26-40) */
int mfo_gemv(const uint8_t* packed, const uint16_t* scales, const uint16_t* biases,
             int bits, size_t m, size_t n, const float* x, float* y);
/* multi-token form: x [t,n] bf16 -> y [t,m] fp32 (dequant_int4.metal:356-446) */
int mfo_gemv_multix(const uint8_t* packed, const uint16_t* scales, const uint16_t* biases,
                    int bits, size_t m, size_t n, size_t t, const uint16_t* x, float* y);
float mfo_silu(float x);
/* routed phase 1: acts[f] = bf16(silu(clamp(gate.x)) * clamp(up.x)), fp32 gate/up
 * (moe.metal:499-529, clamp :27-34).  limit <= 0 disables the clamp. */
int mfo_gemv_group(const uint8_t* packed, const uint16_t* scales, const uint16_t* biases,
                   int bits, size_t m, size_t n, size_t group, const float* x, float* y);
int mfo_expert_phase1_gate(const uint8_t* blob, const mfo_expert_offsets* off, int bits,
                           size_t d, size_t f, size_t gate_group, float limit, int maple,
                           const uint16_t* x, uint16_t* acts);
int mfo_expert_phase1(const uint8_t* blob, const mfo_expert_offsets* off, int bits,
                      size_t d, size_t f, float swiglu_limit, int maple, const uint16_t* x,
                      uint16_t* acts);
/* int8_gelu_pytorch_tanh (dequant_int8.metal:44-49) with tanh(z) = 1 - 2 / (mfo_exp(2 z) + 1) */
float mfo_gelu_tanh(float x);
/* SharedExpertInt8.encode (SharedExpertInt8.swift:78-181; dequant_int8.metal:66-164) for one token row:
 * gate / up / down are 8-bit affine tensors [f,d], [f,d], [d,f] with bf16 tables per 64; rows are summed
 * in the lane order of mfo_dot_int8_laneorder; silu != 0 selects SiLU instead of the tanh GELU */
int mfo_shared_expert_int8(const uint8_t* gw, const uint16_t* gs, const uint16_t* gb, const uint8_t* uw,
                           const uint16_t* us, const uint16_t* ub, const uint8_t* dw, const uint16_t* ds,
                           const uint16_t* db, size_t d, size_t f, int silu, const uint16_t* x, uint16_t* y);
/* MapleMoE's activation, every intermediate narrowed to bf16 (maple_moe.metal:153-164);
 * selected in mfo_expert_phase1 by maple != 0 (swiglu_limit is ignored then) */
float mfo_maple_swiglu(float gate_projection, float up_projection);
/* v[d] = down . acts (fp32) (moe.metal:349-404) */
int mfo_expert_down(const uint8_t* blob, const mfo_expert_offsets* off, int bits,
                    size_t d, size_t f, const uint16_t* acts, float* v);
/* shared expert with the reference's extra narrowings
 * (dequant_int4.metal:216-246, :177-180): y = bf16(down . bf16(silu(bf16(g)) * bf16(u))) */
int mfo_shared_expert(const uint8_t* gw, const uint16_t* gs, const uint16_t* gb,
                      const uint8_t* uw, const uint16_t* us, const uint16_t* ub,
                      const uint8_t* dw, const uint16_t* ds, const uint16_t* db,
                      int bits, size_t d, size_t f, const uint16_t* x, uint16_t* y);
/* y[i] = bf16(y[i] / (1 + exp(-gate))) (utility.metal:49-59) */
void mfo_sigmoid_scalar_mul(uint16_t* y, size_t n, uint16_t gate_bits);

/* hidden += delta (delta may be NULL), then out = narrow(hidden * rsqrt(mean(hidden^2) + eps) * weight)
 * (utility.metal:83-92, rmsnorm.metal:30-92) */
void mfo_residual_rmsnorm(uint16_t* hidden, const uint16_t* delta, const uint16_t* weight,
                          uint16_t* out, size_t d, float eps);

typedef struct {
  size_t d, f, e, k;         /* hidden, routed intermediate, experts, top-k */
  size_t fs;                 /* shared intermediate (0 = no shared expert)  */
  int bits;                  /* routed expert format                        */
  int shared_bits;           /* shared expert format                        */
  int router_mode;           /* 0 = select on logits, softmax over selected */
                             /* 1 = full softmax, argmax, renormalise       */
  float swiglu_limit;        /* <= 0: none                                  */
  const uint16_t* router_w;  /* [e,d] bf16                                  */
  const uint8_t* experts;    /* e blobs, expert_stride bytes apart          */
  size_t expert_stride;
  mfo_expert_offsets off;
  const uint8_t* sgw; const uint16_t* sgs; const uint16_t* sgb; /* shared gate */
  const uint8_t* suw; const uint16_t* sus; const uint16_t* sub; /* shared up   */
  const uint8_t* sdw; const uint16_t* sds; const uint16_t* sdb; /* shared down */
  const uint16_t* w_sg;      /* [d] bf16 scalar shared gate, may be NULL    */
  int maple_rounding;        /* MapleMoE's activation and bf16 down outputs */
  int gate_group;            /* group of the routed gate tables: 0 / 64, or 32 */
  /* the scalar shared gate as an 8-bit affine row [1,d] (RealForwardRunner.swift:2925-2941,
   * dequant_int8.metal:66-107); used instead of w_sg when gqw != NULL */
  const uint8_t* gqw; const uint16_t* gqs; const uint16_t* gqb;
  /* a route's down output narrowed to a 16-bit number (bf16) before it meets its weight, the rule of the
   * reference's prefill kernels (prefill.metal:817-819 writes 16-bit route_partials, :644-651 reads them) */
  int narrow_routes;
} mfo_layer;

/* one token through router -> routed experts -> shared expert -> combine.
 * y = bf16(h1 + sum_k w_k v_k), rank order (moe.metal:1262-1270).
 * Optional outputs (may be NULL): idx[k], w[k], logits[e]. */
int mfo_moe_layer(const mfo_layer* L, const uint16_t* x, uint16_t* y,
                  uint32_t* idx, float* w, float* logits);
/* t tokens, each exactly as mfo_moe_layer (ragged == per-token invariant) */
int mfo_moe_layer_tokens(const mfo_layer* L, const uint16_t* x, size_t t, uint16_t* y,
                         uint32_t* idx, float* w, int threads);

/* ---- ragged grouping --------------------------------------------------- */
/* PrefillRouter.makeTokenExpertPairs (PrefillRouter.swift:91-111) */
void mfo_make_pairs(const uint32_t* idx, const uint32_t* weight_bits, size_t t, size_t k,
                    mfo_pair* out);
/* PrefillMoEGrouping.groupTokenExpertPairs (PrefillMoEGrouping.swift:91-192).
 * Returns 0 or a negative mfo error code mirroring PrefillMoEGroupingError. */
enum {
  MFO_ERR_QUERY_COUNT = -1, MFO_ERR_TOPK = -2, MFO_ERR_NUM_EXPERTS = -3,
  MFO_ERR_TILE_COUNT = -4, MFO_ERR_PAIR_COUNT = -5, MFO_ERR_TOKEN_RANGE = -6,
  MFO_ERR_RANK_RANGE = -7, MFO_ERR_EXPERT_RANGE = -8, MFO_ERR_DUPLICATE = -9,
  MFO_ERR_SORT_KEYS = -10, MFO_ERR_ARG = -20
};
int mfo_group_pairs(const mfo_pair* pairs, size_t n_pairs, int query_count, int top_k,
                    int num_experts, int tile_expert_count, const uint64_t* sort_keys,
                    size_t n_sort_keys, mfo_pair* sorted, uint32_t* offsets,
                    uint32_t* counts, mfo_group* groups, size_t* n_groups,
                    mfo_tile* tiles, size_t* n_tiles);
/* h2[t,d] = sum_r w[t,r] * partial[t,r,d], fma in rank order (prefill.metal:631-652) */
void mfo_reduce_token_major(const float* partials, const float* w, size_t t, size_t k,
                            size_t d, float* h2);

#ifdef __cplusplus
}
#endif
#endif
