// Host-side state and kernel launchers behind the C ABI (include/mfmoe.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/mfmoe.h"

struct mf_ctx {
  int device = 0;
  int num_cu = 0;
  char hip_error[256] = {0};
};

// Per-operator device workspace (the routerLogits buffer and argument table the
// reference's MoE class owns, MoE.swift:136-150).
struct mf_moe_workspace {
  float* logits;        // [256, num_experts]: MF_MAX_TOKENS rows for the decode calls, 256 for mf_moe_router
  uint32_t* idx;        // [MF_MAX_TOKENS, top_k]
  float* w;             // [MF_MAX_TOKENS, top_k]
  uint16_t* acts;       // [MF_MAX_TOKENS, top_k, f]
  uint16_t* shared_act; // [MF_MAX_TOKENS, shared_f]
  uint16_t* shared_y;   // [MF_MAX_TOKENS, d]
  uint16_t* gate;       // [MF_MAX_TOKENS]
  uint16_t* xn;         // [MF_MAX_TOKENS, d]: the normalised rows of mf_moe_decode_layer_normed when it takes two launches
  // exchange buffers of the fused launch: every word carries an epoch tag
  unsigned long long* t_logits;  // [MF_MAX_TOKENS, num_experts]
  uint32_t* t_sact;              // [MF_MAX_TOKENS, shared_f]
  uint32_t* t_acts;              // [MF_MAX_TOKENS, top_k, f]
  uint32_t* epoch;               // [512] one launch counter per workgroup
  uint32_t* status;              // non-zero once a bounded wait gave up
  uint32_t* group_tmp;           // grouping scratch: [512, 1024) starts, [1536] status word, [2048, ...) per-chunk counts,
                                 // flags, and the per-chunk route words and count bytes of the prefill layer call
};

struct mf_moe {
  mf_ctx* ctx = nullptr;
  mf_moe_config cfg{};
  bool fused = true;  // mf_moe_set_fused
  bool generic_shape = false;  // mf_moe_set_fused(h, 2): the fused launch through the instance that reads every dimension from its arguments
  bool narrow_routes = false;  // mf_moe_set_prefill_route_rounding
  unsigned long long* trace = nullptr;  // mf_moe_set_phase_trace
  size_t trace_bytes = 0;
  void* ws_base = nullptr;
  size_t ws_bytes = 0;
  mf_moe_workspace ws{};
};

namespace mf {

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned2(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 1u) == 0; }

// lanes of a wave that share one row of n elements (power of two, <= 64)
inline uint32_t lanes_per_row_log2(uint32_t n, int elems_per_lane) {
  uint32_t need = (n + elems_per_lane - 1) / elems_per_lane;
  uint32_t l = 0;
  while ((1u << l) < need && l < 6) ++l;
  return l;
}

// format.hip
hipError_t launch_quantize(hipStream_t s, const float* w, size_t rows, size_t n, int bits,
                           void* packed, uint16_t* scales, uint16_t* biases);
hipError_t launch_dequantize(hipStream_t s, const mf_qtensor& q, size_t rows, size_t n, int bits,
                             float* out);

// gemv.hip
// `lane_order`: keep the per-row lane partition of gemv_kernel (the fused decode kernel sums in
// that order; the chain of separate launches of a decode layer asks for it so that both give
// the same bits).  Without it wide matrices may take the matrix-core kernels, whose sums differ
// in the last bits.
hipError_t launch_gemv(hipStream_t s, const mf_qtensor& w, int bits, const uint16_t* x, void* y,
                       uint32_t m, uint32_t n, uint32_t t, bool out_f32, bool lane_order = false);
hipError_t launch_gate_up_act(hipStream_t s, const mf_qtensor& gate, const mf_qtensor& up,
                              int bits, const uint16_t* x, uint16_t* act, uint32_t f, uint32_t d,
                              uint32_t t, bool lane_order = false);
hipError_t launch_gate_up_act_q8(hipStream_t s, const mf_qtensor& gate, const mf_qtensor& up, const uint16_t* x,
                                 uint16_t* act, uint32_t f, uint32_t d, uint32_t t, bool silu);
hipError_t launch_residual_rmsnorm(hipStream_t s, uint16_t* hidden, const uint16_t* delta,
                                   const uint16_t* weight, uint16_t* out, uint32_t d, uint32_t t, float eps);
hipError_t launch_silu_mul(hipStream_t s, const uint16_t* gate, const uint16_t* up, uint16_t* out,
                           uint32_t count);
hipError_t launch_sigmoid_scalar_mul(hipStream_t s, uint16_t* y, const uint16_t* gate,
                                     uint32_t row, uint32_t rows);
hipError_t launch_residual_add(hipStream_t s, uint16_t* hidden, const uint16_t* delta,
                               uint32_t count);

// router.hip
hipError_t launch_router_logits(hipStream_t s, const uint16_t* w, const uint16_t* x, uint32_t e,
                                uint32_t d, uint32_t t, uint32_t x_stride, float* logits,
                                uint16_t* logits_bf16);
hipError_t launch_topk(hipStream_t s, const float* logits, uint32_t e, uint32_t k, uint32_t t,
                       int mode, uint32_t* idx, float* w);

// router_family.hip
hipError_t launch_router_logits_int8(hipStream_t s, const uint8_t* codes, const uint16_t* scales,
                                     const uint16_t* biases, const uint16_t* x, const uint16_t* eff,
                                     uint32_t e, uint32_t d, uint32_t t, uint32_t x_stride, float* logits);
hipError_t launch_select_sqrtsoftplus(hipStream_t s, const float* logits, const float* bias, uint32_t e,
                                      uint32_t k, uint32_t t, float route_scale, uint32_t* idx, float* w);
hipError_t launch_hash_weights(hipStream_t s, const float* logits, const uint32_t* given, uint32_t e,
                               uint32_t k, uint32_t t, float route_scale, float* w);
hipError_t launch_select_inkling(hipStream_t s, const float* logits, const float* bias,
                                 const float* global_scale, uint32_t n_routed, uint32_t n_shared, uint32_t k,
                                 uint32_t t, float route_scale, uint32_t* idx, float* w, float* gammas);
hipError_t launch_select_scaled_softmax(hipStream_t s, const float* logits, const uint16_t* expert_scale,
                                        uint32_t e, uint32_t k, uint32_t t, uint32_t* idx, float* w);

// static_scratch.hip: this device's address of the library's built-in scratch array (device = current device)
hipError_t static_scratch_init(int device);

// moe_decode.hip
hipError_t launch_phase1(hipStream_t s, const mf_moe_config& cfg, const void* base, size_t stride,
                         const mf_expert_offsets& off, const uint32_t* idx, const uint16_t* x,
                         uint32_t t, uint32_t x_stride, uint16_t* acts, const uint32_t* subset = nullptr,
                         uint32_t n_subset = 0, const uint64_t* slot_offsets = nullptr,
                         const uint32_t* all_hit = nullptr);
hipError_t launch_phase2(hipStream_t s, const mf_moe_config& cfg, const void* base, size_t stride,
                         const mf_expert_offsets& off, const uint32_t* idx, const float* w,
                         const uint16_t* acts, const uint16_t* residual, uint32_t t, uint16_t* y,
                         const uint64_t* slot_offsets = nullptr, const uint32_t* all_hit = nullptr);
hipError_t launch_slot_lookup(hipStream_t s, const uint32_t* idx, const int16_t* slot_of, uint32_t n_slots_in,
                              uint32_t num_experts, uint64_t slot_stride, uint64_t* out_offsets,
                              uint32_t* out_all_hit);


// moe_fused.hip
bool fused_supported(const mf_moe& h, const mf_moe_layer_weights& w, const void* x, const void* y,
                     const void* hidden, uint32_t t);
// the step in front of the layer made inside the fused launch (hidden += delta, x = RMSNorm(hidden) * weight)
struct FusedNorm {
  const uint16_t* delta;   // [t, d] or null
  const uint16_t* weight;  // [d]
  float eps;
};
bool fused_norm_supported(const mf_moe& h, const mf_moe_layer_weights& w, const void* y, const void* hidden,
                          const void* delta, const void* norm_w, uint32_t t);
hipError_t launch_fused_decode(hipStream_t s, const mf_moe& h, const mf_moe_layer_weights& w,
                               const uint16_t* x, uint32_t t, uint16_t* y, uint16_t* hidden,
                               uint32_t* out_idx, float* out_w, const FusedNorm* norm = nullptr);

}  // namespace mf

// moe_prefill.hip
namespace mf {
hipError_t launch_group(hipStream_t s, const uint32_t* idx, const float* w, uint32_t t, uint32_t K,
                        uint32_t E, uint32_t* counts, uint32_t* offsets, uint32_t* starts,
                        mf_pair* sorted, void* tiles, uint32_t tile_slots, uint32_t* n_tiles,
                        uint32_t* status, uint32_t* chunk_hist);
size_t group_scratch_words();
size_t prefill_workspace_bytes(const mf_moe_config& c, uint32_t t);
hipError_t launch_tile_experts(hipStream_t s, const mf_moe_config& c, const void* src, size_t expert_stride,
                               const mf_expert_offsets& off, void* dst);
bool prefill_supported(const mf_moe_config& c);
hipError_t launch_prefill_layer(hipStream_t s, const mf_moe& h, const mf_moe_layer_weights& w,
                                const uint16_t* x, uint32_t t, uint16_t* y, void* workspace,
                                uint32_t* out_idx, float* out_w);
hipError_t launch_ragged_qmm(hipStream_t s, const mf_moe& h, const void* expert_base, size_t expert_stride,
                             const mf_expert_offsets& off, const uint16_t* x, const mf_pair* sorted,
                             const uint32_t* counts, uint32_t t, float* partials, void* workspace);
hipError_t launch_unpermute(hipStream_t s, const mf_moe_config& c, const float* partials, const float* w,
                            const uint32_t* idx, const uint16_t* residual, uint32_t t, uint16_t* y);
// dense projections over many rows through the matrix-core matmul (moe_prefill.hip)
bool dense_qmm_takes(const mf_qtensor& w, int bits, const void* x, const void* y, uint32_t m, uint32_t n, uint32_t k);
size_t dense_qmm_workspace_bytes(uint32_t m, uint32_t n, uint32_t k);
hipError_t launch_dense_qmm(hipStream_t s, const mf_qtensor& w, int bits, const uint16_t* x, void* y, uint32_t m,
                            uint32_t n, uint32_t k, bool out_f32, void* workspace);
bool dense_mlp_takes(const mf_qtensor& gate, const mf_qtensor& up, const mf_qtensor& down, const void* x,
                     const void* y, const void* scratch, uint32_t d, uint32_t f, uint32_t t);
size_t dense_mlp_scratch_bytes(uint32_t d, uint32_t f, uint32_t t);
hipError_t launch_dense_mlp(hipStream_t s, const mf_qtensor& gate, const mf_qtensor& up, const mf_qtensor& down,
                            int bits, const uint16_t* x, uint16_t* y, uint32_t d, uint32_t f, uint32_t t, void* scratch);
hipError_t launch_prefill_router(hipStream_t s, const uint16_t* W, const uint16_t* x, uint32_t E,
                                 uint32_t D, uint32_t T, uint32_t x_stride, float* logits);
}  // namespace mf
