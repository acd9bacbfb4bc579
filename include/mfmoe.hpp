// mfmoe.hpp — C++ host-side mirror of Mference's Swift operator surface over the C ABI
// of libmfmoe (mfmoe.h).  Header only, C++17.
//
// The reference's host code is Swift: a set of operator classes under
// Sources/Mference/Kernels/ built from a MetalContext, whose encode…() methods append
// dispatches to a caller-owned MTLCommandBuffer and `throw` typed errors.  The classes below
// keep the reference's class and method names, argument order and error behaviour; a command
// buffer becomes a hipStream_t (passed as mf_stream), an (MTLBuffer, offset) pair becomes a
// device pointer (the caller adds the offset), `throws` becomes mf::Error carrying the
// mf_status.  Nothing here allocates device memory or touches the HIP runtime: every call
// goes straight to the C ABI.
#ifndef MFMOE_HPP
#define MFMOE_HPP

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "mfmoe.h"

namespace mf {

// `throws` of the reference (SharedExpertError, PrefillMoEGroupingError, MetalError, …):
// one exception type carrying the status code; detail[] holds the payload of the grouping
// errors (PrefillMoEGrouping.swift:52-88).
class Error : public std::runtime_error {
 public:
  Error(mf_status s, const std::string& what_arg, uint32_t d0 = 0, uint32_t d1 = 0)
      : std::runtime_error(what_arg), status(s), detail{d0, d1} {}
  mf_status status;
  uint32_t detail[2];
};

inline void check(mf_status s, const mf_ctx* ctx = nullptr) {
  if (s == MF_OK) return;
  std::string text = mf_status_string(s);
  if (s == MF_ERR_LAUNCH && ctx) text += std::string(": ") + mf_last_hip_error(ctx);
  throw Error(s, text);
}

// MetalContext (Infrastructure/Metal/MetalContext.swift:45-65): the device and its kernels.
class MetalContext {
 public:
  explicit MetalContext(int device = 0) { check(mf_ctx_create(device, &ctx_)); }
  ~MetalContext() { mf_ctx_destroy(ctx_); }
  MetalContext(const MetalContext&) = delete;
  MetalContext& operator=(const MetalContext&) = delete;
  mf_ctx* raw() const { return ctx_; }
  int computeUnits() const { return mf_ctx_num_cu(ctx_); }

 private:
  mf_ctx* ctx_ = nullptr;
};

// Quantization (Infrastructure/ModelIO/Quantization.swift:3-119), on device.
class Quantization {
 public:
  static constexpr int groupSize = MF_GROUP_SIZE;
  explicit Quantization(const MetalContext& context) : ctx_(context.raw()) {}
  // quantizeInt4Affine (:50-102) for every row of w; bits 4 or 2
  void quantizeInt4Affine(mf_stream stream, const float* w, size_t rows, size_t n, void* packed,
                          uint16_t* scales, uint16_t* biases, mf_bits bits = MF_BITS_4) const {
    check(mf_quantize_affine(ctx_, stream, w, rows, n, bits, packed, scales, biases), ctx_);
  }
  // dequantizeInt4Affine (:104-119)
  void dequantizeInt4Affine(mf_stream stream, mf_qtensor q, size_t rows, size_t n, float* out,
                            mf_bits bits = MF_BITS_4) const {
    check(mf_dequantize(ctx_, stream, q, rows, n, bits, out), ctx_);
  }

 private:
  mf_ctx* ctx_;
};

// DequantInt4GEMV (Kernels/Quant/DequantInt4GEMV.swift:57-103); any supported bit width.
class DequantInt4GEMV {
 public:
  explicit DequantInt4GEMV(const MetalContext& context, mf_bits bits = MF_BITS_4)
      : ctx_(context.raw()), bits_(bits) {}
  void encode(mf_stream commandBuffer, mf_qtensor weights, const uint16_t* x, void* y, uint32_t m,
              uint32_t n, bool outputFloat32 = false) const {
    check(mf_gemv(ctx_, commandBuffer, weights, bits_, x, y, m, n, 1, outputFloat32 ? 1 : 0), ctx_);
  }

 protected:
  mf_ctx* ctx_;
  mf_bits bits_;
};

// DequantInt4GEMVMultiX (Kernels/Quant/DequantInt4GEMVMultiX.swift:48-82): t <= 8 token rows.
class DequantInt4GEMVMultiX : public DequantInt4GEMV {
 public:
  static constexpr uint32_t maxTokens = MF_MAX_TOKENS;
  using DequantInt4GEMV::DequantInt4GEMV;
  void encode(mf_stream commandBuffer, mf_qtensor weights, const uint16_t* x, void* y, uint32_t m,
              uint32_t n, uint32_t t, bool outputFloat32 = false) const {
    check(mf_gemv(ctx_, commandBuffer, weights, bits_, x, y, m, n, t, outputFloat32 ? 1 : 0), ctx_);
  }
};

// Elementwise (Kernels/Primitives/Elementwise.swift:60-87)
class Elementwise {
 public:
  explicit Elementwise(const MetalContext& context) : ctx_(context.raw()) {}
  void encodeSiluMul(mf_stream cb, const uint16_t* gate, const uint16_t* up, uint16_t* out,
                     uint32_t count) const {
    check(mf_silu_mul(ctx_, cb, gate, up, out, count), ctx_);
  }
  void encodeSigmoidScalarMul(mf_stream cb, uint16_t* y, const uint16_t* gate, uint32_t count,
                              uint32_t rows = 1) const {
    check(mf_sigmoid_scalar_mul(ctx_, cb, y, gate, count, rows), ctx_);
  }
  void encodeResidualAdd(mf_stream cb, uint16_t* hidden, const uint16_t* delta, uint32_t count) const {
    check(mf_residual_add(ctx_, cb, hidden, delta, count), ctx_);
  }

 private:
  mf_ctx* ctx_;
};

// RMSNorm.encodeBF16W (Kernels/Primitives/RMSNorm.swift:52-64); `delta`, when given, is the residual
// add the runner issues in front of it (RealForwardRunner.swift:2799-2808), in the same launch
class RMSNorm {
 public:
  explicit RMSNorm(const MetalContext& context) : ctx_(context.raw()) {}
  void encodeBF16W(mf_stream cb, uint16_t* x, const uint16_t* weight, uint16_t* out, uint32_t d, float eps,
                   uint32_t t = 1, const uint16_t* delta = nullptr) const {
    check(mf_residual_rmsnorm(ctx_, cb, x, delta, weight, out, d, t, eps), ctx_);
  }

 private:
  mf_ctx* ctx_;
};

// The router calls of MoEDeepseekV4 (Kernels/MoE/MoEDeepseekV4.swift:92-151): learned top-k on
// sqrt(softplus(logit)) + correction bias, and weighting of hash-routed experts.  routeScale is the
// operator's constant as in the reference (:31-87); `logits` fp32 [tokens, numExperts] stands in for
// its internal routerLogits buffer.
class MoEDeepseekV4Router {
 public:
  MoEDeepseekV4Router(const MetalContext& context, float routeScale, uint32_t topK = 6)
      : ctx_(context.raw()), routeScale_(routeScale), topK_(topK) {}
  void encodeRouterTopK(mf_stream cb, const uint16_t* weights, const uint16_t* hidden,
                        const float* correctionBias, uint32_t* outIndices, float* outWeights,
                        uint32_t numExperts, uint32_t d, float* logits, uint32_t tokens = 1) const {
    check(mf_router_sqrtsoftplus(ctx_, cb, weights, hidden, tokens, d, numExperts, d, topK_, correctionBias,
                                 routeScale_, logits, outIndices, outWeights), ctx_);
  }
  void encodeRouterHashWeights(mf_stream cb, const uint16_t* weights, const uint16_t* hidden,
                               const uint32_t* indices, float* outWeights, uint32_t numExperts, uint32_t d,
                               float* logits, uint32_t tokens = 1) const {
    check(mf_router_hash_weights(ctx_, cb, weights, hidden, tokens, d, numExperts, d, topK_, indices,
                                 routeScale_, logits, outWeights), ctx_);
  }

 private:
  mf_ctx* ctx_;
  float routeScale_;
  uint32_t topK_;
};

// InklingKernels.encodeRouter / encodeRouterPrefill (Kernels/Inkling/InklingKernels.swift:377-476)
class InklingRouter {
 public:
  explicit InklingRouter(const MetalContext& context) : ctx_(context.raw()) {}
  void encodeRouter(mf_stream cb, const uint16_t* weights, const uint16_t* hidden, const float* gateBias,
                    const float* globalScale, uint32_t* outIndices, float* outWeights, float* gammasOut,
                    uint32_t numRouted, uint32_t numShared, uint32_t topK, float routeScale, uint32_t d,
                    float* logits, uint32_t tokens = 1) const {
    check(mf_router_inkling(ctx_, cb, weights, hidden, tokens, d, numRouted, numShared, d, topK, gateBias,
                            globalScale, routeScale, logits, outIndices, outWeights, gammasOut), ctx_);
  }

 private:
  mf_ctx* ctx_;
};

// MoE.encodeRouterGemma4 (Kernels/MoE/MoE.swift:153-202): 8-bit affine router rows
class Gemma4Router {
 public:
  explicit Gemma4Router(const MetalContext& context) : ctx_(context.raw()) {}
  void encodeRouterGemma4(mf_stream cb, const uint8_t* weights, const uint16_t* scales, const uint16_t* biases,
                          const uint16_t* hidden, const uint16_t* effectiveScale, const uint16_t* perExpertScale,
                          uint32_t* outIndices, float* outWeights, uint32_t numExperts, uint32_t d, uint32_t topK,
                          float* logits, uint32_t tokens = 1) const {
    check(mf_router_gemma4(ctx_, cb, weights, scales, biases, hidden, tokens, d, effectiveScale, perExpertScale,
                           numExperts, d, topK, logits, outIndices, outWeights), ctx_);
  }

 private:
  mf_ctx* ctx_;
};

// SharedExpertInt4 (Kernels/MoE/SharedExpertInt4.swift:70-165), also the dense SwiGLU MLP.
// Errors: MF_ERR_DIMENSION_MISMATCH / MF_ERR_SCRATCH_TOO_SMALL / MF_ERR_UNSUPPORTED_BITS are
// SharedExpertError.dimensionMismatch / .scratchTooSmall / .unsupportedWeightBits (:4-19).
class SharedExpertInt4 {
 public:
  explicit SharedExpertInt4(const MetalContext& context, mf_bits bits = MF_BITS_4)
      : ctx_(context.raw()), bits_(bits) {}
  void encode(mf_stream commandBuffer, const uint16_t* x, mf_qtensor gate, mf_qtensor up,
              mf_qtensor down, uint32_t d, uint32_t f, uint16_t* y, uint16_t* scratchAct,
              size_t scratchActBytes, uint32_t tokens = 1) const {
    check(mf_shared_expert(ctx_, commandBuffer, x, gate, up, down, bits_, d, f, tokens, y, scratchAct,
                           scratchActBytes), ctx_);
  }
  // scratch the block form (PrefillSharedExpert.encodeBlock, from 32 rows on) can use
  static size_t scratchBytes(uint32_t d, uint32_t f, uint32_t tokens) { return mf_shared_expert_scratch_bytes(d, f, tokens); }
  // the same operator without a scratch argument and without device allocation (the activations go
  // through a device array inside the library; tokens * f <= MF_STATIC_ACT_ELEMS, calls must not overlap)
  void encodeStatic(mf_stream commandBuffer, const uint16_t* x, mf_qtensor gate, mf_qtensor up, mf_qtensor down,
                    uint32_t d, uint32_t f, uint16_t* y, uint32_t tokens = 1) const {
    check(mf_shared_expert_static(ctx_, commandBuffer, x, gate, up, down, bits_, d, f, tokens, y), ctx_);
  }

 private:
  mf_ctx* ctx_;
  mf_bits bits_;
};

// SharedExpertInt8 (Kernels/MoE/SharedExpertInt8.swift:78-181): the dense MLP on 8-bit affine tensors; the
// activation is the tanh form of GELU, or SiLU with siluActivation
class SharedExpertInt8 {
 public:
  explicit SharedExpertInt8(const MetalContext& context, bool siluActivation = false)
      : ctx_(context.raw()), silu_(siluActivation) {}
  void encode(mf_stream commandBuffer, const uint16_t* x, mf_qtensor gate, mf_qtensor up, mf_qtensor down,
              uint32_t d, uint32_t f, uint16_t* y, uint16_t* scratchAct, size_t scratchActBytes,
              uint32_t tokens = 1) const {
    check(mf_shared_expert_int8(ctx_, commandBuffer, x, gate, up, down, d, f, tokens, silu_ ? 1 : 0, y, scratchAct,
                                scratchActBytes), ctx_);
  }

 private:
  mf_ctx* ctx_;
  bool silu_;
};

// MPPPrefillInt4QMM (Kernels/TensorCore/MPPPrefillInt4QMM.swift:34-78): y[m, n] = x[m, k] . deq(W[n, k])^T.
// encode returns the path like the reference: Unavailable for sizes or offsets it rejects.
class MPPPrefillInt4QMM {
 public:
  enum class Path { AffineMatrixCoreBF16, AffineRowsGEMV, Unavailable };
  static constexpr int tileM = 64, tileN = 32, tileK = MF_GROUP_SIZE;
  explicit MPPPrefillInt4QMM(const MetalContext& context, mf_bits bits = MF_BITS_4) : ctx_(context.raw()), bits_(bits) {}
  static size_t workspaceBytes(uint32_t m, uint32_t n, uint32_t k) { return mf_qmm_workspace_bytes(m, n, k); }
  Path encode(mf_stream commandBuffer, mf_qtensor weights, const uint16_t* x, void* y, uint32_t m, uint32_t n,
              uint32_t k, void* workspace, size_t workspaceBytes, bool outputFloat32 = false) const {
    const int path = mf_qmm_path(weights, bits_, x, y, m, n, k, workspace, workspaceBytes);
    if (path < 0) return Path::Unavailable;
    check(mf_qmm(ctx_, commandBuffer, weights, bits_, x, y, m, n, k, outputFloat32 ? 1 : 0, workspace, workspaceBytes),
          ctx_);
    return path == MF_QMM_PATH_MATRIX_CORE ? Path::AffineMatrixCoreBF16 : Path::AffineRowsGEMV;
  }

 private:
  mf_ctx* ctx_;
  mf_bits bits_;
};

using MoEExpertOffsets = mf_expert_offsets;  // Kernels/MoE/MoE.swift:4-29
// offsets, blob size and page-rounded stride of one routed expert in the repacker's blob order
// (RepackPlanner.swift:544-712, ModelExpertIO.swift:20-35)
inline MoEExpertOffsets expertBlobLayout(uint32_t d, uint32_t f, mf_bits bits, uint32_t align, size_t* blobBytes,
                                         size_t* stride) {
  MoEExpertOffsets off{};
  check(mf_expert_blob_layout(d, f, bits, align, &off, blobBytes, stride), nullptr);
  return off;
}

// MoE (Kernels/MoE/MoE.swift), MoEDeepseekV4 (2-bit, top-6) and MapleMoE (ternary, full-softmax
// router) in one class, selected by the configuration — the specialisation arguments of
// MoE.init (MoE.swift:65-151).  An instance owns its device workspace and is serial
// (MapleMoE.swift:3-6).
class MoE {
 public:
  MoE(const MetalContext& context, uint32_t specializedD, uint32_t specializedF,
      uint32_t specializedNumExperts, uint32_t specializedTopK = 8, mf_bits bits = MF_BITS_4,
      mf_router_mode routerMode = MF_ROUTER_TOPK_SOFTMAX, float swigluLimit = 0.0f,
      uint32_t sharedF = 0, mf_bits sharedBits = MF_BITS_4, bool mapleRounding = false,
      uint32_t gateGroupSize = 0)  // 32: MoEDeepseekV4.encodeRoutedPhase1(gateGroupSize:), MoEDeepseekV4.swift:199
      : ctx_(context.raw()) {
    cfg_ = mf_moe_config{specializedD, specializedF, specializedNumExperts, specializedTopK, bits,
                         routerMode,   swigluLimit,  sharedF,               sharedBits,
                         mapleRounding ? 1u : 0u, gateGroupSize};
    check(mf_moe_create(ctx_, &cfg_, &h_), ctx_);
  }
  ~MoE() { mf_moe_destroy(h_); }
  MoE(const MoE&) = delete;
  MoE& operator=(const MoE&) = delete;
  const mf_moe_config& config() const { return cfg_; }

  // encodeRouterGemma4 / encodeRouterTopK / encodeRouterTop8 (MoE.swift:153-203,
  // MoEDeepseekV4.swift:92-100, MapleMoE.swift:81-131)
  void encodeRouter(mf_stream cb, const uint16_t* weights, const uint16_t* hidden, uint32_t* outIndices,
                    float* outWeights, uint32_t queryCount = 1, float* outLogits = nullptr) const {
    check(mf_moe_router(h_, cb, weights, hidden, queryCount, cfg_.d, outIndices, outWeights, outLogits),
          ctx_);
  }
  // encodeRoutedPersistentPhase1U16Load (MoE.swift:220-253)
  void encodeRoutedPersistentPhase1U16Load(mf_stream cb, const void* experts, size_t expertStride,
                                           const MoEExpertOffsets& routedOffsets, const uint32_t* indices,
                                           const uint16_t* x, uint16_t* acts, uint32_t tokens = 1) const {
    check(mf_moe_phase1(h_, cb, experts, expertStride, &routedOffsets, indices, x, tokens, cfg_.d, acts),
          ctx_);
  }
  // encodeRoutedPersistentPhase1SubsetU16Load (MoE.swift:255-298): only the listed slots
  void encodeRoutedPersistentPhase1SubsetU16Load(mf_stream cb, const void* experts, size_t expertStride,
                                                 const MoEExpertOffsets& routedOffsets, const uint32_t* indices,
                                                 const uint16_t* x, uint16_t* acts, const uint32_t* activeSlots,
                                                 uint32_t activeCount, uint32_t tokens = 1) const {
    check(mf_moe_phase1_subset(h_, cb, experts, expertStride, &routedOffsets, indices, x, tokens, cfg_.d, acts,
                               activeSlots, activeCount), ctx_);
  }
  // encodeRoutedPersistentPhase2Reduce (MoE.swift:400-440)
  void encodeRoutedPersistentPhase2Reduce(mf_stream cb, const void* experts, size_t expertStride,
                                          const MoEExpertOffsets& routedOffsets, const uint32_t* indices,
                                          const float* routingWeights, const uint16_t* acts,
                                          const uint16_t* residual, uint16_t* y, uint32_t tokens = 1) const {
    check(mf_moe_phase2(h_, cb, experts, expertStride, &routedOffsets, indices, routingWeights, acts,
                        residual, tokens, y), ctx_);
  }
  // the whole decode layer in one launch (RealForwardRunner.swift:2811-3218 steps, no readback)
  void encodeDecodeLayer(mf_stream cb, const mf_moe_layer_weights& weights, const uint16_t* x,
                         uint16_t* y, uint32_t tokens = 1, uint16_t* hidden = nullptr,
                         uint32_t* outIndices = nullptr, float* outWeights = nullptr) const {
    check(mf_moe_decode_layer(h_, cb, &weights, x, tokens, y, hidden, outIndices, outWeights), ctx_);
  }
  // router_slot_lookup_k8 + encodeSlotMapGuardedFFN's two routed launches (MoE.swift:333-407), and the
  // routed-argument-buffer forms (MoE.swift:205-253, 409-440: slab == nullptr, the table holds addresses)
  void encodeSlotLookup(mf_stream cb, const uint32_t* indices, const int16_t* slotOf, uint64_t slotStride,
                        uint64_t* outSlotOffsets, uint32_t* outAllHit, uint32_t tokens = 1) const {
    check(mf_moe_slot_lookup(h_, cb, indices, tokens, slotOf, slotStride, outSlotOffsets, outAllHit), ctx_);
  }
  void encodeRoutedPhase1Slots(mf_stream cb, const void* slab, const uint64_t* slotOffsets, const uint32_t* allHit,
                               const MoEExpertOffsets& routedOffsets, const uint16_t* x, uint16_t* acts,
                               uint32_t tokens = 1) const {
    check(mf_moe_phase1_slots(h_, cb, slab, slotOffsets, allHit, &routedOffsets, x, tokens, cfg_.d, acts), ctx_);
  }
  void encodeRoutedPhase2ReduceSlots(mf_stream cb, const void* slab, const uint64_t* slotOffsets,
                                     const uint32_t* allHit, const MoEExpertOffsets& routedOffsets,
                                     const float* routingWeights, const uint16_t* acts, const uint16_t* residual,
                                     uint16_t* y, uint32_t tokens = 1) const {
    check(mf_moe_phase2_slots(h_, cb, slab, slotOffsets, allHit, &routedOffsets, routingWeights, acts, residual,
                              tokens, y), ctx_);
  }
  // PrefillGroupedRoutedMoE.encodeStreamedBatched + PrefillMoE.encodeReduceTokenMajor +
  // PrefillSharedExpert.encodeBlock (PrefillGroupedRoutedMoE.swift:392-466, PrefillMoE.swift:11-38,
  // PrefillSharedExpert.swift:81-99) for `tokens` rows
  size_t prefillWorkspaceBytes(uint32_t tokens) const { return mf_moe_prefill_workspace_bytes(h_, tokens); }
  void encodePrefillLayer(mf_stream cb, const mf_moe_layer_weights& weights, const uint16_t* x,
                          uint16_t* y, uint32_t tokens, void* workspace, size_t workspaceBytes,
                          uint32_t* outIndices = nullptr, float* outWeights = nullptr) const {
    check(mf_moe_prefill_layer(h_, cb, &weights, x, tokens, y, workspace, workspaceBytes, outIndices,
                               outWeights), ctx_);
  }
  // PrefillRouter.makeTokenExpertPairs + PrefillMoEGrouping.groupTokenExpertPairs on device
  void encodeGroup(mf_stream cb, const uint32_t* indices, const float* routingWeights, uint32_t tokens,
                   mf_pair* sortedPairs, uint32_t* expertOffsets, uint32_t* expertCounts) const {
    check(mf_moe_group(h_, cb, indices, routingWeights, tokens, sortedPairs, expertOffsets, expertCounts),
          ctx_);
  }
  void groupStatus(mf_stream cb) const { check(mf_moe_group_status(h_, cb), ctx_); }
  // PrefillGroupedRoutedMoE.encodeStreamedBatched (PrefillGroupedRoutedMoE.swift:392-466) over a
  // grouping the caller holds; routePartials is fp32 [tokens * topK, d], row token * topK + rank
  void encodeStreamedBatched(mf_stream cb, const void* expertBase, size_t expertStride,
                             const mf_expert_offsets& offsets, const uint16_t* hidden,
                             const mf_pair* sortedPairs, const uint32_t* expertCounts, uint32_t tokens,
                             float* routePartials, void* workspace, size_t workspaceBytes) const {
    check(mf_moe_ragged_qmm(h_, cb, expertBase, expertStride, &offsets, hidden, sortedPairs, expertCounts,
                            tokens, routePartials, workspace, workspaceBytes), ctx_);
  }
  // PrefillMoE.encodeReduceTokenMajor (PrefillMoE.swift:11-38)
  void encodeReduceTokenMajor(mf_stream cb, const float* routePartials, const float* routeWeights,
                              uint16_t* h2, uint32_t tokens, const uint32_t* indices = nullptr,
                              const uint16_t* residual = nullptr) const {
    check(mf_moe_unpermute(h_, cb, routePartials, routeWeights, indices, residual, tokens, h2), ctx_);
  }
  // the residual add and RMSNorm in front of the layer, the layer and the residual add behind it in one call
  void encodeDecodeLayerNormed(mf_stream cb, const mf_moe_layer_weights& weights, uint16_t* hidden, const uint16_t* delta,
                               const uint16_t* normWeight, float eps, uint16_t* y, uint32_t tokens = 1,
                               uint32_t* outIndices = nullptr, float* outWeights = nullptr) const {
    check(mf_moe_decode_layer_normed(h_, cb, &weights, hidden, delta, normWeight, eps, tokens, y, outIndices, outWeights), ctx_);
  }
  void setFused(bool enabled) const { check(mf_moe_set_fused(h_, enabled ? 1 : 0), ctx_); }
  // a copy of the expert pool in the prefill matmul's own order (mf_moe_layer_weights.expert_tiled)
  void tileExperts(mf_stream cb, const void* expertBase, size_t expertStride, const mf_expert_offsets& offsets,
                   void* tiled) const {
    check(mf_moe_tile_experts(h_, cb, expertBase, expertStride, &offsets, tiled), ctx_);
  }
  void setPrefillRouteRounding(bool narrow) const { check(mf_moe_set_prefill_route_rounding(h_, narrow ? 1 : 0), ctx_); }
  void status(mf_stream cb) const { check(mf_moe_status(h_, cb), ctx_); }

 private:
  mf_ctx* ctx_;
  mf_moe_config cfg_{};
  mf_moe* h_ = nullptr;
};

// PrefillTokenExpertPair (Kernels/Prefill/MoE/PrefillRouter.swift:4-28)
using PrefillTokenExpertPair = mf_pair;

// PrefillMoEGroupedRoutes (PrefillMoEGrouping.swift:3-50)
struct PrefillMoEGroupedRoutes {
  std::vector<PrefillTokenExpertPair> sortedPairs;
  std::vector<uint32_t> expertOffsets, expertCounts;
  std::vector<mf_group> groups;
  std::vector<mf_tile> tiles;
  uint32_t maxPairsPerExpert() const {
    uint32_t m = 0;
    for (const auto& g : groups) m = g.pair_count > m ? g.pair_count : m;
    return m;
  }
  uint32_t maxPairsPerTile() const {
    uint32_t m = 0;
    for (const auto& t : tiles) m = t.pair_count > m ? t.pair_count : m;
    return m;
  }
};

// PrefillMoEGrouping (Kernels/Prefill/MoE/PrefillMoEGrouping.swift:91-192), host side.
struct PrefillMoEGrouping {
  // makeTokenExpertPairs (PrefillRouter.swift:91-111): token-major (token, rank) records
  static std::vector<PrefillTokenExpertPair> makeTokenExpertPairs(const uint32_t* indices,
                                                                  const uint32_t* weightBits,
                                                                  uint32_t queryCount, uint32_t topK) {
    std::vector<PrefillTokenExpertPair> pairs(static_cast<size_t>(queryCount) * topK);
    for (uint32_t t = 0; t < queryCount; ++t)
      for (uint32_t r = 0; r < topK; ++r) {
        const size_t i = static_cast<size_t>(t) * topK + r;
        pairs[i] = PrefillTokenExpertPair{t, indices[i], r, weightBits[i]};
      }
    return pairs;
  }
  // groupTokenExpertPairs; throws mf::Error with the PrefillMoEGroupingError case as status
  static PrefillMoEGroupedRoutes groupTokenExpertPairs(const std::vector<PrefillTokenExpertPair>& pairs,
                                                       int queryCount, int topK, int numExperts,
                                                       int tileExpertCount = 16,
                                                       const std::vector<uint64_t>* sortKeys = nullptr) {
    PrefillMoEGroupedRoutes r;
    const size_t ne = numExperts > 0 ? static_cast<size_t>(numExperts) : 1;
    const size_t cap = pairs.size() < ne ? (pairs.empty() ? 1 : pairs.size()) : ne;
    r.sortedPairs.resize(pairs.size());
    r.expertOffsets.resize(ne);
    r.expertCounts.resize(ne);
    r.groups.resize(cap);
    r.tiles.resize(cap);
    size_t ng = 0, nt = 0;
    uint32_t detail[2] = {0, 0};
    const mf_status s = mf_group_pairs_host(
        pairs.data(), pairs.size(), queryCount, topK, numExperts, tileExpertCount,
        sortKeys ? sortKeys->data() : nullptr, sortKeys ? sortKeys->size() : 0, r.sortedPairs.data(),
        r.expertOffsets.data(), r.expertCounts.data(), r.groups.data(), &ng, r.tiles.data(), &nt, detail);
    if (s != MF_OK) throw Error(s, mf_status_string(s), detail[0], detail[1]);
    r.groups.resize(ng);
    r.tiles.resize(nt);
    return r;
  }
};

}  // namespace mf

#endif  // MFMOE_HPP
