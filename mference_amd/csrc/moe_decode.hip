// Routed expert decode: phase 1 (gate/up/activation), phase 2 (down + weighted
// rank-ordered reduce) as separate launches.  Experts are resident in HBM and
// addressed on device as expert_base + idx * expert_stride.
#include "mf_device.h"
#include "mf_internal.h"

#pragma clang fp contract(off)

namespace mf {

// Slots named directly instead of through expert indices: slot s of the call reads the blob at
// base + offsets[s] (base null: the table holds device addresses).  all_hit (optional): a device word
// that switches the launch off when zero (the reference's slot-map lookup found a routed expert
// missing from its slots, router_slot_lookup_k8, moe.metal:594-617).
struct SlotMap {
  const uint64_t* offsets;
  const uint32_t* all_hit;
};

struct BlobView {
  const uint8_t* gw; const uint16_t* gs; const uint16_t* gb;
  const uint8_t* uw; const uint16_t* us; const uint16_t* ub;
  const uint8_t* dw; const uint16_t* ds; const uint16_t* db;
};

__device__ __forceinline__ BlobView view_blob(const uint8_t* blob, const mf_expert_offsets& o) {
  BlobView v;
  v.gw = blob + o.gate_w;
  v.gs = reinterpret_cast<const uint16_t*>(blob + o.gate_s);
  v.gb = reinterpret_cast<const uint16_t*>(blob + o.gate_b);
  v.uw = blob + o.up_w;
  v.us = reinterpret_cast<const uint16_t*>(blob + o.up_s);
  v.ub = reinterpret_cast<const uint16_t*>(blob + o.up_b);
  v.dw = blob + o.down_w;
  v.ds = reinterpret_cast<const uint16_t*>(blob + o.down_s);
  v.db = reinterpret_cast<const uint16_t*>(blob + o.down_b);
  return v;
}

// acts[(t*K+k)*F + f] for every routed (token, slot): one lane group per row,
// gate and up rows share the x loads (moe_phase1_gate_up_act_u16load,
// moe.metal:499-583; 2-bit twin :966-1116; ternary maple_moe_phase1,
// maple_moe.metal:190-221; `maple` selects its bf16-stepped activation, :153-164).
// G32 (2-bit experts only): the gate projection's tables hold an entry per 32 weights
// (moe_int2_gate_up_rows_simd_dev_vec with gate_group_size 32, moe.metal:962-1060); up stays at 64.
template <int BITS, bool ALIGNED, bool G32 = false>
__global__ __launch_bounds__(256) void phase1_kernel(const uint8_t* __restrict__ base,
                                                     size_t stride, mf_expert_offsets off,
                                                     const uint32_t* __restrict__ idx,
                                                     const uint16_t* __restrict__ x,
                                                     uint32_t x_stride,
                                                     uint16_t* __restrict__ acts, uint32_t D,
                                                     uint32_t F, uint32_t E, uint32_t pairs,
                                                     uint32_t K, float limit, int maple,
                                                     uint32_t lpr_log2,
                                                     const uint32_t* __restrict__ subset,
                                                     uint32_t all_pairs, const SlotMap slots) {
  constexpr int EPL = Fmt<BITS>::kElemsPer16B;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const uint32_t lpr = 1u << lpr_log2;
  const uint32_t rpw = 64u >> lpr_log2;
  const uint32_t waves_per_pair = (F + rpw - 1) / rpw;
  uint32_t pair = wave / waves_per_pair;
  if (pair >= pairs) return;
  if (subset) {  // moe_phase1_gate_up_act_subset_u16load (moe.metal:531-565): only the listed slots
    pair = subset[pair];
    if (pair >= all_pairs) return;  // a slot past the table does nothing (:551)
  }
  const uint32_t row = (wave % waves_per_pair) * rpw + (lane >> lpr_log2);
  const uint32_t sub = lane & (lpr - 1);
  const bool row_ok = row < F;
  if (slots.all_hit && *slots.all_hit == 0u) return;  // guarded form: nothing unless every slot was found
  const uint8_t* blob;
  if (slots.offsets) {  // the slot's blob is named directly (moe_phase1_gate_up_act_slotmap, moe.metal:619-708)
    blob = base + slots.offsets[pair];
  } else {
    const uint32_t expert = idx[pair];
    if (expert >= E) {  // router sentinel: the slot contributes nothing
      if (row_ok && sub == 0) acts[static_cast<size_t>(pair) * F + row] = 0;
      return;
    }
    blob = base + static_cast<size_t>(expert) * stride;
  }
  const BlobView bv = view_blob(blob, off);
  const uint16_t* xt = x + static_cast<size_t>(pair / K) * x_stride;
  const uint32_t n_groups = D / kGroup;
  const size_t row_bytes = static_cast<size_t>(D) * Store<BITS>::kBits / 8;
  const size_t r = row_ok ? row : 0;
  float ga = 0.0f, ua = 0.0f;
  for (uint32_t e0 = sub * EPL; e0 < D; e0 += lpr * EPL) {
    if (!row_ok) break;
    const size_t boff = r * row_bytes + static_cast<size_t>(e0) * Store<BITS>::kBits / 8;
    const uint4 gc = load_codes16<ALIGNED>(bv.gw + boff);
    const uint4 uc = load_codes16<ALIGNED>(bv.uw + boff);
    float gs, gb, us, ub, gd, ud, sum, sum2;
    load_scale_bias<BITS>(bv.us + r * n_groups, bv.ub + r * n_groups, e0, us, ub);
    lane_dot<BITS, ALIGNED>(uc, xt + e0, ud, sum2);
    if constexpr (G32 && BITS == kBits2) {
      // the lane's 64 weights are two gate groups: entries e0 / 32 and e0 / 32 + 1 of a row of D / 32
      const uint16_t* gsr = bv.gs + r * (2 * n_groups) + e0 / 32;
      const uint16_t* gbr = bv.gb + r * (2 * n_groups) + e0 / 32;
      float hd[2], hs[2];
      lane_dot_halves_q2<ALIGNED>(gc, xt + e0, hd, hs);
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        ga = __builtin_fmaf(bf16_to_f(gsr[half]), hd[half], ga);
        ga = __builtin_fmaf(bf16_to_f(gbr[half]), hs[half], ga);
      }
      (void)gs; (void)gb; (void)gd; (void)sum;
    } else {
      load_scale_bias<BITS>(bv.gs + r * n_groups, bv.gb + r * n_groups, e0, gs, gb);
      lane_dot<BITS, ALIGNED>(gc, xt + e0, gd, sum);
      ga = __builtin_fmaf(gs, gd, ga);
      ga = __builtin_fmaf(gb, sum, ga);
    }
    ua = __builtin_fmaf(us, ud, ua);
    ua = __builtin_fmaf(ub, sum2, ua);
  }
  const float g = group_sum(ga, static_cast<int>(lpr));
  const float u = group_sum(ua, static_cast<int>(lpr));
  if (row_ok && sub == 0) acts[static_cast<size_t>(pair) * F + row] = routed_activation(g, u, limit, maple != 0);
}

// y[t,d] = bf16(residual[t,d] + sum_k w[t,k] * (down_k[d,:] . acts[t,k,:])):
// residual first, slots in rank order, product then add, one narrowing
// (moe_phase2_down_reduce_k8, moe.metal:1235-1271); with `maple` every expert's down output is a
// bf16 number before it meets its routing weight (maple_moe_phase2, maple_moe.metal:243-264).
template <int BITS, bool ALIGNED>
__global__ __launch_bounds__(256) void phase2_kernel(const uint8_t* __restrict__ base,
                                                     size_t stride, mf_expert_offsets off,
                                                     const uint32_t* __restrict__ idx,
                                                     const float* __restrict__ w,
                                                     const uint16_t* __restrict__ acts,
                                                     const uint16_t* __restrict__ residual,
                                                     uint16_t* __restrict__ y, uint32_t D,
                                                     uint32_t F, uint32_t E, uint32_t T,
                                                     uint32_t K, int maple, uint32_t lpr_log2,
                                                     const SlotMap slots) {
  constexpr int EPL = Fmt<BITS>::kElemsPer16B;
  if (slots.all_hit && *slots.all_hit == 0u) return;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const uint32_t lpr = 1u << lpr_log2;
  const uint32_t rpw = 64u >> lpr_log2;
  const uint32_t waves_per_tok = (D + rpw - 1) / rpw;
  const uint32_t tok = wave / waves_per_tok;
  if (tok >= T) return;
  const uint32_t row = (wave % waves_per_tok) * rpw + (lane >> lpr_log2);
  const uint32_t sub = lane & (lpr - 1);
  const bool row_ok = row < D;
  const size_t r = row_ok ? row : 0;
  const uint32_t n_groups = F / kGroup;
  const size_t row_bytes = static_cast<size_t>(F) * Store<BITS>::kBits / 8;
  float acc = residual ? bf16_to_f(residual[static_cast<size_t>(tok) * D + r]) : 0.0f;
  for (uint32_t k = 0; k < K; ++k) {
    const uint32_t pair = tok * K + k;
    const uint8_t* blob;
    if (slots.offsets) {
      blob = base + slots.offsets[pair];
    } else {
      const uint32_t expert = idx[pair];
      if (expert >= E) continue;
      blob = base + static_cast<size_t>(expert) * stride;
    }
    const BlobView bv = view_blob(blob, off);
    const uint16_t* a = acts + static_cast<size_t>(pair) * F;
    float part = 0.0f;
    for (uint32_t e0 = sub * EPL; e0 < F; e0 += lpr * EPL) {
      if (!row_ok) break;
      const uint4 dc = load_codes16<ALIGNED>(bv.dw + r * row_bytes +
                                             static_cast<size_t>(e0) * Store<BITS>::kBits / 8);
      float s, b, dot, sum;
      load_scale_bias<BITS>(bv.ds + r * n_groups, bv.db + r * n_groups, e0, s, b);
      lane_dot<BITS, ALIGNED>(dc, a + e0, dot, sum);
      part = __builtin_fmaf(s, dot, part);
      part = __builtin_fmaf(b, sum, part);
    }
    const float v = group_sum(part, static_cast<int>(lpr));
    const float weighted = w[pair] * (maple ? round_bf16(v) : v);
    acc = acc + weighted;
  }
  if (row_ok && sub == 0) y[static_cast<size_t>(tok) * D + row] = f_to_bf16(acc);
}

// router_slot_lookup_k8 (moe.metal:594-617): the slot of every routed expert from the caller's
// expert -> slot table (negative: not resident), as a byte offset into the slab, and whether all of
// them were found.  One workgroup; n routes.
__global__ __launch_bounds__(256) void slot_lookup_kernel(const uint32_t* __restrict__ idx,
                                                          const int16_t* __restrict__ slot_of, uint32_t n,
                                                          uint32_t E, uint64_t slot_stride,
                                                          uint64_t* __restrict__ out_offsets,
                                                          uint32_t* __restrict__ out_all_hit) {
  bool miss = false;
  for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
    const uint32_t e = min(idx[i], E - 1u);
    const int slot = slot_of[e];
    miss |= slot < 0;
    out_offsets[i] = slot < 0 ? 0ull : static_cast<uint64_t>(slot) * slot_stride;
  }
  const int any_miss = __syncthreads_or(miss ? 1 : 0);
  if (threadIdx.x == 0) *out_all_hit = any_miss ? 0u : 1u;
}

namespace {

bool blob_aligned(const void* base, size_t stride, const mf_expert_offsets& o) {
  const uint32_t all = o.gate_w | o.up_w | o.down_w;
  return aligned16(base) && (stride % 16 == 0) && (all % 16 == 0);
}

}  // namespace

hipError_t launch_phase1(hipStream_t s, const mf_moe_config& cfg, const void* base, size_t stride,
                         const mf_expert_offsets& off, const uint32_t* idx, const uint16_t* x,
                         uint32_t t, uint32_t x_stride, uint16_t* acts, const uint32_t* subset,
                         uint32_t n_subset, const uint64_t* slot_offsets, const uint32_t* all_hit) {
  const uint32_t all_pairs = t * cfg.top_k;
  const uint32_t pairs = subset ? n_subset : all_pairs;
  if (!pairs) return hipSuccess;
  // one wave per group of rows of a route: the count has to fit the 32-bit indexing of the kernel
  if (static_cast<uint64_t>(pairs) * cfg.f >= (1ull << 31)) return hipErrorInvalidValue;
  const bool al = blob_aligned(base, slot_offsets ? 0 : stride, off) && aligned16(x) && (x_stride % 8 == 0);
  const auto* b = static_cast<const uint8_t*>(base);
#define MF_P1(BITS, AL)                                                                          \
  {                                                                                              \
    const uint32_t lpr_log2 = lanes_per_row_log2(cfg.d, Fmt<BITS>::kElemsPer16B);                \
    const uint32_t rpw = 64u >> lpr_log2;                                                        \
    const uint32_t waves = pairs * ((cfg.f + rpw - 1) / rpw);                                    \
    phase1_kernel<BITS, AL><<<dim3((waves + 3) / 4), dim3(256), 0, s>>>(                         \
        b, stride, off, idx, x, x_stride, acts, cfg.d, cfg.f, cfg.num_experts, pairs, cfg.top_k, \
        cfg.swiglu_limit, static_cast<int>(cfg.maple_rounding), lpr_log2, subset, all_pairs,     \
        SlotMap{slot_offsets, all_hit});                                                         \
  }
  switch (cfg.bits) {
    case MF_BITS_4: if (al) MF_P1(kBits4, true) else MF_P1(kBits4, false) break;
    case MF_BITS_2:
      if (cfg.gate_group_size == 32) {
        const uint32_t lpr_log2 = lanes_per_row_log2(cfg.d, Fmt<kBits2>::kElemsPer16B);
        const uint32_t rpw = 64u >> lpr_log2;
        const uint32_t waves = pairs * ((cfg.f + rpw - 1) / rpw);
#define MF_P1G(AL)                                                                                  \
  phase1_kernel<kBits2, AL, true><<<dim3((waves + 3) / 4), dim3(256), 0, s>>>(                      \
      b, stride, off, idx, x, x_stride, acts, cfg.d, cfg.f, cfg.num_experts, pairs, cfg.top_k,      \
      cfg.swiglu_limit, static_cast<int>(cfg.maple_rounding), lpr_log2, subset, all_pairs,          \
      SlotMap{slot_offsets, all_hit})
        if (al) MF_P1G(true); else MF_P1G(false);
#undef MF_P1G
        break;
      }
      if (al) MF_P1(kBits2, true) else MF_P1(kBits2, false) break;
    case MF_BITS_TERNARY: if (al) MF_P1(kBitsTernary, true) else MF_P1(kBitsTernary, false) break;
    default: return hipErrorInvalidValue;
  }
#undef MF_P1
  return hipGetLastError();
}

hipError_t launch_slot_lookup(hipStream_t s, const uint32_t* idx, const int16_t* slot_of, uint32_t n_slots_in,
                              uint32_t num_experts, uint64_t slot_stride, uint64_t* out_offsets,
                              uint32_t* out_all_hit) {
  slot_lookup_kernel<<<dim3(1), dim3(256), 0, s>>>(idx, slot_of, n_slots_in, num_experts, slot_stride, out_offsets,
                                                   out_all_hit);
  return hipGetLastError();
}

hipError_t launch_phase2(hipStream_t s, const mf_moe_config& cfg, const void* base, size_t stride,
                         const mf_expert_offsets& off, const uint32_t* idx, const float* w,
                         const uint16_t* acts, const uint16_t* residual, uint32_t t, uint16_t* y,
                         const uint64_t* slot_offsets, const uint32_t* all_hit) {
  if (!t) return hipSuccess;
  if (static_cast<uint64_t>(t) * cfg.d >= (1ull << 31)) return hipErrorInvalidValue;  // 32-bit wave and row indices
  // (with a slot table the caller promises blobs on 16-byte boundaries; `stride` is not used)
  const bool al = blob_aligned(base, slot_offsets ? 0 : stride, off) && aligned16(acts);
  const auto* b = static_cast<const uint8_t*>(base);
#define MF_P2(BITS, AL)                                                                      \
  {                                                                                          \
    const uint32_t lpr_log2 = lanes_per_row_log2(cfg.f, Fmt<BITS>::kElemsPer16B);            \
    const uint32_t rpw = 64u >> lpr_log2;                                                    \
    const uint32_t waves = t * ((cfg.d + rpw - 1) / rpw);                                    \
    phase2_kernel<BITS, AL><<<dim3((waves + 3) / 4), dim3(256), 0, s>>>(                     \
        b, stride, off, idx, w, acts, residual, y, cfg.d, cfg.f, cfg.num_experts, t,         \
        cfg.top_k, static_cast<int>(cfg.maple_rounding), lpr_log2,                           \
        SlotMap{slot_offsets, all_hit});                                                     \
  }
  switch (cfg.bits) {
    case MF_BITS_4: if (al) MF_P2(kBits4, true) else MF_P2(kBits4, false) break;
    case MF_BITS_2: if (al) MF_P2(kBits2, true) else MF_P2(kBits2, false) break;
    case MF_BITS_TERNARY: if (al) MF_P2(kBitsTernary, true) else MF_P2(kBitsTernary, false) break;
    default: return hipErrorInvalidValue;
  }
#undef MF_P2
  return hipGetLastError();
}

}  // namespace mf
