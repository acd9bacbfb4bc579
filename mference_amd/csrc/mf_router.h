// Router device functions shared by the stand-alone router kernels and the
// fused decode layer: the fixed-order bf16 row dot and the one-wave top-k
// selectors.  Both are bit-exact against the CPU checker.
#pragma once

#include "mf_device.h"
#include "../../include/mfmoe.h"

#pragma clang fp contract(off)

namespace mf {

// One wave per (token, expert) row.  Elements are split into 8-wide chunks;
// chunk c belongs to lane c % 64; a lane accumulates its elements in ascending
// order with fmaf into one fp32 accumulator; lanes are combined by an xor
// butterfly with strides 1..32 (neighbours first).  Replaces router_gemv_bf16_r4
// (moe.metal:162-185) / maple_router_bf16_gemv (maple_moe.metal:25-60).
__device__ __forceinline__ float dot_bf16_row(const uint16_t* __restrict__ w,
                                              const uint16_t* __restrict__ x, uint32_t d,
                                              uint32_t lane, bool aligned) {
  float acc = 0.0f;
  const uint32_t chunks = d / 8;
  for (uint32_t c = lane; c < chunks; c += kWave) {
    uint4 wv, xv;
    if (aligned) {
      wv = load_x8<true>(w + c * 8);
      xv = load_x8<true>(x + c * 8);
    } else {
      wv = load_x8<false>(w + c * 8);
      xv = load_x8<false>(x + c * 8);
    }
    acc = __builtin_fmaf(bf16_lo(wv.x), bf16_lo(xv.x), acc);
    acc = __builtin_fmaf(bf16_hi(wv.x), bf16_hi(xv.x), acc);
    acc = __builtin_fmaf(bf16_lo(wv.y), bf16_lo(xv.y), acc);
    acc = __builtin_fmaf(bf16_hi(wv.y), bf16_hi(xv.y), acc);
    acc = __builtin_fmaf(bf16_lo(wv.z), bf16_lo(xv.z), acc);
    acc = __builtin_fmaf(bf16_hi(wv.z), bf16_hi(xv.z), acc);
    acc = __builtin_fmaf(bf16_lo(wv.w), bf16_lo(xv.w), acc);
    acc = __builtin_fmaf(bf16_hi(wv.w), bf16_hi(xv.w), acc);
  }
  return wave_sum(acc);
}

constexpr int kMaxPerLane = MF_MAX_EXPERTS / kWave;  // 8
constexpr uint32_t kNoWinner = 0xFFFFFFFFu;

// mode 0 selector, all-register form: lane l owns the PER consecutive experts
// from l*PER (the blocked ownership of router_topk_select_k8_par,
// moe.metal:262-345) and first sorts them by (score descending, index
// ascending).  Each of the k rounds takes the wave maximum of the lanes' heads;
// among the lanes whose head equals it the lowest lane wins and pops its head.
// Lower lane = lower index, so this is the serial kernel's "strictly greater
// wins, equal score keeps the earlier expert".  NaN and -inf are never selected;
// a round without a winner gives index 0, score -inf.  Rank r's result lives in
// lane r; weights are exp(s_r - s_0) / sum with the sum taken in rank order.
// All 64 lanes call it.
// MODE 1: lg holds probabilities of the full softmax; the weights are p_r / (sum + 1e-20)
// with the sum in rank order (maple_moe.metal:100-118).  MODE 2: lg holds selection scores of a
// family router, only the indices are written.
template <int PER, int MODE = 0>
__device__ __forceinline__ void topk_select_sorted(const float* lg, uint32_t e, uint32_t k,
                                                   uint32_t* idx, float* w, uint32_t lane) {
  const float ninf = -__builtin_inff();
  const uint32_t base = lane * PER;
  float v[PER];
  uint32_t id[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    id[j] = base + j;
    const float x = (base + j < e) ? lg[base + j] : ninf;
    v[j] = (x > ninf) ? x : ninf;  // NaN and -inf are not candidates
  }
  // odd-even transposition, swapping only on strictly smaller: stable
#pragma unroll
  for (int pass = 0; pass < PER; ++pass) {
#pragma unroll
    for (int a = pass & 1; a + 1 < PER; a += 2) {
      const bool sw = v[a] < v[a + 1];
      const float tv = sw ? v[a + 1] : v[a];
      const float bv = sw ? v[a] : v[a + 1];
      const uint32_t ti = sw ? id[a + 1] : id[a];
      const uint32_t bi = sw ? id[a] : id[a + 1];
      v[a] = tv; v[a + 1] = bv; id[a] = ti; id[a + 1] = bi;
    }
  }
  float my_score = ninf;
  uint32_t my_idx = 0;
  for (uint32_t r = 0; r < k; ++r) {
    const float m = wave_max(v[0]);
    const bool cand = v[0] == m && m > ninf;
    const unsigned long long mask = __ballot(cand);
    uint32_t widx = 0;
    float ws = ninf;
    if (mask != 0) {
      const int wl = __ffsll(static_cast<long long>(mask)) - 1;
      widx = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(id[0]), wl));
      ws = m;
      if (static_cast<int>(lane) == wl) {  // pop the head
#pragma unroll
        for (int j = 0; j + 1 < PER; ++j) {
          v[j] = v[j + 1];
          id[j] = id[j + 1];
        }
        v[PER - 1] = ninf;
      }
    }
    if (lane == r) {
      my_score = ws;
      my_idx = widx;
    }
  }
  if constexpr (MODE == 2) {  // indices only: the caller weighs them
    if (lane < k) idx[lane] = my_idx;
    return;
  }
  if constexpr (MODE == 1) {
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < MF_MAX_TOPK; ++i)
      if (static_cast<uint32_t>(i) < k) sum += readlane_f(my_score, i);
    if (lane < k) {
      idx[lane] = my_idx;
      w[lane] = my_score / (sum + 1.0e-20f);
    }
    return;
  }
  const float s0 = readlane_f(my_score, 0);
  const float my_e = mf_exp(my_score - s0);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < MF_MAX_TOPK; ++i)
    if (static_cast<uint32_t>(i) < k) sum += readlane_f(my_e, i);
  if (lane < k) {
    idx[lane] = my_idx;
    w[lane] = my_e / sum;
  }
}

// Full softmax over e logits in the reference's order (maple_moe.metal:62-99): maximum, then
// exp(l - max) summed as 32-wide blocks, each block by a 16,8,4,2,1 tree, the blocks added in
// order, + 1e-20; p written to `p` (may alias lg).  Returns false (nothing written) when a
// logit is not finite.  All 64 lanes call it; lg and p are read and written by this wave only.
__device__ __forceinline__ bool full_softmax_probs(const float* lg, float* p, uint32_t e,
                                                   uint32_t lane) {
  const uint32_t per = (e + kWave - 1) / kWave;
  float ch[kMaxPerLane];
  bool bad = false;
  float mx = -1.0e30f;
#pragma unroll
  for (int j = 0; j < kMaxPerLane; ++j) {
    const uint32_t x = lane + j * kWave;
    ch[j] = 0.0f;
    if (static_cast<uint32_t>(j) < per && x < e) {
      ch[j] = lg[x];
      if (!__builtin_isfinite(ch[j])) bad = true;
      if (ch[j] > mx) mx = ch[j];
    }
  }
  if (__any(bad)) return false;
  mx = wave_max(mx);
  float total = 0.0f;
#pragma unroll
  for (int j = 0; j < kMaxPerLane; ++j) {
    if (static_cast<uint32_t>(j) < per) {  // uniform: rows past the last expert cost nothing
      const uint32_t x = lane + j * kWave;
      const bool live = x < e;
      ch[j] = live ? mf_exp(ch[j] - mx) : 0.0f;
      float part = ch[j];
#pragma unroll
      for (int o = 16; o > 0; o >>= 1) part = part + __shfl_xor(part, o, kWave);
      const float lo = readlane_f(part, 0), hi = readlane_f(part, 32);
      if (static_cast<uint32_t>(2 * j) < e / 32) total += lo;
      if (static_cast<uint32_t>(2 * j + 1) < e / 32) total += hi;
    }
  }
  const float recip = 1.0f / (total + 1.0e-20f);
#pragma unroll
  for (int j = 0; j < kMaxPerLane; ++j) {
    const uint32_t x = lane + j * kWave;
    if (static_cast<uint32_t>(j) < per && x < e) p[x] = ch[j] * recip;
  }
  return true;
}

// mode 1 selector: full softmax, then k rounds of arg-max on the probabilities (strictly
// greater wins, so equal probabilities keep the lower index), renormalised.  `p` is scratch
// of e floats owned by this wave (LDS).  A non-finite logit gives indices = e, weights = 0.
__device__ __forceinline__ void topk_full_softmax_fast(const float* lg, float* p, uint32_t e,
                                                       uint32_t k, uint32_t* idx, float* w,
                                                       uint32_t lane) {
  if (!full_softmax_probs(lg, p, e, lane)) {
    if (lane < k) {
      idx[lane] = e;
      w[lane] = 0.0f;
    }
    return;
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): p is re-read by other lanes of this wave
  __builtin_amdgcn_wave_barrier();
  const uint32_t per = (e + kWave - 1) / kWave;
  if (per <= 1) topk_select_sorted<1, 1>(p, e, k, idx, w, lane);
  else if (per <= 2) topk_select_sorted<2, 1>(p, e, k, idx, w, lane);
  else if (per <= 4) topk_select_sorted<4, 1>(p, e, k, idx, w, lane);
  else topk_select_sorted<8, 1>(p, e, k, idx, w, lane);
}

__device__ __forceinline__ void topk_select_fast(const float* lg, uint32_t e, uint32_t k,
                                                 uint32_t* idx, float* w, uint32_t lane) {
  const uint32_t per = (e + kWave - 1) / kWave;
  if (per <= 1) topk_select_sorted<1>(lg, e, k, idx, w, lane);
  else if (per <= 2) topk_select_sorted<2>(lg, e, k, idx, w, lane);
  else if (per <= 4) topk_select_sorted<4>(lg, e, k, idx, w, lane);
  else topk_select_sorted<8>(lg, e, k, idx, w, lane);
}

// indices of the k best selection scores (same tie rule), for the family routers
__device__ __forceinline__ void topk_select_indices(const float* score, uint32_t e, uint32_t k,
                                                    uint32_t* idx, uint32_t lane) {
  const uint32_t per = (e + kWave - 1) / kWave;
  if (per <= 1) topk_select_sorted<1, 2>(score, e, k, idx, nullptr, lane);
  else if (per <= 2) topk_select_sorted<2, 2>(score, e, k, idx, nullptr, lane);
  else if (per <= 4) topk_select_sorted<4, 2>(score, e, k, idx, nullptr, lane);
  else topk_select_sorted<8, 2>(score, e, k, idx, nullptr, lane);
}

}  // namespace mf
