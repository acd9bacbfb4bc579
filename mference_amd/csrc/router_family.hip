// Family-specific routers: DeepSeek-V4 sqrtsoftplus selection and hash weighting, the Inkling
// sigmoid router with shared sinks, and Gemma's 8-bit affine router rows with per-expert scales.
// All share the tie rule of the plain top-k selector and are bit-exact against the CPU checker:
// exp, log and the summation orders are fixed IEEE sequences, divide and sqrt are correctly rounded.
#include "mf_device.h"
#include "mf_internal.h"
#include "mf_router.h"

#include <algorithm>

#pragma clang fp contract(off)

namespace mf {

namespace {

// One wave per (token, expert) row of router_gemv_gemma4_body (moe.metal:102-139).  8-wide chunks
// are dealt to the 64 lanes; a chunk lies inside one group of 64, its sum q*x' and sum x' are built
// in ascending order from 0 and enter the lane's accumulator as fma(s, dot, acc), fma(b, sum, acc);
// x' = x * effective_scale is exact in fp32 for bf16 factors.
__global__ __launch_bounds__(256) void router_logits_int8_kernel(
    const uint8_t* __restrict__ codes, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ x,
    const uint16_t* __restrict__ eff, uint32_t e, uint32_t d, uint32_t t, uint32_t x_stride,
    float* __restrict__ logits, int aligned) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (wave >= e * t) return;
  const uint32_t tok = wave / e, row = wave % e;
  const uint8_t* q_row = codes + static_cast<size_t>(row) * d;
  const uint16_t* s_row = scales + static_cast<size_t>(row) * (d / MF_GROUP_SIZE);
  const uint16_t* b_row = biases + static_cast<size_t>(row) * (d / MF_GROUP_SIZE);
  const uint16_t* x_row = x + static_cast<size_t>(tok) * x_stride;
  float acc = 0.0f;
  for (uint32_t c = lane; c < d / 8; c += kWave) {
    uint32_t q[2];
    uint4 xv, ev;
    if (aligned) {
      const uint2 qq = *reinterpret_cast<const uint2*>(q_row + c * 8);
      q[0] = qq.x; q[1] = qq.y;
      xv = load_x8<true>(x_row + c * 8);
      ev = load_x8<true>(eff + c * 8);
    } else {
      const uint8_t* p = q_row + c * 8;
      q[0] = p[0] | (p[1] << 8) | (p[2] << 16) | (static_cast<uint32_t>(p[3]) << 24);
      q[1] = p[4] | (p[5] << 8) | (p[6] << 16) | (static_cast<uint32_t>(p[7]) << 24);
      xv = load_x8<false>(x_row + c * 8);
      ev = load_x8<false>(eff + c * 8);
    }
    const uint32_t xs[4] = {xv.x, xv.y, xv.z, xv.w}, es[4] = {ev.x, ev.y, ev.z, ev.w};
    float dot = 0.0f, sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float x0 = bf16_lo(xs[j]) * bf16_lo(es[j]);
      const float x1 = bf16_hi(xs[j]) * bf16_hi(es[j]);
      const uint32_t word = q[j >> 1] >> ((j & 1) * 16);
      dot = __builtin_fmaf(static_cast<float>(word & 0xFFu), x0, dot);
      sum = sum + x0;
      dot = __builtin_fmaf(static_cast<float>((word >> 8) & 0xFFu), x1, dot);
      sum = sum + x1;
    }
    const uint32_t g = c * 8 / MF_GROUP_SIZE;
    acc = __builtin_fmaf(bf16_to_f(s_row[g]), dot, acc);
    acc = __builtin_fmaf(bf16_to_f(b_row[g]), sum, acc);
  }
  acc = wave_sum(acc);
  if (lane == 0) logits[static_cast<size_t>(tok) * e + row] = acc;
}

// The same rows for many tokens, bit-exact with the kernel above: a wave keeps R expert rows in
// registers (lane l holds the chunks l, l+64, ... of each row as floats, with their group's scale and
// bias) together with effective_scale, and streams token rows past them; sum x' of a chunk is the
// same for every row and is built once per token.  Needs 16-byte aligned x and effective_scale, 8-byte
// aligned code rows.
template <int CPL, int R>
__global__ __launch_bounds__(256) void router_logits_int8_tiled_kernel(
    const uint8_t* __restrict__ codes, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, const uint16_t* __restrict__ x,
    const uint16_t* __restrict__ eff, uint32_t e, uint32_t d, uint32_t t, uint32_t x_stride,
    float* __restrict__ logits, uint32_t tokens_per_block) {
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const uint32_t row0 = (blockIdx.x * 4 + wv) * R;
  if (row0 >= e) return;
  const uint32_t chunks = d / 8, groups = d / MF_GROUP_SIZE;
  float qf[R][CPL][8], sf[R][CPL], bf[R][CPL], ef[CPL][8];
#pragma unroll
  for (int c = 0; c < CPL; ++c) {
    const uint32_t ci = lane + 64 * c;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (ci < chunks) v = load_x8<true>(eff + ci * 8);
    ef[c][0] = bf16_lo(v.x); ef[c][1] = bf16_hi(v.x); ef[c][2] = bf16_lo(v.y); ef[c][3] = bf16_hi(v.y);
    ef[c][4] = bf16_lo(v.z); ef[c][5] = bf16_hi(v.z); ef[c][6] = bf16_lo(v.w); ef[c][7] = bf16_hi(v.w);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const bool live = ci < chunks && row0 + r < e;
      uint2 q = make_uint2(0, 0);
      if (live) q = *reinterpret_cast<const uint2*>(codes + static_cast<size_t>(row0 + r) * d + ci * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) qf[r][c][j] = static_cast<float>(((j < 4 ? q.x : q.y) >> (8 * (j & 3))) & 0xFFu);
      const size_t g = static_cast<size_t>(row0 + r) * groups + ci * 8 / MF_GROUP_SIZE;
      sf[r][c] = live ? bf16_to_f(scales[g]) : 0.0f;
      bf[r][c] = live ? bf16_to_f(biases[g]) : 0.0f;
    }
  }
  const uint32_t t0 = blockIdx.y * tokens_per_block;
  const uint32_t t1 = min(t, t0 + tokens_per_block);
  for (uint32_t tok = t0; tok < t1; ++tok) {
    const uint16_t* xt = x + static_cast<size_t>(tok) * x_stride;
    float xs[CPL][8], sum[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const uint32_t ci = lane + 64 * c;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (ci < chunks) v = load_x8<true>(xt + ci * 8);
      const float xv[8] = {bf16_lo(v.x), bf16_hi(v.x), bf16_lo(v.y), bf16_hi(v.y),
                           bf16_lo(v.z), bf16_hi(v.z), bf16_lo(v.w), bf16_hi(v.w)};
      sum[c] = 0.0f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        xs[c][j] = xv[j] * ef[c][j];
        sum[c] = sum[c] + xs[c][j];
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float acc = 0.0f;
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        if (lane + 64 * c < chunks) {
          float dot = 0.0f;
#pragma unroll
          for (int j = 0; j < 8; ++j) dot = __builtin_fmaf(qf[r][c][j], xs[c][j], dot);
          acc = __builtin_fmaf(sf[r][c], dot, acc);
          acc = __builtin_fmaf(bf[r][c], sum[c], acc);
        }
      }
      acc = wave_sum(acc);
      if (lane == 0 && row0 + r < e) logits[static_cast<size_t>(tok) * e + row0 + r] = acc;
    }
  }
}

enum Family { kSqrtSoftplus = 0, kHash = 1, kInkling = 2, kScaledSoftmax = 3 };

struct FamilyArgs {
  const float* logits;            // [t, e + n_shared]
  const float* bias;              // [e] selection bias (sqrtsoftplus, Inkling)
  const float* global_scale;      // [1] (Inkling)
  const uint16_t* expert_scale;   // [e] bf16 (scaled softmax)
  const uint32_t* given;          // [t, k] (hash)
  uint32_t e, n_shared, k;
  float route_scale;
  uint32_t* idx;                  // [t, k]
  float* w;                       // [t, k]
  float* gammas;                  // [t, n_shared]
};

__device__ __forceinline__ void lds_settle() {
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  __builtin_amdgcn_wave_barrier();
}

// sum of v over lanes 0..n-1 in ascending order, n <= 16 (the reference's serial tails)
__device__ __forceinline__ float ordered_sum(float v, uint32_t n) {
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < 16; ++i)
    if (static_cast<uint32_t>(i) < n) sum += readlane_f(v, i);
  return sum;
}

// One wave per token.
template <int FAMILY>
__global__ __launch_bounds__(64) void family_select_kernel(FamilyArgs a) {
  __shared__ float s_sel[MF_MAX_EXPERTS];
  __shared__ uint32_t s_idx[MF_MAX_TOPK];
  __shared__ float s_w[MF_MAX_TOPK];
  const uint32_t lane = threadIdx.x, tok = blockIdx.x, k = a.k;
  const float* lg = a.logits + static_cast<size_t>(tok) * (a.e + a.n_shared);
  uint32_t* idx = a.idx + static_cast<size_t>(tok) * k;
  float* w = a.w + static_cast<size_t>(tok) * k;

  if constexpr (FAMILY == kScaledSoftmax) {
    // router_topk_select_k8 (moe.metal:190-240): softmax over the selected, times per_expert_scale
    topk_select_fast(lg, a.e, k, s_idx, s_w, lane);
    lds_settle();
    if (lane < k) {
      const uint32_t my = s_idx[lane];
      idx[lane] = my;
      w[lane] = s_w[lane] * bf16_to_f(a.expert_scale[my]);
    }
    return;
  }

  uint32_t my = 0;
  if constexpr (FAMILY == kHash) {
    if (lane < k) my = a.given[static_cast<size_t>(tok) * k + lane];
  } else {
    for (uint32_t x = lane; x < a.e; x += kWave) {
      const float l = lg[x];
      s_sel[x] = (FAMILY == kSqrtSoftplus ? mf_sqrtsoftplus(l) : 1.0f / (1.0f + mf_exp(-l))) + a.bias[x];
    }
    lds_settle();
    topk_select_indices(s_sel, a.e, k, s_idx, lane);
    lds_settle();
    if (lane < k) {
      my = s_idx[lane];
      idx[lane] = my;
    }
  }

  if constexpr (FAMILY == kInkling) {
    // inkling.metal:540-565: softmax over logsigmoid of the raw logits of the selected experts and
    // the sinks, times route_scale * global_scale
    const uint32_t total = k + a.n_shared;
    float lp = -__builtin_inff();
    if (lane < total) {
      const float x = lane < k ? lg[my] : lg[a.e + (lane - k)];
      lp = (x < 0.0f ? x : 0.0f) - mf_log_1to2(1.0f + mf_exp(-__builtin_fabsf(x)));
    }
    const float mx = wave_max(lp);
    const float ex = lane < total ? mf_exp(lp - mx) : 0.0f;
    const float denom = ordered_sum(ex, total);
    const float s_all = a.route_scale * a.global_scale[0] / denom;
    if (lane < k) w[lane] = ex * s_all;
    else if (lane < total) a.gammas[static_cast<size_t>(tok) * a.n_shared + (lane - k)] = ex * s_all;
  } else {
    // moe.metal:773-785 / :855-865: raw sqrtsoftplus scores of the chosen experts, renormalised.
    // An expert index past the table (possible only for given indices) weighs nothing.
    const float raw = (lane < k && my < a.e) ? mf_sqrtsoftplus(lg[my]) : 0.0f;
    const float inv = a.route_scale / (ordered_sum(raw, k) + 1e-20f);
    if (lane < k) w[lane] = raw * inv;
  }
}

template <int FAMILY>
hipError_t launch_family(hipStream_t s, const FamilyArgs& a, uint32_t t) {
  if (!t) return hipSuccess;
  family_select_kernel<FAMILY><<<dim3(t), dim3(64), 0, s>>>(a);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_router_logits_int8(hipStream_t s, const uint8_t* codes, const uint16_t* scales,
                                     const uint16_t* biases, const uint16_t* x, const uint16_t* eff,
                                     uint32_t e, uint32_t d, uint32_t t, uint32_t x_stride, float* logits) {
  const uint32_t waves = e * t;
  if (!waves) return hipSuccess;
  const int al = (reinterpret_cast<uintptr_t>(codes) % 8 == 0) && aligned16(x) && aligned16(eff) &&
                 x_stride % 8 == 0 && d % 8 == 0;
  const uint32_t cpl = (d / 8 + 63) / 64;
  if (al && t >= 16 && cpl <= 8) {  // many tokens: rows stay in registers
    const uint32_t tpb = std::max(1u, std::min(64u, t / 64));
#define MF_R8(CPL, R)                                                                                \
  router_logits_int8_tiled_kernel<CPL, R><<<dim3((e + 4 * R - 1) / (4 * R), (t + tpb - 1) / tpb), dim3(256), 0, \
                                            s>>>(codes, scales, biases, x, eff, e, d, t, x_stride, logits, tpb)
    if (cpl <= 2) MF_R8(2, 4);
    else if (cpl <= 4) MF_R8(4, 2);
    else if (cpl <= 6) MF_R8(6, 2);
    else MF_R8(8, 1);
#undef MF_R8
    return hipGetLastError();
  }
  router_logits_int8_kernel<<<dim3((waves + 3) / 4), dim3(256), 0, s>>>(codes, scales, biases, x, eff, e, d, t,
                                                                       x_stride, logits, al);
  return hipGetLastError();
}

hipError_t launch_select_sqrtsoftplus(hipStream_t s, const float* logits, const float* bias, uint32_t e,
                                      uint32_t k, uint32_t t, float route_scale, uint32_t* idx, float* w) {
  FamilyArgs a{};
  a.logits = logits; a.bias = bias; a.e = e; a.k = k; a.route_scale = route_scale; a.idx = idx; a.w = w;
  return launch_family<kSqrtSoftplus>(s, a, t);
}

hipError_t launch_hash_weights(hipStream_t s, const float* logits, const uint32_t* given, uint32_t e,
                               uint32_t k, uint32_t t, float route_scale, float* w) {
  FamilyArgs a{};
  a.logits = logits; a.given = given; a.e = e; a.k = k; a.route_scale = route_scale; a.w = w;
  return launch_family<kHash>(s, a, t);
}

hipError_t launch_select_inkling(hipStream_t s, const float* logits, const float* bias,
                                 const float* global_scale, uint32_t n_routed, uint32_t n_shared, uint32_t k,
                                 uint32_t t, float route_scale, uint32_t* idx, float* w, float* gammas) {
  FamilyArgs a{};
  a.logits = logits; a.bias = bias; a.global_scale = global_scale; a.e = n_routed; a.n_shared = n_shared;
  a.k = k; a.route_scale = route_scale; a.idx = idx; a.w = w; a.gammas = gammas;
  return launch_family<kInkling>(s, a, t);
}

hipError_t launch_select_scaled_softmax(hipStream_t s, const float* logits, const uint16_t* expert_scale,
                                        uint32_t e, uint32_t k, uint32_t t, uint32_t* idx, float* w) {
  FamilyArgs a{};
  a.logits = logits; a.expert_scale = expert_scale; a.e = e; a.k = k; a.idx = idx; a.w = w;
  return launch_family<kScaledSoftmax>(s, a, t);
}

}  // namespace mf
