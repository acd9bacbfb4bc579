// Group-quantized GEMV (1..8 token rows against one read of each weight row),
// the fused shared-expert gate/up/activation kernel, and the three elementwise
// ops of the path.  One wave64 owns one or more rows; each lane reads 16 bytes
// of packed codes per step (32 four-bit / 64 two-bit elements), dequantizes in
// registers with the factored form s*sum(q*x) + b*sum(x)
// (Metal/Quant/dequant_int4.metal:14-17) and the row is finished by a wave
// butterfly.
#include "mf_device.h"
#include "mf_internal.h"

#pragma clang fp contract(off)

namespace mf {

// y[t, row] = sum_n deq(W[row, n]) * x[t, n].
// Semantics of dequant_int4_gemv_simd / _f32out (dequant_int4.metal:248-288) for
// T = 1 and dequant_int4_gemv_simd_multix (:356-446) for T > 1.
// lpr = lanes per row (1 << lpr_log2); a wave holds 64 / lpr rows.
template <int BITS, int T, bool ALIGNED>
__global__ __launch_bounds__(256) void gemv_kernel(const uint8_t* __restrict__ W,
                                                   const uint16_t* __restrict__ S,
                                                   const uint16_t* __restrict__ B,
                                                   const uint16_t* __restrict__ x,
                                                   void* __restrict__ y, uint32_t M, uint32_t N,
                                                   uint32_t lpr_log2, int out_f32) {
  constexpr int EPL = Fmt<BITS>::kElemsPer16B;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const uint32_t lpr = 1u << lpr_log2;
  const uint32_t row = (wave << (6 - lpr_log2)) + (lane >> lpr_log2);
  const uint32_t sub = lane & (lpr - 1);
  const bool row_ok = row < M;
  const uint32_t n_groups = N / kGroup;
  const size_t row_bytes = static_cast<size_t>(N) * Store<BITS>::kBits / 8;
  const uint8_t* wrow = W + static_cast<size_t>(row_ok ? row : 0) * row_bytes;
  const uint16_t* srow = S + static_cast<size_t>(row_ok ? row : 0) * n_groups;
  const uint16_t* brow = (BITS == kBitsTernary) ? nullptr
                                                : B + static_cast<size_t>(row_ok ? row : 0) * n_groups;
  float acc[T];
#pragma unroll
  for (int t = 0; t < T; ++t) acc[t] = 0.0f;

  for (uint32_t e0 = sub * EPL; e0 < N; e0 += lpr * EPL) {
    if (!row_ok) break;
    const uint4 codes = load_codes16<ALIGNED>(wrow + static_cast<size_t>(e0) * Store<BITS>::kBits / 8);
    float s, b;
    load_scale_bias<BITS>(srow, brow, e0, s, b);
#pragma unroll
    for (int t = 0; t < T; ++t) {
      float dot, sum;
      lane_dot<BITS, ALIGNED>(codes, x + static_cast<size_t>(t) * N + e0, dot, sum);
      acc[t] = __builtin_fmaf(s, dot, acc[t]);
      acc[t] = __builtin_fmaf(b, sum, acc[t]);
    }
  }
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const float v = group_sum(acc[t], static_cast<int>(lpr));
    if (row_ok && sub == 0) {
      if (out_f32) static_cast<float*>(y)[static_cast<size_t>(t) * M + row] = v;
      else static_cast<uint16_t*>(y)[static_cast<size_t>(t) * M + row] = f_to_bf16(v);
    }
  }
}

// Shared expert / dense MLP phase 1 (shared_int4_gate_up_act_simd,
// dequant_int4.metal:216-246): gate and up rows share the x loads; both fp32
// results are narrowed before the activation and the product is narrowed again.
template <int BITS, int T, bool ALIGNED>
__global__ __launch_bounds__(256) void gate_up_act_kernel(
    const uint8_t* __restrict__ gW, const uint16_t* __restrict__ gS, const uint16_t* __restrict__ gB,
    const uint8_t* __restrict__ uW, const uint16_t* __restrict__ uS, const uint16_t* __restrict__ uB,
    const uint16_t* __restrict__ x, uint16_t* __restrict__ act, uint32_t F, uint32_t D,
    uint32_t lpr_log2) {
  constexpr int EPL = Fmt<BITS>::kElemsPer16B;
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const uint32_t lpr = 1u << lpr_log2;
  const uint32_t row = (wave << (6 - lpr_log2)) + (lane >> lpr_log2);
  const uint32_t sub = lane & (lpr - 1);
  const bool row_ok = row < F;
  const uint32_t n_groups = D / kGroup;
  const size_t row_bytes = static_cast<size_t>(D) * Store<BITS>::kBits / 8;
  const size_t r = row_ok ? row : 0;
  float ga[T], ua[T];
#pragma unroll
  for (int t = 0; t < T; ++t) ga[t] = ua[t] = 0.0f;

  for (uint32_t e0 = sub * EPL; e0 < D; e0 += lpr * EPL) {
    if (!row_ok) break;
    const size_t boff = r * row_bytes + static_cast<size_t>(e0) * Store<BITS>::kBits / 8;
    const uint4 gc = load_codes16<ALIGNED>(gW + boff);
    const uint4 uc = load_codes16<ALIGNED>(uW + boff);
    float gs, gb, us, ub;
    load_scale_bias<BITS>(gS + r * n_groups, (BITS == kBitsTernary) ? nullptr : gB + r * n_groups, e0, gs, gb);
    load_scale_bias<BITS>(uS + r * n_groups, (BITS == kBitsTernary) ? nullptr : uB + r * n_groups, e0, us, ub);
#pragma unroll
    for (int t = 0; t < T; ++t) {
      float gd, ud, sum, sum2;
      const uint16_t* xt = x + static_cast<size_t>(t) * D + e0;
      lane_dot<BITS, ALIGNED>(gc, xt, gd, sum);
      lane_dot<BITS, ALIGNED>(uc, xt, ud, sum2);
      ga[t] = __builtin_fmaf(gs, gd, ga[t]);
      ga[t] = __builtin_fmaf(gb, sum, ga[t]);
      ua[t] = __builtin_fmaf(us, ud, ua[t]);
      ua[t] = __builtin_fmaf(ub, sum, ua[t]);
    }
  }
#pragma unroll
  for (int t = 0; t < T; ++t) {
    const float g = group_sum(ga[t], static_cast<int>(lpr));
    const float u = group_sum(ua[t], static_cast<int>(lpr));
    if (row_ok && sub == 0) {
      const float rg = round_bf16(g), ru = round_bf16(u);
      act[static_cast<size_t>(t) * F + row] = f_to_bf16(mf_silu(rg) * ru);
    }
  }
}

// silu_mul_fp16 (utility.metal:21-33)
__global__ void silu_mul_kernel(const uint16_t* gate, const uint16_t* up, uint16_t* out,
                                uint32_t count) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const float g = bf16_to_f(gate[i]), u = bf16_to_f(up[i]);
  out[i] = f_to_bf16(mf_silu(g) * u);
}

// sigmoid_scalar_mul_fp16 (utility.metal:49-59), one gate per row
// (block form prefill_qwen_shared_scalar_gate, prefill.metal:74-79)
__global__ void sigmoid_scalar_mul_kernel(uint16_t* y, const uint16_t* gate, uint32_t row,
                                          uint32_t rows) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= row * rows) return;
  const float g = bf16_to_f(gate[i / row]);
  y[i] = f_to_bf16(bf16_to_f(y[i]) / (1.0f + mf_exp(-g)));
}

// residual_add_fp16 (utility.metal:83-92)
__global__ void residual_add_kernel(uint16_t* hidden, const uint16_t* delta, uint32_t count) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  hidden[i] = f_to_bf16(bf16_to_f(hidden[i]) + bf16_to_f(delta[i]));
}

namespace {

template <int BITS, bool ALIGNED>
hipError_t gemv_dispatch_t(hipStream_t s, const mf_qtensor& w, const uint16_t* x, void* y,
                           uint32_t m, uint32_t n, uint32_t t, bool out_f32) {
  const uint32_t lpr_log2 = lanes_per_row_log2(n, Fmt<BITS>::kElemsPer16B);
  const uint32_t rows_per_wave = 64u >> lpr_log2;
  const uint32_t waves = (m + rows_per_wave - 1) / rows_per_wave;
  const dim3 grid((waves + 3) / 4), block(256);
  const auto* W = static_cast<const uint8_t*>(w.weights);
#define MF_GEMV_CASE(TT)                                                                     \
  case TT:                                                                                   \
    gemv_kernel<BITS, TT, ALIGNED><<<grid, block, 0, s>>>(W, w.scales, w.biases, x, y, m, n, \
                                                          lpr_log2, out_f32 ? 1 : 0);        \
    break;
  switch (t) {
    MF_GEMV_CASE(1) MF_GEMV_CASE(2) MF_GEMV_CASE(3) MF_GEMV_CASE(4)
    MF_GEMV_CASE(5) MF_GEMV_CASE(6) MF_GEMV_CASE(7) MF_GEMV_CASE(8)
    default: return hipErrorInvalidValue;
  }
#undef MF_GEMV_CASE
  return hipGetLastError();
}

template <int BITS, bool ALIGNED>
hipError_t gate_up_dispatch_t(hipStream_t s, const mf_qtensor& g, const mf_qtensor& u,
                              const uint16_t* x, uint16_t* act, uint32_t f, uint32_t d,
                              uint32_t t) {
  const uint32_t lpr_log2 = lanes_per_row_log2(d, Fmt<BITS>::kElemsPer16B);
  const uint32_t rows_per_wave = 64u >> lpr_log2;
  const uint32_t waves = (f + rows_per_wave - 1) / rows_per_wave;
  const dim3 grid((waves + 3) / 4), block(256);
  const auto* gW = static_cast<const uint8_t*>(g.weights);
  const auto* uW = static_cast<const uint8_t*>(u.weights);
#define MF_GU_CASE(TT)                                                                         \
  case TT:                                                                                     \
    gate_up_act_kernel<BITS, TT, ALIGNED><<<grid, block, 0, s>>>(                              \
        gW, g.scales, g.biases, uW, u.scales, u.biases, x, act, f, d, lpr_log2);               \
    break;
  switch (t) {
    MF_GU_CASE(1) MF_GU_CASE(2) MF_GU_CASE(3) MF_GU_CASE(4)
    MF_GU_CASE(5) MF_GU_CASE(6) MF_GU_CASE(7) MF_GU_CASE(8)
    default: return hipErrorInvalidValue;
  }
#undef MF_GU_CASE
  return hipGetLastError();
}

}  // namespace

hipError_t launch_gemv(hipStream_t s, const mf_qtensor& w, int bits, const uint16_t* x, void* y,
                       uint32_t m, uint32_t n, uint32_t t, bool out_f32) {
  const bool al = aligned16(w.weights) && aligned16(x);
  switch (bits) {
    case kBits4:
      return al ? gemv_dispatch_t<kBits4, true>(s, w, x, y, m, n, t, out_f32)
                : gemv_dispatch_t<kBits4, false>(s, w, x, y, m, n, t, out_f32);
    case kBits2:
      return al ? gemv_dispatch_t<kBits2, true>(s, w, x, y, m, n, t, out_f32)
                : gemv_dispatch_t<kBits2, false>(s, w, x, y, m, n, t, out_f32);
    case kBitsTernary:
      return al ? gemv_dispatch_t<kBitsTernary, true>(s, w, x, y, m, n, t, out_f32)
                : gemv_dispatch_t<kBitsTernary, false>(s, w, x, y, m, n, t, out_f32);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_gate_up_act(hipStream_t s, const mf_qtensor& gate, const mf_qtensor& up,
                              int bits, const uint16_t* x, uint16_t* act, uint32_t f, uint32_t d,
                              uint32_t t) {
  const bool al = aligned16(gate.weights) && aligned16(up.weights) && aligned16(x);
  switch (bits) {
    case kBits4:
      return al ? gate_up_dispatch_t<kBits4, true>(s, gate, up, x, act, f, d, t)
                : gate_up_dispatch_t<kBits4, false>(s, gate, up, x, act, f, d, t);
    case kBits2:
      return al ? gate_up_dispatch_t<kBits2, true>(s, gate, up, x, act, f, d, t)
                : gate_up_dispatch_t<kBits2, false>(s, gate, up, x, act, f, d, t);
    case kBitsTernary:
      return al ? gate_up_dispatch_t<kBitsTernary, true>(s, gate, up, x, act, f, d, t)
                : gate_up_dispatch_t<kBitsTernary, false>(s, gate, up, x, act, f, d, t);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_silu_mul(hipStream_t s, const uint16_t* gate, const uint16_t* up, uint16_t* out,
                           uint32_t count) {
  if (!count) return hipSuccess;
  silu_mul_kernel<<<dim3((count + 255) / 256), dim3(256), 0, s>>>(gate, up, out, count);
  return hipGetLastError();
}

hipError_t launch_sigmoid_scalar_mul(hipStream_t s, uint16_t* y, const uint16_t* gate,
                                     uint32_t row, uint32_t rows) {
  if (!row || !rows) return hipSuccess;
  sigmoid_scalar_mul_kernel<<<dim3((row * rows + 255) / 256), dim3(256), 0, s>>>(y, gate, row, rows);
  return hipGetLastError();
}

hipError_t launch_residual_add(hipStream_t s, uint16_t* hidden, const uint16_t* delta,
                               uint32_t count) {
  if (!count) return hipSuccess;
  residual_add_kernel<<<dim3((count + 255) / 256), dim3(256), 0, s>>>(hidden, delta, count);
  return hipGetLastError();
}

}  // namespace mf
