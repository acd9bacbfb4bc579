// Router: bf16 GEMV to fp32 logits and the top-k selectors.  Both are
// bit-exact against the CPU checker: the logit summation order is fixed (see
// dot_bf16_row) and exp/divide are IEEE sequences shared with it.
#include "mf_device.h"
#include "mf_internal.h"
#include "mf_router.h"

#pragma clang fp contract(off)

namespace mf {

__global__ __launch_bounds__(256) void router_logits_kernel(const uint16_t* __restrict__ w,
                                                            const uint16_t* __restrict__ x,
                                                            uint32_t e, uint32_t d, uint32_t t,
                                                            uint32_t x_stride,
                                                            float* __restrict__ logits,
                                                            uint16_t* __restrict__ logits_bf16,
                                                            int aligned) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (wave >= e * t) return;
  const uint32_t tok = wave / e, row = wave % e;
  const float v = dot_bf16_row(w + static_cast<size_t>(row) * d,
                               x + static_cast<size_t>(tok) * x_stride, d, lane, aligned != 0);
  if (lane == 0) {
    if (logits) logits[static_cast<size_t>(tok) * e + row] = v;
    if (logits_bf16) logits_bf16[static_cast<size_t>(tok) * e + row] = f_to_bf16(v);
  }
}

// one wave per token
__global__ __launch_bounds__(64) void topk_kernel(const float* __restrict__ logits, uint32_t e,
                                                  uint32_t k, int mode,
                                                  uint32_t* __restrict__ idx,
                                                  float* __restrict__ w) {
  const uint32_t tok = blockIdx.x;
  if (mode == 0)
    topk_select_fast(logits + static_cast<size_t>(tok) * e, e, k, idx + static_cast<size_t>(tok) * k,
                     w + static_cast<size_t>(tok) * k, threadIdx.x);
  else {
    __shared__ float s_p[MF_MAX_EXPERTS];
    topk_full_softmax_fast(logits + static_cast<size_t>(tok) * e, s_p, e, k, idx + static_cast<size_t>(tok) * k,
                           w + static_cast<size_t>(tok) * k, threadIdx.x);
  }
}

hipError_t launch_router_logits(hipStream_t s, const uint16_t* w, const uint16_t* x, uint32_t e,
                                uint32_t d, uint32_t t, uint32_t x_stride, float* logits,
                                uint16_t* logits_bf16) {
  const uint32_t waves = e * t;
  if (!waves) return hipSuccess;
  const int al = aligned16(w) && aligned16(x) && (x_stride % 8 == 0) && (d % 8 == 0);
  router_logits_kernel<<<dim3((waves + 3) / 4), dim3(256), 0, s>>>(w, x, e, d, t, x_stride, logits,
                                                                  logits_bf16, al);
  return hipGetLastError();
}

hipError_t launch_topk(hipStream_t s, const float* logits, uint32_t e, uint32_t k, uint32_t t,
                       int mode, uint32_t* idx, float* w) {
  if (!t) return hipSuccess;
  topk_kernel<<<dim3(t), dim3(64), 0, s>>>(logits, e, k, mode, idx, w);
  return hipGetLastError();
}

}  // namespace mf
