// MLX-affine group quantization on device: the quantizer and the bit-exact
// dequantizer of Infrastructure/ModelIO/Quantization.swift:50-119.
#include "mf_device.h"
#include "mf_internal.h"

#pragma clang fp contract(off)

namespace mf {

// 16 lanes share one group of 64 values (4 each).  Ties between equal values
// (only observable for +0/-0) keep the earlier element, as the reference's
// sequential `if w < wmin` scan does.
template <int BITS>
__global__ __launch_bounds__(256) void quantize_kernel(const float* __restrict__ w,
                                                       size_t n_groups,
                                                       uint8_t* __restrict__ packed,
                                                       uint16_t* __restrict__ scales,
                                                       uint16_t* __restrict__ biases) {
  constexpr int kQMax = (BITS == kBits8) ? 255 : (BITS == kBits4) ? 15 : 3;  // 8-bit: Quantization.swift:135-176
  constexpr int kCodeBits = (BITS == kBits8) ? 8 : Store<BITS>::kBits;
  const size_t g = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) >> 4;
  const int l16 = threadIdx.x & 15;
  const bool live = g < n_groups;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (live) {
    const float4 q = *reinterpret_cast<const float4*>(w + g * kGroup + l16 * 4);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  }
  float wmin = v[0], wmax = v[0];
#pragma unroll
  for (int i = 1; i < 4; ++i) {
    if (v[i] < wmin) wmin = v[i];
    if (v[i] > wmax) wmax = v[i];
  }
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) {
    const float omin = __shfl_xor(wmin, o, kWave);
    const float omax = __shfl_xor(wmax, o, kWave);
    const bool partner_is_earlier = (l16 & o) != 0;
    if (omin < wmin || (omin == wmin && partner_is_earlier)) wmin = omin;
    if (omax > wmax || (omax == wmax && partner_is_earlier)) wmax = omax;
  }
  float scale_f, bias_f;
  if (wmax == wmin) {  // constant group: exact reconstruction (Quantization.swift:70-76)
    scale_f = 1.0f;
    bias_f = wmin;
  } else {
    scale_f = (wmax - wmin) / static_cast<float>(kQMax);
    bias_f = wmin;
  }
  const uint16_t sb = f_to_bf16(scale_f), bb = f_to_bf16(bias_f);
  const float scale = bf16_to_f(sb), bias = bf16_to_f(bb);
  const float inv = scale == 0.0f ? 0.0f : 1.0f / scale;
  uint32_t code = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float t = (v[i] - bias) * inv;
    const float rq = __builtin_roundf(t);  // Swift .rounded(): half away from zero
    const int q = rq >= static_cast<float>(kQMax) ? kQMax : (rq <= 0.0f ? 0 : static_cast<int>(rq));
    code |= static_cast<uint32_t>(q) << (kCodeBits * i);
  }
  if (!live) return;
  if (l16 == 0) {
    scales[g] = sb;
    biases[g] = bb;
  }
  if constexpr (BITS == kBits8) {
    uint8_t* o = packed + g * 64 + l16 * 4;  // (2-byte aligned at least: written as two halves)
    *reinterpret_cast<uint16_t*>(o) = static_cast<uint16_t>(code);
    *reinterpret_cast<uint16_t*>(o + 2) = static_cast<uint16_t>(code >> 16);
  } else if constexpr (BITS == kBits4) {
    *reinterpret_cast<uint16_t*>(packed + g * 32 + l16 * 2) = static_cast<uint16_t>(code);
  } else {
    packed[g * 16 + l16] = static_cast<uint8_t>(code);
  }
}

// One thread per 8 consecutive elements: out = float(q) * scale + bias, the
// multiply and the add rounded separately (Quantization.swift:115).
template <int BITS>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t* __restrict__ packed,
                                                         const uint16_t* __restrict__ scales,
                                                         const uint16_t* __restrict__ biases,
                                                         size_t n_elems, float* __restrict__ out) {
  const size_t i8 = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t e0 = i8 * 8;
  if (e0 >= n_elems) return;
  const size_t g = e0 / kGroup;
  const float s = bf16_to_f(scales[g]);
  const float b = (BITS == kBitsTernary) ? -s : bf16_to_f(biases[g]);
  uint32_t w;
  if constexpr (BITS == kBits8) {  // a byte per code (Quantization.swift:179-190)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float prod = static_cast<float>(packed[e0 + i]) * s;
      out[e0 + i] = prod + b;
    }
    return;
  } else if constexpr (BITS == kBits4) {
    w = load_u32_bytes(packed + e0 / 2);
  } else {
    const uint8_t* p = packed + e0 / 4;
    w = static_cast<uint32_t>(p[0]) | (static_cast<uint32_t>(p[1]) << 8);
  }
  constexpr int kW = BITS == kBits8 ? 8 : Store<BITS>::kBits;
  constexpr uint32_t kMask = (1u << kW) - 1u;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float q = static_cast<float>((w >> (kW * i)) & kMask);
    const float prod = q * s;
    out[e0 + i] = prod + b;
  }
}

hipError_t launch_quantize(hipStream_t s, const float* w, size_t rows, size_t n, int bits,
                           void* packed, uint16_t* scales, uint16_t* biases) {
  const size_t n_groups = rows * (n / kGroup);
  if (n_groups == 0) return hipSuccess;
  const size_t blocks = (n_groups * 16 + 255) / 256;
  auto* p = static_cast<uint8_t*>(packed);
  if (bits == kBits8)
    quantize_kernel<kBits8><<<dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, s>>>(
        w, n_groups, p, scales, biases);
  else if (bits == kBits4)
    quantize_kernel<kBits4><<<dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, s>>>(
        w, n_groups, p, scales, biases);
  else
    quantize_kernel<kBits2><<<dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, s>>>(
        w, n_groups, p, scales, biases);
  return hipGetLastError();
}

hipError_t launch_dequantize(hipStream_t s, const mf_qtensor& q, size_t rows, size_t n, int bits,
                             float* out) {
  const size_t n_elems = rows * n;
  if (n_elems == 0) return hipSuccess;
  const size_t blocks = (n_elems / 8 + 255) / 256;
  const auto* p = static_cast<const uint8_t*>(q.weights);
  const dim3 grid(static_cast<uint32_t>(blocks)), block(256);
  if (bits == kBits8)
    dequantize_kernel<kBits8><<<grid, block, 0, s>>>(p, q.scales, q.biases, n_elems, out);
  else if (bits == kBits4)
    dequantize_kernel<kBits4><<<grid, block, 0, s>>>(p, q.scales, q.biases, n_elems, out);
  else if (bits == kBits2)
    dequantize_kernel<kBits2><<<grid, block, 0, s>>>(p, q.scales, q.biases, n_elems, out);
  else
    dequantize_kernel<kBitsTernary><<<grid, block, 0, s>>>(p, q.scales, q.biases, n_elems, out);
  return hipGetLastError();
}

}  // namespace mf
