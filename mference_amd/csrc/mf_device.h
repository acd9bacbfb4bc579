// Device-side building blocks shared by every kernel: bf16 helpers, the
// deterministic exp, wave64 reductions and the per-lane packed-code dot products.
//
// Compile with -ffp-contract=off: every fused multiply-add below is spelled
// fmaf(); any other a*b+c is two roundings on purpose (the bit-exact paths
// rely on it).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mf {

constexpr int kWave = 64;    // gfx950 wavefront
constexpr int kGroup = 64;   // quantization group (Quantization.swift:5)

enum : int { kBitsTernary = 1, kBits2 = 2, kBits4 = 4 };

// elements covered by one 16-byte load of packed codes
template <int BITS> struct Fmt { static constexpr int kElemsPer16B = (BITS == kBits4) ? 32 : 64; };

// ------------------------------------------------------------------ bf16

__device__ __forceinline__ float bf16_to_f(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}
__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xFFFF0000u); }

// Quantization.swift:17-23: (bits + 0x7FFF + lsb) >> 16, no NaN special case.
__device__ __forceinline__ uint16_t f_to_bf16(float x) {
  uint32_t b = __float_as_uint(x);
  return static_cast<uint16_t>((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float round_bf16(float x) { return bf16_to_f(f_to_bf16(x)); }

// ------------------------------------------------------------------- exp

// Deterministic exp: the same sequence of IEEE operations as the CPU checker,
// so routing weights agree bit for bit.  Results below e^-86 are 0.
__device__ __forceinline__ float mf_exp(float x) {
  if (x != x) return x;
  if (x < -86.0f) return 0.0f;
  if (x > 88.0f) return __builtin_inff();
  float n = __builtin_rintf(x * 1.44269504088896341f);
  float r = __builtin_fmaf(-n, 0.693145751953125f, x);
  r = __builtin_fmaf(-n, 1.42860682030941723212e-6f, r);
  float p = 1.9875691500e-4f;
  p = __builtin_fmaf(p, r, 1.3981999507e-3f);
  p = __builtin_fmaf(p, r, 8.3334519073e-3f);
  p = __builtin_fmaf(p, r, 4.1665795894e-2f);
  p = __builtin_fmaf(p, r, 1.6666665459e-1f);
  p = __builtin_fmaf(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  p = __builtin_fmaf(p, r2, r);
  p = p + 1.0f;
  int e = static_cast<int>(n) + 127;
  return p * __uint_as_float(static_cast<uint32_t>(e) << 23);
}

// moe.metal:79-84
__device__ __forceinline__ float mf_silu(float x) { return x / (1.0f + mf_exp(-x)); }

// --------------------------------------------------------- wave reductions

// xor butterfly over the low `lanes` lanes of each aligned lane group
// (lanes = power of two <= 64); every lane of the group ends with the sum.
// Strides run from lanes/2 down to 1: this order is part of the router's
// bit-exact contract.
__device__ __forceinline__ float group_sum(float v, int lanes) {
  for (int o = lanes >> 1; o > 0; o >>= 1) v = v + __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_sum(float v) { return group_sum(v, kWave); }

// ------------------------------------------------------------- raw loads

__device__ __forceinline__ uint32_t load_u32_bytes(const uint8_t* p) {
  return static_cast<uint32_t>(p[0]) | (static_cast<uint32_t>(p[1]) << 8) |
         (static_cast<uint32_t>(p[2]) << 16) | (static_cast<uint32_t>(p[3]) << 24);
}

// 16 bytes of packed codes; ALIGNED = pointer is 16-byte aligned.
template <bool ALIGNED>
__device__ __forceinline__ uint4 load_codes16(const uint8_t* p) {
  if constexpr (ALIGNED) {
    return *reinterpret_cast<const uint4*>(p);
  } else {
    uint4 r;
    r.x = load_u32_bytes(p);
    r.y = load_u32_bytes(p + 4);
    r.z = load_u32_bytes(p + 8);
    r.w = load_u32_bytes(p + 12);
    return r;
  }
}

// 8 bf16 values as 4 packed pairs; ALIGNED = pointer is 16-byte aligned
// (otherwise 2-byte aligned).
template <bool ALIGNED>
__device__ __forceinline__ uint4 load_x8(const uint16_t* p) {
  if constexpr (ALIGNED) {
    return *reinterpret_cast<const uint4*>(p);
  } else {
    uint4 r;
    r.x = static_cast<uint32_t>(p[0]) | (static_cast<uint32_t>(p[1]) << 16);
    r.y = static_cast<uint32_t>(p[2]) | (static_cast<uint32_t>(p[3]) << 16);
    r.z = static_cast<uint32_t>(p[4]) | (static_cast<uint32_t>(p[5]) << 16);
    r.w = static_cast<uint32_t>(p[6]) | (static_cast<uint32_t>(p[7]) << 16);
    return r;
  }
}

// ------------------------------------------------- per-lane code x x dots

// byte i of v as float (v_cvt_f32_ubyte{i})
__device__ __forceinline__ float ubyte_f(uint32_t v, int i) {
  return static_cast<float>((v >> (8 * i)) & 0xFFu);
}

// 8 consecutive 4-bit codes (one uint32, element j at bit 4j) against 8 bf16
// (four packed pairs).  dot += sum q*x, sum += sum x.
__device__ __forceinline__ void dot8_q4(uint32_t w, const uint4& x, float& dot, float& sum) {
  const uint32_t lo = w & 0x0F0F0F0Fu;         // byte i = code of element 2i
  const uint32_t hi = (w >> 4) & 0x0F0F0F0Fu;  // byte i = code of element 2i+1
  const uint32_t xs[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float x0 = bf16_lo(xs[i]), x1 = bf16_hi(xs[i]);
    dot = __builtin_fmaf(ubyte_f(lo, i), x0, dot);
    dot = __builtin_fmaf(ubyte_f(hi, i), x1, dot);
    sum += x0 + x1;
  }
}

// 16 consecutive 2-bit codes (one uint32, element j at bit 2j) against 16 bf16.
__device__ __forceinline__ void dot16_q2(uint32_t w, const uint4& xa, const uint4& xb,
                                         float& dot, float& sum) {
  // plane p, byte i = code of element 4i + p
  const uint32_t p0 = w & 0x03030303u;
  const uint32_t p1 = (w >> 2) & 0x03030303u;
  const uint32_t p2 = (w >> 4) & 0x03030303u;
  const uint32_t p3 = (w >> 6) & 0x03030303u;
  const uint32_t xs[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {  // byte i covers elements 4i..4i+3 = pairs 2i, 2i+1
    const float x0 = bf16_lo(xs[2 * i]), x1 = bf16_hi(xs[2 * i]);
    const float x2 = bf16_lo(xs[2 * i + 1]), x3 = bf16_hi(xs[2 * i + 1]);
    dot = __builtin_fmaf(ubyte_f(p0, i), x0, dot);
    dot = __builtin_fmaf(ubyte_f(p1, i), x1, dot);
    dot = __builtin_fmaf(ubyte_f(p2, i), x2, dot);
    dot = __builtin_fmaf(ubyte_f(p3, i), x3, dot);
    sum += (x0 + x1) + (x2 + x3);
  }
}

// One lane's share of a row: 16 bytes of codes (32 four-bit or 64 two-bit
// elements, never straddling a 64-group for 4-bit: a lane covers half a
// group; exactly one group for 2-bit) against the matching slice of x.
template <int BITS, bool ALIGNED>
__device__ __forceinline__ void lane_dot(const uint4& codes, const uint16_t* x, float& dot,
                                         float& sum) {
  dot = 0.0f;
  sum = 0.0f;
  if constexpr (BITS == kBits4) {
    dot8_q4(codes.x, load_x8<ALIGNED>(x), dot, sum);
    dot8_q4(codes.y, load_x8<ALIGNED>(x + 8), dot, sum);
    dot8_q4(codes.z, load_x8<ALIGNED>(x + 16), dot, sum);
    dot8_q4(codes.w, load_x8<ALIGNED>(x + 24), dot, sum);
  } else {
    dot16_q2(codes.x, load_x8<ALIGNED>(x), load_x8<ALIGNED>(x + 8), dot, sum);
    dot16_q2(codes.y, load_x8<ALIGNED>(x + 16), load_x8<ALIGNED>(x + 24), dot, sum);
    dot16_q2(codes.z, load_x8<ALIGNED>(x + 32), load_x8<ALIGNED>(x + 40), dot, sum);
    dot16_q2(codes.w, load_x8<ALIGNED>(x + 48), load_x8<ALIGNED>(x + 56), dot, sum);
  }
}

// Same with the code part only (x already turned into fp32 by the caller,
// `xf` holds kElemsPer16B values): used when one x slice meets many rows.
template <int BITS>
__device__ __forceinline__ float lane_dot_xf(const uint4& codes, const float* xf) {
  float dot = 0.0f;
  const uint32_t ws[4] = {codes.x, codes.y, codes.z, codes.w};
  if constexpr (BITS == kBits4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t lo = ws[j] & 0x0F0F0F0Fu, hi = (ws[j] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dot = __builtin_fmaf(ubyte_f(lo, i), xf[8 * j + 2 * i], dot);
        dot = __builtin_fmaf(ubyte_f(hi, i), xf[8 * j + 2 * i + 1], dot);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w = ws[j];
      const uint32_t p0 = w & 0x03030303u, p1 = (w >> 2) & 0x03030303u;
      const uint32_t p2 = (w >> 4) & 0x03030303u, p3 = (w >> 6) & 0x03030303u;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        dot = __builtin_fmaf(ubyte_f(p0, i), xf[16 * j + 4 * i], dot);
        dot = __builtin_fmaf(ubyte_f(p1, i), xf[16 * j + 4 * i + 1], dot);
        dot = __builtin_fmaf(ubyte_f(p2, i), xf[16 * j + 4 * i + 2], dot);
        dot = __builtin_fmaf(ubyte_f(p3, i), xf[16 * j + 4 * i + 3], dot);
      }
    }
  }
  return dot;
}

// scale / bias of the group that holds element e0 of a row whose tables start
// at srow / brow; ternary rows carry no bias table (bias = -scale).
template <int BITS>
__device__ __forceinline__ void load_scale_bias(const uint16_t* srow, const uint16_t* brow,
                                                uint32_t e0, float& s, float& b) {
  const uint32_t g = e0 / kGroup;
  s = bf16_to_f(srow[g]);
  if constexpr (BITS == kBitsTernary) b = -s;
  else b = bf16_to_f(brow[g]);
}

// lanes of a wave that share one row of n elements (power of two, <= 64)
__host__ __device__ __forceinline__ uint32_t lanes_per_row_log2_dev(uint32_t n, uint32_t elems_per_lane) {
  const uint32_t need = (n + elems_per_lane - 1) / elems_per_lane;
  uint32_t l = 0;
  while ((1u << l) < need && l < 6) ++l;
  return l;
}

// storage width of a format in bits per element
template <int BITS> struct Store { static constexpr int kBits = (BITS == kBits4) ? 4 : 2; };

// the dot-product flavour of a format (ternary shares the 2-bit unpack)
template <int BITS> struct DotBits { static constexpr int k = (BITS == kBits4) ? kBits4 : kBits2; };

}  // namespace mf
