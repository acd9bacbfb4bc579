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

enum : int { kBitsTernary = 1, kBits2 = 2, kBits4 = 4, kBits8 = 8 };  // 8: GEMV, quantizer and scalar gate only

// elements covered by one 16-byte load of packed codes
template <int BITS> struct Fmt { static constexpr int kElemsPer16B = (BITS == kBits4) ? 32 : 64; };
// storage width of a format in bits per element (ternary is stored as 2-bit codes)
template <int BITS> struct Store { static constexpr int kBits = (BITS == kBits4) ? 4 : 2; };

// lanes of a wave that share one row of n elements (power of two, <= 64)
__host__ __device__ __forceinline__ uint32_t lanes_per_row_log2_dev(uint32_t n,
                                                                    uint32_t elems_per_lane) {
  const uint32_t need = (n + elems_per_lane - 1) / elems_per_lane;
  uint32_t l = 0;
  while ((1u << l) < need && l < 6) ++l;
  return l;
}

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

// log(t) for 1 <= t <= 2 (t = 1 + exp(-|x|) in the routers): 2*atanh((t-1)/(t+1)), odd series
// through s^15; the same IEEE sequence as the CPU checker.
__device__ __forceinline__ float mf_log_1to2(float t) {
  const float s = (t - 1.0f) / (t + 1.0f);
  const float z = s * s;
  float p = 6.6666666667e-2f;
  p = __builtin_fmaf(p, z, 7.6923076923e-2f);
  p = __builtin_fmaf(p, z, 9.0909090909e-2f);
  p = __builtin_fmaf(p, z, 1.1111111111e-1f);
  p = __builtin_fmaf(p, z, 1.4285714286e-1f);
  p = __builtin_fmaf(p, z, 2.0e-1f);
  p = __builtin_fmaf(p, z, 3.3333333333e-1f);
  float r = s * z;
  r = __builtin_fmaf(r, p, s);
  return r + r;
}

// moe.metal:736-740
__device__ __forceinline__ float mf_sqrtsoftplus(float x) {
  const float sp = (x > 0.0f ? x : 0.0f) + mf_log_1to2(1.0f + mf_exp(-__builtin_fabsf(x)));
  return __builtin_sqrtf(sp);
}

// moe.metal:79-84
__device__ __forceinline__ float mf_silu(float x) { return x / (1.0f + mf_exp(-x)); }

// int8_gelu_pytorch_tanh (Metal/Quant/dequant_int8.metal:44-49): 0.5 x (1 + tanh(c (x + 0.044715 x^3))), the
// argument clamped to +-20; tanh(z) = 1 - 2 / (exp(2 z) + 1) on this build's exp, the same IEEE sequence as the
// CPU checker.
__device__ __forceinline__ float mf_gelu_tanh(float x) {
  const float x3 = x * x * x;
  float inner = 0.7978845608028654f * (x + 0.044715f * x3);
  inner = fminf(fmaxf(inner, -20.0f), 20.0f);
  const float th = 1.0f - 2.0f / (mf_exp(2.0f * inner) + 1.0f);
  return 0.5f * x * (1.0f + th);
}

// MapleMoE's activation (maple_swiglu, maple_moe.metal:153-164): every intermediate is a bf16 number.
// min / clamp of bf16 numbers against +-7 and |x| stay bf16 numbers, so only the five arithmetic
// results are narrowed here.
__device__ __forceinline__ float maple_swiglu(float gate_projection, float up_projection) {
  const float gate = fminf(round_bf16(gate_projection), 7.0f);
  const float up = fminf(fmaxf(round_bf16(up_projection), -7.0f), 7.0f);
  const float exponent = round_bf16(mf_exp(fabsf(gate)));
  const float reciprocal = round_bf16(1.0f / round_bf16(1.0f + exponent));
  const float sigmoid = gate < 0.0f ? reciprocal : round_bf16(1.0f - reciprocal);
  return round_bf16(round_bf16(gate * sigmoid) * up);
}

// the routed experts' activation, narrowed once (moe.metal:27-34, 528) or in Maple's steps
__device__ __forceinline__ uint16_t routed_activation(float g, float u, float limit, bool maple) {
  if (maple) return f_to_bf16(maple_swiglu(g, u));
  if (limit > 0.0f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  return f_to_bf16(mf_silu(g) * u);
}

// --------------------------------------------------------- wave reductions

// cross-lane move inside a row of 16 lanes (DPP); CTRL: 0xB1 = swap lanes
// (l, l^1), 0x4E = (l, l^2), 0x141 = mirror inside 8, 0x140 = mirror inside 16
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float readlane_f(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

// Sum over aligned groups of `lanes` lanes (power of two <= 64); every lane of
// a group ends with the group's sum.  The tree pairs neighbours first:
// (l, l^1), then (l, l^2), 4, 8, 16, 32 -- identical to an xor butterfly with
// ascending strides, which is the order the router's bit-exact contract names.
__device__ __forceinline__ float group_sum(float v, int lanes) {
  if (lanes >= 2) v = v + dpp_f<0xB1>(v);
  if (lanes >= 4) v = v + dpp_f<0x4E>(v);
  if (lanes >= 8) v = v + dpp_f<0x141>(v);
  if (lanes >= 16) v = v + dpp_f<0x140>(v);
  if (lanes >= 32) {
    const float r0 = readlane_f(v, 0), r1 = readlane_f(v, 16);
    const float r2 = readlane_f(v, 32), r3 = readlane_f(v, 48);
    const float lo = r0 + r1, hi = r2 + r3;
    if (lanes >= 64) v = lo + hi;
    else v = (threadIdx.x & 32) ? hi : lo;
  }
  return v;
}
__device__ __forceinline__ float wave_sum(float v) { return group_sum(v, kWave); }

// maximum over the wave, returned in every lane (no NaN inputs)
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f<0xB1>(v));
  v = fmaxf(v, dpp_f<0x4E>(v));
  v = fmaxf(v, dpp_f<0x141>(v));
  v = fmaxf(v, dpp_f<0x140>(v));
  const float r0 = readlane_f(v, 0), r1 = readlane_f(v, 16);
  const float r2 = readlane_f(v, 32), r3 = readlane_f(v, 48);
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// ------------------------------------------- device-coherent accesses
//
// Data that workgroups on different XCDs exchange inside one launch goes
// through these: `sc1` makes a store write through, and a load miss, every
// cache that is private to a CU or an XCD, so no bulk cache write-back or
// invalidate is needed around the grid barriers.

__device__ __forceinline__ void store_u16_agent(uint16_t* p, uint16_t v) {
  const uint32_t vv = v;
  asm volatile("global_store_short %0, %1, off sc1" : : "v"(p), "v"(vv) : "memory");
}
__device__ __forceinline__ uint16_t load_u16_agent(const uint16_t* p) {
  uint32_t r;
  asm volatile("global_load_ushort %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(r) : "v"(p) : "memory");
  return static_cast<uint16_t>(r);
}
__device__ __forceinline__ void store_u32_agent(uint32_t* p, uint32_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// 16 bytes (16-byte aligned) written through as one request; readers rely on nothing wider than
// the 4-byte words being whole
__device__ __forceinline__ void store_u32x4_agent(uint32_t* p, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  const u32x4 v = {a, b, c, d};
  asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void store_u32x4_agent(uint32_t* p, uint32_t a) { store_u32x4_agent(p, a, a, a, a); }
__device__ __forceinline__ void store_f32_agent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_f32_agent(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint4 load_u32x4_agent(const void* p) {
  uint4 r;
  asm volatile("global_load_dwordx4 %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(r) : "v"(p) : "memory");
  return r;
}
// Device-coherent 16-byte loads the compiler can schedule and wait for itself
// (several may be in flight): a raw buffer over [p, p + 2 GiB) read with sc1.
typedef __attribute__((ext_vector_type(4))) unsigned int mf_u32x4;
struct AgentBuf {
  __amdgpu_buffer_rsrc_t rsrc;
};
__device__ __forceinline__ AgentBuf make_agent_buf(const void* p) {
  AgentBuf b;
  b.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, 0x7FFFFFFF, 0x00020000);
  return b;
}
__device__ __forceinline__ uint4 load_u32x4_agentbuf(const AgentBuf& b, uint32_t byte_offset) {
  const mf_u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(b.rsrc, static_cast<int>(byte_offset), 0,
                                                           16 /* sc1 */);
  return make_uint4(v.x, v.y, v.z, v.w);
}

// Nothing is moved across this point by the compiler: placed behind a group of loads it keeps
// them one batch of requests (the compiler otherwise sinks some of them below the arithmetic on
// the others, which turns one memory round trip into several).
__device__ __forceinline__ void issue_fence() { asm volatile("" ::: "memory"); }

// every store this wave has issued is acknowledged at its scope
__device__ __forceinline__ void wait_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// 32 bf16 (64 bytes) of exchanged activations
__device__ __forceinline__ void load_x32_agent(const uint16_t* p, uint4 (&x)[4]) {
  asm volatile(
      "global_load_dwordx4 %0, %4, off sc1\n\t"
      "global_load_dwordx4 %1, %4, off offset:16 sc1\n\t"
      "global_load_dwordx4 %2, %4, off offset:32 sc1\n\t"
      "global_load_dwordx4 %3, %4, off offset:48 sc1\n\t"
      "s_waitcnt vmcnt(0)"
      : "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3])
      : "v"(p)
      : "memory");
}

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
//
// One lane's share of a row is 16 bytes of codes: 32 four-bit elements (half a
// quantization group) or 64 two-bit elements (one group).  The dot product
// sum(q*x) runs on v_dot2c_f32_bf16: two codes are masked out of the packed
// word straight into the mantissas of a bf16 pair (0x4100 | q << 3 = 8 + q/2
// for 4-bit codes, 0x4080 | q << 5 = 4 + q for 2-bit codes, both exact),
// multiplied with a matching bf16 pair of x and accumulated in fp32; the
// offset * sum(x) this adds is taken off once per lane share.  Codes are
// paired (j, j + 4) for 4-bit and (j, j + 8) for 2-bit because those pairs sit
// 16 bits apart in the packed word; the x slice is permuted once to match and
// reused for every row that meets it (gate and up, several tokens' rows).

typedef __attribute__((ext_vector_type(2))) short mf_bf16x2;

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float acc) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(mf_bf16x2, a),
                                         __builtin_bit_cast(mf_bf16x2, b), acc, false);
}

constexpr uint32_t kMagic128 = 0x43004300u;  // bf16 pair (128.0, 128.0)
// A masked code lands in the mantissa of a bf16 whose exponent is the smallest that leaves
// room for it: 4-bit codes in mantissa bits 3..6 under 2^3 (the number 8 + q/2), 2-bit codes
// in bits 5..6 under 2^2 (4 + q).  The dot product then carries offset * sum(x), removed in
// fp32 afterwards; the smaller the offset, the less of the fp32 mantissa that cancellation eats.
constexpr uint32_t kMagic8 = 0x41004100u;    // bf16 pair (8.0, 8.0)
constexpr uint32_t kMagic4 = 0x40804080u;    // bf16 pair (4.0, 4.0)
constexpr uint32_t kOnes = 0x3F803F80u;      // bf16 pair (1.0, 1.0)

// (v & mask) | magic in one instruction (v_and_or_b32).  A VOP3 instruction of this ISA takes
// one scalar source and no literal, so the mask has to sit in a scalar register and the magic in
// a vector register; the two empty asm statements only pin the constants there (they are pure,
// so the compiler hoists them out of loops) and the and-or itself stays an ordinary instruction
// the compiler schedules and guards: written as inline asm it would escape the hazard checks
// between a matrix instruction that still reads an operand and the next write of that register.
__device__ __forceinline__ uint32_t pin_sgpr(uint32_t x) {
  uint32_t r;
  asm("" : "=s"(r) : "0"(x));
  return r;
}
__device__ __forceinline__ uint32_t pin_vgpr(uint32_t x) {
  uint32_t r;
  asm("" : "=v"(r) : "0"(x));
  return r;
}
__device__ __forceinline__ uint32_t and_or(uint32_t v, uint32_t mask, uint32_t magic) {
  return (v & pin_sgpr(mask)) | pin_vgpr(magic);
}

// ---- matrix-core forms of the same embedding
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

__device__ __forceinline__ f32x16_t mfma_bf16(const uint4& a, const uint4& b, const f32x16_t& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// one packed word of 4-bit codes -> MFMA operand: pairs (q0,q4),(q1,q5),(q2,q6),(q3,q7) as the
// bf16 numbers 8 + q/2 (exponent 2^3, the code in mantissa bits 3..6).  16 is the smallest offset
// a mask-and-or can give a 4-bit code, and the offset matters: the matrix core accumulates
// offset * sum(x) alongside the signal and the correction term takes it out again in fp32.
__device__ __forceinline__ uint4 expand_q4(uint32_t w) {
  return make_uint4(and_or(w << 3, 0x00780078u, kMagic8), and_or(w >> 1, 0x00780078u, kMagic8),
                    and_or(w >> 5, 0x00780078u, kMagic8), and_or(w >> 9, 0x00780078u, kMagic8));
}

// one packed word of sixteen 2-bit codes -> two MFMA operands in the same pairing: the byte swap
// (B0, B2, B1, B3) puts code r and code r + 4 sixteen bits apart, and likewise 8 + r and 12 + r, so
// a = (q0,q4),(q1,q5),(q2,q6),(q3,q7) and b = (q8,q12),...,(q11,q15) as the bf16 numbers 4 + q
// (exponent 2^2, the code in mantissa bits 5..6): the x order of the 4-bit form serves both.
__device__ __forceinline__ void expand_q2(uint32_t w, uint4& a, uint4& b) {
  const uint32_t v = __builtin_amdgcn_perm(w, w, 0x03010200u);
  a = make_uint4(and_or(v << 5, 0x00600060u, kMagic4), and_or(v << 3, 0x00600060u, kMagic4),
                 and_or(v << 1, 0x00600060u, kMagic4), and_or(v >> 1, 0x00600060u, kMagic4));
  b = make_uint4(and_or(v >> 3, 0x00600060u, kMagic4), and_or(v >> 5, 0x00600060u, kMagic4),
                 and_or(v >> 7, 0x00600060u, kMagic4), and_or(v >> 9, 0x00600060u, kMagic4));
}

// What the quantized matmuls need to know about a code width: a lane's share of one 64-wide group
// of its weight row is half the group -- 16 bytes of 4-bit codes or 8 bytes of 2-bit codes (ternary
// weights are 2-bit codes) -- and it becomes four MFMA operands of 8 bf16 numbers offset + q * step.
template <int BITS> struct QmmCodes;
template <> struct QmmCodes<4> {
  static constexpr uint32_t kGroupBytes = 32;     // one group of one row
  static constexpr uint32_t kNegOffsetAdd = 0x02000200u;  // exponent + 4: 16 * scale (offset 8 at step 1/2)
  static constexpr float kScaleMul = 2.0f;        // codes enter as 8 + q/2
  uint32_t w[4];
  __device__ __forceinline__ void load(const uint8_t* p) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
  }
};
template <> struct QmmCodes<2> {
  static constexpr uint32_t kGroupBytes = 16;
  static constexpr uint32_t kNegOffsetAdd = 0x01000100u;  // exponent + 2: 4 * scale (offset 4 at step 1)
  static constexpr float kScaleMul = 1.0f;        // codes enter as 4 + q
  uint32_t w[2];
  __device__ __forceinline__ void load(const uint8_t* p) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    w[0] = v.x; w[1] = v.y;
  }
};

// tmp[token block] += x * codes over one group: 8 MFMAs; `after(s)` runs once both token blocks have
// issued theirs on operand s (the caller may then overwrite bx[.][s])
// (NTA = 1: only the first token block holds routes, the second is left alone)
template <int BITS, int NTA = 2, typename After>
__device__ __forceinline__ void group_products(const QmmCodes<BITS>& c, const uint4 (&bx)[2][4], f32x16_t (&tmp)[2],
                                               After after) {
  if constexpr (BITS == 4) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint4 av = expand_q4(c.w[s]);
      tmp[0] = mfma_bf16(bx[0][s], av, tmp[0]);
      if constexpr (NTA > 1) tmp[1] = mfma_bf16(bx[1][s], av, tmp[1]);
      after(s);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      uint4 a, b;
      expand_q2(c.w[j], a, b);
      tmp[0] = mfma_bf16(bx[0][2 * j], a, tmp[0]);
      if constexpr (NTA > 1) tmp[1] = mfma_bf16(bx[1][2 * j], a, tmp[1]);
      after(2 * j);
      tmp[0] = mfma_bf16(bx[0][2 * j + 1], b, tmp[0]);
      if constexpr (NTA > 1) tmp[1] = mfma_bf16(bx[1][2 * j + 1], b, tmp[1]);
      after(2 * j + 1);
    }
  }
}

// 8 bf16 from p, of which only the first `avail` exist (the rest read as 0)
__device__ __forceinline__ uint4 load_bf16x8_guarded(const uint16_t* p, uint32_t avail) {
  if (avail >= 8) return load_x8<false>(p);
  uint32_t v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = static_cast<uint32_t>(i) < avail ? p[i] : 0u;
  return make_uint4(v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16));
}

// The activations one lane meets, permuted for the pairing above, plus their sum.
template <int BITS> struct XSlice {
  static constexpr int kPairs = Fmt<BITS>::kElemsPer16B / 2;
  uint32_t p[kPairs];
  float sum;
};

// raw: consecutive bf16 pairs (x0,x1),(x2,x3),... of the lane's slice
template <int BITS>
__device__ __forceinline__ void permute_x(const uint32_t* raw, XSlice<BITS>& xs) {
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < XSlice<BITS>::kPairs; ++i) sum = dot2_bf16(raw[i], kOnes, sum);
  xs.sum = sum;
  if constexpr (BITS == kBits4) {
    // per packed word: 8 elements = raw pairs r0..r3 -> (x0,x4),(x1,x5),(x2,x6),(x3,x7)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t r0 = raw[4 * j], r1 = raw[4 * j + 1], r2 = raw[4 * j + 2], r3 = raw[4 * j + 3];
      xs.p[4 * j + 0] = __builtin_amdgcn_perm(r2, r0, 0x05040100u);
      xs.p[4 * j + 1] = __builtin_amdgcn_perm(r2, r0, 0x07060302u);
      xs.p[4 * j + 2] = __builtin_amdgcn_perm(r3, r1, 0x05040100u);
      xs.p[4 * j + 3] = __builtin_amdgcn_perm(r3, r1, 0x07060302u);
    }
  } else {
    // per packed word: 16 elements = raw pairs r0..r7 -> (x_i, x_{i+8}), i = 0..7
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t lo = raw[8 * j + i], hi = raw[8 * j + 4 + i];
        xs.p[8 * j + 2 * i] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        xs.p[8 * j + 2 * i + 1] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);
      }
    }
  }
}

enum XLoad : int { kXAligned = 0, kXUnaligned = 1, kXAgent = 2 };

// loads and permutes the lane's slice of x starting at element pointer x
template <int BITS, int MODE>
__device__ __forceinline__ XSlice<BITS> load_xslice(const uint16_t* x) {
  constexpr int kQuads = Fmt<BITS>::kElemsPer16B / 8;
  uint32_t raw[kQuads * 4];
  if constexpr (MODE == kXAgent) {
#pragma unroll
    for (int q = 0; q < kQuads; q += 4) {
      uint4 a[4];
      load_x32_agent(x + 8 * q, a);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        raw[4 * (q + i)] = a[i].x; raw[4 * (q + i) + 1] = a[i].y;
        raw[4 * (q + i) + 2] = a[i].z; raw[4 * (q + i) + 3] = a[i].w;
      }
    }
  } else {
#pragma unroll
    for (int q = 0; q < kQuads; ++q) {
      const uint4 a = load_x8<MODE == kXAligned>(x + 8 * q);
      raw[4 * q] = a.x; raw[4 * q + 1] = a.y; raw[4 * q + 2] = a.z; raw[4 * q + 3] = a.w;
    }
  }
  XSlice<BITS> xs;
  permute_x<BITS>(raw, xs);
  return xs;
}

// the same in two steps: request the lane's slice (16-byte aligned), permute it later
template <int BITS> struct XRaw { uint4 q[Fmt<BITS>::kElemsPer16B / 8]; };
template <int BITS>
__device__ __forceinline__ XRaw<BITS> load_xraw(const uint16_t* x) {
  XRaw<BITS> r;
#pragma unroll
  for (int q = 0; q < Fmt<BITS>::kElemsPer16B / 8; ++q) r.q[q] = load_x8<true>(x + 8 * q);
  return r;
}
template <int BITS>
__device__ __forceinline__ XSlice<BITS> make_xslice(const XRaw<BITS>& r) {
  constexpr int kQuads = Fmt<BITS>::kElemsPer16B / 8;
  uint32_t raw[kQuads * 4];
#pragma unroll
  for (int q = 0; q < kQuads; ++q) {
    raw[4 * q] = r.q[q].x; raw[4 * q + 1] = r.q[q].y; raw[4 * q + 2] = r.q[q].z; raw[4 * q + 3] = r.q[q].w;
  }
  XSlice<BITS> xs;
  permute_x<BITS>(raw, xs);
  return xs;
}

// sum over the lane's share of q * x
template <int BITS>
__device__ __forceinline__ float codes_dot(const uint4& codes, const XSlice<BITS>& xs) {
  const uint32_t ws[4] = {codes.x, codes.y, codes.z, codes.w};
  float dot = 0.0f;
  if constexpr (BITS == kBits4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w = ws[j];
      dot = dot2_bf16(and_or(w << 3, 0x00780078u, kMagic8), xs.p[4 * j + 0], dot);
      dot = dot2_bf16(and_or(w >> 1, 0x00780078u, kMagic8), xs.p[4 * j + 1], dot);
      dot = dot2_bf16(and_or(w >> 5, 0x00780078u, kMagic8), xs.p[4 * j + 2], dot);
      dot = dot2_bf16(and_or(w >> 9, 0x00780078u, kMagic8), xs.p[4 * j + 3], dot);
    }
    return 2.0f * __builtin_fmaf(-8.0f, xs.sum, dot);  // sum((8 + q/2) x) -> sum(q x)
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t w = ws[j];
      dot = dot2_bf16(and_or(w << 5, 0x00600060u, kMagic4), xs.p[8 * j + 0], dot);
      dot = dot2_bf16(and_or(w << 3, 0x00600060u, kMagic4), xs.p[8 * j + 1], dot);
      dot = dot2_bf16(and_or(w << 1, 0x00600060u, kMagic4), xs.p[8 * j + 2], dot);
#pragma unroll
      for (int i = 3; i < 8; ++i)
        dot = dot2_bf16(and_or(w >> (2 * i - 5), 0x00600060u, kMagic4), xs.p[8 * j + i], dot);
    }
    return __builtin_fmaf(-4.0f, xs.sum, dot);  // sum((4 + q) x) -> sum(q x)
  }
}

// convenience form: one row against a slice loaded on the spot
template <int BITS, bool ALIGNED>
__device__ __forceinline__ void lane_dot(const uint4& codes, const uint16_t* x, float& dot,
                                         float& sum) {
  const XSlice<BITS> xs = load_xslice<BITS, ALIGNED ? kXAligned : kXUnaligned>(x);
  dot = codes_dot<BITS>(codes, xs);
  sum = xs.sum;
}

// A lane's 64 two-bit codes as two runs of 32 (a gate projection quantized at group 32 has a
// scale / bias entry for each): sum(q x) and sum(x) of either run.
template <bool ALIGNED>
__device__ __forceinline__ void lane_dot_halves_q2(const uint4& codes, const uint16_t* x, float (&dot)[2],
                                                   float (&sum)[2]) {
  uint32_t raw[32];
#pragma unroll
  for (int q = 0; q < 8; ++q) {
    const uint4 a = load_x8<ALIGNED>(x + 8 * q);
    raw[4 * q] = a.x; raw[4 * q + 1] = a.y; raw[4 * q + 2] = a.z; raw[4 * q + 3] = a.w;
  }
  const uint32_t ws[4] = {codes.x, codes.y, codes.z, codes.w};
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    float s = 0.0f, d = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s = dot2_bf16(raw[16 * half + i], kOnes, s);
#pragma unroll
    for (int j = 2 * half; j < 2 * half + 2; ++j) {
      const uint32_t w = ws[j];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        // code i of the word pairs with code i + 8: raw pairs (x_2i', x_2i'+1) regrouped as (x_i, x_i+8)
        const uint32_t lo = raw[8 * j + (i >> 1)], hi = raw[8 * j + 4 + (i >> 1)];
        const uint32_t xp = (i & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u) : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        const uint32_t cw = i < 3 ? w << (5 - 2 * i) : w >> (2 * i - 5);
        d = dot2_bf16(and_or(cw, 0x00600060u, kMagic4), xp, d);
      }
    }
    sum[half] = s;
    dot[half] = __builtin_fmaf(-4.0f, s, d);  // sum((4 + q) x) -> sum(q x)
  }
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

}  // namespace mf
