// Group-quantized GEMV (1..8 token rows against one read of each weight row),
// the fused shared-expert gate/up/activation kernel, and the three elementwise
// ops of the path.  One wave64 owns one or more rows; each lane reads 16 bytes
// of packed codes per step (32 four-bit / 64 two-bit elements), dequantizes in
// registers with the factored form s*sum(q*x) + b*sum(x)
// (Metal/Quant/dequant_int4.metal:14-17) and the row is finished by a wave
// butterfly.
#include "mf_device.h"
#include "mf_internal.h"
#include "mf_router.h"

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

// Streaming form of the two kernels above for wide matrices: a wave keeps its
// slices of x (already permuted, with their sums) in registers for the whole
// launch and walks down the rows, so the only traffic per row is the codes and
// the scale/bias entries.  The next row's loads are issued before the current
// row's arithmetic.  ITS (compile time) bounds the 16-byte steps a lane takes
// along a row; wpr waves (1, 2 or 4) split a row when it is longer than one
// wave can hold in registers, and their partial sums meet in LDS in wave order.
// NPROJ 2 is the gate/up pair with the shared-expert activation
// (dequant_int4.metal:216-246); NPROJ 1 is the plain GEMV.
struct RowsArgs {
  const uint8_t* W[2];
  const uint16_t* S[2];
  const uint16_t* B[2];
  const uint16_t* x;   // [T, N]
  void* y;             // NPROJ 1: [T, M] bf16 or fp32; NPROJ 2: act [T, M] bf16
  uint32_t M, N;
  uint32_t wpr;        // waves per row
  int out_f32;
};

template <int BITS, int T, int ITS, int NPROJ>
__global__ __launch_bounds__(256) void rows_stream_kernel(const RowsArgs a) {
  // rows in flight per wave: HBM under load answers in 2-3 us and a row's arithmetic is under 1 us
  constexpr int DEPTH = 2;
  constexpr int EPL = Fmt<BITS>::kElemsPer16B;
  __shared__ float s_part[4][T][NPROJ];
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const uint32_t wpr = a.wpr, slot = wv / wpr, part = wv % wpr, rows_per_wg = 4 / wpr;
  const uint32_t n_groups = a.N / kGroup;
  const size_t row_bytes = static_cast<size_t>(a.N) * Store<BITS>::kBits / 8;

  // the lane's columns: step it covers elements [(it * wpr + part) * 64 + lane] * EPL ...
  uint32_t e0[ITS];
  bool live[ITS];
  XSlice<BITS> xs[T][ITS];
#pragma unroll
  for (int it = 0; it < ITS; ++it) {
    e0[it] = ((it * wpr + part) * 64 + lane) * EPL;
    live[it] = e0[it] < a.N;
    if (!live[it]) e0[it] = 0;
#pragma unroll
    for (int t = 0; t < T; ++t) {
      xs[t][it] = load_xslice<BITS, kXAligned>(a.x + static_cast<size_t>(t) * a.N + e0[it]);
      if (!live[it]) {
#pragma unroll
        for (int i = 0; i < XSlice<BITS>::kPairs; ++i) xs[t][it].p[i] = 0;
        xs[t][it].sum = 0.0f;
      }
    }
  }

  // The scale / bias entries of one row: this wave's steps meet GPS = 64 * EPL / 64 groups
  // each; one load per table brings them in (lane l holds entry l of step-major order, the
  // wave's steps being wpr * GPS apart in the row), a cross-lane read hands each lane its own.
  constexpr int GPS = EPL;                         // groups per wave step
  constexpr int TW = (ITS * GPS + 63) / 64;        // table words per lane
  uint32_t tab_g[TW];                              // group index this lane fetches
  bool tab_ok[TW];
#pragma unroll
  for (int k = 0; k < TW; ++k) {
    const uint32_t j = k * 64 + lane, it = j / GPS;
    tab_g[k] = (it * wpr + part) * GPS + j % GPS;
    tab_ok[k] = it < static_cast<uint32_t>(ITS) && tab_g[k] < n_groups;
    if (!tab_ok[k]) tab_g[k] = 0;
  }
  int tab_src[ITS];                                // lane holding this lane's entry of step it,
#pragma unroll                                     // in table word (it * GPS) / 64
  for (int it = 0; it < ITS; ++it) tab_src[it] = static_cast<int>((it * GPS + lane * EPL / kGroup) & 63u) << 2;
  uint4 codes[DEPTH][NPROJ][ITS];
  uint32_t sraw[DEPTH][NPROJ][TW], braw[DEPTH][NPROJ][TW];
  const uint32_t stride = gridDim.x * rows_per_wg;
  const uint32_t row0 = blockIdx.x * rows_per_wg + slot;
  const uint32_t row_end = (a.M + stride - 1) / stride * stride;  // every wave runs the same trip count
#define MF_FETCH(U, ROW)                                                                            \
  do {                                                                                              \
    const size_t fr = (ROW) < a.M ? (ROW) : a.M - 1;                                                \
    _Pragma("unroll") for (int p = 0; p < NPROJ; ++p) {                                             \
      _Pragma("unroll") for (int it = 0; it < ITS; ++it)                                            \
        codes[U][p][it] = *reinterpret_cast<const uint4*>(                                          \
            a.W[p] + fr * row_bytes + static_cast<size_t>(e0[it]) * Store<BITS>::kBits / 8);        \
      _Pragma("unroll") for (int k = 0; k < TW; ++k) {                                              \
        sraw[U][p][k] = a.S[p][fr * n_groups + tab_g[k]];                                           \
        if constexpr (BITS != kBitsTernary) braw[U][p][k] = a.B[p][fr * n_groups + tab_g[k]];       \
      }                                                                                             \
    }                                                                                               \
  } while (0)
#pragma unroll
  for (int u = 0; u < DEPTH; ++u) MF_FETCH(u, row0 + u * stride);

  for (uint32_t base = row0; base < row_end; base += DEPTH * stride) {
#pragma unroll
  for (int u = 0; u < DEPTH; ++u) {
    const uint32_t row = base + u * stride;
    if (row >= row_end) break;
    float sc[NPROJ][ITS], bi[NPROJ][ITS];
#pragma unroll
    for (int p = 0; p < NPROJ; ++p)
#pragma unroll
      for (int it = 0; it < ITS; ++it) {
        uint32_t sv = 0, bv = 0;
        sv = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(tab_src[it], static_cast<int>(sraw[u][p][(it * GPS) / 64])));
        if constexpr (BITS != kBitsTernary)
          bv = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(tab_src[it], static_cast<int>(braw[u][p][(it * GPS) / 64])));
        sc[p][it] = __uint_as_float(sv << 16);
        if constexpr (BITS == kBitsTernary) bi[p][it] = -sc[p][it];
        else bi[p][it] = __uint_as_float(bv << 16);
      }

    float acc[T][NPROJ];
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int p = 0; p < NPROJ; ++p) acc[t][p] = 0.0f;
#pragma unroll
    for (int it = 0; it < ITS; ++it)
#pragma unroll
      for (int p = 0; p < NPROJ; ++p)
#pragma unroll
        for (int t = 0; t < T; ++t) {
          const float dot = codes_dot<BITS>(codes[u][p][it], xs[t][it]);
          acc[t][p] = __builtin_fmaf(sc[p][it], dot, acc[t][p]);
          acc[t][p] = __builtin_fmaf(bi[p][it], xs[t][it].sum, acc[t][p]);
        }
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int p = 0; p < NPROJ; ++p) acc[t][p] = wave_sum(acc[t][p]);
    if (wpr > 1) {
      if (lane == 0) {
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
          for (int p = 0; p < NPROJ; ++p) s_part[wv][t][p] = acc[t][p];
      }
      __syncthreads();
      if (part == 0) {
#pragma unroll
        for (int t = 0; t < T; ++t)
#pragma unroll
          for (int p = 0; p < NPROJ; ++p) {
            float v = s_part[wv][t][p];
            for (uint32_t q = 1; q < wpr; ++q) v = v + s_part[wv + q][t][p];
            acc[t][p] = v;
          }
      }
      __syncthreads();
    }
    if (part == 0 && lane == 0 && row < a.M) {
#pragma unroll
      for (int t = 0; t < T; ++t) {
        const size_t at = static_cast<size_t>(t) * a.M + row;
        if constexpr (NPROJ == 2) {
          const float rg = round_bf16(acc[t][0]), ru = round_bf16(acc[t][1]);
          static_cast<uint16_t*>(a.y)[at] = f_to_bf16(mf_silu(rg) * ru);
        } else if (a.out_f32) {
          static_cast<float*>(a.y)[at] = acc[t][0];
        } else {
          static_cast<uint16_t*>(a.y)[at] = f_to_bf16(acc[t][0]);
        }
      }
    }
    if (row + DEPTH * stride < row_end) MF_FETCH(u, row + DEPTH * stride);  // refill the slot just consumed
  }
  }
#undef MF_FETCH
}

// Matrix-core form of the same two operations (4-bit codes, T <= 8).  The vector ALU is what
// limits the streaming kernel: extracting a code and feeding it to a dot product costs about
// three instructions per code.  Here a code costs one (mask-and-or into a bf16 operand) and the
// bf16 matrix core does the products: per 64-wide K group, D[token, row] = sum x * (8 + q/2) over
// four 32x32x16 MFMAs with the tokens as the (mostly empty) M side, so a lane ends up with ONE
// weight row and the group's scale is a per-lane scalar, applied to the T live accumulator rows
// only.  A workgroup is one block of 32 weight rows; its KS waves split K, each keeps the x rows
// of its K range (pre-ordered for the code pairing, with their group sums) in its own part of
// LDS, and the partial sums meet in LDS in wave order.  Bias and offset terms are MFMAs over the
// group index, as in the prefill matmul.
struct RowsMfmaArgs {
  const uint8_t* W[2];
  const uint16_t* S[2];
  const uint16_t* B[2];
  const uint16_t* x;   // [T, N]
  void* y;             // NPROJ 1: [T, M] bf16 or fp32; NPROJ 2: act [T, M] bf16
  uint32_t M, N, T;
  uint32_t gps;        // K groups per wave (a multiple of 4)
  int out_f32;
};

template <int NPROJ, int KS>
__global__ __launch_bounds__(KS * 64) void rows_mfma_kernel(const RowsMfmaArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const uint32_t lane = threadIdx.x & 63, ks = threadIdx.x >> 6, n_ks = KS;
  const uint32_t m = lane & 31, h = lane >> 5;
  const uint32_t T = a.T, ng = a.N / kGroup;
  const uint32_t gps = a.gps;                               // K groups per wave
  const uint32_t g_begin = min(ng, ks * gps), g_end = min(ng, g_begin + gps), n_g = g_end - g_begin;
  const uint32_t row = blockIdx.x * 32 + m, row_c = min(row, a.M - 1);
  const size_t row_bytes = static_cast<size_t>(a.N) / 2;

  // this wave's LDS: x operands [group][s][h][token] x 16 B, then group sums [token][group] fp32
  uint4* s_xw = reinterpret_cast<uint4*>(smem + static_cast<size_t>(ks) * gps * (8 * T * 16 + T * 4));
  float* s_sum = reinterpret_cast<float*>(s_xw + gps * 8 * T);

  // codes of the first four groups are on their way while x is staged
  const uint8_t* wrow[NPROJ];
  uint4 cur[NPROJ][4], nxt[NPROJ][4];
#pragma unroll
  for (int p = 0; p < NPROJ; ++p) {
    wrow[p] = a.W[p] + row_c * row_bytes + static_cast<size_t>(g_begin) * 32 + h * 16;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      cur[p][u] = make_uint4(0, 0, 0, 0);
      if (static_cast<uint32_t>(u) < n_g) cur[p][u] = *reinterpret_cast<const uint4*>(wrow[p] + u * 32);
    }
  }

  // ---- stage x: 8-value runs re-ordered to (0,4,1,5,2,6,3,7), one lane per run
  const uint32_t runs = n_g * 8;
  for (uint32_t i0 = 0; i0 < T * runs; i0 += kWave) {
    const uint32_t i = i0 + lane;
    const bool in = i < T * runs;
    const uint32_t t = in ? i / runs : 0, c = in ? i % runs : 0;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (in) v = *reinterpret_cast<const uint4*>(a.x + static_cast<size_t>(t) * a.N + (g_begin * 8 + c) * 8);
    float sum = ((bf16_lo(v.x) + bf16_hi(v.x)) + (bf16_lo(v.y) + bf16_hi(v.y))) +
                ((bf16_lo(v.z) + bf16_hi(v.z)) + (bf16_lo(v.w) + bf16_hi(v.w)));
    sum = group_sum(sum, 8);
    if (in) {
      const uint32_t gl = c >> 3, ci = c & 7;
      s_xw[((gl * 4 + (ci & 3)) * 2 + (ci >> 2)) * T + t] =
          make_uint4(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u), __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                     __builtin_amdgcn_perm(v.w, v.y, 0x05040100u), __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));
      if (ci == 0) s_sum[t * gps + gl] = sum;
    }
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave reads back what its lanes wrote
  __builtin_amdgcn_wave_barrier();

  const uint32_t tok = m < T ? m : 0;  // accumulator rows past T read token 0 and are never stored
  f32x16_t acc[NPROJ];
#pragma unroll
  for (int p = 0; p < NPROJ; ++p)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[p][r] = 0.0f;

  // ---- bias and offset terms: acc[token, row] += sumx[token, g] * (B[row, g] - 16 S[row, g])
  for (uint32_t g0 = 0; g0 < n_g; g0 += 16) {
    const uint32_t gl = g0 + 8 * h;
    const bool have = gl < n_g;
    const uint32_t gc = have ? gl : 0;
    uint4 ab[NPROJ], as[NPROJ];
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      const size_t at = static_cast<size_t>(row_c) * ng + g_begin + gc;
      ab[p] = load_bf16x8_guarded(a.B[p] + at, n_g - gc);
      const uint4 sv = load_bf16x8_guarded(a.S[p] + at, n_g - gc);
      as[p] = make_uint4((sv.x + 0x02000200u) ^ 0x80008000u, (sv.y + 0x02000200u) ^ 0x80008000u,
                         (sv.z + 0x02000200u) ^ 0x80008000u, (sv.w + 0x02000200u) ^ 0x80008000u);
      if (!have) ab[p] = as[p] = make_uint4(0, 0, 0, 0);
    }
    uint32_t hi[8], mid[8], lo[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = (m < T && gc + e < n_g) ? s_sum[tok * gps + gc + e] : 0.0f;
      hi[e] = __float_as_uint(v) & 0xFFFF0000u;
      const float r1 = v - __uint_as_float(hi[e]);
      mid[e] = __float_as_uint(r1) & 0xFFFF0000u;
      lo[e] = __float_as_uint(r1 - __uint_as_float(mid[e]));
    }
    const uint4 b_hi = make_uint4((hi[0] >> 16) | hi[1], (hi[2] >> 16) | hi[3], (hi[4] >> 16) | hi[5],
                                  (hi[6] >> 16) | hi[7]);
    const uint4 b_mid = make_uint4((mid[0] >> 16) | mid[1], (mid[2] >> 16) | mid[3], (mid[4] >> 16) | mid[5],
                                   (mid[6] >> 16) | mid[7]);
    const uint4 b_lo = make_uint4(__builtin_amdgcn_perm(lo[1], lo[0], 0x07060302u),
                                  __builtin_amdgcn_perm(lo[3], lo[2], 0x07060302u),
                                  __builtin_amdgcn_perm(lo[5], lo[4], 0x07060302u),
                                  __builtin_amdgcn_perm(lo[7], lo[6], 0x07060302u));
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      acc[p] = mfma_bf16(b_hi, ab[p], acc[p]);
      acc[p] = mfma_bf16(b_hi, as[p], acc[p]);
      acc[p] = mfma_bf16(b_mid, ab[p], acc[p]);
      acc[p] = mfma_bf16(b_mid, as[p], acc[p]);
      acc[p] = mfma_bf16(b_lo, ab[p], acc[p]);
      acc[p] = mfma_bf16(b_lo, as[p], acc[p]);
    }
  }

  // ---- main loop, four K groups per step; the next step's codes and scales are in flight
  for (uint32_t g0 = 0; g0 < n_g; g0 += 4) {
    uint2 sraw[NPROJ];
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      const uint16_t* sp = a.S[p] + static_cast<size_t>(row_c) * ng + g_begin + g0;
      if (g0 + 4 <= n_g) {
        sraw[p] = *reinterpret_cast<const uint2*>(sp);  // 8-byte aligned: ng, gps and g0 are multiples of 4
      } else {
        uint32_t q[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) q[e] = g0 + e < n_g ? sp[e] : 0u;
        sraw[p] = make_uint2(q[0] | (q[1] << 16), q[2] | (q[3] << 16));
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        nxt[p][v] = cur[p][v];
        if (g0 + 4 + v < n_g) nxt[p][v] = *reinterpret_cast<const uint4*>(wrow[p] + (g0 + 4 + v) * 32);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t gl = g0 + u;
      if (gl >= n_g) break;
      uint4 ax[4];
#pragma unroll
      for (int s4 = 0; s4 < 4; ++s4) ax[s4] = s_xw[((gl * 4 + s4) * 2 + h) * T + tok];
#pragma unroll
      for (int p = 0; p < NPROJ; ++p) {
        const uint32_t cw[4] = {cur[p][u].x, cur[p][u].y, cur[p][u].z, cur[p][u].w};
        const uint32_t sw = u < 2 ? sraw[p].x : sraw[p].y;
        const float sc = 2.0f * ((u & 1) ? bf16_hi(sw) : bf16_lo(sw));
        f32x16_t tmp;
#pragma unroll
        for (int r = 0; r < 16; ++r) tmp[r] = 0.0f;
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) tmp = mfma_bf16(ax[s4], expand_q4(cw[s4]), tmp);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[p][r] = __builtin_fmaf(sc, tmp[r], acc[p][r]);  // tokens 4h + r
      }
    }
#pragma unroll
    for (int p = 0; p < NPROJ; ++p)
#pragma unroll
      for (int v = 0; v < 4; ++v) cur[p][v] = nxt[p][v];
  }

  // ---- the K splits meet: [wave][projection][token 0..7][32 rows], over the x area
  __syncthreads();
  float* s_comb = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int p = 0; p < NPROJ; ++p)
#pragma unroll
    for (int r = 0; r < 4; ++r) s_comb[((ks * NPROJ + p) * 8 + 4 * h + r) * 32 + m] = acc[p][r];
  __syncthreads();
  if (threadIdx.x < T * 32) {
    const uint32_t t = threadIdx.x >> 5, mm = threadIdx.x & 31, orow = blockIdx.x * 32 + mm;
    float v[NPROJ];
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      v[p] = 0.0f;
      for (uint32_t q = 0; q < n_ks; ++q) v[p] = v[p] + s_comb[((q * NPROJ + p) * 8 + t) * 32 + mm];
    }
    if (orow < a.M) {
      const size_t at = static_cast<size_t>(t) * a.M + orow;
      if constexpr (NPROJ == 2) {
        const float rg = round_bf16(v[0]), ru = round_bf16(v[1]);
        static_cast<uint16_t*>(a.y)[at] = f_to_bf16(mf_silu(rg) * ru);
      } else if (a.out_f32) {
        static_cast<float*>(a.y)[at] = v[0];
      } else {
        static_cast<uint16_t*>(a.y)[at] = f_to_bf16(v[0]);
      }
    }
  }
}

// Quad form for 1..4 token rows of a wide 4-bit matrix.  v_mfma_f32_4x4x4_16b_bf16 multiplies
// sixteen independent 4x4x4 blocks, one per quad of lanes.  Block b takes the K positions of the
// 16-byte code chunks b, b + 16, ... of a row, so the lanes of a wave read 4 weight rows x 256
// contiguous bytes per load, and the x values a lane meets never change: they stay in registers
// as the A operand (lane (b, r) holds token r), pre-ordered for the code pairing of expand_q4,
// next to their per-chunk sums.  The B operand is the chunk's codes of weight row c = lane % 4 as
// the bf16 numbers 8 + q/2, so the result D[token, row] puts ONE weight row in a lane (its four
// token sums in four registers) and the group's scale is a per-lane scalar:
//   acc[t] += 2 s * (sum x (8 + q/2))            4 fma per chunk
//   acc[t] += b * sum(x) - 16 s * sum(x)         two more matrix instructions per chunk (sum(x) as
//                                                three bf16 terms: exact products)
// Every token count 1..4 runs the same instructions on its own A rows: a token's result does
// not depend on how many tokens ride along.  The waves of a workgroup split the chunks of a row
// set (4 rows); partial sums meet in LDS in a fixed order.
struct RowsQuadArgs {
  const uint8_t* W[2];
  const uint16_t* S[2];
  const uint16_t* B[2];
  const uint16_t* x;   // [T, N]
  void* y;             // NPROJ 1: [T, M] bf16 or fp32; NPROJ 2: act [T, M] bf16
  uint32_t M, N, T;    // M % 4 == 0, N % 64 == 0, T <= 4
  int out_f32;
};

typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

__device__ __forceinline__ f32x4_t mfma_quad(uint2 a, uint2 b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4_t, a), __builtin_bit_cast(s16x4_t, b), c,
                                                0, 0, 0);
}

constexpr uint32_t kQuadMaxWaves = 8;

template <int NPROJ, int ITS>
__global__ __launch_bounds__(kQuadMaxWaves * 64) void rows_quad_kernel(const RowsQuadArgs a) {
  // partial sums [buffer][projection][wave][16-lane row][weight row][token]
  __shared__ __attribute__((aligned(16))) float s_part[2][NPROJ][kQuadMaxWaves][4][4][4];
  // scale / bias pieces [wave][ring slot][(table, row, piece)][8 groups]
  __shared__ __attribute__((aligned(16))) uint16_t s_tab[kQuadMaxWaves][2][64 * 8];
  const uint32_t lane = threadIdx.x & 63, wsub = threadIdx.x >> 6, wpr = blockDim.x >> 6;
  const uint32_t b = lane >> 2, c = lane & 3;
  const uint32_t n_chunks = a.N / 32, ng = a.N / kGroup, n_sets = a.M / 4;
  const size_t row_bytes = static_cast<size_t>(a.N) / 2;

  // chunk of every slot of this lane: (wsub * ITS + j) * 16 + b
  uint32_t chc[ITS];
  uint2 xa[ITS][8], sx[ITS];  // this lane's x operands and chunk sums (filled below)
#pragma unroll
  for (int j = 0; j < ITS; ++j)
    chc[j] = min((wsub * ITS + j) * 16 + b, n_chunks - 1);  // a slot past the row reads the last chunk against x = 0

  // Codes and table entries of two stages (a stage = one projection of one row set) live in a
  // ring of registers: a slot is refilled, as soon as it has been used, with the same slot of
  // the stage two ahead, so between one and two stages of loads are in flight all the time.
  // The scales and biases a wave needs for one stage are 8 * ITS consecutive groups of each of its
  // 4 rows: lanes 0 .. 8 * ITS - 1 fetch them as 16-byte pieces ((table, row, piece) per lane) in
  // ONE load instruction issued with the first refill of the stage that frees the ring slot; the
  // piece goes to the wave's own LDS area when that stage ends, and a lane picks the two values of
  // each slot from there (LDS reads cost no vector-memory issue slot,
  // which is what limits this kernel).
  uint4 cw[2][ITS];
  // (lanes past 8 * ITS fetch and store a copy nobody reads: no branch around the load)
  const uint32_t tb_lane = lane % (8 * ITS);
  const uint32_t tb_bias = tb_lane / (4 * ITS), tb_row = (tb_lane / ITS) & 3u, tb_piece = tb_lane % ITS;
  const uint32_t tb_g = (wsub * ITS + tb_piece) * 8;
  const uint32_t tb_group = tb_g < ng ? tb_g : 0u;  // a piece past the row is never used: read piece 0
  uint16_t* my_tab = &s_tab[wsub][0][0];
  auto fetch = [&](int buf, int j, uint32_t set, int p) __attribute__((always_inline)) {
    const size_t row = static_cast<size_t>(set) * 4 + c;
    cw[buf][j] = *reinterpret_cast<const uint4*>(a.W[p] + row * row_bytes + static_cast<size_t>(chc[j]) * 16);
  };
  auto fetch_tables = [&](uint32_t set, int p) __attribute__((always_inline)) {
    return *reinterpret_cast<const uint4*>((tb_bias ? a.B[p] : a.S[p]) + (static_cast<size_t>(set) * 4 + tb_row) * ng +
                                           tb_group);
  };
  // the wave's part of D[token, row] for one row set; then the four blocks of each 16-lane row
  // are added and lanes 0..3 of the row leave [weight row][token] in LDS.  `refill` is the row
  // set whose stage takes over the ring slots.
  auto compute = [&](int buf, int p, uint32_t pb, uint32_t refill) __attribute__((always_inline)) {
    f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
    uint16_t* tab = my_tab + buf * (64 * 8);
    __builtin_amdgcn_wave_barrier();  // the wave reads back what its own lanes wrote (LDS keeps order)
    uint4 tbn = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int j = 0; j < ITS; ++j) {
      const uint32_t w[4] = {cw[buf][j].x, cw[buf][j].y, cw[buf][j].z, cw[buf][j].w};
      f32x4_t tmp = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint4 e = expand_q4(w[i]);
        tmp = mfma_quad(xa[j][2 * i], make_uint2(e.x, e.y), tmp);
        tmp = mfma_quad(xa[j][2 * i + 1], make_uint2(e.z, e.w), tmp);
      }
      const uint32_t sb = tab[((c * ITS) + j) * 8 + (b >> 1)], bb = tab[(((4 + c) * ITS) + j) * 8 + (b >> 1)];
      const uint32_t ms = ((sb + 0x0200u) ^ 0x8000u) & 0xFFFFu;  // -16 s: exponent + 4, sign flipped
      acc = mfma_quad(sx[j], make_uint2(bb | (bb << 16), bb), acc);
      acc = mfma_quad(sx[j], make_uint2(ms | (ms << 16), ms), acc);
      const float s2 = 2.0f * __uint_as_float(sb << 16);
      fetch(buf, j, refill, p);
      if (j == 0) tbn = fetch_tables(refill, p);
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[t] = __builtin_fmaf(s2, tmp[t], acc[t]);
    }
    // every read of this ring slot's tables is issued: the refill stage's pieces take their place
    __builtin_amdgcn_wave_barrier();
    *reinterpret_cast<uint4*>(tab + lane * 8) = tbn;
    float v[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      v[t] = acc[t] + dpp_f<0x124>(acc[t]);  // + lane - 4 (rotation inside the 16-lane row)
      v[t] = v[t] + dpp_f<0x128>(v[t]);      // + lane - 8
    }
    if ((lane & 12u) == 0)
      *reinterpret_cast<float4*>(&s_part[pb][p][wsub][lane >> 4][c][0]) = make_float4(v[0], v[1], v[2], v[3]);
  };
  // threads 0..15: (weight row, token) totals in wave then row order
  auto combine = [&](uint32_t set, uint32_t pb) __attribute__((always_inline)) {
    if (threadIdx.x >= 16) return;
    const uint32_t cc = threadIdx.x & 3, t = threadIdx.x >> 2;
    float v[NPROJ];
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      v[p] = 0.0f;
      for (uint32_t w = 0; w < wpr; ++w)
#pragma unroll
        for (int r = 0; r < 4; ++r) v[p] = v[p] + s_part[pb][p][w][r][cc][t];
    }
    if (t >= a.T) return;
    const size_t at = static_cast<size_t>(t) * a.M + set * 4 + cc;
    if constexpr (NPROJ == 2) {
      const float rg = round_bf16(v[0]), ru = round_bf16(v[1]);
      static_cast<uint16_t*>(a.y)[at] = f_to_bf16(mf_silu(rg) * ru);
    } else if (a.out_f32) {
      static_cast<float*>(a.y)[at] = v[0];
    } else {
      static_cast<uint16_t*>(a.y)[at] = f_to_bf16(v[0]);
    }
  };

  // Refills past the last row set read the last row set again (loaded, never used): no branch
  // splits the unrolled stage.
  const uint32_t G = gridDim.x, last = n_sets - 1;
  uint32_t set = blockIdx.x, pb = 0;
  if (set >= n_sets) return;
  const uint32_t set1 = NPROJ == 2 ? set : min(set + G, last);
  const uint4 t0 = fetch_tables(set, 0), t1 = fetch_tables(set1, NPROJ == 2 ? 1 : 0);
#pragma unroll
  for (int j = 0; j < ITS; ++j) {
    fetch(0, j, set, 0);
    fetch(1, j, set1, NPROJ == 2 ? 1 : 0);
  }
  // ---- this lane's x: token c, chunks (wsub * ITS + j) * 16 + b.  The first two stages' weight
  // loads are already on their way: the x rows come from L2 behind them.
#pragma unroll
  for (int j = 0; j < ITS; ++j) {
    const uint32_t ch = (wsub * ITS + j) * 16 + b;
    const bool live = ch < n_chunks && c < a.T;
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint4 v = make_uint4(0, 0, 0, 0);
      if (live) v = *reinterpret_cast<const uint4*>(a.x + static_cast<size_t>(c) * a.N + chc[j] * 32 + 8 * i);
      xa[j][2 * i] = make_uint2(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u),   // (e0, e4)
                                __builtin_amdgcn_perm(v.z, v.x, 0x07060302u));  // (e1, e5)
      xa[j][2 * i + 1] = make_uint2(__builtin_amdgcn_perm(v.w, v.y, 0x05040100u),   // (e2, e6)
                                    __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));  // (e3, e7)
      const uint32_t pr[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) sum = (sum + bf16_lo(pr[e])) + bf16_hi(pr[e]);
    }
    const uint32_t hi = __float_as_uint(sum) & 0xFFFF0000u;
    const float r1 = sum - __uint_as_float(hi);
    const uint32_t mid = __float_as_uint(r1) & 0xFFFF0000u;
    const uint32_t lo = __float_as_uint(r1 - __uint_as_float(mid));
    sx[j] = make_uint2((hi >> 16) | mid, lo >> 16);  // K slots: hi, mid, lo, 0
  }

  *reinterpret_cast<uint4*>(my_tab + lane * 8) = t0;
  *reinterpret_cast<uint4*>(my_tab + 64 * 8 + lane * 8) = t1;
  if constexpr (NPROJ == 2) {
    for (; set < n_sets; set += G) {
      const uint32_t nxt = min(set + G, last);
      compute(0, 0, pb, nxt);
      compute(1, 1, pb, nxt);
      __syncthreads();  // the other buffer stays untouched until every wave has passed this point again
      combine(set, pb);
      pb ^= 1u;
    }
  } else {
    for (;;) {
      compute(0, 0, pb, min(set + 2 * G, last));
      __syncthreads();
      combine(set, pb);
      pb ^= 1u;
      const uint32_t s1 = set + G;
      if (s1 >= n_sets) break;
      compute(1, 0, pb, min(s1 + 2 * G, last));
      __syncthreads();
      combine(s1, pb);
      pb ^= 1u;
      set = s1 + G;
      if (set >= n_sets) break;
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

// 8-bit affine rows (dequant_int8_gemv_simd, Metal/Quant/dequant_int8.metal:66-107): one wave per
// (token, row) in the lane order of dot_q8_row, so a token's value does not depend on how many tokens ride along.
__global__ __launch_bounds__(256) void gemv_q8_kernel(const uint8_t* __restrict__ W, const uint16_t* __restrict__ S,
                                                      const uint16_t* __restrict__ B, const uint16_t* __restrict__ x,
                                                      void* __restrict__ y, uint32_t m, uint32_t n, uint32_t t,
                                                      int out_f32, int aligned) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (wave >= m * t) return;
  const uint32_t tok = wave / m, row = wave % m;
  const uint32_t ng = n / kGroup;
  const float v = dot_q8_row(W + static_cast<size_t>(row) * n, S + static_cast<size_t>(row) * ng,
                             B + static_cast<size_t>(row) * ng, x + static_cast<size_t>(tok) * n, n, lane, aligned != 0);
  if (lane == 0) {
    const size_t at = static_cast<size_t>(tok) * m + row;
    if (out_f32) static_cast<float*>(y)[at] = v;
    else static_cast<uint16_t*>(y)[at] = f_to_bf16(v);
  }
}

// shared_int8_gate_up_act_simd (dequant_int8.metal:110-164): the gate and up rows of an 8-bit MLP in one pass,
// both narrowed to 16 bits, act = narrow(activation(gate) * up); the activation is the tanh form of GELU or,
// with the reference's FC_SHARED_INT8_ACT_SILU, SiLU.  One wave per (token, row), dot_q8_row's lane order.
template <bool SILU>
__global__ __launch_bounds__(256) void gate_up_act_q8_kernel(const uint8_t* __restrict__ Wg, const uint16_t* __restrict__ Sg,
                                                             const uint16_t* __restrict__ Bg, const uint8_t* __restrict__ Wu,
                                                             const uint16_t* __restrict__ Su, const uint16_t* __restrict__ Bu,
                                                             const uint16_t* __restrict__ x, uint16_t* __restrict__ act,
                                                             uint32_t m, uint32_t n, uint32_t t, int aligned) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (wave >= m * t) return;
  const uint32_t tok = wave / m, row = wave % m;
  const uint32_t ng = n / kGroup;
  const uint16_t* xt = x + static_cast<size_t>(tok) * n;
  const float g = dot_q8_row(Wg + static_cast<size_t>(row) * n, Sg + static_cast<size_t>(row) * ng,
                             Bg + static_cast<size_t>(row) * ng, xt, n, lane, aligned != 0);
  const float u = dot_q8_row(Wu + static_cast<size_t>(row) * n, Su + static_cast<size_t>(row) * ng,
                             Bu + static_cast<size_t>(row) * ng, xt, n, lane, aligned != 0);
  if (lane == 0) {
    const float gh = round_bf16(g), uh = round_bf16(u);
    const float a = SILU ? mf_silu(gh) : mf_gelu_tanh(gh);
    act[static_cast<size_t>(tok) * m + row] = f_to_bf16(a * uh);
  }
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

// Picks the streaming kernel when the shape fits one of its instantiations:
// 16-byte aligned operands, N a multiple of the group, T in {1, 2, 4}, and a
// (wpr, ITS) split with T * ITS x-slices small enough to stay in registers.
uint32_t device_cu_count() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (!cached[dev]) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return static_cast<uint32_t>(cached[dev]);
}

template <int BITS, int NPROJ>
bool rows_stream_try(hipStream_t s, const RowsArgs& in, uint32_t t, uint32_t num_cu, hipError_t& err) {
  constexpr int EPL = Fmt<BITS>::kElemsPer16B;
  if (in.N % kGroup || in.N < 64 * EPL || (t != 1 && t != 2 && t != 4) || in.M < 1024) return false;
  const uint32_t steps = (in.N + 64 * EPL - 1) / (64 * EPL);  // 16-byte steps of one wave along a row
  // x slices live in registers for the whole launch: T x its x (pairs + sum).  A 2-bit slice is 33
  // registers, and with two projections in flight the 9-step and the 4-token 3-step instances spill.
  constexpr bool wide_slices = BITS == kBits2 && NPROJ == 2;
  const uint32_t max_its = t == 1 ? (wide_slices ? 3 : 9) : (wide_slices && t == 4 ? 1 : 3);
  if (BITS == kBitsTernary) return false;
  uint32_t wpr = 1;
  while (wpr < 4 && (steps + wpr - 1) / wpr > max_its) wpr *= 2;
  // few rows and long rows: split the rows so that every wave still walks a useful number of them
  while (wpr < 4 && in.M / wpr < num_cu * 8 * 4 && (steps + wpr - 1) / wpr > 2) wpr *= 2;
  const uint32_t its = (steps + wpr - 1) / wpr;
  if (its > max_its) return false;
  RowsArgs a = in;
  a.wpr = wpr;
  const uint32_t rows_per_wg = 4 / wpr;
  const uint32_t grid = std::min<uint32_t>((a.M + rows_per_wg - 1) / rows_per_wg, num_cu * (t == 1 ? 3u : 2u));
#define MF_ROWS(TT, II)                                                                      \
  rows_stream_kernel<BITS, TT, II, NPROJ><<<dim3(grid), dim3(256), 0, s>>>(a)
  if constexpr (BITS != kBitsTernary) {
    if (t == 1) {
      if (its == 1) MF_ROWS(1, 1);
      else if (its <= 3) MF_ROWS(1, 3);
      else if constexpr (!wide_slices) MF_ROWS(1, 9);
    } else if (t == 2) {
      if (its == 1) MF_ROWS(2, 1); else MF_ROWS(2, 3);
    } else {
      if (its == 1) MF_ROWS(4, 1);
      else if constexpr (!wide_slices) MF_ROWS(4, 3);
    }
  }
#undef MF_ROWS
  err = hipGetLastError();
  return true;
}

// The matrix-core kernel takes 4-bit matrices with at least 1024 rows whose K is a multiple of
// 256 (so that the per-wave group ranges start on 8-byte boundaries of the scale table), up to 8
// token rows, when the x rows of one workgroup fit LDS.
template <int NPROJ>
bool rows_mfma_try(hipStream_t s, const RowsMfmaArgs& a, uint32_t num_cu, hipError_t& err) {
  const uint32_t ng = a.N / kGroup;
  // one or two token rows stream faster through rows_stream_kernel (1 KB contiguous per load
  // instruction against 32-byte pieces of 32 rows here); from three rows on the dot products
  // outweigh that
  if (a.N % (4 * kGroup) || a.N < 2048 || a.T < 3 || a.T > 8 || a.M < 1024) return false;
  const uint32_t blocks = (a.M + 31) / 32;
  // enough waves to fill the chip: 4 K-splits when there are many row blocks, 16 when few
  uint32_t n_ks = blocks * 4 >= num_cu * 8 ? 4 : 16;
  while (n_ks > 4 && ng / n_ks < 4) n_ks /= 2;
  uint32_t gps = (ng + n_ks - 1) / n_ks;
  gps = (gps + 3) / 4 * 4;  // multiples of 4 groups per wave
  const size_t lds = std::max<size_t>(static_cast<size_t>(n_ks) * gps * (8 * a.T * 16 + a.T * 4),
                                      static_cast<size_t>(n_ks) * NPROJ * 8 * 32 * 4);
  if (lds > 156 * 1024 || (n_ks != 4 && n_ks != 16) || (NPROJ == 2 && n_ks != 4)) return false;
  RowsMfmaArgs b = a;
  b.gps = gps;
  const void* fn = n_ks == 4 ? reinterpret_cast<const void*>(rows_mfma_kernel<NPROJ, 4>)
                             : reinterpret_cast<const void*>(rows_mfma_kernel<1, 16>);
  if (lds > 48 * 1024) {
    err = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
    if (err != hipSuccess) return true;
  }
  if (n_ks == 4) rows_mfma_kernel<NPROJ, 4><<<dim3(blocks), dim3(256), lds, s>>>(b);
  else rows_mfma_kernel<1, 16><<<dim3(blocks), dim3(1024), lds, s>>>(b);
  err = hipGetLastError();
  return true;
}

// The quad kernel takes 4-bit matrices with at least 1024 rows (a multiple of 4) and up to 4
// token rows when the 32-element chunks of a row split over (waves, ITS slots of 16 chunks)
// with little waste.
template <int NPROJ>
bool rows_quad_try(hipStream_t s, const RowsQuadArgs& a, uint32_t num_cu, hipError_t& err) {
  if (a.N % (8 * kGroup) || a.T < 1 || a.T > 4 || a.M < 1024 || a.M % 4) return false;
  const uint32_t chunks = a.N / 32;
  uint32_t best_its = 0, best_wpr = 0, best_waste = ~0u;
  for (uint32_t its = 6; its >= 4; --its) {
    const uint32_t wpr = (chunks + 16 * its - 1) / (16 * its);
    if (wpr > kQuadMaxWaves) continue;
    const uint32_t waste = 16 * its * wpr - chunks;
    if (waste < best_waste) { best_waste = waste; best_its = its; best_wpr = wpr; }
  }
  if (!best_its || best_waste * 10 > chunks) return false;
  const uint32_t n_sets = a.M / 4;
  const uint32_t grid = std::min<uint32_t>(n_sets, num_cu * std::max(1u, 8u / best_wpr));
  const dim3 block(best_wpr * 64);
  if (best_its == 4) rows_quad_kernel<NPROJ, 4><<<dim3(grid), block, 0, s>>>(a);
  else if (best_its == 5) rows_quad_kernel<NPROJ, 5><<<dim3(grid), block, 0, s>>>(a);
  else rows_quad_kernel<NPROJ, 6><<<dim3(grid), block, 0, s>>>(a);
  err = hipGetLastError();
  return true;
}

}  // namespace

hipError_t launch_gemv(hipStream_t s, const mf_qtensor& w, int bits, const uint16_t* x, void* y,
                       uint32_t m, uint32_t n, uint32_t t, bool out_f32, bool lane_order) {
  if (bits == kBits8) {  // one wave per (token, row); any number of token rows
    const uint64_t waves = static_cast<uint64_t>(m) * t;
    if (!waves) return hipSuccess;
    if (waves >= (1ull << 30)) return hipErrorInvalidValue;
    const int al8 = (reinterpret_cast<uintptr_t>(w.weights) % 8 == 0) && n % 8 == 0 && aligned16(x);
    gemv_q8_kernel<<<dim3(static_cast<uint32_t>((waves + 3) / 4)), dim3(256), 0, s>>>(
        static_cast<const uint8_t*>(w.weights), w.scales, w.biases, x, y, m, n, t, out_f32 ? 1 : 0, al8);
    return hipGetLastError();
  }
  const bool al = aligned16(w.weights) && aligned16(x);
  if (!lane_order && al && bits == kBits4 && aligned16(w.scales) && aligned16(w.biases)) {
    RowsMfmaArgs ma{};
    ma.W[0] = static_cast<const uint8_t*>(w.weights); ma.S[0] = w.scales; ma.B[0] = w.biases;
    ma.x = x; ma.y = y; ma.M = m; ma.N = n; ma.T = t; ma.out_f32 = out_f32 ? 1 : 0;
    hipError_t err = hipSuccess;
    RowsQuadArgs qa{};
    qa.W[0] = ma.W[0]; qa.S[0] = ma.S[0]; qa.B[0] = ma.B[0];
    qa.x = x; qa.y = y; qa.M = m; qa.N = n; qa.T = t; qa.out_f32 = ma.out_f32;
    if (rows_quad_try<1>(s, qa, device_cu_count(), err)) return err;
    // Five to eight token rows of a matrix the quad kernel takes: two launches, rows 0..3 and the
    // rest.  The quad kernel runs the same instructions for a token whatever rides along, so every row
    // keeps the bits of a single-token call (MultiXKernelParityTests.swift:50-77); the weights stream
    // twice.  (y rows are m elements apart, 2 or 4 bytes each: 16-byte aligned since m % 4 == 0 and t > 4
    // only reaches here with m >= 1024.)
    if (t > 4 && t <= 8) {
      RowsQuadArgs q0 = qa, q1 = qa;
      q0.T = 4;
      q1.T = t - 4;
      q1.x = x + static_cast<size_t>(4) * n;
      q1.y = static_cast<uint8_t*>(y) + static_cast<size_t>(4) * m * (out_f32 ? 4 : 2);
      if (rows_quad_try<1>(s, q0, device_cu_count(), err)) {
        if (err != hipSuccess) return err;
        if (rows_quad_try<1>(s, q1, device_cu_count(), err)) return err;
        return hipErrorUnknown;  // (not reached: the second launch has the shape of the first)
      }
    }
    if (rows_mfma_try<1>(s, ma, device_cu_count(), err)) return err;
  }
  if (!lane_order && al && (bits == kBits4 || bits == kBits2)) {
    RowsArgs a{};
    a.W[0] = static_cast<const uint8_t*>(w.weights); a.S[0] = w.scales; a.B[0] = w.biases;
    a.x = x; a.y = y; a.M = m; a.N = n; a.out_f32 = out_f32 ? 1 : 0;
    hipError_t err = hipSuccess;
    if (bits == kBits4 ? rows_stream_try<kBits4, 1>(s, a, t, device_cu_count(), err)
                       : rows_stream_try<kBits2, 1>(s, a, t, device_cu_count(), err))
      return err;
  }
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
                              uint32_t t, bool lane_order) {
  const bool al = aligned16(gate.weights) && aligned16(up.weights) && aligned16(x);
  if (!lane_order && al && bits == kBits4 && aligned16(gate.scales) && aligned16(gate.biases) && aligned16(up.scales) &&
      aligned16(up.biases)) {
    RowsMfmaArgs ma{};
    ma.W[0] = static_cast<const uint8_t*>(gate.weights); ma.S[0] = gate.scales; ma.B[0] = gate.biases;
    ma.W[1] = static_cast<const uint8_t*>(up.weights); ma.S[1] = up.scales; ma.B[1] = up.biases;
    ma.x = x; ma.y = act; ma.M = f; ma.N = d; ma.T = t;
    hipError_t err = hipSuccess;
    RowsQuadArgs qa{};
    for (int p = 0; p < 2; ++p) { qa.W[p] = ma.W[p]; qa.S[p] = ma.S[p]; qa.B[p] = ma.B[p]; }
    qa.x = x; qa.y = act; qa.M = f; qa.N = d; qa.T = t;
    if (rows_quad_try<2>(s, qa, device_cu_count(), err)) return err;
    if (t > 4 && t <= 8) {  // as in launch_gemv: rows 0..3, then the rest, same bits as single-token calls
      RowsQuadArgs q0 = qa, q1 = qa;
      q0.T = 4;
      q1.T = t - 4;
      q1.x = x + static_cast<size_t>(4) * d;
      q1.y = act + static_cast<size_t>(4) * f;
      if (rows_quad_try<2>(s, q0, device_cu_count(), err)) {
        if (err != hipSuccess) return err;
        if (rows_quad_try<2>(s, q1, device_cu_count(), err)) return err;
        return hipErrorUnknown;
      }
    }
    if (rows_mfma_try<2>(s, ma, device_cu_count(), err)) return err;
  }
  if (!lane_order && al && (bits == kBits4 || bits == kBits2)) {
    RowsArgs a{};
    a.W[0] = static_cast<const uint8_t*>(gate.weights); a.S[0] = gate.scales; a.B[0] = gate.biases;
    a.W[1] = static_cast<const uint8_t*>(up.weights); a.S[1] = up.scales; a.B[1] = up.biases;
    a.x = x; a.y = act; a.M = f; a.N = d;
    hipError_t err = hipSuccess;
    if (bits == kBits4 ? rows_stream_try<kBits4, 2>(s, a, t, device_cu_count(), err)
                       : rows_stream_try<kBits2, 2>(s, a, t, device_cu_count(), err))
      return err;
  }
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

// The step in front of the MoE layer (RealForwardRunner.swift:2799-2808): hidden += delta
// (residual_add_fp16, utility.metal:83-92; skipped when delta is null), then
// out = narrow(hidden * rsqrt(mean(hidden^2) + eps) * weight) (rmsnorm_bf16w, rmsnorm.metal:68-92:
// fp32 sum of squares by fma, the sum is taken over the narrowed hidden).  One workgroup per row.
__global__ __launch_bounds__(256) void residual_rmsnorm_kernel(uint16_t* __restrict__ hidden,
                                                               const uint16_t* __restrict__ delta,
                                                               const uint16_t* __restrict__ weight,
                                                               uint16_t* __restrict__ out, uint32_t d,
                                                               float eps) {
  __shared__ float s_part[4];
  uint16_t* h = hidden + static_cast<size_t>(blockIdx.x) * d;
  const uint16_t* dl = delta ? delta + static_cast<size_t>(blockIdx.x) * d : nullptr;
  uint16_t* o = out + static_cast<size_t>(blockIdx.x) * d;
  float acc = 0.0f;
  for (uint32_t i = threadIdx.x; i < d; i += blockDim.x) {
    uint16_t hb = h[i];
    if (dl) {
      hb = f_to_bf16(bf16_to_f(hb) + bf16_to_f(dl[i]));
      h[i] = hb;
    }
    const float v = bf16_to_f(hb);
    acc = __builtin_fmaf(v, v, acc);
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = acc;
  __syncthreads();
  const float total = (s_part[0] + s_part[1]) + (s_part[2] + s_part[3]);
  const float inv = 1.0f / __builtin_sqrtf(total / static_cast<float>(d) + eps);
  for (uint32_t i = threadIdx.x; i < d; i += blockDim.x)
    o[i] = f_to_bf16(bf16_to_f(h[i]) * inv * bf16_to_f(weight[i]));
}

hipError_t launch_gate_up_act_q8(hipStream_t s, const mf_qtensor& gate, const mf_qtensor& up, const uint16_t* x,
                                 uint16_t* act, uint32_t f, uint32_t d, uint32_t t, bool silu) {
  const uint64_t waves = static_cast<uint64_t>(f) * t;
  if (!waves) return hipSuccess;
  if (waves >= (1ull << 30)) return hipErrorInvalidValue;
  const int al8 = (reinterpret_cast<uintptr_t>(gate.weights) % 8 == 0) && (reinterpret_cast<uintptr_t>(up.weights) % 8 == 0) &&
                  d % 8 == 0 && aligned16(x);
  const dim3 grid(static_cast<uint32_t>((waves + 3) / 4)), block(256);
  if (silu)
    gate_up_act_q8_kernel<true><<<grid, block, 0, s>>>(static_cast<const uint8_t*>(gate.weights), gate.scales, gate.biases,
                                                        static_cast<const uint8_t*>(up.weights), up.scales, up.biases, x,
                                                        act, f, d, t, al8);
  else
    gate_up_act_q8_kernel<false><<<grid, block, 0, s>>>(static_cast<const uint8_t*>(gate.weights), gate.scales, gate.biases,
                                                         static_cast<const uint8_t*>(up.weights), up.scales, up.biases, x,
                                                         act, f, d, t, al8);
  return hipGetLastError();
}

hipError_t launch_residual_rmsnorm(hipStream_t s, uint16_t* hidden, const uint16_t* delta,
                                   const uint16_t* weight, uint16_t* out, uint32_t d, uint32_t t, float eps) {
  if (!t) return hipSuccess;
  residual_rmsnorm_kernel<<<dim3(t), dim3(256), 0, s>>>(hidden, delta, weight, out, d, eps);
  return hipGetLastError();
}

hipError_t launch_residual_add(hipStream_t s, uint16_t* hidden, const uint16_t* delta,
                               uint32_t count) {
  if (!count) return hipSuccess;
  residual_add_kernel<<<dim3((count + 255) / 256), dim3(256), 0, s>>>(hidden, delta, count);
  return hipGetLastError();
}

}  // namespace mf
