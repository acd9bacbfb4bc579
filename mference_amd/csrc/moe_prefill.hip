// Ragged prefill: router for many tokens, device-side grouping of the
// (token, expert) routes, and the tokens-sorted-by-expert quantized matmul on
// the bf16 matrix cores.
//
// The matmul keeps the 4-bit codes EXACT: a lane's packed uint32 (8 codes of
// one weight row) is masked straight into four bf16 pairs 128+q
// (0x4300 | q), which is an MFMA A operand as it stands -- no LDS staging of
// weights.  x is staged through LDS once per 64-wide K group, permuted to the
// same (j, j+4) pairing.  Per K group the matrix core yields
// sum((128+q)*x) exactly (bf16 x bf16 products are exact in fp32), and the
// group's bf16 scale is applied in fp32: acc += s * tmp -- the reference's own
// factoring s*sum(q*x) + b*sum(x) (Metal/Quant/dequant_int4.metal:14-17), so
// no weight is ever rounded to bf16 (rounding q*s+b to bf16 would cost ~1.6e-3
// relative error per weight, above the layer tolerance).  The b*sum(x) and
// -128*s*sum(x) terms are two more small matmuls over the group index
// (A = the bf16 bias / scale tables, exact; B = sum(x) split into three bf16
// terms, exact), run on the matrix core after the K loop.
//
// Replaces prefill_grouped_routed_moe_batched_{phase1,down}
// (Metal/Prefill/prefill.metal:748-820), prefill_moe_reduce_token_major
// (:631-652) and the staged-affine tensor-core QMM
// mpp_prefill_affine_threadgroup_f16 (Metal/TensorCore/tensorops.metal:13-105).
#include "mf_device.h"
#include "mf_internal.h"
#include "mf_router.h"

#pragma clang fp contract(off)

namespace mf {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

constexpr uint32_t kTileTokens = 64;   // tokens of one expert a workgroup handles
constexpr uint32_t kQmmWaves = 4;      // waves per workgroup, 32 weight rows each
constexpr uint32_t kQmmRows = kQmmWaves * 32;

struct Tile {
  uint32_t expert, pair_start, count, pad;
};

// ------------------------------------------------------------------ router

// logits[t, e] for many tokens, bit-exact with dot_bf16_row: a wave keeps R
// expert rows in registers (lane l holds the chunks l, l+64, ... of each row)
// and streams token rows past them.
template <int CPL, int R>
__global__ __launch_bounds__(256) void prefill_router_kernel(const uint16_t* __restrict__ W,
                                                             const uint16_t* __restrict__ x,
                                                             uint32_t E, uint32_t D, uint32_t T,
                                                             uint32_t x_stride,
                                                             float* __restrict__ logits,
                                                             uint32_t tokens_per_block) {
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const uint32_t row0 = (blockIdx.x * 4 + wv) * R;
  if (row0 >= E) return;
  const uint32_t chunks = D / 8;
  float wf[R][CPL][8];
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const uint32_t ci = lane + 64 * c;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (ci < chunks && row0 + r < E) v = load_x8<true>(W + static_cast<size_t>(row0 + r) * D + ci * 8);
      wf[r][c][0] = bf16_lo(v.x); wf[r][c][1] = bf16_hi(v.x);
      wf[r][c][2] = bf16_lo(v.y); wf[r][c][3] = bf16_hi(v.y);
      wf[r][c][4] = bf16_lo(v.z); wf[r][c][5] = bf16_hi(v.z);
      wf[r][c][6] = bf16_lo(v.w); wf[r][c][7] = bf16_hi(v.w);
    }
  }
  const uint32_t t0 = blockIdx.y * tokens_per_block;
  const uint32_t t1 = min(T, t0 + tokens_per_block);
  for (uint32_t t = t0; t < t1; ++t) {
    const uint16_t* xt = x + static_cast<size_t>(t) * x_stride;
    float xf[CPL][8];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const uint32_t ci = lane + 64 * c;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (ci < chunks) v = load_x8<true>(xt + ci * 8);
      xf[c][0] = bf16_lo(v.x); xf[c][1] = bf16_hi(v.x);
      xf[c][2] = bf16_lo(v.y); xf[c][3] = bf16_hi(v.y);
      xf[c][4] = bf16_lo(v.z); xf[c][5] = bf16_hi(v.z);
      xf[c][6] = bf16_lo(v.w); xf[c][7] = bf16_hi(v.w);
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float acc = 0.0f;
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        if (lane + 64 * c < chunks) {
#pragma unroll
          for (int j = 0; j < 8; ++j) acc = __builtin_fmaf(wf[r][c][j], xf[c][j], acc);
        }
      }
      const float v = wave_sum(acc);
      if (lane == 0 && row0 + r < E) logits[static_cast<size_t>(t) * E + row0 + r] = v;
    }
  }
}

// ---------------------------------------------------------------- grouping
//
// PrefillMoEGrouping.groupTokenExpertPairs (PrefillMoEGrouping.swift:91-192) on
// device: pairs come token-major (token, rank), so "sorted by (expert, token,
// rank)" is a stable partition by expert.  One wave per expert counts its
// routes, a single block scans the counts, one wave per expert emits its
// routes in order.

__global__ __launch_bounds__(256) void group_count_kernel(const uint32_t* __restrict__ idx,
                                                          uint32_t n_pairs, uint32_t E,
                                                          uint32_t* __restrict__ counts,
                                                          uint32_t* __restrict__ status) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t e = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (e >= E) return;
  uint32_t cnt = 0;
  bool bad = false;
  for (uint32_t p0 = 0; p0 < n_pairs; p0 += kWave) {
    const uint32_t p = p0 + lane;
    const uint32_t v = p < n_pairs ? idx[p] : 0xFFFFFFFFu;
    cnt += __popcll(__ballot(v == e));
    if (e == 0 && p < n_pairs && v >= E) bad = true;
  }
  if (lane == 0) counts[e] = cnt;
  if (__any(bad) && lane == 0) atomicOr(status, 2u);
}

// offsets (0xFFFFFFFF for an empty expert), running starts, and the tile list
// of the matmul (every expert's routes cut into runs of kTileTokens).
__global__ __launch_bounds__(512) void group_scan_kernel(const uint32_t* __restrict__ counts,
                                                         uint32_t E, uint32_t* __restrict__ offsets,
                                                         uint32_t* __restrict__ starts,
                                                         Tile* __restrict__ tiles,
                                                         uint32_t* __restrict__ n_tiles) {
  __shared__ uint32_t s_cnt[MF_MAX_EXPERTS], s_tile[MF_MAX_EXPERTS];
  const uint32_t e = threadIdx.x;
  const uint32_t c = e < E ? counts[e] : 0;
  s_cnt[e] = c;
  s_tile[e] = (c + kTileTokens - 1) / kTileTokens;
  __syncthreads();
  for (uint32_t o = 1; o < MF_MAX_EXPERTS; o <<= 1) {  // inclusive scans
    const uint32_t a = e >= o ? s_cnt[e - o] : 0, b = e >= o ? s_tile[e - o] : 0;
    __syncthreads();
    s_cnt[e] += a;
    s_tile[e] += b;
    __syncthreads();
  }
  if (e < E) {
    const uint32_t start = s_cnt[e] - c;
    starts[e] = start;
    offsets[e] = c ? start : 0xFFFFFFFFu;
    if (tiles) {
      const uint32_t nt = (c + kTileTokens - 1) / kTileTokens, t0 = s_tile[e] - nt;
      for (uint32_t j = 0; j < nt; ++j)
        tiles[t0 + j] = Tile{e, start + j * kTileTokens, min(kTileTokens, c - j * kTileTokens), 0};
    }
  }
  if (n_tiles && e == MF_MAX_EXPERTS - 1) *n_tiles = s_tile[e];
}

__global__ __launch_bounds__(256) void group_emit_kernel(const uint32_t* __restrict__ idx,
                                                         const float* __restrict__ w,
                                                         uint32_t n_pairs, uint32_t K, uint32_t E,
                                                         const uint32_t* __restrict__ starts,
                                                         mf_pair* __restrict__ sorted) {
  const uint32_t lane = threadIdx.x & 63;
  const uint32_t e = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (e >= E) return;
  uint32_t running = starts[e];
  for (uint32_t p0 = 0; p0 < n_pairs; p0 += kWave) {
    const uint32_t p = p0 + lane;
    const bool m = p < n_pairs && idx[p] == e;
    const unsigned long long mask = __ballot(m);
    if (m) {
      const uint32_t pos = running + __popcll(mask & ((1ull << lane) - 1ull));
      mf_pair r;
      r.token = p / K;
      r.expert = e;
      r.rank = p % K;
      r.weight_bits = __float_as_uint(w[p]);
      sorted[pos] = r;
    }
    running += __popcll(mask);
  }
}

__global__ void zero_words_kernel(uint32_t* p, uint32_t n) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// --------------------------------------------------------------- the matmul

struct QmmArgs {
  // weights: routed = blobs of the expert pool, dense = one projection set
  const uint8_t* expert_base;
  size_t expert_stride;
  uint32_t w_off[2], s_off[2], b_off[2];
  mf_qtensor dense[2];
  int dense_mode;       // 1: the "expert" is dense[], tiles are runs of consecutive rows
  uint32_t dense_rows;  // number of x rows in dense mode
  // activations: rows of kdim bf16
  const uint16_t* x;
  uint32_t x_stride;
  int gather;           // 1: x row = sorted[pair].token, 0: x row = pair index
  const mf_pair* sorted;
  const Tile* tiles;
  const uint32_t* n_tiles;
  uint32_t rows, kdim;  // weight rows (output width) and contraction length
  // epilogue
  int epi;              // 0 swiglu -> bf16 [pair, rows]; 1 fp32 [token*K+rank, rows]; 2 bf16 [pair, rows]
  int narrow;           // shared-expert rounding points (dequant_int4.metal:240-245)
  void* out;
  uint32_t top_k;
  float limit;
};

__device__ __forceinline__ f32x16_t mfma_bf16(const uint4& a, const uint4& b, const f32x16_t& c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// one packed word of 4-bit codes -> MFMA operand: pairs (q0,q4),(q1,q5),(q2,q6),(q3,q7) as 128+q
__device__ __forceinline__ uint4 expand_q4(uint32_t w) {
  return make_uint4((w & 0x000F000Fu) | kMagic128, ((w >> 4) & 0x000F000Fu) | kMagic128,
                    ((w >> 8) & 0x000F000Fu) | kMagic128, ((w >> 12) & 0x000F000Fu) | kMagic128);
}

// 8 bf16 from p, of which only the first `avail` exist (the rest read as 0)
__device__ __forceinline__ uint4 load_bf16x8_guarded(const uint16_t* p, uint32_t avail) {
  if (avail >= 8) return load_x8<false>(p);
  uint32_t v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = static_cast<uint32_t>(i) < avail ? p[i] : 0u;
  return make_uint4(v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16));
}

// three exact bf16 terms of 8 fp32 values as MFMA operands: term k of +x and of -128*x
__device__ __forceinline__ void split_terms(const float (&sx)[8], int k, uint4& pos, uint4& neg) {
  float t[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float t0 = __uint_as_float(__float_as_uint(sx[e]) & 0xFFFF0000u);
    const float r1 = sx[e] - t0;
    const float t1 = __uint_as_float(__float_as_uint(r1) & 0xFFFF0000u);
    const float t2 = r1 - t1;
    t[e] = k == 0 ? t0 : (k == 1 ? t1 : t2);
  }
  pos = make_uint4((__float_as_uint(t[0]) >> 16) | (__float_as_uint(t[1]) & 0xFFFF0000u),
                   (__float_as_uint(t[2]) >> 16) | (__float_as_uint(t[3]) & 0xFFFF0000u),
                   (__float_as_uint(t[4]) >> 16) | (__float_as_uint(t[5]) & 0xFFFF0000u),
                   (__float_as_uint(t[6]) >> 16) | (__float_as_uint(t[7]) & 0xFFFF0000u));
#pragma unroll
  for (int e = 0; e < 8; ++e) t[e] = -128.0f * t[e];
  neg = make_uint4((__float_as_uint(t[0]) >> 16) | (__float_as_uint(t[1]) & 0xFFFF0000u),
                   (__float_as_uint(t[2]) >> 16) | (__float_as_uint(t[3]) & 0xFFFF0000u),
                   (__float_as_uint(t[4]) >> 16) | (__float_as_uint(t[5]) & 0xFFFF0000u),
                   (__float_as_uint(t[6]) >> 16) | (__float_as_uint(t[7]) & 0xFFFF0000u));
}

__device__ __forceinline__ uint32_t pack_bf16_trunc(float lo, float hi) {
  return (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xFFFF0000u);
}

// LDS layout (dynamic): x tile double buffer 2 x [2 nt][4 s][2 h][32 n] x 16 B,
// sumx [ng][64] fp32, scale tables [NPROJ][4 waves][ng][32 rows] bf16, rows[64] u32.
template <int NPROJ>
__global__ __launch_bounds__(256) void qmm_kernel(const QmmArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const uint32_t n_slices = a.rows / kQmmRows;
  const uint32_t tile_id = blockIdx.x / n_slices, slice = blockIdx.x % n_slices;
  const uint32_t ng = a.kdim / kGroup;

  uint32_t expert = 0, pair_start, count;
  if (a.dense_mode) {
    pair_start = tile_id * kTileTokens;
    if (pair_start >= a.dense_rows) return;
    count = min(kTileTokens, a.dense_rows - pair_start);
  } else {
    if (tile_id >= *a.n_tiles) return;
    const Tile t = a.tiles[tile_id];
    expert = t.expert;
    pair_start = t.pair_start;
    count = t.count;
  }

  uint4* s_x = reinterpret_cast<uint4*>(smem);                                   // 2 * 512 uint4
  float* s_sumx = reinterpret_cast<float*>(smem + 2 * 512 * 16);                 // [ng][64]
  uint16_t* s_scale = reinterpret_cast<uint16_t*>(smem + 2 * 512 * 16 + ng * 64 * 4);
  uint32_t* s_rows = reinterpret_cast<uint32_t*>(smem + 2 * 512 * 16 + ng * 64 * 4 +
                                                 NPROJ * kQmmWaves * ng * 32 * 2);

  // weight pointers of this workgroup's projections
  const uint8_t* Wp[NPROJ];
  const uint16_t* Sp[NPROJ];
  const uint16_t* Bp[NPROJ];
#pragma unroll
  for (int p = 0; p < NPROJ; ++p) {
    if (a.dense_mode) {
      Wp[p] = static_cast<const uint8_t*>(a.dense[p].weights);
      Sp[p] = a.dense[p].scales;
      Bp[p] = a.dense[p].biases;
    } else {
      const uint8_t* blob = a.expert_base + static_cast<size_t>(expert) * a.expert_stride;
      Wp[p] = blob + a.w_off[p];
      Sp[p] = reinterpret_cast<const uint16_t*>(blob + a.s_off[p]);
      Bp[p] = reinterpret_cast<const uint16_t*>(blob + a.b_off[p]);
    }
  }
  const uint32_t row_base = slice * kQmmRows + wv * 32;  // first of this wave's 32 weight rows
  const uint32_t m = lane & 31, h = lane >> 5;
  const size_t row_bytes = static_cast<size_t>(a.kdim) / 2;

  // x rows of the tile
  if (threadIdx.x < kTileTokens) {
    uint32_t r = 0xFFFFFFFFu;
    if (threadIdx.x < count)
      r = a.gather ? a.sorted[pair_start + threadIdx.x].token : pair_start + threadIdx.x;
    s_rows[threadIdx.x] = r;
  }
  // scale tables of the wave's rows, transposed to [g][row]
  {
    uint16_t* dst = s_scale;
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      uint16_t* tab = dst + (p * kQmmWaves + wv) * ng * 32;
      const uint16_t* src = Sp[p] + static_cast<size_t>(row_base + m) * ng;
      for (uint32_t g0 = h * 8; g0 < ng; g0 += 16) {  // lane: row m, 8 groups from g0
        const uint4 v = load_bf16x8_guarded(src + g0, ng - g0);
        const uint32_t pr[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (g0 + 2 * i < ng) tab[(g0 + 2 * i) * 32 + m] = static_cast<uint16_t>(pr[i] & 0xFFFFu);
          if (g0 + 2 * i + 1 < ng) tab[(g0 + 2 * i + 1) * 32 + m] = static_cast<uint16_t>(pr[i] >> 16);
        }
      }
    }
  }
  __syncthreads();

  f32x16_t acc[NPROJ][2];
#pragma unroll
  for (int p = 0; p < NPROJ; ++p)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[p][nt][r] = 0.0f;

  // staging role of this thread: token i, 16 K values from 16 * q
  const uint32_t st_i = threadIdx.x >> 2, st_q = threadIdx.x & 3;
  const uint32_t st_row = s_rows[st_i];
  const uint16_t* st_src = a.x + static_cast<size_t>(st_row == 0xFFFFFFFFu ? 0 : st_row) * a.x_stride + st_q * 16;

  uint4 codes[NPROJ];
#pragma unroll
  for (int p = 0; p < NPROJ; ++p)
    codes[p] = *reinterpret_cast<const uint4*>(Wp[p] + (row_base + m) * row_bytes + h * 16);

  for (uint32_t g = 0; g < ng; ++g) {
    // ---- stage x tile of group g (buffer g & 1) and its row sums
    {
      uint4 v0 = make_uint4(0, 0, 0, 0), v1 = v0;
      if (st_row != 0xFFFFFFFFu) {
        v0 = *reinterpret_cast<const uint4*>(st_src + g * kGroup);
        v1 = *reinterpret_cast<const uint4*>(st_src + g * kGroup + 8);
      }
      float sum = 0.0f;
      sum = dot2_bf16(v0.x, kOnes, sum); sum = dot2_bf16(v0.y, kOnes, sum);
      sum = dot2_bf16(v0.z, kOnes, sum); sum = dot2_bf16(v0.w, kOnes, sum);
      sum = dot2_bf16(v1.x, kOnes, sum); sum = dot2_bf16(v1.y, kOnes, sum);
      sum = dot2_bf16(v1.z, kOnes, sum); sum = dot2_bf16(v1.w, kOnes, sum);
      sum = sum + dpp_f<0xB1>(sum);
      sum = sum + dpp_f<0x4E>(sum);
      if (st_q == 0) s_sumx[g * 64 + st_i] = sum;
      uint4* buf = s_x + (g & 1) * 512;
      const uint32_t nt = st_i >> 5, n = st_i & 31;
      // chunk c = 2q (+1): K 8c..8c+7 -> (h = c / 4, s = c % 4)
      const uint32_t c0 = 2 * st_q, c1 = c0 + 1;
      buf[((nt * 4 + (c0 & 3)) * 2 + (c0 >> 2)) * 32 + n] =
          make_uint4(__builtin_amdgcn_perm(v0.z, v0.x, 0x05040100u), __builtin_amdgcn_perm(v0.z, v0.x, 0x07060302u),
                     __builtin_amdgcn_perm(v0.w, v0.y, 0x05040100u), __builtin_amdgcn_perm(v0.w, v0.y, 0x07060302u));
      buf[((nt * 4 + (c1 & 3)) * 2 + (c1 >> 2)) * 32 + n] =
          make_uint4(__builtin_amdgcn_perm(v1.z, v1.x, 0x05040100u), __builtin_amdgcn_perm(v1.z, v1.x, 0x07060302u),
                     __builtin_amdgcn_perm(v1.w, v1.y, 0x05040100u), __builtin_amdgcn_perm(v1.w, v1.y, 0x07060302u));
    }
    // next group's codes
    uint4 next[NPROJ];
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      next[p] = codes[p];
      if (g + 1 < ng)
        next[p] = *reinterpret_cast<const uint4*>(Wp[p] + (row_base + m) * row_bytes + (g + 1) * 32 + h * 16);
    }
    __syncthreads();

    // ---- matrix core: tmp = sum over the group of (128+q) * x
    const uint4* buf = s_x + (g & 1) * 512;
    uint4 bx[2][4];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int s = 0; s < 4; ++s) bx[nt][s] = buf[((nt * 4 + s) * 2 + h) * 32 + m];
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      const uint32_t cw[4] = {codes[p].x, codes[p].y, codes[p].z, codes[p].w};
      f32x16_t tmp[2];
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int r = 0; r < 16; ++r) tmp[nt][r] = 0.0f;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const uint4 av = expand_q4(cw[s]);
        tmp[0] = mfma_bf16(av, bx[0][s], tmp[0]);
        tmp[1] = mfma_bf16(av, bx[1][s], tmp[1]);
      }
      // per-group scale of the 16 rows this lane holds: row = 8j + 4h + i
      const uint16_t* tab = s_scale + ((p * kQmmWaves + wv) * ng + g) * 32 + 4 * h;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint2 sv = *reinterpret_cast<const uint2*>(tab + 8 * j);
        const float s0 = bf16_lo(sv.x), s1 = bf16_hi(sv.x), s2 = bf16_lo(sv.y), s3 = bf16_hi(sv.y);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          acc[p][nt][4 * j + 0] = __builtin_fmaf(s0, tmp[nt][4 * j + 0], acc[p][nt][4 * j + 0]);
          acc[p][nt][4 * j + 1] = __builtin_fmaf(s1, tmp[nt][4 * j + 1], acc[p][nt][4 * j + 1]);
          acc[p][nt][4 * j + 2] = __builtin_fmaf(s2, tmp[nt][4 * j + 2], acc[p][nt][4 * j + 2]);
          acc[p][nt][4 * j + 3] = __builtin_fmaf(s3, tmp[nt][4 * j + 3], acc[p][nt][4 * j + 3]);
        }
      }
      codes[p] = next[p];
    }
  }
  __syncthreads();

  // ---- bias and offset terms: acc += B[row, g] * sumx[g, n] - 128 * S[row, g] * sumx[g, n]
  for (uint32_t g0 = 0; g0 < ng; g0 += 16) {
    const uint32_t gl = g0 + 8 * h;  // this lane's 8 groups
    uint4 ab[NPROJ], as[NPROJ];
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      ab[p] = as[p] = make_uint4(0, 0, 0, 0);
      if (gl < ng) {
        ab[p] = load_bf16x8_guarded(Bp[p] + static_cast<size_t>(row_base + m) * ng + gl, ng - gl);
        as[p] = load_bf16x8_guarded(Sp[p] + static_cast<size_t>(row_base + m) * ng + gl, ng - gl);
      }
    }
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      float sx[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) sx[e] = gl + e < ng ? s_sumx[(gl + e) * 64 + nt * 32 + m] : 0.0f;
#pragma unroll
      for (int k = 0; k < 3; ++k) {
        uint4 bpos, bneg;
        split_terms(sx, k, bpos, bneg);
#pragma unroll
        for (int p = 0; p < NPROJ; ++p) {
          acc[p][nt] = mfma_bf16(ab[p], bpos, acc[p][nt]);
          acc[p][nt] = mfma_bf16(as[p], bneg, acc[p][nt]);
        }
      }
    }
  }

  // ---- epilogue: lane holds token n = m of each token tile, rows 8j + 4h + i
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const uint32_t ti = nt * 32 + m;
    if (ti >= count) continue;
    const uint32_t pair = pair_start + ti;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t row = row_base + 8 * j + 4 * h;
      if (a.epi == 0) {
        uint16_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float gv = acc[0][nt][4 * j + i], uv = acc[NPROJ - 1][nt][4 * j + i];
          if (a.narrow) {
            gv = round_bf16(gv);
            uv = round_bf16(uv);
          }
          if (a.limit > 0.0f) {
            gv = fminf(gv, a.limit);
            uv = fminf(fmaxf(uv, -a.limit), a.limit);
          }
          o[i] = f_to_bf16(mf_silu(gv) * uv);
        }
        uint2 pk;
        pk.x = static_cast<uint32_t>(o[0]) | (static_cast<uint32_t>(o[1]) << 16);
        pk.y = static_cast<uint32_t>(o[2]) | (static_cast<uint32_t>(o[3]) << 16);
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(a.out) + static_cast<size_t>(pair) * a.rows + row) = pk;
      } else if (a.epi == 1) {
        const mf_pair pr = a.sorted[pair];
        const size_t slot = static_cast<size_t>(pr.token) * a.top_k + pr.rank;
        *reinterpret_cast<float4*>(static_cast<float*>(a.out) + slot * a.rows + row) =
            make_float4(acc[0][nt][4 * j], acc[0][nt][4 * j + 1], acc[0][nt][4 * j + 2], acc[0][nt][4 * j + 3]);
      } else {
        uint2 pk;
        pk.x = static_cast<uint32_t>(f_to_bf16(acc[0][nt][4 * j])) |
               (static_cast<uint32_t>(f_to_bf16(acc[0][nt][4 * j + 1])) << 16);
        pk.y = static_cast<uint32_t>(f_to_bf16(acc[0][nt][4 * j + 2])) |
               (static_cast<uint32_t>(f_to_bf16(acc[0][nt][4 * j + 3])) << 16);
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(a.out) + static_cast<size_t>(pair) * a.rows + row) = pk;
      }
    }
  }
}

// y[t,d] = bf16(h1[t,d] + sum_r w[t,r] * partial[t*K+r, d]), residual first, rank
// order, product then add (moe.metal:1262-1270; reduce of prefill.metal:631-652).
// h1 = bf16(hs / (1 + exp(-gate_t))) when a scalar gate is given (utility.metal:49-59).
__global__ __launch_bounds__(256) void prefill_reduce_kernel(const float* __restrict__ partials,
                                                             const float* __restrict__ w,
                                                             const uint32_t* __restrict__ idx,
                                                             const uint16_t* __restrict__ hs,
                                                             const uint16_t* __restrict__ gate,
                                                             uint16_t* __restrict__ y, uint32_t T,
                                                             uint32_t K, uint32_t D, uint32_t E) {
  const size_t i4 = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
  if (i4 >= static_cast<size_t>(T) * D) return;
  const uint32_t t = static_cast<uint32_t>(i4 / D), d = static_cast<uint32_t>(i4 % D);
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (hs) {
    const uint2 hv = *reinterpret_cast<const uint2*>(hs + i4);
    acc[0] = bf16_lo(hv.x); acc[1] = bf16_hi(hv.x); acc[2] = bf16_lo(hv.y); acc[3] = bf16_hi(hv.y);
    if (gate) {
      const float den = 1.0f + mf_exp(-bf16_to_f(gate[t]));
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = round_bf16(acc[i] / den);
    }
  }
  for (uint32_t r = 0; r < K; ++r) {
    if (idx[t * K + r] >= E) continue;
    const float wt = w[t * K + r];
    const float4 v = *reinterpret_cast<const float4*>(partials + (static_cast<size_t>(t) * K + r) * D + d);
    const float p0 = wt * v.x, p1 = wt * v.y, p2 = wt * v.z, p3 = wt * v.w;
    acc[0] = acc[0] + p0; acc[1] = acc[1] + p1; acc[2] = acc[2] + p2; acc[3] = acc[3] + p3;
  }
  uint2 o;
  o.x = static_cast<uint32_t>(f_to_bf16(acc[0])) | (static_cast<uint32_t>(f_to_bf16(acc[1])) << 16);
  o.y = static_cast<uint32_t>(f_to_bf16(acc[2])) | (static_cast<uint32_t>(f_to_bf16(acc[3])) << 16);
  *reinterpret_cast<uint2*>(y + i4) = o;
}

// ------------------------------------------------------------------ launchers

hipError_t launch_prefill_router(hipStream_t s, const uint16_t* W, const uint16_t* x, uint32_t E,
                                 uint32_t D, uint32_t T, uint32_t x_stride, float* logits) {
  const uint32_t cpl = (D / 8 + 63) / 64;
  const uint32_t tpb = 64;
#define MF_PR(CPL, R)                                                                              \
  prefill_router_kernel<CPL, R><<<dim3((E + 4 * R - 1) / (4 * R), (T + tpb - 1) / tpb), dim3(256), 0, s>>>( \
      W, x, E, D, T, x_stride, logits, tpb)
  if (cpl <= 1) MF_PR(1, 4);
  else if (cpl <= 2) MF_PR(2, 4);
  else if (cpl <= 4) MF_PR(4, 4);
  else if (cpl <= 8) MF_PR(8, 2);
  else return hipErrorInvalidValue;
#undef MF_PR
  return hipGetLastError();
}

hipError_t launch_group(hipStream_t s, const uint32_t* idx, const float* w, uint32_t t, uint32_t K,
                        uint32_t E, uint32_t* counts, uint32_t* offsets, uint32_t* starts,
                        mf_pair* sorted, void* tiles, uint32_t* n_tiles, uint32_t* status) {
  const uint32_t n_pairs = t * K;
  zero_words_kernel<<<dim3(1), dim3(64), 0, s>>>(status, 1);  // a fill kernel: safe under graph capture
  group_count_kernel<<<dim3((E + 3) / 4), dim3(256), 0, s>>>(idx, n_pairs, E, counts, status);
  group_scan_kernel<<<dim3(1), dim3(MF_MAX_EXPERTS), 0, s>>>(counts, E, offsets, starts,
                                                             static_cast<Tile*>(tiles), n_tiles);
  group_emit_kernel<<<dim3((E + 3) / 4), dim3(256), 0, s>>>(idx, w, n_pairs, K, E, starts, sorted);
  return hipGetLastError();
}

size_t qmm_lds_bytes(uint32_t kdim, int nproj) {
  const uint32_t ng = kdim / kGroup;
  return 2 * 512 * 16 + static_cast<size_t>(ng) * 64 * 4 + static_cast<size_t>(nproj) * kQmmWaves * ng * 32 * 2 +
         kTileTokens * 4;
}

hipError_t launch_qmm(hipStream_t s, const QmmArgs& a, int nproj, uint32_t max_tiles) {
  const size_t lds = qmm_lds_bytes(a.kdim, nproj);
  const dim3 grid(max_tiles * (a.rows / kQmmRows)), block(256);
  if (grid.x == 0) return hipSuccess;
  if (nproj == 2) {
    if (lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(qmm_kernel<2>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
      if (e != hipSuccess) return e;
    }
    qmm_kernel<2><<<grid, block, lds, s>>>(a);
  } else {
    if (lds > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(qmm_kernel<1>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
      if (e != hipSuccess) return e;
    }
    qmm_kernel<1><<<grid, block, lds, s>>>(a);
  }
  return hipGetLastError();
}

namespace {
size_t up256(size_t v) { return (v + 255) / 256 * 256; }
}  // namespace

// workspace carve-up of one prefill layer call
struct PrefillWs {
  float* logits; uint32_t* idx; float* w; uint32_t* counts; uint32_t* offsets; uint32_t* starts;
  uint32_t* n_tiles; uint32_t* status; Tile* tiles; mf_pair* sorted; uint16_t* acts; float* partials;
  uint16_t* sact; uint16_t* hs; uint16_t* gate;
  size_t bytes;
};

PrefillWs prefill_carve(const mf_moe_config& c, uint32_t t, void* base) {
  PrefillWs p{};
  size_t pos = 0;
  auto take = [&](size_t bytes) {
    uint8_t* at = static_cast<uint8_t*>(base) + pos;
    pos += up256(bytes);
    return static_cast<void*>(base ? at : nullptr);
  };
  const size_t pairs = static_cast<size_t>(t) * c.top_k;
  const size_t max_tiles = std::min<size_t>(c.num_experts, pairs) + pairs / kTileTokens + 1;
  p.logits = static_cast<float*>(take(sizeof(float) * t * c.num_experts));
  p.idx = static_cast<uint32_t*>(take(sizeof(uint32_t) * pairs));
  p.w = static_cast<float*>(take(sizeof(float) * pairs));
  p.counts = static_cast<uint32_t*>(take(sizeof(uint32_t) * MF_MAX_EXPERTS));
  p.offsets = static_cast<uint32_t*>(take(sizeof(uint32_t) * MF_MAX_EXPERTS));
  p.starts = static_cast<uint32_t*>(take(sizeof(uint32_t) * MF_MAX_EXPERTS));
  p.n_tiles = static_cast<uint32_t*>(take(256));
  p.status = p.n_tiles ? p.n_tiles + 1 : nullptr;
  p.tiles = static_cast<Tile*>(take(sizeof(Tile) * max_tiles));
  p.sorted = static_cast<mf_pair*>(take(sizeof(mf_pair) * pairs));
  p.acts = static_cast<uint16_t*>(take(sizeof(uint16_t) * pairs * c.f));
  p.partials = static_cast<float*>(take(sizeof(float) * pairs * c.d));
  p.sact = static_cast<uint16_t*>(take(sizeof(uint16_t) * static_cast<size_t>(t) * std::max<uint32_t>(c.shared_f, 64)));
  p.hs = static_cast<uint16_t*>(take(sizeof(uint16_t) * static_cast<size_t>(t) * c.d));
  p.gate = static_cast<uint16_t*>(take(sizeof(uint16_t) * t));
  p.bytes = pos;
  return p;
}

size_t prefill_workspace_bytes(const mf_moe_config& c, uint32_t t) {
  return prefill_carve(c, t, nullptr).bytes;
}

bool prefill_supported(const mf_moe_config& c) {
  if (c.bits != MF_BITS_4 || (c.shared_f && c.shared_bits != MF_BITS_4)) return false;
  if (c.d % kQmmRows || c.f % kQmmRows || (c.shared_f % kQmmRows)) return false;
  if (c.d > 8192 || c.f > 8192 || c.shared_f > 8192) return false;
  return true;
}

hipError_t launch_prefill_layer(hipStream_t s, const mf_moe& h, const mf_moe_layer_weights& w,
                                const uint16_t* x, uint32_t t, uint16_t* y, void* workspace,
                                uint32_t* out_idx, float* out_w) {
  const mf_moe_config& c = h.cfg;
  const PrefillWs ws = prefill_carve(c, t, workspace);
  hipError_t e;
#define MF_TRY(call) do { e = (call); if (e != hipSuccess) return e; } while (0)
  MF_TRY(launch_prefill_router(s, w.router_w, x, c.num_experts, c.d, t, c.d, ws.logits));
  MF_TRY(launch_topk(s, ws.logits, c.num_experts, c.top_k, t, c.router_mode, ws.idx, ws.w));
  MF_TRY(launch_group(s, ws.idx, ws.w, t, c.top_k, c.num_experts, ws.counts, ws.offsets, ws.starts,
                      ws.sorted, ws.tiles, ws.n_tiles, ws.status));
  const size_t pairs = static_cast<size_t>(t) * c.top_k;
  const uint32_t max_tiles =
      static_cast<uint32_t>(std::min<size_t>(c.num_experts, pairs) + pairs / kTileTokens + 1);

  QmmArgs q{};
  q.expert_base = static_cast<const uint8_t*>(w.expert_base);
  q.expert_stride = w.expert_stride;
  q.sorted = ws.sorted;
  q.tiles = ws.tiles;
  q.n_tiles = ws.n_tiles;
  q.top_k = c.top_k;
  q.limit = c.swiglu_limit;
  // routed phase 1: gate/up -> acts [pair, F]
  q.w_off[0] = w.offsets.gate_w; q.s_off[0] = w.offsets.gate_s; q.b_off[0] = w.offsets.gate_b;
  q.w_off[1] = w.offsets.up_w; q.s_off[1] = w.offsets.up_s; q.b_off[1] = w.offsets.up_b;
  q.x = x; q.x_stride = c.d; q.gather = 1; q.rows = c.f; q.kdim = c.d; q.epi = 0; q.out = ws.acts;
  MF_TRY(launch_qmm(s, q, 2, max_tiles));
  // routed phase 2: down -> fp32 partials [token*K+rank, D]
  q.w_off[0] = w.offsets.down_w; q.s_off[0] = w.offsets.down_s; q.b_off[0] = w.offsets.down_b;
  q.x = ws.acts; q.x_stride = c.f; q.gather = 0; q.rows = c.d; q.kdim = c.f; q.epi = 1; q.out = ws.partials;
  q.limit = 0.0f;
  MF_TRY(launch_qmm(s, q, 1, max_tiles));
  const uint16_t* hs = nullptr;
  const uint16_t* gate = nullptr;
  if (c.shared_f) {
    QmmArgs d{};
    d.dense_mode = 1; d.dense_rows = t; d.top_k = c.top_k; d.narrow = 1;
    d.dense[0] = w.shared_gate; d.dense[1] = w.shared_up;
    d.x = x; d.x_stride = c.d; d.rows = c.shared_f; d.kdim = c.d; d.epi = 0; d.out = ws.sact;
    const uint32_t dense_tiles = (t + kTileTokens - 1) / kTileTokens;
    MF_TRY(launch_qmm(s, d, 2, dense_tiles));
    d.dense[0] = w.shared_down;
    d.x = ws.sact; d.x_stride = c.shared_f; d.rows = c.d; d.kdim = c.shared_f; d.epi = 2; d.out = ws.hs;
    MF_TRY(launch_qmm(s, d, 1, dense_tiles));
    hs = ws.hs;
    if (w.w_sg) {
      MF_TRY(launch_router_logits(s, w.w_sg, x, 1, c.d, t, c.d, nullptr, ws.gate));
      gate = ws.gate;
    }
  }
  const size_t n4 = static_cast<size_t>(t) * c.d / 4;
  prefill_reduce_kernel<<<dim3(static_cast<uint32_t>((n4 + 255) / 256)), dim3(256), 0, s>>>(
      ws.partials, ws.w, ws.idx, hs, gate, y, t, c.top_k, c.d, c.num_experts);
  MF_TRY(hipGetLastError());
  if (out_idx) MF_TRY(hipMemcpyAsync(out_idx, ws.idx, sizeof(uint32_t) * pairs, hipMemcpyDeviceToDevice, s));
  if (out_w) MF_TRY(hipMemcpyAsync(out_w, ws.w, sizeof(float) * pairs, hipMemcpyDeviceToDevice, s));
#undef MF_TRY
  return hipSuccess;
}

}  // namespace mf
