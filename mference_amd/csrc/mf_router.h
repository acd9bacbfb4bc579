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
  // four steps' loads are requested before the first product is taken: a lane's chunks are one
  // memory round trip, not one per step (the order of the fmaf chain is unchanged)
  for (uint32_t c0 = lane; c0 < chunks; c0 += 4 * kWave) {
    uint4 wv[4], xv[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const uint32_t c = c0 + s * kWave;
      if (c < chunks) {
        if (aligned) {
          wv[s] = load_x8<true>(w + c * 8);
          xv[s] = load_x8<true>(x + c * 8);
        } else {
          wv[s] = load_x8<false>(w + c * 8);
          xv[s] = load_x8<false>(x + c * 8);
        }
      }
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      if (c0 + s * kWave < chunks) {
        acc = __builtin_fmaf(bf16_lo(wv[s].x), bf16_lo(xv[s].x), acc);
        acc = __builtin_fmaf(bf16_hi(wv[s].x), bf16_hi(xv[s].x), acc);
        acc = __builtin_fmaf(bf16_lo(wv[s].y), bf16_lo(xv[s].y), acc);
        acc = __builtin_fmaf(bf16_hi(wv[s].y), bf16_hi(xv[s].y), acc);
        acc = __builtin_fmaf(bf16_lo(wv[s].z), bf16_lo(xv[s].z), acc);
        acc = __builtin_fmaf(bf16_hi(wv[s].z), bf16_hi(xv[s].z), acc);
        acc = __builtin_fmaf(bf16_lo(wv[s].w), bf16_lo(xv[s].w), acc);
        acc = __builtin_fmaf(bf16_hi(wv[s].w), bf16_hi(xv[s].w), acc);
      }
    }
  }
  return wave_sum(acc);
}

// The same for a row of 8-bit affine codes (dequant_int8_gemv_simd, Metal/Quant/dequant_int8.metal:66-107:
// w = q * scale + bias per group of 64, fma(s, sum q x, acc), fma(b, sum x, acc)): chunk c of 8 codes
// belongs to lane c % 64 and lies inside one group; its sum q*x and sum x are built in ascending order
// from 0 and enter the lane's accumulator as the two fmas; lanes combine neighbours first.
__device__ __forceinline__ float dot_q8_row(const uint8_t* __restrict__ q_row, const uint16_t* __restrict__ s_row,
                                            const uint16_t* __restrict__ b_row, const uint16_t* __restrict__ x,
                                            uint32_t d, uint32_t lane, bool aligned) {
  float acc = 0.0f;
  for (uint32_t c = lane; c < d / 8; c += kWave) {
    uint32_t q[2];
    uint4 xv;
    if (aligned) {
      const uint2 qq = *reinterpret_cast<const uint2*>(q_row + c * 8);
      q[0] = qq.x; q[1] = qq.y;
      xv = load_x8<true>(x + c * 8);
    } else {
      const uint8_t* p = q_row + c * 8;
      q[0] = p[0] | (p[1] << 8) | (p[2] << 16) | (static_cast<uint32_t>(p[3]) << 24);
      q[1] = p[4] | (p[5] << 8) | (p[6] << 16) | (static_cast<uint32_t>(p[7]) << 24);
      xv = load_x8<false>(x + c * 8);
    }
    const uint32_t xs[4] = {xv.x, xv.y, xv.z, xv.w};
    float dot = 0.0f, sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float x0 = bf16_lo(xs[j]), x1 = bf16_hi(xs[j]);
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

// ---- workgroup-collective selection (the fused decode launch)
//
// The rank of expert i is the number of experts that beat it under the selectors' total order
// (higher score first, equal scores: lower index first; NaN counts as -inf), so the expert of
// rank r is exactly what round r of the serial selector picks.
__device__ __forceinline__ float score_or_ninf(float x) {
  const float ninf = -__builtin_inff();
  return (x > ninf) ? x : ninf;
}
// a score (no NaN) as an unsigned number that orders like the score; -0 and +0 get one key
__device__ __forceinline__ uint32_t score_key(float x) {
  const uint32_t b = __float_as_uint(x + 0.0f);
  return b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}
__device__ __forceinline__ float key_score(uint32_t k) {
  return __uint_as_float(k ^ ((k >> 31) ? 0x80000000u : 0xFFFFFFFFu));
}
// does (q, j) beat (v, i)?  q, v hold no NaN
__device__ __forceinline__ uint32_t beats(float q, uint32_t j, float v, uint32_t i) {
  return (q > v || (q == v && j < i)) ? 1u : 0u;
}

// Full rank count: every wave takes a block of 64 candidates (one per lane) and a slice of the
// experts to compare them with, read from LDS four at a time as broadcasts, and adds its count to
// rank[] with an LDS atomic.  vals, rank: LDS [t_count][e], vals without NaN, e a multiple of 4,
// rank zero on entry.  A workgroup barrier has to follow before topk_rank_emit.
template <int ORDER>  // -1: every j < i (an equal score beats), +1: every j > i, 0: mixed
__device__ __forceinline__ uint32_t count_beats(const float* lg, uint32_t j0, uint32_t j1, float v, uint32_t i) {
  uint32_t cnt = 0;
  for (uint32_t j = j0; j + 4 <= j1; j += 4) {
    const float4 q = *reinterpret_cast<const float4*>(lg + j);
    if constexpr (ORDER < 0) cnt += (q.x >= v) + (q.y >= v) + (q.z >= v) + (q.w >= v);
    else if constexpr (ORDER > 0) cnt += (q.x > v) + (q.y > v) + (q.z > v) + (q.w > v);
    else cnt += beats(q.x, j, v, i) + beats(q.y, j + 1, v, i) + beats(q.z, j + 2, v, i) + beats(q.w, j + 3, v, i);
  }
  return cnt;
}
__device__ __forceinline__ void topk_rank_count(const float* vals, uint32_t* rank, uint32_t t_count,
                                                uint32_t e, uint32_t wv, uint32_t lane, uint32_t nwaves) {
  const uint32_t eb = (e + kWave - 1) / kWave;  // candidate blocks per token
  const uint32_t blocks = t_count * eb;
  uint32_t split = 1;  // slices of the comparison range, each a multiple of 4 long
  while (blocks * split * 2 <= nwaves && e % (8 * split) == 0) split *= 2;
  const uint32_t jr = e / split;
  for (uint32_t item = wv; item < blocks * split; item += nwaves) {
    const uint32_t b = item / split, js = item % split;
    const uint32_t t = b / eb, i0 = (b % eb) * kWave, i = i0 + lane;
    const float* lg = vals + t * e;
    const float v = i < e ? lg[i] : 0.0f;
    const uint32_t j0 = js * jr, j1 = j0 + jr;
    uint32_t cnt;
    if (j1 <= i0) cnt = count_beats<-1>(lg, j0, j1, v, i);
    else if (j0 >= i0 + kWave) cnt = count_beats<1>(lg, j0, j1, v, i);
    else cnt = count_beats<0>(lg, j0, j1, v, i);
    if (i < e) atomicAdd(&rank[t * e + i], cnt);
  }
}
// Every expert whose rank is below k writes itself to idx / sc [t_count][k] (a value that is not a
// candidate -- -inf -- gives index 0, score -inf, like a round without a winner).  idx / sc
// entries of ranks that no expert takes (k > e) must have been set to 0 / -inf by the caller.
__device__ __forceinline__ void topk_rank_emit(const float* vals, const uint32_t* rank, uint32_t t_count,
                                               uint32_t e, uint32_t k, uint32_t* idx, float* sc,
                                               uint32_t tid, uint32_t nthreads) {
  const float ninf = -__builtin_inff();
  for (uint32_t p = tid; p < t_count * e; p += nthreads) {
    const uint32_t r = rank[p];
    if (r < k) {
      const uint32_t t = p / e, i = p % e;
      const float x = vals[p];
      const bool valid = x > ninf;
      idx[t * k + r] = valid ? i : 0u;
      sc[t * k + r] = valid ? x : ninf;
    }
  }
}

// Selection with a prefilter, for e a multiple of 64 with e / 16 >= k and one wave per block of 64
// experts (t_count * e / 64 <= nwaves).  The k-th largest of the maxima of the 16-expert
// sub-blocks, L, is a lower bound of the k-th largest score: k distinct experts reach it.  So
// every selected expert has a score >= L, and so has everything that beats such an expert: the
// ranks of the experts with score >= L among themselves are their ranks among all.  There are
// usually a dozen of them; they are compacted into a list and one wave per token ranks the list.
// More than 64 of them (many equal scores, or fewer than k finite ones) raise *fallback and the
// caller counts ranks over everything instead.
// scr: LDS words, zero on entry: [0, 256) sub-block maxima, [256, 264) list lengths per token,
// [512, 512 + t_count * 128) the lists of (~index, score key).  Contains workgroup barriers: all
// threads call it.
constexpr uint32_t kPrefilterScratchWords = 512 + MF_MAX_TOKENS * 128;
__device__ __forceinline__ bool topk_prefilter_fits(uint32_t t_count, uint32_t e, uint32_t k, uint32_t nwaves) {
  return e % 64 == 0 && e / 16 >= k && t_count * (e / 64) <= nwaves && t_count * (e / 16) <= 256;
}
__device__ __forceinline__ void topk_prefilter(const float* vals, uint32_t* scr, uint32_t* fallback,
                                               uint32_t t_count, uint32_t e, uint32_t k, uint32_t* idx,
                                               float* sc, uint32_t wv, uint32_t lane) {
  const float ninf = -__builtin_inff();
  float* smax = reinterpret_cast<float*>(scr);
  uint32_t* n_list = scr + 256;
  uint32_t* lists = scr + 512;
  const uint32_t eb = e / kWave, nsb = e / 16;
  const bool mine = wv < t_count * eb;  // this wave has a block
  const uint32_t t = mine ? wv / eb : 0, b = mine ? wv % eb : 0;
  const uint32_t i = b * kWave + lane;
  const float v = mine ? vals[t * e + i] : ninf;
  if (mine) {  // maximum of each row of 16 lanes
    float m = v;
    m = fmaxf(m, dpp_f<0xB1>(m));
    m = fmaxf(m, dpp_f<0x4E>(m));
    m = fmaxf(m, dpp_f<0x141>(m));
    m = fmaxf(m, dpp_f<0x140>(m));
    if ((lane & 15) == 0) smax[t * nsb + b * 4 + lane / 16] = m;
  }
  __syncthreads();
  if (mine) {
    // L: the k-th largest sub-block maximum = the largest maximum that at least k maxima reach
    // (equal maxima need no tie rule here: only the value matters)
    const float* sm = smax + t * nsb;
    const float ml = lane < nsb ? sm[lane] : ninf;
    uint32_t ge = 0;
    for (uint32_t j0 = 0; j0 < nsb; j0 += 16) {  // four LDS reads in flight; maxima past nsb read as -inf
      float4 q[4];
#pragma unroll
      for (uint32_t u = 0; u < 4; ++u)
        q[u] = j0 + 4 * u < nsb ? *reinterpret_cast<const float4*>(sm + j0 + 4 * u) : make_float4(ninf, ninf, ninf, ninf);
#pragma unroll
      for (uint32_t u = 0; u < 4; ++u) ge += (q[u].x >= ml) + (q[u].y >= ml) + (q[u].z >= ml) + (q[u].w >= ml);
    }
    // lanes past nsb hold -inf and count the -inf padding: they never raise the maximum below
    float L = (lane < nsb && ge >= k) ? ml : ninf;
    L = wave_max(L);
    // the experts that reach L join their token's list (in any order: the list is ranked below)
    const bool c = v >= L;
    const unsigned long long cm = __ballot(c);
    const uint32_t n = static_cast<uint32_t>(__popcll(cm));
    uint32_t base = 0;
    if (lane == 0) base = atomicAdd(&n_list[t], n);
    base = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(base)));
    const uint32_t pos = base + __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(cm >> 32),
                                                          __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(cm), 0u));
    if (c && pos < kWave) {  // (score as an unsigned key that sorts like the score, ~index): one 64-bit
                             // comparison then says "beats", ties to the lower index included
      lists[t * 128 + 2 * pos] = ~i;
      lists[t * 128 + 2 * pos + 1] = score_key(v);
    }
  }
  __syncthreads();
  if (wv < t_count) {  // wave t ranks the list of token t
    const uint32_t n = n_list[wv];
    if (n > kWave) {
      if (lane == 0) *fallback = 1u;
    } else {
      const unsigned long long* lst = reinterpret_cast<const unsigned long long*>(lists + wv * 128);
      const unsigned long long me = lane < n ? lst[lane] : 0ull;
      uint32_t r = 0;
      for (uint32_t j0 = 0; j0 < n; j0 += 8) {  // eight entries per step, their LDS reads in flight together
        uint4 o[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) o[u] = *reinterpret_cast<const uint4*>(lists + wv * 128 + 2 * (j0 + 2 * u));
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {  // entries past the list's end beat nothing
          const uint32_t j = j0 + 2 * u;
          const unsigned long long k0 = (static_cast<unsigned long long>(o[u].y) << 32) | o[u].x;
          const unsigned long long k1 = (static_cast<unsigned long long>(o[u].w) << 32) | o[u].z;
          r += (j < n && k0 > me ? 1u : 0u) + (j + 1 < n && k1 > me ? 1u : 0u);
        }
      }
      const float vc = key_score(static_cast<uint32_t>(me >> 32));
      const uint32_t ic = ~static_cast<uint32_t>(me);
      if (lane < n && r < k) {
        const bool valid = vc > ninf;
        idx[wv * k + r] = valid ? ic : 0u;
        sc[wv * k + r] = valid ? vc : ninf;
      }
    }
  }
  __syncthreads();
}

// Routing weight of rank `lane` from the selected scores (my_score in lanes < k): MODE 0
// exp(s_r - s_0) / sum, MODE 1 p_r / (sum + 1e-20); sums in rank order -- the tails of
// topk_select_sorted.  All 64 lanes call it.
template <int MODE>
__device__ __forceinline__ float topk_weight_of_rank(float my_score, uint32_t k) {
  if constexpr (MODE == 1) {
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < MF_MAX_TOPK; ++i)
      if (static_cast<uint32_t>(i) < k) sum += readlane_f(my_score, i);
    return my_score / (sum + 1.0e-20f);
  } else {
    const float s0 = readlane_f(my_score, 0);
    const float my_e = mf_exp(my_score - s0);
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < MF_MAX_TOPK; ++i)
      if (static_cast<uint32_t>(i) < k) sum += readlane_f(my_e, i);
    return my_e / sum;
  }
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
