/*
 * mf_oracle.c — CPU restatement of Mference's MoE expert hot path.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels.  Nothing in the
 * product library links, loads or calls this file.
 *
 * Build: gcc -O3 -march=native -ffp-contract=off -fopenmp (see Makefile).
 * -ffp-contract=off is part of the contract: every place below that wants a
 * fused multiply-add says fmaf(); every other a*b+c is two roundings, as in the
 * Swift/Metal sources it follows.
 *
 * Paths are relative to the Mference repository root.
 *
 * Parity status (what pins each function; "unpinned" = no independent check):
 *   mfo_bf16_bits / to_float      closed form, Quantization.swift:17-28; checked
 *                                 against torch bf16 RNE and spot values.
 *   mfo_quantize_affine bits 4/8  Quantization.swift:50-102 / :135-181; checked
 *                                 by the reference's invariants (nibble order,
 *                                 constant group, codebook ends, error bound,
 *                                 edge list) and by brute-force nearest-code.
 *   mfo_quantize_affine bits 2    PARITY UNPINNED against the reference, which
 *                                 has no 2-bit quantizer to compare with (only
 *                                 random-code fixtures,
 *                                 DSV4ToySynthetic.swift:319-337).  Defined by
 *                                 analogy (scale=(max-min)/3) and checked the
 *                                 way the 4-bit one is: brute-force nearest of
 *                                 the four levels.  The 2-bit DEQUANT / element
 *                                 order is pinned.
 *   mfo_dequantize                closed form q*s+b, two roundings
 *                                 (Quantization.swift:104-119); element order
 *                                 pinned by hand-built byte KATs
 *                                 (moe.metal:898-901 for 2-bit).
 *   mfo_rng_*                     integer closed forms (SplitMix64.swift:11-23,
 *                                 SeedTree.swift:12-19); SplitMix64 checked on
 *                                 its published first outputs for seed 0 and
 *                                 1234567; FNV-1a on published hash values.
 *   mfo_exp                       this build's own deterministic exp (shared
 *                                 bit-for-bit with the HIP kernels); checked
 *                                 against libm to 2 ulp.
 *   mfo_router_logits_bf16        exact products, summation order defined here;
 *                                 checked against fp64 and x=e_i / x=1 cases.
 *   mfo_topk_softmax              moe.metal:190-240; checked against
 *                                 sort-by-(score desc,index asc) on the
 *                                 reference's tie-heavy logit families
 *                                 (RouterTopKParityTests.swift:34,109-127).
 *   mfo_topk_full_softmax         maple_moe.metal:62-119; checked on the
 *                                 reference's tied-score fixture
 *                                 (MapleMoETests.swift:24-40) and sentinels.
 *   mfo_log_1to2,                 this build's own deterministic log on [1,2] (shared
 *   mfo_sqrtsoftplus              bit for bit with the HIP kernels) and moe.metal:736-740;
 *                                 checked against libm (1.2e-7), sqrt(ln 2) at 0, exactly
 *                                 sqrt(x) / 0 beyond |x| = 20, fp64 on [-4, 12].
 *   mfo_router_sqrtsoftplus,      moe.metal:744-786, :847-866; selection checked against
 *   mfo_router_hash_weights       sort-by-(score desc, index asc) on the reference's
 *                                 tie-heavy logits and duplicated biases
 *                                 (RouterTopKParityTests.swift:52-104), weights against
 *                                 fp64 and sum = route_scale; repeated experts.
 *   mfo_router_inkling            inkling.metal:503-566; selection as above, weights against
 *                                 the closed form sigmoid(x_i) / sum sigmoid(x_j) over the
 *                                 picked experts and the sinks, sum = route * global scale.
 *                                 A NaN logit is undefined behaviour in the reference
 *                                 (writes past top_score); here it is never picked.
 *   mfo_router_logits_int8,       moe.metal:102-139 with this build's summation order;
 *   mfo_topk_softmax_scaled       checked against fp64, x = e_i (the two-rounding
 *                                 dequantized weight), effective_scale = 2; the scaled
 *                                 top-k on the reference's per-expert-scale draw
 *                                 (RouterTopKParityTests.swift:30-47).
 *   mfo_gemv / mfo_gemv_multix    DequantInt4Gemv.swift:26-40; checked by
 *                                 x=e_i, x=1, linearity, fp64 brute force.
 *   mfo_expert_*, mfo_shared_*    Moe.swift:58-88 with the rounding points of
 *                                 moe.metal:526-528, dequant_int4.metal:240-245;
 *                                 checked against an independent fp64 numpy
 *                                 composition within the reference tolerance.
 *   mfo_maple_swiglu, the         maple_moe.metal:153-164, 243-264; the bf16 steps
 *   maple_rounding layer          checked on seven inputs followed by hand (clamp
 *                                 sides, both sigmoid branches, overflow, a bf16
 *                                 tie); the layer rebuilt from the phase-1 and
 *                                 down functions.  exp is mfo_exp, not Metal's:
 *                                 PARITY UNPINNED where an exp result sits on a
 *                                 bf16 rounding boundary.
 *   mfo_gelu_tanh,                dequant_int8.metal:44-49, SharedExpertInt8.swift:78-181; the activation
 *   mfo_shared_expert_int8        checked against fp64 tanh (1e-6), 0, +-large; the MLP against an fp64
 *                                 composition of the dequantized weights.  tanh is built on mfo_exp:
 *                                 PARITY UNPINNED against Metal's tanh where a result sits on a bf16
 *                                 rounding boundary.
 *   mfo_residual_rmsnorm          utility.metal:83-92 + rmsnorm.metal:30-92; closed
 *                                 form, checked on hand-computed rows (3-4-0
 *                                 vector, unit vector, eps only) and fp64 numpy.
 *   mfo_group_pairs               PrefillMoEGrouping.swift:91-192; checked on
 *                                 the literal integer KATs of
 *                                 PrefillMoEGroupingTests.swift:5-203.
 *   mfo_reduce_token_major        prefill.metal:631-652; closed form.
 */
#include "mf_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define GROUP 64

/* ------------------------------------------------------------------ bf16 */

/* Quantization.swift:17-23: (bits + 0x7FFF + lsb) >> 16, no NaN special case */
uint16_t mfo_bf16_bits(float x) {
  uint32_t bits;
  memcpy(&bits, &x, 4);
  uint32_t lsb = (bits >> 16) & 1u;
  uint32_t rounded = (bits + 0x7FFFu + lsb) >> 16;
  return (uint16_t)rounded;
}

/* Quantization.swift:25-28 */
float mfo_bf16_to_float(uint16_t b) {
  uint32_t bits = (uint32_t)b << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

void mfo_bf16_encode(const float* x, size_t n, uint16_t* out) {
  for (size_t i = 0; i < n; ++i) out[i] = mfo_bf16_bits(x[i]);
}

void mfo_bf16_decode(const uint16_t* x, size_t n, float* out) {
  for (size_t i = 0; i < n; ++i) out[i] = mfo_bf16_to_float(x[i]);
}

static inline float bfr(float x) { return mfo_bf16_to_float(mfo_bf16_bits(x)); }

/* ------------------------------------------------------------------ PRNG */

mfo_rng mfo_rng_seed(uint64_t seed) {
  mfo_rng r = {seed};
  return r;
}

/* SeedTree.swift:12-19: root ^ FNV-1a-64(label) */
mfo_rng mfo_seed_tree_key(uint64_t root, const char* label) {
  uint64_t h = 0xCBF29CE484222325ull;
  for (const unsigned char* p = (const unsigned char*)label; *p; ++p) {
    h ^= (uint64_t)*p;
    h *= 0x100000001B3ull;
  }
  return mfo_rng_seed(root ^ h);
}

/* SplitMix64.swift:11-17 */
uint64_t mfo_rng_next(mfo_rng* r) {
  r->state += 0x9E3779B97F4A7C15ull;
  uint64_t z = r->state;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

/* SplitMix64.swift:19-23: 24-bit mantissa uniform in [lo, hi) */
float mfo_rng_uniform(mfo_rng* r, float lo, float hi) {
  float u = (float)(mfo_rng_next(r) >> 40) / (float)(1 << 24);
  return lo + (hi - lo) * u;
}

void mfo_rng_uniform_fill(mfo_rng* r, float lo, float hi, float* out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = mfo_rng_uniform(r, lo, hi);
}

void mfo_rng_normal(mfo_rng* r, float mean, float sigma, float* out, size_t n) {
  const double two_pi = 6.283185307179586476925286766559;
  for (size_t i = 0; i < n; i += 2) {
    double u1 = ((double)(mfo_rng_next(r) >> 11) + 1.0) / 9007199254740992.0;
    double u2 = (double)(mfo_rng_next(r) >> 11) / 9007199254740992.0;
    double rad = sqrt(-2.0 * log(u1));
    out[i] = (float)((double)mean + (double)sigma * rad * cos(two_pi * u2));
    if (i + 1 < n) out[i + 1] = (float)((double)mean + (double)sigma * rad * sin(two_pi * u2));
  }
}

/* ---------------------------------------------------------- quantization */

static int codes_per_byte(int bits) {
  switch (bits) {
    case MFO_BITS_8: return 1;
    case MFO_BITS_4: return 2;
    case MFO_BITS_2:
    case MFO_BITS_TERNARY: return 4;
    default: return 0;
  }
}

size_t mfo_packed_row_bytes(int bits, size_t n) {
  int c = codes_per_byte(bits);
  return c ? n / (size_t)c : 0;
}

/* element k of a row: 4-bit low nibble = even index (Quantization.swift:92-98);
 * 2-bit element j at bit 2*(j%4) of byte j/4 (moe.metal:948-951) */
static inline void put_code(uint8_t* row, size_t k, int bits, unsigned q) {
  if (bits == MFO_BITS_8) {
    row[k] = (uint8_t)q;
  } else if (bits == MFO_BITS_4) {
    size_t b = k >> 1;
    if ((k & 1) == 0) row[b] = (uint8_t)((row[b] & 0xF0u) | (q & 0x0Fu));
    else row[b] = (uint8_t)((row[b] & 0x0Fu) | ((q & 0x0Fu) << 4));
  } else {
    size_t b = k >> 2;
    unsigned sh = 2u * (unsigned)(k & 3);
    row[b] = (uint8_t)((row[b] & ~(0x3u << sh)) | ((q & 0x3u) << sh));
  }
}

static inline unsigned get_code(const uint8_t* row, size_t k, int bits) {
  if (bits == MFO_BITS_8) return row[k];
  if (bits == MFO_BITS_4) return (k & 1) == 0 ? (row[k >> 1] & 0x0Fu) : (unsigned)(row[k >> 1] >> 4);
  return (row[k >> 2] >> (2u * (unsigned)(k & 3))) & 0x3u;
}

/* Quantization.swift:50-102 (4-bit), :135-181 (8-bit); 2-bit by analogy */
int mfo_quantize_affine(const float* w, size_t rows, size_t n, int bits,
                        uint8_t* packed, uint16_t* scales, uint16_t* biases) {
  if (n % GROUP != 0) return MFO_ERR_ARG;
  int qmax;
  switch (bits) {
    case MFO_BITS_8: qmax = 255; break;
    case MFO_BITS_4: qmax = 15; break;
    case MFO_BITS_2: qmax = 3; break;
    default: return MFO_ERR_ARG;
  }
  const size_t ngroups = n / GROUP;
  const size_t row_bytes = mfo_packed_row_bytes(bits, n);
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; ++r) {
    const float* row = w + r * n;
    uint8_t* prow = packed + r * row_bytes;
    memset(prow, 0, row_bytes);
    for (size_t g = 0; g < ngroups; ++g) {
      float wmin = INFINITY, wmax = -INFINITY;
      for (size_t k = 0; k < GROUP; ++k) {
        float v = row[g * GROUP + k];
        if (v < wmin) wmin = v;
        if (v > wmax) wmax = v;
      }
      float scale_f, bias_f;
      if (wmax == wmin) {
        scale_f = 1.0f;
        bias_f = wmin;
      } else {
        scale_f = (wmax - wmin) / (float)qmax;
        bias_f = wmin;
      }
      uint16_t sb = mfo_bf16_bits(scale_f), bb = mfo_bf16_bits(bias_f);
      scales[r * ngroups + g] = sb;
      biases[r * ngroups + g] = bb;
      float scale = mfo_bf16_to_float(sb), bias = mfo_bf16_to_float(bb);
      float inv = scale == 0.0f ? 0.0f : 1.0f / scale;
      for (size_t k = 0; k < GROUP; ++k) {
        float t = (row[g * GROUP + k] - bias) * inv;
        /* Swift .rounded() = round half away from zero */
        float rq = roundf(t);
        int q = rq >= (float)qmax ? qmax : (rq <= 0.0f ? 0 : (int)rq);
        put_code(prow, g * GROUP + k, bits, (unsigned)q);
      }
    }
  }
  return 0;
}

int mfo_pack_codes(const uint8_t* codes, size_t rows, size_t n, int bits, uint8_t* packed) {
  if (!codes_per_byte(bits)) return MFO_ERR_ARG;
  const size_t row_bytes = mfo_packed_row_bytes(bits, n);
  memset(packed, 0, rows * row_bytes);
  for (size_t r = 0; r < rows; ++r)
    for (size_t k = 0; k < n; ++k) put_code(packed + r * row_bytes, k, bits, codes[r * n + k]);
  return 0;
}

/* Quantization.swift:104-119: Float(q) * scale + bias, two roundings.
 * Ternary: bias = -scale (RepackPlanner.swift:629,640; MapleMoETests.swift:327-332) */
static void dequant_row_group(const uint8_t* prow, const uint16_t* s, const uint16_t* b, size_t n,
                              int bits, size_t group, float* out) {
  const size_t ngroups = n / group;
  for (size_t g = 0; g < ngroups; ++g) {
    float scale = mfo_bf16_to_float(s[g]);
    float bias = bits == MFO_BITS_TERNARY ? -scale : mfo_bf16_to_float(b[g]);
    for (size_t k = 0; k < group; ++k) {
      float q = (float)get_code(prow, g * group + k, bits);
      float prod = q * scale;
      out[g * group + k] = prod + bias;
    }
  }
}

static void dequant_row(const uint8_t* prow, const uint16_t* s, const uint16_t* b, size_t n,
                        int bits, float* out) {
  dequant_row_group(prow, s, b, n, bits, GROUP, out);
}

int mfo_dequantize(const uint8_t* packed, const uint16_t* scales, const uint16_t* biases,
                   size_t rows, size_t n, int bits, float* out) {
  if (n % GROUP != 0 || !codes_per_byte(bits)) return MFO_ERR_ARG;
  const size_t ngroups = n / GROUP, row_bytes = mfo_packed_row_bytes(bits, n);
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; ++r)
    dequant_row(packed + r * row_bytes, scales + r * ngroups,
                biases ? biases + r * ngroups : NULL, n, bits, out + r * n);
  return 0;
}

/* ---------------------------------------------------------------- router */

/* Deterministic exp shared bit-for-bit with the HIP kernels: range reduction
 * by ln2 (hi/lo), degree-6 polynomial in fmaf form, exact power-of-two scale.
 * Results below e^-86 are 0 so no denormal is ever produced. */
float mfo_exp(float x) {
  if (x != x) return x;
  if (x < -86.0f) return 0.0f;
  if (x > 88.0f) return INFINITY;
  float n = rintf(x * 1.44269504088896341f);
  float r = fmaf(-n, 0.693145751953125f, x);
  r = fmaf(-n, 1.42860682030941723212e-6f, r);
  float p = 1.9875691500e-4f;
  p = fmaf(p, r, 1.3981999507e-3f);
  p = fmaf(p, r, 8.3334519073e-3f);
  p = fmaf(p, r, 4.1665795894e-2f);
  p = fmaf(p, r, 1.6666665459e-1f);
  p = fmaf(p, r, 5.0000001201e-1f);
  float r2 = r * r;
  p = fmaf(p, r2, r);
  p = p + 1.0f;
  int32_t e = (int32_t)n + 127;
  uint32_t sb = (uint32_t)e << 23;
  float scale;
  memcpy(&scale, &sb, 4);
  return p * scale;
}

/* bf16 x bf16 dot in the order the HIP kernel uses, so logits match bit for
 * bit: elements are split into 8-wide chunks; chunk c belongs to lane c % 64;
 * each lane accumulates its elements in ascending order with fmaf into one
 * fp32 accumulator; the 64 lane sums are combined by an xor butterfly with
 * strides 1,2,4,8,16,32 (p[l] = p[l] + p[l^s]): neighbours first.  The reference's order is one
 * Metal SIMD's (moe.metal:162-185); only a fixed order is needed, because the
 * reference itself compares logits under tolerances. */
float mfo_dot_bf16_laneorder(const uint16_t* w, const uint16_t* x, size_t d) {
  float p[64];
  for (int l = 0; l < 64; ++l) p[l] = 0.0f;
  size_t chunks = d / 8;
  for (size_t c = 0; c < chunks; ++c) {
    int l = (int)(c % 64);
    float acc = p[l];
    for (int j = 0; j < 8; ++j)
      acc = fmaf(mfo_bf16_to_float(w[c * 8 + j]), mfo_bf16_to_float(x[c * 8 + j]), acc);
    p[l] = acc;
  }
  for (int s = 1; s <= 32; s <<= 1) {
    float q[64];
    for (int l = 0; l < 64; ++l) q[l] = p[l] + p[l ^ s];
    memcpy(p, q, sizeof p);
  }
  return p[0];
}

void mfo_router_logits_bf16(const uint16_t* w, const uint16_t* x, size_t e, size_t d,
                            float* logits) {
  for (size_t i = 0; i < e; ++i) logits[i] = mfo_dot_bf16_laneorder(w + i * d, x, d);
}

/* moe.metal:190-240 generalised to any k: strictly greater wins, equal score
 * keeps the lower index; weights = exp(s_i - s_0) / sum over the selected. */
void mfo_topk_softmax(const float* logits, size_t e, size_t k, uint32_t* idx, float* w) {
  float* score = (float*)malloc(k * sizeof(float));
  float* ex = (float*)malloc(k * sizeof(float));
  for (size_t i = 0; i < k; ++i) {
    idx[i] = 0;
    score[i] = -INFINITY;
  }
  for (size_t x = 0; x < e; ++x) {
    float s = logits[x];
    if (s <= score[k - 1]) continue;
    size_t pos = k;
    for (size_t i = 0; i < k; ++i) {
      if (s > score[i] || (s == score[i] && x < idx[i])) {
        pos = i;
        break;
      }
    }
    if (pos >= k) continue;
    for (size_t i = k - 1; i > pos; --i) {
      idx[i] = idx[i - 1];
      score[i] = score[i - 1];
    }
    idx[pos] = (uint32_t)x;
    score[pos] = s;
  }
  float max_s = score[0], sum = 0.0f;
  for (size_t i = 0; i < k; ++i) {
    ex[i] = mfo_exp(score[i] - max_s);
    sum += ex[i];
  }
  for (size_t i = 0; i < k; ++i) w[i] = ex[i] / sum;
  free(score);
  free(ex);
}

/* maple_moe.metal:62-119 generalised to e experts (e % 32 == 0 for the
 * blocked tree sum): non-finite logit -> idx = e, w = 0. */
void mfo_topk_full_softmax(const float* logits, size_t e, size_t k, uint32_t* idx, float* w) {
  float* scores = (float*)malloc(e * sizeof(float));
  float maximum = -1.0e30f;
  for (size_t i = 0; i < e; ++i) {
    float l = logits[i];
    if (!isfinite(l)) {
      for (size_t r = 0; r < k; ++r) {
        idx[r] = (uint32_t)e;
        w[r] = 0.0f;
      }
      free(scores);
      return;
    }
    if (l > maximum) maximum = l;
  }
  for (size_t i = 0; i < e; ++i) scores[i] = mfo_exp(logits[i] - maximum);
  float sum = 0.0f;
  for (size_t g = 0; g < e / 32; ++g) {
    float partial[32];
    for (int l = 0; l < 32; ++l) partial[l] = scores[g * 32 + l];
    for (int off = 16; off > 0; off >>= 1)
      for (int l = 0; l < off; ++l) partial[l] += partial[l + off];
    sum += partial[0];
  }
  float recip = 1.0f / (sum + 1.0e-20f);
  for (size_t i = 0; i < e; ++i) scores[i] *= recip;
  float selected = 0.0f;
  for (size_t r = 0; r < k; ++r) {
    float best = -1.0e30f;
    uint32_t bi = 0;
    for (size_t i = 0; i < e; ++i) {
      if (scores[i] > best) {
        best = scores[i];
        bi = (uint32_t)i;
      }
    }
    w[r] = best;
    idx[r] = bi;
    scores[bi] = -1.0e30f;
  }
  for (size_t r = 0; r < k; ++r) selected += w[r];
  for (size_t r = 0; r < k; ++r) w[r] = w[r] / (selected + 1.0e-20f);
  free(scores);
}

/* ------------------------------------------------------- family routers */

/* The selection rule every router of the reference shares (moe.metal:209-225,
 * :764-780; inkling.metal:526-538): scan the experts in ascending order, a
 * strictly greater score goes ahead, an equal score stays behind the earlier
 * expert.  NaN and -inf are never taken; slots nobody filled keep index 0. */
static void select_topk(const float* s, size_t e, size_t k, uint32_t* idx, float* score) {
  for (size_t i = 0; i < k; ++i) {
    idx[i] = 0;
    score[i] = -INFINITY;
  }
  for (size_t x = 0; x < e; ++x) {
    float v = s[x];
    if (!(v > score[k - 1])) continue;
    size_t pos = k - 1;
    while (pos > 0 && score[pos - 1] < v) --pos;
    for (size_t i = k - 1; i > pos; --i) {
      idx[i] = idx[i - 1];
      score[i] = score[i - 1];
    }
    idx[pos] = (uint32_t)x;
    score[pos] = v;
  }
}

/* log(t) for 1 <= t <= 2, the only range the routers need (t = 1 + exp(-|x|)):
 * 2*atanh(s) with s = (t-1)/(t+1) <= 1/3, odd series through s^15 in fmaf
 * form.  t-1 and t+1 are exact, the truncated tail is below 2e-9 relative.  The
 * HIP kernels run the same IEEE sequence, so results agree bit for bit. */
float mfo_log_1to2(float t) {
  float s = (t - 1.0f) / (t + 1.0f);
  float z = s * s;
  float p = 6.6666666667e-2f;          /* 1/15 */
  p = fmaf(p, z, 7.6923076923e-2f);    /* 1/13 */
  p = fmaf(p, z, 9.0909090909e-2f);    /* 1/11 */
  p = fmaf(p, z, 1.1111111111e-1f);    /* 1/9 */
  p = fmaf(p, z, 1.4285714286e-1f);    /* 1/7 */
  p = fmaf(p, z, 2.0e-1f);             /* 1/5 */
  p = fmaf(p, z, 3.3333333333e-1f);    /* 1/3 */
  float r = s * z;
  r = fmaf(r, p, s);
  return r + r;
}

/* moe.metal:736-740: sqrt(max(x,0) + log(1 + exp(-|x|))) */
float mfo_sqrtsoftplus(float x) {
  float sp = (x > 0.0f ? x : 0.0f) + mfo_log_1to2(1.0f + mfo_exp(-fabsf(x)));
  return sqrtf(sp);
}

/* router_topk_select_sqrtsoftplus_k6 (moe.metal:744-786) for any k <= 8: the
 * selection score carries the correction bias, the weights do not; weights are
 * kept fp32 (the reference narrows them to fp16 at :784). */
void mfo_router_sqrtsoftplus(const float* logits, const float* correction_bias, size_t e, size_t k,
                             float route_scale, uint32_t* idx, float* w) {
  float* sel = (float*)malloc(e * sizeof(float));
  float score[8];
  for (size_t x = 0; x < e; ++x) sel[x] = mfo_sqrtsoftplus(logits[x]) + correction_bias[x];
  select_topk(sel, e, k, idx, score);
  free(sel);
  mfo_router_hash_weights(logits, idx, k, route_scale, w);
}

/* router_hash_weights_k6 (moe.metal:847-866): the experts are given. */
void mfo_router_hash_weights(const float* logits, const uint32_t* idx, size_t k, float route_scale,
                             float* w) {
  float sum = 0.0f;
  for (size_t i = 0; i < k; ++i) {
    w[i] = mfo_sqrtsoftplus(logits[idx[i]]);
    sum += w[i];
  }
  const float inv = route_scale / (sum + 1e-20f);
  for (size_t i = 0; i < k; ++i) w[i] = w[i] * inv;
}

/* inkling_router_select (inkling.metal:503-566): selection on sigmoid(logit) +
 * bias over the routed experts; weights are a softmax over the logsigmoid of
 * the RAW logits of the selected experts and the n_shared sink rows that follow
 * the routed ones, times route_scale * global_scale.  k <= 8, n_shared <= 8. */
void mfo_router_inkling(const float* logits, const float* bias, float global_scale,
                        size_t n_routed, size_t n_shared, size_t k, float route_scale,
                        uint32_t* idx, float* w, float* gammas) {
  float* sel = (float*)malloc(n_routed * sizeof(float));
  float score[8], lp[16], ex[16];
  for (size_t x = 0; x < n_routed; ++x) sel[x] = 1.0f / (1.0f + mfo_exp(-logits[x])) + bias[x];
  select_topk(sel, n_routed, k, idx, score);
  free(sel);
  const size_t total = k + n_shared;
  for (size_t i = 0; i < total; ++i) {
    const float x = i < k ? logits[idx[i]] : logits[n_routed + (i - k)];
    lp[i] = (x < 0.0f ? x : 0.0f) - mfo_log_1to2(1.0f + mfo_exp(-fabsf(x)));
  }
  float mx = -INFINITY;
  for (size_t i = 0; i < total; ++i) mx = lp[i] > mx ? lp[i] : mx;
  float denom = 0.0f;
  for (size_t i = 0; i < total; ++i) {
    ex[i] = mfo_exp(lp[i] - mx);
    denom += ex[i];
  }
  const float s_all = route_scale * global_scale / denom;
  for (size_t i = 0; i < k; ++i) w[i] = ex[i] * s_all;
  for (size_t i = 0; i < n_shared; ++i) gammas[i] = ex[k + i] * s_all;
}

/* router_gemv_gemma4_body (moe.metal:102-139): 8-bit affine router rows, x
 * scaled element-wise by effective_scale, per group acc = fma(s, sum q*x', acc);
 * acc = fma(b, sum x', acc).  The summation order is this build's (the
 * reference's is one 32-wide Metal SIMD's): 8-wide chunks dealt to 64 lanes as
 * in mfo_dot_bf16_laneorder, a chunk's two sums by fmaf / add in ascending
 * order from 0, then the two fmas into the lane's accumulator, then the
 * neighbour-first butterfly. */
float mfo_dot_int8_laneorder(const uint8_t* codes, const uint16_t* scales, const uint16_t* biases,
                             const uint16_t* x, const uint16_t* effective_scale, size_t d) {
  float p[64];
  for (int l = 0; l < 64; ++l) p[l] = 0.0f;
  for (size_t c = 0; c < d / 8; ++c) {
    float dot = 0.0f, sum = 0.0f;
    for (int j = 0; j < 8; ++j) {
      const float xs = mfo_bf16_to_float(x[c * 8 + j]) * mfo_bf16_to_float(effective_scale[c * 8 + j]);
      dot = fmaf((float)codes[c * 8 + j], xs, dot);
      sum = sum + xs;
    }
    const size_t g = c * 8 / GROUP;
    float acc = p[c % 64];
    acc = fmaf(mfo_bf16_to_float(scales[g]), dot, acc);
    acc = fmaf(mfo_bf16_to_float(biases[g]), sum, acc);
    p[c % 64] = acc;
  }
  for (int s = 1; s <= 32; s <<= 1) {
    float q[64];
    for (int l = 0; l < 64; ++l) q[l] = p[l] + p[l ^ s];
    memcpy(p, q, sizeof p);
  }
  return p[0];
}

void mfo_router_logits_int8(const uint8_t* codes, const uint16_t* scales, const uint16_t* biases,
                            const uint16_t* x, const uint16_t* effective_scale, size_t e, size_t d,
                            float* logits) {
  for (size_t i = 0; i < e; ++i)
    logits[i] = mfo_dot_int8_laneorder(codes + i * d, scales + i * (d / GROUP), biases + i * (d / GROUP), x,
                                       effective_scale, d);
}

/* router_topk_select_k8 with its per-expert scale (moe.metal:190-240): the
 * softmax weight over the selected, times bf16 per_expert_scale[expert]. */
void mfo_topk_softmax_scaled(const float* logits, const uint16_t* per_expert_scale, size_t e, size_t k,
                             uint32_t* idx, float* w) {
  mfo_topk_softmax(logits, e, k, idx, w);
  for (size_t i = 0; i < k; ++i) w[i] = w[i] * mfo_bf16_to_float(per_expert_scale[idx[i]]);
}

/* ------------------------------------------------------------------ GEMV */

/* DequantInt4Gemv.swift:26-40 with the scalar loop of
 * DequantInt4GEMVReferenceTests.swift:17-30 in place of vDSP_dotpr. */
int mfo_gemv(const uint8_t* packed, const uint16_t* scales, const uint16_t* biases,
             int bits, size_t m, size_t n, const float* x, float* y) {
  return mfo_gemv_group(packed, scales, biases, bits, m, n, GROUP, x, y);
}

/* The same with a scale / bias entry per `group` weights (32 or 64): the gate projection of the
 * DeepSeek-V4 conversion, whose kernel derives the table entry of an element as elem / gate_group_size
 * (moe_int2_gate_up_rows_simd_dev_vec, moe.metal:962-1060); the packed codes do not depend on the group. */
int mfo_gemv_group(const uint8_t* packed, const uint16_t* scales, const uint16_t* biases,
                   int bits, size_t m, size_t n, size_t group, const float* x, float* y) {
  if ((group != 32 && group != GROUP) || n % GROUP != 0 || !codes_per_byte(bits)) return MFO_ERR_ARG;
  const size_t ngroups = n / group, row_bytes = mfo_packed_row_bytes(bits, n);
#pragma omp parallel
  {
    float* wrow = (float*)malloc(n * sizeof(float));
#pragma omp for schedule(static)
    for (size_t r = 0; r < m; ++r) {
      dequant_row_group(packed + r * row_bytes, scales + r * ngroups,
                        biases ? biases + r * ngroups : NULL, n, bits, group, wrow);
      float sum = 0.0f;
      for (size_t i = 0; i < n; ++i) {
        float prod = wrow[i] * x[i];
        sum += prod;
      }
      y[r] = sum;
    }
    free(wrow);
  }
  return 0;
}

int mfo_gemv_multix(const uint8_t* packed, const uint16_t* scales, const uint16_t* biases,
                    int bits, size_t m, size_t n, size_t t, const uint16_t* x, float* y) {
  float* xf = (float*)malloc(n * sizeof(float));
  int rc = 0;
  for (size_t i = 0; i < t && rc == 0; ++i) {
    mfo_bf16_decode(x + i * n, n, xf);
    rc = mfo_gemv(packed, scales, biases, bits, m, n, xf, y + i * m);
  }
  free(xf);
  return rc;
}

/* moe.metal:79-84: x / (1 + exp(-x)) */
float mfo_silu(float x) { return x / (1.0f + mfo_exp(-x)); }

/* int8_gelu_pytorch_tanh (dequant_int8.metal:44-49) */
float mfo_gelu_tanh(float x) {
  const float x3 = x * x * x;
  float inner = 0.7978845608028654f * (x + 0.044715f * x3);
  inner = fminf(fmaxf(inner, -20.0f), 20.0f);
  const float th = 1.0f - 2.0f / (mfo_exp(2.0f * inner) + 1.0f);
  return 0.5f * x * (1.0f + th);
}

/* SharedExpertInt8.encode (SharedExpertInt8.swift:78-181): shared_int8_gate_up_act_simd
 * (dequant_int8.metal:110-164), then dequant_int8_gemv_simd (:66-107) */
int mfo_shared_expert_int8(const uint8_t* gw, const uint16_t* gs, const uint16_t* gb, const uint8_t* uw,
                           const uint16_t* us, const uint16_t* ub, const uint8_t* dw, const uint16_t* ds,
                           const uint16_t* db, size_t d, size_t f, int silu, const uint16_t* x, uint16_t* y) {
  if (d == 0 || f == 0 || d % GROUP || f % GROUP) return MFO_ERR_ARG;
  const size_t longest = d > f ? d : f;
  uint16_t* ones = (uint16_t*)malloc(longest * sizeof(uint16_t));
  uint16_t* act = (uint16_t*)malloc(f * sizeof(uint16_t));
  if (!ones || !act) { free(ones); free(act); return MFO_ERR_ARG; }
  for (size_t i = 0; i < longest; ++i) ones[i] = 0x3F80;
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < f; ++r) {
    const float g = mfo_dot_int8_laneorder(gw + r * d, gs + r * (d / GROUP), gb + r * (d / GROUP), x, ones, d);
    const float u = mfo_dot_int8_laneorder(uw + r * d, us + r * (d / GROUP), ub + r * (d / GROUP), x, ones, d);
    const float gh = mfo_bf16_to_float(mfo_bf16_bits(g)), uh = mfo_bf16_to_float(mfo_bf16_bits(u));
    const float a = silu ? gh / (1.0f + mfo_exp(-gh)) : mfo_gelu_tanh(gh);
    act[r] = mfo_bf16_bits(a * uh);
  }
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < d; ++r)
    y[r] = mfo_bf16_bits(mfo_dot_int8_laneorder(dw + r * f, ds + r * (f / GROUP), db + r * (f / GROUP), act, ones, f));
  free(ones);
  free(act);
  return 0;
}

/* maple_swiglu (maple_moe.metal:153-164): every intermediate is a bf16 number */
static float bf16r(float x) { return mfo_bf16_to_float(mfo_bf16_bits(x)); }
float mfo_maple_swiglu(float gate_projection, float up_projection) {
  const float limit = 7.0f;
  const float gate = bf16r(fminf(bf16r(gate_projection), limit));
  const float up = bf16r(fminf(fmaxf(bf16r(up_projection), -limit), limit));
  const float absolute = gate < 0.0f ? bf16r(-gate) : gate;
  const float exponent = bf16r(mfo_exp(absolute));
  const float denominator = bf16r(1.0f + exponent);
  const float reciprocal = bf16r(1.0f / denominator);
  const float sigmoid = gate < 0.0f ? reciprocal : bf16r(1.0f - reciprocal);
  const float silu = bf16r(gate * sigmoid);
  return bf16r(silu * up);
}

static const uint16_t* u16_at(const uint8_t* base, uint32_t off) {
  return (const uint16_t*)(const void*)(base + off);
}

int mfo_expert_phase1(const uint8_t* blob, const mfo_expert_offsets* off, int bits,
                      size_t d, size_t f, float limit, int maple, const uint16_t* x, uint16_t* acts) {
  return mfo_expert_phase1_gate(blob, off, bits, d, f, GROUP, limit, maple, x, acts);
}

int mfo_expert_phase1_gate(const uint8_t* blob, const mfo_expert_offsets* off, int bits,
                           size_t d, size_t f, size_t gate_group, float limit, int maple,
                           const uint16_t* x, uint16_t* acts) {
  if ((off->gate_s | off->gate_b | off->up_s | off->up_b) & 1u) return MFO_ERR_ARG;
  float* xf = (float*)malloc(d * sizeof(float));
  float* g = (float*)malloc(f * sizeof(float));
  float* u = (float*)malloc(f * sizeof(float));
  mfo_bf16_decode(x, d, xf);
  const int tern = bits == MFO_BITS_TERNARY;
  int rc = mfo_gemv_group(blob + off->gate_w, u16_at(blob, off->gate_s),
                          tern ? NULL : u16_at(blob, off->gate_b), bits, f, d, gate_group, xf, g);
  if (!rc)
    rc = mfo_gemv(blob + off->up_w, u16_at(blob, off->up_s),
                  tern ? NULL : u16_at(blob, off->up_b), bits, f, d, xf, u);
  if (!rc) {
    for (size_t i = 0; i < f; ++i) {
      float gv = g[i], uv = u[i];
      if (maple) { /* maple_moe.metal:203 */
        acts[i] = mfo_bf16_bits(mfo_maple_swiglu(gv, uv));
        continue;
      }
      if (limit > 0.0f) { /* moe.metal:27-34 */
        gv = fminf(gv, limit);
        uv = fminf(fmaxf(uv, -limit), limit);
      }
      float a = mfo_silu(gv) * uv;
      acts[i] = mfo_bf16_bits(a); /* moe.metal:528 narrows the product once */
    }
  }
  free(xf);
  free(g);
  free(u);
  return rc;
}

int mfo_expert_down(const uint8_t* blob, const mfo_expert_offsets* off, int bits,
                    size_t d, size_t f, const uint16_t* acts, float* v) {
  if ((off->down_s | off->down_b) & 1u) return MFO_ERR_ARG;
  float* af = (float*)malloc(f * sizeof(float));
  mfo_bf16_decode(acts, f, af);
  int rc = mfo_gemv(blob + off->down_w, u16_at(blob, off->down_s),
                    bits == MFO_BITS_TERNARY ? NULL : u16_at(blob, off->down_b), bits, d, f,
                    af, v);
  free(af);
  return rc;
}

/* dequant_int4.metal:216-246 (gate and up each narrowed before the activation,
 * then the product narrowed) and :177-180 (down output narrowed) */
int mfo_shared_expert(const uint8_t* gw, const uint16_t* gs, const uint16_t* gb,
                      const uint8_t* uw, const uint16_t* us, const uint16_t* ub,
                      const uint8_t* dw, const uint16_t* ds, const uint16_t* db,
                      int bits, size_t d, size_t f, const uint16_t* x, uint16_t* y) {
  float* xf = (float*)malloc(d * sizeof(float));
  float* g = (float*)malloc(f * sizeof(float));
  float* u = (float*)malloc(f * sizeof(float));
  float* a = (float*)malloc(f * sizeof(float));
  float* o = (float*)malloc(d * sizeof(float));
  mfo_bf16_decode(x, d, xf);
  int rc = mfo_gemv(gw, gs, gb, bits, f, d, xf, g);
  if (!rc) rc = mfo_gemv(uw, us, ub, bits, f, d, xf, u);
  if (!rc) {
    for (size_t i = 0; i < f; ++i) {
      float rg = bfr(g[i]), ru = bfr(u[i]);
      float prod = mfo_silu(rg) * ru;
      a[i] = bfr(prod);
    }
    rc = mfo_gemv(dw, ds, db, bits, d, f, a, o);
  }
  if (!rc) mfo_bf16_encode(o, d, y);
  free(xf);
  free(g);
  free(u);
  free(a);
  free(o);
  return rc;
}

/* utility.metal:49-59 */
void mfo_sigmoid_scalar_mul(uint16_t* y, size_t n, uint16_t gate_bits) {
  float g = mfo_bf16_to_float(gate_bits);
  float den = 1.0f + mfo_exp(-g);
  for (size_t i = 0; i < n; ++i) y[i] = mfo_bf16_bits(mfo_bf16_to_float(y[i]) / den);
}

/* residual_add_fp16 (utility.metal:83-92) + rmsnorm_bf16w (rmsnorm.metal:30-92): hidden is
 * narrowed after the add; the sum of squares of the narrowed values is taken here in double
 * (the kernels sum in fp32 in an order of their own: a test compares within one bf16 step);
 * out = narrow(h * inv * w), two fp32 products, left to right. */
void mfo_residual_rmsnorm(uint16_t* hidden, const uint16_t* delta, const uint16_t* weight,
                          uint16_t* out, size_t d, float eps) {
  double sum = 0.0;
  for (size_t i = 0; i < d; ++i) {
    if (delta) hidden[i] = mfo_bf16_bits(mfo_bf16_to_float(hidden[i]) + mfo_bf16_to_float(delta[i]));
    const double v = mfo_bf16_to_float(hidden[i]);
    sum += v * v;
  }
  const float inv = (float)(1.0 / sqrt(sum / (double)d + (double)eps));
  for (size_t i = 0; i < d; ++i) {
    float v = mfo_bf16_to_float(hidden[i]) * inv;
    v = v * mfo_bf16_to_float(weight[i]);
    out[i] = mfo_bf16_bits(v);
  }
}

/* Moe.swift:58-88 (y = residual + sum_slot w * FFN(x), slot order) with the
 * kernels' rounding points: phase-2 product then add, residual first, one
 * narrowing at the end (moe.metal:1262-1270).  With maple_rounding: MapleMoE's
 * activation and bf16 down outputs (maple_moe.metal:153-164, 243-264; the sum
 * there starts from the first product, which 0 + w*v reproduces exactly). */
int mfo_moe_layer(const mfo_layer* L, const uint16_t* x, uint16_t* y, uint32_t* idx_out,
                  float* w_out, float* logits_out) {
  const size_t d = L->d, f = L->f, e = L->e, k = L->k;
  if (d % GROUP || f % GROUP || k == 0 || k > e) return MFO_ERR_ARG;
  float* logits = (float*)malloc(e * sizeof(float));
  uint32_t* idx = (uint32_t*)malloc(k * sizeof(uint32_t));
  float* w = (float*)malloc(k * sizeof(float));
  uint16_t* acts = (uint16_t*)malloc(f * sizeof(uint16_t));
  float* v = (float*)malloc(d * sizeof(float));
  float* acc = (float*)malloc(d * sizeof(float));
  uint16_t* h1 = (uint16_t*)calloc(d, sizeof(uint16_t));
  int rc = 0;

  mfo_router_logits_bf16(L->router_w, x, e, d, logits);
  if (L->router_mode == 1) mfo_topk_full_softmax(logits, e, k, idx, w);
  else mfo_topk_softmax(logits, e, k, idx, w);

  if (L->fs > 0) {
    rc = mfo_shared_expert(L->sgw, L->sgs, L->sgb, L->suw, L->sus, L->sub, L->sdw, L->sds,
                           L->sdb, L->shared_bits, d, L->fs, x, h1);
    if (!rc && L->gqw) {
      /* the 8-bit row in the lane order of mfo_router_logits_int8, x unscaled (effective scale 1) */
      uint16_t* ones = (uint16_t*)malloc(d * sizeof(uint16_t));
      for (size_t i = 0; i < d; ++i) ones[i] = 0x3F80;
      uint16_t gate = mfo_bf16_bits(mfo_dot_int8_laneorder(L->gqw, L->gqs, L->gqb, x, ones, d));
      free(ones);
      mfo_sigmoid_scalar_mul(h1, d, gate);
    } else if (!rc && L->w_sg) {
      uint16_t gate = mfo_bf16_bits(mfo_dot_bf16_laneorder(L->w_sg, x, d));
      mfo_sigmoid_scalar_mul(h1, d, gate);
    }
  }
  for (size_t i = 0; i < d; ++i) acc[i] = mfo_bf16_to_float(h1[i]);
  for (size_t s = 0; s < k && !rc; ++s) {
    if (idx[s] >= e) continue; /* sentinel route: contributes nothing */
    const uint8_t* blob = L->experts + (size_t)idx[s] * L->expert_stride;
    rc = mfo_expert_phase1_gate(blob, &L->off, L->bits, d, f, L->gate_group ? (size_t)L->gate_group : GROUP,
                                L->swiglu_limit, L->maple_rounding, x, acts);
    if (!rc) rc = mfo_expert_down(blob, &L->off, L->bits, d, f, acts, v);
    if (!rc)
      for (size_t i = 0; i < d; ++i) {
        /* maple_moe.metal:258: the down output is a bf16 number before it meets its weight */
        /* prefill.metal:817-819: the prefill kernels keep a route's result as a 16-bit number */
        float partial = w[s] * (L->maple_rounding || L->narrow_routes ? bf16r(v[i]) : v[i]);
        acc[i] += partial;
      }
  }
  if (!rc) mfo_bf16_encode(acc, d, y);
  if (idx_out) memcpy(idx_out, idx, k * sizeof(uint32_t));
  if (w_out) memcpy(w_out, w, k * sizeof(float));
  if (logits_out) memcpy(logits_out, logits, e * sizeof(float));
  free(logits);
  free(idx);
  free(w);
  free(acts);
  free(v);
  free(acc);
  free(h1);
  return rc;
}

int mfo_moe_layer_tokens(const mfo_layer* L, const uint16_t* x, size_t t, uint16_t* y,
                         uint32_t* idx, float* w, int threads) {
  (void)threads;
  int rc = 0;
  for (size_t i = 0; i < t && !rc; ++i)
    rc = mfo_moe_layer(L, x + i * L->d, y + i * L->d, idx ? idx + i * L->k : NULL,
                       w ? w + i * L->k : NULL, NULL);
  return rc;
}

/* -------------------------------------------------------------- grouping */

void mfo_make_pairs(const uint32_t* idx, const uint32_t* weight_bits, size_t t, size_t k,
                    mfo_pair* out) {
  for (size_t tok = 0; tok < t; ++tok)
    for (size_t r = 0; r < k; ++r) {
      size_t i = tok * k + r;
      out[i].token = (uint32_t)tok;
      out[i].expert = idx[i];
      out[i].rank = (uint32_t)r;
      out[i].weight_bits = weight_bits[i];
    }
}

static const uint64_t* g_sort_keys;

static int pair_cmp(const void* pa, const void* pb) {
  const mfo_pair* a = (const mfo_pair*)pa;
  const mfo_pair* b = (const mfo_pair*)pb;
  if (g_sort_keys) {
    uint64_t ka = g_sort_keys[a->expert], kb = g_sort_keys[b->expert];
    if (ka != kb) return ka < kb ? -1 : 1;
  }
  if (a->expert != b->expert) return a->expert < b->expert ? -1 : 1;
  if (a->token != b->token) return a->token < b->token ? -1 : 1;
  if (a->rank != b->rank) return a->rank < b->rank ? -1 : 1;
  return 0;
}

int mfo_group_pairs(const mfo_pair* pairs, size_t n_pairs, int query_count, int top_k,
                    int num_experts, int tile_expert_count, const uint64_t* sort_keys,
                    size_t n_sort_keys, mfo_pair* sorted, uint32_t* offsets,
                    uint32_t* counts, mfo_group* groups, size_t* n_groups,
                    mfo_tile* tiles, size_t* n_tiles) {
  if (query_count < 0) return MFO_ERR_QUERY_COUNT;
  if (top_k <= 0) return MFO_ERR_TOPK;
  if (num_experts <= 0) return MFO_ERR_NUM_EXPERTS;
  if (tile_expert_count < 1 || tile_expert_count > 16) return MFO_ERR_TILE_COUNT;
  if (sort_keys && n_sort_keys != (size_t)num_experts) return MFO_ERR_SORT_KEYS;
  if (n_pairs != (size_t)query_count * (size_t)top_k) return MFO_ERR_PAIR_COUNT;

  uint8_t* seen = (uint8_t*)calloc(n_pairs ? n_pairs : 1, 1);
  for (size_t i = 0; i < n_pairs; ++i) {
    int rc = 0;
    if (pairs[i].token >= (uint32_t)query_count) rc = MFO_ERR_TOKEN_RANGE;
    else if (pairs[i].rank >= (uint32_t)top_k) rc = MFO_ERR_RANK_RANGE;
    else if (pairs[i].expert >= (uint32_t)num_experts) rc = MFO_ERR_EXPERT_RANGE;
    else {
      size_t key = (size_t)pairs[i].token * (size_t)top_k + pairs[i].rank;
      if (seen[key]) rc = MFO_ERR_DUPLICATE;
      seen[key] = 1;
    }
    if (rc) {
      free(seen);
      return rc;
    }
  }
  free(seen);

  memcpy(sorted, pairs, n_pairs * sizeof(mfo_pair));
  g_sort_keys = sort_keys;
  qsort(sorted, n_pairs, sizeof(mfo_pair), pair_cmp);
  g_sort_keys = NULL;

  for (int e = 0; e < num_experts; ++e) {
    offsets[e] = 0xFFFFFFFFu;
    counts[e] = 0;
  }
  size_t ng = 0, i = 0;
  while (i < n_pairs) {
    uint32_t expert = sorted[i].expert;
    size_t start = i;
    while (i < n_pairs && sorted[i].expert == expert) ++i;
    offsets[expert] = (uint32_t)start;
    counts[expert] = (uint32_t)(i - start);
    groups[ng].expert = expert;
    groups[ng].pair_start = (uint32_t)start;
    groups[ng].pair_count = (uint32_t)(i - start);
    ++ng;
  }
  size_t nt = 0, gs = 0;
  while (gs < ng) {
    size_t ge = gs + (size_t)tile_expert_count < ng ? gs + (size_t)tile_expert_count : ng;
    tiles[nt].group_start = (uint32_t)gs;
    tiles[nt].group_count = (uint32_t)(ge - gs);
    tiles[nt].pair_start = groups[gs].pair_start;
    tiles[nt].pair_count =
        groups[ge - 1].pair_start + groups[ge - 1].pair_count - groups[gs].pair_start;
    ++nt;
    gs = ge;
  }
  *n_groups = ng;
  *n_tiles = nt;
  return 0;
}

/* prefill.metal:631-652 */
void mfo_reduce_token_major(const float* partials, const float* w, size_t t, size_t k,
                            size_t d, float* h2) {
  for (size_t tok = 0; tok < t; ++tok)
    for (size_t i = 0; i < d; ++i) {
      float acc = 0.0f;
      for (size_t r = 0; r < k; ++r)
        acc = fmaf(w[tok * k + r], partials[(tok * k + r) * d + i], acc);
      h2[tok * d + i] = acc;
    }
}
