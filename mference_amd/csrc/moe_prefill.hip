// Ragged prefill: router for many tokens, device-side grouping of the
// (token, expert) routes, and the tokens-sorted-by-expert quantized matmul on
// the bf16 matrix cores.
//
// The matmul keeps the 4-bit codes EXACT: a lane's packed uint32 (8 codes of
// one weight row) is masked straight into four bf16 pairs 8 + q/2
// (0x4100 | q << 3), which is a matrix-core operand as it stands -- no LDS
// staging of weights.  x rows are pre-permuted once per call to the same
// (j, j+4) pairing and staged through LDS per 64-wide K group.  Per K group the
// matrix core yields sum((8 + q/2) * x) (bf16 x bf16 products are exact in
// fp32), and the group's bf16 scale is applied in fp32: acc += 2s * tmp -- the
// reference's own factoring s*sum(q*x) + b*sum(x)
// (Metal/Quant/dequant_int4.metal:14-17), so no weight is ever rounded to bf16
// (rounding q*s+b to bf16 would cost ~1.6e-3 relative error per weight, above
// the layer tolerance).  The b*sum(x) and -16*s*sum(x) terms are two more small
// matmuls over the group index (operands: the bf16 bias / scale tables, exact,
// and sum(x) split into three bf16 terms, exact).
//
// Replaces prefill_grouped_routed_moe_batched_{phase1,down}
// (Metal/Prefill/prefill.metal:748-820), prefill_moe_reduce_token_major
// (:631-652) and the staged-affine tensor-core QMM
// mpp_prefill_affine_threadgroup_f16 (Metal/TensorCore/tensorops.metal:13-105).
#include <type_traits>

#include "mf_device.h"
#include "mf_internal.h"
#include "mf_router.h"

#pragma clang fp contract(off)

namespace mf {

constexpr uint32_t kTileTokens = 64;   // tokens of one expert a workgroup handles
constexpr uint32_t kQmmWaves = 4;      // waves per workgroup, 32 weight rows each
constexpr uint32_t kQmmRows = kQmmWaves * 32;
constexpr uint32_t kQmmXBytes = 2 * 2 * 512 * 16;  // x tile ring: 2 stages of 2 K groups

struct Tile {
  uint32_t expert, pair_start, count, pad;
};

// ------------------------------------------------------------------ router

// logits[t, e] for many tokens, bit-exact with dot_bf16_row: a wave keeps R
// expert rows in registers (lane l holds the chunks l, l+64, ... of each row)
// and streams token rows past them.
template <int CPL, int R>
__device__ __forceinline__ void router_rows(const uint16_t* __restrict__ W, const uint16_t* __restrict__ x,
                                            uint32_t E, uint32_t D, uint32_t T, uint32_t x_stride,
                                            float* __restrict__ logits, uint32_t tokens_per_block, uint32_t ld,
                                            uint32_t lane, uint32_t wv);

// What a short batch hangs on the router launch so that it needs no launch of its own: the x
// preparation (matmul order, group sums, scalar shared gate) in extra workgroup columns.  (The top-k of
// a token block by the last workgroup to finish that block's logits was tried and lost: the
// device-wide fence every workgroup needs for it costs more than the launch it saves.)
struct RouterTail {
  uint16_t* xp;          // null: none of this
  uint32_t router_cols;  // workgroup columns that compute logits; the columns behind them prepare x
  const uint16_t* w_sg;  // null: no scalar gate
  float* sums;
  uint16_t* gate;
};

__device__ __forceinline__ void prep_x_row(const uint16_t* __restrict__ x, uint16_t* __restrict__ xp,
                                           float* __restrict__ sums, const uint16_t* __restrict__ w_sg,
                                           uint16_t* __restrict__ gate, uint32_t row, uint32_t d, uint32_t lane);

template <int CPL, int R>
__global__ __launch_bounds__(256) void prefill_router_kernel(const uint16_t* __restrict__ W,
                                                             const uint16_t* __restrict__ x,
                                                             uint32_t E, uint32_t D, uint32_t T,
                                                             uint32_t x_stride,
                                                             float* __restrict__ logits,
                                                             uint32_t tokens_per_block, uint32_t ld,
                                                             const RouterTail tail) {
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  if (tail.xp && blockIdx.x >= tail.router_cols) {  // an x-preparation workgroup: one row per wave
    const uint32_t row = ((blockIdx.x - tail.router_cols) * gridDim.y + blockIdx.y) * 4 + wv;
    if (row < T) prep_x_row(x + static_cast<size_t>(row) * x_stride, tail.xp, tail.sums, tail.w_sg, tail.gate, row, D, lane);
    return;
  }
  router_rows<CPL, R>(W, x, E, D, T, x_stride, logits, tokens_per_block, ld, lane, wv);
}

template <int CPL, int R>
__device__ __forceinline__ void router_rows(const uint16_t* __restrict__ W, const uint16_t* __restrict__ x,
                                            uint32_t E, uint32_t D, uint32_t T, uint32_t x_stride,
                                            float* __restrict__ logits, uint32_t tokens_per_block, uint32_t ld,
                                            uint32_t lane, uint32_t wv) {
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
      if (lane == 0 && row0 + r < E) logits[static_cast<size_t>(t) * ld + row0 + r] = v;
    }
  }
}

// The same logits on the fp32 matrix core, still bit for bit: a K=1 outer-product MFMA adds
// exactly one product to every accumulator element, c <- fl(c + x*w), and x*w is exact for
// bf16 inputs -- so a run of K=1 MFMAs is the per-lane fmaf chain of dot_bf16_row for a whole
// 32-token x 32-expert block at once.  "Lane l" of the reference order becomes chain l: the K
// values 8l..8l+7, then +512, +1024, ...  The two blocks of one instruction carry chains l and
// l+1; their accumulators are added (the stride-1 level of the butterfly), then combined with
// the later pairs as a binary counter, which reproduces the ascending-stride tree.  Each of the
// four waves of a workgroup owns 16 chains; the last two levels go through LDS.
// Needs D % 512 == 0 (all 64 chains the same length) and E % 32 == 0.
typedef __attribute__((ext_vector_type(32))) float f32x32_t;

// N_I = D / 512 as a compile-time constant unrolls the whole walk (a wave's 8 chain pairs x N_I runs): the
// operand offsets, the ring slots and the levels of the binary counter are then literals, the operand ring
// needs no register moves and a chain's first instruction takes the constant 0 as its accumulator -- 3.9
// vector instructions per matrix instruction where the loop for any width (N_I = 0) issues 10.6, and the
// matrix instructions of a SIMD wait for its vector instructions (T=2048: 38.6 -> 34.1 us, T=512: 18.5 ->
// 14.8 us).  (The unrolled form needs 123 registers; eight waves of 8 chains per block, four to a SIMD,
// measured no faster than these four of 16 chains: 34.7 / 15.8 us.)  Three waves per SIMD: the x-preparation
// workgroups behind the router's then share the CUs with them instead of waiting for a second round (-1.3 us).
template <int N_I>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(N_I > 0 ? 3 : 2, N_I > 0 ? 3 : 2)))
void prefill_router_mfma_kernel(const uint16_t* __restrict__ W,
                                                                  const uint16_t* __restrict__ x,
                                                                  uint32_t E, uint32_t D, uint32_t T,
                                                                  uint32_t x_stride,
                                                                  float* __restrict__ logits, uint32_t ld,
                                                                  const RouterTail tail) {
  constexpr int WAVES = 4, kPairs = 32 / WAVES;  // waves of a workgroup, chain pairs of one wave
  __shared__ float s_part[WAVES - 1][16 * 64];
  __shared__ uint4 s_stage[N_I > 0 ? WAVES : 1][2][N_I > 0 ? 2 * 128 : 1];  // per wave: x and w, two buffers of 32 rows x 64 B
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  if (tail.xp && blockIdx.y >= tail.router_cols) {  // an x-preparation workgroup (rows behind the expert blocks)
    const uint32_t row = ((blockIdx.y - tail.router_cols) * gridDim.x + blockIdx.x) * WAVES + wv;
    if (row < T) prep_x_row(x + static_cast<size_t>(row) * x_stride, tail.xp, tail.sums, tail.w_sg, tail.gate, row, D, lane);
    return;
  }
  const uint32_t m = lane & 31, b = lane >> 5;
  // token tiles vary fastest: workgroups go to the XCDs round-robin, so each XCD's L2 sees an
  // eighth of the token rows (and all of the small router matrix)
  const uint32_t t0 = blockIdx.x * 32, e0 = blockIdx.y * 32;
  const uint32_t n_i = D / 512;
  const uint16_t* xrow = x + static_cast<size_t>(min(t0 + m, T - 1)) * x_stride + 8 * (2 * kPairs * wv + b);
  const uint16_t* wrow = W + static_cast<size_t>(e0 + m) * D + 8 * (2 * kPairs * wv + b);

  float lev0[16], lev1[16], lev2[16], total[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) lev0[r] = lev1[r] = lev2[r] = total[r] = 0.0f;
  if constexpr (N_I > 0) {
    // A lane needs 16 bytes of its token row and of its expert row per step -- read straight from memory
    // that is 32 rows, 32 cache lines, per load instruction, and the L1's line rate, not the matrix core,
    // sets the pace.  So the wave fetches 64 contiguous bytes of every row at a time (the operands of two
    // chain pairs: four lanes side by side, 16 lines per instruction) and hands them to itself through a
    // wave-private LDS buffer.  A stage is (pair group pg, K run i): 2 steps, 16 matrix instructions.  The
    // two chain pairs of a group keep an accumulator each across the runs.
    constexpr int kGroups = kPairs / 2, kStages = kGroups * N_I;
    const uint32_t ld_row = lane >> 2, ld_chunk = lane & 3;  // fetch: rows ld_row, ld_row + 16; 16-byte chunk
    const uint16_t* xsrc[2];
    const uint16_t* wsrc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      xsrc[j] = x + static_cast<size_t>(min(t0 + ld_row + 16 * j, T - 1)) * x_stride + 8 * (2 * kPairs * wv + ld_chunk);
      wsrc[j] = W + static_cast<size_t>(e0 + ld_row + 16 * j) * D + 8 * (2 * kPairs * wv + ld_chunk);
    }
    // LDS rows of 64 bytes; chunk c of row r sits in slot c ^ ((r >> 2) & 3): 16 lanes that read the same
    // chunk of 16 consecutive rows then cover 256 bytes of distinct banks
    uint4* stage_x = s_stage[wv][0];
    uint4* stage_w = s_stage[wv][1];
    uint32_t st_at[2], rd_at[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t r = ld_row + 16 * j;
      st_at[j] = r * 4 + (ld_chunk ^ ((r >> 2) & 3));
      rd_at[j] = m * 4 + ((2 * j + b) ^ ((m >> 2) & 3));  // pair j of the group, block b
    }
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    u32x4_t fx0, fx1, fw0, fw1;  // the stage on its way from memory to LDS
#define MF_ROUTER_FETCH(ST)                                                                          \
  do {                                                                                               \
    const int f_off = 32 * ((ST) / N_I) + 512 * ((ST) % N_I);                                        \
    fx0 = *reinterpret_cast<const u32x4_t*>(xsrc[0] + f_off);                                        \
    fx1 = *reinterpret_cast<const u32x4_t*>(xsrc[1] + f_off);                                        \
    fw0 = *reinterpret_cast<const u32x4_t*>(wsrc[0] + f_off);                                        \
    fw1 = *reinterpret_cast<const u32x4_t*>(wsrc[1] + f_off);                                        \
  } while (0)
#define MF_ROUTER_PUT(BUF)                                                                           \
  do {                                                                                               \
    *reinterpret_cast<u32x4_t*>(stage_x + (BUF) * 128 + st_at[0]) = fx0;                             \
    *reinterpret_cast<u32x4_t*>(stage_x + (BUF) * 128 + st_at[1]) = fx1;                             \
    *reinterpret_cast<u32x4_t*>(stage_w + (BUF) * 128 + st_at[0]) = fw0;                             \
    *reinterpret_cast<u32x4_t*>(stage_w + (BUF) * 128 + st_at[1]) = fw1;                             \
  } while (0)
    MF_ROUTER_FETCH(0);
    MF_ROUTER_PUT(0);
    if (kStages > 1) MF_ROUTER_FETCH(1);
    f32x32_t acc[2];
#pragma unroll
    for (int st = 0; st < kStages; ++st) {
      const int pg = st / N_I, i = st % N_I;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const uint4 cxq = stage_x[(st & 1) * 128 + rd_at[j]], cwq = stage_w[(st & 1) * 128 + rd_at[j]];
        const uint32_t xw[4] = {cxq.x, cxq.y, cxq.z, cxq.w}, ww[4] = {cwq.x, cwq.y, cwq.z, cwq.w};
        float xa[8], wa[8];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          xa[2 * u] = bf16_lo(xw[u]); xa[2 * u + 1] = bf16_hi(xw[u]);
          wa[2 * u] = bf16_lo(ww[u]); wa[2 * u + 1] = bf16_hi(ww[u]);
        }
        // all 16 operands in registers of their own before the step's first matrix instruction (see below)
        asm volatile("" : "+v"(xa[0]), "+v"(xa[1]), "+v"(xa[2]), "+v"(xa[3]), "+v"(xa[4]), "+v"(xa[5]), "+v"(xa[6]), "+v"(xa[7]),
                          "+v"(wa[0]), "+v"(wa[1]), "+v"(wa[2]), "+v"(wa[3]), "+v"(wa[4]), "+v"(wa[5]), "+v"(wa[6]), "+v"(wa[7]));
        if (i == 0) {  // a chain's first product lands on 0
          f32x32_t zero;
#pragma unroll
          for (int r = 0; r < 32; ++r) zero[r] = 0.0f;
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x1f32(xa[0], wa[0], zero, 0, 0, 0);
        } else {
          acc[j] = __builtin_amdgcn_mfma_f32_32x32x1f32(xa[0], wa[0], acc[j], 0, 0, 0);
        }
#pragma unroll
        for (int u = 1; u < 8; ++u) acc[j] = __builtin_amdgcn_mfma_f32_32x32x1f32(xa[u], wa[u], acc[j], 0, 0, 0);
      }
      if (st + 1 < kStages) {  // the next stage into the other buffer (read last a stage ago), the one after it on its way
        MF_ROUTER_PUT((st + 1) & 1);
        if (st + 2 < kStages) MF_ROUTER_FETCH(st + 2);
      }
      if (i == N_I - 1) {  // two pairs of chains are complete: stride-1 level, then the binary counter
        constexpr int kLevels = kPairs == 8 ? 3 : 2;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int pp = 2 * pg + j;
          float carry[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) carry[r] = acc[j][r] + acc[j][16 + r];
          int level = 0;
#pragma unroll
          for (; level < kLevels && ((pp >> level) & 1); ++level) {
            float* lv = level == 0 ? lev0 : level == 1 ? lev1 : lev2;
#pragma unroll
            for (int r = 0; r < 16; ++r) carry[r] = lv[r] + carry[r];
          }
          float* dst = level == kLevels ? total : level == 0 ? lev0 : level == 1 ? lev1 : lev2;
#pragma unroll
          for (int r = 0; r < 16; ++r) dst[r] = carry[r];
        }
      }
    }
#undef MF_ROUTER_FETCH
#undef MF_ROUTER_PUT
  } else {
  // step q = pp * n_i + i: chain pair pp (chains 16 wv + 2 pp + b), K run i; operands run 4 steps ahead
  const uint32_t steps = 8 * n_i;
  uint4 cx[4], cw[4], nx[4], nw[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const uint32_t q = min(static_cast<uint32_t>(u), steps - 1), off = 16 * (q / n_i) + 512 * (q % n_i);
    cx[u] = *reinterpret_cast<const uint4*>(xrow + off);
    cw[u] = *reinterpret_cast<const uint4*>(wrow + off);
  }
  f32x32_t acc;
#pragma unroll
  for (int r = 0; r < 32; ++r) acc[r] = 0.0f;
  uint32_t pp = 0, i = 0;
  for (uint32_t q0 = 0; q0 < steps; q0 += 4) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t q = min(q0 + 4 + u, steps - 1), off = 16 * (q / n_i) + 512 * (q % n_i);
      nx[u] = *reinterpret_cast<const uint4*>(xrow + off);
      nw[u] = *reinterpret_cast<const uint4*>(wrow + off);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (q0 + u >= steps) break;
      // The 16 operands of the step's 8 matrix instructions, each in a register of its own, before the
      // first of them issues: a vector instruction that writes a register an MFMA in flight still reads
      // as A or B waits until that MFMA is done (64 cycles here), so operands made one at a time in a
      // recycled register pair cost 89 instead of 65 cycles per instruction.
      const uint32_t xw[4] = {cx[u].x, cx[u].y, cx[u].z, cx[u].w}, ww[4] = {cw[u].x, cw[u].y, cw[u].z, cw[u].w};
      float xa[8], wa[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        xa[2 * j] = bf16_lo(xw[j]); xa[2 * j + 1] = bf16_hi(xw[j]);
        wa[2 * j] = bf16_lo(ww[j]); wa[2 * j + 1] = bf16_hi(ww[j]);
      }
      asm volatile("" : "+v"(xa[0]), "+v"(xa[1]), "+v"(xa[2]), "+v"(xa[3]), "+v"(xa[4]), "+v"(xa[5]), "+v"(xa[6]), "+v"(xa[7]),
                        "+v"(wa[0]), "+v"(wa[1]), "+v"(wa[2]), "+v"(wa[3]), "+v"(wa[4]), "+v"(wa[5]), "+v"(wa[6]), "+v"(wa[7]));
#pragma unroll
      for (int j = 0; j < 8; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x1f32(xa[j], wa[j], acc, 0, 0, 0);
      if (++i == n_i) {  // the pair of chains is complete: stride-1 level, then the binary counter
        float carry[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) carry[r] = acc[r] + acc[16 + r];
#pragma unroll
        for (int r = 0; r < 32; ++r) acc[r] = 0.0f;
        if (pp & 1) {
#pragma unroll
          for (int r = 0; r < 16; ++r) carry[r] = lev0[r] + carry[r];
          if (pp & 2) {
#pragma unroll
            for (int r = 0; r < 16; ++r) carry[r] = lev1[r] + carry[r];
            if (pp & 4) {
#pragma unroll
              for (int r = 0; r < 16; ++r) total[r] = lev2[r] + carry[r];
            } else {
#pragma unroll
              for (int r = 0; r < 16; ++r) lev2[r] = carry[r];
            }
          } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) lev1[r] = carry[r];
          }
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) lev0[r] = carry[r];
        }
        i = 0;
        ++pp;
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      cx[u] = nx[u];
      cw[u] = nw[u];
    }
  }
  }  // the loop for any width
  if (wv > 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) s_part[wv - 1][r * 64 + lane] = total[r];
  }
  __syncthreads();
  if (wv == 0) {  // the last levels of the tree: neighbouring waves first
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float v[WAVES];
      v[0] = total[r];
#pragma unroll
      for (int u = 1; u < WAVES; ++u) v[u] = s_part[u - 1][r * 64 + lane];
#pragma unroll
      for (int stride = 1; stride < WAVES; stride *= 2)
#pragma unroll
        for (int u = 0; u < WAVES; u += 2 * stride) v[u] = v[u] + v[u + stride];
      const uint32_t t = t0 + 8 * (r / 4) + 4 * b + (r % 4);
      if (t < T) logits[static_cast<size_t>(t) * ld + e0 + m] = v[0];
    }
  }
}

// ---------------------------------------------------------------- grouping
//
// PrefillMoEGrouping.groupTokenExpertPairs (PrefillMoEGrouping.swift:91-192) on
// device: pairs come token-major (token, rank), so "sorted by (expert, token,
// rank)" is a stable counting sort by expert.  The pair list is cut into at
// most kGroupChunks chunks; every chunk counts its routes per expert, one
// block turns the counts into per-(chunk, expert) start positions, and every
// chunk then places its routes in order.

constexpr uint32_t kGroupChunks = 256;   // rows of the per-chunk count matrix
constexpr uint32_t kGroupBlock = 256;    // pairs one workgroup handles per step

__global__ __launch_bounds__(256) void group_count_kernel(const uint32_t* __restrict__ idx,
                                                          uint32_t n_pairs, uint32_t E,
                                                          uint32_t chunk_pairs,
                                                          uint32_t* __restrict__ chunk_hist,
                                                          uint32_t* __restrict__ chunk_bad) {
  __shared__ uint32_t s_hist[MF_MAX_EXPERTS];
  for (uint32_t e = threadIdx.x; e < E; e += blockDim.x) s_hist[e] = 0;
  __syncthreads();
  const uint32_t p0 = blockIdx.x * chunk_pairs, p1 = min(n_pairs, p0 + chunk_pairs);
  bool bad = false;
  for (uint32_t p = p0 + threadIdx.x; p < p1; p += blockDim.x) {
    const uint32_t e = idx[p];
    if (e < E) atomicAdd(&s_hist[e], 1u);
    else bad = true;
  }
  // one flag per chunk, always written: nothing has to be cleared before the launch
  const int any_bad = __syncthreads_or(bad ? 1 : 0);
  if (threadIdx.x == 0) chunk_bad[blockIdx.x] = any_bad ? 1u : 0u;
  for (uint32_t e = threadIdx.x; e < E; e += blockDim.x) chunk_hist[blockIdx.x * E + e] = s_hist[e];
}

// From every expert's count (thread e holds c; threads past MF_MAX_EXPERTS only keep the barriers
// company): counts, offsets (0xFFFFFFFF for an empty expert), the start of every expert's run and
// the tile list of the matmul (runs of kTileTokens routes).
__device__ __forceinline__ void group_layout(uint32_t c, uint32_t E, uint32_t* __restrict__ counts,
                                             uint32_t* __restrict__ offsets, uint32_t* __restrict__ starts,
                                             Tile* __restrict__ tiles, uint32_t tile_slots,
                                             uint32_t* __restrict__ n_tiles, uint32_t* s_cnt, uint32_t* s_tile,
                                             bool publish = true) {
  const uint32_t e = threadIdx.x;
  const bool act = e < MF_MAX_EXPERTS;
  if (!publish) tiles = nullptr, n_tiles = nullptr;  // the scans only (s_cnt, s_tile): another workgroup writes
  if (publish && e < E) counts[e] = c;
  // inclusive scans of the counts and of the tile counts over the MF_MAX_EXPERTS entries: inside a wave
  // by shuffles, the eight wave totals through the last slots of the two arrays' neighbours
  __shared__ uint32_t s_wave_cnt[MF_MAX_EXPERTS / 64], s_wave_tile[MF_MAX_EXPERTS / 64];
  uint32_t run_c = act ? c : 0u, run_t = act ? (c + kTileTokens - 1) / kTileTokens : 0u;
  const uint32_t lane = e & 63u;
  for (uint32_t o = 1; o < 64; o <<= 1) {
    const uint32_t a = static_cast<uint32_t>(__shfl_up(static_cast<int>(run_c), o, 64));
    const uint32_t b = static_cast<uint32_t>(__shfl_up(static_cast<int>(run_t), o, 64));
    if (lane >= o) {
      run_c += a;
      run_t += b;
    }
  }
  if (act && lane == 63) {
    s_wave_cnt[e >> 6] = run_c;
    s_wave_tile[e >> 6] = run_t;
  }
  __syncthreads();
  if (act) {
    for (uint32_t v = 0; v < (e >> 6); ++v) {
      run_c += s_wave_cnt[v];
      run_t += s_wave_tile[v];
    }
    s_cnt[e] = run_c;
    s_tile[e] = run_t;
  }
  __syncthreads();
  // The tile list has tile_slots entries (a multiple of 8).  The matmul sends the workgroups of
  // slot range k * tile_slots/8 .. to XCD k, so every eighth of the list gets an eighth of the
  // live tiles, in expert order; the rest of each eighth stays empty (count 0).
  if (tiles) {
    for (uint32_t i = e; i < tile_slots; i += blockDim.x) tiles[i] = Tile{0, 0, 0, 0};
    __syncthreads();
  }
  if (publish && e < E) {
    const uint32_t start = s_cnt[e] - c;
    starts[e] = start;
    offsets[e] = c ? start : 0xFFFFFFFFu;
    if (tiles) {
      const uint32_t total = s_tile[MF_MAX_EXPERTS - 1], per_live = (total + 7) / 8, per_slot = tile_slots / 8;
      const uint32_t nt = (c + kTileTokens - 1) / kTileTokens, t0 = s_tile[e] - nt;
      for (uint32_t j = 0; j < nt; ++j) {
        const uint32_t id = t0 + j;
        tiles[(id / per_live) * per_slot + id % per_live] =
            Tile{e, start + j * kTileTokens, min(kTileTokens, c - j * kTileTokens), 0};
      }
    }
  }
  if (n_tiles && e == MF_MAX_EXPERTS - 1) *n_tiles = s_tile[e];
}

// counts, offsets (0xFFFFFFFF for an empty expert), the start of every expert's
// run, chunk_hist turned into each chunk's first position inside its expert's
// run, and the tile list of the matmul (runs of kTileTokens routes).
__global__ __launch_bounds__(512) void group_scan_kernel(uint32_t* __restrict__ chunk_hist,
                                                         uint32_t n_chunks, uint32_t E,
                                                         uint32_t* __restrict__ counts,
                                                         uint32_t* __restrict__ offsets,
                                                         uint32_t* __restrict__ starts,
                                                         Tile* __restrict__ tiles,
                                                         uint32_t tile_slots,
                                                         uint32_t* __restrict__ n_tiles,
                                                         const uint32_t* __restrict__ chunk_bad,
                                                         uint32_t* __restrict__ status,
                                                         int drop_if_bad = 0) {
  __shared__ uint32_t s_cnt[MF_MAX_EXPERTS], s_tile[MF_MAX_EXPERTS];
  const uint32_t e = threadIdx.x;
  // status word: 2 when any chunk met an expert index out of range (n_chunks <= blockDim)
  const int any_bad = __syncthreads_or(e < n_chunks && chunk_bad[e] ? 1 : 0);
  if (e == 0) *status = any_bad ? 2u : 0u;
  uint32_t c = 0;
  if (e < E && !(any_bad && drop_if_bad)) {  // a caller's grouping that failed its check yields no tiles
    uint32_t k = 0;
    for (; k + 32 <= n_chunks; k += 32) {  // 32 independent loads in flight: the loop is all latency
      uint32_t v[32];
#pragma unroll
      for (int u = 0; u < 32; ++u) v[u] = chunk_hist[(k + u) * E + e];
#pragma unroll
      for (int u = 0; u < 32; ++u) {
        chunk_hist[(k + u) * E + e] = c;
        c += v[u];
      }
    }
    for (; k < n_chunks; ++k) {
      const uint32_t v = chunk_hist[k * E + e];
      chunk_hist[k * E + e] = c;
      c += v;
    }
  }
  group_layout(c, E, counts, offsets, starts, tiles, tile_slots, n_tiles, s_cnt, s_tile);
}

__global__ __launch_bounds__(256) void group_emit_kernel(const uint32_t* __restrict__ idx,
                                                         const float* __restrict__ w,
                                                         uint32_t n_pairs, uint32_t K, uint32_t E,
                                                         uint32_t chunk_pairs,
                                                         const uint32_t* __restrict__ chunk_base,
                                                         const uint32_t* __restrict__ starts,
                                                         mf_pair* __restrict__ sorted) {
  __shared__ uint32_t s_base[MF_MAX_EXPERTS];      // next free position of every expert's run
  __shared__ uint32_t s_wave[4][MF_MAX_EXPERTS];   // routes per expert of each wave in this step
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  for (uint32_t e = threadIdx.x; e < E; e += blockDim.x) {
    s_base[e] = starts[e] + chunk_base[blockIdx.x * E + e];
    s_wave[0][e] = s_wave[1][e] = s_wave[2][e] = s_wave[3][e] = 0;
  }
  __syncthreads();
  const uint32_t p0 = blockIdx.x * chunk_pairs, p1 = min(n_pairs, p0 + chunk_pairs);
  for (uint32_t q0 = p0; q0 < p1; q0 += kGroupBlock) {
    const uint32_t p = q0 + threadIdx.x;
    const bool valid = p < p1;
    const uint32_t e = valid ? idx[p] : 0xFFFFFFFFu;
    // rank of this route among the routes of its expert in this wave, in pair order
    bool open = valid && e < E;
    uint32_t rank = 0;
    unsigned long long todo = __ballot(open);
    while (todo) {
      const int leader = __ffsll(static_cast<long long>(todo)) - 1;
      const uint32_t e0 = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(e), leader));
      const unsigned long long same = __ballot(open && e == e0);
      if (open && e == e0) {
        rank = __popcll(same & ((1ull << lane) - 1ull));
        open = false;
      }
      if (lane == static_cast<uint32_t>(leader)) s_wave[wv][e0] = __popcll(same);
      todo &= ~same;
    }
    __syncthreads();
    if (valid && e < E) {
      uint32_t pos = s_base[e] + rank;
      for (uint32_t v = 0; v < wv; ++v) pos += s_wave[v][e];
      mf_pair r;
      r.token = p / K;
      r.expert = e;
      r.rank = p % K;
      r.weight_bits = __float_as_uint(w[p]);
      sorted[pos] = r;
    }
    __syncthreads();
    if (q0 + kGroupBlock < p1) {  // another step follows: advance the bases, clear the wave counts
      for (uint32_t x = threadIdx.x; x < E; x += blockDim.x) {
        s_base[x] += s_wave[0][x] + s_wave[1][x] + s_wave[2][x] + s_wave[3][x];
        s_wave[0][x] = s_wave[1][x] = s_wave[2][x] = s_wave[3][x] = 0;
      }
      __syncthreads();
    }
  }
}

// The stable counting sort by ballots, in one workgroup of 16 waves: each wave is a "chunk" (a contiguous
// run of the pair list) with its per-expert counts in LDS (s_hist: [16][MF_MAX_EXPERTS]).
__device__ __forceinline__ void group_serial(const uint32_t* __restrict__ idx, const float* __restrict__ w,
                                             uint32_t n_pairs, uint32_t K, uint32_t E,
                                             uint32_t* __restrict__ counts, uint32_t* __restrict__ offsets,
                                             uint32_t* __restrict__ starts, mf_pair* __restrict__ sorted,
                                             Tile* __restrict__ tiles, uint32_t tile_slots,
                                             uint32_t* __restrict__ n_tiles, uint32_t* s_hist_flat,
                                             uint32_t* s_cnt, uint32_t* s_tile) {
  uint32_t (*s_hist)[MF_MAX_EXPERTS] = reinterpret_cast<uint32_t (*)[MF_MAX_EXPERTS]>(s_hist_flat);
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < 16 * MF_MAX_EXPERTS; i += blockDim.x) s_hist_flat[i] = 0;
  __syncthreads();
  const uint32_t chunk = ((n_pairs + 15) / 16 + 63) / 64 * 64;
  const uint32_t p0 = min(n_pairs, wv * chunk), p1 = min(n_pairs, p0 + chunk);
  for (uint32_t p = p0 + lane; p < p1; p += 64) {
    const uint32_t e = idx[p];
    if (e < E) atomicAdd(&s_hist[wv][e], 1u);
  }
  __syncthreads();
  uint32_t c = 0;
  if (threadIdx.x < E) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const uint32_t n = s_hist[v][threadIdx.x];
      s_hist[v][threadIdx.x] = c;
      c += n;
    }
  }
  group_layout(c, E, counts, offsets, starts, tiles, tile_slots, n_tiles, s_cnt, s_tile);
  __syncthreads();
  // s_cnt holds the inclusive scan: an expert's run starts at s_cnt[e - 1]; the waves' bases are
  // relative to that start
  for (uint32_t q0 = p0; q0 < p1; q0 += 64) {
    const uint32_t p = q0 + lane;
    const bool valid = p < p1;
    const uint32_t e = valid ? idx[p] : 0xFFFFFFFFu;
    bool open = valid && e < E;
    const bool mine = open;
    uint32_t pos = 0;
    unsigned long long todo = __ballot(open);
    while (todo) {  // rank of this route among the routes of its expert in this step, in pair order
      const int leader = __ffsll(static_cast<long long>(todo)) - 1;
      const uint32_t e0 = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(e), leader));
      const unsigned long long same = __ballot(open && e == e0);
      const uint32_t base = s_hist[wv][e0];
      if (open && e == e0) {
        pos = base + __popcll(same & ((1ull << lane) - 1ull));
        open = false;
      }
      if (lane == static_cast<uint32_t>(leader)) s_hist[wv][e0] = base + __popcll(same);
      todo &= ~same;
    }
    if (mine) {
      const uint32_t run = (e ? s_cnt[e - 1] : 0u);
      mf_pair r;
      r.token = p / K;
      r.expert = e;
      r.rank = p % K;
      r.weight_bits = __float_as_uint(w[p]);
      sorted[run + pos] = r;
    }
  }
}

// The three steps above in one workgroup, for token counts whose (expert x token) bit matrix fits LDS.
// A token names an expert at most once (a top-k does), so "the routes of expert e in token order" is row
// e of that matrix: a route's place in its expert's run is the number of set bits before its token's, i.e.
// a per-word prefix count plus a popcount -- no serial ranking at all.  Every thread marks its routes
// (LDS atomic OR), the rows are prefix-counted (several threads per row), the expert counts go through the
// same layout step as the three-launch form, and every thread places its routes.  Input that does name
// an expert twice in one token (legal for the reference's grouping, never produced by a router) is
// noticed when the bit is already set; the workgroup then does the stable ranking the slow way (each of
// its 16 waves a chunk of the pair list, ballots per step) -- same result, same launch.
constexpr uint32_t kGroupOnePairs = 8192;  // beyond this the pair list is worth several workgroups (T=2048, K=8: 31 us in one, 20 us in three launches)
constexpr uint32_t kGroupOneMaxBytes = 112 * 1024;  // bit matrix + prefix counts the single workgroup may hold

__host__ __device__ __forceinline__ uint32_t group_one_row_words(uint32_t t) { return ((t + 31) / 32) | 1u; }  // odd: rows fall on different banks
__host__ __device__ __forceinline__ size_t group_one_lds_bytes(uint32_t t, uint32_t E) {
  const size_t bits = static_cast<size_t>(E) * group_one_row_words(t) * 6;  // u32 words + u16 prefix counts
  const size_t serial = 16 * MF_MAX_EXPERTS * 4;                            // the slow path's per-wave counts
  return (bits > serial ? bits : serial) + 16;
}

__global__ __launch_bounds__(1024) void group_one_kernel(const uint32_t* __restrict__ idx,
                                                         const float* __restrict__ w, uint32_t n_pairs,
                                                         uint32_t K, uint32_t E, uint32_t tpe_log2,
                                                         uint32_t* __restrict__ counts,
                                                         uint32_t* __restrict__ offsets,
                                                         uint32_t* __restrict__ starts,
                                                         mf_pair* __restrict__ sorted, Tile* __restrict__ tiles,
                                                         uint32_t tile_slots, uint32_t* __restrict__ n_tiles,
                                                         uint32_t* __restrict__ status) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  __shared__ uint32_t s_cnt[MF_MAX_EXPERTS], s_tile[MF_MAX_EXPERTS];
  const uint32_t T = n_pairs / K, W = group_one_row_words(T);
  uint32_t* bm = reinterpret_cast<uint32_t*>(smem);                 // [E][W] bits: token t of row e
  uint16_t* pref = reinterpret_cast<uint16_t*>(smem + static_cast<size_t>(E) * W * 4);  // [E][W] set bits before word
  // a thread's routes (at most kGroupOnePairs / 1024 = 8) stay in registers from the marking pass to the
  // placing pass: one round trip to memory instead of two
  constexpr uint32_t kMine = kGroupOnePairs / 1024;
  static_assert(kGroupOnePairs % 1024 == 0, "the launch has 1024 threads");
  uint32_t my_e[kMine], my_w[kMine];
#pragma unroll
  for (uint32_t u = 0; u < kMine; ++u) {
    const uint32_t p = threadIdx.x + u * 1024;
    my_e[u] = p < n_pairs ? idx[p] : 0xFFFFFFFFu;
    my_w[u] = p < n_pairs ? __float_as_uint(w[p]) : 0u;
  }
  for (uint32_t i = threadIdx.x; i < E * W; i += blockDim.x) bm[i] = 0;
  __syncthreads();
  bool bad = false, dup = false;
#pragma unroll
  for (uint32_t u = 0; u < kMine; ++u) {
    const uint32_t p = threadIdx.x + u * 1024;
    if (p >= n_pairs) break;
    const uint32_t e = my_e[u], t = p / K;
    if (e < E) {
      const uint32_t bit = 1u << (t & 31u);
      dup |= (atomicOr(&bm[e * W + (t >> 5)], bit) & bit) != 0u;
    } else {
      bad = true;
    }
  }
  const int any_bad = __syncthreads_or(bad ? 1 : 0);
  const int any_dup = __syncthreads_or(dup ? 1 : 0);
  if (threadIdx.x == 0) *status = any_bad ? 2u : 0u;
  if (any_dup) {
    group_serial(idx, w, n_pairs, K, E, counts, offsets, starts, sorted, tiles, tile_slots, n_tiles,
                 reinterpret_cast<uint32_t*>(smem), s_cnt, s_tile);
    return;
  }
  // prefix counts of every row: 2^tpe_log2 threads per row, each a run of words
  const uint32_t tpe = 1u << tpe_log2, row = threadIdx.x >> tpe_log2, part = threadIdx.x & (tpe - 1u);
  const uint32_t per = (W + tpe - 1) / tpe, w0 = min(W, part * per), w1 = min(W, w0 + per);
  uint32_t mine = 0;
  if (row < E)
    for (uint32_t j = w0; j < w1; ++j) mine += __popc(bm[row * W + j]);
  // exclusive scan of `mine` over the row's threads (they are neighbours in one wave: tpe <= 16)
  uint32_t before = 0, total = mine;
  for (uint32_t o = 1; o < tpe; o <<= 1) {
    const uint32_t v = static_cast<uint32_t>(__shfl_up(static_cast<int>(total), o, 64));
    if (part >= o) total += v;
  }
  before = total - mine;
  const uint32_t row_total = static_cast<uint32_t>(__shfl(static_cast<int>(total), (threadIdx.x & 63u) | (tpe - 1u), 64));
  if (row < E) {
    uint32_t c = before;
    for (uint32_t j = w0; j < w1; ++j) {
      pref[row * W + j] = static_cast<uint16_t>(c);
      c += __popc(bm[row * W + j]);
    }
    if (part == 0) s_tile[row] = row_total;  // parked for the layout step below
  }
  __syncthreads();
  const uint32_t c = threadIdx.x < E ? s_tile[threadIdx.x] : 0u;
  __syncthreads();
  group_layout(c, E, counts, offsets, starts, tiles, tile_slots, n_tiles, s_cnt, s_tile);
  __syncthreads();
#pragma unroll
  for (uint32_t u = 0; u < kMine; ++u) {
    const uint32_t p = threadIdx.x + u * 1024, e = my_e[u];
    if (p >= n_pairs || e >= E) continue;
    const uint32_t t = p / K, at = e * W + (t >> 5);
    const uint32_t pos = (e ? s_cnt[e - 1] : 0u) + pref[at] + __popc(bm[at] & ((1u << (t & 31u)) - 1u));
    mf_pair r;
    r.token = t;
    r.expert = e;
    r.rank = p - t * K;
    r.weight_bits = my_w[u];
    sorted[pos] = r;
  }
}

// The layer call selects the routes itself, so selection and grouping share launches: two instead of the
// selector's one plus the grouping's one or three.  A top-k names an expert at most once per token, so the
// routes of expert e inside a chunk of up to 64 consecutive tokens are a 64-bit word (bit i: token i of
// the chunk routes to e) and "how many routes of e come before mine" is a popcount.
//
// First launch: a workgroup selects the routes of one chunk (a wave a token at a time, the selectors of
// topk_kernel), stores them, and leaves the chunk's word per expert and, as a row of bytes, its number of
// routes per expert.
constexpr uint32_t kSelectWaves = 16;
constexpr uint32_t kChunkTokensMax = 64;
static_assert(kChunkTokensMax * MF_MAX_TOPK <= MF_MAX_EXPERTS, "a chunk's routes are placed by one workgroup in one step");

__global__ __launch_bounds__(kSelectWaves * 64) void topk_chunk_kernel(const float* __restrict__ logits, uint32_t T,
                                                                       uint32_t E, uint32_t K, int mode,
                                                                       uint32_t chunk_tokens,
                                                                       uint32_t* __restrict__ idx,
                                                                       float* __restrict__ w,
                                                                       unsigned long long* __restrict__ chunk_bits,
                                                                       uint8_t* __restrict__ chunk_cnt,
                                                                       uint32_t* __restrict__ chunk_bad) {
  __shared__ uint32_t s_bits[2][MF_MAX_EXPERTS];
  __shared__ float s_p[kSelectWaves][MF_MAX_EXPERTS];  // the full softmax's probabilities, a row per wave
  __shared__ uint32_t s_i[kSelectWaves][MF_MAX_TOPK];
  __shared__ float s_wt[kSelectWaves][MF_MAX_TOPK];
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  for (uint32_t e = threadIdx.x; e < E; e += blockDim.x) s_bits[0][e] = s_bits[1][e] = 0u;
  __syncthreads();
  const uint32_t t0 = blockIdx.x * chunk_tokens, t1 = min(T, t0 + chunk_tokens);
  bool bad = false;
  for (uint32_t t = t0 + wv; t < t1; t += kSelectWaves) {
    const float* lg = logits + static_cast<size_t>(t) * E;
    if (mode == 0) topk_select_fast(lg, E, K, s_i[wv], s_wt[wv], lane);
    else topk_full_softmax_fast(lg, s_p[wv], E, K, s_i[wv], s_wt[wv], lane);
    if (lane < K) {
      const uint32_t e = s_i[wv][lane];
      idx[static_cast<size_t>(t) * K + lane] = e;
      w[static_cast<size_t>(t) * K + lane] = s_wt[wv][lane];
      const uint32_t i = t - t0;
      if (e < E) atomicOr(&s_bits[i >> 5][e], 1u << (i & 31u));
      else bad = true;  // the full softmax's "routes nowhere"
    }
  }
  // one flag per chunk, always written: nothing has to be cleared before the launch
  const int any_bad = __syncthreads_or(bad ? 1 : 0);
  if (threadIdx.x == 0) chunk_bad[blockIdx.x] = any_bad ? 1u : 0u;
  for (uint32_t e = threadIdx.x; e < E; e += blockDim.x) {
    const uint32_t lo = s_bits[0][e], hi = s_bits[1][e];
    chunk_bits[static_cast<size_t>(blockIdx.x) * E + e] =
        static_cast<unsigned long long>(lo) | (static_cast<unsigned long long>(hi) << 32);
    chunk_cnt[static_cast<size_t>(blockIdx.x) * E + e] = static_cast<uint8_t>(__popc(lo) + __popc(hi));
  }
}

// Second launch: every workgroup adds up the chunks' counts per expert (an expert's total, and its routes
// in the chunks before the workgroup's own), repeats the layout scans for itself, and places the routes of
// its chunk; the first workgroup also publishes counts, offsets, starts, the tile list and the status word.
__global__ __launch_bounds__(MF_MAX_EXPERTS) void group_place_kernel(const uint32_t* __restrict__ idx,
                                                                    const float* __restrict__ w, uint32_t T,
                                                                    uint32_t K, uint32_t E, uint32_t chunk_tokens,
                                                                    uint32_t n_chunks,
                                                                    const unsigned long long* __restrict__ chunk_bits,
                                                                    const uint8_t* __restrict__ chunk_cnt,
                                                                    const uint32_t* __restrict__ chunk_bad,
                                                                    uint32_t* __restrict__ counts,
                                                                    uint32_t* __restrict__ offsets,
                                                                    uint32_t* __restrict__ starts,
                                                                    mf_pair* __restrict__ sorted,
                                                                    Tile* __restrict__ tiles, uint32_t tile_slots,
                                                                    uint32_t* __restrict__ n_tiles,
                                                                    uint32_t* __restrict__ status) {
  __shared__ uint32_t s_cnt[MF_MAX_EXPERTS], s_tile[MF_MAX_EXPERTS], s_base[MF_MAX_EXPERTS];
  __shared__ unsigned long long s_mine[MF_MAX_EXPERTS];
  const uint32_t e = threadIdx.x, me = blockIdx.x;
  const bool first = me == 0;
  // this workgroup's routes, requested before anything is waited for
  const uint32_t t0 = me * chunk_tokens, t1 = min(T, t0 + chunk_tokens);
  const uint32_t n = (t1 - t0) * K;  // <= kChunkTokensMax * MF_MAX_TOPK <= blockDim
  const size_t p = static_cast<size_t>(t0) * K + threadIdx.x;
  uint32_t ex = 0xFFFFFFFFu, wbits = 0u;
  if (threadIdx.x < n) {
    ex = idx[p];
    wbits = __float_as_uint(w[p]);
  }
  uint32_t c = 0, before = 0;
  if (e < E) {
    s_mine[e] = chunk_bits[static_cast<size_t>(me) * E + e];
    uint32_t k = 0;
    for (; k + 32 <= n_chunks; k += 32) {  // 32 independent byte loads in flight
      uint32_t v[32];
#pragma unroll
      for (int u = 0; u < 32; ++u) v[u] = chunk_cnt[static_cast<size_t>(k + u) * E + e];
#pragma unroll
      for (int u = 0; u < 32; ++u) {
        c += v[u];
        before += k + u < me ? v[u] : 0u;
      }
    }
    for (; k < n_chunks; ++k) {
      const uint32_t v = chunk_cnt[static_cast<size_t>(k) * E + e];
      c += v;
      before += k < me ? v : 0u;
    }
  }
  const int any_bad = __syncthreads_or(e < n_chunks && chunk_bad[e] ? 1 : 0);  // n_chunks <= blockDim
  if (first && e == 0) *status = any_bad ? 2u : 0u;
  group_layout(c, E, counts, offsets, starts, tiles, tile_slots, n_tiles, s_cnt, s_tile, first);
  if (e < E) s_base[e] = s_cnt[e] - c + before;  // s_cnt is the inclusive scan of the counts
  __syncthreads();
  if (ex < E) {
    const uint32_t i = threadIdx.x / K;
    mf_pair r;
    r.token = t0 + i;
    r.expert = ex;
    r.rank = threadIdx.x - i * K;
    r.weight_bits = wbits;
    sorted[s_base[ex] + __popcll(s_mine[ex] & ((1ull << i) - 1ull))] = r;
  }
}

// ---- the expert pool in the matmul's order
// A lane of the matmul reads half a K group of ONE weight row per load (16 bytes of 4-bit codes, 8 of 2-bit):
// row by row that is 32 rows, 32 memory lines, per load instruction, and the L1's line rate is a large part
// of what a work item costs (Qwen shape, 2048 tokens: layer 273 -> 255 us with the loads below).  In the
// tiled pool every sub-tensor keeps its place in the blob and its size; inside it, the pieces of the 32 rows
// of a block for one K group sit side by side in lane order: piece (row block rb, group g, lane l = m + 32 h)
// = row 32 rb + m, bytes [g * GB + h * GB / 2, + GB / 2) of the row, GB = 32 (4-bit) or 16 (2-bit, ternary)
// bytes per group.  A load instruction then reads 1 KB (512 B) of consecutive bytes.  Scale and bias tables
// stay row by row.  One thread per piece; sub-tensor w of every expert in one launch.
__global__ __launch_bounds__(256) void tile_codes_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                         size_t expert_stride, uint32_t w_off, uint32_t rows,
                                                         uint32_t ng, uint32_t group_bytes) {
  const uint32_t half = group_bytes / 2;
  const uint64_t pieces = static_cast<uint64_t>(rows) * ng * 2;
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= pieces) return;
  const uint32_t l = static_cast<uint32_t>(i & 63u), m = l & 31u, h = l >> 5;
  const uint64_t bg = i >> 6;  // rb * ng + g
  const uint32_t g = static_cast<uint32_t>(bg % ng), rb = static_cast<uint32_t>(bg / ng);
  const size_t base = static_cast<size_t>(blockIdx.y) * expert_stride + w_off;
  const uint8_t* from = src + base + (static_cast<size_t>(32u * rb + m) * ng + g) * group_bytes + h * half;
  uint8_t* to = dst + base + i * half;
  if (half == 16) *reinterpret_cast<uint4*>(to) = *reinterpret_cast<const uint4*>(from);
  else *reinterpret_cast<uint2*>(to) = *reinterpret_cast<const uint2*>(from);
}

// dst = the pool `src` (E blobs, expert_stride apart) with the three code sub-tensors of every blob tiled
hipError_t launch_tile_experts(hipStream_t s, const mf_moe_config& c, const void* src, size_t expert_stride,
                               const mf_expert_offsets& off, void* dst) {
  hipError_t e = hipMemcpyAsync(dst, src, expert_stride * c.num_experts, hipMemcpyDeviceToDevice, s);
  if (e != hipSuccess) return e;
  const uint32_t gb = c.bits == MF_BITS_4 ? 32u : 16u;
  const struct { uint32_t off, rows, k; } parts[3] = {{off.gate_w, c.f, c.d}, {off.up_w, c.f, c.d}, {off.down_w, c.d, c.f}};
  for (const auto& p : parts) {
    const uint64_t pieces = static_cast<uint64_t>(p.rows) * (p.k / kGroup) * 2;
    tile_codes_kernel<<<dim3(static_cast<uint32_t>((pieces + 255) / 256), c.num_experts), dim3(256), 0, s>>>(
        static_cast<const uint8_t*>(src), static_cast<uint8_t*>(dst), expert_stride, p.off, p.rows, p.k / kGroup, gb);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

// --------------------------------------------------------------- the matmul

// Activation rows as the matmul wants them: inside every run of 8 K values the
// order is (0,4,1,5,2,6,3,7) -- the pairing a packed code word expands to --
// and the fp32 sum of every 64-wide K group is kept beside them.  One lane per
// run of 8; `dst` may be null when `src` is already in that order.
struct PrepArgs {  // up to two row sets per launch: the second starts at workgroup `blocks0`
  const uint16_t* src[2];
  uint16_t* dst[2];
  float* sums[2];
  uint32_t chunks[2];
  uint32_t blocks0;
};

__global__ __launch_bounds__(256) void prep_rows_kernel(const PrepArgs a) {
  const int part = blockIdx.x >= a.blocks0 ? 1 : 0;
  const uint16_t* src = a.src[part];
  uint16_t* dst = a.dst[part];
  float* sums = a.sums[part];
  const uint32_t chunks = a.chunks[part];
  const uint32_t c = (blockIdx.x - (part ? a.blocks0 : 0u)) * blockDim.x + threadIdx.x;
  uint4 v = make_uint4(0, 0, 0, 0);
  if (c < chunks) v = *reinterpret_cast<const uint4*>(src + static_cast<size_t>(c) * 8);
  float sum = ((bf16_lo(v.x) + bf16_hi(v.x)) + (bf16_lo(v.y) + bf16_hi(v.y))) +
              ((bf16_lo(v.z) + bf16_hi(v.z)) + (bf16_lo(v.w) + bf16_hi(v.w)));
  sum = group_sum(sum, 8);
  if (c >= chunks) return;
  if (dst)
    *reinterpret_cast<uint4*>(dst + static_cast<size_t>(c) * 8) =
        make_uint4(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u), __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                   __builtin_amdgcn_perm(v.w, v.y, 0x05040100u), __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));
  if ((c & 7) == 0) sums[c >> 3] = sum;
}

// The same for the layer's input rows and, in the same pass, the scalar shared gate's logit
// w_sg . x of every row (prefill_qwen_shared_scalar_gate, prefill.metal:42-80) in the router's lane
// order (dot_bf16_row: lane l takes the chunks l, l+64, ... of a row, neighbour-first butterfly), so
// the gate has the bits of the stand-alone router-row launch it replaces.  One wave per row.
__device__ __forceinline__ void prep_x_row(const uint16_t* __restrict__ xr, uint16_t* __restrict__ xp,
                                           float* __restrict__ sums, const uint16_t* __restrict__ w_sg,
                                           uint16_t* __restrict__ gate, uint32_t row, uint32_t d, uint32_t lane) {
  const uint32_t chunks = d / 8;  // a multiple of 8: the 8 lanes of a K group are live together
  const size_t base = static_cast<size_t>(row) * chunks;
  float acc = 0.0f;
  for (uint32_t c0 = 0; c0 < chunks; c0 += kWave) {
    const uint32_t c = c0 + lane;
    const bool live = c < chunks;
    uint4 v = make_uint4(0, 0, 0, 0), wv = make_uint4(0, 0, 0, 0);
    if (live) {
      v = *reinterpret_cast<const uint4*>(xr + static_cast<size_t>(c) * 8);
      if (w_sg) wv = *reinterpret_cast<const uint4*>(w_sg + static_cast<size_t>(c) * 8);
    }
    float sum = ((bf16_lo(v.x) + bf16_hi(v.x)) + (bf16_lo(v.y) + bf16_hi(v.y))) +
                ((bf16_lo(v.z) + bf16_hi(v.z)) + (bf16_lo(v.w) + bf16_hi(v.w)));
    sum = group_sum(sum, 8);
    if (live) {
      *reinterpret_cast<uint4*>(xp + (base + c) * 8) =
          make_uint4(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u), __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                     __builtin_amdgcn_perm(v.w, v.y, 0x05040100u), __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));
      if ((c & 7) == 0) sums[(base + c) >> 3] = sum;
      acc = __builtin_fmaf(bf16_lo(wv.x), bf16_lo(v.x), acc);
      acc = __builtin_fmaf(bf16_hi(wv.x), bf16_hi(v.x), acc);
      acc = __builtin_fmaf(bf16_lo(wv.y), bf16_lo(v.y), acc);
      acc = __builtin_fmaf(bf16_hi(wv.y), bf16_hi(v.y), acc);
      acc = __builtin_fmaf(bf16_lo(wv.z), bf16_lo(v.z), acc);
      acc = __builtin_fmaf(bf16_hi(wv.z), bf16_hi(v.z), acc);
      acc = __builtin_fmaf(bf16_lo(wv.w), bf16_lo(v.w), acc);
      acc = __builtin_fmaf(bf16_hi(wv.w), bf16_hi(v.w), acc);
    }
  }
  acc = wave_sum(acc);
  if (w_sg && lane == 0) gate[row] = f_to_bf16(acc);
}

__global__ __launch_bounds__(256) void prep_x_gate_kernel(const uint16_t* __restrict__ x,
                                                          uint16_t* __restrict__ xp, float* __restrict__ sums,
                                                          const uint16_t* __restrict__ w_sg,
                                                          uint16_t* __restrict__ gate, uint32_t t, uint32_t d) {
  const uint32_t lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= t) return;
  prep_x_row(x + static_cast<size_t>(row) * d, xp, sums, w_sg, gate, row, d, lane);
}

struct QmmArgs {
  // weights: routed = blobs of the expert pool, dense = one projection set
  const uint8_t* expert_base;
  size_t expert_stride;
  uint32_t w_off[2], s_off[2], b_off[2];
  mf_qtensor dense[2];
  int pair_rows;        // 1: the NPROJ blocks of a wave are consecutive 32-row blocks of projection 0
  int tiled;            // 1: the routed experts' codes are in the matmul's own order (tile_codes_kernel), not row by row
  int dense_mode;       // 1: the "expert" is dense[], tiles are runs of consecutive rows
  uint32_t dense_rows;  // number of x rows in dense mode
  // activations: rows of kdim bf16 in prep_rows_kernel order + their group sums [row, kdim/64]
  const uint16_t* x;
  const float* sumx;
  uint32_t x_stride;
  int gather;           // 1: x row = sorted[pair].token, 0: x row = pair index
  const mf_pair* sorted;
  const Tile* tiles;
  const uint32_t* n_tiles;
  uint32_t rows, kdim;  // weight rows (output width) and contraction length
  // a launch may take a window of the contraction (long K is cut into windows whose fp32 results are
  // added afterwards): rows of weights, tables and group sums are ng_ld groups apart (0: kdim / 64)
  // and the window starts at group g_off (a multiple of 8)
  uint32_t ng_ld, g_off;
  // several windows in one launch (dense mode): window w covers the groups from
  // dense_window_start(ng_ld, n_win, w) on and writes its fp32 result out_win_stride elements behind the
  // previous window's
  uint32_t n_win;
  size_t out_win_stride;
  // epilogue
  int epi;              // 0 swiglu -> bf16 [pair, rows] in prep order; 1 fp32 [token*K+rank, rows]; 2 bf16 [pair, rows];
                        // 3 bf16 [token*K+rank, rows]
  int narrow;           // shared-expert rounding points (dequant_int4.metal:240-245)
  int tab_aligned;      // scale / bias rows start on 16-byte boundaries (set by the launcher)
  int ternary;          // 2-bit codes {0,1,2} with bias = -scale: b_off / dense[].biases name the SCALE table
  int maple;            // MapleMoE's bf16-stepped activation in the SwiGLU epilogue
  void* out;
  void* out2;           // epi 1 / 2 with two projections that are not row blocks of one: where projection 1 goes (null: dropped)
  uint32_t top_k;
  float limit;
  // dense mode: number of 64-row tiles and of work items; every XCD gets an eighth of the items however few
  // tiles there are.  With few tiles (tile_major = 0: x is small, the weights are not) work item w is tile
  // w % dense_tiles of row slice (w / dense_tiles) % slices: the items that read the same weight rows follow
  // one another (same XCD, same moment).  With many tiles (tile_major = 1) the slices of one tile follow one
  // another and an XCD's L2 holds the x rows of the few tiles it works on.  The window is w / (tiles * slices).
  uint32_t dense_tiles, dense_items;
  int tile_major;
  // optional stage stamps: 8 per work item, 100 MHz clock
  unsigned long long* trace;
  uint32_t trace_items;
};

// first K group of window wdx when ng groups are cut into n_win windows (multiples of 8 groups)
__host__ __device__ __forceinline__ uint32_t dense_window_start(uint32_t ng, uint32_t n_win, uint32_t wdx) {
  if (wdx >= n_win) return ng;
  return static_cast<uint32_t>(static_cast<uint64_t>(ng) * wdx / n_win) & ~7u;
}

__device__ __forceinline__ void qmm_trace(const QmmArgs& a, uint32_t work, uint32_t k) {
  if (a.trace && threadIdx.x == 0 && work < a.trace_items) a.trace[work * 8 + k] = wall_clock64();
}

// silu with the hardware exp2 / reciprocal (1 ulp each): the result is narrowed to bf16 right after
__device__ __forceinline__ float fast_silu(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

// One workgroup: 64 routes of one expert x 128 weight rows (4 waves x 32) x
// NPROJ projections, the whole K.  The matrix core computes the TRANSPOSED
// product: the A operand is the x tile (tokens are the rows), the B operand is
// the expanded codes, so a lane ends up holding ONE weight row (its column
// m = lane % 32) for 16 tokens of each 32-token block, and the per-group scale
// is one scalar per lane.  With two row blocks per wave two waves per SIMD stay
// resident (the register budget of 256 keeps the matrix-core results in ordinary
// registers, where the scale multiply reads them directly); with one row block the
// kernel fits 168 registers and three waves stay resident.
// LDS (dynamic): x tile ring, 2 stages x 2 K groups x [2 nt][4 s][2 h][32 n] x 16 B,
// scale tables [NPROJ][4 waves][ng][32 rows] fp32, out slots [64] u32.
// One launch can carry two independent problems of the same instantiation (the routed experts
// and the shared expert of the same phase): the second problem's work items follow the first's
// on every XCD, so they fill the slots the first problem's last round leaves empty instead of
// running as a launch of their own that covers a quarter of the chip.
struct QmmLaunch {
  QmmArgs part[2];
  uint32_t per_xcd[2];  // work items of each part on one XCD (grid = 8 * their sum)
};

template <int BITS, int NPROJ, bool NG8, bool TAB16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(NPROJ == 1 ? 3 : 2, NPROJ == 1 ? 3 : 2)))
void qmm_kernel(const QmmLaunch launch) {
  constexpr uint32_t kGB = QmmCodes<BITS>::kGroupBytes;  // bytes of one K group of one weight row
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const uint32_t m = lane & 31, h = lane >> 5;
  // Workgroups go to the 8 XCDs round-robin by blockIdx; consecutive work items (the row slices of
  // one tile share its x rows, the tiles of one expert share its weights) are laid on ONE XCD so
  // that its L2 serves the re-reads.  The tile list is laid out by group_scan_kernel so that every
  // eighth of it holds an eighth of the live tiles.
  const uint32_t xcd_slot = blockIdx.x >> 3;
  const bool second = xcd_slot >= launch.per_xcd[0];
  const QmmArgs& a = launch.part[second ? 1 : 0];
  const uint32_t work = (blockIdx.x & 7u) * launch.per_xcd[second ? 1 : 0] + (xcd_slot - (second ? launch.per_xcd[0] : 0u));
  const uint32_t wave_rows = a.pair_rows ? 32u * NPROJ : 32u;  // weight rows of one wave
  const uint32_t n_slices = a.rows / (kQmmWaves * wave_rows);
  uint32_t tile_id = work / n_slices, slice = work % n_slices, win = 0;
  if (a.dense_mode) {
    if (work >= a.dense_items) return;
    const uint32_t inner = a.tile_major ? n_slices : a.dense_tiles, outer = a.tile_major ? a.dense_tiles : n_slices;
    const uint32_t lo = work % inner, rest = work / inner, hi = rest % outer;
    tile_id = a.tile_major ? hi : lo;
    slice = a.tile_major ? lo : hi;
    win = rest / outer;
    if (tile_id >= a.dense_tiles) return;
  }
  uint32_t ng = a.kdim / kGroup, g_off = a.g_off;
  uint8_t* out_base = static_cast<uint8_t*>(a.out);
  uint8_t* out2_base = static_cast<uint8_t*>(a.out2);
  if (a.n_win > 1) {  // this work item's window of the contraction
    g_off = dense_window_start(a.ng_ld, a.n_win, win);
    ng = dense_window_start(a.ng_ld, a.n_win, win + 1) - g_off;
    out_base += win * a.out_win_stride * sizeof(float);
    if (out2_base) out2_base += win * a.out_win_stride * sizeof(float);
  }
  qmm_trace(a, work, 0);

  uint32_t expert = 0, pair_start, count;
  if (a.dense_mode) {
    pair_start = tile_id * kTileTokens;
    count = min(kTileTokens, a.dense_rows - pair_start);
  } else {
    // (the whole 16-byte record in one load: read field by field, the count was fetched, tested, and the rest
    // fetched in a second round trip)
    const uint4 tv = *reinterpret_cast<const uint4*>(a.tiles + tile_id);
    const Tile t{tv.x, tv.y, tv.z, tv.w};
    if (t.count == 0) return;
    expert = t.expert;
    pair_start = t.pair_start;
    count = t.count;
  }

  uint4* s_x = reinterpret_cast<uint4*>(smem);                      // 2 stages x 2 groups x 512 uint4
  // The scale of every (row, group): fp32, or (TAB16, long contractions) a bf16 number -- 2 * scale for 4-bit
  // codes is one (exponent + 1), so the upper half of the fp32 product is all of it.  That is half the LDS,
  // which lets two workgroups share a CU up to 112 K groups (K = 7168), for one more instruction per read.
  using tab_t = std::conditional_t<TAB16, uint16_t, float>;
  tab_t* s_scale = reinterpret_cast<tab_t*>(smem + kQmmXBytes);  // [NPROJ][4][ng][32]
  uint32_t* s_slot = reinterpret_cast<uint32_t*>(smem + kQmmXBytes + ((NPROJ * kQmmWaves * ng * 32 * sizeof(tab_t) + 15) & ~15u));

  // weight pointers of this workgroup's projections
  const uint8_t* Wp[NPROJ];
  const uint16_t* Sp[NPROJ];
  const uint16_t* Bp[NPROJ];
  uint32_t row_base[NPROJ];  // first weight row of each of this wave's 32-row blocks
#pragma unroll
  for (int p = 0; p < NPROJ; ++p) {
    const int t = a.pair_rows ? 0 : p;
    if (a.dense_mode) {
      Wp[p] = static_cast<const uint8_t*>(a.dense[t].weights);
      Sp[p] = a.dense[t].scales;
      Bp[p] = a.dense[t].biases;
    } else {
      const uint8_t* blob = a.expert_base + static_cast<size_t>(expert) * a.expert_stride;
      Wp[p] = blob + a.w_off[t];
      Sp[p] = reinterpret_cast<const uint16_t*>(blob + a.s_off[t]);
      Bp[p] = reinterpret_cast<const uint16_t*>(blob + a.b_off[t]);
    }
    row_base[p] = (slice * kQmmWaves + wv) * wave_rows + (a.pair_rows ? 32u * p : 0u);
  }
  const uint32_t ng_ld = a.ng_ld ? a.ng_ld : ng;
  const size_t row_bytes = static_cast<size_t>(ng_ld) * kGB;

  // ---- everything the tile needs that depends only on the tile: issued back to back.
  // Routes past `count` read the tile's last route instead (finite data, results discarded).
  const uint32_t st_i = threadIdx.x >> 2, st_q = threadIdx.x & 3;  // staging: token i, K values 16q..16q+15
  const uint32_t st_pair = pair_start + min(st_i, count - 1);
  const uint32_t ti_pair[2] = {pair_start + min(m, count - 1), pair_start + min(32 + m, count - 1)};
  uint32_t st_row = st_pair, xrow[2] = {ti_pair[0], ti_pair[1]};
  uint32_t slot = pair_start + min(threadIdx.x & 63u, count - 1);
  // the routes' records are requested here and looked at behind the code loads below, which do not depend on
  // them: the first codes are then on their way one memory round trip earlier
  mf_pair pr{};
  uint32_t tok_st = 0, tok_0 = 0, tok_1 = 0;
  if (!a.dense_mode) {
    pr = a.sorted[slot];
    if (a.gather) {
      tok_st = a.sorted[st_pair].token;
      tok_0 = a.sorted[ti_pair[0]].token;
      tok_1 = a.sorted[ti_pair[1]].token;
    }
  }
  const uint8_t* wrow[NPROJ];
  const uint32_t gstride = a.tiled ? 32u * kGB : kGB;  // bytes from a group's codes to the next group's
  QmmCodes<BITS> cur[NPROJ][4];
#pragma unroll
  for (int p = 0; p < NPROJ; ++p) {
    // row by row: the lane's half group of its row, groups kGB apart.  Tiled: the 32 rows' pieces of a group are
    // one run of 64 x kGB / 2 bytes in lane order (one load instruction reads 1 KB of consecutive bytes)
    wrow[p] = a.tiled ? Wp[p] + row_base[p] * row_bytes + static_cast<size_t>(g_off) * gstride + lane * (kGB / 2)
                      : Wp[p] + (row_base[p] + m) * row_bytes + static_cast<size_t>(g_off) * gstride + h * (kGB / 2);
#pragma unroll
    for (int u = 0; u < 4; ++u) cur[p][u].load(wrow[p] + min(static_cast<uint32_t>(u), ng - 1) * gstride);
  }
  __builtin_amdgcn_sched_barrier(0);  // (keeps the look at the routes behind the code loads)
  if (!a.dense_mode) {
    if (a.gather) {
      st_row = tok_st;
      xrow[0] = tok_0;
      xrow[1] = tok_1;
    }
    if (a.epi == 1 || a.epi == 3) slot = pr.token * a.top_k + pr.rank;
  }
  // x rows of groups 0..2 and, for the bias terms, the group sums of the lane's two routes
  const uint16_t* st_src = a.x + static_cast<size_t>(st_row) * a.x_stride + static_cast<size_t>(g_off) * kGroup + st_q * 16;
  // K groups travel in pairs (ng is even: kdim is a multiple of 128)
  // (arrays of a native vector type: arrays of the uint4 struct were kept in scratch memory)
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  u32x4_t xs[2][2];  // the pair after the one in LDS, on its way there
  u32x4_t x0[2][2];
#pragma unroll
  for (int gi = 0; gi < 2; ++gi) {
    x0[gi][0] = *reinterpret_cast<const u32x4_t*>(st_src + gi * kGroup);
    x0[gi][1] = *reinterpret_cast<const u32x4_t*>(st_src + gi * kGroup + 8);
    xs[gi][0] = xs[gi][1] = u32x4_t{0, 0, 0, 0};
    if (NG8 || ng > 2) {
      xs[gi][0] = *reinterpret_cast<const u32x4_t*>(st_src + (2 + gi) * kGroup);
      xs[gi][1] = *reinterpret_cast<const u32x4_t*>(st_src + (2 + gi) * kGroup + 8);
    }
  }
  // Scale and bias words of the lane's row and the group sums of its two routes, 8 K groups at a time
  // (groups gl = g0 + 8h .. gl + 7 for g0 = 0, 16, ...); the loads of the first step leave now, with the
  // codes and the x rows, the loads of every later step one step ahead of their use.
  struct TabStep {
    uint4 S[NPROJ], B[NPROJ];
    float sx[2][8];
  };
  auto tab_fetch = [&](uint32_t g0) {
    TabStep t;
    const uint32_t gl = g0 + 8 * h;
    const uint32_t gc = gl < ng ? gl : 0;  // a lane without groups reads group 0 and drops it
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      const size_t at = static_cast<size_t>(row_base[p] + m) * ng_ld + g_off + gc;
      t.B[p] = NG8 ? (a.tab_aligned ? load_x8<true>(Bp[p] + at) : load_x8<false>(Bp[p] + at))
                   : load_bf16x8_guarded(Bp[p] + at, ng - gc);
      t.S[p] = NG8 ? (a.tab_aligned ? load_x8<true>(Sp[p] + at) : load_x8<false>(Sp[p] + at))
                   : load_bf16x8_guarded(Sp[p] + at, ng - gc);
    }
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const float* sp = a.sumx + static_cast<size_t>(xrow[nt]) * ng_ld + g_off + gc;
      if (NG8) {
        const float4 s0 = *reinterpret_cast<const float4*>(sp), s1 = *reinterpret_cast<const float4*>(sp + 4);
        t.sx[nt][0] = s0.x; t.sx[nt][1] = s0.y; t.sx[nt][2] = s0.z; t.sx[nt][3] = s0.w;
        t.sx[nt][4] = s1.x; t.sx[nt][5] = s1.y; t.sx[nt][6] = s1.z; t.sx[nt][7] = s1.w;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) t.sx[nt][e] = gc + e < ng ? sp[e] : 0.0f;
      }
    }
    return t;
  };
  TabStep tab_cur = tab_fetch(0);
  qmm_trace(a, work, 1);

  if (threadIdx.x < kTileTokens) s_slot[threadIdx.x] = threadIdx.x < count ? slot : 0xFFFFFFFFu;

  f32x16_t acc[NPROJ][2];
#pragma unroll
  for (int p = 0; p < NPROJ; ++p)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[p][nt][r] = 0.0f;

  // ---- per step: scale / code step (4-bit codes enter as 8 + q/2: 2 * scale; 2-bit codes as 4 + q: scale)
  // of the wave's rows into the [g][row] fp32 table, and the bias and offset terms:
  // acc[token, row] += sumx[token, g] * B[row, g] + sumx[token, g] * (-offset S[row, g]), offset 16 or 4.
  // -offset * S is formed in place (exponent + 4 or + 2, sign flipped: exact; a zero scale becomes 2^-123 / 2^-125).
  // sumx enters as three bf16 terms, which hold all 24 bits: the -offset * S * sumx term cancels the
  // offset * sum(x) the matrix core accumulated with the codes, so it has to be exact.
  // A tile of at most 32 routes fills only the first token block: the second block's matrix
  // instructions and scale multiplies are left out (NTA = 1); its accumulators stay zero and its
  // output slots are empty.
  auto tile_body = [&](auto nta_c) {
  constexpr int NTA = decltype(nta_c)::value;
  for (uint32_t g0 = 0; g0 < ng; g0 += 16) {
    const TabStep t = tab_cur;
    tab_cur = tab_fetch(g0 + 16 < ng ? g0 + 16 : g0);  // past the end: the same step again, unused
    const uint32_t gl = g0 + 8 * h;
    const bool have = gl < ng;
    uint4 ab[NPROJ], as[NPROJ];
#pragma unroll
    for (int p = 0; p < NPROJ; ++p) {
      tab_t* tab = s_scale + (p * kQmmWaves + wv) * ng * 32;
      auto entry = [](float v) -> tab_t {
        if constexpr (TAB16) return static_cast<uint16_t>(__float_as_uint(v) >> 16);
        else return v;
      };
      const uint32_t pr[4] = {t.S[p].x, t.S[p].y, t.S[p].z, t.S[p].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (have && (NG8 || gl + 2 * i < ng)) tab[(gl + 2 * i) * 32 + m] = entry(QmmCodes<BITS>::kScaleMul * bf16_lo(pr[i]));
        if (have && (NG8 || gl + 2 * i + 1 < ng)) tab[(gl + 2 * i + 1) * 32 + m] = entry(QmmCodes<BITS>::kScaleMul * bf16_hi(pr[i]));
      }
      constexpr uint32_t kAdd = QmmCodes<BITS>::kNegOffsetAdd;
      // ternary rows store no biases: the bias is -scale (the table pointer is the scale table then)
      ab[p] = a.ternary ? make_uint4(t.B[p].x ^ 0x80008000u, t.B[p].y ^ 0x80008000u, t.B[p].z ^ 0x80008000u,
                                     t.B[p].w ^ 0x80008000u)
                        : t.B[p];
      as[p] = make_uint4((t.S[p].x + kAdd) ^ 0x80008000u, (t.S[p].y + kAdd) ^ 0x80008000u,
                         (t.S[p].z + kAdd) ^ 0x80008000u, (t.S[p].w + kAdd) ^ 0x80008000u);
      if (!have) ab[p] = as[p] = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int nt = 0; nt < NTA; ++nt) {
      uint32_t hi[8], mid[8], lo[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float v = t.sx[nt][e];
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
        acc[p][nt] = mfma_bf16(b_hi, ab[p], acc[p][nt]);
        acc[p][nt] = mfma_bf16(b_hi, as[p], acc[p][nt]);
        acc[p][nt] = mfma_bf16(b_mid, ab[p], acc[p][nt]);
        acc[p][nt] = mfma_bf16(b_mid, as[p], acc[p][nt]);
        acc[p][nt] = mfma_bf16(b_lo, ab[p], acc[p][nt]);
        acc[p][nt] = mfma_bf16(b_lo, as[p], acc[p][nt]);
      }
    }
  }
  qmm_trace(a, work, 2);

  // run c = 2q (+1): K 8c..8c+7 -> slot (h = c / 4, s = c % 4)
  const uint32_t st_nt = st_i >> 5, st_n = st_i & 31, c0 = 2 * st_q, c1 = c0 + 1;
  // inside a 32-token block the column is rotated by 4 * ((s >> 1) + 2h): the four lanes that
  // stage one token then hit four different bank groups
  const uint32_t st_rot = 4 * ((c0 & 3) >> 1) + 8 * (c0 >> 2);
  const uint32_t st_slot0 = ((st_nt * 4 + (c0 & 3)) * 2 + (c0 >> 2)) * 32 + ((st_n + st_rot) & 31);
  const uint32_t st_slot1 = ((st_nt * 4 + (c1 & 3)) * 2 + (c1 >> 2)) * 32 + ((st_n + st_rot) & 31);
  uint32_t rd_col[4];
#pragma unroll
  for (int sidx = 0; sidx < 4; ++sidx) rd_col[sidx] = (m + 4 * (sidx >> 1) + 8 * h) & 31;
#pragma unroll
  for (int gi = 0; gi < 2; ++gi) {
    *reinterpret_cast<u32x4_t*>(s_x + gi * 512 + st_slot0) = x0[gi][0];
    *reinterpret_cast<u32x4_t*>(s_x + gi * 512 + st_slot1) = x0[gi][1];
  }

  // Weight codes run four K groups ahead in a ring of registers (the expert's bytes come
  // from HBM); x rows come from L2 in pairs of groups, one pair in registers behind
  // the pair in the LDS stage that is not being read.

  for (uint32_t g0 = 0; g0 < ng; g0 += 4) {
#pragma unroll
    for (int uu = 0; uu < 2; ++uu) {  // pair of K groups g0 + 2uu, g0 + 2uu + 1 in stage uu
      const uint32_t gu = g0 + 2 * uu;
      if (!NG8 && gu >= ng) break;
      __syncthreads();  // stage uu is complete, stage uu ^ 1 is no longer read
      // ---- the next pair into the other stage, fetch the pair after it into the freed registers.
      // With whole steps of 8 groups the body has no branch (past the end the last pair is fetched
      // again and the write goes to the stage nobody reads any more): every pass issues the same
      // loads in the same order, so a wait for the codes of this pass never covers the x rows
      // requested a moment before it.
      if (NG8 || gu + 2 < ng) {
        uint4* wbuf = s_x + (uu ^ 1) * 1024;
#pragma unroll
        for (int gi = 0; gi < 2; ++gi) {
          *reinterpret_cast<u32x4_t*>(wbuf + gi * 512 + st_slot0) = xs[gi][0];
          *reinterpret_cast<u32x4_t*>(wbuf + gi * 512 + st_slot1) = xs[gi][1];
        }
        if (NG8 || gu + 4 < ng) {
          const uint32_t gx = NG8 ? min(gu + 4, ng - 2) : gu + 4;
#pragma unroll
          for (int gi = 0; gi < 2; ++gi) {
            xs[gi][0] = *reinterpret_cast<const u32x4_t*>(st_src + (gx + gi) * kGroup);
            xs[gi][1] = *reinterpret_cast<const u32x4_t*>(st_src + (gx + gi) * kGroup + 8);
          }
        }
      }
#pragma unroll
      for (int gi = 0; gi < 2; ++gi) {
        const uint32_t g = gu + gi;
        // ---- matrix core: tmp[token, row] = sum over the group of x * (8 + q/2)
        const uint4* buf = s_x + uu * 1024 + gi * 512;
        uint4 bx[2][4];
#pragma unroll
        for (int nt = 0; nt < NTA; ++nt)
#pragma unroll
          for (int s = 0; s < 4; ++s) bx[nt][s] = buf[((nt * 4 + s) * 2 + h) * 32 + rd_col[s]];
#pragma unroll
        for (int p = 0; p < NPROJ; ++p) {
          float sc;
          if constexpr (TAB16) sc = bf16_to_f(s_scale[((p * kQmmWaves + wv) * ng + g) * 32 + m]);
          else sc = s_scale[((p * kQmmWaves + wv) * ng + g) * 32 + m];
          f32x16_t tmp[2];
#pragma unroll
          for (int nt = 0; nt < NTA; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) tmp[nt][r] = 0.0f;
          group_products<BITS, NTA>(cur[p][2 * uu + gi], bx, tmp, [](int) {});
          // the register that held this group's codes takes those of the group four ahead
          // (past the end the last group is read again: no branch inside the unrolled body)
          cur[p][2 * uu + gi].load(wrow[p] + min(g + 4, ng - 1) * gstride);
#pragma unroll
          for (int nt = 0; nt < NTA; ++nt)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[p][nt][r] = __builtin_fmaf(sc, tmp[nt][r], acc[p][nt][r]);
        }
      }
    }
  }
  };  // tile_body
  // (the one-projection form keeps to its budget of 168 registers, three waves per SIMD, with one body only)
  if (NPROJ == 1 || count > 32) tile_body(std::integral_constant<int, 2>{});
  else tile_body(std::integral_constant<int, 1>{});

  qmm_trace(a, work, 3);
  // ---- epilogue: the lane holds weight row row_base[p] + m for tokens 8j + 4h + i of each 32-token block
  if (a.epi == 0) {
    // SwiGLU, narrowed to bf16, transposed through the (now free) x ring so that a lane stores
    // 16 bytes of one token: [token][32 rows] per wave, the rows of a run of 8 in the
    // (0,4,1,5,2,6,3,7) order phase 2 reads, i.e. rows r and r + 4 share a 32-bit word.
    __syncthreads();  // every wave is past its last read of the ring
    uint32_t* so = reinterpret_cast<uint32_t*>(s_x) + wv * 1024;
    const bool upper = (m >> 2) & 1u;
    const uint32_t dw = ((m & ~7u) >> 1) + (m & 3u);  // word of the row pair (r, r + 4)
    // The activation's variants are chosen outside the element loops (one uniform branch: Maple's or the
    // ordinary one) and, for the ordinary one, by selects -- narrowed or not, clamped or not -- so that the
    // 64 exponentials and reciprocals of a lane are one block of code the compiler can interleave (with
    // the three tests inside the loops every element was a block of its own).
    const bool clamp = a.limit > 0.0f, narrow = a.narrow != 0;
    auto swiglu_block = [&](auto maple_tag) __attribute__((always_inline)) {
      constexpr bool kMaple = decltype(maple_tag)::value;
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        if (nt == 1 && count <= 32) break;  // no route in the second block: its slots are empty
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t bits[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float gv = acc[0][nt][4 * j + i], uv = acc[NPROJ - 1][nt][4 * j + i];
            if constexpr (kMaple) {  // maple_moe.metal:153-164
              bits[i] = f_to_bf16(maple_swiglu(gv, uv));
            } else {
              const float gr = round_bf16(gv), ur = round_bf16(uv);
              const float g0 = narrow ? gr : gv, u0 = narrow ? ur : uv;
              gv = clamp ? fminf(g0, a.limit) : g0;  // (selects, so that a NaN stays one without a clamp)
              uv = clamp ? fminf(fmaxf(u0, -a.limit), a.limit) : u0;
              bits[i] = f_to_bf16(fast_silu(gv) * uv);
            }
          }
          // lanes m and m ^ 4 trade halves: the lower lane ends with tokens i = 0, 1 of both rows,
          // the upper lane with tokens i = 2, 3
          const uint32_t t01 = bits[0] | (bits[1] << 16), t23 = bits[2] | (bits[3] << 16);
          const uint32_t keep = upper ? t23 : t01;
          const uint32_t got = static_cast<uint32_t>(
              __builtin_amdgcn_ds_swizzle(static_cast<int>(upper ? t01 : t23), 0x101F));  // lane ^ 4
          const uint32_t lo_row = upper ? got : keep, hi_row = upper ? keep : got;
          const uint32_t tok = nt * 32 + 8 * j + 4 * h + (upper ? 2u : 0u);
          so[tok * 16 + dw] = __builtin_amdgcn_perm(hi_row, lo_row, 0x05040100u);
          so[(tok + 1) * 16 + dw] = __builtin_amdgcn_perm(hi_row, lo_row, 0x07060302u);
        }
      }
    };
    if (a.maple) swiglu_block(std::true_type{});
    else swiglu_block(std::false_type{});
    __builtin_amdgcn_wave_barrier();  // the wave reads back only what it wrote itself
    const uint32_t lane = threadIdx.x & 63u;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      if (it == 2 && count <= 32) break;
      const uint32_t c = it * 64 + lane, tok = c >> 2, part = c & 3u;
      const uint32_t sl = s_slot[tok];
      const uint4 v = reinterpret_cast<const uint4*>(so)[c];
      if (sl != 0xFFFFFFFFu)
        *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(out_base) + static_cast<size_t>(sl) * a.rows + row_base[0] +
                                  part * 8) = v;
    }
  } else {
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      if (nt == 1 && count <= 32) break;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint4 sl = *reinterpret_cast<const uint4*>(s_slot + nt * 32 + 8 * j + 4 * h);
        const uint32_t slot[4] = {sl.x, sl.y, sl.z, sl.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (slot[i] == 0xFFFFFFFFu) continue;
          const size_t at = static_cast<size_t>(slot[i]) * a.rows;
#pragma unroll
          for (int p = 0; p < NPROJ; ++p) {
            if (p > 0 && !a.pair_rows && !out2_base) break;
            uint8_t* ob = (p > 0 && !a.pair_rows) ? out2_base : out_base;  // the second projection's own buffer
            if (a.epi == 1) reinterpret_cast<float*>(ob)[at + row_base[p] + m] = acc[p][nt][4 * j + i];
            else reinterpret_cast<uint16_t*>(ob)[at + row_base[p] + m] = f_to_bf16(acc[p][nt][4 * j + i]);
          }
        }
      }
    }
  }
  qmm_trace(a, work, 4);
}

// ---- the same product for a short contraction (K <= 512: the down projections) ----
// With K this short the x tile of a workgroup (64 routes x K bf16 <= 64 KB) stays in LDS whole, so a
// workgroup stages it once and then walks over `slices` consecutive 256-row slices of the weight matrix
// without any further workgroup barrier: the waves run free, each wave's next-slice codes and scale / bias
// words are requested while it still multiplies the current slice, and the stores of a finished slice
// drain while the next one starts.  (qmm_kernel re-stages x through a two-stage ring for every 128 or 256
// rows, four barriers per 8 groups, and pays its set-up -- tile, routes, tables, 3 us -- per slice.)
// A wave owns two consecutive 32-row blocks (64 rows).  Routes past the tile's count repeat the tile's
// last route in every respect, its output slot included: they store the same values to the same place,
// and no store needs a branch.
struct KresLaunch {
  QmmArgs part[2];
  uint32_t per_xcd[2];   // work items of each part on one XCD (grid = 8 * their sum)
  uint32_t slices[2];    // 256-row slices one work item walks (divides rows / 256)
};

template <int NG> __device__ __forceinline__ uint4 load_groups_bf16(const uint16_t* p) {  // NG bf16, zero-padded to 8
  if constexpr (NG >= 8) {
    return *reinterpret_cast<const uint4*>(p);
  } else if constexpr (NG == 4) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    return make_uint4(v.x, v.y, 0, 0);
  } else {
    return make_uint4(*reinterpret_cast<const uint32_t*>(p), 0, 0, 0);
  }
}

template <int BITS, int NG>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void qmm_kres_kernel(const KresLaunch launch) {
  static_assert(NG == 2 || NG == 4 || NG == 8, "K is 128, 256 or 512");
  constexpr uint32_t kGB = QmmCodes<BITS>::kGroupBytes;  // bytes of one K group of one weight row
  constexpr int kRing = NG < 4 ? NG : 4;  // code registers in flight per projection
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const uint32_t m = lane & 31, h = lane >> 5;
  const uint32_t xcd_slot = blockIdx.x >> 3;
  const bool second = xcd_slot >= launch.per_xcd[0];
  const QmmArgs& a = launch.part[second ? 1 : 0];
  const uint32_t work = (blockIdx.x & 7u) * launch.per_xcd[second ? 1 : 0] + (xcd_slot - (second ? launch.per_xcd[0] : 0u));
  const uint32_t n_walk = launch.slices[second ? 1 : 0];
  const uint32_t items_per_tile = a.rows / (256u * n_walk);
  uint32_t tile_id = work / items_per_tile, slice0 = (work % items_per_tile) * n_walk;
  if (a.dense_mode) {
    if (work >= a.dense_items) return;
    tile_id = a.tile_major ? work / items_per_tile : work % a.dense_tiles;
    slice0 = (a.tile_major ? work % items_per_tile : work / a.dense_tiles) * n_walk;
    if (tile_id >= a.dense_tiles) return;
  }
  qmm_trace(a, work, 0);

  uint32_t expert = 0, pair_start, count;
  if (a.dense_mode) {
    pair_start = tile_id * kTileTokens;
    count = min(kTileTokens, a.dense_rows - pair_start);
  } else {
    // (the whole 16-byte record in one load: read field by field, the count was fetched, tested, and the rest
    // fetched in a second round trip)
    const uint4 tv = *reinterpret_cast<const uint4*>(a.tiles + tile_id);
    const Tile t{tv.x, tv.y, tv.z, tv.w};
    if (t.count == 0) return;
    expert = t.expert;
    pair_start = t.pair_start;
    count = t.count;
  }
  uint4* s_x = reinterpret_cast<uint4*>(smem);                       // [NG groups][512]
  uint32_t* s_slot = reinterpret_cast<uint32_t*>(smem + NG * 8192);  // [64]
  float* s_sum = reinterpret_cast<float*>(smem + NG * 8192 + kTileTokens * 4);  // [64 routes][NG]

  const uint8_t* W;
  const uint16_t* Sp;
  const uint16_t* Bp;
  if (a.dense_mode) {
    W = static_cast<const uint8_t*>(a.dense[0].weights);
    Sp = a.dense[0].scales;
    Bp = a.dense[0].biases;
  } else {
    const uint8_t* blob = a.expert_base + static_cast<size_t>(expert) * a.expert_stride;
    W = blob + a.w_off[0];
    Sp = reinterpret_cast<const uint16_t*>(blob + a.s_off[0]);
    Bp = reinterpret_cast<const uint16_t*>(blob + a.b_off[0]);
  }
  constexpr uint32_t kRowBytes = NG * kGB;
  // the lane's weight row of block p of slice w: row0 + 256 w + 32 p
  const uint32_t row0 = (slice0 * kQmmWaves + wv) * 64 + m;
  const uint32_t gstride = a.tiled ? 32u * kGB : kGB;
  const uint8_t* wrow = a.tiled ? W + static_cast<size_t>(row0 - m) * kRowBytes + lane * (kGB / 2)
                                : W + static_cast<size_t>(row0) * kRowBytes + h * (kGB / 2);
  const uint16_t* srow = Sp + static_cast<size_t>(row0) * NG;
  const uint16_t* brow = Bp + static_cast<size_t>(row0) * NG;

  // ---- everything issued back to back: codes of the first slice, its scale / bias words, the x tile
  QmmCodes<BITS> cur[2][kRing];
#pragma unroll
  for (int p = 0; p < 2; ++p)
#pragma unroll
    for (int u = 0; u < kRing; ++u) cur[p][u].load(wrow + p * 32 * kRowBytes + u * gstride);
  uint4 nS[2], nB[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    nS[p] = load_groups_bf16<NG>(srow + p * 32 * NG);
    nB[p] = load_groups_bf16<NG>(brow + p * 32 * NG);
  }
  const uint32_t st_i = threadIdx.x >> 2, st_q = threadIdx.x & 3;  // staging: route i, K values 16q..16q+15 of a group
  const uint16_t* st_src = a.x + static_cast<size_t>(pair_start + min(st_i, count - 1)) * a.x_stride + st_q * 16;
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  u32x4_t xv[2 * NG];
#pragma unroll
  for (int g = 0; g < 2 * NG; ++g) xv[g] = *reinterpret_cast<const u32x4_t*>(st_src + (g >> 1) * kGroup + (g & 1) * 8);
  uint32_t slot = 0;
  if (threadIdx.x < kTileTokens) {
    const uint32_t pi = pair_start + min(threadIdx.x, count - 1);
    slot = pi;
    if (!a.dense_mode && (a.epi == 1 || a.epi == 3)) {
      const mf_pair pr = a.sorted[pi];
      slot = pr.token * a.top_k + pr.rank;
    }
  }
  qmm_trace(a, work, 1);

  // ---- x tile into LDS (the layout qmm_kernel's ring uses for one group, NG times)
  {
    const uint32_t st_nt = st_i >> 5, st_n = st_i & 31, c0 = 2 * st_q, c1 = c0 + 1;
    const uint32_t st_rot = 4 * ((c0 & 3) >> 1) + 8 * (c0 >> 2);
    const uint32_t st_slot0 = ((st_nt * 4 + (c0 & 3)) * 2 + (c0 >> 2)) * 32 + ((st_n + st_rot) & 31);
    const uint32_t st_slot1 = ((st_nt * 4 + (c1 & 3)) * 2 + (c1 >> 2)) * 32 + ((st_n + st_rot) & 31);
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      *reinterpret_cast<u32x4_t*>(s_x + g * 512 + st_slot0) = xv[2 * g];
      *reinterpret_cast<u32x4_t*>(s_x + g * 512 + st_slot1) = xv[2 * g + 1];
    }
    if (threadIdx.x < kTileTokens) s_slot[threadIdx.x] = slot;
    // the fp32 sum of every 64-wide group of every route, for the bias and offset terms: the four
    // threads that stage a route each hold 16 of a group's values
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      float part = 0.0f;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const u32x4_t v = xv[2 * g + u];
        part += ((bf16_lo(v.x) + bf16_hi(v.x)) + (bf16_lo(v.y) + bf16_hi(v.y))) +
                ((bf16_lo(v.z) + bf16_hi(v.z)) + (bf16_lo(v.w) + bf16_hi(v.w)));
      }
      part = group_sum(part, 4);
      if (st_q == 0) s_sum[st_i * NG + g] = part;
    }
  }
  uint32_t rd_col[4];
#pragma unroll
  for (int sidx = 0; sidx < 4; ++sidx) rd_col[sidx] = (m + 4 * (sidx >> 1) + 8 * h) & 31;
  __syncthreads();  // the only workgroup barrier: from here on the waves run on their own
  qmm_trace(a, work, 2);
  // sum(x) of a group as three bf16 terms (all 24 bits), see qmm_kernel.  Both halves of the wave hold
  // the sums of groups 0..7 of the lane's two routes: K slots 8h..8h+7 of the bias product are those
  // groups again, multiplied by the biases for h = 0 and by -offset * scale for h = 1.
  // A tile of at most 32 routes fills only the first route block (NTA = 1): the second block, whose routes
  // would all repeat the last route, is left out of the products, the scale multiplies and the stores.
  auto tile_body = [&](auto nta_c) {
  constexpr int NTA = decltype(nta_c)::value;
  uint4 b_term[2][3];
#pragma unroll
  for (int nt = 0; nt < NTA; ++nt) {
    float sx[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sx[e] = e < NG ? s_sum[(nt * 32 + m) * NG + e] : 0.0f;
    uint32_t hi[8], mid[8], lo[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = sx[e];
      hi[e] = __float_as_uint(v) & 0xFFFF0000u;
      const float r1 = v - __uint_as_float(hi[e]);
      mid[e] = __float_as_uint(r1) & 0xFFFF0000u;
      lo[e] = __float_as_uint(r1 - __uint_as_float(mid[e]));
    }
    b_term[nt][0] = make_uint4((hi[0] >> 16) | hi[1], (hi[2] >> 16) | hi[3], (hi[4] >> 16) | hi[5], (hi[6] >> 16) | hi[7]);
    b_term[nt][1] = make_uint4((mid[0] >> 16) | mid[1], (mid[2] >> 16) | mid[3], (mid[4] >> 16) | mid[5],
                               (mid[6] >> 16) | mid[7]);
    b_term[nt][2] = make_uint4(__builtin_amdgcn_perm(lo[1], lo[0], 0x07060302u), __builtin_amdgcn_perm(lo[3], lo[2], 0x07060302u),
                               __builtin_amdgcn_perm(lo[5], lo[4], 0x07060302u), __builtin_amdgcn_perm(lo[7], lo[6], 0x07060302u));
  }

  for (uint32_t w = 0; w < n_walk; ++w) {
    const uint32_t step = w + 1 < n_walk ? 1u : 0u;  // the last slice requests itself again: no branch around loads
    const uint8_t* wnext = wrow + static_cast<size_t>(step) * 256 * kRowBytes;
    // scale words of this slice; bias operand: the biases for K slots 0..7, -offset * scale for K slots
    // 8..15 (formed in place: exponent + 4 or + 2, sign flipped -- exact; a zero scale becomes 2^-123 / 2^-125);
    // ternary rows store no biases: theirs is -scale (the bias pointer is the scale table then)
    uint4 Sv[2], bop[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      constexpr uint32_t kAdd = QmmCodes<BITS>::kNegOffsetAdd;
      Sv[p] = nS[p];
      const uint4 neg = make_uint4((nS[p].x + kAdd) ^ 0x80008000u, (nS[p].y + kAdd) ^ 0x80008000u,
                                   (nS[p].z + kAdd) ^ 0x80008000u, (nS[p].w + kAdd) ^ 0x80008000u);
      const uint32_t flip = a.ternary ? 0x80008000u : 0u;
      bop[p] = h ? neg : make_uint4(nB[p].x ^ flip, nB[p].y ^ flip, nB[p].z ^ flip, nB[p].w ^ flip);
    }
    f32x16_t acc[2][2];
#pragma unroll
    for (int p = 0; p < 2; ++p)
#pragma unroll
      for (int nt = 0; nt < NTA; ++nt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[p][nt][r] = 0.0f;
#pragma unroll
        for (int term = 0; term < 3; ++term) acc[p][nt] = mfma_bf16(b_term[nt][term], bop[p], acc[p][nt]);
      }
    // the next slice's scale / bias words (the registers are free again)
    srow += step * 256 * NG;
    brow += step * 256 * NG;
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      nS[p] = load_groups_bf16<NG>(srow + p * 32 * NG);
      nB[p] = load_groups_bf16<NG>(brow + p * 32 * NG);
    }
    // x of a group comes out of LDS one group ahead, into the registers the matrix core has just read
    uint4 bx[2][4];
    if (w == 0) {
#pragma unroll
      for (int nt = 0; nt < NTA; ++nt)
#pragma unroll
        for (int s = 0; s < 4; ++s) bx[nt][s] = s_x[((nt * 4 + s) * 2 + h) * 32 + rd_col[s]];
    }
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const uint4* nbuf = s_x + ((g + 1) % NG) * 512;  // after the last group: group 0 again, for the next slice
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const uint32_t sw[4] = {Sv[p].x, Sv[p].y, Sv[p].z, Sv[p].w};
        const float sc = QmmCodes<BITS>::kScaleMul * ((g & 1) ? bf16_hi(sw[g >> 1]) : bf16_lo(sw[g >> 1]));
        f32x16_t tmp[2];
#pragma unroll
        for (int nt = 0; nt < NTA; ++nt)
#pragma unroll
          for (int r = 0; r < 16; ++r) tmp[nt][r] = 0.0f;
        group_products<BITS, NTA>(cur[p][g % kRing], bx, tmp, [&](int s) {
          if (p == 1) {  // both row blocks have read x slot s of this group
            bx[0][s] = nbuf[((0 * 4 + s) * 2 + h) * 32 + rd_col[s]];
            if (NTA > 1) bx[1][s] = nbuf[((1 * 4 + s) * 2 + h) * 32 + rd_col[s]];
          }
        });
        // the register takes the codes kRing groups on: of this slice, or of the next one
        const int ahead = g + kRing;
        cur[p][g % kRing].load(ahead < NG ? wrow + p * 32 * kRowBytes + ahead * gstride
                                          : wnext + p * 32 * kRowBytes + (ahead - NG) * gstride);
#pragma unroll
        for (int nt = 0; nt < NTA; ++nt)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[p][nt][r] = __builtin_fmaf(sc, tmp[nt][r], acc[p][nt][r]);
        // the sums are wanted here, not after the last group: without this the compiler keeps every
        // group's products and adds them up at the end of the slice, out of scratch memory
        if constexpr (NTA > 1) asm volatile("" : "+v"(acc[p][0]), "+v"(acc[p][1]));
        else asm volatile("" : "+v"(acc[p][0]));
        __builtin_amdgcn_sched_barrier(0);  // one unit at a time: hoisted loads would cost more registers than exist
      }
    }
    if (w + 1 == n_walk) qmm_trace(a, work, 3);
    // ---- stores: the lane holds rows row + 32 p for routes 8j + 4h + i of each 32-route block
    const uint32_t row = row0 + w * 256;
    // byte offsets fit 32 bits (the launcher checks): one multiply-add per route, the base stays scalar
    if (a.epi == 1) {
      uint8_t* out = static_cast<uint8_t*>(a.out);
      const uint32_t pitch = a.rows * 4, col = row * 4;
#pragma unroll
      for (int nt = 0; nt < NTA; ++nt) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint4 sl = *reinterpret_cast<const uint4*>(s_slot + nt * 32 + 8 * j + 4 * h);
          const uint32_t sl4[4] = {sl.x, sl.y, sl.z, sl.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float* o = reinterpret_cast<float*>(out + (sl4[i] * pitch + col));
            o[0] = acc[0][nt][4 * j + i];
            o[32] = acc[1][nt][4 * j + i];
          }
        }
      }
    } else {
      uint8_t* out = static_cast<uint8_t*>(a.out);
      const uint32_t pitch = a.rows * 2, col = row * 2;
#pragma unroll
      for (int nt = 0; nt < NTA; ++nt) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint4 sl = *reinterpret_cast<const uint4*>(s_slot + nt * 32 + 8 * j + 4 * h);
          const uint32_t sl4[4] = {sl.x, sl.y, sl.z, sl.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            uint16_t* o = reinterpret_cast<uint16_t*>(out + (sl4[i] * pitch + col));
            o[0] = f_to_bf16(acc[0][nt][4 * j + i]);
            o[32] = f_to_bf16(acc[1][nt][4 * j + i]);
          }
        }
      }
    }
    wrow = wnext;
  }
  };  // tile_body
  if (count > 32) tile_body(std::integral_constant<int, 2>{});
  else tile_body(std::integral_constant<int, 1>{});
  qmm_trace(a, work, 4);
}

// y[t,d] = bf16(h1[t,d] + sum_r w[t,r] * partial[t*K+r, d]), residual first, rank
// order, product then add (moe.metal:1262-1270; reduce of prefill.metal:631-652).
// h1 = bf16(hs / (1 + exp(-gate_t))) when a scalar gate is given (utility.metal:49-59).
template <bool NARROW>  // the per-route results are bf16 numbers (stored as such) instead of fp32
__global__ __launch_bounds__(256) void prefill_reduce_kernel(const float* __restrict__ partials,
                                                             const float* __restrict__ w,
                                                             const uint32_t* __restrict__ idx,
                                                             const uint16_t* __restrict__ hs,
                                                             const uint16_t* __restrict__ gate,
                                                             uint16_t* __restrict__ y, uint32_t T,
                                                             uint32_t K, uint32_t D, uint32_t E, int maple) {
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
  // all of a token's routes are requested before the first is used (a short batch has few waves: a loop
  // that tests a route's expert before it asks for the route's row walks K round trips one after another);
  // the row of a route without an expert is read and dropped
  uint32_t ex[MF_MAX_TOPK];
  float wt[MF_MAX_TOPK];
  float4 v[MF_MAX_TOPK];
#pragma unroll
  for (uint32_t r = 0; r < MF_MAX_TOPK; ++r) {
    if (r < K) {
      ex[r] = idx ? idx[t * K + r] : 0u;
      wt[r] = w[t * K + r];
      if constexpr (NARROW) {
        const uint2 q = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(partials) +
                                                        (static_cast<size_t>(t) * K + r) * D + d);
        v[r] = make_float4(bf16_lo(q.x), bf16_hi(q.x), bf16_lo(q.y), bf16_hi(q.y));
      } else {
        v[r] = *reinterpret_cast<const float4*>(partials + (static_cast<size_t>(t) * K + r) * D + d);
      }
    }
  }
#pragma unroll
  for (uint32_t r = 0; r < MF_MAX_TOPK; ++r) {
    if (r < K && ex[r] < E) {  // a route without an expert adds nothing
      float4 q = v[r];
      if (maple && !NARROW) {  // maple_moe.metal:258: the down output is a bf16 number before its weight
        q.x = round_bf16(q.x); q.y = round_bf16(q.y); q.z = round_bf16(q.z); q.w = round_bf16(q.w);
      }
      const float p0 = wt[r] * q.x, p1 = wt[r] * q.y, p2 = wt[r] * q.z, p3 = wt[r] * q.w;
      acc[0] = acc[0] + p0; acc[1] = acc[1] + p1; acc[2] = acc[2] + p2; acc[3] = acc[3] + p3;
    }
  }
  uint2 o;
  o.x = static_cast<uint32_t>(f_to_bf16(acc[0])) | (static_cast<uint32_t>(f_to_bf16(acc[1])) << 16);
  o.y = static_cast<uint32_t>(f_to_bf16(acc[2])) | (static_cast<uint32_t>(f_to_bf16(acc[3])) << 16);
  *reinterpret_cast<uint2*>(y + i4) = o;
}

// The caller's counts as the one-chunk histogram of the scan, and the check's flag cleared (a kernel,
// not a memset or a copy node, so that the call can be captured into a graph).
__global__ __launch_bounds__(512) void ragged_begin_kernel(const uint32_t* __restrict__ counts, uint32_t E,
                                                           uint32_t* __restrict__ hist, uint32_t* __restrict__ bad) {
  if (threadIdx.x < E) hist[threadIdx.x] = counts[threadIdx.x];
  if (threadIdx.x == 0) *bad = 0;
}

// A caller's grouping before the matmuls trust it: the counts cover at most T*K routes, and every
// route the counts cover names a token below T and a rank below K.  Sets *bad otherwise.
__global__ __launch_bounds__(256) void ragged_check_kernel(const mf_pair* __restrict__ sorted,
                                                           const uint32_t* __restrict__ counts,
                                                           uint32_t E, uint32_t T, uint32_t K,
                                                           uint32_t* __restrict__ bad) {
  __shared__ unsigned long long s_total;
  if (threadIdx.x == 0) s_total = 0;
  __syncthreads();
  unsigned long long part = 0;
  for (uint32_t e = threadIdx.x; e < E; e += blockDim.x) part += counts[e];
  if (part) atomicAdd(&s_total, part);
  __syncthreads();
  const unsigned long long total = s_total, pairs = static_cast<unsigned long long>(T) * K;
  if (total > pairs) {
    if (blockIdx.x == 0 && threadIdx.x == 0) atomicOr(bad, 1u);
    return;
  }
  bool wrong = false;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const mf_pair p = sorted[i];
    wrong |= p.token >= T || p.rank >= K;
  }
  if (wrong) atomicOr(bad, 1u);
}

// ------------------------------------------------------------------ launchers

// `tail` (optional): the x preparation a short batch wants done in the same launch; on return
// tail->xp is null when the launch did not take it on (the caller then launches it).
hipError_t launch_prefill_router(hipStream_t s, const uint16_t* W, const uint16_t* x, uint32_t E,
                                 uint32_t D, uint32_t T, uint32_t x_stride, float* logits, RouterTail* tail) {
  RouterTail fused{};
  if (tail) {
    fused = *tail;
    tail->xp = nullptr;
  }
  // Up to 192 tokens the matrix-core kernel has too few workgroups (T/32 x E/32) to cover the chip: the
  // register-tiled kernel is faster there (Qwen shape, layer time: 128 tokens 79 against 82 us, equal at 192,
  // 256 tokens 98.4 against 96.4 us; it holds rows of up to 4096 elements).  Both give the same bits.  The
  // matrix-core kernel takes whole blocks of 32 rows; rows left over (the two sink rows of a 258-row
  // Inkling router) go through the register-tiled kernel behind it.
  const uint32_t e32 = (T > 192 || D > 4096) && D % 512 == 0 && aligned16(W) && aligned16(x) && x_stride % 8 == 0
                           ? E & ~31u : 0u;
  // rows of more than 4096 elements that the matrix-core kernel does not take (a width that is no
  // multiple of 512, rows left over by the blocks of 32, unaligned operands): the register-tiled
  // kernel cannot hold them, so the whole call goes one wave per (token, row) -- the same bits
  if ((D / 8 + 63) / 64 > 8 && e32 != E) return launch_router_logits(s, W, x, E, D, T, x_stride, logits, nullptr);
  const bool tail_ok = fused.xp && x_stride == D && D % 64 == 0 && aligned16(x) && aligned16(fused.xp) &&
                       (!fused.w_sg || aligned16(fused.w_sg));
  if (e32) {
    RouterTail mt{};
    uint32_t prep_rows = 0;
    if (tail_ok) {  // the x preparation rides in this launch: workgroup rows behind the expert blocks
      mt = fused;
      mt.router_cols = e32 / 32;
      fused.xp = nullptr;  // done here: the register-tiled launch for left-over rows does not repeat it
      tail->xp = mt.xp;
    }
    if (tail_ok) prep_rows = ((T + 3) / 4 + (T + 31) / 32 - 1) / ((T + 31) / 32);
    const dim3 grid((T + 31) / 32, e32 / 32 + prep_rows);
    if (D == 1024) prefill_router_mfma_kernel<2><<<grid, dim3(256), 0, s>>>(W, x, e32, D, T, x_stride, logits, E, mt);
    else if (D == 2048) prefill_router_mfma_kernel<4><<<grid, dim3(256), 0, s>>>(W, x, e32, D, T, x_stride, logits, E, mt);
    else if (D == 4096) prefill_router_mfma_kernel<8><<<grid, dim3(256), 0, s>>>(W, x, e32, D, T, x_stride, logits, E, mt);
    else prefill_router_mfma_kernel<0><<<grid, dim3(256), 0, s>>>(W, x, e32, D, T, x_stride, logits, E, mt);
    if (e32 == E) return hipGetLastError();
  }
  const uint32_t rest = E - e32;
  const uint16_t* Wr = W + static_cast<size_t>(e32) * D;
  float* lr = logits + e32;
  const uint32_t cpl = (D / 8 + 63) / 64;
  // about a thousand workgroups, >= 4 tokens per row load; the few rows left over by the matrix-core kernel
  // fill one workgroup column only, so they take the shortest token runs
  const uint32_t tpb = e32 ? 4u : std::max(4u, std::min(64u, T / 64));
  const uint32_t token_blocks = (T + tpb - 1) / tpb;
  // the whole call in this kernel, x rows as the preparation reads them: the launch takes the tail on
  const bool take_tail = tail_ok && fused.xp && !e32 && cpl <= 8;
  if (!take_tail) fused = RouterTail{};
  const uint32_t prep_cols = take_tail ? ((T + 3) / 4 + token_blocks - 1) / token_blocks : 0u;
#define MF_PR(CPL, R)                                                                              \
  do {                                                                                             \
    fused.router_cols = (rest + 4 * R - 1) / (4 * R);                                              \
    prefill_router_kernel<CPL, R><<<dim3(fused.router_cols + prep_cols, token_blocks), dim3(256), 0, s>>>( \
        Wr, x, rest, D, T, x_stride, lr, tpb, E, fused);                                           \
  } while (0)
  if (cpl <= 1) MF_PR(1, 4);
  else if (cpl <= 2) MF_PR(2, 4);
  else if (cpl <= 4) MF_PR(4, 4);
  else if (cpl <= 8) MF_PR(8, 2);
  else return hipErrorInvalidValue;
#undef MF_PR
  if (take_tail) tail->xp = fused.xp;
  return hipGetLastError();
}

hipError_t launch_prefill_router(hipStream_t s, const uint16_t* W, const uint16_t* x, uint32_t E,
                                 uint32_t D, uint32_t T, uint32_t x_stride, float* logits) {
  return launch_prefill_router(s, W, x, E, D, T, x_stride, logits, nullptr);
}

hipError_t launch_group(hipStream_t s, const uint32_t* idx, const float* w, uint32_t t, uint32_t K,
                        uint32_t E, uint32_t* counts, uint32_t* offsets, uint32_t* starts,
                        mf_pair* sorted, void* tiles, uint32_t tile_slots, uint32_t* n_tiles,
                        uint32_t* status, uint32_t* chunk_hist) {
  const uint32_t n_pairs = t * K;
  if (n_pairs && n_pairs <= kGroupOnePairs && group_one_lds_bytes(t, E) <= kGroupOneMaxBytes) {
    const size_t lds = group_one_lds_bytes(t, E);
    uint32_t tpe_log2 = 0;  // threads per row of the bit matrix: as many as 1024 threads give, at most 16
    while (tpe_log2 < 4 && (E << (tpe_log2 + 1)) <= 1024) ++tpe_log2;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(group_one_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kGroupOneMaxBytes));
    if (e != hipSuccess) return e;
    group_one_kernel<<<dim3(1), dim3(1024), lds, s>>>(idx, w, n_pairs, K, E, tpe_log2, counts, offsets, starts, sorted,
                                                      static_cast<Tile*>(tiles), tile_slots, n_tiles, status);
    return hipGetLastError();
  }
  if (n_pairs == 0) {  // no routes: the scan over no chunks writes empty experts and a clean status word
    group_scan_kernel<<<dim3(1), dim3(MF_MAX_EXPERTS), 0, s>>>(chunk_hist, 0, E, counts, offsets, starts,
                                                               static_cast<Tile*>(tiles), tile_slots, n_tiles,
                                                               chunk_hist, status);
    return hipGetLastError();
  }
  // at most kGroupChunks chunks, each a whole number of kGroupBlock-pair steps
  const uint32_t steps = (n_pairs + kGroupBlock - 1) / kGroupBlock;
  const uint32_t chunk_pairs = (steps + kGroupChunks - 1) / kGroupChunks * kGroupBlock;
  const uint32_t n_chunks = (n_pairs + chunk_pairs - 1) / chunk_pairs;
  uint32_t* chunk_bad = chunk_hist + static_cast<size_t>(kGroupChunks) * MF_MAX_EXPERTS;
  group_count_kernel<<<dim3(n_chunks), dim3(256), 0, s>>>(idx, n_pairs, E, chunk_pairs, chunk_hist, chunk_bad);
  group_scan_kernel<<<dim3(1), dim3(MF_MAX_EXPERTS), 0, s>>>(chunk_hist, n_chunks, E, counts, offsets, starts,
                                                             static_cast<Tile*>(tiles), tile_slots, n_tiles,
                                                             chunk_bad, status);
  group_emit_kernel<<<dim3(n_chunks), dim3(256), 0, s>>>(idx, w, n_pairs, K, E, chunk_pairs, chunk_hist, starts,
                                                         sorted);
  return hipGetLastError();
}

// words of the handle's grouping scratch: 2048 of small tables, the per-chunk counts and flags of the
// three-launch grouping, and behind them the per-chunk 64-bit words and the [chunk][expert] count bytes of
// the layer call's own grouping
constexpr size_t kGroupBitsAt = 2048 + static_cast<size_t>(kGroupChunks) * MF_MAX_EXPERTS + kGroupChunks;  // even
constexpr size_t kGroupCntAt = kGroupBitsAt + 2 * static_cast<size_t>(kGroupChunks) * MF_MAX_EXPERTS;
size_t group_scratch_words() { return kGroupCntAt + static_cast<size_t>(kGroupChunks) * MF_MAX_EXPERTS / 4; }

// Selection and grouping of the layer call's own routes in two launches (topk_chunk_kernel,
// group_place_kernel); false when the batch is too long for chunks of 64 tokens.
bool topk_group_takes(uint32_t t) { return t != 0 && t <= kGroupChunks * kChunkTokensMax; }

hipError_t launch_topk_group(hipStream_t s, const float* logits, uint32_t t, uint32_t K, uint32_t E, int mode,
                             uint32_t* idx, float* w, uint32_t* counts, uint32_t* offsets, uint32_t* starts,
                             mf_pair* sorted, void* tiles, uint32_t tile_slots, uint32_t* n_tiles, uint32_t* status,
                             uint32_t* group_tmp) {
  // a token per wave while that gives at most 128 chunks, then longer chunks, then more of them
  uint32_t chunk_tokens = ((t + 127) / 128 + kSelectWaves - 1) / kSelectWaves * kSelectWaves;
  chunk_tokens = std::min(std::max(chunk_tokens, kSelectWaves), kChunkTokensMax);
  const uint32_t n_chunks = (t + chunk_tokens - 1) / chunk_tokens;
  auto* bits = reinterpret_cast<unsigned long long*>(group_tmp + kGroupBitsAt);
  auto* cnt = reinterpret_cast<uint8_t*>(group_tmp + kGroupCntAt);
  uint32_t* bad = group_tmp + 2048 + static_cast<size_t>(kGroupChunks) * MF_MAX_EXPERTS;
  topk_chunk_kernel<<<dim3(n_chunks), dim3(kSelectWaves * 64), 0, s>>>(logits, t, E, K, mode, chunk_tokens, idx, w, bits,
                                                                       cnt, bad);
  group_place_kernel<<<dim3(n_chunks), dim3(MF_MAX_EXPERTS), 0, s>>>(idx, w, t, K, E, chunk_tokens, n_chunks, bits, cnt,
                                                                    bad, counts, offsets, starts, sorted,
                                                                    static_cast<Tile*>(tiles), tile_slots, n_tiles,
                                                                    status);
  return hipGetLastError();
}

size_t qmm_lds_bytes(uint32_t kdim, int nproj, bool tab16) {
  const uint32_t ng = kdim / kGroup;
  return kQmmXBytes + ((static_cast<size_t>(nproj) * kQmmWaves * ng * 32 * (tab16 ? 2 : 4) + 15) & ~static_cast<size_t>(15)) +
         kTileTokens * 4;
}
// the scale tables as bf16 where fp32 tables would leave a CU (160 KB of LDS) room for one workgroup only
bool qmm_tab16(uint32_t kdim, int nproj) { return 2 * qmm_lds_bytes(kdim, nproj, false) > 160 * 1024; }

hipError_t launch_prep_rows(hipStream_t s, const uint16_t* src, uint16_t* dst, float* sums, size_t elems,
                            const uint16_t* src1 = nullptr, uint16_t* dst1 = nullptr, float* sums1 = nullptr,
                            size_t elems1 = 0) {
  PrepArgs a{};
  a.src[0] = src; a.dst[0] = dst; a.sums[0] = sums; a.chunks[0] = static_cast<uint32_t>(elems / 8);
  a.src[1] = src1; a.dst[1] = dst1; a.sums[1] = sums1; a.chunks[1] = static_cast<uint32_t>(elems1 / 8);
  a.blocks0 = (a.chunks[0] + 255) / 256;
  const uint32_t blocks = a.blocks0 + (a.chunks[1] + 255) / 256;
  if (!blocks) return hipSuccess;
  prep_rows_kernel<<<dim3(blocks), dim3(256), 0, s>>>(a);
  return hipGetLastError();
}

// Work items of a dense problem that one XCD gets: an eighth, but at least 4 while there are any -- a handful
// of items (the shared expert beside the routed experts of a short batch) runs faster on few XCDs, whose L2
// serves the x rows and weight rows they share, than spread one to an XCD (Qwen shape, 128 tokens: layer 81 us
// against 89 us).
static uint32_t dense_per_xcd(uint32_t items) { return std::max((items + 7) / 8, std::min(items, 4u)); }
// Whether an XCD should own tiles (and stream all weight rows) or row slices (and stream all of x): whichever
// streams fewer bytes.  code_bits: 4 or 2.
static int dense_tile_major(uint32_t rows, uint32_t x_rows, int code_bits) {
  return static_cast<uint64_t>(rows) * code_bits <= static_cast<uint64_t>(x_rows) * 16;
}

// Whether qmm_kres_kernel takes the problem: a down-projection epilogue, K of 128, 256 or 512, whole
// 256-row slices, tables aligned for vector loads.
bool kres_takes(const QmmArgs& q, size_t out_rows) {
  const uint32_t ng = q.kdim / kGroup;
  if (q.epi == 0 || q.gather || q.kdim % kGroup || !(ng == 2 || ng == 4 || ng == 8) || q.rows % 256) return false;
  if (static_cast<uint64_t>(out_rows) * q.rows * 4 >= (1ull << 32)) return false;  // 32-bit store offsets
  if (q.dense_mode) return aligned16(q.dense[0].scales) && aligned16(q.dense[0].biases) && aligned16(q.dense[0].weights);
  return aligned16(q.expert_base) && q.expert_stride % 16 == 0 && (q.w_off[0] | q.s_off[0] | q.b_off[0]) % 16 == 0;
}

// bits: 4, or 2 for 2-bit and ternary codes (both problems of one launch have the same width)
hipError_t launch_qmm_kres(hipStream_t s, int bits, const QmmArgs& a, uint32_t tile_slots, const QmmArgs* b,
                           uint32_t b_tile_slots) {
  KresLaunch launch{};
  for (int part = 0; part < (b ? 2 : 1); ++part) {
    QmmArgs& q = launch.part[part];
    q = part ? *b : a;
    const uint32_t slots = part ? b_tile_slots : tile_slots;
    const uint32_t n_slices = q.rows / 256;
    // two slices per work item halve the set-up per slice and still leave several rounds of work items
    // (Qwen shape, 2048 tokens, whole layer: 331 us with one slice, 325 with two, 330 with four, 334 with eight)
    const uint32_t walk = n_slices % 2 == 0 ? 2 : 1;
    launch.slices[part] = walk;
    if (q.dense_mode) {
      q.dense_tiles = slots;
      q.tile_major = dense_tile_major(q.rows, q.dense_rows, bits);
      q.dense_items = slots * (n_slices / walk);
      launch.per_xcd[part] = dense_per_xcd(q.dense_items);
    } else {
      launch.per_xcd[part] = slots / 8 * (n_slices / walk);
    }
  }
  const dim3 grid(8 * (launch.per_xcd[0] + launch.per_xcd[1])), block(256);
  if (grid.x == 0) return hipSuccess;
  const uint32_t ng = a.kdim / kGroup;
  const size_t lds = static_cast<size_t>(ng) * 8192 + kTileTokens * 4 + kTileTokens * ng * 4;
#define MF_KRES(B, N)                                                                                  \
  do {                                                                                                 \
    if (lds > 48 * 1024) {                                                                             \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(qmm_kres_kernel<B, N>),         \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
      if (e != hipSuccess) return e;                                                                   \
    }                                                                                                  \
    qmm_kres_kernel<B, N><<<grid, block, lds, s>>>(launch);                                            \
  } while (0)
  if (bits == 4) {
    if (ng == 8) MF_KRES(4, 8); else if (ng == 4) MF_KRES(4, 4); else MF_KRES(4, 2);
  } else {
    if (ng == 8) MF_KRES(2, 8); else if (ng == 4) MF_KRES(2, 4); else MF_KRES(2, 2);
  }
#undef MF_KRES
  return hipGetLastError();
}

// tile_slots: entries of the tile list (routed; a multiple of 8) or number of 64-row tiles (dense).
// `b` (optional) is a second problem for the same instantiation, run behind `a` in the same launch.
hipError_t launch_qmm(hipStream_t s, int bits, QmmArgs a, int nproj, uint32_t tile_slots, const QmmArgs* b,
                      uint32_t b_tile_slots) {
  QmmLaunch launch{};
  size_t lds = 0;
  bool ng8 = true, tab16 = false;
  for (int part = 0; part < (b ? 2 : 1); ++part) {
    QmmArgs& q = launch.part[part];
    q = part ? *b : a;
    const uint32_t slots = part ? b_tile_slots : tile_slots;
    const uint32_t n_slices = q.rows / (kQmmRows * (q.pair_rows ? nproj : 1));
    if (q.dense_mode) {
      q.dense_tiles = slots;
      q.tile_major = dense_tile_major(q.rows * (q.pair_rows ? 1 : nproj), q.dense_rows, bits);
      q.dense_items = slots * n_slices * std::max(1u, q.n_win);
      launch.per_xcd[part] = dense_per_xcd(q.dense_items);
    } else {
      launch.per_xcd[part] = slots / 8 * n_slices;
    }
    q.tab_aligned = q.dense_mode
        ? aligned16(q.dense[0].scales) && aligned16(q.dense[0].biases) && aligned16(q.dense[1].scales) &&
              aligned16(q.dense[1].biases)
        : aligned16(q.expert_base) && q.expert_stride % 16 == 0 &&
              (q.s_off[0] | q.b_off[0] | q.s_off[1] | q.b_off[1]) % 16 == 0;
    tab16 = tab16 || qmm_tab16(q.kdim, nproj);  // with windows: kdim is the longest window
    ng8 = ng8 && (q.n_win > 1 ? q.ng_ld : q.kdim / kGroup) % 8 == 0;
  }
  for (int part = 0; part < (b ? 2 : 1); ++part) lds = std::max(lds, qmm_lds_bytes(launch.part[part].kdim, nproj, tab16));
  const dim3 grid(8 * (launch.per_xcd[0] + launch.per_xcd[1])), block(256);
  if (grid.x == 0) return hipSuccess;
#define MF_QMM(B, P, G, T)                                                                             \
  do {                                                                                                 \
    if (lds > 48 * 1024) {                                                                             \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(qmm_kernel<B, P, G, T>),        \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)); \
      if (e != hipSuccess) return e;                                                                   \
    }                                                                                                  \
    qmm_kernel<B, P, G, T><<<grid, block, lds, s>>>(launch);                                           \
  } while (0)
#define MF_QMM_G(B, P, G)                                            \
  do {                                                               \
    if (tab16) MF_QMM(B, P, G, true); else MF_QMM(B, P, G, false);   \
  } while (0)
#define MF_QMM_B(B)                                                        \
  do {                                                                     \
    if (nproj == 2) { if (ng8) MF_QMM_G(B, 2, true); else MF_QMM_G(B, 2, false); } \
    else { if (ng8) MF_QMM_G(B, 1, true); else MF_QMM_G(B, 1, false); }    \
  } while (0)
  if (bits == 4) MF_QMM_B(4); else MF_QMM_B(2);
#undef MF_QMM_B
#undef MF_QMM_G
#undef MF_QMM
  return hipGetLastError();
}

namespace {
size_t up256(size_t v) { return (v + 255) / 256 * 256; }
}  // namespace

// ---- dense projections over many rows: MPPPrefillInt4QMM.encode (MPPPrefillInt4QMM.swift:34-78) and the
// block form of the shared expert / dense MLP (PrefillSharedExpert.encodeBlock, PrefillSharedExpert.swift:81-172)
//
// y[m, n] = x[m, k] . W[n, k]^T through qmm_kernel in dense mode.  The kernel keeps the scales of a
// workgroup's rows for the whole contraction in LDS, so a long K is cut into windows of at most
// kDenseWindow groups (multiples of 8 groups, the last takes the rest): every window is a launch that
// writes fp32 [m, n], and dense_combine_kernel adds the windows in order and narrows the sum.
// A gate / up pair whose K does not fit one launch's tables (kDenseFusedMax groups) goes the same way:
// both projections as fp32 per window, then dense_swiglu_combine_kernel.
constexpr uint32_t kDenseWindow = 64;   // K groups per launch (4096 values)
constexpr uint32_t kDenseFusedMax = 112;  // K groups a gate/up + SwiGLU launch can hold (both projections' scales in LDS)
__global__ __launch_bounds__(256) void dense_combine_kernel(const float* __restrict__ parts, uint32_t n_parts,
                                                            size_t part_stride, void* __restrict__ y, size_t count,
                                                            int out_f32) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float acc = parts[i];
  for (uint32_t p = 1; p < n_parts; ++p) acc = acc + parts[p * part_stride + i];
  if (out_f32) static_cast<float*>(y)[i] = acc;
  else static_cast<uint16_t*>(y)[i] = f_to_bf16(acc);
}

// windows of a contraction of length k
static uint32_t dense_windows(uint32_t k, uint32_t max_groups = kDenseWindow) {
  return std::max(1u, (k / kGroup + max_groups - 1) / max_groups);
}

// bytes of fp32 window results a projection of n rows over m tokens needs (0: one window, written directly)
static size_t dense_parts_bytes(uint32_t m, uint32_t n, uint32_t k) {
  const uint32_t n_win = dense_windows(k);
  return n_win > 1 ? up256(sizeof(float) * static_cast<size_t>(m) * n) * n_win : 0;
}
// ... and of the gate / up pair of an MLP (both projections of a work item: kQmmRows rows each)
static uint32_t dense_gate_up_windows(uint32_t d) {
  return dense_windows(d, kDenseFusedMax);
}
static size_t dense_gate_up_parts_bytes(uint32_t t, uint32_t f, uint32_t d) {
  const uint32_t n_win = dense_gate_up_windows(d);
  return n_win > 1 ? 2 * up256(sizeof(float) * static_cast<size_t>(t) * f) * n_win : 0;
}

// The windows of a gate / up pair meet here: sums in window order, gate and up narrowed to bf16
// (dequant_int4.metal:240-245), act = bf16(silu(gate) * up) written in the matmul's order (0,4,1,5,2,6,3,7 inside
// every run of 8) with the fp32 sum of every 64-wide group beside it -- what the SwiGLU epilogue of the
// one-window launch and prep_rows_kernel produce together.  One thread per run of 8.
__global__ __launch_bounds__(256) void dense_swiglu_combine_kernel(const float* __restrict__ pg, const float* __restrict__ pu,
                                                                   uint32_t n_parts, size_t part_stride,
                                                                   uint16_t* __restrict__ act, float* __restrict__ sums,
                                                                   size_t chunks, float limit) {
  const size_t c = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  float g[8], u[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) g[i] = u[i] = 0.0f;
  if (c < chunks) {
    for (uint32_t p = 0; p < n_parts; ++p) {
      const float4 g0 = *reinterpret_cast<const float4*>(pg + p * part_stride + c * 8);
      const float4 g1 = *reinterpret_cast<const float4*>(pg + p * part_stride + c * 8 + 4);
      const float4 u0 = *reinterpret_cast<const float4*>(pu + p * part_stride + c * 8);
      const float4 u1 = *reinterpret_cast<const float4*>(pu + p * part_stride + c * 8 + 4);
      const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
      const float uv[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        g[i] = p == 0 ? gv[i] : g[i] + gv[i];
        u[i] = p == 0 ? uv[i] : u[i] + uv[i];
      }
    }
  }
  uint32_t a[8];
  float v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float gr = round_bf16(g[i]), ur = round_bf16(u[i]);
    if (limit > 0.0f) {
      gr = fminf(gr, limit);
      ur = fminf(fmaxf(ur, -limit), limit);
    }
    a[i] = f_to_bf16(fast_silu(gr) * ur);
    v[i] = bf16_to_f(static_cast<uint16_t>(a[i]));
  }
  float sum = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
  sum = group_sum(sum, 8);
  if (c >= chunks) return;
  *reinterpret_cast<uint4*>(act + c * 8) = make_uint4(a[0] | (a[4] << 16), a[1] | (a[5] << 16), a[2] | (a[6] << 16),
                                                      a[3] | (a[7] << 16));
  if ((c & 7) == 0) sums[c >> 3] = sum;
}

bool dense_qmm_takes(const mf_qtensor& w, int bits, const void* x, const void* y, uint32_t m, uint32_t n, uint32_t k) {
  if (n % kQmmRows || k % (2 * kGroup) || m == 0) return false;
  if (!aligned16(w.weights) || !aligned16(x) || !aligned16(y)) return false;
  if (static_cast<uint64_t>(m) * n >= (1ull << 31)) return false;
  return true;
}

size_t dense_qmm_workspace_bytes(uint32_t m, uint32_t n, uint32_t k) {
  return up256(sizeof(uint16_t) * static_cast<size_t>(m) * k) + up256(sizeof(float) * static_cast<size_t>(m) * (k / kGroup)) +
         dense_parts_bytes(m, n, k);
}

// x_prepared: rows already in the matmul's order with their group sums in sumx (x is then ignored)
static hipError_t dense_project(hipStream_t s, const mf_qtensor& w, int bits, const uint16_t* xp, const float* sumx,
                                void* y, uint32_t m, uint32_t n, uint32_t k, bool out_f32, void* parts) {
  const uint32_t ng = k / kGroup, n_win = dense_windows(k);
  const int code_bits = bits == MF_BITS_4 ? 4 : 2;
  QmmArgs d{};
  d.dense_mode = 1; d.dense_rows = m; d.top_k = 1;
  d.dense[0] = d.dense[1] = w;
  if (bits == MF_BITS_TERNARY) {  // bias = -scale: the kernel reads the scale table as bias table
    d.ternary = 1;
    d.dense[0].biases = d.dense[1].biases = w.scales;
  }
  d.x = xp; d.sumx = sumx; d.x_stride = k; d.rows = n;
  d.pair_rows = n % (2 * kQmmRows) == 0;
  const uint32_t tiles = (m + kTileTokens - 1) / kTileTokens;
  const size_t part_stride = up256(sizeof(float) * static_cast<size_t>(m) * n) / sizeof(float);
  d.ng_ld = ng;
  if (n_win == 1) {
    d.kdim = k; d.epi = out_f32 ? 1 : 2; d.out = y;
  } else {  // all windows in one launch, each writing fp32 into its own buffer
    uint32_t longest = 0;
    for (uint32_t wdx = 0; wdx < n_win; ++wdx)
      longest = std::max(longest, dense_window_start(ng, n_win, wdx + 1) - dense_window_start(ng, n_win, wdx));
    d.kdim = longest * kGroup; d.n_win = n_win; d.out_win_stride = part_stride; d.epi = 1; d.out = parts;
  }
  {
    const hipError_t e = launch_qmm(s, code_bits, d, d.pair_rows ? 2 : 1, tiles, nullptr, 0);
    if (e != hipSuccess) return e;
  }
  if (n_win > 1) {
    const size_t count = static_cast<size_t>(m) * n;
    dense_combine_kernel<<<dim3(static_cast<uint32_t>((count + 255) / 256)), dim3(256), 0, s>>>(
        static_cast<const float*>(parts), n_win, part_stride, y, count, out_f32 ? 1 : 0);
    return hipGetLastError();
  }
  return hipSuccess;
}

hipError_t launch_dense_qmm(hipStream_t s, const mf_qtensor& w, int bits, const uint16_t* x, void* y, uint32_t m,
                            uint32_t n, uint32_t k, bool out_f32, void* workspace) {
  uint8_t* base = static_cast<uint8_t*>(workspace);
  uint16_t* xp = reinterpret_cast<uint16_t*>(base);
  float* sumx = reinterpret_cast<float*>(base + up256(sizeof(uint16_t) * static_cast<size_t>(m) * k));
  void* parts = reinterpret_cast<uint8_t*>(sumx) + up256(sizeof(float) * static_cast<size_t>(m) * (k / kGroup));
  const hipError_t e = launch_prep_rows(s, x, xp, sumx, static_cast<size_t>(m) * k);
  if (e != hipSuccess) return e;
  return dense_project(s, w, bits, xp, sumx, y, m, n, k, out_f32, parts);
}

// The block form of the shared expert / dense SwiGLU MLP: gate and up in one launch with the SwiGLU epilogue
// (gate and up narrowed first, dequant_int4.metal:240-245), then the down projection.
bool dense_mlp_takes(const mf_qtensor& gate, const mf_qtensor& up, const mf_qtensor& down, const void* x,
                     const void* y, const void* scratch, uint32_t d, uint32_t f, uint32_t t) {
  if (d % kQmmRows || f % kQmmRows || t == 0) return false;
  return aligned16(gate.weights) && aligned16(up.weights) && aligned16(down.weights) && aligned16(x) && aligned16(y) &&
         aligned16(scratch) && static_cast<uint64_t>(t) * std::max(d, f) < (1ull << 31);
}

size_t dense_mlp_scratch_bytes(uint32_t d, uint32_t f, uint32_t t) {
  return up256(sizeof(uint16_t) * static_cast<size_t>(t) * f) + up256(sizeof(uint16_t) * static_cast<size_t>(t) * d) +
         up256(sizeof(float) * static_cast<size_t>(t) * (d / kGroup)) + up256(sizeof(float) * static_cast<size_t>(t) * (f / kGroup)) +
         std::max(dense_parts_bytes(t, d, f), dense_gate_up_parts_bytes(t, f, d));  // (the two uses follow one another)
}

hipError_t launch_dense_mlp(hipStream_t s, const mf_qtensor& gate, const mf_qtensor& up, const mf_qtensor& down,
                            int bits, const uint16_t* x, uint16_t* y, uint32_t d, uint32_t f, uint32_t t, void* scratch) {
  uint8_t* base = static_cast<uint8_t*>(scratch);
  uint16_t* act = reinterpret_cast<uint16_t*>(base);
  base += up256(sizeof(uint16_t) * static_cast<size_t>(t) * f);
  uint16_t* xp = reinterpret_cast<uint16_t*>(base);
  base += up256(sizeof(uint16_t) * static_cast<size_t>(t) * d);
  float* sumx = reinterpret_cast<float*>(base);
  base += up256(sizeof(float) * static_cast<size_t>(t) * (d / kGroup));
  float* sum_act = reinterpret_cast<float*>(base);
  base += up256(sizeof(float) * static_cast<size_t>(t) * (f / kGroup));
  hipError_t e = launch_prep_rows(s, x, xp, sumx, static_cast<size_t>(t) * d);
  if (e != hipSuccess) return e;
  const int code_bits = bits == MF_BITS_4 ? 4 : 2;
  QmmArgs q{};
  q.dense_mode = 1; q.dense_rows = t; q.top_k = 1; q.narrow = 1;
  q.dense[0] = gate; q.dense[1] = up;
  if (bits == MF_BITS_TERNARY) {
    q.ternary = 1;
    q.dense[0].biases = gate.scales;
    q.dense[1].biases = up.scales;
  }
  q.x = xp; q.sumx = sumx; q.x_stride = d; q.rows = f; q.kdim = d; q.epi = 0; q.out = act;
  const uint32_t gu_win = dense_gate_up_windows(d);
  if (gu_win > 1) {
    // few rows (or a K too long for one launch's scale tables): the contraction in windows, both projections as
    // fp32 per window, then one pass that adds the windows, activates and sums the groups
    const uint32_t ng = d / kGroup;
    const size_t part_stride = up256(sizeof(float) * static_cast<size_t>(t) * f) / sizeof(float);
    float* pg = reinterpret_cast<float*>(base);
    float* pu = pg + part_stride * gu_win;
    uint32_t longest = 0;
    for (uint32_t wdx = 0; wdx < gu_win; ++wdx)
      longest = std::max(longest, dense_window_start(ng, gu_win, wdx + 1) - dense_window_start(ng, gu_win, wdx));
    q.ng_ld = ng; q.kdim = longest * kGroup; q.n_win = gu_win; q.out_win_stride = part_stride;
    q.epi = 1; q.out = pg; q.out2 = pu;
    e = launch_qmm(s, code_bits, q, 2, (t + kTileTokens - 1) / kTileTokens, nullptr, 0);
    if (e != hipSuccess) return e;
    const size_t chunks = static_cast<size_t>(t) * f / 8;
    dense_swiglu_combine_kernel<<<dim3(static_cast<uint32_t>((chunks + 255) / 256)), dim3(256), 0, s>>>(
        pg, pu, gu_win, part_stride, act, sum_act, chunks, 0.0f);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  } else {
    e = launch_qmm(s, code_bits, q, 2, (t + kTileTokens - 1) / kTileTokens, nullptr, 0);
    if (e != hipSuccess) return e;
    e = launch_prep_rows(s, act, nullptr, sum_act, static_cast<size_t>(t) * f);  // the activations are in matmul order already
    if (e != hipSuccess) return e;
  }
  return dense_project(s, down, bits, act, sum_act, y, t, d, f, false, base);
}

// entries of the tile list: every live expert may end in a partial tile; a multiple of 8
uint32_t prefill_tile_slots(const mf_moe_config& c, uint32_t t) {
  const size_t pairs = static_cast<size_t>(t) * c.top_k;
  const size_t n = std::min<size_t>(c.num_experts, pairs) + pairs / kTileTokens + 1;
  return static_cast<uint32_t>((n + 7) / 8 * 8);
}

// workspace carve-up of one prefill layer call
struct PrefillWs {
  float* logits; uint32_t* idx; float* w; uint32_t* counts; uint32_t* offsets; uint32_t* starts;
  uint32_t* n_tiles; uint32_t* status; Tile* tiles; mf_pair* sorted; uint16_t* acts; float* partials;
  uint16_t* sact; uint16_t* hs; uint16_t* gate;
  uint16_t* xp; float* sum_x; float* sum_acts; float* sum_sact;
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
  const size_t max_tiles = prefill_tile_slots(c, t);
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
  p.xp = static_cast<uint16_t*>(take(sizeof(uint16_t) * static_cast<size_t>(t) * c.d));
  p.sum_x = static_cast<float*>(take(sizeof(float) * static_cast<size_t>(t) * (c.d / kGroup)));
  p.sum_acts = static_cast<float*>(take(sizeof(float) * pairs * (c.f / kGroup)));
  p.sum_sact = static_cast<float*>(take(sizeof(float) * static_cast<size_t>(t) * (std::max<uint32_t>(c.shared_f, 64) / kGroup)));
  p.bytes = pos;
  return p;
}

size_t prefill_workspace_bytes(const mf_moe_config& c, uint32_t t) {
  return prefill_carve(c, t, nullptr).bytes;
}

bool prefill_supported(const mf_moe_config& c) {
  if (c.bits != MF_BITS_4 && c.bits != MF_BITS_2 && c.bits != MF_BITS_TERNARY) return false;
  if (c.shared_f && c.shared_bits != MF_BITS_4) return false;
  if (c.gate_group_size == 32) return false;  // the matmul's tables hold one entry per 64 weights
  if (c.d % kQmmRows || c.f % kQmmRows || (c.shared_f % kQmmRows)) return false;
  if (c.d > 8192 || c.f > 8192 || c.shared_f > 8192) return false;
  return true;
}

struct RaggedOnly {
  const mf_pair* sorted;    // [t * top_k] by (expert, token, rank)
  const uint32_t* counts;   // [num_experts]
  float* partials;          // [t * top_k, d] fp32, row token * top_k + rank
};
hipError_t launch_prefill_layer(hipStream_t s, const mf_moe& h, const mf_moe_layer_weights& w,
                                const uint16_t* x, uint32_t t, uint16_t* y, void* workspace,
                                uint32_t* out_idx, float* out_w, const RaggedOnly* ragged);

// The routed experts alone over a grouping the caller holds (sorted pairs + per-expert counts):
// PrefillGroupedRoutedMoE.encodeStreamedBatched.  Runs the layer call's matmul launches and stops
// before the un-permute; the per-route results go to the caller's fp32 buffer.
hipError_t launch_ragged_qmm(hipStream_t s, const mf_moe& h, const void* expert_base, size_t expert_stride,
                             const mf_expert_offsets& off, const uint16_t* x, const mf_pair* sorted,
                             const uint32_t* counts, uint32_t t, float* partials, void* workspace) {
  RaggedOnly r{sorted, counts, partials};
  mf_moe_layer_weights w{};
  w.expert_base = expert_base;
  w.expert_stride = expert_stride;
  w.offsets = off;
  return launch_prefill_layer(s, h, w, x, t, nullptr, workspace, nullptr, nullptr, &r);
}

hipError_t launch_unpermute(hipStream_t s, const mf_moe_config& c, const float* partials, const float* w,
                            const uint32_t* idx, const uint16_t* residual, uint32_t t, uint16_t* y) {
  const size_t n4 = static_cast<size_t>(t) * c.d / 4;
  if (!n4) return hipSuccess;
  prefill_reduce_kernel<false><<<dim3(static_cast<uint32_t>((n4 + 255) / 256)), dim3(256), 0, s>>>(
      partials, w, idx, residual, nullptr, y, t, c.top_k, c.d, c.num_experts, static_cast<int>(c.maple_rounding));
  return hipGetLastError();
}

hipError_t launch_prefill_layer(hipStream_t s, const mf_moe& h, const mf_moe_layer_weights& w,
                                const uint16_t* x, uint32_t t, uint16_t* y, void* workspace,
                                uint32_t* out_idx, float* out_w, const RaggedOnly* ragged) {
  const mf_moe_config& cfg_in = h.cfg;
  mf_moe_config c = cfg_in;
  if (ragged) c.shared_f = 0;  // the routed experts only
  PrefillWs ws = prefill_carve(cfg_in, t, workspace);
  // the caller's routing outputs, when given, are the routing buffers of the whole call
  if (out_idx) ws.idx = out_idx;
  if (out_w) ws.w = out_w;
  hipError_t e;
#define MF_TRY(call) do { e = (call); if (e != hipSuccess) return e; } while (0)
  const size_t pairs = static_cast<size_t>(t) * c.top_k;
  const uint32_t max_tiles = prefill_tile_slots(c, t);
  bool x_prepared = false, fused_group = false;
  if (ragged) {
    // the caller's grouping: its per-expert counts are a one-chunk histogram for the scan that lays
    // out the tile list (the runs start at 0 in expert order, as mf_moe_group writes them)
    uint32_t* hist = h.ws.group_tmp + 2048;
    uint32_t* bad = hist + static_cast<size_t>(kGroupChunks) * MF_MAX_EXPERTS;
    ws.status = h.ws.group_tmp + 3 * 512;  // the word mf_moe_group_status reads
    ragged_begin_kernel<<<dim3(1), dim3(MF_MAX_EXPERTS), 0, s>>>(ragged->counts, c.num_experts, hist, bad);
    const uint32_t check_wgs = static_cast<uint32_t>(std::min<size_t>((pairs + 255) / 256, 2048));
    ragged_check_kernel<<<dim3(std::max(check_wgs, 1u)), dim3(256), 0, s>>>(ragged->sorted, ragged->counts, c.num_experts,
                                                                           t, c.top_k, bad);
    MF_TRY(hipGetLastError());
    group_scan_kernel<<<dim3(1), dim3(MF_MAX_EXPERTS), 0, s>>>(hist, 1, c.num_experts, ws.counts, ws.offsets, ws.starts,
                                                               ws.tiles, max_tiles, ws.n_tiles, bad, ws.status, 1);
    MF_TRY(hipGetLastError());
    ws.sorted = const_cast<mf_pair*>(ragged->sorted);
    ws.partials = ragged->partials;
  } else {
    if (w.router_w) {  // else the routing in out_idx / out_w is the caller's
      RouterTail tail{};
      tail.xp = ws.xp;
      tail.w_sg = c.shared_f && !w.w_sg_q8.weights ? w.w_sg : nullptr;  // (an 8-bit gate row: its own launch below)
      tail.sums = ws.sum_x;
      tail.gate = ws.gate;
      MF_TRY(launch_prefill_router(s, w.router_w, x, c.num_experts, c.d, t, c.d, ws.logits, &tail));
      x_prepared = tail.xp != nullptr;
      fused_group = topk_group_takes(t) && pairs > kGroupOnePairs;
      if (fused_group)
        MF_TRY(launch_topk_group(s, ws.logits, t, c.top_k, c.num_experts, c.router_mode, ws.idx, ws.w, ws.counts,
                                 ws.offsets, ws.starts, ws.sorted, ws.tiles, max_tiles, ws.n_tiles, ws.status,
                                 h.ws.group_tmp));
      else MF_TRY(launch_topk(s, ws.logits, c.num_experts, c.top_k, t, c.router_mode, ws.idx, ws.w));
    }
    if (!fused_group)
      MF_TRY(launch_group(s, ws.idx, ws.w, t, c.top_k, c.num_experts, ws.counts, ws.offsets, ws.starts,
                          ws.sorted, ws.tiles, max_tiles, ws.n_tiles, ws.status, h.ws.group_tmp + 2048));
  }

  const bool gate_q8 = c.shared_f && w.w_sg_q8.weights;
  const bool want_gate = c.shared_f && (w.w_sg || gate_q8);
  if (x_prepared) {
    // the router launch has prepared x (and the gate's logits) on the side
  } else if (want_gate && !gate_q8) {  // one pass over x: matmul order, group sums and the shared gate's logits
    prep_x_gate_kernel<<<dim3((t + 3) / 4), dim3(256), 0, s>>>(x, ws.xp, ws.sum_x, w.w_sg, ws.gate, t, c.d);
    MF_TRY(hipGetLastError());
  } else {
    MF_TRY(launch_prep_rows(s, x, ws.xp, ws.sum_x, static_cast<size_t>(t) * c.d));
  }
  // the scalar gate stored as an 8-bit row (RealForwardRunner.swift:2925-2941): one wave per token, the
  // bits of mf_gemv(MF_BITS_8) -- and of the decode launch
  if (gate_q8) MF_TRY(launch_gemv(s, w.w_sg_q8, MF_BITS_8, x, ws.gate, 1, c.d, t, false));

  QmmArgs q{};
  // the routed experts' blobs: the pool in the matmul's order when the caller built one (mf_moe_tile_experts)
  q.expert_base = static_cast<const uint8_t*>(w.expert_tiled ? w.expert_tiled : w.expert_base);
  q.tiled = w.expert_tiled != nullptr;
  q.expert_stride = w.expert_stride;
  q.sorted = ws.sorted;
  q.tiles = ws.tiles;
  q.n_tiles = ws.n_tiles;
  q.top_k = c.top_k;
  q.limit = c.swiglu_limit;
  // ternary experts are 2-bit codes whose bias is -scale: the kernels take the scale table as bias table
  const int code_bits = c.bits == MF_BITS_4 ? 4 : 2;
  const bool ternary = c.bits == MF_BITS_TERNARY;
  q.ternary = ternary;
  q.maple = static_cast<int>(c.maple_rounding);
  // the (4-bit) shared expert rides in the routed launches when the routed experts are 4-bit too;
  // otherwise its matmuls are launches of their own
  const bool shared_rides = c.shared_f && code_bits == 4;
  if (h.trace && h.trace_bytes >= 64) {  // stage stamps of the routed gate/up matmul
    q.trace = h.trace;
    q.trace_items = static_cast<uint32_t>(std::min<size_t>(h.trace_bytes / 64, 1u << 30));
  }
  // The shared expert's two matmuls ride in the routed launches of the same phase.
  QmmArgs d{};
  const uint32_t dense_tiles = c.shared_f ? (t + kTileTokens - 1) / kTileTokens : 0;
  if (c.shared_f) {
    d.dense_mode = 1; d.dense_rows = t; d.top_k = c.top_k; d.narrow = 1;
    d.dense[0] = w.shared_gate; d.dense[1] = w.shared_up;
    d.x = ws.xp; d.sumx = ws.sum_x; d.x_stride = c.d; d.rows = c.shared_f; d.kdim = c.d; d.epi = 0; d.out = ws.sact;
  }
  // phase 1: routed gate/up -> acts [pair, F]; shared gate/up -> sact [token, Fs]
  q.w_off[0] = w.offsets.gate_w; q.s_off[0] = w.offsets.gate_s; q.b_off[0] = ternary ? w.offsets.gate_s : w.offsets.gate_b;
  q.w_off[1] = w.offsets.up_w; q.s_off[1] = w.offsets.up_s; q.b_off[1] = ternary ? w.offsets.up_s : w.offsets.up_b;
  q.x = ws.xp; q.sumx = ws.sum_x; q.x_stride = c.d; q.gather = 1; q.rows = c.f; q.kdim = c.d; q.epi = 0;
  q.out = ws.acts;
  // The shared expert's work items (whole 64-row tiles, the longest of the launch) go first: a short batch
  // leaves workgroup slots over, and up to about 4096 tokens the launch ends sooner with them out of the way
  // (Qwen shape, layer: 2048 tokens 280.5 -> 274.5 us, 1024 tokens 191 -> 187 us, 4096 tokens 506 -> 503 us;
  // at 16 384 tokens they are better last, 1763 against 1776 us, where they fill the holes of the last round).
  const bool dense_first = shared_rides && pairs <= 32768;
  if (dense_first) MF_TRY(launch_qmm(s, code_bits, d, 2, dense_tiles, &q, max_tiles));
  else MF_TRY(launch_qmm(s, code_bits, q, 2, max_tiles, shared_rides ? &d : nullptr, dense_tiles));
  if (c.shared_f && !shared_rides) MF_TRY(launch_qmm(s, 4, d, 2, dense_tiles, nullptr, 0));
  // phase 2: routed down -> fp32 partials [token*K+rank, D]; shared down -> hs [token, D]
  q.w_off[0] = w.offsets.down_w; q.s_off[0] = w.offsets.down_s; q.b_off[0] = ternary ? w.offsets.down_s : w.offsets.down_b;
  q.w_off[1] = q.s_off[1] = q.b_off[1] = 0;
  // Per-route results as bf16 numbers where the rounding rule narrows them anyway before they meet their
  // weights -- MapleMoE's (maple_moe.metal:258), or on request (mf_moe_set_prefill_route_rounding; the
  // reference's prefill keeps 16-bit per-route results, prefill.metal:817-819, 644-651): half the bytes
  // written here and read by the reduce.  The caller's buffer of a ragged call stays fp32.
  const bool narrow_routes = !ragged && (c.maple_rounding || h.narrow_routes);
  q.x = ws.acts; q.sumx = ws.sum_acts; q.x_stride = c.f; q.gather = 0; q.rows = c.d; q.kdim = c.f;
  q.epi = narrow_routes ? 3 : 1; q.out = ws.partials;
  q.limit = 0.0f;
  q.trace = nullptr;
  q.pair_rows = c.d % (2 * kQmmRows) == 0;
  if (c.shared_f) {
    d.dense[0] = w.shared_down;
    d.x = ws.sact; d.sumx = ws.sum_sact; d.x_stride = c.shared_f; d.rows = c.d; d.kdim = c.shared_f; d.epi = 2; d.out = ws.hs;
    d.pair_rows = q.pair_rows;
  }
  const bool kres_q = kres_takes(q, pairs), kres_d = c.shared_f && kres_takes(d, t);
  {
    // group sums of the activation rows for qmm_kernel (qmm_kres_kernel sums the rows it stages itself);
    // routes past the last tile's count were never written: only pairs rows exist, all written
    const bool q_ring = !(kres_q && (!shared_rides || (kres_d && d.kdim == q.kdim)));
    const bool d_ring = c.shared_f && !(kres_d && (!shared_rides || (kres_q && d.kdim == q.kdim)));
    if (q_ring || d_ring)
      MF_TRY(launch_prep_rows(s, q_ring ? ws.acts : nullptr, nullptr, ws.sum_acts, q_ring ? pairs * c.f : 0,
                              d_ring ? ws.sact : nullptr, nullptr, ws.sum_sact,
                              d_ring ? static_cast<size_t>(t) * c.shared_f : 0));
  }
  if (shared_rides) {
    if (kres_q && kres_d && d.kdim == q.kdim) {
      if (dense_first) MF_TRY(launch_qmm_kres(s, 4, d, dense_tiles, &q, max_tiles));
      else MF_TRY(launch_qmm_kres(s, 4, q, max_tiles, &d, dense_tiles));
    } else if (dense_first) MF_TRY(launch_qmm(s, 4, d, q.pair_rows ? 2 : 1, dense_tiles, &q, max_tiles));
    else MF_TRY(launch_qmm(s, 4, q, q.pair_rows ? 2 : 1, max_tiles, &d, dense_tiles));
  } else {
    if (kres_q) MF_TRY(launch_qmm_kres(s, code_bits, q, max_tiles, nullptr, 0));
    else MF_TRY(launch_qmm(s, code_bits, q, q.pair_rows ? 2 : 1, max_tiles, nullptr, 0));
    if (c.shared_f) {
      if (kres_d) MF_TRY(launch_qmm_kres(s, 4, d, dense_tiles, nullptr, 0));
      else MF_TRY(launch_qmm(s, 4, d, d.pair_rows ? 2 : 1, dense_tiles, nullptr, 0));
    }
  }
  if (ragged) return hipSuccess;  // the per-route results are the caller's: mf_moe_unpermute reduces them
  const uint16_t* hs = nullptr;
  const uint16_t* gate = nullptr;
  if (c.shared_f) {
    hs = ws.hs;
    if (want_gate) gate = ws.gate;
  }
  const size_t n4 = static_cast<size_t>(t) * c.d / 4;
  const dim3 reduce_grid(static_cast<uint32_t>((n4 + 255) / 256));
  if (narrow_routes)
    prefill_reduce_kernel<true><<<reduce_grid, dim3(256), 0, s>>>(ws.partials, ws.w, ws.idx, hs, gate, y, t, c.top_k, c.d,
                                                                  c.num_experts, static_cast<int>(c.maple_rounding));
  else
    prefill_reduce_kernel<false><<<reduce_grid, dim3(256), 0, s>>>(ws.partials, ws.w, ws.idx, hs, gate, y, t, c.top_k, c.d,
                                                                   c.num_experts, static_cast<int>(c.maple_rounding));
  MF_TRY(hipGetLastError());
#undef MF_TRY
  return hipSuccess;
}

hipError_t launch_prefill_layer(hipStream_t s, const mf_moe& h, const mf_moe_layer_weights& w,
                                const uint16_t* x, uint32_t t, uint16_t* y, void* workspace,
                                uint32_t* out_idx, float* out_w) {
  return launch_prefill_layer(s, h, w, x, t, y, workspace, out_idx, out_w, nullptr);
}

}  // namespace mf
