// The fused decode layer: one launch per MoE layer.
//
// A grid of one 1024-thread workgroup per CU stays resident for the whole layer
// and runs three stages separated by two grid-wide barriers:
//
//   A  router logits (one wave per expert row), the scalar shared gate w_sg.x,
//      shared-expert gate/up/activation rows
//   --- barrier 1: logits, gate and shared activations are complete ---
//      every workgroup recomputes the (cheap, deterministic) top-k itself
//   B  routed gate/up/activation rows of the K selected experts of every token,
//      shared-expert down rows (-> gated h1)
//   --- barrier 2: routed activations and h1 are complete ---
//   C  down rows: K waves of a workgroup take the K slots of one group of output
//      rows, weight them, and one thread per row adds them to h1 in rank order.
//
// Nothing but the router decides which weights are read, so stage C's packed
// codes are requested right after a workgroup has arrived at barrier 2: their
// HBM latency hides behind the wait.
//
// The barriers need every workgroup of the grid to be resident at once; the
// launcher never asks for more workgroups than CUs and the kernel needs a whole
// CU (1024 threads, <= 128 VGPRs).  Waits are bounded: a barrier that does not
// complete within kSpinLimit polls sets the status word and lets the grid drain.
// (The logits buffer is read 16 bytes at a time: [T, E] fp32 with E % 4 == 0.)
#include "mf_device.h"
#include "mf_internal.h"
#include "mf_router.h"

#pragma clang fp contract(off)

namespace mf {

constexpr uint32_t kFusedThreads = 1024;
constexpr uint32_t kFusedWaves = kFusedThreads / kWave;
constexpr uint32_t kSpinLimit = 1u << 22;  // x ~50 ns per poll

template <int BITS> struct Chunk {
  uint4 codes;
  float s, b;
};

template <int BITS>
__device__ __forceinline__ Chunk<BITS> load_chunk(const uint8_t* wrow, const uint16_t* srow,
                                                  const uint16_t* brow, uint32_t e0) {
  Chunk<BITS> c;
  c.codes = load_codes16<true>(wrow + static_cast<size_t>(e0) * Store<BITS>::kBits / 8);
  load_scale_bias<BITS>(srow, brow, e0, c.s, c.b);
  return c;
}

// lane partial of one row of N elements against x (16-byte aligned bf16);
// `first` may carry the already loaded chunk of the first step.  AGENT_X: x was
// written by other workgroups during this launch.
template <int BITS, bool AGENT_X>
__device__ __forceinline__ float row_partial(const uint8_t* wrow, const uint16_t* srow,
                                             const uint16_t* brow, const uint16_t* x, uint32_t N,
                                             uint32_t sub, uint32_t lpr, bool have_first,
                                             const Chunk<BITS>& first) {
  constexpr uint32_t EPL = Fmt<BITS>::kElemsPer16B;
  float acc = 0.0f;
  for (uint32_t e0 = sub * EPL; e0 < N; e0 += lpr * EPL) {
    const Chunk<BITS> c = (have_first && e0 == sub * EPL) ? first
                                                           : load_chunk<BITS>(wrow, srow, brow, e0);
    float dot, sum;
    const XSlice<BITS> xs = load_xslice<BITS, AGENT_X ? kXAgent : kXAligned>(x + e0);
    dot = codes_dot<BITS>(c.codes, xs);
    sum = xs.sum;
    acc = __builtin_fmaf(c.s, dot, acc);
    acc = __builtin_fmaf(c.b, sum, acc);
  }
  return acc;
}

// gate and up rows of one projection pair sharing the x loads
template <int BITS>
__device__ __forceinline__ void gate_up_partial(const uint8_t* gw, const uint16_t* gs,
                                                const uint16_t* gb, const uint8_t* uw,
                                                const uint16_t* us, const uint16_t* ub,
                                                const uint16_t* x, uint32_t N, uint32_t sub,
                                                uint32_t lpr, float& ga, float& ua) {
  constexpr uint32_t EPL = Fmt<BITS>::kElemsPer16B;
  ga = ua = 0.0f;
  for (uint32_t e0 = sub * EPL; e0 < N; e0 += lpr * EPL) {
    const Chunk<BITS> g = load_chunk<BITS>(gw, gs, gb, e0);
    const Chunk<BITS> u = load_chunk<BITS>(uw, us, ub, e0);
    const XSlice<BITS> xs = load_xslice<BITS, kXAligned>(x + e0);
    const float gd = codes_dot<BITS>(g.codes, xs), ud = codes_dot<BITS>(u.codes, xs);
    const float sum = xs.sum;
    ga = __builtin_fmaf(g.s, gd, ga);
    ga = __builtin_fmaf(g.b, sum, ga);
    ua = __builtin_fmaf(u.s, ud, ua);
    ua = __builtin_fmaf(u.b, sum, ua);
  }
}

struct FusedArgs {
  const uint16_t* router_w;
  const uint8_t* expert_base;
  size_t expert_stride;
  mf_expert_offsets off;
  mf_qtensor sg, su, sd;
  const uint16_t* w_sg;
  const uint16_t* x;
  uint16_t* y;
  uint16_t* hidden;
  uint32_t* out_idx;
  float* out_w;
  float* logits;
  uint16_t* acts;
  uint16_t* shared_act;
  uint16_t* shared_y;
  float* gate;  // bf16-rounded scalar shared gate per token
  unsigned long long* trace;  // phase timestamps, 8 per workgroup, or nullptr
  uint32_t* sync;  // kMaxGrid flags of barrier 1, kMaxGrid of barrier 2, status word
  uint32_t D, F, E, K, T, Fs;
  int router_mode;
  float limit;
};

// Grid barrier without read-modify-write atomics (256 workgroups adding to one
// counter serialise at the memory side for microseconds): every workgroup owns
// one flag per barrier and raises it by one each time it arrives; a waiter
// polls all flags with one 16-byte device-coherent load per lane until none
// lags behind its own.  Flags only ever count up, so nothing has to be reset
// between launches (HIP-graph replay safe).  Exchanged data is written with
// device-coherent stores that are acknowledged before the flag is raised.
constexpr uint32_t kMaxGrid = 512;  // flags per barrier
constexpr uint32_t kSyncFlags1 = 0, kSyncFlags2 = kMaxGrid, kSyncStatus = 2 * kMaxGrid;

__device__ __forceinline__ void grid_arrive(uint32_t* flags, uint32_t target) {
  wait_stores();
  __syncthreads();
  if (threadIdx.x == 0) store_u32_agent(&flags[blockIdx.x], target);
}

__device__ __forceinline__ void grid_wait(const uint32_t* flags, uint32_t target, uint32_t G,
                                          uint32_t* status) {
  if (threadIdx.x < kWave) {
    const uint32_t lane = threadIdx.x;
    uint32_t spins = 0;
    for (;;) {
      bool ok = true;
      for (uint32_t b = 0; b < G; b += 4 * kWave) {
        const uint32_t i = b + 4 * lane;
        const uint4 f = load_u32x4_agent(flags + i);
        ok = ok && (i + 0 >= G || static_cast<int32_t>(f.x - target) >= 0) &&
             (i + 1 >= G || static_cast<int32_t>(f.y - target) >= 0) &&
             (i + 2 >= G || static_cast<int32_t>(f.z - target) >= 0) &&
             (i + 3 >= G || static_cast<int32_t>(f.w - target) >= 0);
      }
      if (__all(ok)) break;
      __builtin_amdgcn_s_sleep(1);
      if (++spins > kSpinLimit) {
        if (lane == 0) store_u32_agent(status, 1u);
        break;
      }
    }
  }
  __syncthreads();
}

// phase trace: the shader clock at every stage boundary, thread 0 of each workgroup
__device__ __forceinline__ void trace_mark(const FusedArgs& a, uint32_t slot) {
  if (a.trace && threadIdx.x == 0) a.trace[blockIdx.x * 8 + slot] = wall_clock64();
}

template <int BITS, int SBITS>
__global__ __launch_bounds__(kFusedThreads) void fused_decode_kernel(const FusedArgs a) {
  __shared__ uint32_t s_idx[MF_MAX_TOKENS * MF_MAX_TOPK];
  __shared__ float s_w[MF_MAX_TOKENS * MF_MAX_TOPK];
  __shared__ float s_v[kFusedWaves][kWave];
  __shared__ float s_lg[MF_MAX_TOKENS][MF_MAX_EXPERTS];

  const uint32_t lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const uint32_t G = gridDim.x, wg = blockIdx.x;
  const uint32_t gw = wv * G + wg;  // consecutive work items land on different CUs
  const uint32_t total_waves = kFusedWaves * G;
  const uint32_t D = a.D, F = a.F, E = a.E, K = a.K, T = a.T, Fs = a.Fs;

  // this launch's barrier targets: one above the workgroup's own flags
  const uint32_t target1 =
      __hip_atomic_load(&a.sync[kSyncFlags1 + wg], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
  const uint32_t target2 =
      __hip_atomic_load(&a.sync[kSyncFlags2 + wg], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
  trace_mark(a, 0);
  // ------------------------------------------------------------- stage A
  {
    const uint32_t lpr_log2 = Fs ? lanes_per_row_log2_dev(D, Fmt<SBITS>::kElemsPer16B) : 0;
    const uint32_t lpr = 1u << lpr_log2, rpw = 64u >> lpr_log2;
    const uint32_t n_router = E * T;
    const uint32_t n_gate = (Fs && a.w_sg) ? T : 0;
    const uint32_t srg = Fs ? (Fs + rpw - 1) / rpw : 0;
    const uint32_t n_items = n_router + n_gate + T * srg;
    for (uint32_t item = gw; item < n_items; item += total_waves) {
      if (item < n_router) {
        const uint32_t tok = item / E, row = item % E;
        const float v = dot_bf16_row(a.router_w + static_cast<size_t>(row) * D,
                                     a.x + static_cast<size_t>(tok) * D, D, lane, true);
        if (lane == 0) store_f32_agent(&a.logits[item], v);
      } else if (item < n_router + n_gate) {
        const uint32_t tok = item - n_router;
        const float v = dot_bf16_row(a.w_sg, a.x + static_cast<size_t>(tok) * D, D, lane, true);
        if (lane == 0) store_f32_agent(&a.gate[tok], round_bf16(v));
      } else {
        const uint32_t it = item - n_router - n_gate;
        const uint32_t tok = it / srg;
        const uint32_t row = (it % srg) * rpw + (lane >> lpr_log2);
        const uint32_t sub = lane & (lpr - 1);
        const bool ok = row < Fs;
        const size_t r = ok ? row : 0;
        const uint32_t ng = D / kGroup;
        const size_t rb = static_cast<size_t>(D) * Store<SBITS>::kBits / 8;
        float ga = 0.0f, ua = 0.0f;
        if (ok)
          gate_up_partial<SBITS>(static_cast<const uint8_t*>(a.sg.weights) + r * rb,
                                 a.sg.scales + r * ng, a.sg.biases + r * ng,
                                 static_cast<const uint8_t*>(a.su.weights) + r * rb,
                                 a.su.scales + r * ng, a.su.biases + r * ng,
                                 a.x + static_cast<size_t>(tok) * D, D, sub, lpr, ga, ua);
        const float g = group_sum(ga, static_cast<int>(lpr));
        const float u = group_sum(ua, static_cast<int>(lpr));
        if (ok && sub == 0) {
          // dequant_int4.metal:240-245: gate and up narrowed before the activation
          const float rg = round_bf16(g), ru = round_bf16(u);
          store_u16_agent(&a.shared_act[static_cast<size_t>(tok) * Fs + row],
                          f_to_bf16(mf_silu(rg) * ru));
        }
      }
    }
  }
  trace_mark(a, 1);
  grid_arrive(a.sync + kSyncFlags1, target1);
  grid_wait(a.sync + kSyncFlags1, target1, G, a.sync + kSyncStatus);
  trace_mark(a, 2);

  // ------------------------------------------------------------- top-k
  if (wv < T) {  // stage the token's logits in LDS: 4 consecutive experts per lane and load
    for (uint32_t e0 = 4 * lane; e0 < E; e0 += 4 * kWave) {
      const uint4 v = load_u32x4_agent(a.logits + static_cast<size_t>(wv) * E + e0);
      s_lg[wv][e0] = __uint_as_float(v.x);
      if (e0 + 1 < E) s_lg[wv][e0 + 1] = __uint_as_float(v.y);
      if (e0 + 2 < E) s_lg[wv][e0 + 2] = __uint_as_float(v.z);
      if (e0 + 3 < E) s_lg[wv][e0 + 3] = __uint_as_float(v.w);
    }
  }
  __syncthreads();
  if (wv < T) {
    if (a.router_mode == 0) topk_select_fast(s_lg[wv], E, K, s_idx + wv * K, s_w + wv * K, lane);
    else topk_wave(s_lg[wv], E, K, a.router_mode, s_idx + wv * K, s_w + wv * K, lane);
  }
  __syncthreads();
  if (wg == 0 && threadIdx.x < T * K) {
    if (a.out_idx) a.out_idx[threadIdx.x] = s_idx[threadIdx.x];
    if (a.out_w) a.out_w[threadIdx.x] = s_w[threadIdx.x];
  }

  trace_mark(a, 3);
  // ------------------------------------------------------------- stage B
  {
    const uint32_t lpr_log2 = lanes_per_row_log2_dev(D, Fmt<BITS>::kElemsPer16B);
    const uint32_t lpr = 1u << lpr_log2, rpw = 64u >> lpr_log2;
    const uint32_t rgf = (F + rpw - 1) / rpw;
    const uint32_t n_routed = T * K * rgf;
    const uint32_t slpr_log2 = Fs ? lanes_per_row_log2_dev(Fs, Fmt<SBITS>::kElemsPer16B) : 0;
    const uint32_t slpr = 1u << slpr_log2, srpw = 64u >> slpr_log2;
    const uint32_t sdrg = Fs ? (D + srpw - 1) / srpw : 0;
    const uint32_t n_items = n_routed + T * sdrg;
    for (uint32_t item = gw; item < n_items; item += total_waves) {
      if (item < n_routed) {
        const uint32_t pair = item / rgf;
        const uint32_t row = (item % rgf) * rpw + (lane >> lpr_log2);
        const uint32_t sub = lane & (lpr - 1);
        const bool ok = row < F;
        const uint32_t expert = s_idx[pair];
        if (expert >= E) {
          if (ok && sub == 0) store_u16_agent(&a.acts[static_cast<size_t>(pair) * F + row], 0);
          continue;
        }
        const uint8_t* blob = a.expert_base + static_cast<size_t>(expert) * a.expert_stride;
        const size_t r = ok ? row : 0;
        const uint32_t ng = D / kGroup;
        const size_t rb = static_cast<size_t>(D) * Store<BITS>::kBits / 8;
        float ga = 0.0f, ua = 0.0f;
        if (ok)
          gate_up_partial<BITS>(
              blob + a.off.gate_w + r * rb,
              reinterpret_cast<const uint16_t*>(blob + a.off.gate_s) + r * ng,
              reinterpret_cast<const uint16_t*>(blob + a.off.gate_b) + r * ng,
              blob + a.off.up_w + r * rb,
              reinterpret_cast<const uint16_t*>(blob + a.off.up_s) + r * ng,
              reinterpret_cast<const uint16_t*>(blob + a.off.up_b) + r * ng,
              a.x + static_cast<size_t>(pair / K) * D, D, sub, lpr, ga, ua);
        float g = group_sum(ga, static_cast<int>(lpr));
        float u = group_sum(ua, static_cast<int>(lpr));
        if (ok && sub == 0) {
          if (a.limit > 0.0f) {  // moe.metal:27-34
            g = fminf(g, a.limit);
            u = fminf(fmaxf(u, -a.limit), a.limit);
          }
          store_u16_agent(&a.acts[static_cast<size_t>(pair) * F + row], f_to_bf16(mf_silu(g) * u));
        }
      } else {
        const uint32_t it = item - n_routed;
        const uint32_t tok = it / sdrg;
        const uint32_t row = (it % sdrg) * srpw + (lane >> slpr_log2);
        const uint32_t sub = lane & (slpr - 1);
        const bool ok = row < D;
        const size_t r = ok ? row : 0;
        const uint32_t ng = Fs / kGroup;
        const size_t rb = static_cast<size_t>(Fs) * Store<SBITS>::kBits / 8;
        float part = 0.0f;
        if (ok)
          part = row_partial<SBITS, true>(static_cast<const uint8_t*>(a.sd.weights) + r * rb,
                                    a.sd.scales + r * ng, a.sd.biases + r * ng,
                                    a.shared_act + static_cast<size_t>(tok) * Fs, Fs, sub, slpr,
                                    false, Chunk<SBITS>{});
        const float v = group_sum(part, static_cast<int>(slpr));
        if (ok && sub == 0) {
          uint16_t h = f_to_bf16(v);  // dequant_int4.metal:177-180
          if (a.w_sg) {               // utility.metal:49-59
            const float gt = load_f32_agent(&a.gate[tok]);
            h = f_to_bf16(bf16_to_f(h) / (1.0f + mf_exp(-gt)));
          }
          store_u16_agent(&a.shared_y[static_cast<size_t>(tok) * D + row], h);
        }
      }
    }
  }

  // ------------------------------------------------------------- stage C
  const uint32_t lpr_log2 = lanes_per_row_log2_dev(F, Fmt<BITS>::kElemsPer16B);
  const uint32_t lpr = 1u << lpr_log2, rpw = 64u >> lpr_log2;
  const uint32_t rg_per_tok = (D + rpw - 1) / rpw;
  const uint32_t units = T * rg_per_tok;
  const uint32_t ub = kFusedWaves / K;  // units a workgroup handles per round
  const uint32_t rounds = (units + G * ub - 1) / (G * ub);
  const uint32_t unit_local = wv / K, slot = wv % K;
  const uint32_t sub = lane & (lpr - 1);
  const uint32_t ng = F / kGroup;
  const size_t rb = static_cast<size_t>(F) * Store<BITS>::kBits / 8;

  trace_mark(a, 4);
  grid_arrive(a.sync + kSyncFlags2, target2);
  // request round 0's codes while the barrier completes
  Chunk<BITS> pre{};
  bool have_pre = false;
  {
    const uint32_t unit = wg * ub + unit_local;
    if (unit_local < ub && unit < units) {
      const uint32_t tok = unit / rg_per_tok;
      const uint32_t row = (unit % rg_per_tok) * rpw + (lane >> lpr_log2);
      const uint32_t expert = s_idx[tok * K + slot];
      if (row < D && expert < E && sub * Fmt<BITS>::kElemsPer16B < F) {
        const uint8_t* blob = a.expert_base + static_cast<size_t>(expert) * a.expert_stride;
        pre = load_chunk<BITS>(blob + a.off.down_w + row * rb,
                               reinterpret_cast<const uint16_t*>(blob + a.off.down_s) + row * ng,
                               reinterpret_cast<const uint16_t*>(blob + a.off.down_b) + row * ng,
                               sub * Fmt<BITS>::kElemsPer16B);
        have_pre = true;
      }
    }
  }
  grid_wait(a.sync + kSyncFlags2, target2, G, a.sync + kSyncStatus);
  trace_mark(a, 5);

  for (uint32_t round = 0; round < rounds; ++round) {
    const uint32_t unit = (round * G + wg) * ub + unit_local;
    const bool active = unit_local < ub && unit < units;
    if (active) {
      const uint32_t tok = unit / rg_per_tok;
      const uint32_t row = (unit % rg_per_tok) * rpw + (lane >> lpr_log2);
      const uint32_t pair = tok * K + slot;
      const uint32_t expert = s_idx[pair];
      const bool ok = row < D;
      float part = 0.0f;
      if (ok && expert < E) {
        const uint8_t* blob = a.expert_base + static_cast<size_t>(expert) * a.expert_stride;
        part = row_partial<BITS, true>(blob + a.off.down_w + row * rb,
                                 reinterpret_cast<const uint16_t*>(blob + a.off.down_s) + row * ng,
                                 reinterpret_cast<const uint16_t*>(blob + a.off.down_b) + row * ng,
                                 a.acts + static_cast<size_t>(pair) * F, F, sub, lpr,
                                 have_pre && round == 0, pre);
      }
      const float v = group_sum(part, static_cast<int>(lpr));
      if (sub == 0) s_v[wv][lane >> lpr_log2] = s_w[pair] * v;  // moe.metal:1262
    }
    __syncthreads();
    if (threadIdx.x < ub * rpw) {
      const uint32_t ul = threadIdx.x / rpw, rr = threadIdx.x % rpw;
      const uint32_t u2 = (round * G + wg) * ub + ul;
      if (u2 < units) {
        const uint32_t tok = u2 / rg_per_tok;
        const uint32_t row = (u2 % rg_per_tok) * rpw + rr;
        if (row < D) {
          const size_t o = static_cast<size_t>(tok) * D + row;
          float acc = Fs ? bf16_to_f(load_u16_agent(&a.shared_y[o])) : 0.0f;  // residual first (moe.metal:1265)
          for (uint32_t k = 0; k < K; ++k)
            if (s_idx[tok * K + k] < E) acc = acc + s_v[ul * K + k][rr];
          const uint16_t yb = f_to_bf16(acc);
          a.y[o] = yb;
          if (a.hidden)  // residual_add_fp16, utility.metal:83-92
            a.hidden[o] = f_to_bf16(bf16_to_f(a.hidden[o]) + bf16_to_f(yb));
        }
      }
    }
    __syncthreads();
  }

  trace_mark(a, 6);
}

bool fused_supported(const mf_moe_config& c, const mf_moe_layer_weights& w, const void* x,
                     const void* y, const void* hidden) {
  if (c.num_experts % 4 != 0) return false;  // logits are staged 4 at a time
  const bool combo = (c.bits == MF_BITS_4 && (!c.shared_f || c.shared_bits == MF_BITS_4)) ||
                     (c.bits == MF_BITS_2 && (!c.shared_f || c.shared_bits == MF_BITS_4 ||
                                              c.shared_bits == MF_BITS_2)) ||
                     (c.bits == MF_BITS_TERNARY && (!c.shared_f || c.shared_bits == MF_BITS_4));
  if (!combo || c.d % 8 != 0) return false;
  const uint32_t offs = w.offsets.gate_w | w.offsets.up_w | w.offsets.down_w;
  if (!aligned16(w.expert_base) || w.expert_stride % 16 || offs % 16) return false;
  if (!aligned16(w.router_w) || !aligned16(x) || !aligned16(y)) return false;
  if (hidden && !aligned16(hidden)) return false;
  if (c.shared_f) {
    if (!aligned16(w.shared_gate.weights) || !aligned16(w.shared_up.weights) ||
        !aligned16(w.shared_down.weights))
      return false;
    if (w.w_sg && !aligned16(w.w_sg)) return false;
  }
  return true;
}

hipError_t launch_fused_decode(hipStream_t s, const mf_moe& h, const mf_moe_layer_weights& w,
                               const uint16_t* x, uint32_t t, uint16_t* y, uint16_t* hidden,
                               uint32_t* out_idx, float* out_w) {
  const mf_moe_config& c = h.cfg;
  FusedArgs a{};
  a.router_w = w.router_w;
  a.expert_base = static_cast<const uint8_t*>(w.expert_base);
  a.expert_stride = w.expert_stride;
  a.off = w.offsets;
  a.sg = w.shared_gate;
  a.su = w.shared_up;
  a.sd = w.shared_down;
  a.w_sg = c.shared_f ? w.w_sg : nullptr;
  a.x = x;
  a.y = y;
  a.hidden = hidden;
  a.out_idx = out_idx;
  a.out_w = out_w;
  a.logits = h.ws.logits;
  a.acts = h.ws.acts;
  a.shared_act = h.ws.shared_act;
  a.shared_y = h.ws.shared_y;
  a.gate = reinterpret_cast<float*>(h.ws.gate);
  a.sync = h.ws.sync;
  a.trace = h.trace;
  a.D = c.d;
  a.F = c.f;
  a.E = c.num_experts;
  a.K = c.top_k;
  a.T = t;
  a.Fs = c.shared_f;
  a.router_mode = c.router_mode;
  a.limit = c.swiglu_limit;
  const dim3 grid(static_cast<uint32_t>(h.ctx->num_cu)), block(kFusedThreads);
#define MF_FUSED(B, SB) fused_decode_kernel<B, SB><<<grid, block, 0, s>>>(a)
  if (c.bits == MF_BITS_4) MF_FUSED(kBits4, kBits4);
  else if (c.bits == MF_BITS_2 && c.shared_f && c.shared_bits == MF_BITS_2) MF_FUSED(kBits2, kBits2);
  else if (c.bits == MF_BITS_2) MF_FUSED(kBits2, kBits4);
  else MF_FUSED(kBitsTernary, kBits4);
#undef MF_FUSED
  return hipGetLastError();
}

}  // namespace mf
