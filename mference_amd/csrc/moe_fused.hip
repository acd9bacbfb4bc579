// The fused decode layer: one launch per MoE layer.
//
// A grid of one 1024-thread workgroup per CU stays resident for the whole layer:
//
//   A  router logits (one wave per expert row), the scalar shared gate w_sg.x,
//      shared-expert gate/up/activation rows
//      -> every workgroup gathers the logits and selects the top-k itself (cheap and
//         deterministic: rank counting over the logits in LDS, all waves)
//   B  routed gate/up/activation rows of the K selected experts of every token
//   C  per token: the shared expert's down rows of this workgroup's output rows
//      (-> gated h1, kept in LDS), then the routed down rows: K waves take the K
//      slots of one group of output rows, weight them, and one thread per row
//      adds them to h1 in rank order.
//
// Workgroups exchange three small vectors through HBM: logits, shared
// activations, routed activations.  There is no grid barrier.  Every exchanged
// word carries the launch's epoch as a tag (fp32 logits: a 32-bit tag beside the
// value; bf16 activations: a 16-bit tag above the value), producers write them
// with device-coherent stores and go on, consumers poll the data itself with
// device-coherent loads into LDS until every tag they need is current.  This
// costs one store propagation plus about one load round trip per exchange
// (0.55 - 0.65 us between two workgroups, on the same XCD or not);
// a barrier built on a flag or counter costs a store acknowledgement, the flag's
// own propagation, a poll and then the data load.  The epoch is a per-workgroup counter
// in the workspace that every workgroup raises by one per launch, so all
// workgroups agree on it without talking, nothing is reset between launches
// and a captured HIP graph can replay the launch.  One token slot of the
// activation buffers (epoch mod 8, if unused by this launch) is re-tagged per
// launch so that no stale word is ever older than 8 launches: a 16-bit tag can
// never alias.
//
// Producers write whole 64-byte pieces.  Work is dealt in chunks of consecutive rows, one chunk
// per workgroup, the waves' results meet in LDS and one store instruction writes the chunk:
// when neighbouring words of a line are written through by different workgroups (different
// XCDs), the partial-line writes serialise in the memory system and the gather of a 16 KiB
// vector by all workgroups takes 3.3 us instead of 1.4 us (2 KiB: 2.4 against 1.2 us).
//
// Nothing but the router decides which weights are read, so stage C's packed
// codes are requested before the routed activations are polled: their HBM
// latency hides behind the wait.
//
// Consumers spin on data other workgroups produce, so every workgroup of the
// grid has to be resident at once: the launcher never asks for more workgroups
// than CUs and the kernel needs a whole CU (1024 threads, <= 128 VGPRs).  Waits
// are bounded: a poll that does not complete within kSpinLimit tries sets the
// status word, the workgroup writes NaN to the output rows it owns and the grid drains.
#include "mf_device.h"
#include "mf_internal.h"
#include "mf_router.h"

#pragma clang fp contract(off)

namespace mf {

constexpr uint32_t kFusedThreads = 1024;
constexpr uint32_t kFusedWaves = kFusedThreads / kWave;
constexpr uint32_t kSpinLimit = 1u << 17;  // x ~0.6 us per poll
constexpr uint32_t kRouterChunk = 8;       // router rows per workgroup chunk: 8 tagged logits = 64 bytes
constexpr uint32_t kRankCountLimit = 1u << 18;  // T * E * E up to which the top-k counts ranks
constexpr uint32_t kRankWords = 2048;      // ... and T * E it may have then
constexpr uint32_t kMaxH1 = 2048;          // output rows of one token a workgroup may own

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

// lane partial of one row of N elements against x (16-byte aligned bf16, global
// or LDS); `first` may carry the already loaded chunk of the first step.
template <int BITS>
__device__ __forceinline__ float row_partial(const uint8_t* wrow, const uint16_t* srow,
                                             const uint16_t* brow, const uint16_t* x, uint32_t N,
                                             uint32_t sub, uint32_t lpr, bool have_first,
                                             const Chunk<BITS> first) {
  constexpr uint32_t EPL = Fmt<BITS>::kElemsPer16B;
  float acc = 0.0f;
  for (uint32_t e0 = sub * EPL; e0 < N; e0 += lpr * EPL) {
    // plain scalars, not a struct select: the prefetched chunk must stay in registers
    uint4 codes = first.codes;
    float s = first.s, b = first.b;
    if (!(have_first && e0 == sub * EPL)) {
      codes = load_codes16<true>(wrow + static_cast<size_t>(e0) * Store<BITS>::kBits / 8);
      load_scale_bias<BITS>(srow, brow, e0, s, b);
    }
    const XSlice<BITS> xs = load_xslice<BITS, kXAligned>(x + e0);
    acc = __builtin_fmaf(s, codes_dot<BITS>(codes, xs), acc);
    acc = __builtin_fmaf(b, xs.sum, acc);
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
    const XRaw<BITS> xr = load_xraw<BITS>(x + e0);
    issue_fence();
    const XSlice<BITS> xs = make_xslice<BITS>(xr);
    const float gd = codes_dot<BITS>(g.codes, xs), ud = codes_dot<BITS>(u.codes, xs);
    ga = __builtin_fmaf(g.s, gd, ga);
    ga = __builtin_fmaf(g.b, xs.sum, ga);
    ua = __builtin_fmaf(u.s, ud, ua);
    ua = __builtin_fmaf(u.b, xs.sum, ua);
  }
}

// The lane slices of x a routed row meets (XSlice: permuted pairs + their sum) depend on the token
// only, so a workgroup builds them once in LDS instead of once per row: slice sl of token t keeps
// its pairs as 16-byte blocks xq[(t * kQ + q) * n_sl + sl] (neighbouring lanes read neighbouring
// blocks) and its sum at xsum[t * n_sl + sl].
template <int BITS>
__device__ __forceinline__ void store_xslice_lds(uint4* xq, float* xsum, uint32_t t, uint32_t n_sl, uint32_t sl,
                                                 const XSlice<BITS>& xs) {
  constexpr uint32_t kQ = XSlice<BITS>::kPairs / 4;
#pragma unroll
  for (uint32_t q = 0; q < kQ; ++q)
    xq[(t * kQ + q) * n_sl + sl] = make_uint4(xs.p[4 * q], xs.p[4 * q + 1], xs.p[4 * q + 2], xs.p[4 * q + 3]);
  xsum[t * n_sl + sl] = xs.sum;
}
template <int BITS>
__device__ __forceinline__ XSlice<BITS> load_xslice_lds(const uint4* xq, const float* xsum, uint32_t t, uint32_t n_sl,
                                                        uint32_t sl) {
  constexpr uint32_t kQ = XSlice<BITS>::kPairs / 4;
  XSlice<BITS> xs;
#pragma unroll
  for (uint32_t q = 0; q < kQ; ++q) {
    const uint4 v = xq[(t * kQ + q) * n_sl + sl];
    xs.p[4 * q] = v.x; xs.p[4 * q + 1] = v.y; xs.p[4 * q + 2] = v.z; xs.p[4 * q + 3] = v.w;
  }
  xs.sum = xsum[t * n_sl + sl];
  return xs;
}

struct FusedArgs {
  const uint16_t* router_w;
  const uint8_t* expert_base;
  size_t expert_stride;
  mf_expert_offsets off;
  mf_qtensor sg, su, sd;
  const uint16_t* w_sg;
  // the scalar gate as 8-bit affine codes [1, D] with its scale / bias tables (null: w_sg, or no gate)
  const uint8_t* gq_w;
  const uint16_t* gq_s;
  const uint16_t* gq_b;
  const uint16_t* x;
  uint16_t* y;
  uint16_t* hidden;
  // NORM instances: x is made inside the launch from hidden (+ delta) -- see the kernel's prologue
  const uint16_t* delta;   // [T, D] added to hidden first, or null
  const uint16_t* norm_w;  // [D] RMSNorm weight
  float norm_eps;
  uint32_t xn_off;         // byte offset of the normalised rows [T, D] in LDS
  uint32_t* out_idx;
  float* out_w;
  // exchange buffers (workspace of the handle)
  unsigned long long* t_logits;  // [T, E] (value bits | epoch << 32)
  uint32_t* t_sact;              // [MF_MAX_TOKENS, Fs + 4] (bf16 | tag << 16); word Fs = gate
  uint32_t* t_acts;              // [MF_MAX_TOKENS, K, F]
  uint32_t* epoch;               // one counter per workgroup
  uint32_t* status;
  unsigned long long* trace;     // phase timestamps, 8 per workgroup, or nullptr
  uint32_t D, F, E, K, T, Fs;
  int router_mode;
  float limit;
  int maple;  // MapleMoE's rounding points (mf_moe_config::maple_rounding)
  uint32_t stage_words;  // words of the LDS staging area
  int xprep;             // the routed rows read x from LDS, permuted and summed once per workgroup
};

__device__ __forceinline__ void store_u64_agent(unsigned long long* p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// a bounded wait ran out: the status word tells the host, the LDS flag makes this workgroup
// write NaN instead of a result
__device__ __forceinline__ void give_up(uint32_t* status, uint32_t* s_fail, uint32_t lane) {
  if (lane == 0) {
    store_u32_agent(status, 1u);
    *s_fail = 1u;
  }
}

// phase trace: the 100 MHz wall clock at every stage boundary, thread 0 of each workgroup
__device__ __forceinline__ void trace_mark(const FusedArgs& a, uint32_t slot) {
  if (a.trace && threadIdx.x == 0) a.trace[blockIdx.x * 8 + slot] = wall_clock64();
}

// Shape specialisation (the reference's FC_MOE_D / FC_MOE_F / FC_MOE_TOP_K function
// constants, moe.metal:13-16): a StaticShape turns the dimensions it names into
// compile-time constants (kDyn leaves one to the arguments), which unrolls the row
// loops and removes most of the control flow -- the launch executes each
// instruction once per wave, so code size is instruction-fetch latency.
// RuntimeShape reads every dimension from the arguments and handles everything else.
// kGiven: the routing is the caller's (written by an earlier launch, e.g. a family router): the kernel
// has no router rows, no logits exchange and no top-k, and reads indices and weights instead of
// writing them.  A compile-time property, so the kernels that route keep their code as it is.
constexpr uint32_t kDyn = 0xFFFFFFFFu;  // a dimension read from the arguments
template <bool GIVEN = false>
struct RuntimeShapeT {
  static constexpr bool kStatic = false, kGiven = GIVEN;
  static constexpr uint32_t D = kDyn, F = kDyn, E = kDyn, K = kDyn, T = kDyn, Fs = kDyn;
  static constexpr uint32_t Mode = kDyn, Maple = kDyn, NoLimit = 0, XPrep = kDyn;
};
using RuntimeShape = RuntimeShapeT<false>;
// MODE_ / MAPLE_: the router mode and the Maple rounding flag as literals (kDyn: from the arguments);
// NOLIMIT_ = 1: the layer has no SwiGLU clamp; XPREP_ = 1: the x slices are kept in LDS.
template <uint32_t D_, uint32_t F_, uint32_t E_, uint32_t K_, uint32_t T_, uint32_t Fs_, bool GIVEN = false,
          uint32_t MODE_ = kDyn, uint32_t MAPLE_ = kDyn, uint32_t NOLIMIT_ = 0, uint32_t XPREP_ = kDyn>
struct StaticShape {
  static constexpr bool kStatic = D_ != kDyn && F_ != kDyn && E_ != kDyn && K_ != kDyn && T_ != kDyn && Fs_ != kDyn;
  static constexpr bool kGiven = GIVEN;
  static constexpr uint32_t D = D_, F = F_, E = E_, K = K_, T = T_, Fs = Fs_;
  static constexpr uint32_t Mode = MODE_, Maple = MAPLE_, NoLimit = NOLIMIT_, XPrep = XPREP_;
};

// rows one wave takes per step when a row has n elements (compile-time twin of
// 64 >> lanes_per_row_log2_dev)
constexpr uint32_t static_rows_per_wave(uint32_t n, uint32_t elems_per_lane) {
  uint32_t need = (n + elems_per_lane - 1) / elems_per_lane, lanes = 1;
  while (lanes < need && lanes < 64) lanes *= 2;
  return 64u / lanes;
}

template <int BITS, int SBITS, class S, bool NORM = false>
__global__ __launch_bounds__(kFusedThreads) void fused_decode_kernel(const FusedArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  const uint32_t D = S::D != kDyn ? S::D : a.D, F = S::F != kDyn ? S::F : a.F;
  const uint32_t E = S::E != kDyn ? S::E : a.E, K = S::K != kDyn ? S::K : a.K;
  const uint32_t T = S::T != kDyn ? S::T : a.T, Fs = S::Fs != kDyn ? S::Fs : a.Fs;
  const int router_mode = S::Mode != kDyn ? static_cast<int>(S::Mode) : a.router_mode;
  const bool maple = S::Maple != kDyn ? S::Maple != 0u : a.maple != 0;
  const float limit = S::NoLimit ? 0.0f : a.limit;
  const bool xprep = S::XPrep != kDyn ? S::XPrep != 0u : a.xprep != 0;
  // LDS carve-up (the launcher sizes it with fused_lds_bytes)
  uint32_t* s_idx = reinterpret_cast<uint32_t*>(smem);                 // [8*8]
  float* s_w = reinterpret_cast<float*>(smem + 256);                    // [8*8]
  float* s_sc = reinterpret_cast<float*>(smem + 512);                   // [8*8] selected scores
  uint32_t* s_flag = reinterpret_cast<uint32_t*>(smem + 768);           // [8] token has a non-finite logit
  uint32_t* s_fail = reinterpret_cast<uint32_t*>(smem + 800);           // a bounded wait gave up; [1]: selection fallback
  float* s_v = reinterpret_cast<float*>(smem + 1024);                   // [16][64]
  float* s_h1 = reinterpret_cast<float*>(smem + 1024 + 4096);           // [kMaxH1]
  uint32_t* s_rank = reinterpret_cast<uint32_t*>(smem + 1024 + 4096 + kMaxH1 * 4);  // [kRankWords]
  uint8_t* dyn = smem + 1024 + 4096 + kMaxH1 * 4 + kRankWords * 4;
  float* s_lg = reinterpret_cast<float*>(dyn);                          // [MF_MAX_TOKENS][E]
  uint32_t* s_sact = reinterpret_cast<uint32_t*>(dyn + MF_MAX_TOKENS * E * 4);  // [(Fs+4)/2]
  uint32_t* s_acts = s_sact + (((Fs + 4) / 2 + 3) & ~3u);               // [K*F/2], 16-byte aligned
  uint32_t* s_stage = s_acts + ((K * F / 2 + 3) & ~3u);                 // chunk staging, a.stage_words
  const uint32_t sact_stride = Fs + 4;  // words per token in t_sact

  const uint32_t lane = threadIdx.x & 63;
  // the wave index as a scalar: what derives from it (rows, experts, base addresses) is then
  // computed once per wave by the scalar unit instead of per lane
  const uint32_t wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t G = gridDim.x, wg = blockIdx.x;
  // x slices of the routed rows, built once per workgroup (when a.xprep)
  constexpr uint32_t kEPL = Fmt<BITS>::kElemsPer16B;
  const uint32_t n_sl = D / kEPL;  // slices per token (the last partial slice, if any, is not kept)
  uint4* s_xq = reinterpret_cast<uint4*>(s_stage + a.stage_words);
  float* s_xsum = reinterpret_cast<float*>(s_xq + T * (XSlice<BITS>::kPairs / 4) * n_sl);

  // The launch epoch comes out of device memory (a captured graph replays the launch with the same
  // arguments) and is first needed when a result is tagged.  The load is requested here; every
  // user takes the value through epoch_now(), whose empty asm statement keeps the compiler from
  // waiting for it any earlier -- in particular not before the first rows' loads are out.
  uint32_t epoch_lane_off = 0;
  asm volatile("" : "+v"(epoch_lane_off));
  const uint32_t epoch_raw =
      __hip_atomic_load(&a.epoch[wg] + epoch_lane_off, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  auto epoch_now = [&]() __attribute__((always_inline)) {
    uint32_t e = epoch_raw;
    asm volatile("" : "+v"(e));
    return e + 1u;
  };
  trace_mark(a, 0);
  // NORM: the step in front of the layer inside the launch (RealForwardRunner.swift:2799-2808: hidden += delta,
  // x = RMSNorm(hidden) * weight).  Every workgroup makes the normalised rows for itself, in LDS, with the
  // instruction order of residual_rmsnorm_kernel (256 threads per row, element i + 256 j on thread i, fmaf
  // chain, neighbour-first butterfly, (s0 + s1) + (s2 + s3)), so x has the bits of that launch; everything
  // below reads x from LDS.  hidden itself is written once, at the end, by the workgroup that owns the
  // element: bf16(bf16(hidden + delta) + y).  A workgroup that other workgroups do not wait for (no row of
  // stages A and B) may read hidden while it is being written: its x then is of no consequence.
  const uint16_t* xin = a.x;
  // (NORM) the first router row of a wave: its weights are requested ahead of the norm, which has a memory
  // round trip of its own to wait for -- rows of up to 2048 elements, four chunks per lane
  uint4 pre_w[4];
  bool pre_router = false;
  if constexpr (NORM && !S::kGiven) {
    const uint32_t row = wg * kRouterChunk + wv;
    pre_router = D <= 2048 && D % 8 == 0 && wv < kRouterChunk && row < E * T;
    if (pre_router) {
      const uint16_t* wr = a.router_w + static_cast<size_t>(row % E) * D;
#pragma unroll
      for (int sidx = 0; sidx < 4; ++sidx) {
        const uint32_t c = lane + sidx * kWave;
        pre_w[sidx] = c < D / 8 ? load_x8<true>(wr + c * 8) : make_uint4(0, 0, 0, 0);
      }
    }
  }
  if constexpr (NORM) {
    uint16_t* s_xn = reinterpret_cast<uint16_t*>(smem + a.xn_off);
    float* s_part = s_v;  // [token][4 waves of its row]; s_v is free until stage C
    // The rows come in as 16-byte pieces, every piece once per workgroup (piece c on thread c % 1024), with
    // the matching piece of delta and of the weights in the same round trip; bf16(hidden + delta) goes to
    // LDS, the sums read it from there in the norm kernel's order, and each piece's owner scales it in
    // place.  (Element by element from global memory, the delta loads sat behind a branch each: eight
    // round trips in a row, 3.9 us before the first row could start.)
    constexpr uint32_t kPc = MF_MAX_TOKENS * 4096 / 8 / kFusedThreads;  // pieces per thread at most
    const uint32_t ppr = D / 8, n_pc = T * ppr;
    const uint16_t* dsrc = a.delta ? a.delta : a.hidden;  // (always a valid address: no branch around the load)
    const bool has_delta = a.delta != nullptr;
    uint4 hv[kPc], nv[kPc];
#pragma unroll
    for (uint32_t p = 0; p < kPc; ++p) {
      const uint32_t c = threadIdx.x + kFusedThreads * p;
      if (c < n_pc) {
        const uint4 h4 = load_x8<true>(a.hidden + static_cast<size_t>(c) * 8);
        const uint4 d4 = load_x8<true>(dsrc + static_cast<size_t>(c) * 8);
        nv[p] = load_x8<true>(a.norm_w + static_cast<size_t>(c % ppr) * 8);
        const uint32_t hw[4] = {h4.x, h4.y, h4.z, h4.w}, dw[4] = {d4.x, d4.y, d4.z, d4.w};
        uint32_t o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint16_t lo = f_to_bf16(bf16_to_f(static_cast<uint16_t>(hw[q] & 0xffffu)) +
                                        bf16_to_f(static_cast<uint16_t>(dw[q] & 0xffffu)));
          const uint16_t hi = f_to_bf16(bf16_to_f(static_cast<uint16_t>(hw[q] >> 16)) +
                                        bf16_to_f(static_cast<uint16_t>(dw[q] >> 16)));
          o[q] = has_delta ? (static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16)) : hw[q];
        }
        hv[p] = make_uint4(o[0], o[1], o[2], o[3]);
        *reinterpret_cast<uint4*>(s_xn + static_cast<size_t>(c) * 8) = hv[p];
      }
    }
    __syncthreads();
    const uint32_t grp = threadIdx.x >> 8, ti = threadIdx.x & 255u;
    for (uint32_t tok0 = 0; tok0 < T; tok0 += 4) {
      const uint32_t tok = tok0 + grp;
      float acc = 0.0f;
      if (tok < T) {
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j) {  // D <= 4096
          const uint32_t i = ti + 256u * j;
          if (i < D) {
            const float v = bf16_to_f(s_xn[static_cast<size_t>(tok) * D + i]);
            acc = __builtin_fmaf(v, v, acc);
          }
        }
      }
      acc = wave_sum(acc);
      if (lane == 0 && tok < T) s_part[4 * tok + (wv & 3u)] = acc;
    }
    __syncthreads();
#pragma unroll
    for (uint32_t p = 0; p < kPc; ++p) {
      const uint32_t c = threadIdx.x + kFusedThreads * p;
      if (c < n_pc) {
        const uint32_t tok = c / ppr;
        const float total = (s_part[4 * tok] + s_part[4 * tok + 1]) + (s_part[4 * tok + 2] + s_part[4 * tok + 3]);
        const float inv = 1.0f / __builtin_sqrtf(total / static_cast<float>(D) + a.norm_eps);
        const uint32_t hw[4] = {hv[p].x, hv[p].y, hv[p].z, hv[p].w}, nw4[4] = {nv[p].x, nv[p].y, nv[p].z, nv[p].w};
        uint32_t o[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint16_t lo = f_to_bf16(bf16_to_f(static_cast<uint16_t>(hw[q] & 0xffffu)) * inv *
                                        bf16_to_f(static_cast<uint16_t>(nw4[q] & 0xffffu)));
          const uint16_t hi = f_to_bf16(bf16_to_f(static_cast<uint16_t>(hw[q] >> 16)) * inv *
                                        bf16_to_f(static_cast<uint16_t>(nw4[q] >> 16)));
          o[q] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
        }
        *reinterpret_cast<uint4*>(s_xn + static_cast<size_t>(c) * 8) = make_uint4(o[0], o[1], o[2], o[3]);
      }
    }
    __syncthreads();
    xin = s_xn;
    trace_mark(a, 7);
  }
  // rank counting selects the top-k when it is cheap enough, else one wave per token sorts
  const bool rank_count = !S::kGiven && T * E * E <= kRankCountLimit && T * E <= kRankWords;
  // Who does what while the logits are on their way: the top waves poll for them (n_poll waves),
  // the waves below those build the x slices, the bottom waves have the rows of stage A.
  const uint32_t n2 = S::kGiven ? 0 : T * E / 2;  // 16-byte pieces of tagged logits (E % 4 == 0)
  const uint32_t n_poll = n2 ? ((n2 + kWave - 1) / kWave < 8 ? (n2 + kWave - 1) / kWave : 8) : 0;
  const uint32_t n_xw = (T * n_sl + kWave - 1) / kWave < kFusedWaves - n_poll - 4
                            ? (T * n_sl + kWave - 1) / kWave : kFusedWaves - n_poll - 4;

  // ------------------------------------------------------------- stage A
  // Router rows are on the critical path and their logits are gathered by everybody: they go in
  // chunks of kRouterChunk consecutive rows to the first workgroups (a wave each; the chunk
  // leaves as one 64-byte store).  The shared expert's rows and the scalar-gate rows are needed
  // much later; they are dealt one at a time over the waves of the other workgroups (their
  // dot products are vector-ALU work: spread thin, they cost no workgroup more than a row or two).
  {
    const uint32_t lpr_log2 = Fs ? lanes_per_row_log2_dev(D, Fmt<SBITS>::kElemsPer16B) : 0;
    const uint32_t lpr = 1u << lpr_log2, rpw = 64u >> lpr_log2;
    const uint32_t n_rows_r = S::kGiven ? 0 : E * T;
    const uint32_t n_rc = (n_rows_r + kRouterChunk - 1) / kRouterChunk;
    unsigned long long* s_stage64 = reinterpret_cast<unsigned long long*>(s_stage);
    for (uint32_t ci = wg; ci < n_rc; ci += G) {
      const uint32_t row = ci * kRouterChunk + wv;
      if (wv < kRouterChunk && row < n_rows_r) {
        const uint32_t tok = row / E, e = row % E;
        float v;
        if (NORM && pre_router && ci == wg) {  // the weights are here already: dot_bf16_row's products in its order
          const uint16_t* xr = xin + static_cast<size_t>(tok) * D;
          float acc = 0.0f;
#pragma unroll
          for (int sidx = 0; sidx < 4; ++sidx) {
            const uint32_t c = lane + sidx * kWave;
            if (c < D / 8) {
              const uint4 xv = load_x8<true>(xr + c * 8), wq = pre_w[sidx];
              acc = __builtin_fmaf(bf16_lo(wq.x), bf16_lo(xv.x), acc);
              acc = __builtin_fmaf(bf16_hi(wq.x), bf16_hi(xv.x), acc);
              acc = __builtin_fmaf(bf16_lo(wq.y), bf16_lo(xv.y), acc);
              acc = __builtin_fmaf(bf16_hi(wq.y), bf16_hi(xv.y), acc);
              acc = __builtin_fmaf(bf16_lo(wq.z), bf16_lo(xv.z), acc);
              acc = __builtin_fmaf(bf16_hi(wq.z), bf16_hi(xv.z), acc);
              acc = __builtin_fmaf(bf16_lo(wq.w), bf16_lo(xv.w), acc);
              acc = __builtin_fmaf(bf16_hi(wq.w), bf16_hi(xv.w), acc);
            }
          }
          v = wave_sum(acc);
        } else {
          v = dot_bf16_row(a.router_w + static_cast<size_t>(e) * D, xin + static_cast<size_t>(tok) * D, D, lane, true);
        }
        if (lane == 0) s_stage64[wv] = (static_cast<unsigned long long>(epoch_now()) << 32) | __float_as_uint(v);
      }
      __syncthreads();
      if (wv == 0 && lane < kRouterChunk && ci * kRouterChunk + lane < n_rows_r)
        store_u64_agent(&a.t_logits[ci * kRouterChunk + lane], s_stage64[lane]);
      if (ci + G < n_rc) __syncthreads();  // the staging words are reused
    }
    const uint32_t skip = n_rc < G ? n_rc : 0;  // workgroups [0, skip) had router rows
    const uint32_t n_gate = (Fs && (a.w_sg || a.gq_w)) ? T : 0;
    const uint32_t srg = Fs ? (Fs + rpw - 1) / rpw : 0;
    const uint32_t n_items = n_gate + T * srg;
    const uint32_t Gs = G - skip;
    for (uint32_t item = wg >= skip ? wv * Gs + (wg - skip) : n_items; item < n_items; item += kFusedWaves * Gs) {
      if (item < n_gate) {
        const uint32_t tok = item;
        const float v = a.gq_w ? dot_q8_row(a.gq_w, a.gq_s, a.gq_b, xin + static_cast<size_t>(tok) * D, D, lane, true)
                               : dot_bf16_row(a.w_sg, xin + static_cast<size_t>(tok) * D, D, lane, true);
        if (lane < 4)  // the gate rides behind the token's shared activations
          store_u32_agent(&a.t_sact[static_cast<size_t>(tok) * sact_stride + Fs + lane],
                          (lane == 0 ? static_cast<uint32_t>(f_to_bf16(v)) : 0u) | (epoch_now() << 16));
      } else {
        const uint32_t it = item - n_gate;
        const uint32_t srg1 = srg ? srg : 1u;  // no shared expert: this branch is never taken
        const uint32_t tok = it / srg1;
        const uint32_t row = (it % srg1) * rpw + (lane >> lpr_log2);
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
                                 xin + static_cast<size_t>(tok) * D, D, sub, lpr, ga, ua);
        const float g = group_sum(ga, static_cast<int>(lpr));
        const float u = group_sum(ua, static_cast<int>(lpr));
        if (ok && sub == 0) {
          // dequant_int4.metal:240-245: gate and up narrowed before the activation
          const float rg = round_bf16(g), ru = round_bf16(u);
          store_u32_agent(&a.t_sact[static_cast<size_t>(tok) * sact_stride + row],
                          static_cast<uint32_t>(f_to_bf16(mf_silu(rg) * ru)) | (epoch_now() << 16));
        }
      }
    }
    // the x slices of the routed rows
    if (xprep && wv + n_poll + n_xw >= kFusedWaves && wv + n_poll < kFusedWaves) {
      for (uint32_t q = (wv + n_poll + n_xw - kFusedWaves) * kWave + lane; q < T * n_sl; q += n_xw * kWave) {
        const uint32_t tok = q / n_sl, sl = q % n_sl;
        store_xslice_lds<BITS>(s_xq, s_xsum, tok, n_sl, sl,
                               load_xslice<BITS, kXAligned>(xin + static_cast<size_t>(tok) * D + sl * kEPL));
      }
    }
  }
  const uint32_t epoch = epoch_now();
  const uint32_t tag16 = epoch & 0xFFFFu;
  for (uint32_t i = threadIdx.x; i < kRankWords; i += kFusedThreads) s_rank[i] = 0u;
  if (threadIdx.x < MF_MAX_TOKENS * MF_MAX_TOPK) {
    s_idx[threadIdx.x] = 0u;
    s_sc[threadIdx.x] = -__builtin_inff();
  }
  if (threadIdx.x < MF_MAX_TOKENS + 2) s_flag[threadIdx.x] = 0u;  // + s_fail and the selection's fallback flag behind it
  {
    // keep every word of the activation buffers recently tagged (see the top)
    const uint32_t ts = epoch % MF_MAX_TOKENS;
    if (ts >= T) {
      const uint32_t gtid = wg * kFusedThreads + threadIdx.x, gthreads = G * kFusedThreads;
      for (uint32_t i = gtid * 4; i < K * F; i += gthreads * 4)  // K * F is a multiple of 64
        store_u32x4_agent(&a.t_acts[static_cast<size_t>(ts) * K * F + i], tag16 << 16);
      for (uint32_t i = gtid; i < (Fs ? sact_stride : 0); i += gthreads)
        store_u32_agent(&a.t_sact[static_cast<size_t>(ts) * sact_stride + i], tag16 << 16);
    }
  }
  trace_mark(a, 1);

  // ------------------------------------------------------- logits, top-k
  if constexpr (!S::kGiven) {
    // every lane takes two tagged logits
    if (wv + n_poll >= kFusedWaves) {
      for (uint32_t p0 = (kFusedWaves - 1 - wv) * kWave; p0 < n2; p0 += n_poll * kWave) {
        const uint32_t p = p0 + lane;
        const bool in = p < n2;
        uint4 v = make_uint4(0, epoch, 0, epoch);
        for (uint32_t spins = 0;; ++spins) {
          if (in) v = load_u32x4_agent(a.t_logits + 2 * p);
          if (__all(!in || (v.y == epoch && v.w == epoch))) break;
          if (spins > kSpinLimit) {
            give_up(a.status, s_fail, lane);
            break;
          }
          __builtin_amdgcn_s_sleep(1);
        }
        if (in) {  // rank counting wants no NaN among the scores it compares
          const bool clean = rank_count && router_mode == 0;
          s_lg[2 * p] = clean ? score_or_ninf(__uint_as_float(v.x)) : __uint_as_float(v.x);
          s_lg[2 * p + 1] = clean ? score_or_ninf(__uint_as_float(v.z)) : __uint_as_float(v.z);
        }
      }
    }
    __syncthreads();
    trace_mark(a, 2);
    if (rank_count) {
      if (router_mode != 0) {  // full softmax first: the probabilities replace the logits
        if (wv < T && !full_softmax_probs(s_lg + wv * E, s_lg + wv * E, E, lane)) {
          if (lane == 0) s_flag[wv] = 1u;  // the token routes nowhere; its scores only have to be comparable
          for (uint32_t i = lane; i < E; i += kWave) s_lg[wv * E + i] = 0.0f;
        }
        __syncthreads();
      }
      bool counted = false;
      if (topk_prefilter_fits(T, E, K, kFusedWaves)) {
        topk_prefilter(s_lg, s_rank, s_fail + 1, T, E, K, s_idx, s_sc, wv, lane);
        counted = s_fail[1] == 0u;  // else too many experts passed the prefilter: rank everything
        if (!counted) {
          __syncthreads();
          for (uint32_t i = threadIdx.x; i < kRankWords; i += kFusedThreads) s_rank[i] = 0u;
          __syncthreads();
        }
      }
      if (!counted) {
        topk_rank_count(s_lg, s_rank, T, E, wv, lane, kFusedWaves);
        __syncthreads();
        topk_rank_emit(s_lg, s_rank, T, E, K, s_idx, s_sc, threadIdx.x, kFusedThreads);
      }
      if (router_mode != 0) {  // a token with a non-finite logit routes nowhere (maple_moe.metal:62-119)
        __syncthreads();
        if (threadIdx.x < T * K && s_flag[threadIdx.x / K]) s_idx[threadIdx.x] = E;
      }
      // the routing weights follow after stage B: nothing needs them before stage C
    } else if (wv < T) {
      if (router_mode == 0) topk_select_fast(s_lg + wv * E, E, K, s_idx + wv * K, s_w + wv * K, lane);
      else topk_full_softmax_fast(s_lg + wv * E, s_lg + wv * E, E, K, s_idx + wv * K, s_w + wv * K, lane);
    }
    __syncthreads();
  } else {  // routing written by an earlier launch on the stream (a family router): read, never written
    trace_mark(a, 2);
    if (threadIdx.x < T * K) {
      s_idx[threadIdx.x] = a.out_idx[threadIdx.x];
      s_w[threadIdx.x] = a.out_w[threadIdx.x];
    }
    __syncthreads();
  }
  trace_mark(a, 3);

  // ------------------------------------------------------------- stage B
  // Every workgroup takes a run of consecutive units (rpw rows of one routed slot), its waves
  // take them in turn; gate and up sums meet in LDS, the first threads turn them into
  // activations (one exp and one division per thread instead of per wave) and the run leaves as
  // one contiguous piece.
  {
    const uint32_t lpr_log2 = lanes_per_row_log2_dev(D, kEPL);
    const uint32_t lpr = 1u << lpr_log2, rpw = 64u >> lpr_log2;
    const uint32_t rgf = (F + rpw - 1) / rpw;   // units per (token, slot)
    const uint32_t n_items = T * K * rgf;
    uint32_t per_wg = (n_items + G - 1) / G;
    per_wg = (per_wg + kFusedWaves - 1) / kFusedWaves * kFusedWaves;
    const uint32_t first = wg * per_wg;
    const uint32_t last = first + per_wg < n_items ? first + per_wg : n_items;
    float* s_gu = reinterpret_cast<float*>(s_stage);  // (gate sum, up sum) per staged row
    const uint32_t sub = lane & (lpr - 1), rloc = lane >> lpr_log2;
    const uint32_t ng = D / kGroup;
    const size_t rb = static_cast<size_t>(D) * Store<BITS>::kBits / 8;
    for (uint32_t item = first + wv; item < last; item += kFusedWaves) {
      const uint32_t pair = item / rgf;
      const uint32_t row = (item % rgf) * rpw + rloc;
      const uint32_t expert = __builtin_amdgcn_readfirstlane(s_idx[pair]);
      // A lane without a row, or a router sentinel, contributes nothing: its sums stay 0.  For 2-bit codes the
      // loads carry no branch (such a lane reads a row that exists and drops it): 29.4 -> 28.3 us on the large
      // 2-bit layer; the 4-bit layers lose 2-3 % at several token rows that way and keep the branch.
      constexpr bool kFreeLoads = BITS == kBits2;
      const bool ok = row < F && expert < E;
      const uint32_t ec = expert < E ? expert : 0u, rc = row < F ? row : 0u;
      float ga = 0.0f, ua = 0.0f;
      if (kFreeLoads || ok) {
        const uint8_t* blob = a.expert_base + static_cast<size_t>(ec) * a.expert_stride;
        const uint8_t* gw = blob + a.off.gate_w + rc * rb;
        const uint8_t* uw = blob + a.off.up_w + rc * rb;
        const uint16_t* gs = reinterpret_cast<const uint16_t*>(blob + a.off.gate_s) + static_cast<size_t>(rc) * ng;
        const uint16_t* gb = reinterpret_cast<const uint16_t*>(blob + a.off.gate_b) + static_cast<size_t>(rc) * ng;
        const uint16_t* us = reinterpret_cast<const uint16_t*>(blob + a.off.up_s) + static_cast<size_t>(rc) * ng;
        const uint16_t* ub = reinterpret_cast<const uint16_t*>(blob + a.off.up_b) + static_cast<size_t>(rc) * ng;
        const uint32_t tok = pair / K;
        for (uint32_t e0 = sub * kEPL; e0 < D; e0 += lpr * kEPL) {  // the steps of gate_up_partial
          const Chunk<BITS> gc = load_chunk<BITS>(gw, gs, gb, e0);
          const Chunk<BITS> uc = load_chunk<BITS>(uw, us, ub, e0);
          issue_fence();
          const XSlice<BITS> xs = xprep ? load_xslice_lds<BITS>(s_xq, s_xsum, tok, n_sl, e0 / kEPL)
                                          : load_xslice<BITS, kXAligned>(xin + static_cast<size_t>(tok) * D + e0);
          const float gd = codes_dot<BITS>(gc.codes, xs), ud = codes_dot<BITS>(uc.codes, xs);
          if (ok) {
            ga = __builtin_fmaf(gc.s, gd, ga);
            ga = __builtin_fmaf(gc.b, xs.sum, ga);
            ua = __builtin_fmaf(uc.s, ud, ua);
            ua = __builtin_fmaf(uc.b, xs.sum, ua);
          }
        }
      }
      const float g = group_sum(ga, static_cast<int>(lpr));
      const float u = group_sum(ua, static_cast<int>(lpr));
      if (sub == 0) {
        float* dst = s_gu + 2 * ((item - first) * rpw + rloc);
        dst[0] = g;
        dst[1] = u;
      }
    }
    __syncthreads();
    // staged row (item - first) * rpw + r is activation (item % rgf) * rpw + r of pair item / rgf
    const uint32_t n_words = first < last ? (last - first) * rpw : 0;
    for (uint32_t i = threadIdx.x; i < n_words; i += kFusedThreads) {
      const uint32_t item = first + i / rpw, row = (item % rgf) * rpw + i % rpw;
      // moe.metal:27-34, 528; maple_moe.metal:153-164
      const uint32_t word =
          static_cast<uint32_t>(routed_activation(s_gu[2 * i], s_gu[2 * i + 1], limit, maple)) | (tag16 << 16);
      if (row < F) store_u32_agent(&a.t_acts[static_cast<size_t>(item / rgf) * F + row], word);
    }
  }
  trace_mark(a, 4);
  // routing weights of token t by the wave 15 - t (rank counting left scores, not weights)
  if (rank_count && wv + T >= kFusedWaves) {
    const uint32_t tok = kFusedWaves - 1 - wv;
    const float my_score = lane < K ? s_sc[tok * K + lane] : -__builtin_inff();
    float wgt = router_mode == 0 ? topk_weight_of_rank<0>(my_score, K) : topk_weight_of_rank<1>(my_score, K);
    if (s_flag[tok]) wgt = 0.0f;  // maple_moe.metal:62-119: a non-finite logit routes nowhere
    if (lane < K) s_w[tok * K + lane] = wgt;
  }

  // ------------------------------------------------------------- stage C
  const uint32_t lpr_log2 = lanes_per_row_log2_dev(F, Fmt<BITS>::kElemsPer16B);
  const uint32_t lpr = 1u << lpr_log2, rpw = 64u >> lpr_log2;
  const uint32_t rg_per_tok = (D + rpw - 1) / rpw;  // units (groups of rpw output rows) per token
  const uint32_t ub = kFusedWaves / K;              // units a workgroup handles per round
  const uint32_t rounds = (rg_per_tok + G * ub - 1) / (G * ub);
  const uint32_t unit_local = wv / K, slot = wv % K;
  const uint32_t sub = lane & (lpr - 1);
  const uint32_t ng = F / kGroup;
  const size_t rb = static_cast<size_t>(F) * Store<BITS>::kBits / 8;
  const uint32_t rows_per_round = ub * rpw;
  // shared-expert down rows: srpw rows per wave step
  const uint32_t slpr_log2 = Fs ? lanes_per_row_log2_dev(Fs, Fmt<SBITS>::kElemsPer16B) : 0;
  const uint32_t slpr = 1u << slpr_log2, srpw = 64u >> slpr_log2;

  // Round 0's routed codes of every token after the first are requested while the token before it is
  // being summed up (a token's turn is otherwise a round trip to HBM longer).  That request has no branch
  // around it -- a lane without a row reads one that exists and drops it, and the last token requests its
  // own row again -- so that the products of the token at hand need not wait for it.  A launch that is
  // compiled for one token has none of this.
  constexpr bool kOneToken = S::T == 1;
  auto request_round0 = [&](uint32_t tok, Chunk<BITS>& c) __attribute__((always_inline)) {
    const uint32_t unit = wg * ub + unit_local;
    const uint32_t row = unit * rpw + (lane >> lpr_log2);
    const uint32_t expert = __builtin_amdgcn_readfirstlane(s_idx[tok * K + slot]);
    const uint32_t e0 = sub * Fmt<BITS>::kElemsPer16B;
    const bool live = unit_local < ub && unit < rg_per_tok && row < D && expert < E && e0 < F;
    const uint32_t ec = expert < E ? expert : 0u, rc = row < D ? row : 0u, e0c = e0 < F ? e0 : 0u;
    const uint8_t* blob = a.expert_base + static_cast<size_t>(ec) * a.expert_stride;
    c = load_chunk<BITS>(blob + a.off.down_w + rc * rb,
                         reinterpret_cast<const uint16_t*>(blob + a.off.down_s) + static_cast<size_t>(rc) * ng,
                         reinterpret_cast<const uint16_t*>(blob + a.off.down_b) + static_cast<size_t>(rc) * ng, e0c);
    return live;
  };
  Chunk<BITS> pre_next{};
  bool have_next = false;
  for (uint32_t tok = 0; tok < T; ++tok) {
    // request round 0's routed codes, then wait for what other workgroups produce
    // (the first token's request in the same branch-free form: 12.7 -> 12.35 us per Qwen-shaped layer; the
    // ternary layer, 13.5 us with the request under its conditions, read 14.5 us without them and keeps them)
    Chunk<BITS> pre = pre_next;
    bool have_pre = have_next;
    if (BITS != kBitsTernary && (kOneToken || tok == 0)) {
      have_pre = request_round0(tok, pre);
    } else if (kOneToken || tok == 0) {
      const uint32_t unit = wg * ub + unit_local;
      if (unit_local < ub && unit < rg_per_tok) {
        const uint32_t row = unit * rpw + (lane >> lpr_log2);
        const uint32_t expert = __builtin_amdgcn_readfirstlane(s_idx[tok * K + slot]);
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
    // first shared-expert down chunk of this wave, requested before the wait as well
    const uint32_t sng = Fs ? Fs / kGroup : 0;
    const size_t srb = static_cast<size_t>(Fs) * Store<SBITS>::kBits / 8;
    const uint32_t n_slots = Fs ? rounds * rows_per_round : 0;
    const uint32_t ssub = lane & (slpr - 1);
    Chunk<SBITS> spre{};
    bool have_spre = false;
    if (Fs) {
      const uint32_t i = wv * srpw + (lane >> slpr_log2);
      const uint32_t round = i / rows_per_round, in_round = i % rows_per_round;
      const uint32_t unit = (round * G + wg) * ub + in_round / rpw;
      const uint32_t row = unit * rpw + in_round % rpw;
      if (i < n_slots && unit < rg_per_tok && row < D && ssub * Fmt<SBITS>::kElemsPer16B < Fs) {
        spre = load_chunk<SBITS>(static_cast<const uint8_t*>(a.sd.weights) + row * srb,
                                 a.sd.scales + static_cast<size_t>(row) * sng,
                                 a.sd.biases + static_cast<size_t>(row) * sng,
                                 ssub * Fmt<SBITS>::kElemsPer16B);
        have_spre = true;
      }
    }
    // Gather what other workgroups produced: the routed activations [K*F] and the shared
    // activations (+ gate) [Fs (+4)], 256 words per wave step, two steps in flight.
    // The shared activations were written in stage A, long ago: when the routed words fit the
    // other waves' first poll step, the workgroup fetches the shared words first (they are there:
    // one round trip, during which the routed words are still on their way anyway) and the few
    // waves that own the shared-expert down rows compute the gated shared output h1 while the
    // rest of the workgroup polls for the routed words -- h1 leaves the critical path.
    const bool gated = a.w_sg || a.gq_w;
    const uint32_t n_a = K * F, n_s = Fs ? (gated ? Fs + 4 : Fs) : 0;
    const AgentBuf ba = make_agent_buf(a.t_acts + static_cast<size_t>(tok) * n_a);
    const AgentBuf bs = make_agent_buf(a.t_sact + static_cast<size_t>(tok) * sact_stride);
    const uint32_t want = tag16 << 16;
    // waves [w0, w0 + nw) gather words [first, first + count) of the virtual array [acts | sact]
    auto gather = [&](uint32_t first, uint32_t count, uint32_t w0, uint32_t nw) __attribute__((always_inline)) {
      const uint32_t step = nw * 4 * kWave, end = first + count;
      for (uint32_t c0 = first + (wv - w0) * 4 * kWave; c0 < end; c0 += 2 * step) {
        const uint32_t i0 = c0 + 4 * lane, i1 = i0 + step;
        const bool in0 = i0 < end, in1 = i1 < end;
        uint4 v0 = make_uint4(want, want, want, want), v1 = v0;
        for (uint32_t spins = 0;; ++spins) {
          if (in0) v0 = i0 < n_a ? load_u32x4_agentbuf(ba, i0 * 4) : load_u32x4_agentbuf(bs, (i0 - n_a) * 4);
          if (in1) v1 = i1 < n_a ? load_u32x4_agentbuf(ba, i1 * 4) : load_u32x4_agentbuf(bs, (i1 - n_a) * 4);
          const uint32_t diff = (v0.x ^ want) | (v0.y ^ want) | (v0.z ^ want) | (v0.w ^ want) |
                                (v1.x ^ want) | (v1.y ^ want) | (v1.z ^ want) | (v1.w ^ want);
          if (__all((diff >> 16) == 0)) break;
          if (spins > kSpinLimit) {
            give_up(a.status, s_fail, lane);
            break;
          }
          __builtin_amdgcn_s_sleep(1);
        }
        if (in0) {
          uint32_t* dst = i0 < n_a ? s_acts + i0 / 2 : s_sact + (i0 - n_a) / 2;
          dst[0] = __builtin_amdgcn_perm(v0.y, v0.x, 0x05040100u);
          dst[1] = __builtin_amdgcn_perm(v0.w, v0.z, 0x05040100u);
        }
        if (in1) {
          uint32_t* dst = i1 < n_a ? s_acts + i1 / 2 : s_sact + (i1 - n_a) / 2;
          dst[0] = __builtin_amdgcn_perm(v1.y, v1.x, 0x05040100u);
          dst[1] = __builtin_amdgcn_perm(v1.w, v1.z, 0x05040100u);
        }
      }
    };
    // gated shared output h1 of the output rows this workgroup owns for this token; waves
    // [0, nw) share the rows
    auto shared_rows = [&](uint32_t nw) __attribute__((always_inline)) {
      const float gate = gated ? bf16_lo(s_sact[Fs / 2]) : 0.0f;
      for (uint32_t s0 = wv * srpw; s0 < n_slots; s0 += nw * srpw) {
        const uint32_t i = s0 + (lane >> slpr_log2);  // slot of (round, unit_local, row in unit)
        const uint32_t round = i / rows_per_round, in_round = i % rows_per_round;
        const uint32_t unit = (round * G + wg) * ub + in_round / rpw;
        const uint32_t row = unit * rpw + in_round % rpw;
        const bool ok = i < n_slots && unit < rg_per_tok && row < D;
        float part = 0.0f;
        if (ok)
          part = row_partial<SBITS>(static_cast<const uint8_t*>(a.sd.weights) + row * srb,
                                    a.sd.scales + static_cast<size_t>(row) * sng,
                                    a.sd.biases + static_cast<size_t>(row) * sng,
                                    reinterpret_cast<const uint16_t*>(s_sact), Fs, ssub, slpr,
                                    have_spre && s0 == wv * srpw, spre);
        const float v = group_sum(part, static_cast<int>(slpr));
        if (ok && ssub == 0) {
          float h = round_bf16(v);  // dequant_int4.metal:177-180
          if (gated) h = round_bf16(h / (1.0f + mf_exp(-gate)));  // utility.metal:49-59
          s_h1[i] = h;
        }
      }
    };
    // waves that own shared rows when the rows are dealt one wave step each
    const uint32_t sh_waves = Fs ? (n_slots + srpw - 1) / srpw : 0;
    // (the first token only: the later tokens' routed words have arrived as well by then, and one fetch of
    // everything is a trip past L2 shorter than two behind each other)
    const bool split = tok == 0 && Fs && sh_waves <= 4 && n_a <= (kFusedWaves - sh_waves) * 8 * kWave;
    if (split) {
      gather(n_a, n_s, 0, kFusedWaves);  // first try succeeds: one round trip
      __syncthreads();
      if (wv < sh_waves) shared_rows(sh_waves);
      else gather(0, n_a, sh_waves, kFusedWaves - sh_waves);
      __syncthreads();
      if (tok == 0) trace_mark(a, 5);
    } else {
      gather(0, n_a + n_s, 0, kFusedWaves);
      __syncthreads();
      if (tok == 0) trace_mark(a, 5);
      if (Fs) shared_rows(kFusedWaves);
    }

    if constexpr (!kOneToken) {
      have_next = request_round0(tok + 1 < T ? tok + 1 : tok, pre_next);
      issue_fence();
    }
    // When a lane's share of a row is one 16-byte step, its slice of the slot's activations is the same in
    // every round: it is built once per token (with several rounds of rows that is a third of the round's
    // vector work).
    // (2-bit codes only: their slices are the longest to build and their layers the ones with several rounds;
    // the 4-bit and ternary launches measured slower with the extra path compiled in)
    const bool one_step = BITS == kBits2 && lpr * Fmt<BITS>::kElemsPer16B >= F && rounds > 1 && unit_local < ub;
    XSlice<BITS> xs_slot{};
    if (one_step && sub * Fmt<BITS>::kElemsPer16B < F)
      xs_slot = load_xslice<BITS, kXAligned>(reinterpret_cast<const uint16_t*>(s_acts) + slot * F +
                                             sub * Fmt<BITS>::kElemsPer16B);
    for (uint32_t round = 0; round < rounds; ++round) {
      const uint32_t unit = (round * G + wg) * ub + unit_local;
      const bool active = unit_local < ub && unit < rg_per_tok;
      if (active) {
        const uint32_t row = unit * rpw + (lane >> lpr_log2);
        const uint32_t pair = tok * K + slot;
        const uint32_t expert = __builtin_amdgcn_readfirstlane(s_idx[pair]);
        float part = 0.0f;
        if (row < D && expert < E) {
          const uint8_t* blob = a.expert_base + static_cast<size_t>(expert) * a.expert_stride;
          const uint8_t* wrow = blob + a.off.down_w + row * rb;
          const uint16_t* srow = reinterpret_cast<const uint16_t*>(blob + a.off.down_s) + row * ng;
          const uint16_t* brow = reinterpret_cast<const uint16_t*>(blob + a.off.down_b) + row * ng;
          if (one_step) {
            const uint32_t e0 = sub * Fmt<BITS>::kElemsPer16B;
            if (e0 < F) {  // the one step of row_partial over the slice at hand
              uint4 codes = pre.codes;
              float sc = pre.s, bi = pre.b;
              if (!(have_pre && round == 0)) {
                codes = load_codes16<true>(wrow + static_cast<size_t>(e0) * Store<BITS>::kBits / 8);
                load_scale_bias<BITS>(srow, brow, e0, sc, bi);
              }
              part = __builtin_fmaf(sc, codes_dot<BITS>(codes, xs_slot), 0.0f);
              part = __builtin_fmaf(bi, xs_slot.sum, part);
            }
          } else {
            part = row_partial<BITS>(wrow, srow, brow, reinterpret_cast<const uint16_t*>(s_acts) + slot * F, F, sub,
                                     lpr, have_pre && round == 0, pre);
          }
        }
        const float v = group_sum(part, static_cast<int>(lpr));
        // moe.metal:1262; maple_moe.metal:258 (the down output is a bf16 number first)
        if (sub == 0) s_v[wv * kWave + (lane >> lpr_log2)] = s_w[pair] * (maple ? round_bf16(v) : v);
      }
      __syncthreads();
      if (threadIdx.x < rows_per_round) {
        const uint32_t ul = threadIdx.x / rpw, rr = threadIdx.x % rpw;
        const uint32_t u2 = (round * G + wg) * ub + ul;
        const uint32_t row = u2 * rpw + rr;
        if (u2 < rg_per_tok && row < D) {
          const size_t o = static_cast<size_t>(tok) * D + row;
          // the K weighted values first (independent LDS reads: one round of latency, not K),
          // then the sum in rank order, residual first
          float vk[MF_MAX_TOPK];
          bool live[MF_MAX_TOPK];
#pragma unroll
          for (uint32_t k = 0; k < MF_MAX_TOPK; ++k) {
            live[k] = k < K && s_idx[tok * K + (k < K ? k : 0)] < E;
            vk[k] = s_v[(ul * K + (k < K ? k : 0)) * kWave + rr];
          }
          float acc = Fs ? s_h1[round * rows_per_round + threadIdx.x] : 0.0f;
#pragma unroll
          for (uint32_t k = 0; k < MF_MAX_TOPK; ++k)
            if (live[k]) acc = acc + vk[k];
          const bool failed = *s_fail != 0u;  // a wait gave up: no result, and hidden stays as it is
          const uint16_t yb = failed ? static_cast<uint16_t>(0x7FC0u) : f_to_bf16(acc);
          a.y[o] = yb;
          if (a.hidden && !failed) {  // residual_add_fp16, utility.metal:83-92
            uint16_t hv = a.hidden[o];
            if constexpr (NORM) {  // the residual add in front of the norm, made here for good
              if (a.delta) hv = f_to_bf16(bf16_to_f(hv) + bf16_to_f(a.delta[o]));
            }
            a.hidden[o] = f_to_bf16(bf16_to_f(hv) + bf16_to_f(yb));
          }
        }
      }
      // The next round (or token) overwrites s_v.  Behind the last round nothing is left to protect, and a
      // barrier there only makes every wave wait for the acknowledgement of the stores of y: the one-token
      // instances leave it out.  (With the token count an argument the same condition, or a barrier that
      // waits for LDS operations only, made the launch slower: the large 2-bit layer at 4 rows 92 -> 111 us.)
      if (!(kOneToken && round + 1 == rounds)) __syncthreads();
    }
  }
  if constexpr (!S::kGiven) {
    if (wg == 0 && threadIdx.x < T * K) {  // s_w was complete before stage C's first barrier
      if (a.out_idx) a.out_idx[threadIdx.x] = s_idx[threadIdx.x];
      if (a.out_w) a.out_w[threadIdx.x] = s_w[threadIdx.x];
    }
  }
  if (threadIdx.x == 0) a.epoch[wg] = epoch;
  trace_mark(a, 6);
}

// words of the LDS staging area: a chunk of router logits in stage A, the (gate, up) sums of a
// workgroup's run of routed rows in stage B
static uint32_t fused_stage_words(const mf_moe_config& c, uint32_t num_cu, uint32_t t) {
  const uint32_t epl = c.bits == MF_BITS_4 ? 32 : 64;
  const uint32_t rpw = 64u >> lanes_per_row_log2_dev(c.d, epl);
  const uint32_t rgf = (c.f + rpw - 1) / rpw;
  uint32_t per_wg = (t * c.top_k * rgf + num_cu - 1) / num_cu;
  per_wg = (per_wg + kFusedWaves - 1) / kFusedWaves * kFusedWaves;
  const uint32_t words = 2 * per_wg * rpw;
  return words < 64 ? 64 : (words + 3) & ~3u;
}
// words of the x slices of the routed rows (permuted pairs + sum per slice)
static uint32_t fused_xprep_words(const mf_moe_config& c, uint32_t t) {
  const uint32_t epl = c.bits == MF_BITS_4 ? 32 : 64;
  return t * (c.d / epl) * (epl / 2 + 1);
}
static size_t fused_lds_base(const mf_moe_config& c, uint32_t num_cu, uint32_t t) {
  const size_t sact_words = ((c.shared_f + 4) / 2 + 3) & ~size_t(3);
  const size_t acts_words = (static_cast<size_t>(c.top_k) * c.f / 2 + 3) & ~size_t(3);
  return 1024 + 4096 + kMaxH1 * 4 + kRankWords * 4 + static_cast<size_t>(MF_MAX_TOKENS) * c.num_experts * 4 +
         4 * (sact_words + acts_words + fused_stage_words(c, num_cu, t));
}
constexpr size_t kFusedLdsLimit = 150 * 1024;
// the x slices are kept in LDS when they fit beside everything else
static bool fused_xprep(const mf_moe_config& c, uint32_t num_cu, uint32_t t) {
  return fused_lds_base(c, num_cu, t) + 4 * static_cast<size_t>(fused_xprep_words(c, t)) <= kFusedLdsLimit;
}
size_t fused_lds_bytes(const mf_moe_config& c, uint32_t num_cu, uint32_t t) {
  const size_t base = fused_lds_base(c, num_cu, t);
  return fused_xprep(c, num_cu, t) ? base + 4 * static_cast<size_t>(fused_xprep_words(c, t)) : base;
}

bool fused_supported(const mf_moe& h, const mf_moe_layer_weights& w, const void* x, const void* y,
                     const void* hidden, uint32_t t) {
  const mf_moe_config& c = h.cfg;
  if (c.num_experts % 4 != 0) return false;  // tagged logits are read two entries per lane
  if (c.gate_group_size == 32) return false;  // a gate projection at group 32 runs on the chain of launches
  const bool combo = (c.bits == MF_BITS_4 && (!c.shared_f || c.shared_bits == MF_BITS_4)) ||
                     (c.bits == MF_BITS_2 && (!c.shared_f || c.shared_bits == MF_BITS_4 ||
                                              c.shared_bits == MF_BITS_2)) ||
                     (c.bits == MF_BITS_TERNARY && (!c.shared_f || c.shared_bits == MF_BITS_4));
  if (!combo || c.d % 8 != 0) return false;
  if (fused_lds_base(c, static_cast<uint32_t>(h.ctx->num_cu), t) > kFusedLdsLimit) return false;
  {  // rows of one token a workgroup owns must fit the h1 array
    const uint32_t epl = c.bits == MF_BITS_4 ? 32 : 64;
    const uint32_t rpw = 64u >> lanes_per_row_log2_dev(c.f, epl);
    const uint32_t rg = (c.d + rpw - 1) / rpw, ub = kFusedWaves / c.top_k;
    const uint32_t G = static_cast<uint32_t>(h.ctx->num_cu);
    const uint32_t rounds = (rg + G * ub - 1) / (G * ub);
    if (rounds * ub * rpw > kMaxH1) return false;
  }
  const uint32_t offs = w.offsets.gate_w | w.offsets.up_w | w.offsets.down_w;
  if (!aligned16(w.expert_base) || w.expert_stride % 16 || offs % 16) return false;
  if (!aligned16(w.router_w) || !aligned16(x) || !aligned16(y)) return false;
  if (hidden && !aligned16(hidden)) return false;
  if (c.shared_f) {
    if (!aligned16(w.shared_gate.weights) || !aligned16(w.shared_up.weights) ||
        !aligned16(w.shared_down.weights))
      return false;
    if (w.w_sg && !w.w_sg_q8.weights && !aligned16(w.w_sg)) return false;
    if (w.w_sg_q8.weights && (reinterpret_cast<uintptr_t>(w.w_sg_q8.weights) & 7u)) return false;
  }
  return true;
}

// Whether the launch can make x itself (NORM instances): own routing, rows of at most 4096 elements, room in
// LDS for the normalised rows, everything the plain launch needs
bool fused_norm_supported(const mf_moe& h, const mf_moe_layer_weights& w, const void* y, const void* hidden,
                          const void* delta, const void* norm_w, uint32_t t) {
  const mf_moe_config& c = h.cfg;
  if (!w.router_w || !hidden || !norm_w || c.d > 4096) return false;
  if (!aligned16(hidden) || !aligned16(norm_w) || (delta && !aligned16(delta))) return false;
  if (!fused_supported(h, w, hidden, y, hidden, t)) return false;  // (x stands in as an aligned pointer)
  const uint32_t num_cu = static_cast<uint32_t>(h.ctx->num_cu);
  return fused_lds_bytes(c, num_cu, t) + 16 + static_cast<size_t>(t) * c.d * 2 <= kFusedLdsLimit;
}

hipError_t launch_fused_decode(hipStream_t s, const mf_moe& h, const mf_moe_layer_weights& w,
                               const uint16_t* x, uint32_t t, uint16_t* y, uint16_t* hidden,
                               uint32_t* out_idx, float* out_w, const FusedNorm* norm) {
  const mf_moe_config& c = h.cfg;
  FusedArgs a{};
  a.router_w = w.router_w;
  a.expert_base = static_cast<const uint8_t*>(w.expert_base);
  a.expert_stride = w.expert_stride;
  a.off = w.offsets;
  a.sg = w.shared_gate;
  a.su = w.shared_up;
  a.sd = w.shared_down;
  const bool gate_q8 = c.shared_f && w.w_sg_q8.weights;
  a.w_sg = c.shared_f && !gate_q8 ? w.w_sg : nullptr;
  a.gq_w = gate_q8 ? static_cast<const uint8_t*>(w.w_sg_q8.weights) : nullptr;
  a.gq_s = gate_q8 ? w.w_sg_q8.scales : nullptr;
  a.gq_b = gate_q8 ? w.w_sg_q8.biases : nullptr;
  a.x = x;
  a.y = y;
  a.hidden = hidden;
  a.out_idx = out_idx;
  a.out_w = out_w;
  a.t_logits = h.ws.t_logits;
  a.t_sact = h.ws.t_sact;
  a.t_acts = h.ws.t_acts;
  a.epoch = h.ws.epoch;
  a.status = h.ws.status;
  a.trace = h.trace;
  a.D = c.d;
  a.F = c.f;
  a.E = c.num_experts;
  a.K = c.top_k;
  a.T = t;
  a.Fs = c.shared_f;
  a.router_mode = c.router_mode;
  a.limit = c.swiglu_limit;
  a.maple = static_cast<int>(c.maple_rounding);
  const dim3 grid(static_cast<uint32_t>(h.ctx->num_cu)), block(kFusedThreads);
  const uint32_t num_cu = static_cast<uint32_t>(h.ctx->num_cu);
  size_t lds = fused_lds_bytes(c, num_cu, t);
  a.stage_words = fused_stage_words(c, num_cu, t);
  a.xprep = fused_xprep(c, num_cu, t) ? 1 : 0;
  if (norm) {  // the normalised rows behind everything else in LDS
    a.delta = norm->delta;
    a.norm_w = norm->weight;
    a.norm_eps = norm->eps;
    a.xn_off = static_cast<uint32_t>((lds + 15) & ~size_t(15));
    lds = a.xn_off + static_cast<size_t>(t) * c.d * 2;
  }
#define MF_FUSED(B, SB, SHAPE)                                                                 \
  do {                                                                                         \
    auto kern = fused_decode_kernel<B, SB, SHAPE>;                                             \
    if (lds > 48 * 1024) {                                                                     \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                  \
                                         hipFuncAttributeMaxDynamicSharedMemorySize,           \
                                         static_cast<int>(lds));                               \
      if (e != hipSuccess) return e;                                                           \
    }                                                                                          \
    kern<<<grid, block, lds, s>>>(a);                                                          \
  } while (0)
  // Shape-specialised instances: a layer shape's dimensions as literals with the token rows read from the
  // arguments (Tn), and the one-token launch with T = 1 as a literal as well (T1: it drops the code of the
  // token loop; Qwen shape 12.3 us against 13.5 us through Tn).  Which literal buys what, Qwen shape, 4
  // token rows: none 40.2 us, T alone 39.8, top_k 37.5, top_k + experts 36.5, d + f 35.1, d + f + top_k 33.9,
  // those + shared_f 29.1, all but T 27.2, all 27.1.
  using QwenT1 = StaticShape<2048, 512, 256, 8, 1, 512, false, 0, 0, 1, 1>;
  using QwenTn = StaticShape<2048, 512, 256, 8, kDyn, 512, false, 0>;
  const bool qwen = c.bits == MF_BITS_4 && c.shared_bits == MF_BITS_4 && c.d == 2048 &&
                    c.f == 512 && c.num_experts == 256 && c.top_k == 8 && c.shared_f == 512 &&
                    c.router_mode == MF_ROUTER_TOPK_SOFTMAX;
  // the large 2-bit layer (hidden 4096, 256 experts of 2048, top-6, 4-bit shared expert of 2048)
  using Big2T1 = StaticShape<4096, 2048, 256, 6, 1, 2048, false, 0, 0, 0, 1>;
  using Big2Tn = StaticShape<4096, 2048, 256, 6, kDyn, 2048, false, 0>;
  const bool big2 = c.bits == MF_BITS_2 && c.shared_bits == MF_BITS_4 && c.d == 4096 && c.f == 2048 &&
                    c.num_experts == 256 && c.top_k == 6 && c.shared_f == 2048 &&
                    c.router_mode == MF_ROUTER_TOPK_SOFTMAX;
  // the ternary layer (hidden 2048, 64 experts of 1024, top-8, no shared expert)
  using TernT1 = StaticShape<2048, 1024, 64, 8, 1, 0, false, 1, 1, 1, 1>;
  using TernTn = StaticShape<2048, 1024, 64, 8, kDyn, 0>;
  const bool tern = c.bits == MF_BITS_TERNARY && c.d == 2048 && c.f == 1024 && c.num_experts == 64 &&
                    c.top_k == 8 && c.shared_f == 0;
  // MaplePreview's ternary layer (ModelTypes.swift:515-560: hidden 2048, 256 experts of 512, top-8, no shared expert)
  using MapleT1 = StaticShape<2048, 512, 256, 8, 1, 0, false, 1, 1, 1, 1>;
  using MapleTn = StaticShape<2048, 512, 256, 8, kDyn, 0>;
  const bool maple = c.bits == MF_BITS_TERNARY && c.d == 2048 && c.f == 512 && c.num_experts == 256 &&
                     c.top_k == 8 && c.shared_f == 0;
  const bool no_limit = c.swiglu_limit == 0.0f;  // the one-token instances of the benchmark shapes have these flags as literals
  // the instances of the shapes listed for the build (fused_shapes.json): declarations here, the branches
  // that pick them below, ahead of the instances that read every dimension from the arguments
#define MF_SHAPES_DECLARE
#include "fused_shapes.inc"
#undef MF_SHAPES_DECLARE
  using Given = RuntimeShapeT<true>;
  using Big2T1Given = StaticShape<4096, 2048, 256, 6, 1, 2048, true>;
  using QwenT1Given = StaticShape<2048, 512, 256, 8, 1, 512, true, kDyn, 0, 1, 1>;
  using QwenTnGiven = StaticShape<2048, 512, 256, 8, kDyn, 512, true>;
  // (with the routing given the router mode plays no part: the shapes are recognised without it)
  const bool qwen_dims = c.bits == MF_BITS_4 && c.shared_bits == MF_BITS_4 && c.d == 2048 && c.f == 512 &&
                         c.num_experts == 256 && c.top_k == 8 && c.shared_f == 512;
  const bool lit = !h.generic_shape;  // shape instances allowed
#define MF_FUSED_N(B, SB, SHAPE)                                                               \
  do {                                                                                         \
    auto kern = fused_decode_kernel<B, SB, SHAPE, true>;                                       \
    if (lds > 48 * 1024) {                                                                     \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                  \
                                         hipFuncAttributeMaxDynamicSharedMemorySize,           \
                                         static_cast<int>(lds));                               \
      if (e != hipSuccess) return e;                                                           \
    }                                                                                          \
    kern<<<grid, block, lds, s>>>(a);                                                          \
  } while (0)
  if (norm) {  // x made inside the launch: the Qwen shape's instances and the ones that read every dimension
    if (lit && qwen && t == 1 && !c.maple_rounding && no_limit && a.xprep) MF_FUSED_N(kBits4, kBits4, QwenT1);
    else if (lit && qwen) MF_FUSED_N(kBits4, kBits4, QwenTn);
    else if (c.bits == MF_BITS_4) MF_FUSED_N(kBits4, kBits4, RuntimeShape);
    else if (c.bits == MF_BITS_2 && c.shared_f && c.shared_bits == MF_BITS_2) MF_FUSED_N(kBits2, kBits2, RuntimeShape);
    else if (c.bits == MF_BITS_2) MF_FUSED_N(kBits2, kBits4, RuntimeShape);
    else MF_FUSED_N(kBitsTernary, kBits4, RuntimeShape);
    return hipGetLastError();
  }
#undef MF_FUSED_N
  if (!w.router_w) {  // caller-given routing
    if (!lit) {
      if (c.bits == MF_BITS_4) MF_FUSED(kBits4, kBits4, Given);
      else if (c.bits == MF_BITS_2 && c.shared_f && c.shared_bits == MF_BITS_2) MF_FUSED(kBits2, kBits2, Given);
      else if (c.bits == MF_BITS_2) MF_FUSED(kBits2, kBits4, Given);
      else MF_FUSED(kBitsTernary, kBits4, Given);
    }
    else if (big2 && t == 1) MF_FUSED(kBits2, kBits4, Big2T1Given);
    else if (qwen_dims && t == 1 && !c.maple_rounding && no_limit && a.xprep) MF_FUSED(kBits4, kBits4, QwenT1Given);
    else if (qwen_dims) MF_FUSED(kBits4, kBits4, QwenTnGiven);
#define MF_SHAPES_PICK_GIVEN
#include "fused_shapes.inc"
#undef MF_SHAPES_PICK_GIVEN
    else if (c.bits == MF_BITS_4) MF_FUSED(kBits4, kBits4, Given);
    else if (c.bits == MF_BITS_2 && c.shared_f && c.shared_bits == MF_BITS_2) MF_FUSED(kBits2, kBits2, Given);
    else if (c.bits == MF_BITS_2) MF_FUSED(kBits2, kBits4, Given);
    else MF_FUSED(kBitsTernary, kBits4, Given);
  } else if (!lit) {
    if (c.bits == MF_BITS_4) MF_FUSED(kBits4, kBits4, RuntimeShape);
    else if (c.bits == MF_BITS_2 && c.shared_f && c.shared_bits == MF_BITS_2) MF_FUSED(kBits2, kBits2, RuntimeShape);
    else if (c.bits == MF_BITS_2) MF_FUSED(kBits2, kBits4, RuntimeShape);
    else MF_FUSED(kBitsTernary, kBits4, RuntimeShape);
  } else if (qwen && t == 1 && !c.maple_rounding && no_limit && a.xprep) MF_FUSED(kBits4, kBits4, QwenT1);
  else if (qwen) MF_FUSED(kBits4, kBits4, QwenTn);
  else if (big2 && t == 1 && !c.maple_rounding && a.xprep) MF_FUSED(kBits2, kBits4, Big2T1);
  else if (big2) MF_FUSED(kBits2, kBits4, Big2Tn);
  else if (tern && t == 1 && c.router_mode == MF_ROUTER_FULL_SOFTMAX && c.maple_rounding && no_limit && a.xprep)
    MF_FUSED(kBitsTernary, kBits4, TernT1);
  else if (tern) MF_FUSED(kBitsTernary, kBits4, TernTn);
  else if (maple && t == 1 && c.router_mode == MF_ROUTER_FULL_SOFTMAX && c.maple_rounding && no_limit && a.xprep)
    MF_FUSED(kBitsTernary, kBits4, MapleT1);
  else if (maple) MF_FUSED(kBitsTernary, kBits4, MapleTn);
#define MF_SHAPES_PICK_OWN
#include "fused_shapes.inc"
#undef MF_SHAPES_PICK_OWN
  else if (c.bits == MF_BITS_4) MF_FUSED(kBits4, kBits4, RuntimeShape);
  else if (c.bits == MF_BITS_2 && c.shared_f && c.shared_bits == MF_BITS_2)
    MF_FUSED(kBits2, kBits2, RuntimeShape);
  else if (c.bits == MF_BITS_2) MF_FUSED(kBits2, kBits4, RuntimeShape);
  else MF_FUSED(kBitsTernary, kBits4, RuntimeShape);
#undef MF_FUSED
  return hipGetLastError();
}

}  // namespace mf
