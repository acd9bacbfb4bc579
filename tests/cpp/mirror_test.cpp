// Drives libmfmoe through the C++ mirror of the reference's operator classes
// (include/mfmoe.hpp) and checks the results against the CPU checker, the way the reference's
// own XCTest cases drive its Swift operators: SeedTree-seeded inputs, one small layer,
// decode == per-token checker, ragged prefill == per-token checker, family routers bit for bit,
// grouping KATs and errors.
//
//   mirror_test cpu   grouping KATs and error cases only (no GPU needed)
//   mirror_test gpu   everything
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "mfmoe.hpp"
extern "C" {
#include "mf_oracle.h"
}

static int g_fail = 0;
#define EXPECT(cond, ...)                                   \
  do {                                                      \
    if (!(cond)) {                                          \
      ++g_fail;                                             \
      std::printf("FAIL %s:%d: ", __FILE__, __LINE__);      \
      std::printf(__VA_ARGS__);                             \
      std::printf("\n");                                    \
    }                                                       \
  } while (0)

#define HIP_OK(call)                                                              \
  do {                                                                            \
    hipError_t e_ = (call);                                                       \
    if (e_ != hipSuccess) {                                                       \
      std::printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
      std::exit(2);                                                               \
    }                                                                             \
  } while (0)

template <typename T> static T* to_device(const std::vector<T>& v) {
  T* p = nullptr;
  HIP_OK(hipMalloc(&p, v.size() * sizeof(T) + 16));
  HIP_OK(hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice));
  return p;
}
template <typename T> static std::vector<T> to_host(const T* p, size_t n) {
  std::vector<T> v(n);
  HIP_OK(hipMemcpy(v.data(), p, n * sizeof(T), hipMemcpyDeviceToHost));
  return v;
}

// ---------------------------------------------------------------- grouping (host)
// PrefillMoEGroupingTests: pairs of 3 tokens x top-2 over 4 experts; sorted by (expert, token,
// rank), offsets 0xFFFFFFFF for the empty expert, error cases carry their payload.
static void test_grouping() {
  const uint32_t idx[6] = {2, 0, 0, 3, 2, 0};
  const uint32_t wb[6] = {10, 11, 12, 13, 14, 15};
  auto pairs = mf::PrefillMoEGrouping::makeTokenExpertPairs(idx, wb, 3, 2);
  auto routes = mf::PrefillMoEGrouping::groupTokenExpertPairs(pairs, 3, 2, 4, 2);
  const uint32_t want_expert[6] = {0, 0, 0, 2, 2, 3};
  const uint32_t want_token[6] = {0, 1, 2, 0, 2, 1};
  const uint32_t want_w[6] = {11, 12, 15, 10, 14, 13};
  for (int i = 0; i < 6; ++i)
    EXPECT(routes.sortedPairs[i].expert == want_expert[i] && routes.sortedPairs[i].token == want_token[i] &&
               routes.sortedPairs[i].weight_bits == want_w[i], "sorted pair %d", i);
  EXPECT(routes.expertOffsets[0] == 0 && routes.expertOffsets[1] == 0xFFFFFFFFu && routes.expertOffsets[2] == 3 &&
             routes.expertOffsets[3] == 5, "offsets");
  EXPECT(routes.expertCounts[0] == 3 && routes.expertCounts[1] == 0 && routes.expertCounts[2] == 2 &&
             routes.expertCounts[3] == 1, "counts");
  EXPECT(routes.groups.size() == 3 && routes.tiles.size() == 2, "groups %zu tiles %zu", routes.groups.size(),
         routes.tiles.size());
  EXPECT(routes.maxPairsPerExpert() == 3 && routes.maxPairsPerTile() == 5, "max pairs");
  // the same result as the checker's restatement
  std::vector<mfo_pair> op(6), os(6);
  mfo_make_pairs(idx, wb, 3, 2, op.data());
  std::vector<uint32_t> oo(4), oc(4);
  std::vector<mfo_group> og(4);
  std::vector<mfo_tile> ot(4);
  size_t ng = 0, nt = 0;
  EXPECT(mfo_group_pairs(op.data(), 6, 3, 2, 4, 2, nullptr, 0, os.data(), oo.data(), oc.data(), og.data(), &ng,
                         ot.data(), &nt) == 0, "checker grouping");
  EXPECT(std::memcmp(os.data(), routes.sortedPairs.data(), 6 * sizeof(mfo_pair)) == 0, "sorted == checker");
  // errors are thrown with the reference's case as status
  bool thrown = false;
  try {
    auto bad = pairs;
    bad[3].expert = 9;
    mf::PrefillMoEGrouping::groupTokenExpertPairs(bad, 3, 2, 4, 2);
  } catch (const mf::Error& e) {
    thrown = e.status == MF_ERR_EXPERT_RANGE && e.detail[0] == 9;
  }
  EXPECT(thrown, "expertOutOfRange(9) not thrown");
  thrown = false;
  try {
    mf::PrefillMoEGrouping::groupTokenExpertPairs(pairs, 3, 2, 4, 0);
  } catch (const mf::Error& e) {
    thrown = e.status == MF_ERR_TILE_EXPERT_COUNT;
  }
  EXPECT(thrown, "invalidTileExpertCount not thrown");
}

// ---------------------------------------------------------------- one layer on the GPU
struct HostLayer {
  size_t d, f, e, k, fs;
  std::vector<uint16_t> router_w, w_sg;
  std::vector<uint8_t> experts;
  size_t stride;
  mfo_expert_offsets off;
  std::vector<uint8_t> sw[3];
  std::vector<uint16_t> ss[3], sb[3];
};

static void quantize(uint64_t root, const std::string& label, size_t rows, size_t cols, std::vector<uint8_t>& w,
                     std::vector<uint16_t>& s, std::vector<uint16_t>& b) {
  mfo_rng r = mfo_seed_tree_key(root, label.c_str());
  std::vector<float> raw(rows * cols);
  mfo_rng_normal(&r, 0.0f, 0.02f, raw.data(), raw.size());
  w.resize(rows * cols / 2);
  s.resize(rows * cols / 64);
  b.resize(rows * cols / 64);
  mfo_quantize_affine(raw.data(), rows, cols, 4, w.data(), s.data(), b.data());
}

static HostLayer make_layer(uint64_t root, size_t d, size_t f, size_t e, size_t k, size_t fs) {
  HostLayer L{d, f, e, k, fs, {}, {}, {}, 0, {}, {}, {}, {}};
  mfo_rng r = mfo_seed_tree_key(root, "router");
  std::vector<float> raw(e * d);
  mfo_rng_normal(&r, 0.0f, 0.02f, raw.data(), raw.size());
  L.router_w.resize(e * d);
  mfo_bf16_encode(raw.data(), raw.size(), L.router_w.data());
  // blob: gate{W,s,b}, up{W,s,b}, down{W,s,b} (RepackPlanner.swift:544-712), stride rounded to 256
  const size_t gu_w = f * d / 2, gu_s = f * (d / 64) * 2, dn_w = d * f / 2, dn_s = d * (f / 64) * 2;
  uint32_t pos = 0;
  uint32_t* o = &L.off.gate_w;
  const size_t sizes[9] = {gu_w, gu_s, gu_s, gu_w, gu_s, gu_s, dn_w, dn_s, dn_s};
  for (int i = 0; i < 9; ++i) {
    o[i] = pos;
    pos += static_cast<uint32_t>(sizes[i]);
  }
  L.stride = (pos + 255) / 256 * 256;
  L.experts.assign(e * L.stride, 0);
  for (size_t x = 0; x < e; ++x) {
    const char* names[3] = {"gate", "up", "down"};
    for (int t = 0; t < 3; ++t) {
      std::vector<uint8_t> w;
      std::vector<uint16_t> s, b;
      const size_t rows = t < 2 ? f : d, cols = t < 2 ? d : f;
      quantize(root, "expert" + std::to_string(x) + "." + names[t], rows, cols, w, s, b);
      uint8_t* blob = L.experts.data() + x * L.stride;
      std::memcpy(blob + o[3 * t], w.data(), w.size());
      std::memcpy(blob + o[3 * t + 1], s.data(), s.size() * 2);
      std::memcpy(blob + o[3 * t + 2], b.data(), b.size() * 2);
    }
  }
  const char* sn[3] = {"shared.gate", "shared.up", "shared.down"};
  for (int t = 0; t < 3; ++t) quantize(root, sn[t], t < 2 ? fs : d, t < 2 ? d : fs, L.sw[t], L.ss[t], L.sb[t]);
  r = mfo_seed_tree_key(root, "w_sg");
  raw.resize(d);
  mfo_rng_normal(&r, 0.0f, 0.02f, raw.data(), d);
  L.w_sg.resize(d);
  mfo_bf16_encode(raw.data(), d, L.w_sg.data());
  return L;
}

static void compare(const std::vector<uint16_t>& got, const std::vector<uint16_t>& ref, const char* what) {
  double max_abs = 0, num = 0, den = 0;
  for (size_t i = 0; i < got.size(); ++i) {
    const double a = mfo_bf16_to_float(got[i]), b = mfo_bf16_to_float(ref[i]);
    max_abs = std::fmax(max_abs, std::fabs(a - b));
    num += (a - b) * (a - b);
    den += b * b;
  }
  const double rel = std::sqrt(num / std::fmax(den, 1e-30));
  std::printf("%-28s max_abs %.3e rel_l2 %.3e\n", what, max_abs, rel);
  EXPECT(max_abs <= 2e-2 && rel <= 1e-3, "%s out of tolerance", what);  // the layer tolerance
}

static void test_layer() {
  const size_t d = 512, f = 256, e = 32, k = 8, fs = 256, t_dec = 3, t_pre = 90;
  const uint64_t root = 0x4D464D4F00000000ull + 0xC99;
  HostLayer L = make_layer(root, d, f, e, k, fs);
  mfo_layer ol{};
  ol.d = d; ol.f = f; ol.e = e; ol.k = k; ol.fs = fs; ol.bits = 4; ol.shared_bits = 4; ol.router_mode = 0;
  ol.router_w = L.router_w.data(); ol.experts = L.experts.data(); ol.expert_stride = L.stride; ol.off = L.off;
  ol.sgw = L.sw[0].data(); ol.sgs = L.ss[0].data(); ol.sgb = L.sb[0].data();
  ol.suw = L.sw[1].data(); ol.sus = L.ss[1].data(); ol.sub = L.sb[1].data();
  ol.sdw = L.sw[2].data(); ol.sds = L.ss[2].data(); ol.sdb = L.sb[2].data();
  ol.w_sg = L.w_sg.data();

  mfo_rng r = mfo_seed_tree_key(root, "x");
  std::vector<float> xf(t_pre * d);
  mfo_rng_normal(&r, 0.0f, 1.0f, xf.data(), xf.size());
  std::vector<uint16_t> x(t_pre * d);
  mfo_bf16_encode(xf.data(), xf.size(), x.data());
  std::vector<uint16_t> ref_y(t_pre * d);
  std::vector<uint32_t> ref_idx(t_pre * k);
  std::vector<float> ref_w(t_pre * k);
  EXPECT(mfo_moe_layer_tokens(&ol, x.data(), t_pre, ref_y.data(), ref_idx.data(), ref_w.data(), 1) == 0, "checker");

  mf::MetalContext context(0);
  mf::MoE moe(context, d, f, e, k, MF_BITS_4, MF_ROUTER_TOPK_SOFTMAX, 0.0f, fs, MF_BITS_4);
  mf_moe_layer_weights w{};
  w.router_w = to_device(L.router_w);
  w.expert_base = to_device(L.experts);
  w.expert_stride = L.stride;
  std::memcpy(&w.offsets, &L.off, sizeof(w.offsets));
  mf_qtensor* sh[3] = {&w.shared_gate, &w.shared_up, &w.shared_down};
  for (int i = 0; i < 3; ++i) *sh[i] = mf_qtensor{to_device(L.sw[i]), to_device(L.ss[i]), to_device(L.sb[i])};
  w.w_sg = to_device(L.w_sg);
  uint16_t* dx = to_device(x);
  uint16_t* dy = nullptr;
  uint32_t* didx = nullptr;
  float* dw = nullptr;
  HIP_OK(hipMalloc(&dy, t_pre * d * 2));
  HIP_OK(hipMalloc(&didx, t_pre * k * 4));
  HIP_OK(hipMalloc(&dw, t_pre * k * 4));

  // decode: the first t_dec tokens in one launch
  moe.encodeDecodeLayer(nullptr, w, dx, dy, t_dec, nullptr, didx, dw);
  moe.status(nullptr);
  auto y = to_host(dy, t_dec * d);
  auto idx = to_host(didx, t_dec * k);
  auto wt = to_host(dw, t_dec * k);
  EXPECT(std::memcmp(idx.data(), ref_idx.data(), t_dec * k * 4) == 0, "decode routing indices");
  EXPECT(std::memcmp(wt.data(), ref_w.data(), t_dec * k * 4) == 0, "decode routing weights (bit-exact)");
  compare(y, std::vector<uint16_t>(ref_y.begin(), ref_y.begin() + t_dec * d), "decode layer");

  // two-phase structure (MoEFusedFFNTests): router, phase 1, phase 2 as separate calls == fused launch
  uint16_t* dacts = nullptr;
  uint16_t* dy2 = nullptr;
  HIP_OK(hipMalloc(&dacts, k * f * 2));
  HIP_OK(hipMalloc(&dy2, d * 2));
  mf::MoE routed(context, d, f, e, k);  // no shared expert: the routed part alone
  routed.encodeRouter(nullptr, w.router_w, dx, didx, dw);
  routed.encodeRoutedPersistentPhase1U16Load(nullptr, w.expert_base, w.expert_stride, w.offsets, didx, dx, dacts);
  routed.encodeRoutedPersistentPhase2Reduce(nullptr, w.expert_base, w.expert_stride, w.offsets, didx, dw, dacts,
                                            nullptr, dy2);
  mf_moe_layer_weights wr = w;
  uint16_t* dy3 = nullptr;
  HIP_OK(hipMalloc(&dy3, d * 2));
  routed.encodeDecodeLayer(nullptr, wr, dx, dy3);
  routed.status(nullptr);
  EXPECT(to_host(dy2, d) == to_host(dy3, d), "two-phase != fused launch");

  // ragged prefill: all t_pre tokens
  const size_t ws_bytes = moe.prefillWorkspaceBytes(t_pre);
  void* ws = nullptr;
  HIP_OK(hipMalloc(&ws, ws_bytes));
  moe.encodePrefillLayer(nullptr, w, dx, dy, t_pre, ws, ws_bytes, didx, dw);
  HIP_OK(hipDeviceSynchronize());
  idx = to_host(didx, t_pre * k);
  EXPECT(std::memcmp(idx.data(), ref_idx.data(), t_pre * k * 4) == 0, "prefill routing indices");
  compare(to_host(dy, t_pre * d), ref_y, "ragged prefill layer");

  // the same layer from the tiled copy of the expert pool: the bits of the row-by-row pool
  {
    auto y_rows = to_host(dy, t_pre * d);
    void* tiled = nullptr;
    HIP_OK(hipMalloc(&tiled, L.stride * e));
    moe.tileExperts(nullptr, w.expert_base, w.expert_stride, w.offsets, tiled);
    mf_moe_layer_weights wt2 = w;
    wt2.expert_tiled = tiled;
    moe.encodePrefillLayer(nullptr, wt2, dx, dy, t_pre, ws, ws_bytes, didx, dw);
    HIP_OK(hipDeviceSynchronize());
    EXPECT(to_host(dy, t_pre * d) == y_rows, "tiled pool != row-by-row pool");
    std::printf("%-28s bit-identical\n", "prefill from the tiled pool");
  }

  // the residual add and the RMSNorm in front of the layer in the layer's launch == the two calls
  {
    std::vector<float> nf(d), df(t_dec * d);
    mfo_rng rn = mfo_seed_tree_key(root, "norm");
    mfo_rng_normal(&rn, 1.0f, 0.1f, nf.data(), nf.size());
    mfo_rng_normal(&rn, 0.0f, 0.5f, df.data(), df.size());
    std::vector<uint16_t> nw(d), dl(t_dec * d);
    mfo_bf16_encode(nf.data(), nf.size(), nw.data());
    mfo_bf16_encode(df.data(), df.size(), dl.data());
    uint16_t* dnw = to_device(nw);
    uint16_t* ddl = to_device(dl);
    std::vector<uint16_t> h0(x.begin(), x.begin() + t_dec * d);
    uint16_t* dh1 = to_device(h0);
    uint16_t* dh2 = to_device(h0);
    uint16_t* dxn = nullptr;
    uint16_t* dya = nullptr;
    uint16_t* dyb = nullptr;
    HIP_OK(hipMalloc(&dxn, t_dec * d * 2));
    HIP_OK(hipMalloc(&dya, t_dec * d * 2));
    HIP_OK(hipMalloc(&dyb, t_dec * d * 2));
    moe.encodeDecodeLayerNormed(nullptr, w, dh1, ddl, dnw, 1e-6f, dya, t_dec);
    mf::RMSNorm norm(context);
    norm.encodeBF16W(nullptr, dh2, dnw, dxn, d, 1e-6f, t_dec, ddl);
    moe.encodeDecodeLayer(nullptr, w, dxn, dyb, t_dec, dh2);
    moe.status(nullptr);
    EXPECT(to_host(dya, t_dec * d) == to_host(dyb, t_dec * d), "normed layer: y != two calls");
    EXPECT(to_host(dh1, t_dec * d) == to_host(dh2, t_dec * d), "normed layer: hidden != two calls");
    std::printf("%-28s bit-identical\n", "normed decode layer");
  }

  // argument errors throw and launch nothing (SharedExpertError.scratchTooSmall)
  bool thrown = false;
  try {
    moe.encodePrefillLayer(nullptr, w, dx, dy, t_pre, ws, 64);
  } catch (const mf::Error& err) {
    thrown = err.status == MF_ERR_SCRATCH_TOO_SMALL;
  }
  EXPECT(thrown, "scratchTooSmall not thrown");
}

// ---------------------------------------------------------------- family routers (GPU)
// The DeepSeek-V4 selector and the Inkling router through the mirror classes, bit for bit against
// the checker on seeded inputs.
static void test_family_routers(const mf::MetalContext& ctx) {
  const uint32_t e = 64, shared = 2, d = 256, t = 3, k = 6;
  mfo_rng rng = mfo_seed_tree_key(0x4D464D4F0000FA40ull, "family");
  std::vector<float> wf((e + shared) * d), xf(t * d), bias(e);
  mfo_rng_normal(&rng, 0.0f, 0.05f, wf.data(), wf.size());
  mfo_rng_normal(&rng, 0.0f, 1.0f, xf.data(), xf.size());
  mfo_rng_uniform_fill(&rng, -0.3f, 0.3f, bias.data(), bias.size());
  std::vector<uint16_t> w(wf.size()), x(xf.size());
  mfo_bf16_encode(wf.data(), wf.size(), w.data());
  mfo_bf16_encode(xf.data(), xf.size(), x.data());
  const std::vector<float> gs = {0.75f};
  uint16_t* dw = to_device(w);
  uint16_t* dx = to_device(x);
  float* dbias = to_device(bias);
  float* dgs = to_device(gs);
  uint32_t* didx = to_device(std::vector<uint32_t>(t * 8));
  float* dwt = to_device(std::vector<float>(t * 8));
  float* dgam = to_device(std::vector<float>(t * shared));
  float* dlg = to_device(std::vector<float>(t * (e + shared)));

  mf::MoEDeepseekV4Router v4(ctx, 1.5f, k);
  v4.encodeRouterTopK(nullptr, dw, dx, dbias, didx, dwt, e, d, dlg, t);
  HIP_OK(hipDeviceSynchronize());
  auto idx = to_host(didx, t * k);
  auto wt = to_host(dwt, t * k);
  for (uint32_t i = 0; i < t; ++i) {
    std::vector<float> lg(e);
    mfo_router_logits_bf16(w.data(), x.data() + i * d, e, d, lg.data());
    uint32_t ri[8];
    float rw[8];
    mfo_router_sqrtsoftplus(lg.data(), bias.data(), e, k, 1.5f, ri, rw);
    EXPECT(!std::memcmp(ri, idx.data() + i * k, k * 4) && !std::memcmp(rw, wt.data() + i * k, k * 4),
           "sqrtsoftplus router row %u", i);
  }
  v4.encodeRouterHashWeights(nullptr, dw, dx, didx, dwt, e, d, dlg, t);
  HIP_OK(hipDeviceSynchronize());
  EXPECT(to_host(dwt, t * k) == wt, "hash weights of the selected experts");

  mf::InklingRouter ink(ctx);
  ink.encodeRouter(nullptr, dw, dx, dbias, dgs, didx, dwt, dgam, e, shared, 8, 2.5f, d, dlg, t);
  HIP_OK(hipDeviceSynchronize());
  idx = to_host(didx, t * 8);
  wt = to_host(dwt, t * 8);
  auto gam = to_host(dgam, t * shared);
  for (uint32_t i = 0; i < t; ++i) {
    std::vector<float> lg(e + shared);
    mfo_router_logits_bf16(w.data(), x.data() + i * d, e + shared, d, lg.data());
    uint32_t ri[8];
    float rw[8], rg[8];
    mfo_router_inkling(lg.data(), bias.data(), 0.75f, e, shared, 8, 2.5f, ri, rw, rg);
    EXPECT(!std::memcmp(ri, idx.data() + i * 8, 32) && !std::memcmp(rw, wt.data() + i * 8, 32) &&
               !std::memcmp(rg, gam.data() + i * shared, shared * 4), "inkling router row %u", i);
  }
  bool threw = false;
  try {
    mf::MoEDeepseekV4Router(ctx, 1.0f, 9).encodeRouterTopK(nullptr, dw, dx, dbias, didx, dwt, e, d, dlg, t);
  } catch (const mf::Error& err) {
    threw = err.status == MF_ERR_TOPK;
  }
  EXPECT(threw, "top-k above the maximum is MF_ERR_TOPK");
  for (void* p : {(void*)dw, (void*)dx, (void*)dbias, (void*)dgs, (void*)didx, (void*)dwt, (void*)dgam, (void*)dlg})
    HIP_OK(hipFree(p));
}

int main(int argc, char** argv) {
  const std::string mode = argc > 1 ? argv[1] : "cpu";
  test_grouping();
  if (mode == "gpu") {
    test_layer();
    mf::MetalContext context(0);
    test_family_routers(context);
  }
  std::printf(g_fail ? "mirror_test: %d FAILED\n" : "mirror_test: ok\n", g_fail);
  return g_fail ? 1 : 0;
}
