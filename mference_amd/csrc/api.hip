// The C ABI (include/mfmoe.h): argument validation, workspace ownership and
// kernel dispatch.  Bad arguments return a negative status and launch nothing.
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <new>
#include <vector>

#include "mf_internal.h"

namespace {

constexpr int kAbiVersion = 2;  // 2: mf_moe_config.gate_group_size
// rows of router logits a handle holds for mf_moe_router calls that bring no logits buffer
constexpr uint32_t kRouterRows = 256;

mf_status fail_hip(mf_ctx* ctx, hipError_t e, const char* what) {
  if (ctx) snprintf(ctx->hip_error, sizeof ctx->hip_error, "%s: %s", what, hipGetErrorString(e));
  return e == hipErrorOutOfMemory ? MF_ERR_OUT_OF_MEMORY : MF_ERR_LAUNCH;
}

#define MF_HIP(ctx, call)                                  \
  do {                                                     \
    hipError_t e_ = (call);                                \
    if (e_ != hipSuccess) return fail_hip(ctx, e_, #call); \
  } while (0)

bool bits_ok(int bits) { return bits == MF_BITS_4 || bits == MF_BITS_2 || bits == MF_BITS_TERNARY; }
// the calls that also take 8-bit affine tensors: quantizer, dequantizer, GEMV
bool bits_ok_rows(int bits) { return bits_ok(bits) || bits == MF_BITS_8; }

bool qtensor_ok(const mf_qtensor& q, int bits) {
  if (!q.weights || !q.scales || !mf::aligned2(q.scales)) return false;
  if (bits != MF_BITS_TERNARY && (!q.biases || !mf::aligned2(q.biases))) return false;
  return true;
}

bool offsets_ok(const mf_expert_offsets& o, int bits) {
  uint32_t tables = o.gate_s | o.up_s | o.down_s;
  if (bits != MF_BITS_TERNARY) tables |= o.gate_b | o.up_b | o.down_b;
  return (tables & 1u) == 0;
}

size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace

extern "C" {

int mf_abi_version(void) { return kAbiVersion; }

const char* mf_status_string(mf_status s) {
  switch (s) {
    case MF_OK: return "ok";
    case MF_ERR_INVALID_ARGUMENT: return "invalid argument";
    case MF_ERR_DIMENSION_MISMATCH: return "dimension mismatch";
    case MF_ERR_UNSUPPORTED_BITS: return "unsupported weight bits";
    case MF_ERR_SCRATCH_TOO_SMALL: return "scratch too small";
    case MF_ERR_NO_DEVICE: return "no device";
    case MF_ERR_OUT_OF_MEMORY: return "out of device memory";
    case MF_ERR_LAUNCH: return "HIP call failed";
    case MF_ERR_QUERY_COUNT: return "queryCount must be non-negative";
    case MF_ERR_TOPK: return "topK must be positive";
    case MF_ERR_NUM_EXPERTS: return "numExperts must be positive";
    case MF_ERR_TILE_EXPERT_COUNT: return "tileExpertCount must be in 1...16";
    case MF_ERR_PAIR_COUNT: return "route pair count mismatch";
    case MF_ERR_TOKEN_RANGE: return "route token out of range";
    case MF_ERR_RANK_RANGE: return "route rank out of range";
    case MF_ERR_EXPERT_RANGE: return "route expert out of range";
    case MF_ERR_DUPLICATE_TOKEN_RANK: return "duplicate route pair";
    case MF_ERR_SORT_KEY_COUNT: return "expert sort key count mismatch";
  }
  return "unknown status";
}

mf_status mf_ctx_create(int device, mf_ctx** out) {
  if (!out) return MF_ERR_INVALID_ARGUMENT;
  *out = nullptr;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count)
    return MF_ERR_NO_DEVICE;
  if (hipSetDevice(device) != hipSuccess) return MF_ERR_NO_DEVICE;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device) != hipSuccess) return MF_ERR_NO_DEVICE;
  auto* ctx = new (std::nothrow) mf_ctx();
  if (!ctx) return MF_ERR_OUT_OF_MEMORY;
  ctx->device = device;
  ctx->num_cu = prop.multiProcessorCount;
  if (mf::static_scratch_init(device) != hipSuccess) {  // mf_shared_expert_static's array on this GPU
    delete ctx;
    return MF_ERR_NO_DEVICE;
  }
  *out = ctx;
  return MF_OK;
}

void mf_ctx_destroy(mf_ctx* ctx) { delete ctx; }

const char* mf_last_hip_error(const mf_ctx* ctx) { return ctx ? ctx->hip_error : ""; }

/* ----------------------------------------------------------------- format */

mf_status mf_quantize_affine(mf_ctx* ctx, mf_stream stream, const float* w, size_t rows,
                             size_t n, mf_bits bits, void* packed, uint16_t* scales,
                             uint16_t* biases) {
  if (!ctx || !w || !packed || !scales || !biases) return MF_ERR_INVALID_ARGUMENT;
  if (bits != MF_BITS_4 && bits != MF_BITS_2 && bits != MF_BITS_8) return MF_ERR_UNSUPPORTED_BITS;
  if (n % MF_GROUP_SIZE != 0) return MF_ERR_INVALID_ARGUMENT;
  if (!mf::aligned16(w) || !mf::aligned2(packed) || !mf::aligned2(scales) || !mf::aligned2(biases))
    return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(ctx, mf::launch_quantize(static_cast<hipStream_t>(stream), w, rows, n, bits, packed,
                                  scales, biases));
  return MF_OK;
}

mf_status mf_dequantize(mf_ctx* ctx, mf_stream stream, mf_qtensor q, size_t rows, size_t n,
                        mf_bits bits, float* out) {
  if (!ctx || !out) return MF_ERR_INVALID_ARGUMENT;
  if (!bits_ok_rows(bits)) return MF_ERR_UNSUPPORTED_BITS;
  if (!qtensor_ok(q, bits) || n % MF_GROUP_SIZE != 0) return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(ctx, mf::launch_dequantize(static_cast<hipStream_t>(stream), q, rows, n, bits, out));
  return MF_OK;
}

/* ------------------------------------------------------------------- GEMV */

mf_status mf_gemv(mf_ctx* ctx, mf_stream stream, mf_qtensor w, mf_bits bits, const uint16_t* x,
                  void* y, uint32_t m, uint32_t n, uint32_t t, int out_f32) {
  if (!ctx || !x || !y) return MF_ERR_INVALID_ARGUMENT;
  if (!bits_ok_rows(bits)) return MF_ERR_UNSUPPORTED_BITS;
  if (!qtensor_ok(w, bits) || !mf::aligned2(x) || !mf::aligned2(y)) return MF_ERR_INVALID_ARGUMENT;
  if (n == 0 || n % MF_GROUP_SIZE != 0 || t == 0 || t > MF_MAX_TOKENS)
    return MF_ERR_INVALID_ARGUMENT;
  if (m == 0) return MF_OK;
  MF_HIP(ctx, mf::launch_gemv(static_cast<hipStream_t>(stream), w, bits, x, y, m, n, t,
                              out_f32 != 0));
  return MF_OK;
}

mf_status mf_silu_mul(mf_ctx* ctx, mf_stream stream, const uint16_t* gate, const uint16_t* up,
                      uint16_t* out, uint32_t count) {
  if (!ctx || !gate || !up || !out) return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(ctx, mf::launch_silu_mul(static_cast<hipStream_t>(stream), gate, up, out, count));
  return MF_OK;
}

mf_status mf_sigmoid_scalar_mul(mf_ctx* ctx, mf_stream stream, uint16_t* y, const uint16_t* gate,
                                uint32_t row, uint32_t rows) {
  if (!ctx || !y || !gate) return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(ctx, mf::launch_sigmoid_scalar_mul(static_cast<hipStream_t>(stream), y, gate, row, rows));
  return MF_OK;
}

mf_status mf_residual_add(mf_ctx* ctx, mf_stream stream, uint16_t* hidden, const uint16_t* delta,
                          uint32_t count) {
  if (!ctx || !hidden || !delta) return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(ctx, mf::launch_residual_add(static_cast<hipStream_t>(stream), hidden, delta, count));
  return MF_OK;
}

mf_status mf_residual_rmsnorm(mf_ctx* ctx, mf_stream stream, uint16_t* hidden, const uint16_t* delta,
                              const uint16_t* weight, uint16_t* out, uint32_t d, uint32_t t, float eps) {
  if (!ctx || !hidden || !weight || !out) return MF_ERR_INVALID_ARGUMENT;
  if (d == 0) return MF_ERR_DIMENSION_MISMATCH;
  if (!mf::aligned2(hidden) || !mf::aligned2(weight) || !mf::aligned2(out) || (delta && !mf::aligned2(delta)))
    return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(ctx, mf::launch_residual_rmsnorm(static_cast<hipStream_t>(stream), hidden, delta, weight, out, d, t, eps));
  return MF_OK;
}

size_t mf_shared_expert_scratch_bytes(uint32_t d, uint32_t f, uint32_t t) {
  if (t <= MF_MAX_TOKENS || d % MF_GROUP_SIZE || f % MF_GROUP_SIZE) return static_cast<size_t>(t) * f * sizeof(uint16_t);
  return mf::dense_mlp_scratch_bytes(d, f, t);
}

mf_status mf_shared_expert(mf_ctx* ctx, mf_stream stream, const uint16_t* x, mf_qtensor gate,
                           mf_qtensor up, mf_qtensor down, mf_bits bits, uint32_t d, uint32_t f,
                           uint32_t t, uint16_t* y, uint16_t* scratch_act,
                           size_t scratch_act_bytes) {
  if (!ctx || !x || !y || !scratch_act) return MF_ERR_INVALID_ARGUMENT;
  if (!bits_ok(bits)) return MF_ERR_UNSUPPORTED_BITS;
  if (d == 0 || f == 0 || d % MF_GROUP_SIZE != 0 || f % MF_GROUP_SIZE != 0)
    return MF_ERR_DIMENSION_MISMATCH;
  if (t == 0 || t > MF_MAX_ROWS) return MF_ERR_INVALID_ARGUMENT;
  if (!qtensor_ok(gate, bits) || !qtensor_ok(up, bits) || !qtensor_ok(down, bits))
    return MF_ERR_INVALID_ARGUMENT;
  if (!mf::aligned2(x) || !mf::aligned2(y) || !mf::aligned2(scratch_act))
    return MF_ERR_INVALID_ARGUMENT;
  if (scratch_act_bytes < static_cast<size_t>(t) * f * sizeof(uint16_t))
    return MF_ERR_SCRATCH_TOO_SMALL;
  auto s = static_cast<hipStream_t>(stream);
  // PrefillSharedExpert.encodeBlock (PrefillSharedExpert.swift:114-172): from 32 rows on the projections
  // go through the matrix-core matmul when the shape allows and the scratch holds its staging rows
  if (t >= 32 && mf::dense_mlp_takes(gate, up, down, x, y, scratch_act, d, f, t) &&
      scratch_act_bytes >= mf::dense_mlp_scratch_bytes(d, f, t)) {
    MF_HIP(ctx, mf::launch_dense_mlp(s, gate, up, down, bits, x, y, d, f, t, scratch_act));
    return MF_OK;
  }
  // row by row otherwise (PrefillSharedExpert.swift:174-190), MF_MAX_TOKENS rows per pair of launches
  for (uint32_t t0 = 0; t0 < t; t0 += MF_MAX_TOKENS) {
    const uint32_t tc = std::min<uint32_t>(t - t0, MF_MAX_TOKENS);
    uint16_t* act = scratch_act + static_cast<size_t>(t0) * f;
    MF_HIP(ctx, mf::launch_gate_up_act(s, gate, up, bits, x + static_cast<size_t>(t0) * d, act, f, d, tc));
    MF_HIP(ctx, mf::launch_gemv(s, down, bits, act, y + static_cast<size_t>(t0) * d, d, f, tc, false));
  }
  return MF_OK;
}

mf_status mf_shared_expert_int8(mf_ctx* ctx, mf_stream stream, const uint16_t* x, mf_qtensor gate, mf_qtensor up,
                                mf_qtensor down, uint32_t d, uint32_t f, uint32_t t, int silu_activation,
                                uint16_t* y, uint16_t* scratch_act, size_t scratch_act_bytes) {
  if (!ctx || !x || !y || !scratch_act) return MF_ERR_INVALID_ARGUMENT;
  if (d == 0 || f == 0 || d % MF_GROUP_SIZE != 0 || f % MF_GROUP_SIZE != 0) return MF_ERR_DIMENSION_MISMATCH;
  if (t == 0 || t > MF_MAX_ROWS) return MF_ERR_INVALID_ARGUMENT;
  if (!qtensor_ok(gate, MF_BITS_8) || !qtensor_ok(up, MF_BITS_8) || !qtensor_ok(down, MF_BITS_8))
    return MF_ERR_INVALID_ARGUMENT;
  if (!mf::aligned2(x) || !mf::aligned2(y) || !mf::aligned2(scratch_act)) return MF_ERR_INVALID_ARGUMENT;
  if (scratch_act_bytes < static_cast<size_t>(t) * f * sizeof(uint16_t)) return MF_ERR_SCRATCH_TOO_SMALL;
  auto s = static_cast<hipStream_t>(stream);
  // rows in runs that keep the launch's wave count in range
  const uint32_t step = 1u << 14;
  for (uint32_t t0 = 0; t0 < t; t0 += step) {
    const uint32_t tc = std::min<uint32_t>(t - t0, step);
    uint16_t* act = scratch_act + static_cast<size_t>(t0) * f;
    MF_HIP(ctx, mf::launch_gate_up_act_q8(s, gate, up, x + static_cast<size_t>(t0) * d, act, f, d, tc, silu_activation != 0));
    MF_HIP(ctx, mf::launch_gemv(s, down, MF_BITS_8, act, y + static_cast<size_t>(t0) * d, d, f, tc, false));
  }
  return MF_OK;
}

size_t mf_qmm_workspace_bytes(uint32_t m, uint32_t n, uint32_t k) {
  if (m == 0 || n == 0 || k == 0 || k % MF_GROUP_SIZE) return 0;
  return mf::dense_qmm_workspace_bytes(m, n, k);
}

// the conditions under which MPPPrefillInt4QMM.encode returns .unavailable (MPPPrefillInt4QMM.swift:43-55),
// then the kernel the call takes
static int qmm_path(mf_qtensor w, mf_bits bits, const uint16_t* x, const void* y, uint32_t m, uint32_t n, uint32_t k,
                    const void* workspace, size_t workspace_bytes) {
  if (!x || !y) return MF_ERR_INVALID_ARGUMENT;
  if (!bits_ok(bits)) return MF_ERR_UNSUPPORTED_BITS;
  if (m == 0 || n == 0 || k == 0 || k % MF_GROUP_SIZE != 0 || m > MF_MAX_ROWS) return MF_ERR_DIMENSION_MISMATCH;
  if (!qtensor_ok(w, bits) || !mf::aligned2(x) || !mf::aligned2(y)) return MF_ERR_INVALID_ARGUMENT;
  if (workspace && mf::aligned16(workspace) && mf::dense_qmm_takes(w, bits, x, y, m, n, k) &&
      workspace_bytes >= mf::dense_qmm_workspace_bytes(m, n, k))
    return MF_QMM_PATH_MATRIX_CORE;
  return MF_QMM_PATH_ROWS;
}

int mf_qmm_path(mf_qtensor w, mf_bits bits, const uint16_t* x, const void* y, uint32_t m, uint32_t n, uint32_t k,
                const void* workspace, size_t workspace_bytes) {
  return qmm_path(w, bits, x, y, m, n, k, workspace, workspace_bytes);
}

mf_status mf_qmm(mf_ctx* ctx, mf_stream stream, mf_qtensor w, mf_bits bits, const uint16_t* x, void* y, uint32_t m,
                 uint32_t n, uint32_t k, int out_f32, void* workspace, size_t workspace_bytes) {
  if (!ctx) return MF_ERR_INVALID_ARGUMENT;
  const int path = qmm_path(w, bits, x, y, m, n, k, workspace, workspace_bytes);
  if (path < 0) return static_cast<mf_status>(path);
  auto s = static_cast<hipStream_t>(stream);
  if (path == MF_QMM_PATH_MATRIX_CORE) {
    MF_HIP(ctx, mf::launch_dense_qmm(s, w, bits, x, y, m, n, k, out_f32 != 0, workspace));
    return MF_OK;
  }
  // any other shape or alignment: the rows MF_MAX_TOKENS at a time through the GEMV kernels
  const size_t ybytes = out_f32 ? sizeof(float) : sizeof(uint16_t);
  for (uint32_t m0 = 0; m0 < m; m0 += MF_MAX_TOKENS) {
    const uint32_t mc = std::min<uint32_t>(m - m0, MF_MAX_TOKENS);
    MF_HIP(ctx, mf::launch_gemv(s, w, bits, x + static_cast<size_t>(m0) * k,
                                static_cast<uint8_t*>(y) + static_cast<size_t>(m0) * n * ybytes, n, k, mc, out_f32 != 0));
  }
  return MF_OK;
}

static mf_status blob_layout(uint32_t d, uint32_t f, mf_bits bits, uint32_t align, bool ternary_bias_tables,
                             mf_expert_offsets* offsets, size_t* blob_bytes, size_t* stride);

mf_status mf_expert_blob_layout(uint32_t d, uint32_t f, mf_bits bits, uint32_t align, mf_expert_offsets* offsets,
                                size_t* blob_bytes, size_t* stride) {
  return blob_layout(d, f, bits, align, false, offsets, blob_bytes, stride);
}

mf_status mf_expert_blob_layout_repacked(uint32_t d, uint32_t f, mf_bits bits, uint32_t align,
                                         mf_expert_offsets* offsets, size_t* blob_bytes, size_t* stride) {
  return blob_layout(d, f, bits, align, true, offsets, blob_bytes, stride);
}

static mf_status blob_layout(uint32_t d, uint32_t f, mf_bits bits, uint32_t align, bool ternary_bias_tables,
                             mf_expert_offsets* offsets, size_t* blob_bytes, size_t* stride) {
  if (!offsets) return MF_ERR_INVALID_ARGUMENT;
  if (!bits_ok(bits)) return MF_ERR_UNSUPPORTED_BITS;
  if (d == 0 || f == 0 || d % MF_GROUP_SIZE != 0 || f % MF_GROUP_SIZE != 0) return MF_ERR_DIMENSION_MISMATCH;
  if (align == 0) return MF_ERR_INVALID_ARGUMENT;
  const uint64_t code_bits = bits == MF_BITS_4 ? 4 : 2;
  const uint64_t gu_w = static_cast<uint64_t>(f) * d * code_bits / 8, gu_s = static_cast<uint64_t>(f) * (d / MF_GROUP_SIZE) * 2;
  const uint64_t dn_w = static_cast<uint64_t>(d) * f * code_bits / 8, dn_s = static_cast<uint64_t>(d) * (f / MF_GROUP_SIZE) * 2;
  const bool has_bias = bits != MF_BITS_TERNARY || ternary_bias_tables;
  const uint64_t sizes[3][2] = {{gu_w, gu_s}, {gu_w, gu_s}, {dn_w, dn_s}};
  uint32_t* out[3][3] = {{&offsets->gate_w, &offsets->gate_s, &offsets->gate_b},
                         {&offsets->up_w, &offsets->up_s, &offsets->up_b},
                         {&offsets->down_w, &offsets->down_s, &offsets->down_b}};
  uint64_t pos = 0;
  for (int p = 0; p < 3; ++p) {
    *out[p][0] = static_cast<uint32_t>(pos); pos += sizes[p][0];
    *out[p][1] = static_cast<uint32_t>(pos); pos += sizes[p][1];
    *out[p][2] = has_bias ? static_cast<uint32_t>(pos) : 0u;
    if (has_bias) pos += sizes[p][1];
    if (pos > 0xFFFFFFFFull) return MF_ERR_DIMENSION_MISMATCH;  // MoEExpertOffsets holds 32-bit offsets
  }
  if (blob_bytes) *blob_bytes = static_cast<size_t>(pos);
  if (stride) *stride = static_cast<size_t>((pos + align - 1) / align * align);
  return MF_OK;
}

/* ---------------------------------------------------------- MoE operator */

mf_status mf_moe_config_check(const mf_moe_config* cfg) {
  if (!cfg) return MF_ERR_INVALID_ARGUMENT;
  if (!bits_ok(cfg->bits)) return MF_ERR_UNSUPPORTED_BITS;
  if (cfg->shared_f && !bits_ok(cfg->shared_bits)) return MF_ERR_UNSUPPORTED_BITS;
  if (cfg->d == 0 || cfg->d % MF_GROUP_SIZE != 0 || cfg->f == 0 || cfg->f % MF_GROUP_SIZE != 0 ||
      cfg->shared_f % MF_GROUP_SIZE != 0)
    return MF_ERR_DIMENSION_MISMATCH;
  if (cfg->num_experts == 0 || cfg->num_experts > MF_MAX_EXPERTS) return MF_ERR_INVALID_ARGUMENT;
  if (cfg->top_k == 0 || cfg->top_k > MF_MAX_TOPK) return MF_ERR_INVALID_ARGUMENT;
  if (cfg->router_mode != MF_ROUTER_TOPK_SOFTMAX && cfg->router_mode != MF_ROUTER_FULL_SOFTMAX)
    return MF_ERR_INVALID_ARGUMENT;
  if (cfg->router_mode == MF_ROUTER_FULL_SOFTMAX && cfg->num_experts % 32 != 0)
    return MF_ERR_INVALID_ARGUMENT;
  if (cfg->maple_rounding > 1) return MF_ERR_INVALID_ARGUMENT;
  if (cfg->gate_group_size != 0 && cfg->gate_group_size != 64 &&
      !(cfg->gate_group_size == 32 && cfg->bits == MF_BITS_2))
    return MF_ERR_INVALID_ARGUMENT;
  return MF_OK;
}

mf_status mf_moe_create(mf_ctx* ctx, const mf_moe_config* cfg, mf_moe** out) {
  if (!ctx || !cfg || !out) return MF_ERR_INVALID_ARGUMENT;
  *out = nullptr;
  const mf_status cfg_status = mf_moe_config_check(cfg);
  if (cfg_status != MF_OK) return cfg_status;

  auto* h = new (std::nothrow) mf_moe();
  if (!h) return MF_ERR_OUT_OF_MEMORY;
  h->ctx = ctx;
  h->cfg = *cfg;
  const size_t T = MF_MAX_TOKENS;
  size_t pos = 0;
  auto take = [&](size_t bytes) {
    size_t at = pos;
    pos = round_up(pos + bytes, 256);
    return at;
  };
  const size_t o_logits = take(kRouterRows * cfg->num_experts * sizeof(float));
  const size_t o_idx = take(T * cfg->top_k * sizeof(uint32_t));
  const size_t o_w = take(T * cfg->top_k * sizeof(float));
  const size_t o_acts = take(T * cfg->top_k * cfg->f * sizeof(uint16_t));
  const size_t o_sact = take(T * std::max<uint32_t>(cfg->shared_f, 64) * sizeof(uint16_t));
  const size_t o_sy = take(T * cfg->d * sizeof(uint16_t));
  const size_t o_gate = take(T * sizeof(uint16_t));
  const size_t o_xn = take(T * cfg->d * sizeof(uint16_t));
  const size_t o_tlogits = take(T * cfg->num_experts * sizeof(uint64_t));
  const size_t o_tsact = take(T * (std::max<uint32_t>(cfg->shared_f, 64) + 4) * sizeof(uint32_t));
  const size_t o_tacts = take(T * cfg->top_k * cfg->f * sizeof(uint32_t));
  const size_t o_epoch = take(512 * sizeof(uint32_t));
  const size_t o_status = take(64);
  const size_t o_group = take(mf::group_scratch_words() * sizeof(uint32_t));
  h->ws_bytes = pos;
  if (hipSetDevice(ctx->device) != hipSuccess) {
    delete h;
    return MF_ERR_NO_DEVICE;
  }
  hipError_t e = hipMalloc(&h->ws_base, h->ws_bytes);
  if (e != hipSuccess) {
    delete h;
    return fail_hip(ctx, e, "hipMalloc(workspace)");
  }
  e = hipMemset(h->ws_base, 0, h->ws_bytes);
  if (e != hipSuccess) {
    (void)hipFree(h->ws_base);
    delete h;
    return fail_hip(ctx, e, "hipMemset(workspace)");
  }
  auto* b = static_cast<uint8_t*>(h->ws_base);
  h->ws.logits = reinterpret_cast<float*>(b + o_logits);
  h->ws.idx = reinterpret_cast<uint32_t*>(b + o_idx);
  h->ws.w = reinterpret_cast<float*>(b + o_w);
  h->ws.acts = reinterpret_cast<uint16_t*>(b + o_acts);
  h->ws.shared_act = reinterpret_cast<uint16_t*>(b + o_sact);
  h->ws.shared_y = reinterpret_cast<uint16_t*>(b + o_sy);
  h->ws.gate = reinterpret_cast<uint16_t*>(b + o_gate);
  h->ws.xn = reinterpret_cast<uint16_t*>(b + o_xn);
  h->ws.t_logits = reinterpret_cast<unsigned long long*>(b + o_tlogits);
  h->ws.t_sact = reinterpret_cast<uint32_t*>(b + o_tsact);
  h->ws.t_acts = reinterpret_cast<uint32_t*>(b + o_tacts);
  h->ws.epoch = reinterpret_cast<uint32_t*>(b + o_epoch);
  h->ws.status = reinterpret_cast<uint32_t*>(b + o_status);
  h->ws.group_tmp = reinterpret_cast<uint32_t*>(b + o_group);
  *out = h;
  return MF_OK;
}

void mf_moe_destroy(mf_moe* h) {
  if (!h) return;
  if (h->ws_base) (void)hipFree(h->ws_base);
  delete h;
}

namespace {
// bf16 router rows for t tokens: the batched kernels of the prefill router from 16 tokens on (the same
// bits: they keep the summation order of the one-row kernel), else one wave per (token, row)
hipError_t family_logits(hipStream_t s, const uint16_t* w, const uint16_t* x, uint32_t rows, uint32_t d,
                         uint32_t t, uint32_t x_stride, float* logits) {
  const bool al = mf::aligned16(w) && mf::aligned16(x) && x_stride % 8 == 0;
  if (t >= 16 && al && ((d % 512 == 0 && rows % 32 == 0) || d <= 4096))
    return mf::launch_prefill_router(s, w, x, rows, d, t, x_stride, logits);
  return mf::launch_router_logits(s, w, x, rows, d, t, x_stride, logits, nullptr);
}
}  // namespace

mf_status mf_moe_router(mf_moe* h, mf_stream stream, const uint16_t* router_w, const uint16_t* x,
                        uint32_t t, uint32_t x_stride, uint32_t* out_idx, float* out_w,
                        float* out_logits) {
  if (!h || !router_w || !x || !out_idx || !out_w) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_ROWS || x_stride < h->cfg.d) return MF_ERR_INVALID_ARGUMENT;
  if (!mf::aligned2(router_w) || !mf::aligned2(x)) return MF_ERR_INVALID_ARGUMENT;
  auto s = static_cast<hipStream_t>(stream);
  const uint32_t e = h->cfg.num_experts;
  // logits go to the caller's buffer when given, else through the handle's (kRouterRows rows at a time)
  for (uint32_t t0 = 0; t0 < t;) {
    const uint32_t tc = out_logits ? t - t0 : std::min<uint32_t>(t - t0, kRouterRows);
    float* lg = out_logits ? out_logits + static_cast<size_t>(t0) * e : h->ws.logits;
    MF_HIP(h->ctx, family_logits(s, router_w, x + static_cast<size_t>(t0) * x_stride, e, h->cfg.d, tc, x_stride, lg));
    MF_HIP(h->ctx, mf::launch_topk(s, lg, e, h->cfg.top_k, tc, h->cfg.router_mode,
                                   out_idx + static_cast<size_t>(t0) * h->cfg.top_k,
                                   out_w + static_cast<size_t>(t0) * h->cfg.top_k));
    t0 += tc;
  }
  return MF_OK;
}

namespace {
// the checks the four family routers share
mf_status family_args_ok(const mf_ctx* ctx, const void* w, const uint16_t* x, uint32_t t, uint32_t x_stride,
                         uint32_t rows, uint32_t d, uint32_t top_k, const float* logits) {
  if (!ctx || !w || !x || !logits) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_ROWS || d == 0 || d % 8 != 0 || x_stride < d) return MF_ERR_INVALID_ARGUMENT;
  if (rows == 0 || rows > MF_MAX_EXPERTS) return MF_ERR_NUM_EXPERTS;
  if (top_k == 0 || top_k > MF_MAX_TOPK) return MF_ERR_TOPK;
  if (!mf::aligned2(x) || (reinterpret_cast<uintptr_t>(logits) & 3u)) return MF_ERR_INVALID_ARGUMENT;
  return MF_OK;
}
}  // namespace

mf_status mf_router_sqrtsoftplus(mf_ctx* ctx, mf_stream stream, const uint16_t* router_w, const uint16_t* x,
                                 uint32_t t, uint32_t x_stride, uint32_t num_experts, uint32_t d,
                                 uint32_t top_k, const float* correction_bias, float route_scale,
                                 float* logits, uint32_t* out_idx, float* out_w) {
  const mf_status st = family_args_ok(ctx, router_w, x, t, x_stride, num_experts, d, top_k, logits);
  if (st != MF_OK) return st;
  if (!correction_bias || !out_idx || !out_w || !mf::aligned2(router_w)) return MF_ERR_INVALID_ARGUMENT;
  auto s = static_cast<hipStream_t>(stream);
  MF_HIP(ctx, family_logits(s, router_w, x, num_experts, d, t, x_stride, logits));
  MF_HIP(ctx, mf::launch_select_sqrtsoftplus(s, logits, correction_bias, num_experts, top_k, t, route_scale,
                                             out_idx, out_w));
  return MF_OK;
}

mf_status mf_router_hash_weights(mf_ctx* ctx, mf_stream stream, const uint16_t* router_w, const uint16_t* x,
                                 uint32_t t, uint32_t x_stride, uint32_t num_experts, uint32_t d,
                                 uint32_t top_k, const uint32_t* indices, float route_scale, float* logits,
                                 float* out_w) {
  const mf_status st = family_args_ok(ctx, router_w, x, t, x_stride, num_experts, d, top_k, logits);
  if (st != MF_OK) return st;
  if (!indices || !out_w || !mf::aligned2(router_w)) return MF_ERR_INVALID_ARGUMENT;
  auto s = static_cast<hipStream_t>(stream);
  MF_HIP(ctx, family_logits(s, router_w, x, num_experts, d, t, x_stride, logits));
  MF_HIP(ctx, mf::launch_hash_weights(s, logits, indices, num_experts, top_k, t, route_scale, out_w));
  return MF_OK;
}

mf_status mf_router_inkling(mf_ctx* ctx, mf_stream stream, const uint16_t* router_w, const uint16_t* x,
                            uint32_t t, uint32_t x_stride, uint32_t n_routed, uint32_t n_shared, uint32_t d,
                            uint32_t top_k, const float* gate_bias, const float* global_scale,
                            float route_scale, float* logits, uint32_t* out_idx, float* out_w,
                            float* out_gammas) {
  if (n_shared > 8) return MF_ERR_INVALID_ARGUMENT;
  const mf_status st = family_args_ok(ctx, router_w, x, t, x_stride, n_routed, d, top_k, logits);
  if (st != MF_OK) return st;
  if (!gate_bias || !global_scale || !out_idx || !out_w || (n_shared && !out_gammas) ||
      !mf::aligned2(router_w))
    return MF_ERR_INVALID_ARGUMENT;
  auto s = static_cast<hipStream_t>(stream);
  MF_HIP(ctx, family_logits(s, router_w, x, n_routed + n_shared, d, t, x_stride, logits));
  MF_HIP(ctx, mf::launch_select_inkling(s, logits, gate_bias, global_scale, n_routed, n_shared, top_k, t,
                                        route_scale, out_idx, out_w, out_gammas));
  return MF_OK;
}

mf_status mf_router_gemma4(mf_ctx* ctx, mf_stream stream, const uint8_t* router_codes,
                           const uint16_t* router_scales, const uint16_t* router_biases, const uint16_t* x,
                           uint32_t t, uint32_t x_stride, const uint16_t* effective_scale,
                           const uint16_t* per_expert_scale, uint32_t num_experts, uint32_t d, uint32_t top_k,
                           float* logits, uint32_t* out_idx, float* out_w) {
  const mf_status st = family_args_ok(ctx, router_codes, x, t, x_stride, num_experts, d, top_k, logits);
  if (st != MF_OK) return st;
  if (d % MF_GROUP_SIZE != 0) return MF_ERR_DIMENSION_MISMATCH;
  if (!router_scales || !router_biases || !effective_scale || !per_expert_scale || !out_idx || !out_w)
    return MF_ERR_INVALID_ARGUMENT;
  if (!mf::aligned2(router_scales) || !mf::aligned2(router_biases) || !mf::aligned2(effective_scale) ||
      !mf::aligned2(per_expert_scale))
    return MF_ERR_INVALID_ARGUMENT;
  auto s = static_cast<hipStream_t>(stream);
  MF_HIP(ctx, mf::launch_router_logits_int8(s, router_codes, router_scales, router_biases, x, effective_scale,
                                            num_experts, d, t, x_stride, logits));
  MF_HIP(ctx, mf::launch_select_scaled_softmax(s, logits, per_expert_scale, num_experts, top_k, t, out_idx,
                                               out_w));
  return MF_OK;
}

mf_status mf_moe_phase1(mf_moe* h, mf_stream stream, const void* expert_base,
                        size_t expert_stride, const mf_expert_offsets* offsets,
                        const uint32_t* idx, const uint16_t* x, uint32_t t, uint32_t x_stride,
                        uint16_t* acts) {
  if (!h || !expert_base || !offsets || !idx || !x || !acts) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_ROWS || x_stride < h->cfg.d) return MF_ERR_INVALID_ARGUMENT;
  if (!offsets_ok(*offsets, h->cfg.bits) || !mf::aligned2(expert_base) || (expert_stride & 1) ||
      !mf::aligned2(x) || !mf::aligned2(acts))
    return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(h->ctx, mf::launch_phase1(static_cast<hipStream_t>(stream), h->cfg, expert_base,
                                   expert_stride, *offsets, idx, x, t, x_stride, acts));
  return MF_OK;
}

mf_status mf_moe_phase1_subset(mf_moe* h, mf_stream stream, const void* expert_base,
                               size_t expert_stride, const mf_expert_offsets* offsets,
                               const uint32_t* idx, const uint16_t* x, uint32_t t, uint32_t x_stride,
                               uint16_t* acts, const uint32_t* active_slots, uint32_t active_count) {
  if (active_count == 0) return MF_OK;  // MoE.swift:269
  if (!active_slots || (reinterpret_cast<uintptr_t>(active_slots) & 3u)) return MF_ERR_INVALID_ARGUMENT;
  if (!h || !expert_base || !offsets || !idx || !x || !acts) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_ROWS || x_stride < h->cfg.d) return MF_ERR_INVALID_ARGUMENT;
  if (!offsets_ok(*offsets, h->cfg.bits) || !mf::aligned2(expert_base) || (expert_stride & 1) ||
      !mf::aligned2(x) || !mf::aligned2(acts))
    return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(h->ctx, mf::launch_phase1(static_cast<hipStream_t>(stream), h->cfg, expert_base, expert_stride,
                                   *offsets, idx, x, t, x_stride, acts, active_slots, active_count));
  return MF_OK;
}

mf_status mf_moe_slot_lookup(mf_moe* h, mf_stream stream, const uint32_t* idx, uint32_t t,
                             const int16_t* slot_of, uint64_t slot_stride, uint64_t* out_slot_offsets,
                             uint32_t* out_all_hit) {
  if (!h || !idx || !slot_of || !out_slot_offsets || !out_all_hit) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_TOKENS) return MF_ERR_INVALID_ARGUMENT;
  if ((reinterpret_cast<uintptr_t>(out_slot_offsets) & 7u) || (reinterpret_cast<uintptr_t>(slot_of) & 1u))
    return MF_ERR_INVALID_ARGUMENT;
  // the routed phases read every blob with 16-byte loads when the slab is 16-byte aligned: the offsets
  // this call writes have to keep that alignment
  if (slot_stride % 16 != 0) return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(h->ctx, mf::launch_slot_lookup(static_cast<hipStream_t>(stream), idx, slot_of, t * h->cfg.top_k,
                                        h->cfg.num_experts, slot_stride, out_slot_offsets, out_all_hit));
  return MF_OK;
}

mf_status mf_moe_phase1_slots(mf_moe* h, mf_stream stream, const void* slab, const uint64_t* slot_offsets,
                              const uint32_t* all_hit, const mf_expert_offsets* offsets, const uint16_t* x,
                              uint32_t t, uint32_t x_stride, uint16_t* acts) {
  if (!h || !slot_offsets || !offsets || !x || !acts) return MF_ERR_INVALID_ARGUMENT;
  // (one guard word covers one lookup, and a lookup covers at most MF_MAX_TOKENS rows)
  if (t == 0 || t > MF_MAX_TOKENS || x_stride < h->cfg.d) return MF_ERR_INVALID_ARGUMENT;
  if (!offsets_ok(*offsets, h->cfg.bits) || !mf::aligned2(slab) || !mf::aligned2(x) || !mf::aligned2(acts) ||
      (reinterpret_cast<uintptr_t>(slot_offsets) & 7u))
    return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(h->ctx, mf::launch_phase1(static_cast<hipStream_t>(stream), h->cfg, slab, 0, *offsets, nullptr, x, t,
                                   x_stride, acts, nullptr, 0, slot_offsets, all_hit));
  return MF_OK;
}

mf_status mf_moe_phase2_slots(mf_moe* h, mf_stream stream, const void* slab, const uint64_t* slot_offsets,
                              const uint32_t* all_hit, const mf_expert_offsets* offsets, const float* w,
                              const uint16_t* acts, const uint16_t* residual, uint32_t t, uint16_t* y) {
  if (!h || !slot_offsets || !offsets || !w || !acts || !y) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_TOKENS) return MF_ERR_INVALID_ARGUMENT;
  if (!offsets_ok(*offsets, h->cfg.bits) || !mf::aligned2(slab) || !mf::aligned2(acts) || !mf::aligned2(y) ||
      (residual && !mf::aligned2(residual)) || (reinterpret_cast<uintptr_t>(slot_offsets) & 7u))
    return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(h->ctx, mf::launch_phase2(static_cast<hipStream_t>(stream), h->cfg, slab, 0, *offsets, nullptr, w, acts,
                                   residual, t, y, slot_offsets, all_hit));
  return MF_OK;
}

mf_status mf_moe_phase2(mf_moe* h, mf_stream stream, const void* expert_base,
                        size_t expert_stride, const mf_expert_offsets* offsets,
                        const uint32_t* idx, const float* w, const uint16_t* acts,
                        const uint16_t* residual, uint32_t t, uint16_t* y) {
  if (!h || !expert_base || !offsets || !idx || !w || !acts || !y) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_ROWS) return MF_ERR_INVALID_ARGUMENT;
  if (!offsets_ok(*offsets, h->cfg.bits) || !mf::aligned2(expert_base) || (expert_stride & 1) ||
      !mf::aligned2(acts) || !mf::aligned2(y) || (residual && !mf::aligned2(residual)))
    return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(h->ctx, mf::launch_phase2(static_cast<hipStream_t>(stream), h->cfg, expert_base,
                                   expert_stride, *offsets, idx, w, acts, residual, t, y));
  return MF_OK;
}

mf_status mf_moe_decode_layer(mf_moe* h, mf_stream stream, const mf_moe_layer_weights* wts,
                              const uint16_t* x, uint32_t t, uint16_t* y, uint16_t* hidden,
                              uint32_t* out_idx, float* out_w) {
  if (!h || !wts || !x || !y) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_TOKENS) return MF_ERR_INVALID_ARGUMENT;
  const mf_moe_config& c = h->cfg;
  // no router weights: the routing in out_idx / out_w is the caller's (a family router wrote it)
  const bool given = !wts->router_w;
  if ((given && (!out_idx || !out_w)) || !wts->expert_base || !offsets_ok(wts->offsets, c.bits) ||
      !mf::aligned2(wts->expert_base) || (wts->expert_stride & 1) || !mf::aligned2(x) ||
      !mf::aligned2(y) || (hidden && !mf::aligned2(hidden)))
    return MF_ERR_INVALID_ARGUMENT;
  if (c.shared_f && (!qtensor_ok(wts->shared_gate, c.shared_bits) ||
                     !qtensor_ok(wts->shared_up, c.shared_bits) ||
                     !qtensor_ok(wts->shared_down, c.shared_bits)))
    return MF_ERR_INVALID_ARGUMENT;
  if (c.shared_f && wts->w_sg_q8.weights && !qtensor_ok(wts->w_sg_q8, MF_BITS_8)) return MF_ERR_INVALID_ARGUMENT;
  auto s = static_cast<hipStream_t>(stream);
  if (h->fused && mf::fused_supported(*h, *wts, x, y, hidden, t)) {
    MF_HIP(h->ctx, mf::launch_fused_decode(s, *h, *wts, x, t, y, hidden, out_idx, out_w));
    return MF_OK;
  }
  uint32_t* idx = given ? out_idx : h->ws.idx;
  float* w = given ? out_w : h->ws.w;
  if (!given) {
    MF_HIP(h->ctx, mf::launch_router_logits(s, wts->router_w, x, c.num_experts, c.d, t, c.d,
                                            h->ws.logits, nullptr));
    MF_HIP(h->ctx, mf::launch_topk(s, h->ws.logits, c.num_experts, c.top_k, t, c.router_mode, idx, w));
  }
  const uint16_t* residual = nullptr;
  if (c.shared_f) {
    // lane order of the fused kernel: both forms of the layer give the same bits
    MF_HIP(h->ctx, mf::launch_gate_up_act(s, wts->shared_gate, wts->shared_up, c.shared_bits, x,
                                          h->ws.shared_act, c.shared_f, c.d, t, true));
    MF_HIP(h->ctx, mf::launch_gemv(s, wts->shared_down, c.shared_bits, h->ws.shared_act,
                                   h->ws.shared_y, c.d, c.shared_f, t, false, true));
    if (wts->w_sg_q8.weights) {  // the gate as the model files store it: an 8-bit row (RealForwardRunner.swift:2925-2941)
      MF_HIP(h->ctx, mf::launch_gemv(s, wts->w_sg_q8, MF_BITS_8, x, h->ws.gate, 1, c.d, t, false));
      MF_HIP(h->ctx, mf::launch_sigmoid_scalar_mul(s, h->ws.shared_y, h->ws.gate, c.d, t));
    } else if (wts->w_sg) {
      MF_HIP(h->ctx, mf::launch_router_logits(s, wts->w_sg, x, 1, c.d, t, c.d, nullptr, h->ws.gate));
      MF_HIP(h->ctx, mf::launch_sigmoid_scalar_mul(s, h->ws.shared_y, h->ws.gate, c.d, t));
    }
    residual = h->ws.shared_y;
  }
  MF_HIP(h->ctx, mf::launch_phase1(s, c, wts->expert_base, wts->expert_stride, wts->offsets, idx, x,
                                   t, c.d, h->ws.acts));
  MF_HIP(h->ctx, mf::launch_phase2(s, c, wts->expert_base, wts->expert_stride, wts->offsets, idx, w,
                                   h->ws.acts, residual, t, y));
  if (hidden) MF_HIP(h->ctx, mf::launch_residual_add(s, hidden, y, t * c.d));
  if (out_idx && !given)
    MF_HIP(h->ctx, hipMemcpyAsync(out_idx, idx, sizeof(uint32_t) * t * c.top_k,
                                  hipMemcpyDeviceToDevice, s));
  if (out_w && !given)
    MF_HIP(h->ctx, hipMemcpyAsync(out_w, w, sizeof(float) * t * c.top_k, hipMemcpyDeviceToDevice, s));
  return MF_OK;
}

mf_status mf_moe_decode_layer_normed(mf_moe* h, mf_stream stream, const mf_moe_layer_weights* wts, uint16_t* hidden,
                                     const uint16_t* delta, const uint16_t* norm_weight, float eps, uint32_t t,
                                     uint16_t* y, uint32_t* out_idx, float* out_w) {
  if (!h || !wts || !hidden || !norm_weight || !y) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_TOKENS) return MF_ERR_INVALID_ARGUMENT;
  if (!mf::aligned2(hidden) || !mf::aligned2(norm_weight) || (delta && !mf::aligned2(delta)) || !mf::aligned2(y))
    return MF_ERR_INVALID_ARGUMENT;
  const mf_moe_config& c = h->cfg;
  auto s = static_cast<hipStream_t>(stream);
  if (h->fused && wts->router_w && wts->expert_base && offsets_ok(wts->offsets, c.bits) &&
      (!c.shared_f || (qtensor_ok(wts->shared_gate, c.shared_bits) && qtensor_ok(wts->shared_up, c.shared_bits) &&
                       qtensor_ok(wts->shared_down, c.shared_bits) &&
                       (!wts->w_sg_q8.weights || qtensor_ok(wts->w_sg_q8, MF_BITS_8)))) &&
      mf::fused_norm_supported(*h, *wts, y, hidden, delta, norm_weight, t)) {
    const mf::FusedNorm norm{delta, norm_weight, eps};
    MF_HIP(h->ctx, mf::launch_fused_decode(s, *h, *wts, nullptr, t, y, hidden, out_idx, out_w, &norm));
    return MF_OK;
  }
  // two launches: the norm into the handle's rows, then the layer on them (the same bits)
  MF_HIP(h->ctx, mf::launch_residual_rmsnorm(s, hidden, delta, norm_weight, h->ws.xn, c.d, t, eps));
  return mf_moe_decode_layer(h, stream, wts, h->ws.xn, t, y, hidden, out_idx, out_w);
}

mf_status mf_moe_set_fused(mf_moe* h, int enabled) {
  if (!h) return MF_ERR_INVALID_ARGUMENT;
  h->fused = enabled != 0;
  h->generic_shape = enabled == 2;
  return MF_OK;
}

mf_status mf_moe_set_prefill_route_rounding(mf_moe* h, int narrow) {
  if (!h) return MF_ERR_INVALID_ARGUMENT;
  h->narrow_routes = narrow != 0;
  return MF_OK;
}

mf_status mf_moe_set_phase_trace(mf_moe* h, uint64_t* device_buffer, size_t bytes) {
  if (!h) return MF_ERR_INVALID_ARGUMENT;
  if (device_buffer && bytes < static_cast<size_t>(h->ctx->num_cu) * 8 * sizeof(uint64_t))
    return MF_ERR_SCRATCH_TOO_SMALL;
  h->trace = reinterpret_cast<unsigned long long*>(device_buffer);
  h->trace_bytes = device_buffer ? bytes : 0;
  return MF_OK;
}

int mf_ctx_num_cu(const mf_ctx* ctx) { return ctx ? ctx->num_cu : 0; }

mf_status mf_moe_status(mf_moe* h, mf_stream stream) {
  if (!h) return MF_ERR_INVALID_ARGUMENT;
  uint32_t word = 0;
  auto s = static_cast<hipStream_t>(stream);
  MF_HIP(h->ctx, hipMemcpyAsync(&word, h->ws.status, sizeof word, hipMemcpyDeviceToHost, s));
  MF_HIP(h->ctx, hipStreamSynchronize(s));
  if (word != 0) {
    snprintf(h->ctx->hip_error, sizeof h->ctx->hip_error,
             "fused decode layer: a bounded wait on exchanged data gave up (status word %u)", word);
    return MF_ERR_LAUNCH;
  }
  return MF_OK;
}

/* ------------------------------------------------------- ragged prefill */

mf_status mf_moe_group(mf_moe* h, mf_stream stream, const uint32_t* idx, const float* w, uint32_t t,
                       mf_pair* sorted_pairs, uint32_t* expert_offsets, uint32_t* expert_counts) {
  if (!h || !expert_offsets || !expert_counts) return MF_ERR_INVALID_ARGUMENT;
  auto s = static_cast<hipStream_t>(stream);
  if (t == 0) {  // queryCount == 0 is valid (PrefillMoEGrouping.swift:99-104): no pairs, every expert empty
    MF_HIP(h->ctx, mf::launch_group(s, nullptr, nullptr, 0, h->cfg.top_k, h->cfg.num_experts, expert_counts,
                                    expert_offsets, h->ws.group_tmp + 512, nullptr, nullptr, 0, nullptr,
                                    h->ws.group_tmp + 3 * 512, h->ws.group_tmp + 2048));
    return MF_OK;
  }
  if (!idx || !w || !sorted_pairs) return MF_ERR_INVALID_ARGUMENT;
  if (t > MF_MAX_ROWS) return MF_ERR_QUERY_COUNT;  // t * top_k stays far inside 32 bits, as in the prefill call
  uint32_t* starts = h->ws.group_tmp + 512;
  uint32_t* status = h->ws.group_tmp + 3 * 512;
  MF_HIP(h->ctx, mf::launch_group(s, idx, w, t, h->cfg.top_k, h->cfg.num_experts, expert_counts,
                                  expert_offsets, starts, sorted_pairs, nullptr, 0, nullptr, status,
                                  h->ws.group_tmp + 2048));
  return MF_OK;
}

mf_status mf_moe_group_status(mf_moe* h, mf_stream stream) {
  if (!h) return MF_ERR_INVALID_ARGUMENT;
  uint32_t word = 0;
  auto s = static_cast<hipStream_t>(stream);
  MF_HIP(h->ctx, hipMemcpyAsync(&word, h->ws.group_tmp + 3 * 512, sizeof word, hipMemcpyDeviceToHost, s));
  MF_HIP(h->ctx, hipStreamSynchronize(s));
  return word ? MF_ERR_EXPERT_RANGE : MF_OK;
}

size_t mf_moe_prefill_workspace_bytes(const mf_moe* h, uint32_t t) {
  if (!h || t == 0 || !mf::prefill_supported(h->cfg)) return 0;
  return mf::prefill_workspace_bytes(h->cfg, t);
}

mf_status mf_moe_prefill_layer(mf_moe* h, mf_stream stream, const mf_moe_layer_weights* wts,
                               const uint16_t* x, uint32_t t, uint16_t* y, void* workspace,
                               size_t workspace_bytes, uint32_t* out_idx, float* out_w) {
  if (!h || !wts || !x || !y) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_ROWS) return MF_ERR_INVALID_ARGUMENT;
  const mf_moe_config& c = h->cfg;
  if (!mf::prefill_supported(c)) {
    // 2-bit / ternary experts, or widths the matmul tiles do not divide: the same rows through
    // the decode launch, MF_MAX_TOKENS at a time (correct for every configuration, not fast)
    for (uint32_t t0 = 0; t0 < t; t0 += MF_MAX_TOKENS) {
      const uint32_t n = t - t0 < MF_MAX_TOKENS ? t - t0 : MF_MAX_TOKENS;
      const mf_status st = mf_moe_decode_layer(
          h, stream, wts, x + static_cast<size_t>(t0) * c.d, n, y + static_cast<size_t>(t0) * c.d, nullptr,
          out_idx ? out_idx + static_cast<size_t>(t0) * c.top_k : nullptr,
          out_w ? out_w + static_cast<size_t>(t0) * c.top_k : nullptr);
      if (st != MF_OK) return st;
    }
    return MF_OK;
  }
  if (!workspace) return MF_ERR_INVALID_ARGUMENT;
  if (workspace_bytes < mf::prefill_workspace_bytes(c, t)) return MF_ERR_SCRATCH_TOO_SMALL;
  const uint32_t offs = wts->offsets.gate_w | wts->offsets.up_w | wts->offsets.down_w;
  if ((!wts->router_w && (!out_idx || !out_w)) || !wts->expert_base || !offsets_ok(wts->offsets, c.bits) ||
      !mf::aligned16(wts->expert_base) || wts->expert_stride % 16 || offs % 16 ||
      !mf::aligned16(wts->router_w) || !mf::aligned16(x) || !mf::aligned16(y) ||
      !mf::aligned16(workspace) || !mf::aligned16(wts->expert_tiled))
    return MF_ERR_INVALID_ARGUMENT;
  if (c.shared_f && (!qtensor_ok(wts->shared_gate, c.shared_bits) ||
                     !qtensor_ok(wts->shared_up, c.shared_bits) ||
                     !qtensor_ok(wts->shared_down, c.shared_bits) ||
                     !mf::aligned16(wts->shared_gate.weights) || !mf::aligned16(wts->shared_up.weights) ||
                     !mf::aligned16(wts->shared_down.weights) ||
                     (wts->w_sg && !wts->w_sg_q8.weights && !mf::aligned16(wts->w_sg))))
    return MF_ERR_INVALID_ARGUMENT;
  if (c.shared_f && wts->w_sg_q8.weights && !qtensor_ok(wts->w_sg_q8, MF_BITS_8)) return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(h->ctx, mf::launch_prefill_layer(static_cast<hipStream_t>(stream), *h, *wts, x, t, y, workspace,
                                          out_idx, out_w));
  return MF_OK;
}

mf_status mf_moe_ragged_qmm(mf_moe* h, mf_stream stream, const void* expert_base, size_t expert_stride,
                            const mf_expert_offsets* offsets, const uint16_t* x, const mf_pair* sorted_pairs,
                            const uint32_t* expert_counts, uint32_t t, float* route_partials, void* workspace,
                            size_t workspace_bytes) {
  if (!h || !offsets || !x || !sorted_pairs || !expert_counts || !route_partials || !expert_base)
    return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_ROWS) return MF_ERR_QUERY_COUNT;
  const mf_moe_config& c = h->cfg;
  if (!mf::prefill_supported(c)) return MF_ERR_DIMENSION_MISMATCH;
  if (!workspace) return MF_ERR_INVALID_ARGUMENT;
  if (workspace_bytes < mf::prefill_workspace_bytes(c, t)) return MF_ERR_SCRATCH_TOO_SMALL;
  const uint32_t offs = offsets->gate_w | offsets->up_w | offsets->down_w;
  if (!offsets_ok(*offsets, c.bits) || !mf::aligned16(expert_base) || expert_stride % 16 || offs % 16 ||
      !mf::aligned16(x) || !mf::aligned16(route_partials) || !mf::aligned16(workspace) ||
      reinterpret_cast<uintptr_t>(sorted_pairs) % 16)
    return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(h->ctx, mf::launch_ragged_qmm(static_cast<hipStream_t>(stream), *h, expert_base, expert_stride, *offsets,
                                       x, sorted_pairs, expert_counts, t, route_partials, workspace));
  return MF_OK;
}

mf_status mf_moe_tile_experts(mf_moe* h, mf_stream stream, const void* expert_base, size_t expert_stride,
                              const mf_expert_offsets* offsets, void* tiled) {
  if (!h || !expert_base || !offsets || !tiled) return MF_ERR_INVALID_ARGUMENT;
  const mf_moe_config& c = h->cfg;
  if (!mf::prefill_supported(c)) return MF_ERR_DIMENSION_MISMATCH;
  const uint32_t offs = offsets->gate_w | offsets->up_w | offsets->down_w;
  if (!offsets_ok(*offsets, c.bits) || !mf::aligned16(expert_base) || !mf::aligned16(tiled) || expert_stride % 16 ||
      offs % 16)
    return MF_ERR_INVALID_ARGUMENT;
  const auto* a = static_cast<const uint8_t*>(expert_base);
  const auto* b = static_cast<const uint8_t*>(tiled);
  const size_t bytes = expert_stride * c.num_experts;
  if (a < b + bytes && b < a + bytes) return MF_ERR_INVALID_ARGUMENT;  // the copy is not done in place
  MF_HIP(h->ctx, mf::launch_tile_experts(static_cast<hipStream_t>(stream), c, expert_base, expert_stride, *offsets, tiled));
  return MF_OK;
}

mf_status mf_moe_unpermute(mf_moe* h, mf_stream stream, const float* route_partials, const float* route_weights,
                           const uint32_t* idx, const uint16_t* residual, uint32_t t, uint16_t* y) {
  if (!h || !route_partials || !route_weights || !y) return MF_ERR_INVALID_ARGUMENT;
  if (t == 0 || t > MF_MAX_ROWS) return MF_ERR_QUERY_COUNT;
  const mf_moe_config& c = h->cfg;
  if (c.d % 4) return MF_ERR_DIMENSION_MISMATCH;
  if (!mf::aligned16(route_partials) || reinterpret_cast<uintptr_t>(y) % 8 ||
      (residual && reinterpret_cast<uintptr_t>(residual) % 8))
    return MF_ERR_INVALID_ARGUMENT;
  MF_HIP(h->ctx, mf::launch_unpermute(static_cast<hipStream_t>(stream), c, route_partials, route_weights, idx,
                                      residual, t, y));
  return MF_OK;
}

mf_status mf_group_pairs_host(const mf_pair* pairs, size_t n_pairs, int query_count, int top_k,
                              int num_experts, int tile_expert_count,
                              const uint64_t* sort_keys, size_t n_sort_keys, mf_pair* sorted,
                              uint32_t* offsets, uint32_t* counts, mf_group* groups,
                              size_t* n_groups, mf_tile* tiles, size_t* n_tiles,
                              uint32_t err_detail[2]) {
  uint32_t dummy[2];
  uint32_t* det = err_detail ? err_detail : dummy;
  det[0] = det[1] = 0;
  // validation order of PrefillMoEGrouping.swift:99-141
  if (query_count < 0) return MF_ERR_QUERY_COUNT;
  if (top_k <= 0) return MF_ERR_TOPK;
  if (num_experts <= 0) return MF_ERR_NUM_EXPERTS;
  if (tile_expert_count < 1 || tile_expert_count > 16) return MF_ERR_TILE_EXPERT_COUNT;
  if (sort_keys && n_sort_keys != static_cast<size_t>(num_experts)) {
    det[0] = static_cast<uint32_t>(num_experts);
    det[1] = static_cast<uint32_t>(n_sort_keys);
    return MF_ERR_SORT_KEY_COUNT;
  }
  const size_t expected = static_cast<size_t>(query_count) * static_cast<size_t>(top_k);
  if (n_pairs != expected) {
    det[0] = static_cast<uint32_t>(expected);
    det[1] = static_cast<uint32_t>(n_pairs);
    return MF_ERR_PAIR_COUNT;
  }
  if (n_pairs && (!pairs || !sorted)) return MF_ERR_INVALID_ARGUMENT;
  if (!offsets || !counts || !groups || !tiles || !n_groups || !n_tiles)
    return MF_ERR_INVALID_ARGUMENT;

  std::vector<uint8_t> seen(n_pairs, 0);
  for (size_t i = 0; i < n_pairs; ++i) {
    const mf_pair& p = pairs[i];
    if (p.token >= static_cast<uint32_t>(query_count)) { det[0] = p.token; return MF_ERR_TOKEN_RANGE; }
    if (p.rank >= static_cast<uint32_t>(top_k)) { det[0] = p.rank; return MF_ERR_RANK_RANGE; }
    if (p.expert >= static_cast<uint32_t>(num_experts)) { det[0] = p.expert; return MF_ERR_EXPERT_RANGE; }
    const size_t key = static_cast<size_t>(p.token) * top_k + p.rank;
    if (seen[key]) { det[0] = p.token; det[1] = p.rank; return MF_ERR_DUPLICATE_TOKEN_RANK; }
    seen[key] = 1;
  }

  std::copy(pairs, pairs + n_pairs, sorted);
  std::sort(sorted, sorted + n_pairs, [&](const mf_pair& a, const mf_pair& b) {
    if (sort_keys) {
      const uint64_t ka = sort_keys[a.expert], kb = sort_keys[b.expert];
      if (ka != kb) return ka < kb;
    }
    if (a.expert != b.expert) return a.expert < b.expert;
    if (a.token != b.token) return a.token < b.token;
    return a.rank < b.rank;
  });
  std::fill(offsets, offsets + num_experts, 0xFFFFFFFFu);
  std::fill(counts, counts + num_experts, 0u);
  size_t ng = 0;
  for (size_t i = 0; i < n_pairs;) {
    const uint32_t expert = sorted[i].expert;
    const size_t start = i;
    while (i < n_pairs && sorted[i].expert == expert) ++i;
    offsets[expert] = static_cast<uint32_t>(start);
    counts[expert] = static_cast<uint32_t>(i - start);
    groups[ng++] = mf_group{expert, static_cast<uint32_t>(start), static_cast<uint32_t>(i - start)};
  }
  size_t nt = 0;
  for (size_t gs = 0; gs < ng;) {
    const size_t ge = std::min(ng, gs + static_cast<size_t>(tile_expert_count));
    const mf_group& first = groups[gs];
    const mf_group& last = groups[ge - 1];
    tiles[nt++] = mf_tile{static_cast<uint32_t>(gs), static_cast<uint32_t>(ge - gs), first.pair_start,
                          last.pair_start + last.pair_count - first.pair_start};
    gs = ge;
  }
  *n_groups = ng;
  *n_tiles = nt;
  return MF_OK;
}

}  // extern "C"
