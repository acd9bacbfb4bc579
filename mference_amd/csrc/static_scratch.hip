// mf_shared_expert_static: the shared expert / dense SwiGLU MLP for callers that cannot allocate
// device memory and bring no scratch buffer (code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc).  The activation vector between the gate/up launch and the
// down launch lives in a device array that is part of the library image; the kernels are the
// ones mf_shared_expert launches and take the array's address as their scratch argument.
//
// Every GPU the library runs on holds its own copy of the array, at its own address, until the
// process ends.  The address is looked up once per device (mf_ctx_create) and host code uses that
// pointer, never the array's name.  All calls on one GPU share the array: calls that overlap on
// one GPU (two streams, two host threads) race on it.  Nothing in it has to start at zero -- the
// gate/up launch writes every element the down launch reads -- so nothing is cleared.
#include <stdio.h>

#include <atomic>

#include "mf_internal.h"

namespace {

constexpr size_t kStaticActBytes = MF_STATIC_ACT_ELEMS * sizeof(uint16_t);  // 512 KiB per GPU
static __device__ __align__(256) unsigned char scratch[kStaticActBytes];

constexpr int kMaxDevices = 64;
// device address of `scratch` on each GPU.  Atomic: contexts may be created from several host threads;
// every thread that looks the address up on a device gets the same value, so the last store wins harmlessly.
std::atomic<void*> g_scratch_ptr[kMaxDevices];

}  // namespace

namespace mf {

// Looks up this device's address of the scratch array; `device` must be the current device.
hipError_t static_scratch_init(int device) {
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  if (g_scratch_ptr[device].load(std::memory_order_acquire)) return hipSuccess;
  void* ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess) return e;
  if (!ptr) return hipErrorInvalidSymbol;
  g_scratch_ptr[device].store(ptr, std::memory_order_release);
  return hipSuccess;
}

}  // namespace mf

extern "C" mf_status mf_shared_expert_static(mf_ctx* ctx, mf_stream stream, const uint16_t* x,
                                             mf_qtensor gate, mf_qtensor up, mf_qtensor down,
                                             mf_bits bits, uint32_t d, uint32_t f, uint32_t t,
                                             uint16_t* y) {
  if (!ctx || !x || !y) return MF_ERR_INVALID_ARGUMENT;
  if (bits != MF_BITS_4 && bits != MF_BITS_2 && bits != MF_BITS_TERNARY) return MF_ERR_UNSUPPORTED_BITS;
  if (d == 0 || f == 0 || d % MF_GROUP_SIZE != 0 || f % MF_GROUP_SIZE != 0)
    return MF_ERR_DIMENSION_MISMATCH;
  if (t == 0 || t > MF_MAX_TOKENS) return MF_ERR_INVALID_ARGUMENT;
  const mf_qtensor* q[3] = {&gate, &up, &down};
  for (const mf_qtensor* p : q) {
    if (!p->weights || !p->scales || !mf::aligned2(p->scales)) return MF_ERR_INVALID_ARGUMENT;
    if (bits != MF_BITS_TERNARY && (!p->biases || !mf::aligned2(p->biases))) return MF_ERR_INVALID_ARGUMENT;
  }
  if (!mf::aligned2(x) || !mf::aligned2(y)) return MF_ERR_INVALID_ARGUMENT;
  if (static_cast<size_t>(t) * f > MF_STATIC_ACT_ELEMS) {
    snprintf(ctx->hip_error, sizeof ctx->hip_error,
             "mf_shared_expert_static: t*f = %zu activations exceed the built-in scratch of %u",
             static_cast<size_t>(t) * f, static_cast<unsigned>(MF_STATIC_ACT_ELEMS));
    return MF_ERR_SCRATCH_TOO_SMALL;
  }
  void* const scratch_ptr =
      ctx->device >= 0 && ctx->device < kMaxDevices ? g_scratch_ptr[ctx->device].load(std::memory_order_acquire) : nullptr;
  if (!scratch_ptr) {
    snprintf(ctx->hip_error, sizeof ctx->hip_error,
             "mf_shared_expert_static: the scratch array's address is unknown on device %d", ctx->device);
    return MF_ERR_LAUNCH;
  }
  auto* act = static_cast<uint16_t*>(scratch_ptr);
  auto s = static_cast<hipStream_t>(stream);
  hipError_t e = mf::launch_gate_up_act(s, gate, up, bits, x, act, f, d, t);
  if (e == hipSuccess) e = mf::launch_gemv(s, down, bits, act, y, d, f, t, false);
  if (e != hipSuccess) {
    snprintf(ctx->hip_error, sizeof ctx->hip_error, "mf_shared_expert_static: %s", hipGetErrorString(e));
    return MF_ERR_LAUNCH;
  }
  return MF_OK;
}
