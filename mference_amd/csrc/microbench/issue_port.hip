// How the vector ALU and the matrix core of a gfx950 SIMD share instruction issue: a stand-alone
// measurement behind the design of the prefill matmul kernels' inner loop.
//   part 1: one MFMA 32x32x16 bf16 followed by N independent vector instructions, per step
//   part 2: the inner loop's instruction mix per 64-wide K group and 32-row block (8 MFMAs, four
//           expansions of packed 4-bit codes, 32 scale fmas on the previous group's products)
// Build and run:
//   hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops -o issue_port issue_port.hip && ./issue_port
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short bf16x8 __attribute__((ext_vector_type(8)));

#define CHECK(call)                                                                       \
  do {                                                                                    \
    hipError_t e_ = (call);                                                               \
    if (e_ != hipSuccess) {                                                               \
      fprintf(stderr, "%s:%d %s\n", __FILE__, __LINE__, hipGetErrorString(e_));           \
      return 1;                                                                           \
    }                                                                                     \
  } while (0)

__device__ __forceinline__ f32x16 mfma(uint4 a, uint4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ uint32_t pin_s(uint32_t v) { asm("" : "+s"(v)); return v; }
__device__ __forceinline__ uint32_t pin_v(uint32_t v) { asm("" : "+v"(v)); return v; }
__device__ __forceinline__ uint32_t and_or(uint32_t v, uint32_t m, uint32_t o) { return (v & pin_s(m)) | pin_v(o); }
// eight 4-bit codes -> eight bf16 numbers 8 + q/2
__device__ __forceinline__ uint4 expand_q4(uint32_t w) {
  return make_uint4(and_or(w << 3, 0x00780078u, 0x41004100u), and_or(w >> 1, 0x00780078u, 0x41004100u),
                    and_or(w >> 5, 0x00780078u, 0x41004100u), and_or(w >> 9, 0x00780078u, 0x41004100u));
}

// part 1: per trip 4 MFMAs on 4 independent chains, each followed by N independent fmas
template <int N, bool WITH_MFMA>
__global__ __launch_bounds__(256) void step_kernel(uint32_t iters, const uint32_t* in, float* out, unsigned long long* clk) {
  const unsigned long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  const uint32_t lane = threadIdx.x & 63;
  const uint4 a = make_uint4(in[lane], in[lane + 1], in[lane + 2], in[lane + 3]);
  const uint4 b = make_uint4(in[lane + 4], in[lane + 5], in[lane + 6], in[lane + 7]);
  f32x16 acc[4];
  for (int c = 0; c < 4; ++c)
    for (int r = 0; r < 16; ++r) acc[c][r] = 0;
  float f[8];
  for (int i = 0; i < 8; ++i) f[i] = in[lane + i] * 1e-9f;
  for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (WITH_MFMA) acc[c] = mfma(a, b, acc[c]);
#pragma unroll
      for (int i = 0; i < N; ++i) f[i] = __builtin_fmaf(f[i], 1.0001f, 0.5f);
      if (WITH_MFMA) {  // keep the order written here: one MFMA, then its N fmas
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, N, 0);
      }
    }
  }
  float r = 0;
  for (int c = 0; c < 4; ++c)
    for (int i = 0; i < 16; ++i) r += acc[c][i];
  for (int i = 0; i < 8; ++i) r += f[i];
  out[blockIdx.x * 256 + threadIdx.x] = r;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clk[0] = __builtin_readcyclecounter() - c0;
    clk[1] = wall_clock64() - w0;
  }
}

// part 2: one unit = 8 MFMAs into `t` from the codes cw, while the 32 scale fmas of the previous unit's `p` go into acc
__device__ __forceinline__ void unit(uint32_t (&cw)[4], const uint4 (&bx)[2][4], f32x16 (&t)[2], const f32x16 (&p)[2],
                                     f32x16 (&acc)[2], float sc) {
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) t[nt][r] = 0.0f;
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    asm volatile("" : "+v"(cw[s]));  // fresh codes every unit: the expansion cannot be hoisted
    const uint4 av = expand_q4(cw[s]);
    t[0] = mfma(bx[0][s], av, t[0]);
    t[1] = mfma(bx[1][s], av, t[1]);
  }
#pragma unroll
  for (int nt = 0; nt < 2; ++nt)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[nt][r] = __builtin_fmaf(sc, p[nt][r], acc[nt][r]);
}

__global__ __launch_bounds__(256) void mix_kernel(uint32_t iters, const uint32_t* in, float* out, unsigned long long* clk) {
  const unsigned long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  const uint32_t lane = threadIdx.x & 63;
  uint4 bx[2][4];
  uint32_t cw[4];
  for (int s = 0; s < 4; ++s) {
    cw[s] = in[lane] + s;
    bx[0][s] = make_uint4(in[lane + s], in[lane + s + 1], 0x3f803f80u, 0x3f803f80u);
    bx[1][s] = make_uint4(in[lane + s + 2], in[lane + s + 3], 0x3f803f80u, 0x3f803f80u);
  }
  f32x16 acc[2], ta[2], tb[2];
  for (int nt = 0; nt < 2; ++nt)
    for (int r = 0; r < 16; ++r) acc[nt][r] = ta[nt][r] = tb[nt][r] = 0;
  float sc = 1.5f;
  for (uint32_t it = 0; it < iters; it += 2) {
    unit(cw, bx, ta, tb, acc, sc);
    asm volatile("" : "+v"(sc));
    unit(cw, bx, tb, ta, acc, sc);
    asm volatile("" : "+v"(sc));
  }
  float r = 0;
  for (int nt = 0; nt < 2; ++nt)
    for (int i = 0; i < 16; ++i) r += acc[nt][i] + ta[nt][i] + tb[nt][i];
  out[blockIdx.x * 256 + threadIdx.x] = r;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clk[0] = __builtin_readcyclecounter() - c0;
    clk[1] = wall_clock64() - w0;
  }
}

struct Bufs {
  uint32_t* in;
  float* out;
  unsigned long long* clk;
};

// 256 CUs x `waves` workgroups of 4 waves: `waves` waves on every SIMD
template <typename Launch> int timed(const Bufs& b, int waves, uint32_t iters, Launch launch, double* ns_per_iter, double* ghz) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  launch(100u);
  CHECK(hipDeviceSynchronize());
  CHECK(hipEventRecord(e0));
  launch(iters);
  CHECK(hipEventRecord(e1));
  CHECK(hipEventSynchronize(e1));
  float ms;
  CHECK(hipEventElapsedTime(&ms, e0, e1));
  unsigned long long hc[2];
  CHECK(hipMemcpy(hc, b.clk, 16, hipMemcpyDeviceToHost));
  *ns_per_iter = ms * 1e6 / iters;
  *ghz = static_cast<double>(hc[0]) / (hc[1] * 10.0);  // wall_clock64 ticks at 100 MHz
  (void)waves;
  return 0;
}

template <int N, bool WITH_MFMA> int run_step(const Bufs& b, int waves) {
  const uint32_t iters = 40000;
  double ns, ghz;
  if (timed(b, waves, iters, [&](uint32_t n) { step_kernel<N, WITH_MFMA><<<256 * waves, 256>>>(n, b.in, b.out, b.clk); }, &ns, &ghz)) return 1;
  printf("step: %s + %d fma, %d wave(s) per SIMD: %5.1f SIMD cycles per step (clock %.2f GHz)\n", WITH_MFMA ? "MFMA" : "no MFMA", N,
         waves, ns * ghz / 4 / waves, ghz);
  return 0;
}

int run_mix(const Bufs& b, int waves) {
  const uint32_t iters = 20000;
  double ns, ghz;
  if (timed(b, waves, iters, [&](uint32_t n) { mix_kernel<<<256 * waves, 256>>>(n, b.in, b.out, b.clk); }, &ns, &ghz)) return 1;
  const double cyc = ns * ghz / waves;
  printf("loop mix (8 MFMA + 32 expansion instructions + 32 fma), %d wave(s) per SIMD: %5.1f SIMD cycles per unit, matrix core busy %.0f%%\n",
         waves, cyc, 100.0 * 256 / cyc);
  return 0;
}

int main() {
  Bufs b;
  CHECK(hipMalloc(&b.in, 4096));
  CHECK(hipMemset(b.in, 0x11, 4096));
  CHECK(hipMalloc(&b.out, 256 * 4 * 256 * 4));
  CHECK(hipMalloc(&b.clk, 16));
  for (int waves = 1; waves <= 2; ++waves) {
    if (run_step<0, true>(b, waves) || run_step<2, true>(b, waves) || run_step<4, true>(b, waves) || run_step<6, true>(b, waves) ||
        run_step<8, true>(b, waves) || run_step<8, false>(b, waves) || run_mix(b, waves))
      return 1;
  }
  return 0;
}
