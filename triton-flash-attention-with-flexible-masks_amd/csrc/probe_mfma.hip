// Measurement aid, not part of the operator: the sustained v_mfma_f32_32x32x16_bf16 rate of the whole
// chip with (a) small-integer operands and (b) random bf16 operands.  On MI355X the second is the
// practical ceiling of any bf16 attention or GEMM kernel: with realistic data the matrix cores draw
// enough power for the clock to drop, and the sustained rate falls well below the 2.5 PFLOP/s
// data-sheet peak.  Built as its own small library (libfa_probe.so) and driven by `bench.py --mfma-probe`;
// it allocates and frees its own two small buffers and synchronises, unlike the operator's library.
#include <hip/hip_runtime.h>
#include <stdlib.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <int RANDOM>
__global__ __launch_bounds__(256) void mfma_loop(const unsigned* rnd, float* out, int iters) {
  bf16x8 a[4], b[4];
  for (int j = 0; j < 4; ++j)
    for (int t = 0; t < 8; ++t) {
      if (RANDOM) {
        const unsigned r = rnd[(threadIdx.x * 64 + j * 8 + t) % 65536];
        a[j][t] = (__bf16)(((r & 0xffff) / 32768.0f - 1.0f) * 2.0f);
        b[j][t] = (__bf16)(((r >> 16) / 32768.0f - 1.0f) * 2.0f);
      } else {
        a[j][t] = (__bf16)(float)((threadIdx.x + j) % 3);
        b[j][t] = (__bf16)(float)((threadIdx.x + t) % 5);
      }
    }
  f32x16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
  for (int i = 0; i < iters; ++i) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[0], c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[1], b[1], c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[2], b[2], c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[3], b[3], c3, 0, 0, 0);
    if (RANDOM) { bf16x8 t = a[0]; a[0] = a[1]; a[1] = a[2]; a[2] = a[3]; a[3] = t; }
  }
  float s = 0;
  for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

// One timed launch of 8 workgroups of 4 waves per CU, nothing but MFMAs in the loop (4 independent
// accumulators per wave).  Returns 0 and the rate in TFLOP/s, or the hipError_t that stopped it.
extern "C" int fa_probe_mfma_rate(int random_operands, int iters, float* tflops) {
  hipDeviceProp_t p;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);   // the device the launch below goes to
  if (e != hipSuccess) return (int)e;
  e = hipGetDeviceProperties(&p, dev);
  if (e != hipSuccess) return (int)e;
  unsigned* h = (unsigned*)malloc(65536 * 4);
  srand(1);
  for (int i = 0; i < 65536; ++i) h[i] = (unsigned)rand() ^ ((unsigned)rand() << 15);
  unsigned* rnd = nullptr;
  float* d = nullptr;
  const int blocks = p.multiProcessorCount * 8;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  float ms = 0.f;
  if ((e = hipMalloc(&rnd, 65536 * 4)) == hipSuccess && (e = hipMalloc(&d, size_t(blocks) * 256 * 4)) == hipSuccess &&
      (e = hipMemcpy(rnd, h, 65536 * 4, hipMemcpyHostToDevice)) == hipSuccess && (e = hipEventCreate(&e0)) == hipSuccess &&
      (e = hipEventCreate(&e1)) == hipSuccess) {
    (void)hipEventRecord(e0, 0);
    if (random_operands) hipLaunchKernelGGL(mfma_loop<1>, dim3(blocks), dim3(256), 0, 0, rnd, d, iters);
    else hipLaunchKernelGGL(mfma_loop<0>, dim3(blocks), dim3(256), 0, 0, rnd, d, iters);
    (void)hipEventRecord(e1, 0);
    if ((e = hipEventSynchronize(e1)) == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (rnd) (void)hipFree(rnd);
  if (d) (void)hipFree(d);
  free(h);
  if (e == hipSuccess && ms > 0.f) *tflops = (float)((double)blocks * 4 * iters * 4 * 32768.0 / ms * 1e-9);
  return (int)e;
}

// The phase structure of the forward's tile loop without any memory access: per wave and round 16 MFMAs
// in 2 chains (the scores), a vector phase that needs their results (32 x fma, exp2, add and 16
// conversions: the softmax of a 64-key tile on its fast path), 16 MFMAs in 4 chains that need those
// (P V), a workgroup barrier.  What this loop reaches is what the forward's instruction mix allows
// before it reads a single operand.
template <int SOFTMAX>
__global__ __launch_bounds__(256) void phase_loop(float* out, int iters, int never) {
  extern __shared__ char smem[];
  if (never == 12345) smem[threadIdx.x] = 1;
  bf16x8 q[8], kf, vf;
  for (int j = 0; j < 8; ++j)
    for (int i = 0; i < 8; ++i) q[j][i] = (__bf16)(0.01f * (threadIdx.x % 7 + i + j));
  for (int i = 0; i < 8; ++i) { kf[i] = (__bf16)(0.02f * (threadIdx.x % 5 + i)); vf[i] = (__bf16)(0.03f * (threadIdx.x % 3 + i)); }
  f32x16 o[4] = {{0}, {0}, {0}, {0}};
  float m = 0.f, l = 0.f;
  for (int it = 0; it < iters; ++it) {
    f32x16 s0 = {0}, s1 = {0};
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, q[ks], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, q[ks], s1, 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    bf16x8 p[4];
    if (SOFTMAX) {
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float a = __builtin_amdgcn_exp2f(s0[i] * 0.125f - m), b = __builtin_amdgcn_exp2f(s1[i] * 0.125f - m);
        sum += a + b;
        p[i / 8][i % 8] = (__bf16)a;
        p[2 + i / 8][i % 8] = (__bf16)b;
      }
      l += sum;
      if (__builtin_expect(sum > 4096.f, 0)) m += 1.f;
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) { p[i / 8][i % 8] = (__bf16)s0[i]; p[2 + i / 8][i % 8] = (__bf16)s1[i]; }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int db = 0; db < 4; ++db) o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(db & 1 ? vf : kf, p[kk], o[db], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
  }
  float s = l + m;
  for (int d = 0; d < 4; ++d)
    for (int i = 0; i < 16; ++i) s += o[d][i];
  out[blockIdx.x * 256 + threadIdx.x] = s;
}

// One timed launch of `wgs_per_cu` (1 or 2) workgroups of 4 waves per CU, held to that residency by
// their LDS size.  Returns 0 and the time of one round in ns (with 2 workgroups: of one round of
// each), or the hipError_t that stopped it.
extern "C" int fa_probe_phase_time(int wgs_per_cu, int softmax, int iters, float* ns_per_round) {
  hipDeviceProp_t p;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);   // the device the launch below goes to
  if (e != hipSuccess) return (int)e;
  e = hipGetDeviceProperties(&p, dev);
  if (e != hipSuccess) return (int)e;
  if (wgs_per_cu != 1 && wgs_per_cu != 2) return (int)hipErrorInvalidValue;
  const int lds = wgs_per_cu == 1 ? 150 * 1024 : 70 * 1024;
  const int blocks = p.multiProcessorCount * wgs_per_cu;
  auto kern = softmax ? phase_loop<1> : phase_loop<0>;
  float* d = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  float ms = 0.f;
  if ((e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds)) == hipSuccess &&
      (e = hipMalloc(&d, size_t(blocks) * 256 * 4)) == hipSuccess && (e = hipEventCreate(&e0)) == hipSuccess &&
      (e = hipEventCreate(&e1)) == hipSuccess) {
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds, 0, d, 16, 0);   // warm
    (void)hipEventRecord(e0, 0);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), lds, 0, d, iters, 0);
    (void)hipEventRecord(e1, 0);
    if ((e = hipEventSynchronize(e1)) == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (d) (void)hipFree(d);
  if (e == hipSuccess && ms > 0.f) *ns_per_round = ms * 1e6f / iters;
  return (int)e;
}
