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
  hipError_t e = hipGetDeviceProperties(&p, 0);
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
