// Stand-alone microbenchmark: sustained v_mfma_f32_32x32x16_bf16 rate of the whole chip with
// (a) small-integer operands and (b) random bf16 operands.  On MI355X the second is the practical
// ceiling of any bf16 attention or GEMM kernel: with realistic data the matrix cores draw enough
// power for the clock to drop, and the sustained rate falls well below the 2.5 PFLOP/s data-sheet peak.
//
//   hipcc --offload-arch=gfx950 -O3 mfma_ceiling.hip -o mfma_ceiling && ./mfma_ceiling
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

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

int main() {
  hipDeviceProp_t p;
  CHECK(hipGetDeviceProperties(&p, 0));
  unsigned* h = (unsigned*)malloc(65536 * 4);
  for (int i = 0; i < 65536; ++i) h[i] = rand() ^ (rand() << 15);
  unsigned* rnd;
  CHECK(hipMalloc(&rnd, 65536 * 4));
  CHECK(hipMemcpy(rnd, h, 65536 * 4, hipMemcpyHostToDevice));
  const int blocks = p.multiProcessorCount * 8, iters = 40000;
  float* d;
  CHECK(hipMalloc(&d, blocks * 256 * 4));
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  for (int mode = 0; mode < 2; ++mode)
    for (int rep = 0; rep < 4; ++rep) {
      CHECK(hipEventRecord(e0));
      if (mode == 0) mfma_loop<0><<<blocks, 256>>>(rnd, d, iters);
      else mfma_loop<1><<<blocks, 256>>>(rnd, d, iters);
      CHECK(hipEventRecord(e1));
      CHECK(hipEventSynchronize(e1));
      float ms;
      CHECK(hipEventElapsedTime(&ms, e0, e1));
      printf("%-18s %.2f ms  %.0f TFLOP/s\n", mode ? "random bf16 data" : "small integers", ms,
             (double)blocks * 4 * iters * 4 * 32768.0 / ms * 1e-9);
    }
  return 0;
}
