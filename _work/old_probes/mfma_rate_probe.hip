// What the matrix cores of one MI355X sustain with operands held in registers: no memory
// traffic, no LDS, independent accumulators.  It is the ceiling the grouped GEMM is priced
// against (2.5 PFLOP/s dense bf16 by the data sheet).  Measurement program, not product code.
//
//   make -C tests/host mfma_rate_probe && tests/host/mfma_rate_probe
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define CK(x)                                                                   \
  do {                                                                          \
    hipError_t e_ = (x);                                                        \
    if (e_ != hipSuccess) {                                                     \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);     \
      exit(1);                                                                  \
    }                                                                           \
  } while (0)

template <int NACC>
__global__ __launch_bounds__(256) void rate_32x32x16(float* out, int iters) {
  f32x16 acc[NACC];
  for (int i = 0; i < NACC; ++i)
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(threadIdx.x * 0.001f + i);
    b[i] = (__bf16)(0.5f + i * 0.01f);
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
  }
  float s = 0;
  for (int i = 0; i < NACC; ++i)
    for (int v = 0; v < 16; ++v) s += acc[i][v];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

template <int NACC>
__global__ __launch_bounds__(256) void rate_16x16x32(float* out, int iters) {
  f32x4 acc[NACC];
  for (int i = 0; i < NACC; ++i)
    for (int v = 0; v < 4; ++v) acc[i][v] = 0.f;
  bf16x8 a, b;
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(threadIdx.x * 0.001f + i);
    b[i] = (__bf16)(0.5f + i * 0.01f);
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < NACC; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[i], 0, 0, 0);
  }
  float s = 0;
  for (int i = 0; i < NACC; ++i)
    for (int v = 0; v < 4; ++v) s += acc[i][v];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

int main() {
  float* out;
  CK(hipMalloc(&out, 512 * 256 * sizeof(float)));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  const int iters = 20000;
#define RUN(KERNEL, NACC, BLOCKS, FLOP, NAME)                                                        \
  {                                                                                                  \
    hipLaunchKernelGGL((KERNEL<NACC>), dim3(BLOCKS), dim3(256), 0, 0, out, 100);                     \
    CK(hipDeviceSynchronize());                                                                      \
    for (int rep = 0; rep < 3; ++rep) {                                                              \
      CK(hipEventRecord(e0));                                                                        \
      hipLaunchKernelGGL((KERNEL<NACC>), dim3(BLOCKS), dim3(256), 0, 0, out, iters);                 \
      CK(hipEventRecord(e1));                                                                        \
      CK(hipEventSynchronize(e1));                                                                   \
      float ms;                                                                                      \
      CK(hipEventElapsedTime(&ms, e0, e1));                                                          \
      const double fl = (double)BLOCKS * 4 * iters * NACC * FLOP;                                    \
      printf("%s, %d accumulators, %d workgroups of 4 waves: %.2f ms, %.0f TFLOP/s\n", NAME, NACC,   \
             BLOCKS, ms, fl / ms / 1e9);                                                             \
    }                                                                                                \
    fflush(stdout);                                                                                  \
  }
  RUN(rate_32x32x16, 16, 256, 32768.0, "32x32x16 bf16, one wave per SIMD")
  RUN(rate_32x32x16, 8, 512, 32768.0, "32x32x16 bf16, two waves per SIMD")
  RUN(rate_32x32x16, 4, 256, 32768.0, "32x32x16 bf16, one wave per SIMD")
  RUN(rate_16x16x32, 16, 256, 16384.0, "16x16x32 bf16, one wave per SIMD")
  RUN(rate_16x16x32, 16, 512, 16384.0, "16x16x32 bf16, two waves per SIMD")
  CK(hipFree(out));
  return 0;
}
