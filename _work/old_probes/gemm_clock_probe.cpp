// The grouped SwiGLU GEMM at the real shape (40 960 rows in 64 groups of 2..6 row tiles,
// H = 7168, H' = 2048) built three ways from moonep_amd/csrc/grouped_gemm.hip -- as it is,
// without its global loads, without its LDS reads and MFMAs -- with a cycle counter and a
// constant-rate counter read at both ends of every tile.  Prints the launch time, the core
// clocks of a tile and the clock the chip sustained (core clocks per wall tick x the tick rate).
// No library, no Python: `make -C tests/host gemm_clock_probe && tests/host/gemm_clock_probe_full` etc.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <vector>

extern "C" int mep_grouped_gemm_nt(const void* A, const void* B, const void* B_up, const int32_t* cu, int G,
                                   void* C, const float* row_scale, int M, int N, int K, int swiglu, void* stream);
extern "C" int mep_gemm_probe_read(unsigned long long* out3, int reset);

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %d at line %d\n", (int)e_, __LINE__); return 1; } } while (0)

// bf16 values in about [-1, 1) from a hash of the index (random bits: the matrix cores' power
// depends on the data they are fed)
__global__ void fill(uint16_t* p, size_t n, uint32_t seed, float scale) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    uint32_t x = (uint32_t)i * 2654435761u + seed;
    x ^= x >> 15; x *= 2246822519u; x ^= x >> 13; x *= 3266489917u; x ^= x >> 16;
    const float f = ((int)(x & 0xffff) - 32768) / 32768.0f * scale;
    p[i] = (uint16_t)(__float_as_uint(f) >> 16);
  }
}

int main() {
  const int M = 40960, H = 7168, Hp = 2048, G = 64;
  const int blocks[8] = {3, 5, 4, 6, 2, 4, 5, 3};
  std::vector<int32_t> cu(G);
  int rows = 0;
  for (int g = 0; g < G; ++g) { rows += 128 * blocks[g % 8]; cu[g] = rows; }
  uint16_t *A, *Bg, *Bu, *C;
  int32_t* dcu;
  CK(hipMalloc(&A, (size_t)M * H * 2)); CK(hipMalloc(&Bg, (size_t)G * Hp * H * 2)); CK(hipMalloc(&Bu, (size_t)G * Hp * H * 2));
  CK(hipMalloc(&C, (size_t)M * Hp * 2)); CK(hipMalloc(&dcu, G * 4));
  CK(hipMemcpy(dcu, cu.data(), G * 4, hipMemcpyHostToDevice));
  hipLaunchKernelGGL(fill, dim3(4096), dim3(256), 0, 0, A, (size_t)M * H, 1u, 1.0f);
  hipLaunchKernelGGL(fill, dim3(4096), dim3(256), 0, 0, Bg, (size_t)G * Hp * H, 2u, 0.02f);
  hipLaunchKernelGGL(fill, dim3(4096), dim3(256), 0, 0, Bu, (size_t)G * Hp * H, 3u, 0.02f);
  CK(hipMemset(C, 0, (size_t)M * Hp * 2));
  CK(hipDeviceSynchronize());
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  const int iters = 8;
  for (int pass = 0; pass < 3; ++pass) {
    for (int i = 0; i < 2; ++i)
      if (mep_grouped_gemm_nt(A, Bg, Bu, dcu, G, C, nullptr, M, Hp, H, 1, nullptr)) { printf("launch failed\n"); return 1; }
    CK(hipDeviceSynchronize());
    unsigned long long c[3];
    if (mep_gemm_probe_read(c, 1)) return 1;
    CK(hipEventRecord(e0));
    for (int i = 0; i < iters; ++i)
      if (mep_grouped_gemm_nt(A, Bg, Bu, dcu, G, C, nullptr, M, Hp, H, 1, nullptr)) { printf("launch failed\n"); return 1; }
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    if (mep_gemm_probe_read(c, 1)) return 1;
    int wall_khz = 0;
    CK(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, 0));
    const double us = ms * 1e3 / iters, flops = 4.0 * rows * H * Hp;
    printf("variant %d pass %d: %7.1f us per launch (%6.1f TFLOP/s-equivalent); per tile %8.0f core clocks, %7.0f wall ticks "
           "at %d kHz -> %5.0f MHz sustained\n", MEP_GEMM_PROBE, pass, us, flops / us / 1e6, (double)c[0] / c[2],
           (double)c[1] / c[2], wall_khz, (double)c[0] / c[1] * wall_khz / 1e3);
    fflush(stdout);
  }
  return 0;
}
