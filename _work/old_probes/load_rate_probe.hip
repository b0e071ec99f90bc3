// How many bytes per second one CU of an MI355X pulls from its L2 and from HBM with tile-shaped
// loads (one instruction = 8 rows x 128 bytes, row stride 14 336 bytes, as the grouped GEMM's
// producers issue them), straight into LDS or into registers, by the number of waves that
// issue them.  One workgroup per CU (100 KB of LDS), two rounds of loads in flight per wave.
// Measurement program, not product code.
//
//   make -C tests/host load_rate_probe && tests/host/load_rate_probe
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#define CK(x)                                                                   \
  do {                                                                          \
    hipError_t e_ = (x);                                                        \
    if (e_ != hipSuccess) {                                                     \
      printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);     \
      exit(1);                                                                  \
    }                                                                           \
  } while (0)

typedef uint32_t u4 __attribute__((ext_vector_type(4)));

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// share != 0: the workgroups of one XCD read the same region (it stays in their L2);
// share == 0: every workgroup streams a region of its own from HBM.
template <int WAVES, int PER, bool TO_LDS, bool HALF = false>
__global__ __launch_bounds__(WAVES * 64, 1) void rate(const char* src, size_t region, size_t stride,
                                                      int rounds, uint32_t* sink, int share) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // HALF: one instruction = 16 rows x 64 bytes (a K step of 32 bf16: half a line per row; the other
  // half is asked for a whole sweep over the row blocks later)
  const int r = HALF ? lane >> 2 : lane >> 3, kv = HALF ? lane & 3 : lane & 7;
  const size_t base = (share ? (size_t)(blockIdx.x & 7) : (size_t)blockIdx.x) * region;
  const char* p0 = src + base + (size_t)r * stride + kv * 16;
  // a wave walks the row blocks wave, wave + WAVES, ... of the region, then the next 128-byte column
  const int nblk = (int)(region / stride / (HALF ? 16 : 8)), ncol = (int)(stride / (HALF ? 64 : 128));
  int rb = wave % nblk, col = 0;
  auto next = [&]() {
    const char* p = p0 + (size_t)rb * (HALF ? 16 : 8) * stride + (size_t)col * (HALF ? 64 : 128);
    rb += WAVES;
    if (rb >= nblk) {
      rb -= nblk;
      col = col + 1 == ncol ? 0 : col + 1;
    }
    return p;
  };
  u4 acc = {0, 0, 0, 0};
  if (TO_LDS) {
    char* mine = lds + wave * PER * 2 * 1024;
    for (int q = 0; q < PER; ++q)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)next(),
                                       (__attribute__((address_space(3))) void*)(mine + q * 1024), 16, 0, 0);
    for (int it = 1; it < rounds; ++it) {
      char* dst = mine + (it & 1) * PER * 1024;
#pragma unroll
      for (int q = 0; q < PER; ++q)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)next(),
                                         (__attribute__((address_space(3))) void*)(dst + q * 1024), 16, 0, 0);
      wait_vmcnt<PER>();
    }
    wait_vmcnt<0>();
    acc = *(u4*)(lds + threadIdx.x * 16);
  } else {
    u4 cur[PER], nxt[PER];
#pragma unroll
    for (int q = 0; q < PER; ++q) cur[q] = *(const u4*)next();
    for (int it = 1; it < rounds; ++it) {
#pragma unroll
      for (int q = 0; q < PER; ++q) nxt[q] = *(const u4*)next();
#pragma unroll
      for (int q = 0; q < PER; ++q) acc ^= cur[q];
#pragma unroll
      for (int q = 0; q < PER; ++q) cur[q] = nxt[q];
    }
#pragma unroll
    for (int q = 0; q < PER; ++q) acc ^= cur[q];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = 1;
}

int main() {
  const size_t stride = 14336;              // bytes per row (7168 bf16)
  const size_t region_l2 = 128 * stride;    // 1.8 MB per XCD when shared: stays in its 4 MB L2
  const size_t region_hbm = 2048 * stride;  // 29 MB per workgroup, 7.5 GB in all
  char* buf;
  CK(hipMalloc(&buf, 256 * region_hbm));
  CK(hipMemset(buf, 1, 256 * region_hbm));
  uint32_t* sink;
  CK(hipMalloc(&sink, 4));
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
#define RUN(W, PER, TO_LDS, SHARE, NAME) RUNH(W, PER, TO_LDS, false, SHARE, NAME)
#define RUNH(W, PER, TO_LDS, HALF, SHARE, NAME)                                                             \
  {                                                                                                    \
    auto k = rate<W, PER, TO_LDS, HALF>;                                                                  \
    CK(hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, 100 * 1024));   \
    const int rounds = (SHARE) ? 32000 / (W * PER) + 8 : (int)(region_hbm / (W * PER * 1024));         \
    const size_t region = (SHARE) ? region_l2 : region_hbm;                                            \
    for (int rep = 0; rep < 2; ++rep) {                                                                \
      CK(hipEventRecord(e0));                                                                          \
      hipLaunchKernelGGL(k, dim3(256), dim3(W * 64), 100 * 1024, 0, buf, region, stride, rounds, sink, \
                         SHARE);                                                                       \
      CK(hipEventRecord(e1));                                                                          \
      CK(hipEventSynchronize(e1));                                                                     \
    }                                                                                                  \
    float ms;                                                                                          \
    CK(hipEventElapsedTime(&ms, e0, e1));                                                              \
    CK(hipGetLastError());                                                                             \
    const double bytes = 256.0 * rounds * W * PER * 1024;                                              \
    printf("%-24s %2d waves, %2d loads each per round: %7.1f us, %6.2f TB/s, %6.1f GB/s per CU\n",     \
           NAME, W, PER, ms * 1e3, bytes / ms / 1e9, bytes / ms / 1e6 / 256);                          \
    fflush(stdout);                                                                                    \
  }
  RUN(2, 24, true, 1, "to LDS, L2 hits")
  RUN(4, 12, true, 1, "to LDS, L2 hits")
  RUN(8, 8, true, 1, "to LDS, L2 hits")
  RUN(16, 4, true, 1, "to LDS, L2 hits")
  RUN(2, 8, false, 1, "to registers, L2 hits")
  RUN(4, 8, false, 1, "to registers, L2 hits")
  RUN(8, 8, false, 1, "to registers, L2 hits")
  RUN(16, 8, false, 1, "to registers, L2 hits")
  RUN(2, 24, true, 0, "to LDS, from HBM")
  RUN(4, 12, true, 0, "to LDS, from HBM")
  RUN(8, 8, true, 0, "to LDS, from HBM")
  RUN(16, 4, true, 0, "to LDS, from HBM")
  RUNH(8, 8, true, true, 1, "to LDS, 64 B, L2 hits")
  RUNH(8, 8, true, true, 0, "to LDS, 64 B, from HBM")
  RUN(8, 8, false, 0, "to registers, from HBM")
  RUN(16, 8, false, 0, "to registers, from HBM")
  CK(hipFree(buf));
  CK(hipFree(sink));
  return 0;
}
