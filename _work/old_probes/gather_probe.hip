// What a top-k gather of the combine's shape can reach on one MI355X, without any of the
// kernel's index arithmetic: S = 4096 tokens, each the sum of K = 8 rows of 14 KiB picked at
// random from 4.8 GB (the 8 shards), seven waves per token with 2 KiB of every row each.
// Variants: the rows loaded into registers or straight into LDS, the 59 MB of sums stored or
// not, and persistent waves that issue the next item's loads before they store the current
// sums.  Sums are integer adds of the raw words (the traffic is what is measured).
// Measurement program, not product code.
//
//   make -C tests/host gather_probe && tests/host/gather_probe
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <stdint.h>
#include <vector>
#include <random>
#include <algorithm>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s at line %d\n",hipGetErrorString(e),__LINE__); exit(1);} }while(0)
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
template <int N> __device__ __forceinline__ void wait_vmcnt() { __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14)); }
constexpr int K = 8, ROWB = 14336, PARTS = 7;   // 7 waves per token, 2 KB each

template <bool TO_LDS, bool STORE>
__global__ __launch_bounds__(256) void gather(const char* shards, const int* rows, char* out, int S) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int gw = blockIdx.x * 4 + wave;
  const int s = gw / PARTS, part = gw - s * PARTS;
  if (s >= S) return;
  int rk = 0; if (lane < K) rk = rows[s * K + lane];
  const size_t c0 = (size_t)part * 2048 + lane * 16;
  u4 acc0 = {0,0,0,0}, acc1 = {0,0,0,0};
  if (TO_LDS) {
    char* mine = lds + wave * (K * 2048);
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const char* row = shards + (size_t)__builtin_amdgcn_readlane(rk, k) * ROWB + c0;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)row, (__attribute__((address_space(3))) void*)(mine + k * 2048), 16, 0, 0);
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(row + 1024), (__attribute__((address_space(3))) void*)(mine + k * 2048 + 1024), 16, 0, 0);
    }
    wait_vmcnt<0>();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const u4 a = *(const u4*)(mine + k * 2048 + lane * 16), b = *(const u4*)(mine + k * 2048 + 1024 + lane * 16);
      acc0 += a; acc1 += b;
    }
  } else {
    u4 v[K][2];
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const char* row = shards + (size_t)__builtin_amdgcn_readlane(rk, k) * ROWB + c0;
      v[k][0] = __builtin_nontemporal_load((const u4*)row);
      v[k][1] = __builtin_nontemporal_load((const u4*)(row + 1024));
    }
#pragma unroll
    for (int k = 0; k < K; ++k) { acc0 += v[k][0]; acc1 += v[k][1]; }
  }
  char* o = out + (size_t)s * ROWB + c0;
  if (STORE) { __builtin_nontemporal_store(acc0, (u4*)o); __builtin_nontemporal_store(acc1, (u4*)(o + 1024)); }
  else if ((acc0.x ^ acc1.y) == 0x12345678u) *(u4*)o = acc0;
}

// persistent waves: the K-row loads of the next item are issued before the sums of the current one are stored
__global__ __launch_bounds__(256) void gather_deferred(const char* shards, const int* rows, char* out, int S) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = gridDim.x * 4, items = S * PARTS;
  int item = blockIdx.x * 4 + wave;
  if (item >= items) return;
  u4 v[K][2], n[K][2];
  auto load = [&](int it, u4 (*d)[2]) {
    const int s = it / PARTS, part = it - s * PARTS;
    int rk = 0; if (lane < K) rk = rows[s * K + lane];
    const size_t c0 = (size_t)part * 2048 + lane * 16;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const char* row = shards + (size_t)__builtin_amdgcn_readlane(rk, k) * ROWB + c0;
      d[k][0] = __builtin_nontemporal_load((const u4*)row);
      d[k][1] = __builtin_nontemporal_load((const u4*)(row + 1024));
    }
  };
  load(item, v);
  while (true) {
    const int nxt = item + nw;
    const bool more = nxt < items;
    if (more) load(nxt, n);
    u4 acc0 = {0,0,0,0}, acc1 = {0,0,0,0};
#pragma unroll
    for (int k = 0; k < K; ++k) { acc0 += v[k][0]; acc1 += v[k][1]; }
    const int s = item / PARTS, part = item - s * PARTS;
    char* o = out + (size_t)s * ROWB + (size_t)part * 2048 + lane * 16;
    __builtin_nontemporal_store(acc0, (u4*)o); __builtin_nontemporal_store(acc1, (u4*)(o + 1024));
    if (!more) break;
#pragma unroll
    for (int k = 0; k < K; ++k) { v[k][0] = n[k][0]; v[k][1] = n[k][1]; }
    item = nxt;
  }
}

int main() {
  const int S = 4096; const long NROWS = 8L * 41984;     // rows of the 8 shards
  char* shards; CK(hipMalloc(&shards, (size_t)NROWS * ROWB)); CK(hipMemset(shards, 1, (size_t)NROWS * ROWB));
  char* out[4]; for (auto& o : out) { CK(hipMalloc(&o, (size_t)S * ROWB)); }
  std::mt19937 g(5); std::vector<int> all(NROWS); for (long i = 0; i < NROWS; ++i) all[i] = (int)i; std::shuffle(all.begin(), all.end(), g);
  int* rows[4];
  for (int b = 0; b < 4; ++b) { std::vector<int> r(all.begin() + b * S * K, all.begin() + (b + 1) * S * K); CK(hipMalloc(&rows[b], S * K * 4)); CK(hipMemcpy(rows[b], r.data(), S * K * 4, hipMemcpyHostToDevice)); }
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
#define RUN(TO_LDS, STORE, LDSB, NAME) { auto k = gather<TO_LDS, STORE>; if (LDSB > 65536) CK(hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, LDSB)); \
    const int blocks = (S * PARTS + 3) / 4; for (int w = 0; w < 4; ++w) hipLaunchKernelGGL(k, dim3(blocks), dim3(256), LDSB, 0, shards, rows[w], out[w], S); CK(hipDeviceSynchronize()); \
    const int it = 12; CK(hipEventRecord(e0)); for (int i = 0; i < it; ++i) hipLaunchKernelGGL(k, dim3(blocks), dim3(256), LDSB, 0, shards, rows[i & 3], out[i & 3], S); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); \
    float ms; CK(hipEventElapsedTime(&ms, e0, e1)); CK(hipGetLastError()); const double us = ms * 1e3 / it; \
    printf("%-44s %6.1f us  read %.2f TB/s%s\n", NAME, us, (double)S * K * ROWB / us / 1e6, STORE ? "  (+59 MB written)" : ""); fflush(stdout); }
  for (int rep = 0; rep < 2; ++rep) {
    RUN(false, false, 0, "registers, no output")
    RUN(true, false, 65536, "LDS-direct (64 KB/WG, 2 WG per CU), no output")
    RUN(false, true, 0, "registers, output stored")
    RUN(true, true, 65536, "LDS-direct, output stored")
    for (int blocks : {512, 1024, 2048, 3584}) {
      for (int w = 0; w < 4; ++w) hipLaunchKernelGGL(gather_deferred, dim3(blocks), dim3(256), 0, 0, shards, rows[w], out[w], S); CK(hipDeviceSynchronize());
      const int it = 12; CK(hipEventRecord(e0)); for (int i = 0; i < it; ++i) hipLaunchKernelGGL(gather_deferred, dim3(blocks), dim3(256), 0, 0, shards, rows[i & 3], out[i & 3], S); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
      float ms; CK(hipEventElapsedTime(&ms, e0, e1)); CK(hipGetLastError()); const double us = ms * 1e3 / it;
      printf("registers, stores deferred behind the next item's loads, %4d workgroups: %6.1f us  read %.2f TB/s  (+59 MB written)\n", blocks, us, (double)S * K * ROWB / us / 1e6); fflush(stdout);
    }
  }
  return 0;
}
