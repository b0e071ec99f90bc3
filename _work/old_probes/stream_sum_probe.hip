// The streams of a slot reduction without its bookkeeping, on one MI355X: G += P over 470 MB of
// fp32 (8 matrices of 7168 x 2048: read the grads, read the slots, write the grads) and 470 MB
// of zeroes into a third region (the own slots to clear).  It measures what the layout of a
// tile, the place of the fills and the number of workgroups are worth before the kernel
// (csrc/prefetch.hip) takes them over:
//   rmw          vectors of a thread 4 KiB apart, loads to registers or straight into LDS,
//                zeroes written as tiles after the sums
//   rmw_strided  vectors STRIDE bytes apart, tiles interleaved in blocks of V * STRIDE bytes
//   rmw_split    fills as short workgroups of their own before / behind the summing ones
//   rmw_split2   the same with a fixed number of fill workgroups that loop
//   rmw_inter    fills as dense 4 KiB pieces that the summing workgroups take between tiles
//   copy_strided a plain copy in the same layouts
// Measurement program, not product code.
//
//   make -C tests/host stream_sum_probe && tests/host/stream_sum_probe
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <stdint.h>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s at line %d\n",hipGetErrorString(e),__LINE__); exit(1);} }while(0)
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
template <int N> __device__ __forceinline__ void wait_vmcnt() { __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14)); }
__device__ __forceinline__ void st_through(void* p, f4 v) { asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 3" : : "v"(p), "v"(v) : "memory"); }

// tile = 256 threads x V vectors of 16 B
template <int V, bool TO_LDS>
__global__ __launch_bounds__(256) void rmw(float* G, const float* P, float* Z, long reduce_tiles, long clear_tiles) {
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long tile_floats = 256L * V * 4;
  const long work = reduce_tiles + clear_tiles;
  if (!TO_LDS) {
    for (long w = blockIdx.x; w < work; w += gridDim.x) {
      if (w >= reduce_tiles) {
        f4* z = (f4*)(Z + (w - reduce_tiles) * tile_floats) + tid;
        const f4 zero = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < V; ++i) st_through(z + i * 256, zero);
        continue;
      }
      f4* g = (f4*)(G + w * tile_floats) + tid;
      const f4* p = (const f4*)(P + w * tile_floats) + tid;
      f4 a[V], b[V];
#pragma unroll
      for (int i = 0; i < V; ++i) a[i] = g[i * 256];
#pragma unroll
      for (int i = 0; i < V; ++i) b[i] = __builtin_nontemporal_load(p + i * 256);
#pragma unroll
      for (int i = 0; i < V; ++i) st_through(g + i * 256, a[i] + b[i]);
    }
  } else {
    // wave-private LDS: [2 buffers][2 streams][V KB]
    char* mine = lds + wave * (4 * V * 1024);
    auto issue = [&](long w, int buf) {
      const char* g = (const char*)(G + w * tile_floats) + wave * 1024 + lane * 16;
      const char* p = (const char*)(P + w * tile_floats) + wave * 1024 + lane * 16;
      char* d = mine + buf * (2 * V * 1024);
#pragma unroll
      for (int i = 0; i < V; ++i) {
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(g + i * 4096), (__attribute__((address_space(3))) void*)(d + i * 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(p + i * 4096), (__attribute__((address_space(3))) void*)(d + (V + i) * 1024), 16, 0, 0);
      }
    };
    long w = blockIdx.x;
    int buf = 0;
    bool have = w < reduce_tiles;
    if (have) issue(w, 0);
    for (; w < work; w += gridDim.x) {
      if (w >= reduce_tiles) {
        f4* z = (f4*)(Z + (w - reduce_tiles) * tile_floats) + tid;
        const f4 zero = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < V; ++i) st_through(z + i * 256, zero);
        continue;
      }
      const long nw = w + gridDim.x;
      const bool more = nw < reduce_tiles;
      if (more) issue(nw, buf ^ 1);
      if (more) wait_vmcnt<2 * V>(); else wait_vmcnt<0>();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const char* d = mine + buf * (2 * V * 1024) + lane * 16;
      char* g = (char*)(G + w * tile_floats) + wave * 1024 + lane * 16;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const f4 a = *(const f4*)(d + i * 1024), b = *(const f4*)(d + (V + i) * 1024);
        st_through(g + i * 4096, a + b);
      }
      buf ^= 1;
    }
  }
}

// register variant with a wave's consecutive vectors STRIDE bytes apart; tiles interleave inside super blocks of V*STRIDE bytes
template <int V, int STRIDE, int POLICY, int CV = 0>
__global__ __launch_bounds__(256) void rmw_strided(float* G, const float* P, float* Z, long reduce_tiles, long clear_tiles) {
  const int tid = threadIdx.x;
  constexpr long per_super = STRIDE / 4096;
  const long work = reduce_tiles + clear_tiles;
  auto off = [&](long w) { const long sup = w / per_super, sub = w - sup * per_super; return sup * (long)V * STRIDE + sub * 4096 + tid * 16; };
  for (long w = blockIdx.x; w < work; w += gridDim.x) {
    if (w >= reduce_tiles) {
      const f4 zero = {0, 0, 0, 0};
      if (CV > 0) {   // dense: CV consecutive 4 KB slabs per work item, one store per thread each
        char* z = (char*)Z + (w - reduce_tiles) * (long)CV * 4096 + tid * 16;
#pragma unroll
        for (int i = 0; i < CV; ++i) st_through(z + (long)i * 4096, zero);
        continue;
      }
      char* z = (char*)Z + off(w - reduce_tiles);
#pragma unroll
      for (int i = 0; i < V; ++i) { if (POLICY == 0) st_through(z + (long)i * STRIDE, zero); else __builtin_nontemporal_store(zero, (f4*)(z + (long)i * STRIDE)); }
      continue;
    }
    char* g = (char*)G + off(w);
    const char* p = (const char*)P + off(w);
    f4 a[V], b[V];
#pragma unroll
    for (int i = 0; i < V; ++i) a[i] = *(const f4*)(g + (long)i * STRIDE);
#pragma unroll
    for (int i = 0; i < V; ++i) b[i] = __builtin_nontemporal_load((const f4*)(p + (long)i * STRIDE));
#pragma unroll
    for (int i = 0; i < V; ++i) { if (POLICY == 0) st_through(g + (long)i * STRIDE, a[i] + b[i]); else __builtin_nontemporal_store(a[i] + b[i], (f4*)(g + (long)i * STRIDE)); }
  }
}

// one launch: fill workgroups (CV dense 4 KB slabs each, not persistent) and RB persistent reduce workgroups
template <int V, int STRIDE, int CV, bool FILL_FIRST>
__global__ __launch_bounds__(256) void rmw_split(float* G, const float* P, float* Z, long reduce_tiles, long fill_blocks, int RB) {
  const int tid = threadIdx.x;
  long b = blockIdx.x;
  bool fill;
  if (FILL_FIRST) { fill = b < fill_blocks; if (!fill) b -= fill_blocks; }
  else { fill = b >= RB; if (fill) b -= RB; }
  if (fill) {
    const f4 zero = {0, 0, 0, 0};
    char* z = (char*)Z + b * (long)CV * 4096 + tid * 16;
#pragma unroll
    for (int i = 0; i < CV; ++i) st_through(z + (long)i * 4096, zero);
    return;
  }
  constexpr long per_super = STRIDE / 4096;
  auto off = [&](long w) { const long sup = w / per_super, sub = w - sup * per_super; return sup * (long)V * STRIDE + sub * 4096 + tid * 16; };
  for (long w = b; w < reduce_tiles; w += RB) {
    char* g = (char*)G + off(w);
    const char* p = (const char*)P + off(w);
    f4 a[V], c[V];
#pragma unroll
    for (int i = 0; i < V; ++i) a[i] = *(const f4*)(g + (long)i * STRIDE);
#pragma unroll
    for (int i = 0; i < V; ++i) c[i] = __builtin_nontemporal_load((const f4*)(p + (long)i * STRIDE));
#pragma unroll
    for (int i = 0; i < V; ++i) st_through(g + (long)i * STRIDE, a[i] + c[i]);
  }
}

// one launch: RB persistent reduce workgroups, then F fill workgroups that take slabs f, f + F, ... (clear_slabs may be 0)
template <int V, int STRIDE>
__global__ __launch_bounds__(256) void rmw_split2(float* G, const float* P, float* Z, long reduce_tiles, long clear_slabs, int RB) {
  const int tid = threadIdx.x;
  long b = blockIdx.x;
  if (b >= RB) {
    const long F = gridDim.x - RB;
    const f4 zero = {0, 0, 0, 0};
    for (long sl = b - RB; sl < clear_slabs; sl += F) st_through((char*)Z + sl * 4096 + tid * 16, zero);
    return;
  }
  constexpr long per_super = STRIDE / 4096;
  auto off = [&](long w) { const long sup = w / per_super, sub = w - sup * per_super; return sup * (long)V * STRIDE + sub * 4096 + tid * 16; };
  for (long w = b; w < reduce_tiles; w += RB) {
    char* g = (char*)G + off(w);
    const char* p = (const char*)P + off(w);
    f4 a[V], c[V];
#pragma unroll
    for (int i = 0; i < V; ++i) a[i] = *(const f4*)(g + (long)i * STRIDE);
#pragma unroll
    for (int i = 0; i < V; ++i) c[i] = __builtin_nontemporal_load((const f4*)(p + (long)i * STRIDE));
#pragma unroll
    for (int i = 0; i < V; ++i) st_through(g + (long)i * STRIDE, a[i] + c[i]);
  }
}

// persistent workgroups that interleave: after each reduce tile, FS fill slabs (dense, in order across the grid)
template <int V, int STRIDE, int FS, bool FILL_BEFORE>
__global__ __launch_bounds__(256) void rmw_inter(float* G, const float* P, float* Z, long reduce_tiles, long clear_slabs) {
  const int tid = threadIdx.x;
  constexpr long per_super = STRIDE / 4096;
  auto off = [&](long w) { const long sup = w / per_super, sub = w - sup * per_super; return sup * (long)V * STRIDE + sub * 4096 + tid * 16; };
  const f4 zero = {0, 0, 0, 0};
  long it = 0;
  for (long w = blockIdx.x; w < reduce_tiles; w += gridDim.x, ++it) {
    const long s0 = (it * gridDim.x + blockIdx.x) * FS;
    if (FILL_BEFORE) {
#pragma unroll
      for (int j = 0; j < FS; ++j) if (s0 + j < clear_slabs) st_through((char*)Z + (s0 + j) * 4096 + tid * 16, zero);
    }
    char* g = (char*)G + off(w);
    const char* p = (const char*)P + off(w);
    f4 a[V], c[V];
#pragma unroll
    for (int i = 0; i < V; ++i) a[i] = *(const f4*)(g + (long)i * STRIDE);
#pragma unroll
    for (int i = 0; i < V; ++i) c[i] = __builtin_nontemporal_load((const f4*)(p + (long)i * STRIDE));
#pragma unroll
    for (int i = 0; i < V; ++i) st_through(g + (long)i * STRIDE, a[i] + c[i]);
    if (!FILL_BEFORE) {
#pragma unroll
      for (int j = 0; j < FS; ++j) if (s0 + j < clear_slabs) st_through((char*)Z + (s0 + j) * 4096 + tid * 16, zero);
    }
  }
  // what the interleave did not reach
  for (long sl = (it * gridDim.x + blockIdx.x) * FS; sl < clear_slabs; sl += gridDim.x) st_through((char*)Z + sl * 4096 + tid * 16, zero);
}

template <int V, int STRIDE>
__global__ __launch_bounds__(256) void copy_strided(const float* S, float* D, long tiles) {
  const int tid = threadIdx.x;
  constexpr long per_super = STRIDE / 4096;
  auto off = [&](long w) { const long sup = w / per_super, sub = w - sup * per_super; return sup * (long)V * STRIDE + sub * 4096 + tid * 16; };
  for (long w = blockIdx.x; w < tiles; w += gridDim.x) {
    const char* s = (const char*)S + off(w);
    char* d = (char*)D + off(w);
    f4 a[V];
#pragma unroll
    for (int i = 0; i < V; ++i) a[i] = __builtin_nontemporal_load((const f4*)(s + (long)i * STRIDE));
#pragma unroll
    for (int i = 0; i < V; ++i) st_through(d + (long)i * STRIDE, a[i]);
  }
}

int main() {
  const long per = 7168L * 2048;            // floats per expert matrix
  const int n = 8;
  float *G, *P, *Z;
  CK(hipMalloc(&G, n * per * 4)); CK(hipMalloc(&P, n * per * 4)); CK(hipMalloc(&Z, n * per * 4));
  CK(hipMemset(G, 0, n * per * 4)); CK(hipMemset(P, 0, n * per * 4));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
#define RUN(V, TO_LDS, BLOCKS, CLEAR, NAME) if ((n * per * 4) % (256L * V * 16) != 0) { printf("skipped\n"); } else { auto k = rmw<V, TO_LDS>; const int ldsb = TO_LDS ? 4 * 4 * V * 1024 : 0; \
    const long rt = n * per / (256L * V * 4), ct = CLEAR ? rt : 0; \
    for (int i = 0; i < 2; ++i) hipLaunchKernelGGL(k, dim3(BLOCKS), dim3(256), ldsb, 0, G, P, Z, rt, ct); CK(hipDeviceSynchronize()); \
    const int it = 6; CK(hipEventRecord(e0)); for (int i = 0; i < it; ++i) hipLaunchKernelGGL(k, dim3(BLOCKS), dim3(256), ldsb, 0, G, P, Z, rt, ct); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); \
    float ms; CK(hipEventElapsedTime(&ms, e0, e1)); CK(hipGetLastError()); const double us = ms * 1e3 / it; const double bytes = (double)n * per * 4 * (CLEAR ? 4 : 3); \
    printf("%-34s V=%d blocks=%4d %s: %7.1f us %5.2f TB/s\n", NAME, V, BLOCKS, CLEAR ? "reduce+clear" : "reduce only ", us, bytes / us / 1e6); fflush(stdout); }
#define RUNS(V, STRIDE, POLICY, BLOCKS, CLEAR) RUNC(V, STRIDE, POLICY, BLOCKS, CLEAR, 0)
#define RUNC(V, STRIDE, POLICY, BLOCKS, CLEAR, CV) if ((n * per * 4) % ((long)V * STRIDE) != 0 || (CV && (n * per * 4) % ((long)CV * 4096) != 0)) { printf("skipped: region not a multiple of the tile pattern\n"); } else { auto k = rmw_strided<V, STRIDE, POLICY, CV>; \
    const long rt = n * per / (256L * V * 4), ct = CLEAR ? (CV ? n * per / (256L * CV * 4) : rt) : 0; if (CV) printf("clear tiles of %d dense slabs: ", CV); \
    for (int i = 0; i < 2; ++i) hipLaunchKernelGGL(k, dim3(BLOCKS), dim3(256), 0, 0, G, P, Z, rt, ct); CK(hipDeviceSynchronize()); \
    const int it = 6; CK(hipEventRecord(e0)); for (int i = 0; i < it; ++i) hipLaunchKernelGGL(k, dim3(BLOCKS), dim3(256), 0, 0, G, P, Z, rt, ct); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); \
    float ms; CK(hipEventElapsedTime(&ms, e0, e1)); CK(hipGetLastError()); const double us = ms * 1e3 / it; const double bytes = (double)n * per * 4 * (CLEAR ? 4 : 3); \
    printf("strided registers V=%d stride=%3dK %s blocks=%4d %s: %7.1f us %5.2f TB/s\n", V, STRIDE / 1024, POLICY ? "nontemporal" : "through    ", BLOCKS, CLEAR ? "reduce+clear" : "reduce only ", us, bytes / us / 1e6); fflush(stdout); }
#define RUNSP(V, STRIDE, CV, FF, RB) if ((n * per * 4) % ((long)V * STRIDE) != 0 || (n * per * 4) % ((long)CV * 4096) != 0) { printf("skipped: region not a multiple of the tile pattern\n"); } else { auto k = rmw_split<V, STRIDE, CV, FF>; const long rt = n * per / (256L * V * 4), fb = n * per / (256L * CV * 4); \
    for (int i = 0; i < 2; ++i) hipLaunchKernelGGL(k, dim3((unsigned)(fb + RB)), dim3(256), 0, 0, G, P, Z, rt, fb, RB); CK(hipDeviceSynchronize()); \
    const int it = 6; CK(hipEventRecord(e0)); for (int i = 0; i < it; ++i) hipLaunchKernelGGL(k, dim3((unsigned)(fb + RB)), dim3(256), 0, 0, G, P, Z, rt, fb, RB); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); \
    float ms; CK(hipEventElapsedTime(&ms, e0, e1)); CK(hipGetLastError()); const double us = ms * 1e3 / it; const double bytes = (double)n * per * 4 * 4; \
    printf("split launch V=%d stride=%dK, fill blocks of %d slabs %s, %d reduce blocks: %7.1f us %5.2f TB/s\n", V, STRIDE / 1024, CV, FF ? "first" : "last ", RB, us, bytes / us / 1e6); fflush(stdout); }
#define RUNS2(V, STRIDE, RB, F, CLEAR) if ((n * per * 4) % ((long)V * STRIDE) != 0) { printf("skipped\n"); } else { auto k = rmw_split2<V, STRIDE>; const long rt = n * per / (256L * V * 4), cs = CLEAR ? n * per * 4 / 4096 : 0; \
    for (int i = 0; i < 2; ++i) hipLaunchKernelGGL(k, dim3(RB + F), dim3(256), 0, 0, G, P, Z, rt, cs, RB); CK(hipDeviceSynchronize()); \
    const int it = 6; CK(hipEventRecord(e0)); for (int i = 0; i < it; ++i) hipLaunchKernelGGL(k, dim3(RB + F), dim3(256), 0, 0, G, P, Z, rt, cs, RB); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); \
    float ms; CK(hipEventElapsedTime(&ms, e0, e1)); CK(hipGetLastError()); const double us = ms * 1e3 / it; const double bytes = (double)n * per * 4 * (CLEAR ? 4 : 3); \
    printf("split2 V=%d stride=%dK, %d reduce blocks, %d fill blocks, %s: %7.1f us %5.2f TB/s\n", V, STRIDE / 1024, RB, F, CLEAR ? "reduce+clear" : "reduce only ", us, bytes / us / 1e6); fflush(stdout); }
#define RUNCP(V, STRIDE, BLOCKS) if ((n * per * 4) % ((long)V * STRIDE) != 0) { printf("skipped\n"); } else { auto k = copy_strided<V, STRIDE>; const long rt = n * per / (256L * V * 4); \
    for (int i = 0; i < 2; ++i) hipLaunchKernelGGL(k, dim3(BLOCKS), dim3(256), 0, 0, P, G, rt); CK(hipDeviceSynchronize()); \
    const int it = 6; CK(hipEventRecord(e0)); for (int i = 0; i < it; ++i) hipLaunchKernelGGL(k, dim3(BLOCKS), dim3(256), 0, 0, P, G, rt); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); \
    float ms; CK(hipEventElapsedTime(&ms, e0, e1)); CK(hipGetLastError()); const double us = ms * 1e3 / it; const double bytes = (double)n * per * 4 * 2; \
    printf("copy V=%d stride=%dK blocks=%d: %7.1f us %5.2f TB/s\n", V, STRIDE / 1024, BLOCKS, us, bytes / us / 1e6); fflush(stdout); }
#define RUNI(V, STRIDE, FS, FB, BLOCKS) if ((n * per * 4) % ((long)V * STRIDE) != 0) { printf("skipped\n"); } else { auto k = rmw_inter<V, STRIDE, FS, FB>; const long rt = n * per / (256L * V * 4), cs = n * per * 4 / 4096; \
    for (int i = 0; i < 2; ++i) hipLaunchKernelGGL(k, dim3(BLOCKS), dim3(256), 0, 0, G, P, Z, rt, cs); CK(hipDeviceSynchronize()); \
    const int it = 6; CK(hipEventRecord(e0)); for (int i = 0; i < it; ++i) hipLaunchKernelGGL(k, dim3(BLOCKS), dim3(256), 0, 0, G, P, Z, rt, cs); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1)); \
    float ms; CK(hipEventElapsedTime(&ms, e0, e1)); CK(hipGetLastError()); const double us = ms * 1e3 / it; const double bytes = (double)n * per * 4 * 4; \
    printf("interleaved V=%d stride=%dK, %d fill slabs %s each tile, %d blocks: %7.1f us %5.2f TB/s\n", V, STRIDE / 1024, FS, FB ? "before" : "after", BLOCKS, us, bytes / us / 1e6); fflush(stdout); }
  for (int rep = 0; rep < 2; ++rep) {
    printf("--- pass %d\n", rep);
    // layout: a thread's vectors 4 KiB apart, zeroes as tiles after the sums
    RUN(8, false, 512, 1, "registers") RUN(4, false, 1024, 1, "registers") RUN(8, false, 512, 0, "registers")
    RUN(4, true, 768, 1, "LDS-direct (64 KB/WG)") RUN(4, true, 512, 0, "LDS-direct (64 KB/WG)")
    // vectors STRIDE apart
    RUNS(8, 4096, 0, 512, 1) RUNS(8, 16384, 0, 512, 1) RUNS(8, 32768, 0, 512, 1) RUNS(8, 65536, 0, 512, 1) RUNS(8, 262144, 0, 512, 1)
    RUNS(14, 32768, 0, 512, 1) RUNS(8, 32768, 1, 512, 1) RUNS(8, 32768, 0, 512, 0) RUNS(8, 4096, 0, 512, 0)
    RUNC(14, 32768, 0, 512, 1, 1)
    // fills as workgroups of their own
    RUNSP(4, 32768, 1, false, 192) RUNSP(4, 32768, 1, false, 256) RUNSP(4, 32768, 1, false, 320) RUNSP(4, 32768, 1, false, 512)
    RUNSP(8, 32768, 1, false, 256) RUNSP(2, 32768, 1, false, 256) RUNSP(4, 4096, 1, false, 256) RUNSP(4, 32768, 1, true, 256)
    RUNS2(4, 32768, 256, 1024, 1) RUNS2(4, 32768, 256, 4096, 1) RUNS2(4, 32768, 256, 16384, 1) RUNS2(4, 32768, 256, 32768, 1) RUNS2(4, 32768, 256, 114688, 1)
    RUNS2(4, 32768, 256, 0, 0) RUNS2(4, 32768, 512, 0, 0) RUNS2(8, 32768, 512, 0, 0) RUNS2(4, 32768, 256, 32768, 0) RUNS2(4, 32768, 256, 458752, 0)
    // fills between the tiles
    RUNI(4, 32768, 4, false, 256) RUNI(4, 32768, 4, true, 256) RUNI(4, 32768, 4, false, 512) RUNI(4, 32768, 4, false, 1024) RUNI(8, 32768, 8, false, 256) RUNI(2, 32768, 2, false, 512)
    // a copy of the same size
    RUNCP(4, 4096, 1792) RUNCP(4, 32768, 1792) RUNCP(4, 32768, 512) RUNCP(4, 4096, 512)
  }
  return 0;
}
