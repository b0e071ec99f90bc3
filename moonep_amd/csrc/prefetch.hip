// Plan-driven expert-weight movement for gfx950:
//   prefetch    -- every owned expert that some rank hosts remotely is read
//                  once and streamed to each requesting (rank, slot);
//   grad reduce -- the fp32 grads accumulated in those slots are summed back
//                  into the owner's grad in (rank, slot) order, then the
//                  rank's own slots are cleared.
// Both are flat 16-byte-vector streaming kernels over a slot table that each
// workgroup rebuilds in LDS from experts_to_copy (a few hundred ints), so no
// host round trip and no second launch is needed to learn the work list.
#include "mep_common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kVecPerThread = 4;                       // 16-byte vectors in flight per thread
constexpr int kTileBytes = kBlock * kVecPerThread * 16;  // 16 KiB per workgroup step
constexpr int kMaxTensors = 6;

// Slot table of `rank`: for each owned (local) expert the slots rb = d*epn+b
// holding it, ascending.  LDS: s_e[R*epn], s_list[R*epn], s_off[epn+1],
// s_active[epn], s_misc[2].
struct SlotTable {
  int* e; int* list; int* off; int* active; int* misc;
  __device__ void carve(int* smem, int R, int epn) {
    e = smem; list = e + R * epn; off = list + R * epn; active = off + epn + 1;
    misc = active + epn;
  }
  // all threads of the workgroup call this
  __device__ void build(const int* etc, int rank, int R, int epn) {
    const int n = R * epn;
    const int lo = rank * epn;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const int v = etc[i] - lo;
      e[i] = ((unsigned)v < (unsigned)epn) ? v : -1;
    }
    __syncthreads();
    // counts per local expert
    for (int le = threadIdx.x; le < epn; le += blockDim.x) {
      int c = 0;
      for (int i = 0; i < n; ++i) c += (e[i] == le);
      off[le + 1] = c;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      int run = 0, na = 0;
      off[0] = 0;
      for (int le = 0; le < epn; ++le) {
        const int c = off[le + 1];
        if (c > 0) active[na++] = le;
        run += c;
        off[le + 1] = run;
      }
      misc[0] = na;
    }
    __syncthreads();
    for (int le = threadIdx.x; le < epn; le += blockDim.x) {
      int p = off[le];
      for (int i = 0; i < n; ++i)
        if (e[i] == le) list[p++] = i;
    }
    __syncthreads();
  }
};

size_t slot_table_bytes(int R, int epn) {
  return ((size_t)2 * R * epn + 2 * (size_t)epn + 4) * sizeof(int);
}

struct PrefetchArgs {
  const char* local[kMaxTensors];
  char* pool[kMaxTensors];
  int64_t rank_stride[kMaxTensors];  // bytes
  int64_t bytes[kMaxTensors];        // per expert
  const int* etc;
  int ntensors, rank, epn, R;
};

__global__ __launch_bounds__(kBlock) void prefetch_kernel(PrefetchArgs a) {
  extern __shared__ int smem[];
  SlotTable t;
  t.carve(smem, a.R, a.epn);
  t.build(a.etc, a.rank, a.R, a.epn);
  const int n_active = t.misc[0];
  if (n_active == 0) return;
  for (int ti = 0; ti < a.ntensors; ++ti) {
    const int64_t bytes = a.bytes[ti];
    const int64_t tiles = (bytes + kTileBytes - 1) / kTileBytes;
    const int64_t work = tiles * n_active;
    for (int64_t w = blockIdx.x; w < work; w += gridDim.x) {
      const int ai = (int)(w / tiles);
      const int64_t tile = w - (int64_t)ai * tiles;
      const int le = t.active[ai];
      const int64_t boff = tile * kTileBytes;
      const char* src = a.local[ti] + (int64_t)le * bytes + boff;
      mep_u4 v[kVecPerThread];
      bool in[kVecPerThread];
#pragma unroll
      for (int i = 0; i < kVecPerThread; ++i) {
        const int64_t o = ((int64_t)i * kBlock + threadIdx.x) * 16;
        in[i] = boff + o < bytes;
        if (in[i]) v[i] = mep_ld16_stream(src + o);
      }
      const int beg = t.off[le], end = t.off[le + 1];
      for (int sidx = beg; sidx < end; ++sidx) {
        const int rb = t.list[sidx];
        const int d = rb / a.epn, b = rb - d * a.epn;
        char* dstp = a.pool[ti] + (int64_t)d * a.rank_stride[ti] + (int64_t)b * bytes + boff;
#pragma unroll
        for (int i = 0; i < kVecPerThread; ++i) {
          const int64_t o = ((int64_t)i * kBlock + threadIdx.x) * 16;
          if (in[i]) mep_st16_stream(dstp + o, v[i]);
        }
      }
    }
  }
}

struct ReduceArgs {
  float* local_grad;
  float* pool;
  int64_t rank_stride;  // elements
  int64_t elems;        // per expert
  const int* etc;
  int rank, epn, R;
};

typedef float mep_f4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(kBlock) void grad_reduce_kernel(ReduceArgs a) {
  extern __shared__ int smem[];
  SlotTable t;
  t.carve(smem, a.R, a.epn);
  t.build(a.etc, a.rank, a.R, a.epn);
  const int n_active = t.misc[0];
  if (n_active == 0) return;
  const int64_t vecs = a.elems / 4;
  constexpr int kTileVecs = kBlock * kVecPerThread;
  const int64_t tiles = (vecs + kTileVecs - 1) / kTileVecs;
  const int64_t work = tiles * n_active;
  for (int64_t w = blockIdx.x; w < work; w += gridDim.x) {
    const int ai = (int)(w / tiles);
    const int64_t tile = w - (int64_t)ai * tiles;
    const int le = t.active[ai];
    mep_f4* g = (mep_f4*)(a.local_grad + (int64_t)le * a.elems) + tile * kTileVecs;
    mep_f4 acc[kVecPerThread];
    bool in[kVecPerThread];
#pragma unroll
    for (int i = 0; i < kVecPerThread; ++i) {
      const int64_t o = (int64_t)i * kBlock + threadIdx.x;
      in[i] = tile * kTileVecs + o < vecs;
      if (in[i]) acc[i] = g[o];
    }
    const int beg = t.off[le], end = t.off[le + 1];
    for (int sidx = beg; sidx < end; ++sidx) {
      const int rb = t.list[sidx];
      const int src = rb / a.epn, b = rb - src * a.epn;
      const mep_f4* p = (const mep_f4*)(a.pool + (int64_t)src * a.rank_stride + (int64_t)b * a.elems) +
                        tile * kTileVecs;
      mep_f4 v[kVecPerThread];
#pragma unroll
      for (int i = 0; i < kVecPerThread; ++i) {
        const int64_t o = (int64_t)i * kBlock + threadIdx.x;
        if (in[i]) v[i] = __builtin_nontemporal_load(p + o);
      }
#pragma unroll
      for (int i = 0; i < kVecPerThread; ++i)
        if (in[i]) acc[i] = acc[i] + v[i];
    }
#pragma unroll
    for (int i = 0; i < kVecPerThread; ++i) {
      const int64_t o = (int64_t)i * kBlock + threadIdx.x;
      if (in[i]) g[o] = acc[i];
    }
  }
}

// zero this rank's own slots that hold any expert
__global__ __launch_bounds__(kBlock) void grad_clear_kernel(ReduceArgs a) {
  const int64_t vecs = a.elems / 4;
  constexpr int kTileVecs = kBlock * kVecPerThread;
  const int64_t tiles = (vecs + kTileVecs - 1) / kTileVecs;
  const int64_t work = tiles * a.epn;
  const mep_f4 zero = {0.f, 0.f, 0.f, 0.f};
  for (int64_t w = blockIdx.x; w < work; w += gridDim.x) {
    const int b = (int)(w / tiles);
    if (a.etc[a.rank * a.epn + b] < 0) continue;
    const int64_t tile = w - (int64_t)b * tiles;
    mep_f4* p = (mep_f4*)(a.pool + (int64_t)a.rank * a.rank_stride + (int64_t)b * a.elems) +
                tile * kTileVecs;
#pragma unroll
    for (int i = 0; i < kVecPerThread; ++i) {
      const int64_t o = (int64_t)i * kBlock + threadIdx.x;
      if (tile * kTileVecs + o < vecs) __builtin_nontemporal_store(zero, p + o);
    }
  }
}

constexpr int kStreamBlocks = 256 * 8;  // persistent workgroups: 8 per CU

}  // namespace

extern "C" int mep_prefetch(int ntensors, const void* const* local, void* const* pool,
                            const int64_t* rank_stride_bytes, const int64_t* bytes_per_expert,
                            const int32_t* experts_to_copy, int rank, int epn, int R,
                            void* stream) {
  MEP_REQUIRE(local && pool && rank_stride_bytes && bytes_per_expert && experts_to_copy,
              MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(ntensors > 0 && ntensors <= kMaxTensors, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(epn > 0 && R > 0 && rank >= 0 && rank < R, MEP_ERR_INVALID_ARG);
  const size_t lds = slot_table_bytes(R, epn);
  MEP_REQUIRE(lds <= 64 * 1024, MEP_ERR_UNSUPPORTED);
  PrefetchArgs a;
  a.ntensors = ntensors; a.rank = rank; a.epn = epn; a.R = R; a.etc = experts_to_copy;
  int64_t max_tiles = 0;
  for (int i = 0; i < ntensors; ++i) {
    MEP_REQUIRE(local[i] && pool[i], MEP_ERR_INVALID_ARG);
    MEP_REQUIRE(bytes_per_expert[i] > 0 && bytes_per_expert[i] % 16 == 0, MEP_ERR_UNSUPPORTED);
    MEP_REQUIRE(rank_stride_bytes[i] >= bytes_per_expert[i] * epn, MEP_ERR_INVALID_ARG);
    MEP_REQUIRE(rank_stride_bytes[i] % 16 == 0 && (uintptr_t)local[i] % 16 == 0 &&
                    (uintptr_t)pool[i] % 16 == 0, MEP_ERR_ALIGNMENT);
    a.local[i] = (const char*)local[i]; a.pool[i] = (char*)pool[i];
    a.rank_stride[i] = rank_stride_bytes[i]; a.bytes[i] = bytes_per_expert[i];
    const int64_t tiles = (bytes_per_expert[i] + kTileBytes - 1) / kTileBytes * epn;
    if (tiles > max_tiles) max_tiles = tiles;
  }
  const int blocks = (int)(max_tiles < kStreamBlocks ? max_tiles : kStreamBlocks);
  hipLaunchKernelGGL(prefetch_kernel, dim3(blocks), dim3(kBlock), lds, (hipStream_t)stream, a);
  return mep_launch_status();
}

extern "C" int mep_grad_reduce(float* local_grad, float* reduce_pool, int64_t rank_stride_elems,
                               const int32_t* experts_to_copy, int rank, int epn, int R,
                               int64_t elems_per_expert, void* stream) {
  MEP_REQUIRE(local_grad && reduce_pool && experts_to_copy, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(epn > 0 && R > 0 && rank >= 0 && rank < R && elems_per_expert > 0,
              MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(elems_per_expert % 4 == 0, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(rank_stride_elems >= elems_per_expert * epn, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(rank_stride_elems % 4 == 0 && (uintptr_t)local_grad % 16 == 0 &&
                  (uintptr_t)reduce_pool % 16 == 0, MEP_ERR_ALIGNMENT);
  const size_t lds = slot_table_bytes(R, epn);
  MEP_REQUIRE(lds <= 64 * 1024, MEP_ERR_UNSUPPORTED);
  ReduceArgs a{local_grad, reduce_pool, rank_stride_elems, elems_per_expert, experts_to_copy,
               rank, epn, R};
  const int64_t tiles = (elems_per_expert / 4 + kBlock * kVecPerThread - 1) /
                        (kBlock * kVecPerThread) * epn;
  const int blocks = (int)(tiles < kStreamBlocks ? tiles : kStreamBlocks);
  hipStream_t st = (hipStream_t)stream;
  // two launches: the clear must not overtake reads of a slot that holds one
  // of this rank's own experts
  hipLaunchKernelGGL(grad_reduce_kernel, dim3(blocks), dim3(kBlock), lds, st, a);
  hipLaunchKernelGGL(grad_clear_kernel, dim3(blocks), dim3(kBlock), 0, st, a);
  return mep_launch_status();
}
