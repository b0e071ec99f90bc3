// Dispatch side of the hot path for gfx950: fused permute (one wave per copy of
// a token row; the row is read with ordinary loads -- it was just produced and
// is shared by the token's K waves through the caches -- and streamed to its
// slot with nontemporal stores, which leave the cached inputs alone), weight
// scatter, padding zero-fill, duplicate-group builder and the destination-side
// duplicate expansion.
#include "mep_common.h"

#include <atomic>

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * MEP_WAVE;

struct DispatchArgs {
  const uint16_t* hidden;  // [S,H] bf16
  const float* w;          // [S,K] or null
  const int* dst;          // [S*K]
  const int* zero_fill;    // [2*epn,2]
  uint16_t* shards;
  float* wslots;
  int64_t shard_stride_rows, wslot_stride;
  int rank, S, H, K, R, NvS, groups, tok_blocks, zblocks, zblocks_per_group;
  unsigned flags;
};

// One wave per (token, k) copy: it reads the token row (the K waves of a token
// share it through the caches) and streams it to its slot.  Waves that issue
// one row of stores each keep the HBM write path busier than one wave issuing
// K rows.  NV > 0: the row is exactly NV 16-byte vectors per lane and passes
// through registers in one go; NV == 0: any H % 8 == 0, strided loop.
template <int NV>
__global__ __launch_bounds__(kBlock) void dispatch_kernel(DispatchArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int H = a.H;
  const size_t row_bytes = (size_t)H * 2;
  // the (few, short) zero-fill workgroups come first in the grid so that they
  // overlap with the copies instead of forming a tail
  if ((int)blockIdx.x >= a.zblocks) {
    const int64_t gw = (int64_t)(blockIdx.x - a.zblocks) * kWavesPerBlock + wave;  // flat (token, k) index
    if (gw >= (int64_t)a.S * a.K) return;
    const int s = (int)(gw / a.K);
    const int dv = a.dst[gw];
    const int raw = dv < 0 ? -dv - 1 : dv;
    const int drank = raw / a.NvS;
    const int loff = raw - drank * a.NvS;
    if (drank >= a.R) return;  // never write outside the shards
    if (a.w && lane == 0) a.wslots[(size_t)drank * a.wslot_stride + loff] = a.w[gw];
    if (dv < 0 && !(a.flags & MEP_DISPATCH_WRITE_DUPS)) return;
    const char* src = (const char*)a.hidden + (size_t)s * row_bytes + (size_t)lane * 16;
    char* row = (char*)a.shards +
                ((uint64_t)drank * (uint64_t)a.shard_stride_rows + (uint64_t)loff) * row_bytes +
                (size_t)lane * 16;
    if (NV > 0) {
      mep_u4 v[NV > 0 ? NV : 1];
#pragma unroll
      for (int i = 0; i < NV; ++i) v[i] = mep_ld16(src + (size_t)i * 1024);
#pragma unroll
      for (int i = 0; i < NV; ++i) mep_st16_stream(row + (size_t)i * 1024, v[i]);
    } else {
      const int nvec = H / 8;
      for (int c0 = 0; c0 < nvec; c0 += 4 * 64) {
        mep_u4 v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (c0 + i * 64 + lane < nvec) v[i] = mep_ld16(src + (size_t)(c0 + i * 64) * 16);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (c0 + i * 64 + lane < nvec) mep_st16_stream(row + (size_t)(c0 + i * 64) * 16, v[i]);
      }
    }
    return;
  }
  // ---- zero-fill of this rank's padding rows (and their weight slots) -----
  const int zb = blockIdx.x;
  const int g = zb / a.zblocks_per_group;
  const int part = zb - g * a.zblocks_per_group;
  if (g >= a.groups) return;
  const int pad_start = a.zero_fill[2 * g];
  int n_pad = a.zero_fill[2 * g + 1];
  if (n_pad <= 0 || pad_start < 0) return;
  if ((int64_t)pad_start + n_pad > a.NvS) n_pad = a.NvS - pad_start;
  // The padding rows of a group are one contiguous byte range: the group's workgroups fill it
  // densely, every thread one 16-byte store per step and consecutive workgroups consecutive
  // 4-KiB pieces -- the store order the memory system takes fastest (a wave per 14-KiB row
  // costs a third more).
  const mep_u4 zero = {0u, 0u, 0u, 0u};
  char* base = (char*)a.shards +
               ((uint64_t)a.rank * (uint64_t)a.shard_stride_rows + (uint64_t)pad_start) * row_bytes;
  const size_t region = (size_t)n_pad * row_bytes;              // a multiple of 16 (H % 8 == 0)
  const size_t step = (size_t)a.zblocks_per_group * kBlock * 16;
  for (size_t off = ((size_t)part * kBlock + threadIdx.x) * 16; off < region; off += step)
    mep_st16_stream(base + off, zero);
  if (a.w && part == 0)
    for (int j = threadIdx.x; j < n_pad; j += kBlock)
      a.wslots[(size_t)a.rank * a.wslot_stride + pad_start + j] = 0.0f;
}

// ---------------------------------------------------------------------------
// duplicate groups of one destination rank from every source rank's dst
// ---------------------------------------------------------------------------
// pass 1: per workgroup of tokens: (#groups, #duplicates) that `rank` holds of them
// pass 2: every workgroup adds up the sums of the workgroups before it, scans its own
//         tokens and emits their groups in token order; the last one stores the totals
struct DedupArgs {
  const int* dst;  // [R, S*K]
  int* dup_groups; int* dup_loffs; int* dup_counts;
  int* blk_sums;   // [2*nblk] per-workgroup (#groups, #dups)
  int rank, S, K, R, NvS, ntok, nblk;
  int vec;         // rows of dst can be read as 16-byte vectors
};

constexpr int kDedupBlock = 256;

// entries of token t that land on `rank`: raw / NvS == rank, as a range test
__device__ __forceinline__ int dedup_entries_on_rank(const DedupArgs& a, int t) {
  const int lo = a.rank * a.NvS, hi = lo + a.NvS;  // fits: the host requires R*NvS <= INT32_MAX
  auto on = [&](int v) { const int raw = v < 0 ? -v - 1 : v; return (int)(raw >= lo && raw < hi); };
  const int* d = a.dst + (size_t)t * a.K;
  int c = 0;
  if (a.vec) {
    const int4* d4 = (const int4*)d;
    for (int k = 0; k < a.K / 4; ++k) {
      const int4 v = d4[k];
      c += on(v.x) + on(v.y) + on(v.z) + on(v.w);
    }
  } else {
    for (int k = 0; k < a.K; ++k) c += on(d[k]);
  }
  return c;
}

// (sum of g, sum of d) over the workgroup, in every thread
__device__ __forceinline__ void dedup_block_sums(int g, int d, int* s_g, int* s_d, int& tg, int& td) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int gs = mep_wave_incl_scan(g), ds = mep_wave_incl_scan(d);
  if (lane == 63) { s_g[wave] = gs; s_d[wave] = ds; }
  __syncthreads();
  tg = 0; td = 0;
  for (int w = 0; w < kDedupBlock / 64; ++w) { tg += s_g[w]; td += s_d[w]; }
  __syncthreads();
}

__global__ __launch_bounds__(kDedupBlock) void dedup_count_kernel(DedupArgs a) {
  __shared__ int s_g[kDedupBlock / 64], s_d[kDedupBlock / 64];
  const int t = blockIdx.x * kDedupBlock + threadIdx.x;
  int nd = 0;
  if (t < a.ntok) {
    const int c = dedup_entries_on_rank(a, t);
    nd = c > 1 ? c - 1 : 0;
  }
  int tg, td;
  dedup_block_sums(nd > 0 ? 1 : 0, nd, s_g, s_d, tg, td);
  if (threadIdx.x == 0) {
    a.blk_sums[2 * blockIdx.x] = tg;
    a.blk_sums[2 * blockIdx.x + 1] = td;
  }
}

__global__ __launch_bounds__(kDedupBlock) void dedup_emit_kernel(DedupArgs a) {
  __shared__ int s_g[kDedupBlock / 64], s_d[kDedupBlock / 64];
  const int t = blockIdx.x * kDedupBlock + threadIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // what the workgroups before this one hold
  int pg = 0, pd = 0;
  for (int b = threadIdx.x; b < (int)blockIdx.x; b += kDedupBlock) {
    pg += a.blk_sums[2 * b];
    pd += a.blk_sums[2 * b + 1];
  }
  int og, od;
  dedup_block_sums(pg, pd, s_g, s_d, og, od);
  int nd = 0;
  if (t < a.ntok) {
    const int c = dedup_entries_on_rank(a, t);
    nd = c > 1 ? c - 1 : 0;
  }
  const int g = nd > 0 ? 1 : 0;
  const int gi = mep_wave_incl_scan(g), di = mep_wave_incl_scan(nd);
  if (lane == 63) { s_g[wave] = gi; s_d[wave] = di; }
  __syncthreads();
  int tg = og, td = od;  // totals up to and including this workgroup
  for (int w = 0; w < kDedupBlock / 64; ++w) {
    if (w < wave) { og += s_g[w]; od += s_d[w]; }
    tg += s_g[w]; td += s_d[w];
  }
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) { a.dup_counts[0] = tg; a.dup_counts[1] = td; }
  if (nd > 0) {
    const int lo = a.rank * a.NvS, hi = lo + a.NvS;
    const int gidx = og + gi - 1;
    int dpos = od + di - nd;
    const int* d = a.dst + (size_t)t * a.K;
    bool first = true;
    for (int k = 0; k < a.K; ++k) {
      const int v = d[k];
      const int raw = v < 0 ? -v - 1 : v;
      if (raw < lo || raw >= hi) continue;
      const int loff = raw - lo;
      if (first) {
        a.dup_groups[3 * gidx] = loff;
        a.dup_groups[3 * gidx + 1] = dpos;
        a.dup_groups[3 * gidx + 2] = nd;
        first = false;
      } else {
        a.dup_loffs[dpos++] = loff;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// duplicate expansion / pre-reduction on one shard: one wave per group
// ---------------------------------------------------------------------------
struct DupArgs {
  uint16_t* shard;
  const int* dup_groups; const int* dup_loffs; const int* dup_counts;
  int NvS, H;
};

// Workgroups of 4 waves by default; of 16 waves when the caller bounds the number of
// compute units (one workgroup per CU then, so each CU still has enough rows in flight).
constexpr int kDupBlockMax = 1024;
constexpr int kDupCH = 2;  // 1-KiB pieces of a row per wave and work item

// A work item is (group, piece of the row): kDupCH consecutive 1-KiB pieces (64 lanes x 16
// bytes).  Consecutive waves take consecutive pieces of one group, the waves grid-stride
// over the items (their number is only known on the device).  A wave reads the group's
// row numbers once, one per lane, before it touches a row, so that no row access waits for
// an index load.
// PROLOGUE: primary <- bf16(fp32 sum of the primary and its duplicates, in list order);
// otherwise: every duplicate row <- the primary.
template <bool PROLOGUE>
__global__ __launch_bounds__(kDupBlockMax) void dup_rows_kernel(DupArgs a) {
  const int lane = threadIdx.x & 63;
  const int wpb = blockDim.x >> 6;
  const int gw = blockIdx.x * wpb + (threadIdx.x >> 6);
  const int nw = gridDim.x * wpb;
  int ng = a.dup_counts[0];
  if (ng > a.NvS) ng = a.NvS;
  const size_t row_bytes = (size_t)a.H * 2;
  const int nvec = a.H / 8;
  const int parts = (nvec + kDupCH * 64 - 1) / (kDupCH * 64);
  const int64_t items = (int64_t)ng * parts;
  for (int64_t it = gw; it < items; it += nw) {
    const int g = (int)(it / parts);
    const int part = (int)(it - (int64_t)g * parts);
    const int p = a.dup_groups[3 * g], start = a.dup_groups[3 * g + 1], n = a.dup_groups[3 * g + 2];
    if ((unsigned)p >= (unsigned)a.NvS || start < 0 || n <= 0 || (int64_t)start + n > a.NvS) continue;
    const int c0 = part * kDupCH * 64 + lane;
    bool ok[kDupCH];
#pragma unroll
    for (int i = 0; i < kDupCH; ++i) ok[i] = c0 + i * 64 < nvec;
    char* prow = (char*)a.shard + (size_t)p * row_bytes + (size_t)c0 * 16;
    mep_u4 v[kDupCH];
#pragma unroll
    for (int i = 0; i < kDupCH; ++i)
      if (ok[i]) v[i] = mep_ld16(prow + (size_t)i * 1024);
    float acc[kDupCH][8];
    if (PROLOGUE) {
#pragma unroll
      for (int i = 0; i < kDupCH; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          acc[i][2 * q] = 0.0f + mep_bf16_lo(v[i][q]);
          acc[i][2 * q + 1] = 0.0f + mep_bf16_hi(v[i][q]);
        }
    }
    for (int j0 = 0; j0 < n; j0 += 64) {
      const int nj = n - j0 < 64 ? n - j0 : 64;
      const int mine = lane < nj ? a.dup_loffs[start + j0 + lane] : -1;
      for (int j = 0; j < nj; ++j) {
        const int lo = __builtin_amdgcn_readlane(mine, j);
        if ((unsigned)lo >= (unsigned)a.NvS) continue;
        char* row = (char*)a.shard + (size_t)lo * row_bytes + (size_t)c0 * 16;
        if (PROLOGUE) {
          mep_u4 d[kDupCH];
#pragma unroll
          for (int i = 0; i < kDupCH; ++i)
            if (ok[i]) d[i] = mep_ld16(row + (size_t)i * 1024);
#pragma unroll
          for (int i = 0; i < kDupCH; ++i)
            if (ok[i]) {
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                acc[i][2 * q] += mep_bf16_lo(d[i][q]);
                acc[i][2 * q + 1] += mep_bf16_hi(d[i][q]);
              }
            }
        } else {
#pragma unroll
          for (int i = 0; i < kDupCH; ++i)
            if (ok[i]) mep_st16(row + (size_t)i * 1024, v[i]);
        }
      }
    }
    if (PROLOGUE) {
#pragma unroll
      for (int i = 0; i < kDupCH; ++i)
        if (ok[i]) {
          mep_u4 o;
#pragma unroll
          for (int q = 0; q < 4; ++q) o[q] = mep_pack_bf16(acc[i][2 * q], acc[i][2 * q + 1]);
          mep_st16(prow + (size_t)i * 1024, o);
        }
    }
  }
}

// Launch shape of the duplicate kernels (they grid-stride over the groups, whose number is
// only known on the device).  max_cus <= 0: up to 2048 workgroups of 4 waves.  max_cus = N:
// at most N workgroups (of 16 waves), so at most N compute units work on it -- the bound
// the reference sizes these two grids with (MOONEP_NUM_SMS_DEDUP, moonep/api.py:100-120).
void dup_launch_shape(int NvS, int max_cus, dim3* grid, dim3* block) {
  if (max_cus > 0) {
    const int wpb = kDupBlockMax / MEP_WAVE;
    int blocks = (NvS + wpb - 1) / wpb;
    if (blocks > max_cus) blocks = max_cus;
    *grid = dim3(blocks > 0 ? blocks : 1);
    *block = dim3(kDupBlockMax);
    return;
  }
  int blocks = (NvS + kWavesPerBlock - 1) / kWavesPerBlock;
  *grid = dim3(blocks < 2048 ? (blocks > 0 ? blocks : 1) : 2048);
  *block = dim3(kBlock);
}

}  // namespace

extern "C" int mep_dispatch(const void* hidden_SH, const float* w_SK, const int32_t* dst,
                            const int32_t* zero_fill, void* shards, int64_t shard_stride_rows,
                            float* wslots, int64_t wslot_stride, int rank, int S, int H, int K,
                            int R, int epn, int NvS, int token_padding, unsigned flags,
                            void* stream) {
  MEP_REQUIRE(hidden_SH && dst && shards, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE((w_SK == nullptr) == (wslots == nullptr), MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(S > 0 && H > 0 && K > 0 && R > 0 && epn > 0 && NvS > 0 && token_padding > 0,
              MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(rank >= 0 && rank < R, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(K <= 32, MEP_ERR_UNSUPPORTED);
  // an entry decodes as (raw / NvS, raw % NvS); raw = R*NvS (rank R) marks an entry nobody copies
  MEP_REQUIRE((int64_t)R * NvS <= INT32_MAX, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(H % 8 == 0, MEP_ERR_UNSUPPORTED);  // 16-byte row vectors (reference dispatch.py:901)
  MEP_REQUIRE(shard_stride_rows >= NvS && (!wslots || wslot_stride >= NvS), MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(((uintptr_t)hidden_SH % 16 == 0) && ((uintptr_t)shards % 16 == 0), MEP_ERR_ALIGNMENT);
  const bool zf = zero_fill && !(flags & MEP_DISPATCH_NO_ZERO_FILL);
  DispatchArgs a;
  a.hidden = (const uint16_t*)hidden_SH; a.w = w_SK; a.dst = dst; a.zero_fill = zero_fill;
  a.shards = (uint16_t*)shards; a.wslots = wslots;
  a.shard_stride_rows = shard_stride_rows; a.wslot_stride = wslot_stride;
  a.rank = rank; a.S = S; a.H = H; a.K = K; a.R = R; a.NvS = NvS; a.flags = flags;
  a.groups = zf ? 2 * epn : 0;
  a.tok_blocks = (int)(((int64_t)S * K + kWavesPerBlock - 1) / kWavesPerBlock);
  int zpg = (token_padding - 1 + kWavesPerBlock - 1) / kWavesPerBlock;
  if (zpg > 32) zpg = 32;
  if (zpg < 1) zpg = 1;
  a.zblocks_per_group = zpg;
  const int zblocks = (zf && token_padding > 1) ? a.groups * zpg : 0;
  if (zblocks == 0) a.groups = 0;
  a.zblocks = zblocks;
  dim3 grid(a.tok_blocks + zblocks);
  hipStream_t st = (hipStream_t)stream;
  // rows that are a whole number of 1-KiB wave tiles (H % 512 == 0, up to H = 8192) pass
  // through registers in one go; any other H % 8 == 0 takes the strided loop
  const int nvec = H / 8;
  const int tiles = nvec % 64 == 0 ? nvec / 64 : 0;
  switch (tiles) {
#define MEP_DISPATCH_CASE(NV) \
    case NV: hipLaunchKernelGGL(dispatch_kernel<NV>, grid, dim3(kBlock), 0, st, a); break;
    MEP_DISPATCH_CASE(1) MEP_DISPATCH_CASE(2) MEP_DISPATCH_CASE(3) MEP_DISPATCH_CASE(4)
    MEP_DISPATCH_CASE(5) MEP_DISPATCH_CASE(6) MEP_DISPATCH_CASE(7) MEP_DISPATCH_CASE(8)
    MEP_DISPATCH_CASE(9) MEP_DISPATCH_CASE(10) MEP_DISPATCH_CASE(11) MEP_DISPATCH_CASE(12)
    MEP_DISPATCH_CASE(13) MEP_DISPATCH_CASE(14) MEP_DISPATCH_CASE(15) MEP_DISPATCH_CASE(16)
#undef MEP_DISPATCH_CASE
    default: hipLaunchKernelGGL(dispatch_kernel<0>, grid, dim3(kBlock), 0, st, a); break;
  }
  return mep_launch_status();
}

extern "C" size_t mep_dedup_scratch_bytes(int S, int R) {
  if (S <= 0 || R <= 0) return 0;
  const size_t ntok = (size_t)S * R;
  const size_t nblk = (ntok + kDedupBlock - 1) / kDedupBlock;
  return (ntok + 2 * nblk) * sizeof(int);
}

namespace {

// Fixed scratch of mep_build_dedup_static: what mep_dedup_scratch_bytes asks for (one
// word per token and the builder's per-workgroup sums; the kernels use the sums), for
// callers that cannot allocate.  1 MiB covers S*R up to 260 000 tokens (the headline shape needs
// 129 KiB).  Every GPU the library runs on holds its own copy at its own
// address until the process ends; host code must never pass the array's name
// to a kernel (on the host it is only a handle for the symbol lookup) but the
// address hipGetSymbolAddress returns for the current device.
constexpr size_t kStaticDedupBytes = (size_t)1 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticDedupBytes];

constexpr int kMaxDevices = 64;
std::atomic<void*> g_static_scratch[kMaxDevices];  // device address per device, null = not looked up

// Device address of `scratch` on the current device; looked up once per device.
int static_scratch_ptr(void** out) {
  int dev = 0;
  MEP_RETURN_IF_HIP(hipGetDevice(&dev));
  MEP_REQUIRE(dev >= 0 && dev < kMaxDevices, MEP_ERR_UNSUPPORTED);
  void* p = g_static_scratch[dev].load(std::memory_order_acquire);
  if (!p) {
    MEP_RETURN_IF_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    MEP_REQUIRE(p != nullptr, MEP_ERR_SCRATCH);
    g_static_scratch[dev].store(p, std::memory_order_release);  // racing threads store the same address
  }
  *out = p;
  return MEP_OK;
}

}  // namespace

extern "C" int mep_build_dedup_static(const int32_t* dst_RN, int rank, int S, int K, int R, int NvS,
                                      int32_t* dup_groups, int32_t* dup_loffs,
                                      int32_t* dup_counts, void* stream) {
  MEP_REQUIRE(dst_RN && dup_groups && dup_loffs && dup_counts, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(S > 0 && K > 0 && R > 0 && NvS > 0 && rank >= 0 && rank < R, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE((int64_t)S * R < INT32_MAX && (int64_t)R * NvS <= INT32_MAX, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(mep_dedup_scratch_bytes(S, R) <= kStaticDedupBytes, MEP_ERR_STATIC_LIMIT);
  void* p = nullptr;
  const int rc = static_scratch_ptr(&p);
  if (rc != MEP_OK) return rc;
  // Nothing needs clearing: the first kernel writes every word of the scratch that
  // the second reads (blk_sums[0, 2*nblk)) within this call.
  return mep_build_dedup(dst_RN, rank, S, K, R, NvS, dup_groups, dup_loffs, dup_counts, p,
                         kStaticDedupBytes, stream);
}

extern "C" int mep_build_dedup(const int32_t* dst_RN, int rank, int S, int K, int R, int NvS,
                               int32_t* dup_groups, int32_t* dup_loffs, int32_t* dup_counts,
                               void* workspace, size_t workspace_bytes, void* stream) {
  MEP_REQUIRE(dst_RN && dup_groups && dup_loffs && dup_counts, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(S > 0 && K > 0 && R > 0 && NvS > 0 && rank >= 0 && rank < R, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE((int64_t)S * R < INT32_MAX && (int64_t)R * NvS <= INT32_MAX, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(workspace && workspace_bytes >= mep_dedup_scratch_bytes(S, R), MEP_ERR_SCRATCH);
  DedupArgs a;
  a.dst = dst_RN; a.dup_groups = dup_groups; a.dup_loffs = dup_loffs; a.dup_counts = dup_counts;
  a.rank = rank; a.S = S; a.K = K; a.R = R; a.NvS = NvS;
  a.ntok = S * R;
  a.nblk = (a.ntok + kDedupBlock - 1) / kDedupBlock;
  a.blk_sums = (int*)workspace;
  a.vec = (K % 4 == 0) && ((uintptr_t)dst_RN % 16 == 0);
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(dedup_count_kernel, dim3(a.nblk), dim3(kDedupBlock), 0, st, a);
  hipLaunchKernelGGL(dedup_emit_kernel, dim3(a.nblk), dim3(kDedupBlock), 0, st, a);
  return mep_launch_status();
}

extern "C" int mep_dispatch_epilogue(void* shard, const int32_t* dup_groups,
                                     const int32_t* dup_loffs, const int32_t* dup_counts, int NvS,
                                     int H, int max_cus, void* stream) {
  MEP_REQUIRE(shard && dup_groups && dup_loffs && dup_counts, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(NvS > 0 && H > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(H % 8 == 0, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE((uintptr_t)shard % 16 == 0, MEP_ERR_ALIGNMENT);
  DupArgs a{(uint16_t*)shard, dup_groups, dup_loffs, dup_counts, NvS, H};
  dim3 grid, block;
  dup_launch_shape(NvS, max_cus, &grid, &block);
  hipLaunchKernelGGL(dup_rows_kernel<false>, grid, block, 0, (hipStream_t)stream, a);
  return mep_launch_status();
}

extern "C" int mep_combine_prologue(void* shard, const int32_t* dup_groups,
                                    const int32_t* dup_loffs, const int32_t* dup_counts, int NvS,
                                    int H, int max_cus, void* stream) {
  MEP_REQUIRE(shard && dup_groups && dup_loffs && dup_counts, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(NvS > 0 && H > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(H % 8 == 0, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE((uintptr_t)shard % 16 == 0, MEP_ERR_ALIGNMENT);
  DupArgs a{(uint16_t*)shard, dup_groups, dup_loffs, dup_counts, NvS, H};
  dim3 grid, block;
  dup_launch_shape(NvS, max_cus, &grid, &block);
  hipLaunchKernelGGL(dup_rows_kernel<true>, grid, block, 0, (hipStream_t)stream, a);
  return mep_launch_status();
}
