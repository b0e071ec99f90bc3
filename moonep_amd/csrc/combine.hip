// Top-k unpermute for gfx950: one wave per token gathers the token's rows
// from the destination shards, accumulates them in fp32 registers in
// ascending k, rounds once to bf16 and streams the row out; the same wave
// gathers the token's K route weights.
#include "mep_common.h"

namespace {

constexpr int kWavesPerBlock = 4;
constexpr int kBlock = kWavesPerBlock * MEP_WAVE;

struct CombineArgs {
  const uint16_t* shards;
  const float* wslots;
  const int* dst;
  uint16_t* out;
  float* out_sk;
  int64_t shard_stride_rows, wslot_stride;
  int S, H, K, R, NvS, mode;
};

__device__ __forceinline__ void acc8(float* acc, mep_u4 v) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    acc[2 * i] += mep_bf16_lo(v[i]);
    acc[2 * i + 1] += mep_bf16_hi(v[i]);
  }
}

// CH: 16-byte chunks a lane keeps in flight per row (unrolled).
template <int CH>
__global__ __launch_bounds__(kBlock) void combine_kernel(CombineArgs a) {
  const int lane = threadIdx.x & 63;
  const int s = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  if (s >= a.S) return;
  const int K = a.K;
  const size_t row_bytes = (size_t)a.H * 2;
  int dv = 0;
  if (lane < K) dv = a.dst[(size_t)s * K + lane];
  const int raw = dv < 0 ? -dv - 1 : dv;
  const int drank = raw / a.NvS;
  const int loff = raw - drank * a.NvS;
  const bool valid = lane < K && drank < a.R;
  if (a.out_sk && lane < K)
    a.out_sk[(size_t)s * K + lane] = valid ? a.wslots[(size_t)drank * a.wslot_stride + loff] : 0.0f;
  const uint64_t off = ((uint64_t)drank * (uint64_t)a.shard_stride_rows + (uint64_t)loff) * row_bytes;
  const uint32_t off_lo = (uint32_t)off, off_hi = (uint32_t)(off >> 32);
  const bool primary = valid && dv >= 0;
  const uint64_t prim_mask = __ballot(primary);
  const uint64_t valid_mask = __ballot(valid);
  const char* base = (const char*)a.shards;
  char* orow = (char*)a.out + (size_t)s * row_bytes;
  const int nvec = a.H / 8;

  if (a.mode != MEP_COMBINE_TWO_LEVEL) {
    const uint64_t sel = a.mode == MEP_COMBINE_ALL ? valid_mask : prim_mask;
    for (int c0 = 0; c0 < nvec; c0 += CH * 64) {
      float acc[CH][8];
#pragma unroll
      for (int i = 0; i < CH; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = 0.0f;
      uint64_t t = sel;
      while (t) {
        const int k = __ffsll((unsigned long long)t) - 1;
        t &= t - 1;
        const uint64_t o = ((uint64_t)__builtin_amdgcn_readlane(off_hi, k) << 32) |
                           (uint32_t)__builtin_amdgcn_readlane(off_lo, k);
        const char* row = base + o;
        mep_u4 v[CH];
#pragma unroll
        for (int i = 0; i < CH; ++i) {
          const int c = c0 + i * 64 + lane;
          v[i] = mep_u4{0u, 0u, 0u, 0u};
          if (c < nvec) v[i] = mep_ld16_stream(row + (size_t)c * 16);
        }
#pragma unroll
        for (int i = 0; i < CH; ++i) acc8(acc[i], v[i]);
      }
#pragma unroll
      for (int i = 0; i < CH; ++i) {
        const int c = c0 + i * 64 + lane;
        if (c < nvec) {
          mep_u4 o;
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = mep_pack_bf16(acc[i][2 * j], acc[i][2 * j + 1]);
          mep_st16_stream(orow + (size_t)c * 16, o);
        }
      }
    }
    return;
  }

  // two-level: per destination-rank group (primary, then its duplicates in
  // ascending k) an fp32 sum rounded to bf16; then the sum of the groups.
  // members of the group led by entry k: later non-primary entries on the
  // same destination rank.
  uint64_t members = 0;  // lane k keeps the member mask of its own group
  {
    for (int k = 0; k < K; ++k) {
      const int dk = __builtin_amdgcn_readlane(drank, k);
      const uint64_t m = __ballot(valid && !primary && drank == dk && lane > k);
      if (lane == k) members = m;
    }
  }
  const uint32_t mem_lo = (uint32_t)members, mem_hi = (uint32_t)(members >> 32);
  for (int c = lane; c < nvec + lane; c += 64) {  // uniform trip count across the wave
    const bool in = c < nvec;
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
    uint64_t t = prim_mask;
    while (t) {
      const int k = __ffsll((unsigned long long)t) - 1;
      t &= t - 1;
      const uint64_t o = ((uint64_t)__builtin_amdgcn_readlane(off_hi, k) << 32) |
                         (uint32_t)__builtin_amdgcn_readlane(off_lo, k);
      uint64_t mem = ((uint64_t)__builtin_amdgcn_readlane(mem_hi, k) << 32) |
                     (uint32_t)__builtin_amdgcn_readlane(mem_lo, k);
      float grp[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) grp[j] = 0.0f;
      mep_u4 v = mep_u4{0u, 0u, 0u, 0u};
      if (in) v = mep_ld16_stream(base + o + (size_t)c * 16);
      acc8(grp, v);
      const bool rounded = mem != 0;
      while (mem) {
        const int j2 = __ffsll((unsigned long long)mem) - 1;
        mem &= mem - 1;
        const uint64_t o2 = ((uint64_t)__builtin_amdgcn_readlane(off_hi, j2) << 32) |
                            (uint32_t)__builtin_amdgcn_readlane(off_lo, j2);
        mep_u4 v2 = mep_u4{0u, 0u, 0u, 0u};
        if (in) v2 = mep_ld16_stream(base + o2 + (size_t)c * 16);
        acc8(grp, v2);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[j] += rounded ? mep_round_bf16(grp[j]) : grp[j];
    }
    if (in) {
      mep_u4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = mep_pack_bf16(acc[2 * j], acc[2 * j + 1]);
      mep_st16_stream(orow + (size_t)c * 16, o);
    }
  }
}

}  // namespace

extern "C" int mep_combine(const void* shards, int64_t shard_stride_rows, const float* wslots,
                           int64_t wslot_stride, const int32_t* dst, void* out_SH, float* out_SK,
                           int S, int H, int K, int R, int NvS, int mode, void* stream) {
  MEP_REQUIRE(shards && dst && out_SH, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(!out_SK || wslots, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(S > 0 && H > 0 && K > 0 && R > 0 && NvS > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(mode >= MEP_COMBINE_PRIMARIES && mode <= MEP_COMBINE_TWO_LEVEL, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(K <= 32, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(H % 8 == 0, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(shard_stride_rows >= NvS && (!out_SK || wslot_stride >= NvS), MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(((uintptr_t)shards % 16 == 0) && ((uintptr_t)out_SH % 16 == 0), MEP_ERR_ALIGNMENT);
  CombineArgs a;
  a.shards = (const uint16_t*)shards; a.wslots = wslots; a.dst = dst;
  a.out = (uint16_t*)out_SH; a.out_sk = out_SK;
  a.shard_stride_rows = shard_stride_rows; a.wslot_stride = wslot_stride;
  a.S = S; a.H = H; a.K = K; a.R = R; a.NvS = NvS; a.mode = mode;
  dim3 grid((S + kWavesPerBlock - 1) / kWavesPerBlock);
  hipLaunchKernelGGL(combine_kernel<2>, grid, dim3(kBlock), 0, (hipStream_t)stream, a);
  return mep_launch_status();
}
