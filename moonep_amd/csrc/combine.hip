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
  int S, H, K, R, NvS, mode, parts;
};

__device__ __forceinline__ void acc8(float* acc, mep_u4 v) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    acc[2 * i] += mep_bf16_lo(v[i]);
    acc[2 * i + 1] += mep_bf16_hi(v[i]);
  }
}

// A wave sums CH consecutive 1-KiB chunks (64 lanes x 16 bytes) of one token's
// rows; a token takes `parts` waves.  EXACT: the row is a whole number of such
// wave tiles, so no bounds checks.  All CH loads of a row are issued before
// they are consumed: with K rows that keeps CH x 1 KiB per wave in flight.
// TWO: the two-level mode (it carries a second accumulator set).
template <int CH, bool EXACT, bool TWO>
__global__ __launch_bounds__(kBlock) void combine_kernel(CombineArgs a) {
  const int lane = threadIdx.x & 63;
  const int gw = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
  const int s = gw / a.parts;
  const int part = gw - s * a.parts;
  if (s >= a.S) return;
  const int K = a.K;
  const size_t row_bytes = (size_t)a.H * 2;
  int dv = 0;
  if (lane < K) dv = a.dst[(size_t)s * K + lane];
  const int raw = dv < 0 ? -dv - 1 : dv;
  const int drank = raw / a.NvS;
  const int loff = raw - drank * a.NvS;
  const bool valid = lane < K && drank < a.R;
  float wk = 0.0f;  // route weight of entry `lane`, read from its slot
  if (a.wslots && valid) wk = a.wslots[(size_t)drank * a.wslot_stride + loff];
  if (a.out_sk && part == 0 && lane < K) a.out_sk[(size_t)s * K + lane] = wk;
  const uint64_t off = ((uint64_t)drank * (uint64_t)a.shard_stride_rows + (uint64_t)loff) * row_bytes;
  const uint32_t off_lo = (uint32_t)off, off_hi = (uint32_t)(off >> 32);
  const bool primary = valid && dv >= 0;
  const uint64_t prim_mask = __ballot(primary);
  const uint64_t valid_mask = __ballot(valid);
  const int nvec = a.H / 8;
  const int c0 = part * CH * 64 + lane;  // this lane's first 16-byte vector
  const char* base = (const char*)a.shards + (size_t)c0 * 16;
  char* orow = (char*)a.out + (size_t)s * row_bytes + (size_t)c0 * 16;

  float acc[CH][8];
#pragma unroll
  for (int i = 0; i < CH; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = 0.0f;

  auto row_of = [&](int k) -> const char* {
    const uint64_t o = ((uint64_t)__builtin_amdgcn_readlane(off_hi, k) << 32) |
                       (uint32_t)__builtin_amdgcn_readlane(off_lo, k);
    return base + o;
  };
  // chunks past the end of a ragged row re-read the row's first vector (their
  // sums are never stored): loads stay unconditional
  int voff[CH];
#pragma unroll
  for (int i = 0; i < CH; ++i) voff[i] = (EXACT || c0 + i * 64 < nvec) ? i * 1024 : -c0 * 16;
  auto load_row = [&](const char* row, mep_u4* v) {
#pragma unroll
    for (int i = 0; i < CH; ++i) v[i] = mep_ld16_stream(row + voff[i]);
  };

  if (!TWO) {
    uint64_t t = a.mode == MEP_COMBINE_PRIMARIES ? prim_mask : valid_mask;
    const bool weighted = a.mode == MEP_COMBINE_WEIGHTED;
    while (t) {
      const int k = __ffsll((unsigned long long)t) - 1;
      t &= t - 1;
      mep_u4 v[CH];
      load_row(row_of(k), v);
      if (weighted) {
        // acc += w * row with the product and the sum rounded separately
        // (no fused multiply-add), in ascending k
#pragma clang fp contract(off)
        const float w = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(wk), k));
#pragma unroll
        for (int i = 0; i < CH; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float p0 = w * mep_bf16_lo(v[i][j]);
            const float p1 = w * mep_bf16_hi(v[i][j]);
            acc[i][2 * j] = acc[i][2 * j] + p0;
            acc[i][2 * j + 1] = acc[i][2 * j + 1] + p1;
          }
      } else {
#pragma unroll
        for (int i = 0; i < CH; ++i) acc8(acc[i], v[i]);
      }
    }
  } else {
    // Per destination-rank group (its primary, then its duplicates in
    // ascending k) an fp32 sum rounded to bf16; then the sum of the groups in
    // the order of their primaries.  Lane k keeps the member mask of the
    // group it leads: later non-primary entries on the same rank.
    uint64_t members = 0;
    for (int k = 0; k < K; ++k) {
      const int dk = __builtin_amdgcn_readlane(drank, k);
      const uint64_t m = __ballot(valid && !primary && drank == dk && lane > k);
      if (lane == k) members = m;
    }
    const uint32_t mem_lo = (uint32_t)members, mem_hi = (uint32_t)(members >> 32);
    uint64_t t = prim_mask;
    while (t) {
      const int k = __ffsll((unsigned long long)t) - 1;
      t &= t - 1;
      uint64_t mem = ((uint64_t)__builtin_amdgcn_readlane(mem_hi, k) << 32) |
                     (uint32_t)__builtin_amdgcn_readlane(mem_lo, k);
      mep_u4 v[CH];
      load_row(row_of(k), v);
      if (mem == 0) {  // a group of one: bf16(row) is the row itself
#pragma unroll
        for (int i = 0; i < CH; ++i) acc8(acc[i], v[i]);
        continue;
      }
      float grp[CH][8];
#pragma unroll
      for (int i = 0; i < CH; ++i) {
#pragma unroll
        for (int j = 0; j < 8; ++j) grp[i][j] = 0.0f;
        acc8(grp[i], v[i]);
      }
      while (mem) {
        const int j2 = __ffsll((unsigned long long)mem) - 1;
        mem &= mem - 1;
        load_row(row_of(j2), v);
#pragma unroll
        for (int i = 0; i < CH; ++i) acc8(grp[i], v[i]);
      }
#pragma unroll
      for (int i = 0; i < CH; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] += mep_round_bf16(grp[i][j]);
    }
  }
#pragma unroll
  for (int i = 0; i < CH; ++i) {
    if (EXACT || c0 + i * 64 < nvec) {
      mep_u4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = mep_pack_bf16(acc[i][2 * j], acc[i][2 * j + 1]);
      // Store policy measured per mode at S=4096, H=7168 (same machine, runs
      // alternated): the one-wave-per-token modes gain 1.2-1.4 us of 87 with
      // stores written through at system scope, the two-level mode loses 4 us
      // of 88 with them (also with 7-chunk tiles) and keeps the nontemporal hint.
      if (TWO) mep_st16_stream(orow + (size_t)i * 1024, o);
      else mep_st16_through(orow + (size_t)i * 1024, o);
    }
  }
}

template <int CH, bool EXACT, bool TWO>
void launch_combine(const CombineArgs& a0, hipStream_t st) {
  CombineArgs a = a0;
  const int nvec = a.H / 8;
  a.parts = (nvec + CH * 64 - 1) / (CH * 64);
  const int64_t waves = (int64_t)a.S * a.parts;
  dim3 grid((unsigned)((waves + kWavesPerBlock - 1) / kWavesPerBlock));
  hipLaunchKernelGGL((combine_kernel<CH, EXACT, TWO>), grid, dim3(kBlock), 0, st, a);
}

}  // namespace

extern "C" int mep_combine(const void* shards, int64_t shard_stride_rows, const float* wslots,
                           int64_t wslot_stride, const int32_t* dst, void* out_SH, float* out_SK,
                           int S, int H, int K, int R, int NvS, int mode, void* stream) {
  MEP_REQUIRE(shards && dst && out_SH, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(!out_SK || wslots, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(S > 0 && H > 0 && K > 0 && R > 0 && NvS > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(mode >= MEP_COMBINE_PRIMARIES && mode <= MEP_COMBINE_WEIGHTED, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(mode != MEP_COMBINE_WEIGHTED || wslots, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(K <= 32, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE((int64_t)R * NvS <= INT32_MAX, MEP_ERR_UNSUPPORTED);  // raw = R*NvS marks an entry to skip
  MEP_REQUIRE(H % 8 == 0, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(shard_stride_rows >= NvS && (!wslots || wslot_stride >= NvS), MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(((uintptr_t)shards % 16 == 0) && ((uintptr_t)out_SH % 16 == 0), MEP_ERR_ALIGNMENT);
  CombineArgs a;
  a.shards = (const uint16_t*)shards; a.wslots = wslots; a.dst = dst;
  a.out = (uint16_t*)out_SH; a.out_sk = out_SK;
  a.shard_stride_rows = shard_stride_rows; a.wslot_stride = wslot_stride;
  a.S = S; a.H = H; a.K = K; a.R = R; a.NvS = NvS; a.mode = mode;
  a.parts = 1;
  hipStream_t st = (hipStream_t)stream;
  const int nvec = H / 8;
  if (mode == MEP_COMBINE_TWO_LEVEL) {
    // two accumulator sets: narrow tiles keep the register count low and more
    // waves resident (88.6 us with 2-chunk tiles vs 90.0 with 7 at H = 7168)
    if (nvec % (2 * 64) == 0) launch_combine<2, true, true>(a, st);
    else launch_combine<2, false, true>(a, st);
  } else {
    if (nvec % (14 * 64) == 0) launch_combine<14, true, false>(a, st);
    else if (nvec % (8 * 64) == 0) launch_combine<8, true, false>(a, st);
    else if (nvec % (4 * 64) == 0) launch_combine<4, true, false>(a, st);
    else launch_combine<2, false, false>(a, st);
  }
  return mep_launch_status();
}
