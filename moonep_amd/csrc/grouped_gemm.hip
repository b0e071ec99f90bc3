// Expert-side consumer of the dispatched rows: grouped bf16 GEMM on the matrix
// cores of gfx950.  Rows [M,K] are split into G consecutive groups by the
// padded end offsets in cu_seqlens (device memory, as the planner wrote them);
// group g multiplies by its own weight matrix B[g] stored [N,K] (K
// contiguous), so C = A * B[g]^T needs no transposition on either operand.
//
// Workgroup: 512 threads, a 128 x 256 tile of (rows x weight rows), K in
// steps of 64 through double-buffered LDS; each of the 8 waves owns 64 x 64 of
// the tile as 2 x 2 MFMA 32x32x16 accumulators.  With token_padding a
// multiple of 128 a row tile never straddles two groups.  The wide weight
// tile is what the kernel's rate hangs on: it is bound by L2 -> LDS traffic
// (a 128 x 128 tile reached 0.7 PFLOP/s at 11 TB/s of tile loads).
// Two epilogues:
//   scale  : C[m,n] = bf16(row_scale[m] * acc)               (down projection)
//   swiglu : C[m,n] = bf16(silu(A*Bg^T) * (A*Bu^T))           (gate/up fused;
//            the tile holds 128 gate rows and the same 128 up rows)
// Tiles are handed out so that the workgroups running at one time on an XCD
// (one L2) work on the same 8 row tiles and neighbouring weight tiles.
#include "mep_common.h"

#include <atomic>

namespace {

typedef __bf16 mep_bf16x8 __attribute__((ext_vector_type(8)));
typedef float mep_f32x16 __attribute__((ext_vector_type(16)));

constexpr int kBM = 128, kBN = 256, kBK = 64;  // rows, weight rows, K per step of a tile
constexpr int kPitch = kBK * 2 + 16;  // bytes per LDS row: 8 lanes of a 16-byte read hit 32 distinct banks
constexpr int kATile = kBM * kPitch, kBTile = kBN * kPitch;
constexpr int kGemmThreads = 512;
constexpr int kPanel = 8;  // row tiles that share a sweep over the weight tiles

struct GemmArgs {
  const uint16_t* A;   // [M,K]
  const uint16_t* B;   // [G,N,K]
  const uint16_t* B2;  // [G,N,K] up weights (swiglu) or null
  const int* cu;       // [G] padded end row of each group
  uint16_t* C;         // [M,N]
  const float* scale;  // [M] or null
  int M, N, K, G, mtiles, ntiles;
};

__device__ __forceinline__ float mep_silu(float x) { return x / (1.0f + __expf(-x)); }

template <bool SWIGLU>
__global__ __launch_bounds__(kGemmThreads, 1) void grouped_gemm_nt_kernel(GemmArgs a) {
  extern __shared__ __attribute__((aligned(16))) char gsm[];
  __shared__ int s_group;
  char* As = gsm;                // [2][kBM][kPitch]
  char* Bs = gsm + 2 * kATile;   // [2][kBN][kPitch]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;  // 2 x 4 waves, 64 x 64 each

  // ---- which tile: XCD x (workgroups x, x+8, ...) walks a contiguous range of
  // tiles; inside a panel of kPanel row tiles the row tile index runs fastest
  const int total = a.mtiles * a.ntiles;
  const int per_xcd = (total + 7) >> 3;
  const int L = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (L >= total || (int)(blockIdx.x >> 3) >= per_xcd) return;
  const int panel = L / (kPanel * a.ntiles);
  const int within = L - panel * (kPanel * a.ntiles);
  const int ph = min(kPanel, a.mtiles - panel * kPanel);
  const int nt = within / ph;
  const int mt = panel * kPanel + (within - nt * ph);
  const int m0 = mt * kBM;
  constexpr int kCols = SWIGLU ? kBN / 2 : kBN;  // output columns per tile
  const int n0 = nt * kCols;

  // ---- group of this row tile: the first whose padded end lies beyond m0
  if (wave == 0) {
    int g = -1;
    for (int c = 0; c < a.G && g < 0; c += 64) {
      const int end = c + lane < a.G ? a.cu[c + lane] : 0;
      const uint64_t m = __ballot(c + lane < a.G && end > m0);
      if (m) g = c + __ffsll((unsigned long long)m) - 1;
    }
    if (lane == 0) s_group = g;
  }
  __syncthreads();
  const int g = s_group;
  if (g < 0) return;  // rows past the last group: nothing to compute

  // ---- global -> register -> LDS staging: 8 threads read the 128 bytes of one
  // row slice; a thread covers rows lrow + 64*i of the row tile (i < 2) and of
  // the weight tile (i < 4)
  const int lrow = tid >> 3, kv = tid & 7;
  const size_t K = (size_t)a.K;
  const uint16_t* Ag = a.A + (size_t)(m0 + lrow) * K + kv * 8;
  const uint16_t* Bg[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (SWIGLU) {  // weight tile = kBN/2 gate rows, then the same kBN/2 up rows
      const uint16_t* base = (i < 2 ? a.B : a.B2) + (size_t)g * a.N * K;
      Bg[i] = base + (size_t)(n0 + lrow + 64 * (i & 1)) * K + kv * 8;
    } else {
      Bg[i] = a.B + (size_t)g * a.N * K + (size_t)(n0 + lrow + 64 * i) * K + kv * 8;
    }
  }
  // two register sets: the loads of K step kt+2 are issued while step kt is
  // multiplied, and staged into LDS one step later, so a load has two steps
  // (and the other resident workgroup) to arrive
  mep_u4 ra[2][2], rb[2][4];
  auto load = [&](int set, int k0) {
#pragma unroll
    for (int i = 0; i < 2; ++i) ra[set][i] = *(const mep_u4*)(Ag + (size_t)i * 64 * K + k0);
#pragma unroll
    for (int i = 0; i < 4; ++i) rb[set][i] = *(const mep_u4*)(Bg[i] + k0);
  };
  auto stage = [&](int set, int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
      *(mep_u4*)(As + buf * kATile + (lrow + 64 * i) * kPitch + kv * 16) = ra[set][i];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      *(mep_u4*)(Bs + buf * kBTile + (lrow + 64 * i) * kPitch + kv * 16) = rb[set][i];
  };

  mep_f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // operand rows of this lane inside the LDS tiles
  const int arow = 64 * wm + (lane & 31);
  const int brow0 = SWIGLU ? 32 * wn + (lane & 31) : 64 * wn + (lane & 31);
  const int brow1 = SWIGLU ? kBN / 2 + 32 * wn + (lane & 31) : brow0 + 32;
  const int koff = (lane >> 5) * 16;

  const int KT = a.K / kBK;
  auto multiply = [&](int cur, int ks0, int ks1) {
    const char* Ab = As + cur * kATile;
    const char* Bb = Bs + cur * kBTile;
#pragma unroll
    for (int ks = ks0; ks < ks1; ++ks) {
      const mep_bf16x8 a0 = *(const mep_bf16x8*)(Ab + arow * kPitch + ks * 32 + koff);
      const mep_bf16x8 a1 = *(const mep_bf16x8*)(Ab + (arow + 32) * kPitch + ks * 32 + koff);
      const mep_bf16x8 b0 = *(const mep_bf16x8*)(Bb + brow0 * kPitch + ks * 32 + koff);
      const mep_bf16x8 b1 = *(const mep_bf16x8*)(Bb + brow1 * kPitch + ks * 32 + koff);
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc[1][1], 0, 0, 0);
    }
  };
  // Loads and stagings are unconditional (steps past the end re-read the last
  // slice): a load behind a branch would force the compiler to wait for every
  // outstanding load before staging, which empties the pipeline.
  const int klast = (KT - 1) * kBK;
  load(0, 0);
  load(1, min(kBK, klast));
  stage(0, 0);
  __syncthreads();
  int kt = 0;
  for (; kt + 1 < KT; kt += 2) {  // buffer 0 holds step kt, register set 1 step kt+1
    load(0, min((kt + 2) * kBK, klast));
    multiply(0, 0, 2);
    stage(1, 1);  // in the middle of the step: the LDS writes hide behind other waves' MFMAs
    multiply(0, 2, 4);
    __syncthreads();
    load(1, min((kt + 3) * kBK, klast));
    multiply(1, 0, 2);
    stage(0, 0);
    multiply(1, 2, 4);
    __syncthreads();
  }
  if (kt < KT) multiply(0, 0, 4);  // odd number of steps

  // ---- epilogue.  acc[i][j][v]: row 64*wm + 32*i + 8*(v/4) + 4*(lane/32) + v%4,
  // column (lane % 32) of the j-th 32-wide block
  const int ldc = a.N;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + 64 * wm + 32 * i + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
      if (SWIGLU) {
        const int n = n0 + 32 * wn + (lane & 31);
        const float r = mep_silu(acc[i][0][v]) * acc[i][1][v];
        a.C[(size_t)m * ldc + n] = (uint16_t)mep_f32_to_bf16_bits(r);
      } else {
        const float sc = a.scale ? a.scale[m] : 1.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int n = n0 + 64 * wn + 32 * j + (lane & 31);
          a.C[(size_t)m * ldc + n] = (uint16_t)mep_f32_to_bf16_bits(sc * acc[i][j][v]);
        }
      }
    }
}

}  // namespace

extern "C" int mep_grouped_gemm_nt(const void* A, const void* B, const void* B_up,
                                   const int32_t* cu_seqlens, int G, void* C,
                                   const float* row_scale, int M, int N, int K, int swiglu,
                                   void* stream) {
  MEP_REQUIRE(A && B && cu_seqlens && C, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(M > 0 && N > 0 && K > 0 && G > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(!swiglu || (B_up && !row_scale), MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(M % kBM == 0 && K % kBK == 0 && N % (swiglu ? kBN / 2 : kBN) == 0, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE((int64_t)M * (N > K ? N : K) < ((int64_t)1 << 40), MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)B % 16 == 0) && ((uintptr_t)B_up % 16 == 0) &&
                  ((uintptr_t)C % 2 == 0), MEP_ERR_ALIGNMENT);
  GemmArgs a;
  a.A = (const uint16_t*)A; a.B = (const uint16_t*)B; a.B2 = (const uint16_t*)B_up;
  a.cu = cu_seqlens; a.C = (uint16_t*)C; a.scale = row_scale;
  a.M = M; a.N = N; a.K = K; a.G = G;
  a.mtiles = M / kBM;
  a.ntiles = N / (swiglu ? kBN / 2 : kBN);
  const int64_t total = (int64_t)a.mtiles * a.ntiles;
  MEP_REQUIRE(total < (1 << 30), MEP_ERR_UNSUPPORTED);
  const int per_xcd = (int)((total + 7) / 8);
  const size_t lds = 2 * (size_t)(kATile + kBTile);
  hipStream_t st = (hipStream_t)stream;
  {  // 108 KB of dynamic LDS needs the opt-in, once per device
    static std::atomic<uint64_t> opted{0};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    const uint64_t bit = 1ull << (dev & 63);
    if (!(opted.load(std::memory_order_acquire) & bit)) {
      e = hipFuncSetAttribute((const void*)grouped_gemm_nt_kernel<true>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e == hipSuccess)
        e = hipFuncSetAttribute((const void*)grouped_gemm_nt_kernel<false>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (e != hipSuccess) return (int)e;
      opted.fetch_or(bit, std::memory_order_release);
    }
  }
  if (swiglu)
    hipLaunchKernelGGL(grouped_gemm_nt_kernel<true>, dim3(per_xcd * 8), dim3(kGemmThreads), lds, st, a);
  else
    hipLaunchKernelGGL(grouped_gemm_nt_kernel<false>, dim3(per_xcd * 8), dim3(kGemmThreads), lds, st, a);
  return mep_launch_status();
}
