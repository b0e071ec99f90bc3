// Expert-side consumer of the dispatched rows: grouped bf16 GEMM on the matrix
// cores of gfx950.  Rows [M,K] are split into G consecutive groups by the
// padded end offsets in cu_seqlens (device memory, as the planner wrote them);
// group g multiplies by its own weight matrix B[g] stored [N,K] (K
// contiguous), so C = A * B[g]^T needs no transposition on either operand.
//
// Workgroup: 640 threads on a 128 x 256 tile of (rows x weight rows), K in
// steps of 64: two producer waves stream the tile slices from global memory
// straight into a ring of three LDS stages, eight consumer waves own 64 x 64
// of the tile each as 2 x 2 MFMA 32x32x16 accumulators.  With token_padding a
// multiple of 128 a row tile never straddles two groups.  The kernel is bound
// by the L2 (its channels are ~75 % busy at 0.8 PFLOP/s), i.e. by tile bytes
// per flop.
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
constexpr int kRowBytes = kBK * 2;             // an LDS row is one 128-byte slice, no padding
constexpr int kATile = kBM * kRowBytes, kBTile = kBN * kRowBytes;
constexpr int kStage = kATile + kBTile;        // 48 KB
constexpr int kStages = 3;
constexpr int kConsumers = 8, kProducers = 2;  // waves
constexpr int kGemmThreads = (kConsumers + kProducers) * 64;
constexpr int kPanel = 8;  // row tiles that share a sweep over the weight tiles
// 1 KB pieces (8 rows x 128 bytes) of a stage that one producer wave moves per step
constexpr int kPiecesPerProducer = (kBM + kBN) / 8 / kProducers;  // 24
static_assert(2 * kPiecesPerProducer < 64, "two steps of loads must fit the 6-bit load counter");

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

// s_waitcnt vmcnt(n) alone (expcnt and lgkmcnt left at "do not wait")
template <int N>
__device__ __forceinline__ void mep_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// Producer / consumer waves.  Two producer waves stream the tiles from global
// memory straight into a ring of three LDS stages (global_load_lds, 16 bytes
// per lane: no registers, no LDS store instructions), always two K steps
// ahead; eight consumer waves only read LDS and feed the matrix cores.  One
// s_barrier per K step hands a filled stage to the consumers and a drained one
// back to the producers.  A stage row is the bare 128-byte slice; the 16-byte
// vector q of row r sits at position q ^ (r & 7), so the eight rows a group of
// eight lanes reads fall into distinct banks.
template <bool SWIGLU>
__global__ __launch_bounds__(kGemmThreads, 1) void grouped_gemm_nt_kernel(GemmArgs a) {
  extern __shared__ __attribute__((aligned(1024))) char gsm[];
  __shared__ int s_group;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // ---- which tile: XCD x (workgroups x, x+8, ...) walks a contiguous range of
  // tiles; inside a panel of kPanel row tiles the row tile index runs fastest
  const int total = a.mtiles * a.ntiles;
  const int per_xcd = (total + 7) >> 3;
  const int L = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (L >= total) return;
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

  const int KT = a.K / kBK;
  const size_t K = (size_t)a.K;

  if (wave >= kConsumers) {
    // =============================== producer ===============================
    const int p = wave - kConsumers;
    const int r = lane >> 3, kv = lane & 7;
    // piece j of a stage: rows 8j .. 8j+7 of the row tile (j < 16), then of the
    // weight tile; this wave moves the pieces j = p, p + kProducers, ...
    // lane (r, kv) fetches vector kv ^ r of its row into slot (r, kv)
    const uint16_t* Ap = a.A + (size_t)(m0 + r) * K + ((kv ^ r) * 8);
    const uint16_t* Bp0 = a.B + (size_t)g * a.N * K + (size_t)(n0 + r) * K + ((kv ^ r) * 8);
    const uint16_t* Bp1 = SWIGLU ? a.B2 + (size_t)g * a.N * K + (size_t)(n0 + r) * K + ((kv ^ r) * 8)
                                 : Bp0 + (size_t)(kBN / 2) * K;
    auto issue = [&](int k0, int stage) {
      char* base = gsm + stage * kStage;
#pragma unroll
      for (int q = 0; q < kPiecesPerProducer; ++q) {
        const int j = p + q * kProducers;  // 0 .. 47
        const uint16_t* src;
        if (j < kBM / 8) src = Ap + (size_t)(8 * j) * K + k0;
        else if (j < kBM / 8 + kBN / 16) src = Bp0 + (size_t)(8 * (j - kBM / 8)) * K + k0;
        else src = Bp1 + (size_t)(8 * (j - kBM / 8 - kBN / 16)) * K + k0;
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                         (__attribute__((address_space(3))) void*)(base + j * 1024),
                                         16, 0, 0);
      }
    };
    const int klast = (KT - 1) * kBK;
    issue(0, 0);
    issue(min(kBK, klast), 1);
    mep_wait_vmcnt<kPiecesPerProducer>();  // step 0 has landed
    __builtin_amdgcn_s_barrier();
    int st = 2;  // stage of step kt + 2
    for (int kt = 0; kt < KT; ++kt) {
      issue(min((kt + 2) * kBK, klast), st);
      st = st == kStages - 1 ? 0 : st + 1;
      mep_wait_vmcnt<kPiecesPerProducer>();  // everything up to step kt + 1 has landed
      __builtin_amdgcn_s_barrier();
    }
    mep_wait_vmcnt<0>();
    return;
  }

  // ================================ consumer =================================
  const int wm = wave & 1, wn = wave >> 1;  // 2 x 4 waves, 64 x 64 each
  mep_f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // operand rows of this lane inside a stage (weight rows follow the kBM rows)
  const int arow = 64 * wm + (lane & 31);
  const int brow0 = kBM + (SWIGLU ? 32 * wn + (lane & 31) : 64 * wn + (lane & 31));
  const int brow1 = SWIGLU ? brow0 + kBN / 2 : brow0 + 32;
  const int sw = lane & 7;      // (row & 7) of every operand row of this lane
  const int half = lane >> 5;   // which 8 of the 16 K values of an MFMA step
  const int oa0 = arow * kRowBytes, oa1 = (arow + 32) * kRowBytes;
  const int ob0 = brow0 * kRowBytes, ob1 = brow1 * kRowBytes;

  __builtin_amdgcn_s_barrier();  // stage 0 is filled
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  int st = 0;
  for (int kt = 0; kt < KT; ++kt) {
    const char* sb = gsm + st * kStage;
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      const int col = ((2 * ks + half) ^ sw) * 16;
      const mep_bf16x8 a0 = *(const mep_bf16x8*)(sb + oa0 + col);
      const mep_bf16x8 a1 = *(const mep_bf16x8*)(sb + oa1 + col);
      const mep_bf16x8 b0 = *(const mep_bf16x8*)(sb + ob0 + col);
      const mep_bf16x8 b1 = *(const mep_bf16x8*)(sb + ob1 + col);
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc[1][1], 0, 0, 0);
    }
    st = st == kStages - 1 ? 0 : st + 1;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // the reads of this stage are done
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  }

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
        const float res = mep_silu(acc[i][0][v]) * acc[i][1][v];
        a.C[(size_t)m * ldc + n] = (uint16_t)mep_f32_to_bf16_bits(res);
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
  const size_t lds = (size_t)kStages * kStage;
  hipStream_t st = (hipStream_t)stream;
  {  // 144 KB of dynamic LDS needs the opt-in, once per device
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
