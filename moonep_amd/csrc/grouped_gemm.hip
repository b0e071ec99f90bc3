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
// Four kinds of launch share the main loop:
//   scale  : C[m,n] = bf16(row_scale[m] * acc)               (down projection)
//   swiglu : C[m,n] = bf16(silu(A*Bg^T) * (A*Bu^T))           (gate/up fused;
//            the tile holds 128 gate rows and the same 128 up rows; the two
//            pre-activations can be stored beside it for the backward pass)
//   dual   : C = bf16(A*B[g]^T + A2*B2[g]^T): the K loop runs over both pairs
//            (input gradient of the gate/up pair)
//   wgrad  : C[g] = At[:, rows of g] * Bt[:, rows of g]^T in fp32: the K range
//            of a tile is the row range of its group (weight gradients from
//            transposed activations)
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
constexpr int kPanel = 8;  // row tiles of a long group that share a sweep over the weight tiles
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
  const uint16_t* A2;  // dual: rows of the second K segment [M,K]
  uint16_t* Cg;        // swiglu: gate pre-activation [M,N] or null
  uint16_t* Cu;        // swiglu: up pre-activation [M,N] or null
  float* Cf;           // wgrad: [G,M,N] fp32
  int64_t ld;          // row stride of A and B in elements (K, or the row count for wgrad)
  int panel;           // row tiles of a long group that share a sweep over the weight tiles
  int skip_from;       // wgrad: groups g >= skip_from without rows are left unwritten
};

enum { kModeScale = 0, kModeSwiglu = 1, kModeDual = 2, kModeWgrad = 3 };

__device__ __forceinline__ float mep_silu(float x) { return x / (1.0f + __expf(-x)); }

// s_waitcnt vmcnt(n) alone (expcnt and lgkmcnt left at "do not wait")
template <int N>
__device__ __forceinline__ void mep_wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

typedef short mep_s16x4 __attribute__((ext_vector_type(4)));
typedef short mep_s16x8 __attribute__((ext_vector_type(8)));

// eight K values of one column from two transposing LDS reads (K rows k .. k+3 and k+4 .. k+7)
__device__ __forceinline__ mep_bf16x8 mep_tr_pair(const char* lo, const char* hi) {
  const mep_s16x4 x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) mep_s16x4*)lo);
  const mep_s16x4 y = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) mep_s16x4*)hi);
  const mep_s16x8 z = __builtin_shufflevector(x, y, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(mep_bf16x8, z);
}

// Producer / consumer waves.  Two producer waves stream the tiles from global
// memory straight into a ring of three LDS stages (global_load_lds, 16 bytes
// per lane: no registers, no LDS store instructions), always two K steps
// ahead; eight consumer waves only read LDS and feed the matrix cores.  One
// s_barrier per K step hands a filled stage to the consumers and a drained one
// back to the producers.  A stage row is the bare 128-byte slice; the 16-byte
// vector q of row r sits at position q ^ (r & 7) ^ ((r >> 3) & 1), so the
// sixteen rows that sixteen consecutive lanes read cover all 64 banks once (a
// 16-byte read runs at 256 bytes per clock then; with q ^ (r & 7) alone, which
// separates only eight rows, at half of that).
//
// BKN: the weights are given as [G, K, N] (the output column contiguous), as the
// backward pass finds them -- dX = dY * W with W stored for Y = X * W^T.  A K
// step of the weight tile is then 64 rows of 512 bytes in LDS, and a consumer
// lane gets its eight K values of one column from two transposing LDS reads
// (ds_read_b64_tr_b16: sixteen lanes read a 4 x 16 block, four rows of 32
// bytes, and each receives one column of it).  The 16-byte vector v of row k
// sits at position v ^ 2 (k & 3): the four rows of such a block then cover all
// banks once.
template <int MODE, bool BKN = false>
__global__ __launch_bounds__(kGemmThreads, 1) void grouped_gemm_nt_kernel(GemmArgs a) {
  constexpr bool SWIGLU = MODE == kModeSwiglu;
  static_assert(!BKN || MODE == kModeScale || MODE == kModeDual, "[K, N] weights: plain and dual products only");
  static_assert(kProducers == 2, "the lane offsets of the pieces assume that a producer wave's pieces share a parity");
  extern __shared__ __attribute__((aligned(1024))) char gsm[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // ---- which tile.  XCD x (workgroups x, x+8, ...) walks a contiguous eighth of
  // the tile list, in launch order, so the tiles that run on an XCD at one time
  // are neighbours in the list.  Only the row tiles below the last group's end
  // are listed (the row buffer is sized for the worst case; what lies beyond
  // would leave the last XCDs idle).
  //
  // Row-tiled products: the list goes group by group, inside a group weight tile
  // by weight tile, the group's row tiles running fastest.  The h row tiles of
  // a group then read a weight tile at the same time (it leaves HBM once), and
  // the 32 tiles an XCD runs cover 32 / h weight tiles of that group, so its
  // rows are fetched ntiles h / 32 times.  (Panels of eight row tiles whatever
  // the groups were, as before, split most groups over two panels: their
  // weights came from HBM twice.)
  const int mtiles = MODE == kModeWgrad ? a.mtiles : min(a.mtiles, (a.cu[a.G - 1] + kBM - 1) / kBM);
  const int per_group = mtiles * a.ntiles;
  const int total = MODE == kModeWgrad ? per_group * a.G : per_group;
  const int per_xcd = (total + 7) >> 3;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  if (idx >= per_xcd) return;
  int tg = 0, mt, nt;
  if (MODE == kModeWgrad) {
    if ((mtiles & 7) == 0) {
      // Weight gradient: every XCD takes an eighth of the row tiles of EVERY group,
      // group after group.  Groups differ in length (slots are often empty), so
      // whole groups per XCD would leave the arithmetic to a few of them; this
      // way all finish together and a group's output is written by all XCDs at once.
      const int mpx = mtiles >> 3;
      tg = idx / (mpx * a.ntiles);
      const int r = idx - tg * (mpx * a.ntiles);
      nt = r / mpx;
      mt = xcd * mpx + (r - nt * mpx);
    } else {
      const int L0 = xcd * per_xcd + idx;
      if (L0 >= total) return;
      tg = L0 / per_group;
      const int L = L0 - tg * per_group;
      nt = L / mtiles;
      mt = L - nt * mtiles;
    }
  } else {
    const int L0 = xcd * per_xcd + idx;
    if (L0 >= total) return;
    // the group whose tiles contain list entry L0: the first whose padded end, counted
    // in tiles, lies beyond it (every wave finds it for itself: 64 groups are one ballot)
    tg = -1;
    int beg_tiles = 0, end_tiles = 0;
    for (int c = 0; c < a.G && tg < 0; c += 64) {
      const int e = c + lane < a.G ? a.cu[c + lane] / kBM : 0;
      const uint64_t m = __ballot(c + lane < a.G && e * a.ntiles > L0);
      if (m) {
        const int src = __ffsll((unsigned long long)m) - 1;
        tg = c + src;
        end_tiles = __shfl(e, src);
        const int prev = __shfl(e, src > 0 ? src - 1 : 0);
        beg_tiles = src > 0 ? prev : (c > 0 ? a.cu[c - 1] / kBM : 0);
      }
    }
    if (tg < 0) return;  // cannot happen: L0 < total
    // a long group goes in panels of a.panel row tiles (its weights are then read once per
    // panel, its rows once per 32 / a.panel weight tiles)
    const int h = end_tiles - beg_tiles;
    const int local = L0 - beg_tiles * a.ntiles;
    const int panel = local / (a.panel * a.ntiles);
    const int within = local - panel * (a.panel * a.ntiles);
    const int ph = min(a.panel, h - panel * a.panel);
    nt = within / ph;
    mt = beg_tiles + panel * a.panel + (within - nt * ph);
  }
  const int m0 = mt * kBM;
  constexpr int kCols = SWIGLU ? kBN / 2 : kBN;  // output columns per tile
  const int n0 = nt * kCols;
  const int g = tg;

  // K steps of this tile and where its K range starts in a row
  int kbeg = 0, KT = a.K / kBK;
  if (MODE == kModeDual) KT *= 2;
  if (MODE == kModeWgrad) {
    kbeg = g > 0 ? a.cu[g - 1] : 0;
    KT = (a.cu[g] - kbeg) / kBK;
  }
  const size_t K = (size_t)a.ld;
  const bool any = KT > 0;  // a group without rows: its weight gradient is zero
  if (MODE == kModeWgrad && !any && g >= a.skip_from) return;  // ... and nobody reads it: an unused slot

  if (wave >= kConsumers) {
    // =============================== producer ===============================
    const int p = wave - kConsumers;
    const int r = lane >> 3, kv = lane & 7;
    // piece j of a stage: rows 8j .. 8j+7 of the row tile (j < 16), then of the
    // weight tile; this wave moves the pieces j = p, p + kProducers, ...
    // lane (r, kv) fetches vector kv ^ r ^ (piece & 1) of its row into slot (r, kv); this
    // wave's pieces all have the parity of p
    if (!any) return;
    const size_t goff = MODE == kModeWgrad ? (size_t)kbeg : (size_t)g * a.N * K;
    const size_t lane_off = (size_t)r * K + ((kv ^ r ^ (p & 1)) * 8);
    const uint16_t* Ap = a.A + (size_t)m0 * K + lane_off + (MODE == kModeWgrad ? (size_t)kbeg : 0);
    // [K, N] weights: piece jb holds the K rows 2 jb and 2 jb + 1 of the step; lane (lk, lv)
    // fetches vector lv ^ 2 (row & 3) of row 2 jb + lk, and (2 jb + lk) & 3 = 2 (p & 1) + lk
    // because this wave's pieces all have the parity of p
    const int lk = lane >> 5, lv = lane & 31;
    const size_t lane_off_kn = (size_t)lk * a.N + (size_t)((lv ^ ((2 * (p & 1) + lk) << 1)) * 8) + n0;
    const uint16_t* Bp0 = BKN ? a.B + goff + lane_off_kn : a.B + goff + (size_t)n0 * K + lane_off;
    const uint16_t* Bp1 = SWIGLU ? a.B2 + goff + (size_t)n0 * K + lane_off : Bp0 + (size_t)(kBN / 2) * K;
    // dual: the second half of the K loop reads the second pair
    const uint16_t* Aq = MODE == kModeDual ? a.A2 + (size_t)m0 * K + lane_off : Ap;
    const uint16_t* Bq0 = MODE != kModeDual ? Bp0
                          : BKN ? a.B2 + goff + lane_off_kn : a.B2 + goff + (size_t)n0 * K + lane_off;
    const uint16_t* Bq1 = Bq0 + (size_t)(kBN / 2) * K;
    auto issue = [&](int k0, int stage) {
      char* base = gsm + stage * kStage;
      const bool second = MODE == kModeDual && k0 >= a.K;
      if (second) k0 -= a.K;
      const uint16_t* pa = second ? Aq : Ap;
      const uint16_t* pb0 = second ? Bq0 : Bp0;
      const uint16_t* pb1 = second ? Bq1 : Bp1;
#pragma unroll
      for (int q = 0; q < kPiecesPerProducer; ++q) {
        const int j = p + q * kProducers;  // 0 .. 47
        const uint16_t* src;
        if (j < kBM / 8) src = pa + (size_t)(8 * j) * K + k0;
        else if (BKN) src = pb0 + (size_t)(k0 + 2 * (j - kBM / 8)) * a.N;
        else if (j < kBM / 8 + kBN / 16) src = pb0 + (size_t)(8 * (j - kBM / 8)) * K + k0;
        else src = pb1 + (size_t)(8 * (j - kBM / 8 - kBN / 16)) * K + k0;
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
  const int sw = (lane & 7) ^ ((lane >> 3) & 1);  // (row & 7) ^ ((row >> 3) & 1) of every operand row of this lane
  const int half = lane >> 5;   // which 8 of the 16 K values of an MFMA step
  const int oa0 = arow * kRowBytes, oa1 = (arow + 32) * kRowBytes;
  const int ob0 = brow0 * kRowBytes, ob1 = brow1 * kRowBytes;
  // [K, N] weights: lane s of a block of sixteen reads 8 bytes of row 8 half + s / 4 (+ 4 for
  // the second read, + 16 per MFMA step) at the columns 64 wn + 32 j + 16 (block & 1) + 4 (s & 3)
  const int ts = lane & 15, tb = (lane >> 4) & 1;
  const int okn0 = kATile + (8 * half + (ts >> 2)) * (kBN * 2) +
                   (((8 * wn + 2 * tb + ((ts & 3) >> 1)) ^ ((ts >> 2) << 1)) * 16) + (ts & 1) * 8;
  const int okn1 = kATile + (8 * half + (ts >> 2)) * (kBN * 2) +
                   (((8 * wn + 4 + 2 * tb + ((ts & 3) >> 1)) ^ ((ts >> 2) << 1)) * 16) + (ts & 1) * 8;

  if (any) {
    __builtin_amdgcn_s_barrier();  // stage 0 is filled
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  }
  int st = 0;
  for (int kt = 0; kt < KT; ++kt) {
    const char* sb = gsm + st * kStage;
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      const int col = ((2 * ks + half) ^ sw) * 16;
      const mep_bf16x8 a0 = *(const mep_bf16x8*)(sb + oa0 + col);
      const mep_bf16x8 a1 = *(const mep_bf16x8*)(sb + oa1 + col);
      mep_bf16x8 b0, b1;
      if (BKN) {
        const int step = ks * 16 * (kBN * 2);
        b0 = mep_tr_pair(sb + okn0 + step, sb + okn0 + step + 4 * (kBN * 2));
        b1 = mep_tr_pair(sb + okn1 + step, sb + okn1 + step + 4 * (kBN * 2));
      } else {
        b0 = *(const mep_bf16x8*)(sb + ob0 + col);
        b1 = *(const mep_bf16x8*)(sb + ob1 + col);
      }
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
  float* cf = MODE == kModeWgrad ? a.Cf + (size_t)g * a.M * a.N : nullptr;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + 64 * wm + 32 * i + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
      if (SWIGLU) {
        const int n = n0 + 32 * wn + (lane & 31);
        const float res = mep_silu(acc[i][0][v]) * acc[i][1][v];
        a.C[(size_t)m * ldc + n] = (uint16_t)mep_f32_to_bf16_bits(res);
        if (a.Cg) a.Cg[(size_t)m * ldc + n] = (uint16_t)mep_f32_to_bf16_bits(acc[i][0][v]);
        if (a.Cu) a.Cu[(size_t)m * ldc + n] = (uint16_t)mep_f32_to_bf16_bits(acc[i][1][v]);
      } else if (MODE == kModeWgrad) {
#pragma unroll
        for (int j = 0; j < 2; ++j)
          // streaming stores: 58 MB of output per group passing through L2 as ordinary
          // writes evicts the operand lines the other tiles of the group still need (9 % slower)
          __builtin_nontemporal_store(acc[i][j][v], &cf[(size_t)m * ldc + n0 + 64 * wn + 32 * j + (lane & 31)]);
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

// ---------------------------------------------------------------------------
// Row-tiled products on tiles of 256 (or 128) rows x 256 weight rows.  These
// kernels are bound by the lines they load, and a 256 x 256 tile needs a third
// fewer of them per flop than a 128 x 256 one.  Groups end on multiples of 128
// rows, so a group of h row blocks is covered by h / 2 tiles of 256 rows and,
// if h is odd, one of 128 (a 256-row tile padded to the next group would load
// and multiply as much again as it saves).  Eight waves of 128 x 64, all of
// them load: every wave moves eight of the 64 one-KB pieces of a K step
// straight into the other of two 64 KB LDS stages before it multiplies the
// current one; one barrier per step.  (K in steps of 32 through a ring of four
// 32 KB stages keeps the request stream going where two stages stop it at
// every step, but asks for every line twice, half by half, and was 12 %
// slower: what bounds the loads is the number of requests.)  A tile of 128
// rows loads no rows for the upper four waves' half and those waves only take
// part in the loads.
// Tile list as in the kernel above: group by group, weight tile by weight
// tile, the group's row tiles fastest; XCD x walks the x-th eighth.
// ---------------------------------------------------------------------------
constexpr int kT2Rows = 256;
constexpr int kT2Stage = (kT2Rows + kBN) * kRowBytes;  // 64 KB
constexpr int kT2Threads = 512;
constexpr int kT2Panel = 8;  // row tiles of a long group that share a sweep over the weight tiles (4: 2-3 % slower at 3-6 per group)
constexpr int kT2BOff = kT2Rows * kRowBytes;           // weight rows follow the 256 rows of the row tile

template <int MODE, bool BKN>
__global__ __launch_bounds__(kT2Threads, 1) void grouped_gemm256_kernel(GemmArgs a) {
  constexpr bool SWIGLU = MODE == kModeSwiglu;
  static_assert(MODE == kModeScale || MODE == kModeSwiglu || MODE == kModeDual, "row-tiled products only");
  static_assert(!BKN || !SWIGLU, "[K, N] weights: plain and dual products only");
  extern __shared__ __attribute__((aligned(1024))) char gsm[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  // ---- tile list: group g has (h + 1) / 2 row tiles, h = its 128-row blocks
  int total_rt = 0;
  for (int c = 0; c < a.G; c += 64) {
    const int gi = c + lane;
    const int end = gi < a.G ? a.cu[gi] : 0;
    const int beg = (gi > 0 && gi < a.G) ? a.cu[gi - 1] : 0;
    const int t = gi < a.G ? ((end - beg) / kBM + 1) >> 1 : 0;
    total_rt += __shfl(mep_wave_incl_scan(t), 63);
  }
  const int total = total_rt * a.ntiles;
  const int per_xcd = (total + 7) >> 3;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  if (idx >= per_xcd) return;
  const int L0 = xcd * per_xcd + idx;
  if (L0 >= total) return;
  int g = -1, m0 = 0, nt = 0;
  bool tall = true;
  {
    int carry = 0;
    for (int c = 0; c < a.G && g < 0; c += 64) {
      const int gi = c + lane;
      const int end = gi < a.G ? a.cu[gi] : 0;
      const int beg = (gi > 0 && gi < a.G) ? a.cu[gi - 1] : 0;
      const int t = gi < a.G ? ((end - beg) / kBM + 1) >> 1 : 0;
      const int incl = carry + mep_wave_incl_scan(t);
      const uint64_t m = __ballot(gi < a.G && incl * a.ntiles > L0);
      if (m) {
        const int src = __ffsll((unsigned long long)m) - 1;
        g = c + src;
        const int hs = __shfl(t, src), first = __shfl(incl - t, src);
        const int gbeg = __shfl(beg, src), gend = __shfl(end, src);
        const int local = L0 - first * a.ntiles;
        // a long group goes in panels of a.panel row tiles
        const int panel = local / (a.panel * a.ntiles);
        const int within = local - panel * (a.panel * a.ntiles);
        const int ph = min(a.panel, hs - panel * a.panel);
        nt = within / ph;
        m0 = gbeg + (panel * a.panel + (within - nt * ph)) * kT2Rows;
        tall = m0 + kT2Rows <= gend;
      }
      carry = __shfl(incl, 63);
    }
  }
  if (g < 0) return;  // cannot happen: L0 < total
  constexpr int kCols = SWIGLU ? kBN / 2 : kBN;  // output columns per tile
  const int n0 = nt * kCols;
  const int KT1 = a.K / kBK;
  const int KT = MODE == kModeDual ? 2 * KT1 : KT1;
  const size_t K = (size_t)a.ld;

  // ---- loads.  Piece j (0 .. 63) is rows 8j .. 8j+7 of the stage (the row tile, then the
  // weight tile); wave w moves the pieces 8w .. 8w+7, so the waves 0-3 load rows and the waves
  // 4-7 weights.  Lane (r, kv) fetches vector kv ^ r ^ (j & 1) of its row into slot (r, kv).
  // [K, N] weights: weight piece jb holds the K rows 2 jb and 2 jb + 1 of the step, lane
  // (lk, lv) fetches vector lv ^ 2 ((2 jb + lk) & 3) of its row.
  const bool loads_rows = wave < 4;
  const bool idle_loader = !tall && (wave == 2 || wave == 3);  // rows 128 .. 255 of a 128-row tile
  const uint16_t* src[8];
  size_t kstep;         // elements per K step
  ptrdiff_t delta = 0;  // distance to the second pair (dual), elements
  {
    const int r = lane >> 3, kv = lane & 7, lk = lane >> 5, lv = lane & 31;
    const size_t goff = (size_t)g * a.N * K;
    kstep = (BKN && !loads_rows) ? (size_t)kBK * a.N : (size_t)kBK;
    if (MODE == kModeDual) delta = loads_rows ? a.A2 - a.A : a.B2 - a.B;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int j = wave * 8 + q;
      if (loads_rows) {
        const int row = 8 * j + r;
        src[q] = a.A + (size_t)(m0 + (idle_loader ? 0 : row)) * K + ((kv ^ r ^ (q & 1)) * 8);
      } else if (BKN) {
        const int jb = j - 32;
        src[q] = a.B + goff + (size_t)(2 * jb + lk) * a.N + n0 + ((lv ^ ((2 * (q & 1) + lk) << 1)) * 8);
      } else {
        const int rb = 8 * (j - 32) + r;  // 0 .. 255
        const uint16_t* base = (SWIGLU && rb >= kBN / 2) ? a.B2 : a.B;
        const int nrow = SWIGLU ? n0 + (rb & (kBN / 2 - 1)) : n0 + rb;
        src[q] = base + goff + (size_t)nrow * K + ((kv ^ r ^ (q & 1)) * 8);
      }
    }
  }
  auto issue = [&](int kt, int stage) {
    if (idle_loader) return;
    ptrdiff_t off = (ptrdiff_t)((size_t)kt * kstep);
    if (MODE == kModeDual && kt >= KT1) off = (ptrdiff_t)((size_t)(kt - KT1) * kstep) + delta;
    char* base = gsm + stage * kT2Stage + wave * 8 * 1024;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src[q] + off),
                                       (__attribute__((address_space(3))) void*)(base + q * 1024), 16, 0, 0);
    }
  };

  // ---- consumers: 2 x 4 waves, 128 x 64 each
  const int wm = wave & 1, wn = wave >> 1;
  const bool works = tall || wm == 0;
  mep_f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
  const int l31 = lane & 31, half = lane >> 5;
  const int sw = (lane & 7) ^ ((lane >> 3) & 1);
  const int oa = (128 * wm + l31) * kRowBytes;
  const int ob0 = kT2BOff + (SWIGLU ? 32 * wn + l31 : 64 * wn + l31) * kRowBytes;
  const int ob1 = ob0 + (SWIGLU ? kBN / 2 : 32) * kRowBytes;
  const int ts = lane & 15, tb = (lane >> 4) & 1;
  const int okn0 = kT2BOff + (8 * half + (ts >> 2)) * (kBN * 2) +
                   (((8 * wn + 2 * tb + ((ts & 3) >> 1)) ^ ((ts >> 2) << 1)) * 16) + (ts & 1) * 8;
  const int okn1 = kT2BOff + (8 * half + (ts >> 2)) * (kBN * 2) +
                   (((8 * wn + 4 + 2 * tb + ((ts & 3) >> 1)) ^ ((ts >> 2) << 1)) * 16) + (ts & 1) * 8;

  issue(0, 0);
  mep_wait_vmcnt<0>();
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  for (int kt = 0; kt < KT; ++kt) {
    const int st = kt & 1;
    if (kt + 1 < KT) issue(kt + 1, st ^ 1);
    const char* sb = gsm + st * kT2Stage;
    if (works) {
#pragma unroll
      for (int ks = 0; ks < kBK / 16; ++ks) {
        const int col = ((2 * ks + half) ^ sw) * 16;
        mep_bf16x8 fa[4], fb[2];
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[i] = *(const mep_bf16x8*)(sb + oa + i * 32 * kRowBytes + col);
        if (BKN) {
          const int step = ks * 16 * (kBN * 2);
          fb[0] = mep_tr_pair(sb + okn0 + step, sb + okn0 + step + 4 * (kBN * 2));
          fb[1] = mep_tr_pair(sb + okn1 + step, sb + okn1 + step + 4 * (kBN * 2));
        } else {
          fb[0] = *(const mep_bf16x8*)(sb + ob0 + col);
          fb[1] = *(const mep_bf16x8*)(sb + ob1 + col);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
    }
    mep_wait_vmcnt<0>();  // the next stage has landed
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();  // ... for everyone, and everyone is done with this one
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  }
  if (!works) return;

  // ---- epilogue.  acc[i][j][v]: row 128 wm + 32 i + 8 (v / 4) + 4 (lane / 32) + v % 4,
  // column lane % 32 of the j-th 32-wide block
  const int ldc = a.N;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + 128 * wm + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
      if (SWIGLU) {
        const int n = n0 + 32 * wn + l31;
        const float res = mep_silu(acc[i][0][v]) * acc[i][1][v];
        a.C[(size_t)m * ldc + n] = (uint16_t)mep_f32_to_bf16_bits(res);
        if (a.Cg) a.Cg[(size_t)m * ldc + n] = (uint16_t)mep_f32_to_bf16_bits(acc[i][0][v]);
        if (a.Cu) a.Cu[(size_t)m * ldc + n] = (uint16_t)mep_f32_to_bf16_bits(acc[i][1][v]);
      } else {
        const float sc = (MODE == kModeScale && a.scale) ? a.scale[m] : 1.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int n = n0 + 64 * wn + 32 * j + l31;
          a.C[(size_t)m * ldc + n] = (uint16_t)mep_f32_to_bf16_bits(sc * acc[i][j][v]);
        }
      }
    }
}

// ---------------------------------------------------------------------------
// Weight gradient on 256 x 256 tiles.  The weight gradient is bound by the
// lines its tiles load (a K loop of only rows / 64 steps, both operands
// activations): a 256 x 256 tile needs a third fewer lines per flop than a
// 128 x 256 one, and both output dimensions are multiples of 256 for the
// shapes of an expert.  Eight waves of 128 x 64 (128 accumulator registers),
// all of them load: every wave moves eight of the 64 one-KB pieces of a K step
// straight into the other of two 64 KB LDS stages before it multiplies the
// current one; one barrier per step.
//
// Tile map: the dimension with more tiles is cut into eight slices, one per
// XCD (mirrored for odd groups, so that 28 tiles give every XCD 3 + 4), and
// every XCD takes its slice of every group, two neighbouring groups at a time
// (pairing every local expert with a slot instead, so that the zeroes of unused
// slots are written beside the products, was 8 % slower): all XCDs
// finish together whatever the groups' lengths, and the tiles an XCD runs at
// one time are one group's slice times the whole other dimension -- each line
// they load is wanted by 3 to 8 of them.
// ---------------------------------------------------------------------------
constexpr int kW2T = 256;                       // tile edge
constexpr int kW2Stage = 2 * kW2T * kRowBytes;  // 64 KB: 256 rows of each operand
constexpr int kW2Threads = 512;

struct Wgrad2Map {
  int sliced, other;  // tiles of the sliced and of the other dimension
  bool slice_m;       // the sliced dimension is the output row
  __host__ __device__ int lo(int x) const { return x * sliced / 8; }
  __host__ __device__ int size(int x) const { return (x + 1) * sliced / 8 - x * sliced / 8; }
  __host__ __device__ int pair_count(int x) const { return (size(x) + size(7 - x)) * other; }
};

// TN: the operands are given as the forward and backward passes hold them, X1 [rows, Ma] and
// X2 [rows, Nb] (a K step is then 64 rows of 512 bytes of each in LDS, read with the transposing
// LDS loads of the [K, N] weight form above); otherwise as transposed copies [Ma, rows], [Nb, rows].
template <bool TN>
__global__ __launch_bounds__(kW2Threads, 1) void wgrad256_kernel(GemmArgs a, Wgrad2Map map) {
  extern __shared__ __attribute__((aligned(1024))) char gsm[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int per_pair = map.pair_count(xcd);
  if (per_pair == 0 || idx >= per_pair * (a.G >> 1)) return;
  const int pair = idx / per_pair;
  int local = idx - pair * per_pair;
  const int n_even = map.size(xcd) * map.other;
  int g = 2 * pair, xe = xcd;
  if (local >= n_even) { local -= n_even; g += 1; xe = 7 - xcd; }
  const int sz = map.size(xe);
  const int u = local / sz, sl = map.lo(xe) + (local - u * sz);
  const int m0 = (map.slice_m ? sl : u) * kW2T, n0 = (map.slice_m ? u : sl) * kW2T;
  const int kbeg = g > 0 ? a.cu[g - 1] : 0;
  const int KT = (a.cu[g] - kbeg) / kBK;
  const size_t ld = (size_t)a.ld;

  // ---- loads: piece j (0 .. 63) is rows 8j .. 8j+7 of the stage (output rows, then output
  // columns); wave w moves the pieces 8w .. 8w+7; lane (r, kv) fetches vector
  // kv ^ r ^ (j & 1) of its row into slot (r, kv).  TN: piece jp of an operand's half of the
  // stage is the K rows 2 jp and 2 jp + 1 of the step (256 columns = 512 bytes each); lane
  // (lk, lv) fetches vector lv ^ 2 ((2 jp + lk) & 3) of its row.
  const int r = lane >> 3, kv = lane & 7;
  const uint16_t* src[8];
  size_t kstep;  // elements per K step
  if (TN) {
    const int lk = lane >> 5, lv = lane & 31;
    const bool first = wave < 4;  // the waves 0-3 load X1, the waves 4-7 X2
    const size_t pitch = first ? (size_t)a.M : (size_t)a.N;
    const uint16_t* base = (first ? a.A + m0 : a.B + n0) + (size_t)kbeg * pitch;
    kstep = (size_t)kBK * pitch;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int jp = (wave & 3) * 8 + q;
      src[q] = base + (size_t)(2 * jp + lk) * pitch + ((lv ^ ((2 * (q & 1) + lk) << 1)) * 8);
    }
  } else {
    kstep = kBK;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int j = wave * 8 + q;
      const int row = 8 * j + r;  // 0 .. 511
      const uint16_t* base = row < kW2T ? a.A + (size_t)(m0 + row) * ld : a.B + (size_t)(n0 + row - kW2T) * ld;
      src[q] = base + kbeg + ((kv ^ r ^ (q & 1)) * 8);
    }
  }
  auto issue = [&](int kt, int stage) {
    char* base = gsm + stage * kW2Stage + wave * 8 * 1024;
#pragma unroll
    for (int q = 0; q < 8; ++q)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src[q] + (size_t)kt * kstep),
                                       (__attribute__((address_space(3))) void*)(base + q * 1024), 16, 0, 0);
  };

  float* cf = a.Cf + (size_t)g * a.M * a.N;
  if (KT == 0 && g >= a.skip_from) return;  // an unused slot whose gradient nobody reads
  if (KT == 0) {
    // a group without rows: its gradient is zero -- whole 1 KB rows of the
    // tile per wave instruction instead of the accumulators' two 128-byte pieces
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int row = wave; row < kW2T; row += kW2Threads / 64)
      __builtin_nontemporal_store(zero, (f32x4*)(cf + (size_t)(m0 + row) * a.N + n0) + lane);
    return;
  }
  const int wm = wave & 1, wn = wave >> 1;  // 2 x 4 waves, 128 x 64 each
  mep_f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
  const int l31 = lane & 31, half = lane >> 5;
  const int sw = (lane & 7) ^ ((lane >> 3) & 1);
  const int oa = (128 * wm + l31) * kRowBytes, ob = (kW2T + 64 * wn + l31) * kRowBytes;
  // TN: lane s of a block of sixteen reads 8 bytes of K row 8 half + s / 4 (+ 4 for the second
  // read, + 16 per MFMA step) at the columns c + 16 (block & 1) + 4 (s & 3) of a 32-column block
  // that starts at column c of its operand's half of the stage
  const int ts = lane & 15, tb = (lane >> 4) & 1;
  const int otn = (8 * half + (ts >> 2)) * (kW2T * 2) + (ts & 1) * 8;
  const int vtn = 2 * tb + ((ts & 3) >> 1), xtn = (ts >> 2) << 1;

  issue(0, 0);
  mep_wait_vmcnt<0>();
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  for (int kt = 0; kt < KT; ++kt) {
    const int st = kt & 1;
    if (kt + 1 < KT) issue(kt + 1, st ^ 1);
    const char* sb = gsm + st * kW2Stage;
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      const int col = ((2 * ks + half) ^ sw) * 16;
      mep_bf16x8 fa[4], fb[2];
      if (TN) {
        // block i (32 columns = 4 vectors) moves the vector index by 4 i; the XOR with xtn
        // (0, 2, 4 or 6) touches the bits 1 and 2 only, so 4 i is added before it
        const int step = ks * 16 * (kW2T * 2);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int o = otn + step + (((16 * wm + 4 * i + vtn) ^ xtn) * 16);
          fa[i] = mep_tr_pair(sb + o, sb + o + 4 * (kW2T * 2));
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int o = kW2T * kRowBytes + otn + step + (((8 * wn + 4 * j + vtn) ^ xtn) * 16);
          fb[j] = mep_tr_pair(sb + o, sb + o + 4 * (kW2T * 2));
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[i] = *(const mep_bf16x8*)(sb + oa + i * 32 * kRowBytes + col);
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[j] = *(const mep_bf16x8*)(sb + ob + j * 32 * kRowBytes + col);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    mep_wait_vmcnt<0>();  // the next stage has landed
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_barrier();  // ... for everyone, and everyone is done with this one
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  }

  // ---- epilogue: acc[i][j][v] is row 128 wm + 32 i + 8 (v / 4) + 4 (lane / 32) + v % 4,
  // column 64 wn + 32 j + lane % 32; streaming stores (see the 128 x 256 kernel)
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + 128 * wm + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        __builtin_nontemporal_store(acc[i][j][v], &cf[(size_t)m * a.N + n0 + 64 * wn + 32 * j + l31]);
    }
}


// ---------------------------------------------------------------------------
// [batch, rows, cols] -> [batch, cols, rows] of 2-byte elements through a
// 64 x 64 LDS tile (rows and cols multiples of 64): 128-byte reads and writes.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void transpose16_kernel(const uint16_t* __restrict__ src,
                                                          uint16_t* __restrict__ dst, int rows, int cols) {
  __shared__ uint16_t tile[64][66];
  const size_t plane = (size_t)rows * cols;
  const uint16_t* s = src + (size_t)blockIdx.z * plane;
  uint16_t* d = dst + (size_t)blockIdx.z * plane;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8 threads, two columns each
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = ty + 8 * i;
    const uint32_t v = *(const uint32_t*)(s + (size_t)(r0 + r) * cols + c0 + 2 * tx);
    tile[r][2 * tx] = (uint16_t)v;
    tile[r][2 * tx + 1] = (uint16_t)(v >> 16);
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int c = ty + 8 * i;  // column of the source = row of the destination
    const uint32_t v = (uint32_t)tile[2 * tx][c] | ((uint32_t)tile[2 * tx + 1][c] << 16);
    *(uint32_t*)(d + (size_t)(c0 + c) * rows + r0 + 2 * tx) = v;
  }
}

// ---------------------------------------------------------------------------
// Backward of h = s * silu(g) * u per element, from the gradient dh' of the
// unscaled activation (dh' = dy * Wdown):
//   dgate = s*dh' * u * silu'(g),  dup = s*dh' * silu(g),  hs = s * silu(g) * u,
//   dscale[m] = sum_n dh'[m,n] * silu(g)*u
// One wave per row; rows at or beyond cu_seqlens[G-1] come out as zeros.
// ---------------------------------------------------------------------------
struct SwigluBwdArgs {
  const uint16_t* dh; const uint16_t* gate; const uint16_t* up; const float* scale; const int* cu;
  uint16_t* dgate; uint16_t* dup; uint16_t* hs; float* dscale;
  int M, N, G;
};

__global__ __launch_bounds__(256) void swiglu_bwd_kernel(SwigluBwdArgs a) {
  const int lane = threadIdx.x & 63;
  const int m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= a.M) return;
  const bool live = m < a.cu[a.G - 1];
  const float s = a.scale ? a.scale[m] : 1.0f;
  const size_t row = (size_t)m * a.N;
  float dot = 0.0f;
  for (int n = lane * 8; n < a.N; n += 512) {
    uint4 od = make_uint4(0, 0, 0, 0), og = od, oh = od;
    if (live) {
      const uint4 vd = *(const uint4*)(a.dh + row + n);
      const uint4 vg = *(const uint4*)(a.gate + row + n);
      const uint4 vu = *(const uint4*)(a.up + row + n);
      const uint32_t wd[4] = {vd.x, vd.y, vd.z, vd.w}, wg[4] = {vg.x, vg.y, vg.z, vg.w},
                     wu[4] = {vu.x, vu.y, vu.z, vu.w};
      uint32_t rg[4], ru[4], rh[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        float fg[2], fu[2], fh[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          const float d = e ? mep_bf16_hi(wd[q]) : mep_bf16_lo(wd[q]);
          const float g = e ? mep_bf16_hi(wg[q]) : mep_bf16_lo(wg[q]);
          const float u = e ? mep_bf16_hi(wu[q]) : mep_bf16_lo(wu[q]);
          const float sig = 1.0f / (1.0f + __expf(-g));
          const float act = g * sig;               // silu(g)
          dot += d * act * u;
          const float dhs = s * d;                 // gradient of the scaled activation
          fg[e] = dhs * u * (sig + act * (1.0f - sig));
          fu[e] = dhs * act;
          fh[e] = s * act * u;
        }
        rg[q] = mep_pack_bf16(fg[0], fg[1]);
        ru[q] = mep_pack_bf16(fu[0], fu[1]);
        rh[q] = mep_pack_bf16(fh[0], fh[1]);
      }
      od = make_uint4(rg[0], rg[1], rg[2], rg[3]);
      og = make_uint4(ru[0], ru[1], ru[2], ru[3]);
      oh = make_uint4(rh[0], rh[1], rh[2], rh[3]);
    }
    *(uint4*)(a.dgate + row + n) = od;
    *(uint4*)(a.dup + row + n) = og;
    *(uint4*)(a.hs + row + n) = oh;
  }
  if (a.dscale) {
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) dot += __shfl_xor(dot, d);
    if (lane == 0) a.dscale[m] = dot;
  }
}

// launch of the 256-row-tile kernel: the grid covers the most row tiles the groups can need
// ((M / 128 + G) / 2, when every group has an odd number of 128-row blocks)
template <int MODE, bool BKN>
int gemm256_launch(const GemmArgs& a0, hipStream_t st) {
  GemmArgs a = a0;
  a.panel = kT2Panel;
  const int64_t row_tiles = ((int64_t)a.M / kBM + a.G + 1) / 2;
  const int64_t total = row_tiles * a.ntiles;
  MEP_REQUIRE(total > 0 && total < (1 << 30), MEP_ERR_UNSUPPORTED);
  const int per_xcd = (int)((total + 7) / 8);
  const size_t lds = 2 * (size_t)kT2Stage;
  const int irc = mep_ensure_init();  // the LDS opt-in of this kernel, once per device
  if (irc != MEP_OK) return irc;
  hipLaunchKernelGGL((grouped_gemm256_kernel<MODE, BKN>), dim3(per_xcd * 8), dim3(kT2Threads), lds, st, a);
  return mep_launch_status();
}

// 144 KB of dynamic LDS: opted in by mep_init_gemm_kernels
template <int MODE, bool BKN = false>
int gemm_launch(const GemmArgs& a0, int64_t total, hipStream_t st) {
  GemmArgs a = a0;
  a.panel = kPanel;
  MEP_REQUIRE(total > 0 && total < (1 << 30), MEP_ERR_UNSUPPORTED);
  const int per_xcd = (int)((total + 7) / 8);
  const size_t lds = (size_t)kStages * kStage;
  const int irc = mep_ensure_init();
  if (irc != MEP_OK) return irc;
  hipLaunchKernelGGL((grouped_gemm_nt_kernel<MODE, BKN>), dim3(per_xcd * 8), dim3(kGemmThreads), lds, st, a);
  return mep_launch_status();
}

// launch of the 256 x 256 weight gradient (a.M, a.N multiples of 256, a.G even)
template <bool TN>
int wgrad256_launch(const GemmArgs& a, hipStream_t st) {
  Wgrad2Map map;
  const int mt = a.M / kW2T, nt = a.N / kW2T;
  map.slice_m = mt >= nt;
  map.sliced = map.slice_m ? mt : nt;
  map.other = map.slice_m ? nt : mt;
  int per_pair = 0;
  for (int x = 0; x < 8; ++x) per_pair = per_pair > map.pair_count(x) ? per_pair : map.pair_count(x);
  const int64_t per_xcd = (int64_t)per_pair * (a.G / 2);
  MEP_REQUIRE(per_xcd > 0 && per_xcd < (1 << 27), MEP_ERR_UNSUPPORTED);
  const size_t lds = 2 * (size_t)kW2Stage;
  const int irc = mep_ensure_init();
  if (irc != MEP_OK) return irc;
  hipLaunchKernelGGL(wgrad256_kernel<TN>, dim3((unsigned)(per_xcd * 8)), dim3(kW2Threads), lds, st, a, map);
  return mep_launch_status();
}

int check_nt_shapes(const void* A, const void* B, const int32_t* cu, const void* C, int M, int N, int K,
                    int G, int cols_per_tile) {
  MEP_REQUIRE(A && B && cu && C, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(M > 0 && N > 0 && K > 0 && G > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(M % kBM == 0 && K % kBK == 0 && N % cols_per_tile == 0, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE((int64_t)M * (N > K ? N : K) < ((int64_t)1 << 40), MEP_ERR_UNSUPPORTED);
  return MEP_OK;
}

GemmArgs nt_args(const void* A, const void* B, const void* B2, const int32_t* cu, void* C, const float* scale,
                 int M, int N, int K, int G, int cols_per_tile) {
  GemmArgs a{};
  a.A = (const uint16_t*)A; a.B = (const uint16_t*)B; a.B2 = (const uint16_t*)B2;
  a.cu = cu; a.C = (uint16_t*)C; a.scale = scale;
  a.M = M; a.N = N; a.K = K; a.G = G;
  a.mtiles = M / kBM;
  a.ntiles = N / cols_per_tile;
  a.ld = K;
  return a;
}

// Which row tiling: 256-row tiles load a third fewer lines per flop, but with two 64 KB
// stages their loads drain at every K step, and there are half as many tiles to spread over
// the CUs.  Measured at 34 688 rows, H = 7168, H' = 2048: 5-8 % faster where a launch has at
// least eight of them per CU (SwiGLU, down, the dual input gradient), 12 % slower at five
// (dy * down, 2048 output columns).
// mep_set_gemm_row_tile(128 or 256) forces one (tests run both on small shapes).
std::atomic<int> g_forced_row_tile{0};

static bool use_256_row_tiles(const GemmArgs& a) {
  const int forced = g_forced_row_tile.load(std::memory_order_relaxed);
  if (forced) return forced == 256;
  const int cus = mep_device_cu_count();
  return (int64_t)(a.M / kT2Rows) * a.ntiles >= 8 * (int64_t)(cus > 0 ? cus : 256);
}

int gemm_nt_forward(const void* A, const void* B, const void* B_up, const int32_t* cu, int G, void* C,
                    void* C_gate, void* C_up, const float* row_scale, int M, int N, int K, int swiglu,
                    void* stream) {
  const int cols = swiglu ? kBN / 2 : kBN;
  const int rc = check_nt_shapes(A, B, cu, C, M, N, K, G, cols);
  if (rc != MEP_OK) return rc;
  MEP_REQUIRE(!swiglu || (B_up && !row_scale), MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(swiglu || (!C_gate && !C_up), MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)B % 16 == 0) && ((uintptr_t)B_up % 16 == 0) &&
                  ((uintptr_t)C % 2 == 0) && ((uintptr_t)C_gate % 2 == 0) && ((uintptr_t)C_up % 2 == 0),
              MEP_ERR_ALIGNMENT);
  GemmArgs a = nt_args(A, B, B_up, cu, C, row_scale, M, N, K, G, cols);
  a.Cg = (uint16_t*)C_gate;
  a.Cu = (uint16_t*)C_up;
  const int64_t total = (int64_t)a.mtiles * a.ntiles;
  if (use_256_row_tiles(a))
    return swiglu ? gemm256_launch<kModeSwiglu, false>(a, (hipStream_t)stream)
                  : gemm256_launch<kModeScale, false>(a, (hipStream_t)stream);
  return swiglu ? gemm_launch<kModeSwiglu>(a, total, (hipStream_t)stream)
                : gemm_launch<kModeScale>(a, total, (hipStream_t)stream);
}

template <class Kern>
int opt_in_lds(Kern kern, size_t bytes) {
  MEP_RETURN_IF_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                        (int)bytes));
  return MEP_OK;
}

}  // namespace

// Every GEMM kernel uses more dynamic LDS than a kernel gets without asking: the opt-ins
// for the current device, made once from mep_init (never from a launch, which may be
// under stream capture).
int mep_init_gemm_kernels() {
  const size_t ring = (size_t)kStages * kStage, two = 2 * (size_t)kT2Stage, w2 = 2 * (size_t)kW2Stage;
  int rc = MEP_OK;
#define MEP_OPT(k, b) if (rc == MEP_OK) rc = opt_in_lds(k, b)
  MEP_OPT((grouped_gemm_nt_kernel<kModeScale, false>), ring);
  MEP_OPT((grouped_gemm_nt_kernel<kModeSwiglu, false>), ring);
  MEP_OPT((grouped_gemm_nt_kernel<kModeDual, false>), ring);
  MEP_OPT((grouped_gemm_nt_kernel<kModeWgrad, false>), ring);
  MEP_OPT((grouped_gemm_nt_kernel<kModeScale, true>), ring);
  MEP_OPT((grouped_gemm_nt_kernel<kModeDual, true>), ring);
  MEP_OPT((grouped_gemm256_kernel<kModeScale, false>), two);
  MEP_OPT((grouped_gemm256_kernel<kModeSwiglu, false>), two);
  MEP_OPT((grouped_gemm256_kernel<kModeDual, false>), two);
  MEP_OPT((grouped_gemm256_kernel<kModeScale, true>), two);
  MEP_OPT((grouped_gemm256_kernel<kModeDual, true>), two);
  MEP_OPT(wgrad256_kernel<false>, w2);
  MEP_OPT(wgrad256_kernel<true>, w2);
#undef MEP_OPT
  return rc;
}

extern "C" int mep_set_gemm_row_tile(int rows) {
  MEP_REQUIRE(rows == 0 || rows == 128 || rows == 256, MEP_ERR_INVALID_ARG);
  g_forced_row_tile.store(rows, std::memory_order_relaxed);
  return MEP_OK;
}

extern "C" int mep_grouped_gemm_nt(const void* A, const void* B, const void* B_up,
                                   const int32_t* cu_seqlens, int G, void* C,
                                   const float* row_scale, int M, int N, int K, int swiglu,
                                   void* stream) {
  return gemm_nt_forward(A, B, B_up, cu_seqlens, G, C, nullptr, nullptr, row_scale, M, N, K, swiglu, stream);
}

extern "C" int mep_grouped_swiglu_nt(const void* A, const void* B_gate, const void* B_up,
                                     const int32_t* cu_seqlens, int G, void* C_act, void* C_gate,
                                     void* C_up, int M, int N, int K, void* stream) {
  return gemm_nt_forward(A, B_gate, B_up, cu_seqlens, G, C_act, C_gate, C_up, nullptr, M, N, K, 1, stream);
}

extern "C" int mep_grouped_gemm_dual_nt(const void* A1, const void* B1, const void* A2, const void* B2,
                                        const int32_t* cu_seqlens, int G, void* C, int M, int N, int K,
                                        void* stream) {
  const int rc = check_nt_shapes(A1, B1, cu_seqlens, C, M, N, K, G, kBN);
  if (rc != MEP_OK) return rc;
  MEP_REQUIRE(A2 && B2, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(2 * (int64_t)K < ((int64_t)1 << 30), MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(((uintptr_t)A1 % 16 == 0) && ((uintptr_t)B1 % 16 == 0) && ((uintptr_t)A2 % 16 == 0) &&
                  ((uintptr_t)B2 % 16 == 0) && ((uintptr_t)C % 2 == 0), MEP_ERR_ALIGNMENT);
  GemmArgs a = nt_args(A1, B1, B2, cu_seqlens, C, nullptr, M, N, K, G, kBN);
  a.A2 = (const uint16_t*)A2;
  if (use_256_row_tiles(a)) return gemm256_launch<kModeDual, false>(a, (hipStream_t)stream);
  return gemm_launch<kModeDual>(a, (int64_t)a.mtiles * a.ntiles, (hipStream_t)stream);
}

extern "C" int mep_grouped_gemm_nn(const void* A, const void* B, const int32_t* cu_seqlens, int G, void* C,
                                   const float* row_scale, int M, int N, int K, void* stream) {
  const int rc = check_nt_shapes(A, B, cu_seqlens, C, M, N, K, G, kBN);
  if (rc != MEP_OK) return rc;
  MEP_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)B % 16 == 0) && ((uintptr_t)C % 2 == 0), MEP_ERR_ALIGNMENT);
  GemmArgs a = nt_args(A, B, nullptr, cu_seqlens, C, row_scale, M, N, K, G, kBN);
  if (use_256_row_tiles(a)) return gemm256_launch<kModeScale, true>(a, (hipStream_t)stream);
  return gemm_launch<kModeScale, true>(a, (int64_t)a.mtiles * a.ntiles, (hipStream_t)stream);
}

extern "C" int mep_grouped_gemm_dual_nn(const void* A1, const void* B1, const void* A2, const void* B2,
                                        const int32_t* cu_seqlens, int G, void* C, int M, int N, int K,
                                        void* stream) {
  const int rc = check_nt_shapes(A1, B1, cu_seqlens, C, M, N, K, G, kBN);
  if (rc != MEP_OK) return rc;
  MEP_REQUIRE(A2 && B2, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(2 * (int64_t)K < ((int64_t)1 << 30), MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(((uintptr_t)A1 % 16 == 0) && ((uintptr_t)B1 % 16 == 0) && ((uintptr_t)A2 % 16 == 0) &&
                  ((uintptr_t)B2 % 16 == 0) && ((uintptr_t)C % 2 == 0), MEP_ERR_ALIGNMENT);
  GemmArgs a = nt_args(A1, B1, B2, cu_seqlens, C, nullptr, M, N, K, G, kBN);
  a.A2 = (const uint16_t*)A2;
  if (use_256_row_tiles(a)) return gemm256_launch<kModeDual, true>(a, (hipStream_t)stream);
  return gemm_launch<kModeDual, true>(a, (int64_t)a.mtiles * a.ntiles, (hipStream_t)stream);
}

extern "C" int mep_grouped_gemm_wgrad(const void* At, const void* Bt, const int32_t* cu_seqlens, int G,
                                      float* C, int Ma, int Nb, int64_t ld, int skip_empty_from, void* stream) {
  MEP_REQUIRE(At && Bt && cu_seqlens && C, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(Ma > 0 && Nb > 0 && G > 0 && ld > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(Ma % kBM == 0 && Nb % kBN == 0 && ld % kBM == 0, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE((int64_t)(Ma > Nb ? Ma : Nb) * ld < ((int64_t)1 << 40), MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(((uintptr_t)At % 16 == 0) && ((uintptr_t)Bt % 16 == 0) && ((uintptr_t)C % 4 == 0),
              MEP_ERR_ALIGNMENT);
  GemmArgs a{};
  a.A = (const uint16_t*)At; a.B = (const uint16_t*)Bt; a.cu = cu_seqlens; a.Cf = C;
  a.M = Ma; a.N = Nb; a.K = 0; a.G = G;
  a.ld = ld;
  MEP_REQUIRE(skip_empty_from >= 0, MEP_ERR_INVALID_ARG);
  a.skip_from = skip_empty_from;
  if (Ma % kW2T == 0 && Nb % kW2T == 0 && G % 2 == 0 && (uintptr_t)C % 16 == 0)  // an expert's shapes: 256 x 256 tiles
    return wgrad256_launch<false>(a, (hipStream_t)stream);
  a.mtiles = Ma / kBM;
  a.ntiles = Nb / kBN;
  return gemm_launch<kModeWgrad>(a, (int64_t)a.mtiles * a.ntiles * G, (hipStream_t)stream);
}

extern "C" int mep_grouped_gemm_wgrad_tn(const void* X1, const void* X2, const int32_t* cu_seqlens, int G,
                                         float* C, int Ma, int Nb, int64_t rows, int skip_empty_from,
                                         void* stream) {
  MEP_REQUIRE(X1 && X2 && cu_seqlens && C, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(Ma > 0 && Nb > 0 && G > 0 && rows > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(Ma % kW2T == 0 && Nb % kW2T == 0 && G % 2 == 0 && rows % kBM == 0, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE((int64_t)(Ma > Nb ? Ma : Nb) * rows < ((int64_t)1 << 40), MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(((uintptr_t)X1 % 16 == 0) && ((uintptr_t)X2 % 16 == 0) && ((uintptr_t)C % 16 == 0),
              MEP_ERR_ALIGNMENT);
  GemmArgs a{};
  a.A = (const uint16_t*)X1; a.B = (const uint16_t*)X2; a.cu = cu_seqlens; a.Cf = C;
  a.M = Ma; a.N = Nb; a.K = 0; a.G = G;
  a.ld = rows;
  MEP_REQUIRE(skip_empty_from >= 0, MEP_ERR_INVALID_ARG);
  a.skip_from = skip_empty_from;
  return wgrad256_launch<true>(a, (hipStream_t)stream);
}

extern "C" int mep_transpose_bf16(const void* src, void* dst, int batch, int rows, int cols, void* stream) {
  MEP_REQUIRE(src && dst && src != dst, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(batch > 0 && rows > 0 && cols > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(rows % 64 == 0 && cols % 64 == 0 && batch <= 65535 && rows / 64 <= 65535, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(((uintptr_t)src % 4 == 0) && ((uintptr_t)dst % 4 == 0), MEP_ERR_ALIGNMENT);
  hipLaunchKernelGGL(transpose16_kernel, dim3(cols / 64, rows / 64, batch), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t*)src, (uint16_t*)dst, rows, cols);
  return mep_launch_status();
}

extern "C" int mep_swiglu_bwd(const void* dh, const void* gate_pre, const void* up_pre,
                              const float* row_scale, const int32_t* cu_seqlens, int G, void* dgate,
                              void* dup, void* hs, float* dscale, int M, int N, void* stream) {
  MEP_REQUIRE(dh && gate_pre && up_pre && cu_seqlens && dgate && dup && hs, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(M > 0 && N > 0 && G > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(N % 8 == 0, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE(((uintptr_t)dh % 16 == 0) && ((uintptr_t)gate_pre % 16 == 0) && ((uintptr_t)up_pre % 16 == 0) &&
                  ((uintptr_t)dgate % 16 == 0) && ((uintptr_t)dup % 16 == 0) && ((uintptr_t)hs % 16 == 0),
              MEP_ERR_ALIGNMENT);
  SwigluBwdArgs a;
  a.dh = (const uint16_t*)dh; a.gate = (const uint16_t*)gate_pre; a.up = (const uint16_t*)up_pre;
  a.scale = row_scale; a.cu = cu_seqlens;
  a.dgate = (uint16_t*)dgate; a.dup = (uint16_t*)dup; a.hs = (uint16_t*)hs; a.dscale = dscale;
  a.M = M; a.N = N; a.G = G;
  hipLaunchKernelGGL(swiglu_bwd_kernel, dim3((M + 3) / 4), dim3(256), 0, (hipStream_t)stream, a);
  return mep_launch_status();
}
