// Write-path probe for MI355X: how fast can 470 MB (32768 rows of 14 KiB, the
// volume one dispatch writes at S=4096, K=8, H=7168) be stored, depending on
// how the stores are laid out over waves and addresses?  No reads: every
// kernel stores constants, so the figures bound any copy kernel that writes
// with the same pattern.  Measurement program, not product code.
//
//   make -C tests/host write_path_probe
//   tests/host/write_path_probe            # every pattern, HIP-event timing
//   rocprofv3 --pmc <counters> -- tests/host/write_path_probe pmc   # 3 launches each
//
// Patterns (a "piece" is the 1 KiB a wave stores with one 16-byte store per lane):
//   dense<PER>     wave w stores pieces w*PER .. w*PER+PER-1; the grid covers the region in order
//   tiled<14>      a wave's 14 stores are 32 KiB apart, the 31 following waves fill the gaps
//   rows seq       one wave per 14 KiB row, rows in order (= dense<14>)
//   rows expert    rows grouped as a dispatch writes them: 256 expert segments, rows
//                  visited in token order (8 random experts per token)
//   rows random    rows drawn at random from the 4.7 GB of the 8 shards
//   runs<16>       a 16-wave workgroup stores 16 adjacent rows (224 KiB) at a random place
//   runs_col<L>    the same runs of L rows, but a wave owns "columns": pieces c, c+32, c+64, ...
//                  of the run, so its consecutive stores are 32 KiB apart
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

typedef uint32_t u4 __attribute__((ext_vector_type(4)));
#define CK(x)                                                                      \
  do {                                                                             \
    hipError_t e_ = (x);                                                           \
    if (e_ != hipSuccess) {                                                        \
      std::printf("FAIL %s: %s (line %d)\n", #x, hipGetErrorString(e_), __LINE__); \
      std::exit(2);                                                                \
    }                                                                              \
  } while (0)

constexpr int kWaves = 4;       // waves per workgroup unless stated
constexpr long kRows = 32768;   // S*K
constexpr int kPieces = 14;     // 1 KiB pieces per row (H = 7168 bf16)
constexpr long kRegionRows = 8 * 40960;  // 8 shards of 40960 rows (4.7 GB): random rows are drawn from all of it

template <int PER>
__global__ __launch_bounds__(kWaves * 64) void dense(char* out, long npieces) {
  const int lane = threadIdx.x & 63;
  const long gw = (long)blockIdx.x * kWaves + (threadIdx.x >> 6);
  const u4 z = {1u, 2u, (uint32_t)gw, 4u};
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const long piece = gw * PER + i;
    if (piece < npieces) __builtin_nontemporal_store(z, (u4*)(out + piece * 1024 + lane * 16));
  }
}

template <int PER>
__global__ __launch_bounds__(kWaves * 64) void tiled(char* out, long npieces) {
  constexpr int SP = 32;  // pieces between a wave's consecutive stores
  const int lane = threadIdx.x & 63;
  const long gw = (long)blockIdx.x * kWaves + (threadIdx.x >> 6);
  const long tile = gw / SP, j = gw % SP;
  const u4 z = {1u, 2u, (uint32_t)gw, 4u};
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const long piece = tile * (long)PER * SP + j + (long)SP * i;
    if (piece < npieces) __builtin_nontemporal_store(z, (u4*)(out + piece * 1024 + lane * 16));
  }
}

// one wave per row; WPB waves per workgroup; LIST only tells the row lists apart in a profile
// (0 in order, 1 expert segments, 2 random)
template <int WPB, int LIST>
__global__ __launch_bounds__(WPB * 64) void rows(char* out, const int* row_of, long nrows) {
  const int lane = threadIdx.x & 63;
  const long gw = (long)blockIdx.x * WPB + (threadIdx.x >> 6);
  if (gw >= nrows) return;
  const long row = row_of[gw];
  const u4 z = {1u, 2u, (uint32_t)gw, 4u};
  char* p = out + row * (kPieces * 1024L) + lane * 16;
#pragma unroll
  for (int i = 0; i < kPieces; ++i) __builtin_nontemporal_store(z, (u4*)(p + i * 1024));
}

// persistent form of `rows`: a fixed grid, every wave takes the rows gw, gw + (waves of the grid), ...
template <int WPB>
__global__ __launch_bounds__(WPB * 64) void rows_persistent(char* out, const int* row_of, long nrows) {
  const int lane = threadIdx.x & 63;
  const long nw = (long)gridDim.x * WPB;
  for (long gw = (long)blockIdx.x * WPB + (threadIdx.x >> 6); gw < nrows; gw += nw) {
    const long row = row_of[gw];
    const u4 z = {1u, 2u, (uint32_t)gw, 4u};
    char* p = out + row * (kPieces * 1024L) + lane * 16;
#pragma unroll
    for (int i = 0; i < kPieces; ++i) __builtin_nontemporal_store(z, (u4*)(p + i * 1024));
  }
}

// one workgroup of 14 waves per row: every thread stores once, the row's 14 KiB leave together
__global__ __launch_bounds__(kPieces * 64) void row_burst(char* out, const int* row_of, long nrows) {
  const long row = row_of[blockIdx.x];
  const u4 z = {1u, 2u, (uint32_t)blockIdx.x, 4u};
  __builtin_nontemporal_store(z, (u4*)(out + row * (kPieces * 1024L) + threadIdx.x * 16));
}

// a WPB-wave workgroup stores WPB adjacent rows starting at start[block]
template <int WPB>
__global__ __launch_bounds__(WPB * 64) void runs(char* out, const int* start, long nblocks) {
  const int lane = threadIdx.x & 63;
  if ((long)blockIdx.x >= nblocks) return;
  const long row = (long)start[blockIdx.x] + (threadIdx.x >> 6);
  const u4 z = {1u, 2u, (uint32_t)row, 4u};
  char* p = out + row * (kPieces * 1024L) + lane * 16;
#pragma unroll
  for (int i = 0; i < kPieces; ++i) __builtin_nontemporal_store(z, (u4*)(p + i * 1024));
}

// an L-wave workgroup stores L adjacent rows (14 L pieces) column-wise: wave w owns the pieces
// c + 32 k of the run for c = w, w + L, ... < 32
template <int L>
__global__ __launch_bounds__(L * 64) void runs_col(char* out, const int* start, long nblocks) {
  constexpr int N = kPieces * L;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if ((long)blockIdx.x >= nblocks) return;
  const long row0 = start[blockIdx.x];
  const u4 z = {1u, 2u, (uint32_t)row0, 4u};
  char* base = out + row0 * (kPieces * 1024L) + lane * 16;
#pragma unroll
  for (int c0 = 0; c0 < 32; c0 += L)
#pragma unroll
    for (int q = 0; q < N; q += 32) {
      const int piece = c0 + w + q;
      if (c0 + w < 32 && piece < N) __builtin_nontemporal_store(z, (u4*)(base + (size_t)piece * 1024));
    }
}

template <class F>
static float time_us(F f, int iters) {
  hipEvent_t a, b;
  CK(hipEventCreate(&a));
  CK(hipEventCreate(&b));
  f();
  CK(hipEventRecord(a));
  for (int i = 0; i < iters; ++i) f();
  CK(hipEventRecord(b));
  CK(hipEventSynchronize(b));
  float ms = 0.f;
  CK(hipEventElapsedTime(&ms, a, b));
  CK(hipGetLastError());
  CK(hipEventDestroy(a));
  CK(hipEventDestroy(b));
  return ms * 1000.f / iters;
}

static int* upload(const std::vector<int>& v) {
  int* d = nullptr;
  CK(hipMalloc(&d, v.size() * sizeof(int)));
  CK(hipMemcpy(d, v.data(), v.size() * sizeof(int), hipMemcpyHostToDevice));
  return d;
}

int main(int argc, char** argv) {
  const bool pmc = argc > 1 && std::strcmp(argv[1], "pmc") == 0;
  const int iters = pmc ? 2 : 12;  // plus one untimed launch each
  const long np = kRows * kPieces;
  const double bytes = (double)np * 1024;
  char* out = nullptr;
  CK(hipMalloc(&out, (size_t)kRegionRows * kPieces * 1024));
  std::mt19937 g(3);

  std::vector<int> seq(kRows), rnd(kRegionRows), expert(kRows), run16(kRows / 16), run8(kRows / 8);
  for (long i = 0; i < kRows; ++i) seq[i] = (int)i;
  for (long i = 0; i < kRegionRows; ++i) rnd[i] = (int)i;
  std::shuffle(rnd.begin(), rnd.end(), g);
  rnd.resize(kRows);
  {  // 8 distinct experts per token out of 256; rank d holds experts 32d..32d+31 in a shard of
     // 40960 rows; an expert's rows are adjacent and filled in token order
    const int S = 4096, K = 8, E = 256, NvS = 40960;
    std::vector<int> ex(S * K), tot(E, 0), base(E), cnt(E, 0);
    for (int s = 0; s < S; ++s)
      for (int got = 0; got < K;) {
        const int e = (int)(g() % E);
        bool dup = false;
        for (int j = 0; j < got; ++j) dup |= ex[s * K + j] == e;
        if (!dup) ex[s * K + got++] = e;
      }
    for (int i = 0; i < S * K; ++i) tot[ex[i]]++;
    for (int d = 0; d < 8; ++d) {
      int o = 0;
      for (int le = 0; le < 32; ++le) {
        const int e = d * 32 + le;
        base[e] = d * NvS + o + 3 * tot[e];  // other ranks' rows sit around this rank's
        o += ((8 * tot[e] + 127) / 128) * 128;
      }
      if (o > NvS) { std::printf("FAIL expert layout does not fit\n"); return 2; }
    }
    for (int i = 0; i < S * K; ++i) expert[i] = base[ex[i]] + cnt[ex[i]]++;
  }
  {
    std::vector<int> slots(kRegionRows / 16);
    for (size_t i = 0; i < slots.size(); ++i) slots[i] = (int)(i * 16);
    std::shuffle(slots.begin(), slots.end(), g);
    for (size_t i = 0; i < run16.size(); ++i) run16[i] = slots[i];
    std::vector<int> slots8(kRegionRows / 8);
    for (size_t i = 0; i < slots8.size(); ++i) slots8[i] = (int)(i * 8);
    std::shuffle(slots8.begin(), slots8.end(), g);
    for (size_t i = 0; i < run8.size(); ++i) run8[i] = slots8[i];
  }
  int *d_seq = upload(seq), *d_rnd = upload(rnd), *d_exp = upload(expert), *d_run = upload(run16), *d_run8 = upload(run8);

  auto report = [&](const char* name, float us) {
    std::printf("%-28s %7.1f us  %5.2f TB/s  %4.1f %% of 8 TB/s\n", name, us, bytes / us / 1e6,
                bytes / us / 1e6 / 8.0 * 100.0);
    std::fflush(stdout);
  };
  const int grid1 = (int)(np / kWaves), grid2 = (int)(np / 2 / kWaves), grid14 = (int)(kRows / kWaves);
  for (int rep = 0; rep < (pmc ? 1 : 2); ++rep) {
    std::printf("--- pass %d (470 MB per launch, %d timed launches each)\n", rep, iters);
    report("dense<1>  1 store/wave", time_us([&] { dense<1><<<grid1, kWaves * 64>>>(out, np); }, iters));
    report("dense<2>  2 stores/wave", time_us([&] { dense<2><<<grid2, kWaves * 64>>>(out, np); }, iters));
    report("dense<14> 14 stores/wave", time_us([&] { dense<14><<<grid14, kWaves * 64>>>(out, np); }, iters));
    report("tiled<14> 32 KiB apart", time_us([&] { tiled<14><<<grid14, kWaves * 64>>>(out, np); }, iters));
    report("rows seq", time_us([&] { rows<4, 0><<<grid14, 256>>>(out, d_seq, kRows); }, iters));
    report("rows expert segments", time_us([&] { rows<4, 1><<<grid14, 256>>>(out, d_exp, kRows); }, iters));
    report("rows random", time_us([&] { rows<4, 2><<<grid14, 256>>>(out, d_rnd, kRows); }, iters));
    report("rows random, 8 waves/wg", time_us([&] { rows<8, 2><<<(int)(kRows / 8), 512>>>(out, d_rnd, kRows); }, iters));
    report("rows expert, 256 persistent wgs", time_us([&] { rows_persistent<4><<<256, 256>>>(out, d_exp, kRows); }, iters));
    report("rows expert, 512 persistent wgs", time_us([&] { rows_persistent<4><<<512, 256>>>(out, d_exp, kRows); }, iters));
    report("rows expert, 2048 persistent wgs", time_us([&] { rows_persistent<4><<<2048, 256>>>(out, d_exp, kRows); }, iters));
    report("row_burst expert (14 waves/row)", time_us([&] { row_burst<<<(int)kRows, kPieces * 64>>>(out, d_exp, kRows); }, iters));
    report("runs<16> 224 KiB random", time_us([&] { runs<16><<<(int)(kRows / 16), 1024>>>(out, d_run, kRows / 16); }, iters));
    report("runs_col<16> same runs", time_us([&] { runs_col<16><<<(int)(kRows / 16), 1024>>>(out, d_run, kRows / 16); }, iters));
    report("runs_col<8> 112 KiB random", time_us([&] { runs_col<8><<<(int)(kRows / 8), 512>>>(out, d_run8, kRows / 8); }, iters));
  }
  CK(hipDeviceSynchronize());
  std::printf("DONE\n");
  return 0;
}
