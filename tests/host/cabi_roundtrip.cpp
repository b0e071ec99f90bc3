// The C ABI used from plain C++: hipMalloc'd buffers, no Python, no torch.
// Plans, dispatches, combines, prefetches and reduces one small emulated
// group on the current GPU and compares every result, bit for bit, with the
// scalar C checker (oracle/mep_oracle.c).  Test program, not product code.
//
//   hipcc tests/host/cabi_roundtrip.cpp -Iinclude -Lmoonep_amd -lmoonep_hip \
//         -Loracle -lmep_oracle -o tests/host/cabi_roundtrip    (see tests/host/Makefile)
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "moonep_hip.h"

extern "C" {
int ora_plan(const int32_t* tpe, const int32_t* topk, int rank, int S, int K, int E, int R, int tp,
             int NvS, int32_t* dst, int32_t* cu_rank, int32_t* etc, int32_t* zf_rank,
             int32_t* stats_rank);
void ora_dispatch(const uint16_t* hidden, const float* w, const int32_t* dst, const int32_t* zf,
                  uint16_t* shards, int64_t stride_rows, float* wslots, int64_t wstride, int rank,
                  int S, int H, int K, int epn, int NvS, int write_dups);
void ora_combine(const uint16_t* shards, int64_t stride_rows, const float* wslots, int64_t wstride,
                 const int32_t* dst, uint16_t* out, float* out_sk, int S, int H, int K, int NvS,
                 int mode, float* acc);
void ora_prefetch(const char* local, char* pool, int64_t rank_stride_bytes, int64_t bytes,
                  const int32_t* etc, int rank, int epn, int R);
void ora_grad_reduce(float* local, float* pool, int64_t rank_stride, int64_t elems,
                     const int32_t* etc, int rank, int epn, int R);
}

#define HIP_OK(x)                                                                        \
  do {                                                                                   \
    hipError_t e_ = (x);                                                                 \
    if (e_ != hipSuccess) {                                                              \
      std::printf("FAIL %s: %s (line %d)\n", #x, hipGetErrorString(e_), __LINE__);       \
      return 2;                                                                          \
    }                                                                                    \
  } while (0)
#define MEP_OK_(x)                                                                       \
  do {                                                                                   \
    int c_ = (x);                                                                        \
    if (c_ != 0) {                                                                       \
      std::printf("FAIL %s: %s (line %d)\n", #x, mep_strerror(c_), __LINE__);            \
      return 2;                                                                          \
    }                                                                                    \
  } while (0)

static uint32_t g_state = 12345u;
static uint32_t rnd() { g_state = g_state * 1664525u + 1013904223u; return g_state >> 8; }

template <class T>
struct Dev {
  T* p = nullptr;
  size_t n = 0;
  hipError_t alloc(size_t count) { n = count; return hipMalloc((void**)&p, count * sizeof(T)); }
  hipError_t up(const std::vector<T>& h) { return hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice); }
  hipError_t down(std::vector<T>& h) const { h.resize(n); return hipMemcpy(h.data(), p, n * sizeof(T), hipMemcpyDeviceToHost); }
  ~Dev() { if (p) (void)hipFree(p); }
};

template <class T>
static int same(const char* what, const std::vector<T>& got, const std::vector<T>& want) {
  if (got.size() == want.size() && std::memcmp(got.data(), want.data(), got.size() * sizeof(T)) == 0) {
    std::printf("ok   %s (%zu elements)\n", what, got.size());
    return 0;
  }
  size_t i = 0;
  while (i < got.size() && i < want.size() && std::memcmp(&got[i], &want[i], sizeof(T)) == 0) ++i;
  std::printf("FAIL %s: first difference at element %zu\n", what, i);
  return 1;
}

int main() {
  const int S = 96, H = 328, K = 4, R = 4, epn = 3, E = R * epn, tp = 8, rank = 1;
  const int NvS = (S * K + (tp - 1) * 2 * epn + tp - 1) / tp * tp;  // reference moonep/api.py:286-290
  const int N = S * K;
  std::printf("libmoonep_hip v%d: S=%d H=%d K=%d E=%d R=%d tp=%d NvS=%d rank=%d\n", mep_version(), S, H,
              K, E, R, tp, NvS, rank);
  int bad = 0;
  if (mep_version() != 200) { std::printf("FAIL header and library disagree on the ABI version\n"); return 2; }
  MEP_OK_(mep_init());   // per-device set-up, outside any capture

  // ---- routing of all ranks (skewed: low expert ids are popular), counts table
  std::vector<int32_t> topk((size_t)R * N), tpe((size_t)R * E, 0);
  for (int r = 0; r < R; ++r)
    for (int s = 0; s < S; ++s)
      for (int k = 0; k < K; ++k) {
        const int e = (int)((rnd() % E) * (rnd() % E) / E);
        topk[((size_t)r * S + s) * K + k] = e;
        ++tpe[(size_t)r * E + e];
      }
  std::vector<int32_t> my_topk(topk.begin() + (size_t)rank * N, topk.begin() + (size_t)(rank + 1) * N);

  // ---- planner
  std::vector<int32_t> dst_ref(N), cu_ref(2 * epn), etc_ref(R * epn), zf_ref(4 * epn), st_ref(2);
  if (ora_plan(tpe.data(), my_topk.data(), rank, S, K, E, R, tp, NvS, dst_ref.data(), cu_ref.data(),
               etc_ref.data(), zf_ref.data(), st_ref.data()) != 0) {
    std::printf("FAIL checker rejected the routing\n");
    return 2;
  }
  Dev<int32_t> d_tpe, d_topk, d_dst, d_cu, d_etc, d_zf, d_st;
  HIP_OK(d_tpe.alloc(tpe.size())); HIP_OK(d_tpe.up(tpe));
  HIP_OK(d_topk.alloc(N)); HIP_OK(d_topk.up(my_topk));
  HIP_OK(d_dst.alloc(N)); HIP_OK(d_cu.alloc(2 * epn)); HIP_OK(d_etc.alloc(R * epn));
  HIP_OK(d_zf.alloc(4 * epn)); HIP_OK(d_st.alloc(2));
  if (mep_plan_scratch_bytes(S, K, E, R, 1) != 0) { std::printf("FAIL unexpected scratch\n"); return 2; }
  MEP_OK_(mep_plan(d_tpe.p, d_topk.p, rank, S, K, E, R, tp, NvS, d_dst.p, d_cu.p, d_etc.p, d_zf.p,
                   d_st.p, nullptr, 0, nullptr));
  HIP_OK(hipDeviceSynchronize());
  std::vector<int32_t> got_i;
  HIP_OK(d_dst.down(got_i)); bad += same("planner dst", got_i, dst_ref);
  HIP_OK(d_cu.down(got_i)); bad += same("planner cu_seqlens", got_i, cu_ref);
  HIP_OK(d_etc.down(got_i)); bad += same("planner experts_to_copy", got_i, etc_ref);
  HIP_OK(d_zf.down(got_i)); bad += same("planner zero_fill_ranges", got_i, zf_ref);
  HIP_OK(d_st.down(got_i)); bad += same("planner remote_stats", got_i, st_ref);

  // ---- dispatch (all K copies) and combine (two-level and primaries) with weights
  std::vector<uint16_t> hidden((size_t)S * H), shards_ref((size_t)R * NvS * H, 0x7f7f);
  std::vector<float> w((size_t)N), ws_ref((size_t)R * NvS, -7.0f);
  for (auto& v : hidden) v = (uint16_t)(0x3c00 + rnd() % 0x0800) ^ (uint16_t)((rnd() & 1) << 15);
  for (auto& v : w) v = (float)(rnd() % 1000) / 1000.0f;
  Dev<uint16_t> d_hidden, d_shards, d_out;
  Dev<float> d_w, d_ws, d_outw;
  HIP_OK(d_hidden.alloc(hidden.size())); HIP_OK(d_hidden.up(hidden));
  HIP_OK(d_shards.alloc(shards_ref.size())); HIP_OK(d_shards.up(shards_ref));
  HIP_OK(d_w.alloc(w.size())); HIP_OK(d_w.up(w));
  HIP_OK(d_ws.alloc(ws_ref.size())); HIP_OK(d_ws.up(ws_ref));
  HIP_OK(d_out.alloc((size_t)S * H)); HIP_OK(d_outw.alloc(N));
  ora_dispatch(hidden.data(), w.data(), dst_ref.data(), zf_ref.data(), shards_ref.data(), NvS,
               ws_ref.data(), NvS, rank, S, H, K, epn, NvS, 1);
  MEP_OK_(mep_dispatch(d_hidden.p, d_w.p, d_dst.p, d_zf.p, d_shards.p, NvS, d_ws.p, NvS, rank, S, H, K,
                       R, epn, NvS, tp, MEP_DISPATCH_WRITE_DUPS, nullptr));
  HIP_OK(hipDeviceSynchronize());
  std::vector<uint16_t> got_h;
  std::vector<float> got_f;
  HIP_OK(d_shards.down(got_h)); bad += same("dispatch rows (poison kept elsewhere)", got_h, shards_ref);
  HIP_OK(d_ws.down(got_f)); bad += same("dispatch weight slots", got_f, ws_ref);

  std::vector<float> acc(2 * (size_t)H);
  const int modes[2] = {MEP_COMBINE_TWO_LEVEL, MEP_COMBINE_PRIMARIES};
  for (int mode : modes) {
    std::vector<uint16_t> out_ref((size_t)S * H);
    std::vector<float> outw_ref(N);
    ora_combine(shards_ref.data(), NvS, ws_ref.data(), NvS, dst_ref.data(), out_ref.data(),
                outw_ref.data(), S, H, K, NvS, mode, acc.data());
    MEP_OK_(mep_combine(d_shards.p, NvS, d_ws.p, NvS, d_dst.p, d_out.p, d_outw.p, S, H, K, R, NvS, mode,
                        nullptr));
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(d_out.down(got_h));
    bad += same(mode == MEP_COMBINE_TWO_LEVEL ? "combine two-level" : "combine primaries", got_h, out_ref);
    HIP_OK(d_outw.down(got_f)); bad += same("combine weight gather", got_f, outw_ref);
  }

  // ---- prefetch (3 tensors of different sizes) and grad reduce on the planner's own slot table
  const int64_t bytes[3] = {4096, 1536, 16};
  std::vector<std::vector<char>> local(3), pool_ref(3);
  Dev<char> d_local[3], d_pool[3];
  const void* lp[3]; void* pp[3]; int64_t stride[3];
  for (int t = 0; t < 3; ++t) {
    local[t].resize((size_t)epn * bytes[t]);
    for (auto& c : local[t]) c = (char)rnd();
    stride[t] = epn * bytes[t] + 64;  // a gap between the ranks' pools
    pool_ref[t].assign((size_t)R * stride[t], (char)0x5a);
    HIP_OK(d_local[t].alloc(local[t].size())); HIP_OK(d_local[t].up(local[t]));
    HIP_OK(d_pool[t].alloc(pool_ref[t].size())); HIP_OK(d_pool[t].up(pool_ref[t]));
    ora_prefetch(local[t].data(), pool_ref[t].data(), stride[t], bytes[t], etc_ref.data(), rank, epn, R);
    lp[t] = d_local[t].p; pp[t] = d_pool[t].p;
  }
  MEP_OK_(mep_prefetch(3, lp, pp, stride, bytes, d_etc.p, rank, epn, R, nullptr));
  HIP_OK(hipDeviceSynchronize());
  for (int t = 0; t < 3; ++t) {
    std::vector<char> got_c;
    HIP_OK(d_pool[t].down(got_c));
    bad += same("prefetch pool", got_c, pool_ref[t]);
  }
  const int64_t elems = 1000;
  std::vector<float> grad((size_t)epn * elems), red((size_t)R * epn * elems);
  for (auto& v : grad) v = (float)(int)(rnd() % 2001 - 1000) * 1e-3f;
  for (auto& v : red) v = (float)(int)(rnd() % 2001 - 1000) * 1e-4f;
  Dev<float> d_grad, d_red;
  HIP_OK(d_grad.alloc(grad.size())); HIP_OK(d_grad.up(grad));
  HIP_OK(d_red.alloc(red.size())); HIP_OK(d_red.up(red));
  ora_grad_reduce(grad.data(), red.data(), epn * elems, elems, etc_ref.data(), rank, epn, R);
  MEP_OK_(mep_grad_reduce(d_grad.p, d_red.p, epn * elems, d_etc.p, rank, epn, R, elems, 0u, nullptr));
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(d_grad.down(got_f)); bad += same("grad reduce local grads", got_f, grad);
  HIP_OK(d_red.down(got_f)); bad += same("grad reduce pool after clears", got_f, red);

  // ---- error path: a bad argument is a return code, not a crash
  if (mep_combine(d_shards.p, NvS, nullptr, 0, d_dst.p, d_out.p, nullptr, S, H + 1, K, R, NvS, 0, nullptr) !=
      MEP_ERR_UNSUPPORTED) {
    std::printf("FAIL H %% 8 != 0 was not rejected\n");
    ++bad;
  }
  std::printf(bad ? "FAILED: %d mismatches\n" : "ALL OK\n", bad);
  return bad ? 1 : 0;
}
