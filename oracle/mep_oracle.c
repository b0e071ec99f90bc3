/*
 * Scalar C restatement of the MoonEP per-rank hot path -- TEST INFRASTRUCTURE.
 *
 * A checker and a timed CPU baseline.  Only tests/, __graft_entry__.smoke()
 * and the cpu_baseline leg of bench.py load this library; the product
 * (moonep_amd, libmoonep_hip.so) never does.
 *
 * Written independently of oracle/planner_oracle.py (plain loops, no shared
 * helpers) so that the two restatements can pin each other on random inputs.
 * Reference lines followed:
 *   planner      tests/planning_reference.py:56-294
 *   dispatch     moonep/dispatch.py:394-433, 467-497
 *   combine      moonep/combine.py:379-435, 485-511;
 *                moonep/combine_prologue.py:380-478 (two-level variant)
 *   prefetch     moonep/prefetch.py:322-368, 398-465
 *   grad reduce  moonep/grad_reduce.py:221-276, 326-389
 *
 * Build: make -C oracle   (gcc -O2 -shared -fPIC)
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static int align_up(int x, int a) { return (x + a - 1) / a * a; }

/* ------------------------------------------------------------------ planner */

/* Rank-independent tables.  alloc_cum [E*R], expert_off [R*E], cu [R*2epn],
 * etc [R*epn], stats [R*2], zf [R*2epn*2], prev_all [R*E] (tokens of the
 * ranks before r).  Returns 0, or a negative code on inconsistent input. */
int ora_plan_global(const int32_t* tpe, int S, int K, int E, int R, int tp, int NvS,
                    int32_t* alloc_cum, int32_t* expert_off, int32_t* cu, int32_t* etc,
                    int32_t* stats, int32_t* zf, int32_t* prev_all) {
  const int epn = E / R, CAP = S * K;
  int64_t* cnt = calloc(E, sizeof(int64_t));
  int64_t* bal = calloc(R, sizeof(int64_t));
  int64_t* z = calloc((size_t)R * R, sizeof(int64_t));
  int64_t* alloc = calloc((size_t)E * R, sizeof(int64_t));
  int64_t* rem = calloc(epn, sizeof(int64_t));
  int64_t* quota = calloc(R, sizeof(int64_t));
  int rc = 0;
  for (int e = 0; e < E; ++e) {
    int64_t run = 0;
    for (int r = 0; r < R; ++r) { prev_all[r * E + e] = (int32_t)run; run += tpe[r * E + e]; }
    cnt[e] = run;
    bal[e / epn] += run;
    alloc[(size_t)e * R + e / epn] = run;
  }
  for (int h = 0; h < R; ++h) bal[h] -= CAP;
  for (;;) { /* receivers: fill the emptiest rank from the fullest group */
    int h = 0, u = 0;
    for (int r = 1; r < R; ++r) { if (bal[r] > bal[h]) h = r; if (bal[r] < bal[u]) u = r; }
    if (bal[h] <= 0) break;
    const int64_t move = -bal[u];
    z[(size_t)h * R + u] = move;
    bal[h] -= move;
    bal[u] = 0;
  }
  for (int h = 0; h < R; ++h) { /* which tokens migrate */
    for (int i = 0; i < epn; ++i) rem[i] = cnt[h * epn + i];
    for (int d = 0; d < R; ++d) quota[d] = z[(size_t)h * R + d];
    for (;;) {
      int d = 0, le = 0;
      for (int r = 1; r < R; ++r) if (quota[r] > quota[d]) d = r;
      if (quota[d] <= 0) break;
      for (int i = 1; i < epn; ++i) if (rem[i] > rem[le]) le = i;
      if (rem[le] <= 0) break;
      const int64_t take = rem[le] < quota[d] ? rem[le] : quota[d];
      alloc[(size_t)(h * epn + le) * R + d] += take;
      alloc[(size_t)(h * epn + le) * R + h] -= take;
      rem[le] -= take;
      quota[d] -= take;
    }
  }
  memset(expert_off, 0, sizeof(int32_t) * (size_t)R * E);
  memset(stats, 0, sizeof(int32_t) * (size_t)R * 2);
  memset(zf, 0, sizeof(int32_t) * (size_t)R * 4 * epn);
  for (int d = 0; d < R; ++d) {
    const int lo = d * epn, hi = lo + epn;
    int nrem = 0;
    for (int b = 0; b < epn; ++b) etc[d * epn + b] = -1;
    for (int e = 0; e < E; ++e) {
      if (alloc[(size_t)e * R + d] > 0 && (e < lo || e >= hi)) {
        if (nrem >= epn) { rc = -2; goto done; }
        etc[d * epn + nrem++] = e;
        stats[(e / epn) * 2 + 1] += 1;
      }
    }
    stats[d * 2] = nrem;
    int start = 0;
    for (int g = 0; g < 2 * epn; ++g) {
      int eid = g < epn ? lo + g : etc[d * epn + g - epn];
      int c = eid >= 0 ? (int)alloc[(size_t)eid * R + d] : 0;
      int padded = c > 0 ? align_up(c, tp) : 0;
      cu[d * 2 * epn + g] = start + padded;
      if (c > 0) {
        expert_off[d * E + eid] = start;
        if (padded > c) {
          zf[(d * 2 * epn + g) * 2] = start + c;
          zf[(d * 2 * epn + g) * 2 + 1] = padded - c;
        }
      }
      start += padded;
    }
    if (start > NvS) { rc = -3; goto done; }
  }
  for (int e = 0; e < E; ++e) {
    int64_t run = 0;
    for (int d = 0; d < R; ++d) { run += alloc[(size_t)e * R + d]; alloc_cum[(size_t)e * R + d] = (int32_t)run; }
    if (run != cnt[e]) { rc = -4; goto done; }
  }
done:
  free(cnt); free(bal); free(z); free(alloc); free(rem); free(quota);
  return rc;
}

/* canonical dst of one rank from the global tables */
int ora_plan_rank(const int32_t* topk, int rank, int S, int K, int E, int R, int NvS,
                  const int32_t* alloc_cum, const int32_t* expert_off, const int32_t* prev_all,
                  int32_t* dst) {
  const int N = S * K;
  int32_t* seen = calloc(E, sizeof(int32_t));
  for (int i = 0; i < N; ++i) {
    const int e = topk[i];
    if (e < 0 || e >= E) { free(seen); return -1; }
    const int g = prev_all[rank * E + e] + seen[e]++;
    int d = 0;
    while (d < R && alloc_cum[(size_t)e * R + d] <= g) ++d;
    if (d >= R) { free(seen); return -5; }
    const int before = d ? alloc_cum[(size_t)e * R + d - 1] : 0;
    dst[i] = d * NvS + expert_off[d * E + e] + (g - before);
  }
  free(seen);
  for (int s = 0; s < S; ++s)
    for (int k = K - 1; k >= 1; --k) { /* later entries on an already used rank */
      const int d = dst[s * K + k] / NvS;
      for (int j = 0; j < k; ++j) {
        const int v = dst[s * K + j];
        if ((v < 0 ? -v - 1 : v) / NvS == d) { dst[s * K + k] = -dst[s * K + k] - 1; break; }
      }
    }
  return 0;
}

/* whole planner for one rank: what the reference returns on `rank` */
int ora_plan(const int32_t* tpe, const int32_t* topk, int rank, int S, int K, int E, int R, int tp,
             int NvS, int32_t* dst, int32_t* cu_rank, int32_t* etc, int32_t* zf_rank,
             int32_t* stats_rank) {
  const int epn = E / R;
  int32_t* ac = malloc(sizeof(int32_t) * (size_t)E * R);
  int32_t* eo = malloc(sizeof(int32_t) * (size_t)E * R);
  int32_t* pv = malloc(sizeof(int32_t) * (size_t)E * R);
  int32_t* cu = malloc(sizeof(int32_t) * (size_t)R * 2 * epn);
  int32_t* zf = malloc(sizeof(int32_t) * (size_t)R * 4 * epn);
  int32_t* st = malloc(sizeof(int32_t) * (size_t)R * 2);
  int rc = ora_plan_global(tpe, S, K, E, R, tp, NvS, ac, eo, cu, etc, st, zf, pv);
  if (rc == 0) rc = ora_plan_rank(topk, rank, S, K, E, R, NvS, ac, eo, pv, dst);
  memcpy(cu_rank, cu + rank * 2 * epn, sizeof(int32_t) * 2 * epn);
  memcpy(zf_rank, zf + rank * 4 * epn, sizeof(int32_t) * 4 * epn);
  memcpy(stats_rank, st + rank * 2, sizeof(int32_t) * 2);
  free(ac); free(eo); free(pv); free(cu); free(zf); free(st);
  return rc;
}

/* ------------------------------------------------------------------ data ops */

static inline float bf2f(uint16_t b) { union { uint32_t u; float f; } x; x.u = (uint32_t)b << 16; return x.f; }
static inline uint16_t f2bf(float f) {
  union { uint32_t u; float f; } x; x.f = f;
  if (f != f) return 0x7fc0;
  return (uint16_t)((x.u + 0x7fffu + ((x.u >> 16) & 1u)) >> 16);
}

/* shards [R, stride_rows, H] bf16; wslots [R, wstride] */
void ora_dispatch(const uint16_t* hidden, const float* w, const int32_t* dst, const int32_t* zf,
                  uint16_t* shards, int64_t stride_rows, float* wslots, int64_t wstride, int rank,
                  int S, int H, int K, int epn, int NvS, int write_dups) {
  for (int s = 0; s < S; ++s)
    for (int k = 0; k < K; ++k) {
      const int v = dst[s * K + k];
      const int raw = v < 0 ? -v - 1 : v;
      const int d = raw / NvS, lo = raw % NvS;
      if (v >= 0 || write_dups)
        memcpy(shards + ((size_t)d * stride_rows + lo) * H, hidden + (size_t)s * H, (size_t)H * 2);
      if (w) wslots[(size_t)d * wstride + lo] = w[s * K + k];
    }
  for (int g = 0; zf && g < 2 * epn; ++g)
    for (int j = 0; j < zf[2 * g + 1]; ++j) {
      const int lo = zf[2 * g] + j;
      memset(shards + ((size_t)rank * stride_rows + lo) * H, 0, (size_t)H * 2);
      if (w) wslots[(size_t)rank * wstride + lo] = 0.0f;
    }
}

/* mode 0 primaries, 1 all, 2 two-level; acc is caller scratch of 2*H floats */
void ora_combine(const uint16_t* shards, int64_t stride_rows, const float* wslots, int64_t wstride,
                 const int32_t* dst, uint16_t* out, float* out_sk, int S, int H, int K, int NvS,
                 int mode, float* acc) {
  float* grp = acc + H;
  for (int s = 0; s < S; ++s) {
    for (int h = 0; h < H; ++h) acc[h] = 0.0f;
    for (int k = 0; k < K; ++k) {
      const int v = dst[s * K + k];
      const int raw = v < 0 ? -v - 1 : v;
      const int d = raw / NvS;
      const uint16_t* row = shards + ((size_t)d * stride_rows + raw % NvS) * H;
      if (out_sk) out_sk[s * K + k] = wslots[(size_t)d * wstride + raw % NvS];
      if (mode == 1 || (mode == 0 && v >= 0)) {
        for (int h = 0; h < H; ++h) acc[h] += bf2f(row[h]);
      } else if (mode == 2 && v >= 0) {
        int members = 0;
        for (int h = 0; h < H; ++h) grp[h] = 0.0f + bf2f(row[h]);
        for (int j = k + 1; j < K; ++j) {
          const int vj = dst[s * K + j];
          if (vj >= 0 || (-vj - 1) / NvS != d) continue;
          const uint16_t* rj = shards + ((size_t)d * stride_rows + (-vj - 1) % NvS) * H;
          for (int h = 0; h < H; ++h) grp[h] += bf2f(rj[h]);
          ++members;
        }
        for (int h = 0; h < H; ++h) acc[h] += members ? bf2f(f2bf(grp[h])) : grp[h];
      }
    }
    for (int h = 0; h < H; ++h) out[(size_t)s * H + h] = f2bf(acc[h]);
  }
}

void ora_prefetch(const char* local, char* pool, int64_t rank_stride_bytes, int64_t bytes,
                  const int32_t* etc, int rank, int epn, int R) {
  for (int d = 0; d < R; ++d)
    for (int b = 0; b < epn; ++b) {
      const int le = etc[d * epn + b] - rank * epn;
      if (le >= 0 && le < epn)
        memcpy(pool + d * rank_stride_bytes + b * bytes, local + le * bytes, (size_t)bytes);
    }
}

void ora_grad_reduce(float* local, float* pool, int64_t rank_stride, int64_t elems,
                     const int32_t* etc, int rank, int epn, int R) {
  for (int src = 0; src < R; ++src)
    for (int b = 0; b < epn; ++b) {
      const int le = etc[src * epn + b] - rank * epn;
      if (le < 0 || le >= epn) continue;
      float* g = local + le * elems;
      const float* p = pool + src * rank_stride + b * elems;
      for (int64_t i = 0; i < elems; ++i) g[i] += p[i];
    }
  for (int b = 0; b < epn; ++b)
    if (etc[rank * epn + b] >= 0) memset(pool + rank * rank_stride + b * elems, 0, (size_t)elems * 4);
}
