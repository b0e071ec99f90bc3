// Online redundant-expert planner for gfx950.
//
// One kernel, no grid-wide synchronisation: every workgroup rebuilds the
// (tiny, rank-independent) balancing plan in its own LDS from the R x E count
// matrix and then resolves the slots of its own slice of the rank's S*K
// routed entries.  Rebuilding the plan per workgroup costs nothing in latency
// (workgroups run side by side on different CUs) and removes the reference's
// rank-0 stage, its broadcast and its three barriers
// (reference moonep/planning.py:577-583, 917-922, 941, 1045).
//
// Results are bit-identical to the reference oracle
// (reference tests/planning_reference.py:25-311).
//
// The kernel is a chain of latencies, not of bandwidth or arithmetic, and is laid
// out for that.  Phases of a workgroup, separated by workgroup barriers:
//   0  issue every global load whose address is known (own entry, count matrix,
//      first part of the routing to count), clear LDS
//   1  counts per expert and per home group
//   2  wave 0: greedy choice of receivers and quotas | other waves: rank of each
//      entry among its wave's entries of the same expert, first part of the count
//      of this rank's earlier (or later) entries per expert
//   3  waves 1..R: which tokens of which expert migrate | wave 0: its own entries'
//      ranks | upper waves: second part of the count
//   4  waves 1..R: slot layout of every destination | upper waves: last part
//   5  every entry: number within its expert -> destination rank -> slot;
//      duplicates of a token on one rank found along DPP rows; store
#include "mep_common.h"

#include <atomic>

namespace {

struct PlanArgs {
  const int* tpe;    // [R,E]
  const int* topk;   // [nranks, S*K]
  int* dst;          // [nranks, S*K]
  int* cu_seqlens;   // [nranks, 2*epn]
  int* etc;          // [R, epn]
  int* zero_fill;    // [nranks, 2*epn, 2]
  int* remote_stats; // [nranks, 2]
  int* scratch;      // alloc/base tables when they do not fit in LDS
  int rank0, S, K, E, R, epn, tp, NvS, tok_per_wg;
  // optional: a byte range the workgroups beyond `groups` read once, so that it
  // sits in the last-level cache when the planner is done (the tokens that the
  // following dispatch copies); the planner itself occupies only a few CUs
  const char* warm;
  size_t warm_vecs;  // 16-byte vectors
  int groups;        // workgroups per rank that plan
};

// LDS layout in ints (must match plan_lds_bytes on the host)
template <int NT>
struct PlanLds {
  static constexpr int NW = NT / MEP_WAVE;
  static constexpr int W4 = (NW + 3) / 4;  // packed per-wave byte counters per expert
  static constexpr int E_ARRAYS = 6 + W4;
  static constexpr int R_ARRAYS = 6;
  static constexpr int FIXED = NT;
};

// RC, KC: the number of ranks and top-k as compile-time constants (0: taken
// from the arguments); the planner is a chain of dependent instructions, and
// a kernel that knows them drops the loops, clamps and alternative paths
template <int NT, bool kLdsTables, int RC = 0, int KC = 0>
__global__ __launch_bounds__(NT) void plan_kernel(PlanArgs a) {
  using L = PlanLds<NT>;
  constexpr int NW = L::NW;
  constexpr int W4 = L::W4;
  extern __shared__ int smem[];
  const int E = a.E, R = RC > 0 ? RC : a.R, epn = a.epn, tp = a.tp, NvS = a.NvS, K = KC > 0 ? KC : a.K;
  const int N = a.S * K;
  const int CAP = N;
  int* s_cnt = smem;             // [E] tokens per expert, all ranks
  int* s_prev = s_cnt + E;       // [E] tokens of the ranks before this one
  int* s_rem = s_prev + E;       // [E] not yet migrated
  int* s_etc = s_rem + E;        // [R*epn] remote experts per destination
  int* s_hist = s_etc + E;       // [E] entries of this rank before my slice, or after it
  int* s_own = s_hist + E;       // [E] tokens of this rank
  int* s_wcnt = s_own + E;       // [E*W4] per-wave counts, one byte per wave
  int* s_gt = s_wcnt + W4 * E;   // [R] tokens per home group
  int* s_from = s_gt + R;        // [R] donor feeding this receiver (-1: none)
  int* s_quota = s_from + R;     // [R] tokens still to receive
  int* s_stat1 = s_quota + R;    // [R] slots elsewhere holding my experts
  int* s_nrem = s_stat1 + R;     // [R] remote experts on this destination
  int* s_bal = s_nrem + R;       // [R] word 0: where counts of invalid expert ids go
  int* s_cd = s_bal + R;         // [NT] destination rank of each entry
  int* tbl = kLdsTables ? (s_cd + NT)
                        : a.scratch + (size_t)(blockIdx.y * a.groups + blockIdx.x) * 2 * E * R;
  int* alloc = tbl;            // [E,R] tokens of expert e landing on rank d
  int* base = tbl + E * R;     // [E,R] first slot of e on d, as an encoded dst

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: roles branch on scalars
  if ((int)blockIdx.x >= a.groups) {
    // cache warmer: plain 16-byte loads, eight in flight.  The values only feed
    // a comparison that guards a sleep, so the loads stay and nothing is written.
    if (blockIdx.y != 0 || a.warm_vecs == 0) return;
    const size_t nthreads = (size_t)(gridDim.x - a.groups) * NT;
    const size_t first = (size_t)(blockIdx.x - a.groups) * NT + tid;
    const mep_u4* w = (const mep_u4*)a.warm;
    mep_u4 x = {0u, 0u, 0u, 0u};
    for (size_t i = first; i < a.warm_vecs; i += 8 * nthreads) {
      mep_u4 t[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const size_t j = i + u * nthreads;
        t[u] = w[j < a.warm_vecs ? j : a.warm_vecs - 1];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) x ^= t[u];
    }
    if ((x[0] ^ x[1]) == 0x9e3779b9u && (x[2] ^ x[3]) == 0x7f4a7c15u) __builtin_amdgcn_s_sleep(1);
    return;
  }
  const int rank = a.rank0 + blockIdx.y;
  const bool writer = blockIdx.x == 0;  // one workgroup per rank stores the small outputs
  const int* topk = a.topk + (size_t)blockIdx.y * N;
  const int t0 = blockIdx.x * a.tok_per_wg;
  const int t1 = min(t0 + a.tok_per_wg, a.S);
  const int e0 = t0 * K;
  const int n = (t1 - t0) * K;  // <= NT

  // ---- every load whose address is known now goes out before anything waits ----
  // (the planner is a chain of latencies; beside a stream of other traffic a
  // load issued late costs two to three times as much)
  int e = -1;  // expert of my entry
  if (tid < n) e = topk[e0 + tid];
  int tv[8];   // counts of expert `tid` on the first eight ranks (clamped row: no branch)
  if (tid < E) {
#pragma unroll
    for (int j = 0; j < 8; ++j) tv[j] = a.tpe[(j < R ? j : R - 1) * E + tid];
  }
  // Per expert, this rank's entries that precede the workgroup's slice - or
  // those that follow it, where these are fewer: tokens_per_expert is the rank's
  // count per expert (reference moonep/api.py:735), so what precedes is the
  // total less the slice less what follows.  The count needs nothing from the
  // plan and is only used when the entries are resolved, so it runs beside the
  // planning phases.  Wave 0 plans alone in the first of them
  // (the serial greedy) while every other wave counts; in the two phases that
  // follow, waves 1..R plan (one per rank) and the waves above them count.  Each
  // part's first loads are issued one phase ahead.  With more ranks than that
  // leaves counting waves for, the first phase takes all of it.
  constexpr int HWB = NW / 2 + 1;       // first wave that counts in the later phases
  constexpr int NA = NT - 64, NB = NT - HWB * 64;
  const int ta = tid - 64, tb = tid - HWB * 64;
  const bool count_a = wave >= 1, count_b = wave >= HWB;
  const bool hist_vec = (((uintptr_t)topk) & 15) == 0;
  const bool spread = R < HWB;
  const bool fwd = e0 <= N - (e0 + n);         // count what precedes the slice
  const int c0 = fwd ? 0 : e0 + n, c1 = fwd ? e0 : N;
  // entries [c0, c1) = a head up to a 16-byte boundary, vectors [v0, v1), a tail
  const int v0 = (c0 + 3) >> 2;
  const int v1 = hist_vec && (c1 >> 2) > v0 ? c1 >> 2 : v0;
  const int head_end = min(4 * v0, c1), tail_start = max(4 * v1, head_end);
  const int hb1 = v0 + (spread ? (int)(((int64_t)(v1 - v0) * 12) >> 5) : v1 - v0);
  const int hb2 = v0 + (spread ? (int)(((int64_t)(v1 - v0) * 22) >> 5) : v1 - v0);
  const int4* t4 = (const int4*)topk;
  // loads v[u] = vector (b + t + u*nt) for those below `end`
  auto hist_load = [&](auto& v, int b, int end, int t, int nt) {
    constexpr int G = sizeof(v) / sizeof(v[0]);
#pragma unroll
    for (int u = 0; u < G; ++u)
      if (b + t + u * nt < end) v[u] = t4[b + t + u * nt];
  };
  // an id outside [0, E) counts into a word nobody reads: no branch per atomic
  auto bin = [&](int x) { return (unsigned)x < (unsigned)E ? s_hist + x : s_bal; };
  auto hist_count = [&](const auto& v, int b, int end, int t, int nt) {
    constexpr int G = sizeof(v) / sizeof(v[0]);
#pragma unroll
    for (int u = 0; u < G; ++u)
      if (b + t + u * nt < end) {
        atomicAdd(bin(v[u].x), 1);
        atomicAdd(bin(v[u].y), 1);
        atomicAdd(bin(v[u].z), 1);
        atomicAdd(bin(v[u].w), 1);
      }
  };
  // counts [b, end) given its first group already loaded into v
  auto hist_part = [&](auto& v, int b, int end, int t, int nt) {
    constexpr int G = sizeof(v) / sizeof(v[0]);
    hist_count(v, b, end, t, nt);
    for (int i = b + G * nt; i < end; i += G * nt) {
      hist_load(v, i, end, t, nt);
      hist_count(v, i, end, t, nt);
    }
  };
  int4 ha[4], hb[6], hc[6];
  if (count_a) hist_load(ha, v0, hb1, ta, NA);

  for (int i = tid; i < R; i += NT) {
    s_gt[i] = 0; s_from[i] = -1; s_quota[i] = 0; s_stat1[i] = 0; s_nrem[i] = 0;
  }
  for (int i = tid; i < W4 * E; i += NT) s_wcnt[i] = 0;
  for (int i = tid; i < E; i += NT) s_hist[i] = 0;
  __syncthreads();

  // ---- counts per expert, per home group --------------------------------
  const int epn_shift = (epn & (epn - 1)) == 0 ? 31 - __clz(epn) : -1;
  for (int ee = tid; ee < E; ee += NT) {
    int c = 0, p = 0, own = 0;
    for (int r0 = 0; r0 < R; r0 += 8) {  // eight independent loads in flight
      int v[8];
      if (ee == tid && r0 == 0) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = tv[j];
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          v[j] = a.tpe[(r0 + j < R ? r0 + j : R - 1) * E + ee];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int x = r0 + j < R ? v[j] : 0;
        p += r0 + j < rank ? x : 0;
        own += r0 + j == rank ? x : 0;
        c += x;
      }
    }
    s_cnt[ee] = c; s_prev[ee] = p; s_rem[ee] = c; s_own[ee] = own;
    const int home = epn_shift >= 0 ? ee >> epn_shift : ee / epn;
    for (int d = 0; d < R; ++d) alloc[ee * R + d] = (d == home) ? c : 0;
    atomicAdd(&s_gt[home], c);
  }
  __syncthreads();

  // ---- receivers and quotas (wave 0) | my entry among those of my wave | histogram
  // Each receiver is filled exactly once (to capacity), so z[h][u] of the
  // reference (tests/planning_reference.py:85-96) is stored per receiver.
  // (value, index) pairs travel through one reduction as value*128 + index
  // code whenever the counts leave 7 bits of room
  const bool packed_key = (int64_t)R * CAP < (1 << 24);
  if (wave == 0) {
    if (packed_key && R <= 16) {
      // One DPP row holds every rank: lane r keeps the balance of rank r and what
      // rank r receives.  No branch inside an iteration; the two reductions are
      // independent and interleave.
      const bool v0 = lane < R;
      int b0 = v0 ? s_gt[lane] - CAP : 0;
      int from = -1, quota = 0;
      for (int it = 0; it < R; ++it) {
        int kx = v0 ? b0 * 128 + (127 - lane) : INT32_MIN;  // max: first index wins ties
        int kn = v0 ? b0 * 128 + lane : INT32_MAX;          // min: first index wins ties
        kx = mep_row_max(kx);
        kn = mep_row_min(kn);
        const int hv2 = kx >> 7, h = 127 - (kx & 127);
        const int uv = kn >> 7, u = kn & 127;
        if (hv2 <= 0 || uv >= 0) break;
        const int move = -uv;
        b0 = lane == h ? b0 - move : b0;
        const bool recv = lane == u;
        b0 = recv ? 0 : b0;
        from = recv ? h : from;
        quota = recv ? move : quota;
      }
      if (v0) { s_from[lane] = from; s_quota[lane] = quota; }
    } else {
      // lane r keeps the balance of rank r (and of rank r + 64)
      int b0 = lane < R ? s_gt[lane] - CAP : 0;
      int b1 = lane + 64 < R ? s_gt[lane + 64] - CAP : 0;
      const bool v0 = lane < R, v1 = lane + 64 < R;
      for (int it = 0; it < R; ++it) {
        int hv2, h, uv, u;
        if (packed_key) {
          int kx = v0 ? b0 * 128 + (127 - lane) : INT32_MIN;
          int kn = v0 ? b0 * 128 + lane : INT32_MAX;
          if (v1) { kx = mep_imax(kx, b1 * 128 + (63 - lane)); kn = mep_imin(kn, b1 * 128 + lane + 64); }
          kx = mep_wave_max(kx);
          kn = mep_wave_min(kn);
          hv2 = kx >> 7; h = 127 - (kx & 127);
          uv = kn >> 7; u = kn & 127;
        } else {
          int mx = v0 ? b0 : INT32_MIN, mxi = lane;
          if (v1 && b1 > mx) { mx = b1; mxi = lane + 64; }
          int mn = v0 ? b0 : INT32_MAX, mni = lane;
          if (v1 && b1 < mn) { mn = b1; mni = lane + 64; }
          mep_wave_argmax_first(mx, mxi, hv2, h);
          mep_wave_argmin_first(mn, mni, uv, u);
        }
        if (hv2 <= 0 || uv >= 0) break;
        const int move = -uv;
        if (lane == (h & 63)) { if (h < 64) b0 -= move; else b1 -= move; }
        if (lane == (u & 63)) { if (u < 64) b0 = 0; else b1 = 0; }
        if (lane == 0) { s_from[u] = h; s_quota[u] = move; }
      }
    }
  }
  // the first loads of the next part of the histogram, before this one's atomics
  if (count_b && spread) hist_load(hb, hb1, hb2, tb, NB);
  // Lanes of my wave before me holding the same expert (one ballot per key bit);
  // the first of them adds the wave's count to the expert's per-wave byte.  Wave 0
  // does this in the next phase, where it has nothing else to do.
  if ((unsigned)e >= (unsigned)E) e = -1;  // invalid id: becomes an entry that nobody copies
  int pos = 0;
  auto rank_in_wave = [&]() {
    uint64_t same = __ballot(e >= 0);
    const int nbits = 32 - __clz(E - 1 > 0 ? E - 1 : 1);
    for (int b = 0; b < nbits; ++b) {
      const bool bit = (e >> b) & 1;
      const uint64_t bb = __ballot(bit);
      same &= bit ? bb : ~bb;
    }
    if (e >= 0) {
      pos = __popcll(same & mep_lanes_lt());
      if (pos == 0)
        atomicAdd(&s_wcnt[e * W4 + (wave >> 2)], __popcll(same) << (8 * (wave & 3)));
    }
  };
  if (count_a) {
    rank_in_wave();
    hist_part(ha, v0, hb1, ta, NA);
    for (int i = c0 + ta; i < head_end; i += NA) atomicAdd(bin(topk[i]), 1);
    for (int i = tail_start + ta; i < c1; i += NA) atomicAdd(bin(topk[i]), 1);
  }
  __syncthreads();

  // ---- which tokens of which expert migrate: one wave per home group -----
  // An (expert, receiver) pair is touched at most once (every step exhausts
  // the expert or the receiver), so alloc[e][d] is a plain store and what
  // stays home is written once at the end.
  // (waves 1..R, so that wave 0 is free)
  if (wave == 0) rank_in_wave();
  if (count_b && spread) {
    hist_load(hc, hb2, v1, tb, NB);
    hist_part(hb, hb1, hb2, tb, NB);
  }
  for (int h = (wave + NW - 1) % NW; h < R; h += NW) {
    const int es = h * epn;
    if (packed_key && R <= 64 && epn <= 64) {
      // lane r keeps the open quota of receiver r, lane le what is left of
      // the home's expert le
      int q = (lane < R && s_from[lane] == h) ? s_quota[lane] : 0;
      int rem = lane < epn ? s_rem[es + lane] : -1;
      if (R <= 16) {  // the receivers fit one DPP row; the two reductions interleave
        for (int it = 0; it < R + epn; ++it) {
          int kq = q > 0 ? q * 128 + (127 - lane) : INT32_MIN;
          int kr = rem >= 0 ? rem * 64 + (63 - lane) : INT32_MIN;
          kq = mep_row_max(kq);
          kr = mep_wave_max(kr);
          const int best = kr >> 6, le = 63 - (kr & 63);
          if (kq < 0 || best <= 0) break;  // no open quota, or nothing left to move
          const int quota = kq >> 7, d = 127 - (kq & 127);
          const int take = best < quota ? best : quota;
          if (lane == le) {
            rem -= take;
            alloc[(es + le) * R + d] = take;
          }
          q = lane == d ? q - take : q;
        }
      } else {
        for (int it = 0; it < R + epn; ++it) {
          int kq = q > 0 ? q * 128 + (127 - lane) : INT32_MIN;
          kq = mep_wave_max(kq);
          if (kq < 0) break;  // no open quota
          const int quota = kq >> 7, d = 127 - (kq & 127);
          int kr = rem >= 0 ? rem * 64 + (63 - lane) : INT32_MIN;
          kr = mep_wave_max(kr);
          const int best = kr >> 6, le = 63 - (kr & 63);
          if (best <= 0) break;
          const int take = best < quota ? best : quota;
          if (lane == le) {
            rem -= take;
            alloc[(es + le) * R + d] = take;
          }
          if (lane == d) q -= take;
        }
      }
      if (lane < epn) alloc[(es + lane) * R + h] = rem;
      continue;
    }
    for (int it = 0; it < R + epn; ++it) {
      int q = INT32_MIN, qi = INT32_MAX;
      for (int d = lane; d < R; d += 64) {
        const int v = (s_from[d] == h) ? s_quota[d] : 0;
        if (v > q) { q = v; qi = d; }
      }
      int quota, d;
      mep_wave_argmax_first(q, qi, quota, d);
      if (quota <= 0) break;
      int rm = INT32_MIN, ri = INT32_MAX;
      for (int le = lane; le < epn; le += 64) {
        const int v = s_rem[es + le];
        if (v > rm) { rm = v; ri = le; }
      }
      int rem, le;
      mep_wave_argmax_first(rm, ri, rem, le);
      if (rem <= 0) break;
      const int take = rem < quota ? rem : quota;
      if (lane == 0) {
        const int ex = es + le;
        alloc[ex * R + d] = take;
        alloc[ex * R + h] = rem - take;
        s_rem[ex] = rem - take;
        s_quota[d] = quota - take;
      }
      mep_wave_sync();
    }
  }
  __syncthreads();

  // ---- layout of every destination: one wave per destination -------------
  if (count_b && spread) hist_part(hc, hb2, v1, tb, NB);
  const bool tp_pow2 = (tp & (tp - 1)) == 0;
  for (int d = (wave + NW - 1) % NW; d < R; d += NW) {
    const int lo = d * epn;
    // Whatever is on d from elsewhere comes from the one home group that feeds d
    // (s_from): its experts with tokens allocated to d, in ascending order.
    const int hs = s_from[d] * epn;  // negative: d receives nothing
    const int cnt_own = lane < epn ? alloc[(lo + lane) * R + d] : 0;  // read early: used after the scan
    int nremote = 0;
    if (hs >= 0) {
      for (int c0 = 0; c0 < epn; c0 += 64) {
        const int ex = hs + c0 + lane;
        const bool sel = c0 + lane < epn && alloc[ex * R + d] > 0;
        const uint64_t m = __ballot(sel);
        if (sel) {
          const int slot = nremote + __popcll(m & mep_lanes_lt());
          if (slot < epn) s_etc[lo + slot] = ex;
        }
        nremote += __popcll(m);
      }
      if (lane == 0 && nremote) atomicAdd(&s_stat1[s_from[d]], nremote);
    }
    for (int b = nremote + lane; b < epn; b += 64) s_etc[lo + b] = -1;
    if (lane == 0) s_nrem[d] = nremote;
    mep_wave_sync();
    if (writer && blockIdx.y == 0)
      for (int b = lane; b < epn; b += 64) a.etc[lo + b] = s_etc[lo + b];
    const bool mine = writer && d == rank;
    int* cu = a.cu_seqlens + (size_t)blockIdx.y * 2 * epn;
    int* zf = a.zero_fill + (size_t)blockIdx.y * 4 * epn;
    int running = 0;
    for (int c = 0; c < 2 * epn; c += 64) {
      const int g = c + lane;
      int eid = -1, cnt = 0;
      if (g < epn) eid = lo + g;
      else if (g < 2 * epn) eid = s_etc[lo + g - epn];
      if (c == 0 && g < epn) cnt = cnt_own;
      else if (eid >= 0) cnt = alloc[eid * R + d];
      const int padded = tp_pow2 ? (cnt + tp - 1) & ~(tp - 1) : ((cnt + tp - 1) / tp) * tp;
      const int incl = mep_wave_incl_scan(padded);
      const int start = running + incl - padded;
      if (cnt > 0) base[eid * R + d] = d * NvS + start;
      if (mine && g < 2 * epn) {
        cu[g] = start + padded;
        zf[2 * g] = padded > cnt ? start + cnt : 0;
        zf[2 * g + 1] = padded - cnt;
      }
      running += __builtin_amdgcn_readlane(incl, 63);
    }
  }
  __syncthreads();

  // ---- my slice of the rank's entries -------------------------------------
  // An entry with an invalid expert id gets destination rank R: dispatch and
  // combine skip such entries (they never write or read outside the R shards),
  // the duplicate-group builder matches no rank to it.
  int* dst = a.dst + (size_t)blockIdx.y * N;
  int dv = R * NvS, dest = -1;  // fits: the host requires R*NvS <= INT32_MAX
  if (e >= 0) {
    // entries of my expert in the waves before mine: one byte per wave, W4 words
    // per expert; with my position in my own wave, my number within the slice
    unsigned words[W4];
#pragma unroll
    for (int w4 = 0; w4 < W4; ++w4) words[w4] = (unsigned)s_wcnt[e * W4 + w4];
    // entries of expert e are numbered over (source rank, flat index) and cut
    // into the destinations' allocations in rank order
    const int counted = s_hist[e], mine_all = s_own[e];
    int g = s_prev[e] + pos;
    int4 c4[4];
    const bool small_row = (R & 3) == 0 && R <= 16;
    const int4* row = (const int4*)(alloc + e * R);  // 16-byte aligned when R % 4 == 0: tables start aligned
    if (small_row) {
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        if (q4 * 4 < R) c4[q4] = row[q4];
    }
#pragma unroll
    for (int w4 = 0; w4 < W4; ++w4) {
      const int m = wave - 4 * w4;  // bytes of this word that belong to earlier waves
      const unsigned mask = m >= 4 ? 0xffffffffu : (m <= 0 ? 0u : (1u << (8 * m)) - 1u);
      g = (int)__builtin_amdgcn_sad_u8(words[w4] & mask, 0u, (unsigned)g);
    }
    if (fwd) {
      g += counted;
    } else {  // the rank's total less my slice less what follows it
      unsigned in_slice = 0;
#pragma unroll
      for (int w4 = 0; w4 < W4; ++w4) in_slice = __builtin_amdgcn_sad_u8(words[w4], 0u, in_slice);
      g += mine_all - (int)in_slice - counted;
    }
    if (small_row) {
      // whole row read at once, then a search without branches
      bool found = false;
      dest = R - 1;
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4)
        if (q4 * 4 < R) {
          const int cs[4] = {c4[q4].x, c4[q4].y, c4[q4].z, c4[q4].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const bool hit = !found && (g < cs[j] || q4 * 4 + j == R - 1);
            dest = hit ? q4 * 4 + j : dest;
            found = found || hit;
            g = found ? g : g - cs[j];
          }
        }
    } else if ((R & 3) == 0) {
      bool found = false;
      dest = 0;
      for (int d4 = 0; d4 < R && !found; d4 += 4) {
        const int4 r4 = row[d4 >> 2];
        const int cs[4] = {r4.x, r4.y, r4.z, r4.w};
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (!found) {
            if (g < cs[j] || d4 + j == R - 1) { dest = d4 + j; found = true; }
            else g -= cs[j];
          }
      }
    } else {
      for (dest = 0; dest < R - 1; ++dest) {
        const int c = alloc[e * R + dest];
        if (g < c) break;
        g -= c;
      }
    }
    dv = base[e * R + dest] + g;
  }
  // a later entry of a token on a destination rank that an earlier entry of the
  // token already has is a duplicate: stored as -dv - 1
  bool dup = false;
  if (16 % K == 0) {
    // the K entries of a token sit in one DPP row: compare along the row
    const int k = tid & (K - 1);
#define MEP_DUP_STEP(J)                                                                      \
  if (J < K) {                                                                               \
    const int pj = __builtin_amdgcn_update_dpp(-2, dest, 0x110 + J, 0xf, 0xf, false);        \
    dup |= J <= k && dest >= 0 && pj == dest;                                                \
  }
    MEP_DUP_STEP(1) MEP_DUP_STEP(2) MEP_DUP_STEP(3) MEP_DUP_STEP(4) MEP_DUP_STEP(5)
    MEP_DUP_STEP(6) MEP_DUP_STEP(7) MEP_DUP_STEP(8) MEP_DUP_STEP(9) MEP_DUP_STEP(10)
    MEP_DUP_STEP(11) MEP_DUP_STEP(12) MEP_DUP_STEP(13) MEP_DUP_STEP(14) MEP_DUP_STEP(15)
#undef MEP_DUP_STEP
  } else {
    s_cd[tid] = dest;
    __syncthreads();
    const int k = tid % K;
    for (int j = tid - k; j < tid; ++j) dup |= (dest >= 0 && s_cd[j] == dest);
  }
  if (tid < n) dst[e0 + tid] = dup ? -dv - 1 : dv;
  if (writer && tid == 0) {
    a.remote_stats[2 * blockIdx.y] = s_nrem[rank];
    a.remote_stats[2 * blockIdx.y + 1] = s_stat1[rank];
  }
}

size_t plan_lds_bytes(int nt, int E, int R, bool lds_tables) {
  const int nw = nt / MEP_WAVE;
  const int w4 = (nw + 3) / 4;
  size_t ints = (size_t)(6 + w4) * E + 6 * (size_t)R + (size_t)nt;
  if (lds_tables) ints += 2 * (size_t)E * R;
  return ints * sizeof(int);
}

constexpr size_t kLdsDefaultLimit = 64 * 1024;   // available to any kernel without opting in
constexpr size_t kLdsOptInLimit = 160 * 1024;    // gfx950: what one workgroup can address

struct PlanConfig {
  int nt;
  bool lds_tables;
  bool opt_in;  // needs more dynamic LDS than the default limit
  size_t lds_bytes;
  int tok_per_wg;
  int groups;
};

// 0 on success
int plan_config(int S, int K, int E, int R, PlanConfig* c) {
  c->opt_in = false;
  if (plan_lds_bytes(1024, E, R, true) <= kLdsDefaultLimit) {
    c->nt = 1024; c->lds_tables = true;
  } else if (plan_lds_bytes(256, E, R, true) <= kLdsDefaultLimit) {
    c->nt = 256; c->lds_tables = true;
  } else if (plan_lds_bytes(256, E, R, false) <= kLdsDefaultLimit) {
    c->nt = 256; c->lds_tables = false;
  } else if (plan_lds_bytes(256, E, R, false) <= kLdsOptInLimit) {
    c->nt = 256; c->lds_tables = false; c->opt_in = true;
  } else {
    return MEP_ERR_UNSUPPORTED;
  }
  c->lds_bytes = plan_lds_bytes(c->nt, E, R, c->lds_tables);
  c->tok_per_wg = c->nt / K;
  c->groups = (S + c->tok_per_wg - 1) / c->tok_per_wg;
  return MEP_OK;
}

}  // namespace

extern "C" size_t mep_plan_scratch_bytes(int S, int K, int E, int R, int nranks) {
  PlanConfig c;
  if (S <= 0 || K <= 0 || K > 32 || E <= 0 || R <= 0 || nranks <= 0) return 0;
  if (plan_config(S, K, E, R, &c) != MEP_OK || c.lds_tables) return 0;
  return (size_t)c.groups * nranks * 2 * (size_t)E * R * sizeof(int);
}

namespace {
int plan_launch(const int32_t* tpe_RE, const int32_t* topk_nSK, int rank0, int nranks, int S, int K,
                int E, int R, int token_padding, int NvS, int32_t* dst, int32_t* cu_seqlens,
                int32_t* experts_to_copy, int32_t* zero_fill, int32_t* remote_stats, void* scratch,
                size_t scratch_bytes, const void* warm, size_t warm_bytes, void* stream) {
  MEP_REQUIRE(tpe_RE && topk_nSK && dst && cu_seqlens && experts_to_copy && zero_fill &&
                  remote_stats, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(S > 0 && K > 0 && E > 0 && R > 0 && token_padding > 0 && NvS > 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(E % R == 0, MEP_ERR_INVALID_ARG);
  MEP_REQUIRE(nranks > 0 && rank0 >= 0 && rank0 + nranks <= R, MEP_ERR_INVALID_ARG);
  // encoding bounds of the reference (moonep/planning.py:1231-1255, api.py:286-290)
  MEP_REQUIRE(K <= 32 && R <= 128, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE((int64_t)S * K < INT32_MAX && (int64_t)S * K <= NvS, MEP_ERR_UNSUPPORTED);
  MEP_REQUIRE((int64_t)R * NvS <= INT32_MAX, MEP_ERR_UNSUPPORTED);
  PlanConfig c;
  int rc = plan_config(S, K, E, R, &c);
  if (rc != MEP_OK) return rc;
  if (!c.lds_tables) {
    const size_t need = (size_t)c.groups * nranks * 2 * (size_t)E * R * sizeof(int);
    MEP_REQUIRE(scratch && scratch_bytes >= need, MEP_ERR_SCRATCH);
    MEP_REQUIRE((uintptr_t)scratch % 16 == 0, MEP_ERR_ALIGNMENT);
  }
  PlanArgs a;
  a.tpe = tpe_RE; a.topk = topk_nSK; a.dst = dst; a.cu_seqlens = cu_seqlens;
  a.etc = experts_to_copy; a.zero_fill = zero_fill; a.remote_stats = remote_stats;
  a.scratch = (int*)scratch;
  a.rank0 = rank0; a.S = S; a.K = K; a.E = E; a.R = R; a.epn = E / R; a.tp = token_padding;
  a.NvS = NvS; a.tok_per_wg = c.tok_per_wg;
  a.groups = c.groups;
  a.warm = (const char*)warm;
  // never more than half of the 256 MB last-level cache: beyond that the read
  // only delays the planner and evicts itself
  constexpr size_t kWarmMax = (size_t)128 << 20;
  a.warm_vecs = warm ? (warm_bytes < kWarmMax ? warm_bytes : kWarmMax) / 16 : 0;
  // eight loads per thread and pass; 1024 threads of warming per CU that the
  // planning workgroups leave free (more gains nothing: 224 or 448 workgroups of
  // 1024 threads read 59 MB in the same 10.7 us)
  int warm_groups = 0;
  if (a.warm_vecs) {
    const size_t per_wg = (size_t)c.nt * 8;
    const size_t want = (a.warm_vecs + per_wg - 1) / per_wg;
    const int cus = mep_device_cu_count();
    if (cus <= 0) return MEP_ERR_INVALID_ARG;
    const int64_t room = ((int64_t)cus - ((int64_t)c.groups * nranks * c.nt + 1023) / 1024) * (1024 / c.nt);
    const size_t cap = room > 0 ? (size_t)room : 0;
    warm_groups = (int)(want < cap ? want : cap);
  }
  dim3 grid(c.groups + warm_groups, nranks);
  hipStream_t st = (hipStream_t)stream;
  // compile-time variants for the usual expert-parallel widths with top-8 routing
  // (7.3 us against 8.8 us for the generic kernel at R = 8)
  if (c.nt == 1024 && K == 8 && R == 8) {
    hipLaunchKernelGGL((plan_kernel<1024, true, 8, 8>), grid, dim3(1024), c.lds_bytes, st, a);
  } else if (c.nt == 1024 && K == 8 && R == 4) {
    hipLaunchKernelGGL((plan_kernel<1024, true, 4, 8>), grid, dim3(1024), c.lds_bytes, st, a);
  } else if (c.nt == 1024 && K == 8 && R == 16) {
    hipLaunchKernelGGL((plan_kernel<1024, true, 16, 8>), grid, dim3(1024), c.lds_bytes, st, a);
  } else if (c.nt == 1024) {
    hipLaunchKernelGGL((plan_kernel<1024, true>), grid, dim3(1024), c.lds_bytes, st, a);
  } else if (c.lds_tables) {
    hipLaunchKernelGGL((plan_kernel<256, true>), grid, dim3(256), c.lds_bytes, st, a);
  } else {
    if (c.opt_in) {  // more dynamic LDS than the default limit: opted in by mep_init_planner_kernels
      const int irc = mep_ensure_init();
      if (irc != MEP_OK) return irc;
    }
    hipLaunchKernelGGL((plan_kernel<256, false>), grid, dim3(256), c.lds_bytes, st, a);
  }
  return mep_launch_status();
}

}  // namespace

// LDS opt-in of the planner variant for very large expert counts, for the current device
int mep_init_planner_kernels() {
  MEP_RETURN_IF_HIP(hipFuncSetAttribute((const void*)plan_kernel<256, false>,
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsOptInLimit));
  return MEP_OK;
}

extern "C" int mep_plan_ranks(const int32_t* tpe_RE, const int32_t* topk_nSK, int rank0, int nranks,
                              int S, int K, int E, int R, int token_padding, int NvS, int32_t* dst,
                              int32_t* cu_seqlens, int32_t* experts_to_copy, int32_t* zero_fill,
                              int32_t* remote_stats, void* scratch, size_t scratch_bytes,
                              void* stream) {
  return plan_launch(tpe_RE, topk_nSK, rank0, nranks, S, K, E, R, token_padding, NvS, dst, cu_seqlens,
                     experts_to_copy, zero_fill, remote_stats, scratch, scratch_bytes, nullptr, 0,
                     stream);
}

extern "C" int mep_plan_warm(const int32_t* tpe_RE, const int32_t* topk_SK, int rank, int S, int K,
                             int E, int R, int token_padding, int NvS, int32_t* dst,
                             int32_t* cu_seqlens, int32_t* experts_to_copy, int32_t* zero_fill,
                             int32_t* remote_stats, void* scratch, size_t scratch_bytes,
                             const void* warm, size_t warm_bytes, void* stream) {
  MEP_REQUIRE(!warm || (uintptr_t)warm % 16 == 0, MEP_ERR_ALIGNMENT);
  return plan_launch(tpe_RE, topk_SK, rank, 1, S, K, E, R, token_padding, NvS, dst, cu_seqlens,
                     experts_to_copy, zero_fill, remote_stats, scratch, scratch_bytes, warm,
                     warm_bytes, stream);
}

extern "C" int mep_plan(const int32_t* tpe_RE, const int32_t* topk_SK, int rank, int S, int K,
                        int E, int R, int token_padding, int NvS, int32_t* dst,
                        int32_t* cu_seqlens, int32_t* experts_to_copy, int32_t* zero_fill,
                        int32_t* remote_stats, void* scratch, size_t scratch_bytes, void* stream) {
  return mep_plan_ranks(tpe_RE, topk_SK, rank, 1, S, K, E, R, token_padding, NvS, dst, cu_seqlens,
                        experts_to_copy, zero_fill, remote_stats, scratch, scratch_bytes, stream);
}
