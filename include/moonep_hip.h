/*
 * libmoonep_hip -- C ABI of the MI355X (gfx950) MoonEP per-rank hot path.
 *
 * The reference has no C FFI on this path: its boundary is one Python
 * launcher per kernel (launch_planning, launch_dispatch, ...), each of which
 * JIT-compiles a CuTe-DSL kernel and launches it on the current stream.
 * Every function below replaces one of those launchers; the cited
 * reference lines are the launcher (host side) and the kernel it starts.
 *
 * Conventions
 *  - plain pointers to DEVICE memory unless a parameter says "host";
 *    sizes and strides are in the unit named by the parameter;
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *    every call only enqueues work: no host synchronisation, no allocation,
 *    safe to record into a HIP graph;
 *  - return value: 0 = ok, negative = MEP_ERR_* (bad argument, nothing was
 *    launched), positive = the hipError_t of a failed launch;
 *    never throws, never exits;
 *  - the R expert-parallel ranks' buffers are addressed as base + rank *
 *    stride, so the same entry points serve one GPU emulating R ranks in
 *    local HBM and a symmetric heap of peer-mapped memory;
 *  - re-entrant for distinct buffers; calls that share output buffers must be
 *    ordered by the caller (same stream or events).
 */
#ifndef MOONEP_HIP_H
#define MOONEP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MEP_OK 0
#define MEP_ERR_INVALID_ARG (-1)   /* null pointer, non-positive size, rank out of range */
#define MEP_ERR_UNSUPPORTED (-2)   /* shape outside what the kernels handle        */
#define MEP_ERR_SCRATCH (-3)       /* scratch buffer missing or too small           */
#define MEP_ERR_ALIGNMENT (-4)     /* pointer/stride not 16-byte aligned            */
#define MEP_ERR_STATIC_LIMIT (-5)  /* input larger than the library's fixed scratch  */

/* dispatch flags */
#define MEP_DISPATCH_WRITE_DUPS 1u /* also copy rows of negative (duplicate) entries */
#define MEP_DISPATCH_NO_ZERO_FILL 2u

/* combine modes */
#define MEP_COMBINE_PRIMARIES 0 /* sum non-negative entries only (reference kernel)      */
#define MEP_COMBINE_ALL 1       /* sum all K entries, one rounding                         */
#define MEP_COMBINE_TWO_LEVEL 2 /* per-destination group sum -> bf16 -> sum (= reference
                                   prologue + combine, without modifying the shards)       */
#define MEP_COMBINE_WEIGHTED 3  /* sum over all K entries of weight_slot * row; product and
                                   sum rounded separately in fp32, one rounding to bf16.
                                   Not a reference mode (its combine is unweighted): the
                                   weighted top-k sum that callers otherwise apply on the
                                   expert side                                              */

/* major*10000 + minor*100 + patch.  200: mep_grad_reduce takes `flags` before `stream`,
 * mep_dispatch_epilogue / mep_combine_prologue take `max_cus` before `stream`; mep_init,
 * mep_prefetch_pull and mep_set_gemm_row_tile exist.  A binding written against another
 * version must refuse to load the library. */
int mep_version(void);
const char* mep_strerror(int code);

/*
 * Per-device set-up that must not happen under stream capture: opts every kernel that
 * uses more than 64 KB of dynamic LDS in (hipFuncSetAttribute).  Call it once per device,
 * with that device current, before the first launch that may be captured into a graph
 * (the Python binding calls it when it loads the library and when a Buffer is made).
 * Idempotent and thread-safe; launches on a device nobody initialised do it themselves,
 * which only works outside capture.  No counterpart in the reference (its kernels are
 * JIT-compiled per shape on first use, moonep/dispatch.py:704-720).
 */
int mep_init(void);

/*
 * A stream whose kernels run on at most `num_cus` compute units (a CU mask on
 * the stream's hardware queue: the low num_cus bits, which the runtime spreads
 * evenly over the XCDs).  This is what Buffer(num_sms=N) of the reference asks
 * for (moonep/api.py:438-451, README.md:13: communication on 32 SMs beside the
 * expert GEMMs): every mep_* call takes a stream, so launching the path on such
 * a stream bounds all of its kernels at once, whatever their grids.  Default
 * priority.  mep_stream_cu_census records, per workgroup of a small probe
 * kernel, which CU it ran on (XCC id << 16 | HW_ID bits 8..15): for checking.
 */
int mep_stream_create_limited(int num_cus, void** stream_out);
int mep_stream_destroy(void* stream);
int mep_stream_cu_census(uint32_t* out, int nblocks, void* stream);

/* Bytes of device scratch mep_plan / mep_plan_ranks need for `nranks` ranks
 * planned in one call (0 when the planner tables fit in LDS). */
size_t mep_plan_scratch_bytes(int S, int K, int E, int R, int nranks);

/*
 * Online redundant-expert planner for one rank.
 * Replaces launch_planning (reference moonep/planning.py:1258-1280) and
 * PlanningKernel (reference moonep/planning.py:328-1101); results equal the
 * reference oracle (reference tests/planning_reference.py:25-311) bit for bit.
 *   tpe_RE          [R,E]  tokens every source rank routes to every expert
 *   topk_SK         [S,K]  this rank's expert ids
 *   dst             [S*K]  out: dest_rank*NvS + slot; later entries of a token
 *                          on the same dest rank are stored as -(value)-1
 *   cu_seqlens      [2*epn] out: padded end offset of each group on `rank`
 *   experts_to_copy [R,epn] out: remote experts every rank hosts (-1 = free)
 *   zero_fill       [2*epn,2] out: (first padding row, padding rows) per group
 *   remote_stats    [2]    out: (remote experts hosted on this rank,
 *                          slots on other ranks that hold this rank's experts)
 * The src_info provenance scratch of the reference (planning.py:1036-1041)
 * is not produced; mep_build_dedup derives the duplicate groups from dst.
 */
int mep_plan(const int32_t* tpe_RE, const int32_t* topk_SK, int rank, int S, int K, int E,
             int R, int token_padding, int NvS, int32_t* dst, int32_t* cu_seqlens,
             int32_t* experts_to_copy, int32_t* zero_fill, int32_t* remote_stats,
             void* scratch, size_t scratch_bytes, void* stream);

/*
 * mep_plan that also warms the last-level cache.  No counterpart in the
 * reference: the planner is latency-bound and occupies a few CUs; the other
 * CUs meanwhile read the `warm_bytes` at `warm` (16-byte aligned; the token
 * rows the following mep_dispatch copies) once, so that dispatch reads them
 * from cache instead of mixing HBM reads into its write stream.  At most the
 * first 128 MiB are read.  warm == NULL is mep_plan.
 */
int mep_plan_warm(const int32_t* tpe_RE, const int32_t* topk_SK, int rank, int S, int K, int E,
                  int R, int token_padding, int NvS, int32_t* dst, int32_t* cu_seqlens,
                  int32_t* experts_to_copy, int32_t* zero_fill, int32_t* remote_stats,
                  void* scratch, size_t scratch_bytes, const void* warm, size_t warm_bytes,
                  void* stream);

/*
 * The same planner for ranks rank0 .. rank0+nranks-1 in one launch (one GPU
 * standing in for several ranks).  topk is [nranks,S,K]; dst, cu_seqlens,
 * zero_fill and remote_stats gain a leading [nranks] dimension;
 * experts_to_copy stays [R,epn].
 */
int mep_plan_ranks(const int32_t* tpe_RE, const int32_t* topk_nSK, int rank0, int nranks, int S,
                   int K, int E, int R, int token_padding, int NvS, int32_t* dst,
                   int32_t* cu_seqlens, int32_t* experts_to_copy, int32_t* zero_fill,
                   int32_t* remote_stats, void* scratch, size_t scratch_bytes, void* stream);

/*
 * Fused permute, source side.  Replaces launch_dispatch (reference
 * moonep/dispatch.py:838-983; kernel :268-692, rows :394-433, zero-fill
 * :467-497).  Copies hidden[s] to shards[drank][loff] for every non-negative
 * dst entry (all entries with MEP_DISPATCH_WRITE_DUPS), scatters w[s,k] to
 * wslots[drank][loff] for every entry, zero-fills rank's padding rows.
 *   hidden_SH [S,H] bf16;  w_SK [S,K] fp32 or NULL;
 *   shards: row r of rank d at shards + (d*shard_stride_rows + r)*H;
 *   wslots: slot r of rank d at wslots + d*wslot_stride + r  (NULL iff w_SK NULL)
 */
int mep_dispatch(const void* hidden_SH, const float* w_SK, const int32_t* dst,
                 const int32_t* zero_fill, void* shards, int64_t shard_stride_rows, float* wslots,
                 int64_t wslot_stride, int rank, int S, int H, int K, int R, int epn, int NvS,
                 int token_padding, unsigned flags, void* stream);

/*
 * Destination-side duplicate groups of `rank` from all ranks' dst.
 * Replaces the dedup builder warps of DispatchKernel (reference
 * moonep/dispatch.py:502-681).  Output order is deterministic (source rank,
 * token) -- the reference's own order is not stable and its tests compare
 * sets.  dst_RN [R, S*K]; dup_groups [NvS,3]; dup_loffs [NvS]; dup_counts [2].
 * scratch: at least mep_dedup_scratch_bytes(S, R) bytes.
 */
size_t mep_dedup_scratch_bytes(int S, int R);
int mep_build_dedup(const int32_t* dst_RN, int rank, int S, int K, int R, int NvS,
                    int32_t* dup_groups, int32_t* dup_loffs, int32_t* dup_counts, void* scratch,
                    size_t scratch_bytes, void* stream);

/*
 * mep_build_dedup without a scratch argument and without any allocation: the
 * builder's scratch is a fixed 1 MiB array in device memory that the library
 * itself holds (one copy per GPU, until the process ends).  It has no
 * counterpart in the reference; it is for callers that cannot allocate --
 * code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  Same outputs as mep_build_dedup, bit for bit.
 * Limit: mep_dedup_scratch_bytes(S, R) <= 1 MiB (S*R up to about 260 000
 * tokens); larger inputs return MEP_ERR_STATIC_LIMIT and launch nothing.
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU
 * (different streams or threads) race; order them.  The first call on a
 * device looks the array's address up (no allocation, no launch): make it
 * outside stream capture.
 */
int mep_build_dedup_static(const int32_t* dst_RN, int rank, int S, int K, int R, int NvS,
                           int32_t* dup_groups, int32_t* dup_loffs, int32_t* dup_counts,
                           void* stream);

/* primary row -> its duplicate rows, in place on one rank's shard.
 * Replaces launch_dispatch_epilogue (reference moonep/dispatch_epilogue.py:366-415).
 * max_cus > 0 bounds the launch to that many workgroups, hence compute units -- the
 * grid the reference sizes from MOONEP_NUM_SMS_DEDUP (moonep/api.py:100-120,
 * dispatch_epilogue.py:366-415); max_cus <= 0: the whole GPU.  Results do not depend on it. */
int mep_dispatch_epilogue(void* shard_NvS_H, const int32_t* dup_groups, const int32_t* dup_loffs,
                          const int32_t* dup_counts, int NvS, int H, int max_cus, void* stream);

/* fp32 sum of primary + duplicates -> bf16 -> primary row, in place.
 * Replaces launch_combine_prologue (reference moonep/combine_prologue.py:544-599).
 * max_cus as for mep_dispatch_epilogue. */
int mep_combine_prologue(void* shard_NvS_H, const int32_t* dup_groups, const int32_t* dup_loffs,
                         const int32_t* dup_counts, int NvS, int H, int max_cus, void* stream);

/*
 * Top-k unpermute + K-sum + weight gather.  Replaces launch_combine
 * (reference moonep/combine.py:565-654; kernel :210-511).  Unweighted fp32
 * accumulation from +0.0 in ascending k, one round-to-nearest-even to bf16.
 *   out_SH [S,H] bf16; out_SK [S,K] fp32 or NULL (then wslots may be NULL unless the
 *   mode is MEP_COMBINE_WEIGHTED)
 */
int mep_combine(const void* shards, int64_t shard_stride_rows, const float* wslots,
                int64_t wslot_stride, const int32_t* dst, void* out_SH, float* out_SK, int S,
                int H, int K, int R, int NvS, int mode, void* stream);

/*
 * Owner-push expert-weight prefetch for `ntensors` (3 or 6) tensors in one
 * launch.  Replaces launch_prefetch (reference moonep/prefetch.py:632-738;
 * kernel :227-470).  For every (d,b) with experts_to_copy[d,b] owned by
 * `rank`: pool_t[d][b] = local_t[expert - rank*epn], bytes copied verbatim.
 *   local, pool, rank_stride_bytes, bytes_per_expert: HOST arrays of length
 *   ntensors; pool_t slot (d,b) at pool[t] + d*rank_stride_bytes[t] +
 *   b*bytes_per_expert[t]; bytes_per_expert % 16 == 0.
 */
int mep_prefetch(int ntensors, const void* const* local, void* const* pool,
                 const int64_t* rank_stride_bytes, const int64_t* bytes_per_expert,
                 const int32_t* experts_to_copy, int rank, int epn, int R, void* stream);

/*
 * Pull view of the same prefetch: fills the occupied slots of ONE rank from all owners in
 * one launch, pool_t[rank][b] = owners_t[e / epn][e % epn] for every b with
 * e = experts_to_copy[rank, b] >= 0 -- what R owner pushes leave in rank's slots, and the
 * compact [2*epn, ...] compute view of a rank when one GPU holds every owner's experts.
 * The reference has no such launcher (its ranks push, moonep/prefetch.py:428-447); its
 * per-rank check of the result is tests/test_prefetch.py:448-464.
 *   owners[t]: expert le of owner o at owners[t] + o*owner_stride_bytes[t] +
 *   le*bytes_per_expert[t]; pool as in mep_prefetch; all four arrays are HOST arrays of
 *   length ntensors (3 or 6).  Slots with -1 and other ranks' slots are not touched.
 */
int mep_prefetch_pull(int ntensors, const void* const* owners, const int64_t* owner_stride_bytes,
                      void* const* pool, const int64_t* rank_stride_bytes,
                      const int64_t* bytes_per_expert, const int32_t* experts_to_copy, int rank,
                      int epn, int R, void* stream);

/*
 * fp32 slot reduction.  Replaces launch_grad_reduce (reference
 * moonep/grad_reduce.py:437-543; kernel :151-389).  local_grad[le] +=
 * reduce[src][b] over the slots holding expert rank*epn+le in (src,b)
 * ascending order; then reduce[rank][b] = 0 for every b with
 * experts_to_copy[rank,b] >= 0.  One launch.  elems_per_expert % 4 == 0.
 * The reference separates the two halves with a cross-rank barrier (every rank
 * has read before any rank clears, grad_reduce.py:369-372); a caller that drives
 * several ranks on one GPU gets the same by calling every rank with
 * MEP_REDUCE_NO_CLEAR first and then every rank with MEP_REDUCE_CLEAR_ONLY.
 */
#define MEP_REDUCE_NO_CLEAR 1u   /* sum only */
#define MEP_REDUCE_CLEAR_ONLY 2u /* zero the rank's own occupied slots only */
int mep_grad_reduce(float* local_grad, float* reduce_pool, int64_t rank_stride_elems,
                    const int32_t* experts_to_copy, int rank, int epn, int R,
                    int64_t elems_per_expert, unsigned flags, void* stream);

/*
 * Expert-side consumer of the dispatched rows: grouped bf16 GEMM on the matrix
 * cores, C = A * B[g]^T with fp32 accumulation.  No counterpart among the
 * reference's launchers: the reference leaves the expert FFN to the caller and
 * only fixes its contract (README.md:43-58: 2*epn groups delimited by
 * cu_seqlens, local experts then prefetch slots).
 *   A [M,K] bf16 rows (a rank's shard); cu_seqlens [G] padded end row of each
 *   group (device memory, as mep_plan wrote it; every end a multiple of 128,
 *   i.e. token_padding % 128 == 0); B [G,N,K] bf16, K contiguous; C [M,N] bf16.
 *   swiglu == 0: C = bf16(row_scale[m] * acc), row_scale [M] fp32 or NULL;
 *   swiglu != 0: C = bf16(silu(A*B[g]^T) * (A*B_up[g]^T)), B_up [G,N,K].
 * Rows at or beyond cu_seqlens[G-1] are not written.
 * M % 128 == 0, K % 64 == 0, N % 256 == 0 (N % 128 == 0 with swiglu).
 */
int mep_grouped_gemm_nt(const void* A, const void* B, const void* B_up, const int32_t* cu_seqlens,
                        int G, void* C, const float* row_scale, int M, int N, int K, int swiglu,
                        void* stream);

/* Test hook: force the row tiling of the grouped GEMMs (128 or 256 rows; 0 = choose by
 * shape, the default).  Process-wide.  No counterpart in the reference. */
int mep_set_gemm_row_tile(int rows);

/*
 * The same fused gate/up GEMM, storing the two pre-activations beside the
 * activation for a backward pass: C_act = bf16(silu(g) * u), C_gate = bf16(g),
 * C_up = bf16(u), g = A*B_gate[g]^T, u = A*B_up[g]^T.  C_gate / C_up may be
 * NULL.  No counterpart in the reference (the expert FFN is the caller's).
 */
int mep_grouped_swiglu_nt(const void* A, const void* B_gate, const void* B_up,
                          const int32_t* cu_seqlens, int G, void* C_act, void* C_gate, void* C_up,
                          int M, int N, int K, void* stream);

/*
 * C = bf16(A1 * B1[g]^T + A2 * B2[g]^T), one K loop over both pairs: the input
 * gradient of the gate/up pair (A1 = d gate, B1 = gate weights [G,N,K] with K
 * the hidden width of the experts, likewise the up pair).  Shapes as
 * mep_grouped_gemm_nt without swiglu.  No counterpart in the reference.
 */
int mep_grouped_gemm_dual_nt(const void* A1, const void* B1, const void* A2, const void* B2,
                             const int32_t* cu_seqlens, int G, void* C, int M, int N, int K,
                             void* stream);

/*
 * C = bf16(row_scale * A * B[g]) with the weights of a group given as [K, N]
 * (B [G,K,N] bf16, the output column contiguous): the input gradient of a
 * projection whose forward pass ran mep_grouped_gemm_nt on the same tensor, with
 * no transposed copy of the weights.  A [M,K], C [M,N], N % 256 == 0,
 * K % 64 == 0, M % 128 == 0; row_scale [M] fp32 or NULL.  No counterpart in
 * the reference.
 */
int mep_grouped_gemm_nn(const void* A, const void* B, const int32_t* cu_seqlens, int G, void* C,
                        const float* row_scale, int M, int N, int K, void* stream);

/*
 * C = bf16(A1 * B1[g] + A2 * B2[g]), weights [G,K,N], one K loop over both
 * pairs: the input gradient of the gate/up pair straight from the forward
 * pass's weight tensors.  No counterpart in the reference.
 */
int mep_grouped_gemm_dual_nn(const void* A1, const void* B1, const void* A2, const void* B2,
                             const int32_t* cu_seqlens, int G, void* C, int M, int N, int K,
                             void* stream);

/*
 * Weight gradients of the grouped GEMMs from TRANSPOSED activations:
 * C[g] [Ma,Nb] fp32 = At[:, rows of g] * Bt[:, rows of g]^T, At [Ma,ld] and
 * Bt [Nb,ld] bf16 with the rank's rows along the contiguous dimension; the rows
 * of group g are [cu_seqlens[g-1], cu_seqlens[g]).  A group without rows gets
 * zeros -- unless its index is >= skip_empty_from, then it is left unwritten
 * (pass the number of local experts when the slots that hold no expert are
 * never read; pass G to have every group written).  Ma % 128 == 0, Nb % 256 == 0, ld % 128 == 0, ld >= cu_seqlens[G-1].
 * The fp32 [G,Ma,Nb] result has the layout mep_grad_reduce sums (local experts
 * first, then the slots).  No counterpart in the reference.
 */
int mep_grouped_gemm_wgrad(const void* At, const void* Bt, const int32_t* cu_seqlens, int G,
                           float* C, int Ma, int Nb, int64_t ld, int skip_empty_from, void* stream);

/*
 * The same weight gradients from the activations as the passes hold them:
 * C[g] [Ma,Nb] fp32 = X1[rows of g]^T * X2[rows of g], X1 [rows,Ma] and X2
 * [rows,Nb] bf16 row-major -- no transposed copies.  Ma % 256 == 0,
 * Nb % 256 == 0, G even (MEP_ERR_UNSUPPORTED otherwise: transpose and call
 * mep_grouped_gemm_wgrad).  No counterpart in the reference.
 */
int mep_grouped_gemm_wgrad_tn(const void* X1, const void* X2, const int32_t* cu_seqlens, int G,
                              float* C, int Ma, int Nb, int64_t rows, int skip_empty_from, void* stream);

/*
 * [batch, rows, cols] -> [batch, cols, rows] of bf16 (any 2-byte element);
 * rows % 64 == 0, cols % 64 == 0, src != dst.  Feeds mep_grouped_gemm_wgrad
 * and the backward GEMMs, which want the other operand orientation.
 */
int mep_transpose_bf16(const void* src, void* dst, int batch, int rows, int cols, void* stream);

/*
 * Backward of the SwiGLU activation with the route weight applied,
 * h = s * silu(g) * u, from dh' = dy * W_down (gradient of the unscaled
 * activation), all [M,N] bf16, row_scale s [M] fp32 or NULL:
 *   dgate = s*dh' * u * silu'(g), dup = s*dh' * silu(g), hs = s * silu(g) * u
 *   (the operand of the down projection's weight gradient),
 *   dscale[m] = sum_n dh'[m,n] * silu(g)*u  (fp32, may be NULL).
 * Rows at or beyond cu_seqlens[G-1] come out as zeros.  N % 8 == 0.
 */
int mep_swiglu_bwd(const void* dh, const void* gate_pre, const void* up_pre, const float* row_scale,
                   const int32_t* cu_seqlens, int G, void* dgate, void* dup, void* hs, float* dscale,
                   int M, int N, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOONEP_HIP_H */
