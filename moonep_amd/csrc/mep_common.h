// Shared device/host helpers for the MoonEP hot-path kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/moonep_hip.h"

#define MEP_WAVE 64

// ---------------------------------------------------------------------------
// host-side launch check: C entry points never throw and never exit
// ---------------------------------------------------------------------------
#define MEP_RETURN_IF_HIP(expr)                         \
  do {                                                  \
    hipError_t _e = (expr);                             \
    if (_e != hipSuccess) return (int)_e;               \
  } while (0)

#define MEP_REQUIRE(cond, code) \
  do {                          \
    if (!(cond)) return (code); \
  } while (0)

static inline int mep_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? MEP_OK : (int)e;
}

// Kernels that use more dynamic LDS than the 64 KB a kernel gets without asking must be
// opted in with hipFuncSetAttribute, per device, and not from inside a stream capture.
// Each source file opts its own kernels in for the current device; mep_ensure_init runs all
// of them once per device (mep_init() is its exported name).  Launch sites of such kernels
// call it too, so a device that nobody initialised still works outside capture.
int mep_init_planner_kernels();
int mep_init_stream_kernels();
int mep_init_gemm_kernels();
int mep_ensure_init();

// CUs of the current device, asked once per device (-1 when the runtime cannot tell)
static inline int mep_device_cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -1;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      return -1;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

#if defined(__HIPCC__)

// ---------------------------------------------------------------------------
// wave64 primitives
// ---------------------------------------------------------------------------
__device__ __forceinline__ int mep_lane() { return __lane_id(); }

__device__ __forceinline__ uint64_t mep_lanes_lt() {
  return (1ull << mep_lane()) - 1ull;
}

// Orders this wave's LDS/global accesses around a point where lanes exchange
// data through memory.  All lanes of a wave run in lock step, so no hardware
// barrier is needed; the fences keep the compiler from moving accesses.
__device__ __forceinline__ void mep_wave_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// DPP row-shift / row-broadcast reduction; the full result lands in lane 63
// and is broadcast through a scalar register.
#define MEP_DPP_STEP(OP, v, ident, ctrl, rowmask)                                   \
  v = OP(v, __builtin_amdgcn_update_dpp((ident), (v), (ctrl), (rowmask), 0xf, false))

__device__ __forceinline__ int mep_imax(int a, int b) { return a > b ? a : b; }
__device__ __forceinline__ int mep_imin(int a, int b) { return a < b ? a : b; }
__device__ __forceinline__ int mep_iadd(int a, int b) { return a + b; }

__device__ __forceinline__ int mep_wave_max(int v) {
  const int id = INT32_MIN;
  MEP_DPP_STEP(mep_imax, v, id, 0x111, 0xf);  // row_shr:1
  MEP_DPP_STEP(mep_imax, v, id, 0x112, 0xf);  // row_shr:2
  MEP_DPP_STEP(mep_imax, v, id, 0x114, 0xf);  // row_shr:4
  MEP_DPP_STEP(mep_imax, v, id, 0x118, 0xf);  // row_shr:8
  MEP_DPP_STEP(mep_imax, v, id, 0x142, 0xa);  // row_bcast:15 -> rows 1,3
  MEP_DPP_STEP(mep_imax, v, id, 0x143, 0xc);  // row_bcast:31 -> rows 2,3
  return __builtin_amdgcn_readlane(v, 63);
}

__device__ __forceinline__ int mep_wave_min(int v) {
  const int id = INT32_MAX;
  MEP_DPP_STEP(mep_imin, v, id, 0x111, 0xf);
  MEP_DPP_STEP(mep_imin, v, id, 0x112, 0xf);
  MEP_DPP_STEP(mep_imin, v, id, 0x114, 0xf);
  MEP_DPP_STEP(mep_imin, v, id, 0x118, 0xf);
  MEP_DPP_STEP(mep_imin, v, id, 0x142, 0xa);
  MEP_DPP_STEP(mep_imin, v, id, 0x143, 0xc);
  return __builtin_amdgcn_readlane(v, 63);
}

// The same over the first 16 lanes only (one DPP row): for tables of at most
// 16 entries; lanes past the table must hold the identity.
__device__ __forceinline__ int mep_row_max(int v) {
  const int id = INT32_MIN;
  MEP_DPP_STEP(mep_imax, v, id, 0x111, 0xf);
  MEP_DPP_STEP(mep_imax, v, id, 0x112, 0xf);
  MEP_DPP_STEP(mep_imax, v, id, 0x114, 0xf);
  MEP_DPP_STEP(mep_imax, v, id, 0x118, 0xf);
  return __builtin_amdgcn_readlane(v, 15);
}

__device__ __forceinline__ int mep_row_min(int v) {
  const int id = INT32_MAX;
  MEP_DPP_STEP(mep_imin, v, id, 0x111, 0xf);
  MEP_DPP_STEP(mep_imin, v, id, 0x112, 0xf);
  MEP_DPP_STEP(mep_imin, v, id, 0x114, 0xf);
  MEP_DPP_STEP(mep_imin, v, id, 0x118, 0xf);
  return __builtin_amdgcn_readlane(v, 15);
}

// Inclusive prefix sum across the wave (lane i gets v_0 + ... + v_i).
__device__ __forceinline__ int mep_wave_incl_scan(int v) {
  MEP_DPP_STEP(mep_iadd, v, 0, 0x111, 0xf);
  MEP_DPP_STEP(mep_iadd, v, 0, 0x112, 0xf);
  MEP_DPP_STEP(mep_iadd, v, 0, 0x114, 0xf);
  MEP_DPP_STEP(mep_iadd, v, 0, 0x118, 0xf);
  MEP_DPP_STEP(mep_iadd, v, 0, 0x142, 0xa);
  MEP_DPP_STEP(mep_iadd, v, 0, 0x143, 0xc);
  return v;
}

// (max value, smallest index holding it); idx must be >= 0 and valid lanes
// pass their candidate, idle lanes pass (INT32_MIN, INT32_MAX).
__device__ __forceinline__ void mep_wave_argmax_first(int v, int idx, int& best, int& best_idx) {
  best = mep_wave_max(v);
  best_idx = mep_wave_min(v == best ? idx : INT32_MAX);
}

__device__ __forceinline__ void mep_wave_argmin_first(int v, int idx, int& best, int& best_idx) {
  best = mep_wave_min(v);
  best_idx = mep_wave_min(v == best ? idx : INT32_MAX);
}

// ---------------------------------------------------------------------------
// bf16 <-> fp32 on raw bit patterns
// ---------------------------------------------------------------------------
__device__ __forceinline__ float mep_bf16_lo(uint32_t packed) {
  return __uint_as_float(packed << 16);
}
__device__ __forceinline__ float mep_bf16_hi(uint32_t packed) {
  return __uint_as_float(packed & 0xffff0000u);
}

// Round to nearest even; NaN maps to the canonical quiet NaN 0x7fc0.
__device__ __forceinline__ uint32_t mep_f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  return (f != f) ? 0x7fc0u : r;
}

__device__ __forceinline__ uint32_t mep_pack_bf16(float lo, float hi) {
  return mep_f32_to_bf16_bits(lo) | (mep_f32_to_bf16_bits(hi) << 16);
}

__device__ __forceinline__ float mep_round_bf16(float f) {
  return __uint_as_float(mep_f32_to_bf16_bits(f) << 16);
}

// 16-byte streaming accesses: rows are touched once, keep them out of the way
// of data that is reused.
typedef uint32_t mep_u4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ mep_u4 mep_ld16_stream(const void* p) {
  return __builtin_nontemporal_load((const mep_u4*)p);
}
__device__ __forceinline__ mep_u4 mep_ld16(const void* p) {
  return *(const mep_u4*)p;
}
__device__ __forceinline__ void mep_st16_stream(void* p, mep_u4 v) {
  __builtin_nontemporal_store(v, (mep_u4*)p);
}
// Store written through at system scope (sc0 sc1).  For long contiguous copy
// streams it measured up to 19 % faster than the nontemporal hint (expert
// weight prefetch); for scattered rows (dispatch, combine) it is no better.
// The s_nop belongs to the store: a store of more than 64 bits reads its data
// registers a few cycles after it issues, and the compiler, which cannot see
// into the asm, would otherwise be free to overwrite them with the very next
// VALU instruction (seen: an address computation landing in v[2:3] of a zero
// vector one instruction after the store, leaving address bits in memory).
__device__ __forceinline__ void mep_st16_through(void* p, mep_u4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 3" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void mep_st16(void* p, mep_u4 v) {
  *(mep_u4*)p = v;
}

#endif  // __HIPCC__
