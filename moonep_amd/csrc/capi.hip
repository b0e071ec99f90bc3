// Version and error strings of the C ABI, and the CU-limited stream behind
// Buffer(num_sms=...).
#include "mep_common.h"

#include <vector>

// major*10000 + minor*100 + patch.  200: mep_grad_reduce takes `flags` before `stream`,
// mep_dispatch_epilogue / mep_combine_prologue take `max_cus`, mep_init and mep_prefetch_pull exist.
extern "C" int mep_version(void) { return 200; }

int mep_ensure_init() {
  static std::atomic<uint64_t> done{0};
  int dev = 0;
  MEP_RETURN_IF_HIP(hipGetDevice(&dev));
  MEP_REQUIRE(dev >= 0 && dev < 64, MEP_ERR_UNSUPPORTED);
  const uint64_t bit = 1ull << dev;
  if (done.load(std::memory_order_acquire) & bit) return MEP_OK;
  int rc = mep_init_planner_kernels();
  if (rc == MEP_OK) rc = mep_init_stream_kernels();
  if (rc == MEP_OK) rc = mep_init_gemm_kernels();
  if (rc == MEP_OK) done.fetch_or(bit, std::memory_order_release);  // racing threads set the same attributes
  return rc;
}

extern "C" int mep_init(void) { return mep_ensure_init(); }

extern "C" const char* mep_strerror(int code) {
  switch (code) {
    case MEP_OK: return "ok";
    case MEP_ERR_INVALID_ARG: return "invalid argument (null pointer, size or rank out of range)";
    case MEP_ERR_UNSUPPORTED: return "shape not supported by the gfx950 kernels";
    case MEP_ERR_SCRATCH: return "scratch buffer missing or too small";
    case MEP_ERR_ALIGNMENT: return "pointer or stride not 16-byte aligned";
    case MEP_ERR_STATIC_LIMIT:
      return "input exceeds the fixed scratch of the allocation-free entry point (use the variant "
             "that takes a scratch buffer)";
    default: break;
  }
  if (code > 0) return hipGetErrorString((hipError_t)code);
  return "unknown error";
}

namespace {

// one record per workgroup: XCC id in bits 16..19, the SE / SH / CU fields of HW_ID in bits 8..15
__global__ void cu_census_kernel(uint32_t* out) {
  if (threadIdx.x == 0) {
    uint32_t hw, xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    out[blockIdx.x] = ((xcc & 0xfu) << 16) | (hw & 0xff00u);
  }
}

}  // namespace

extern "C" int mep_stream_create_limited(int num_cus, void** stream_out) {
  MEP_REQUIRE(stream_out, MEP_ERR_INVALID_ARG);
  int dev = 0, cus = 0;
  MEP_RETURN_IF_HIP(hipGetDevice(&dev));
  MEP_RETURN_IF_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
  MEP_REQUIRE(num_cus >= 1 && num_cus <= cus, MEP_ERR_INVALID_ARG);
  // The low num_cus bits: the runtime spreads consecutive bits over the XCDs (32 bits = 4 CUs on
  // each of 8 XCDs).  Only such contiguous masks are used: they were run from 16 to 256 CUs.
  std::vector<uint32_t> mask((size_t)(cus + 31) / 32, 0u);
  for (int i = 0; i < num_cus; ++i) mask[i / 32] |= 1u << (i % 32);
  hipStream_t st = nullptr;
  MEP_RETURN_IF_HIP(hipExtStreamCreateWithCUMask(&st, (uint32_t)mask.size(), mask.data()));
  *stream_out = (void*)st;
  return MEP_OK;
}

extern "C" int mep_stream_destroy(void* stream) {
  MEP_REQUIRE(stream, MEP_ERR_INVALID_ARG);
  MEP_RETURN_IF_HIP(hipStreamDestroy((hipStream_t)stream));
  return MEP_OK;
}

extern "C" int mep_stream_cu_census(uint32_t* out, int nblocks, void* stream) {
  MEP_REQUIRE(out && nblocks > 0, MEP_ERR_INVALID_ARG);
  hipLaunchKernelGGL(cu_census_kernel, dim3(nblocks), dim3(64), 0, (hipStream_t)stream, out);
  return mep_launch_status();
}
