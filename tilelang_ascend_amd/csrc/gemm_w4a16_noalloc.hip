// tlq_gemm_w4a16_noalloc: the weight-only GEMM of tlq_gemm_w4a16_ws for callers that cannot allocate device memory
// (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The workspace that
// tlq_gemm_w4a16_ws takes from its caller -- fp32 partial sums of the K slices, or the dequantised weight matrix of
// the two-pass path -- lives in a file-scope device array instead.  Each GPU the library runs on holds its own copy
// of that array, at its own address, until the process ends; the address is looked up once per device.
//
// The array keeps the previous call's contents.  Nothing here needs it cleared: every K slice writes its whole
// partial tile before the reduction reads it, and the two-pass path writes the whole dequantised matrix before the
// GEMM reads it.  Calls that overlap on one GPU (different streams, different threads) share the array and race.
#include <mutex>

#include "tlq_common.h"

namespace tlq {
namespace {

static __device__ __align__(256) uint8_t scratch[TLQ_NOALLOC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
uint8_t* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, null until looked up
std::mutex g_scratch_mutex;

// Device address of the array on the current GPU.  In host code the name `scratch` is only a handle for
// hipGetSymbolAddress, never a pointer a kernel could use.
int scratch_of_current_device(uint8_t** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    set_error("tlq_gemm_w4a16_noalloc: hipGetDevice failed: %s", hipGetErrorString(e));
    return 1;
  }
  if (dev < 0 || dev >= kMaxDevices) {
    set_error("tlq_gemm_w4a16_noalloc: device index %d outside 0..%d", dev, kMaxDevices - 1);
    return 1;
  }
  std::lock_guard<std::mutex> hold(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr) {
      set_error("tlq_gemm_w4a16_noalloc: cannot find the built-in scratch array on device %d: %s", dev, hipGetErrorString(e));
      return 1;
    }
    g_scratch_ptr[dev] = (uint8_t*)p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

}  // namespace
}  // namespace tlq

using namespace tlq;

extern "C" {

int tlq_gemm_w4a16_noalloc_init(void) {
  uint8_t* p = nullptr;
  return scratch_of_current_device(&p);
}

int tlq_gemm_w4a16_noalloc(const void* A, const void* w_packed, const void* scales, const void* zeros, void* C, int64_t M,
                           int64_t N, int64_t K, int64_t group, float zero_scalar, int in_dtype, int out_dtype, int algo,
                           void* stream) {
  // The array must hold what the preferred kernel for this shape needs, or at least what the next best one does (the
  // call then equals tlq_gemm_w4a16_ws with a workspace of TLQ_NOALLOC_SCRATCH_BYTES bytes, which takes what fits).
  int64_t need = tlq_w4a16_workspace_bytes(M, N, K);
  if (need > (int64_t)TLQ_NOALLOC_SCRATCH_BYTES) need = tlq_w4a16_workspace_bytes_min(M, N, K);
  // Not even that: the kernels that need no scratch at all (the fused tile kernel for large M) take the problem, as
  // tlq_gemm_w4a16_ws does when it is handed no workspace -- a caller who cannot allocate has nowhere else to go.
  if (need > (int64_t)TLQ_NOALLOC_SCRATCH_BYTES)
    return tlq_gemm_w4a16_ws(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, algo, nullptr, 0, stream);
  uint8_t* ws = nullptr;
  if (scratch_of_current_device(&ws)) return 1;
  // from here on only `ws`, the device address, stands for the array
  return tlq_gemm_w4a16_ws(A, w_packed, scales, zeros, C, M, N, K, group, zero_scalar, in_dtype, out_dtype, algo, ws,
                           (int64_t)TLQ_NOALLOC_SCRATCH_BYTES, stream);
}

}  // extern "C"
