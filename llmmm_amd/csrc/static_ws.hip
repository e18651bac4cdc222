// llmmm_fp8_gemm_static_ws: the FP8 blockwise GEMM for callers that cannot allocate device memory and have no
// workspace to hand over (code under HIP graph capture, tight serving loops).  The split-K planes -- the fp32 partial
// sums that llmmm_fp8_gemm keeps in its caller's workspace -- live in a fixed array inside the library's device image
// instead.  Everything else (kernel choice, arithmetic, outputs) is llmmm_fp8_gemm's.
#include "../../include/llmmm.h"
#include "kernels.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>

namespace {

// Every GPU the library runs on holds its own copy of this array, at its own address, until the process ends.  Plain
// scratch: the kernels write every element of a plane before the reduce kernel reads it, so nothing has to start at
// zero; what the previous call left behind is never read.
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[LLMMM_STATIC_WS_BYTES];

constexpr int      MAX_DEVICES = 64;
std::atomic<void*> g_scratch[MAX_DEVICES];  // device address of `scratch` per device, resolved on first use
std::mutex         g_resolve;

// The array's name is only a host-side handle; the address kernels and copies can use comes from the runtime, once
// per device, with that device current.
int scratch_on_current_device(void** out)
{
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return llmmm::report_error(LLMMM_ERR_RUNTIME, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= MAX_DEVICES) return llmmm::report_error(LLMMM_ERR_RUNTIME, "device ordinal %d beyond the %d this entry point keeps track of", dev, MAX_DEVICES);
  void* p = g_scratch[dev].load(std::memory_order_acquire);
  if (!p) {
    std::lock_guard<std::mutex> lock(g_resolve);
    p = g_scratch[dev].load(std::memory_order_relaxed);
    if (!p) {
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess || !p) return llmmm::report_error(LLMMM_ERR_RUNTIME, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
      g_scratch[dev].store(p, std::memory_order_release);
    }
  }
  *out = p;
  return LLMMM_OK;
}

}  // namespace

extern "C" int llmmm_fp8_gemm_static_ws(int out_kind, const void* A, const float* As, const void* Bt, const float* Bs, void* C, float* Cs, int M, int N,
                                        int K, void* stream)
{
  if (out_kind < LLMMM_OUT_F32 || out_kind > LLMMM_OUT_FP8Q_SWIGLU) return llmmm::report_error(LLMMM_ERR_INVALID_ARGUMENT, "unknown output kind %d", out_kind);
  llmmm_gemm_cfg cfg;
  const int      rc = llmmm_fp8_gemm_query(out_kind, M, N, K, &cfg);  // shape checks, with the reference's texts
  if (rc) return rc;
  // the planes of the split the library picks for this shape must fit the array: no silent fall-back to a smaller split
  const size_t need = llmmm_fp8_gemm_workspace(out_kind, M, N, K);
  if (need > (size_t)LLMMM_STATIC_WS_BYTES)
    return llmmm::report_error(LLMMM_ERR_WORKSPACE, "M = %d, N = %d, K = %d needs %zu bytes of split-K planes, the built-in array holds %zu: use llmmm_fp8_gemm with a workspace",
                               M, N, K, need, (size_t)LLMMM_STATIC_WS_BYTES);
  // The two runtime queries of this path -- the array's address and the device's CU count -- are made on every call,
  // whatever the shape needs: both are answered from memory after the first, so any warm-up call on a device makes
  // every later call on it free of runtime queries, as stream capture requires.
  void*     ws  = nullptr;
  const int rcs = scratch_on_current_device(&ws);
  if (rcs) return rcs;
  (void)llmmm::num_cus();
  return llmmm_fp8_gemm_ex(out_kind, A, As, Bt, Bs, C, Cs, M, N, K, need ? ws : nullptr, need, nullptr, stream);
}
