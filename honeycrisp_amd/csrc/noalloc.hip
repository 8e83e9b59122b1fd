// hc_reduce_noalloc: hc_reduce for callers that cannot allocate device memory (code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc). The partial results that
// hc_reduce keeps in pool blocks (split column reductions, segmented long rows) live in a fixed
// array in device memory that belongs to this library, so the call allocates and frees nothing.
//
// The array's name is a host-side stand-in, not a device address: its address on a device comes
// from hipGetSymbolAddress, once per device with that device current (hc_noalloc_setup, called by
// hc_init), and only that address is handed to kernels.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <mutex>

#include "../../include/hchip.h"

// Each device the library runs on holds its own copy until the process ends.
static __device__ __align__(256) unsigned char scratch[HC_NOALLOC_SCRATCH_BYTES];

static const int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_setup_mu;
// One per device, held for the whole of a call: a split reduction is two launches that meet in the
// array, and with the lock both are enqueued back to back, so that calls from several threads
// through one context run one after the other in its stream's order.
static std::mutex g_call_mu[kMaxDevices];

// hchip.cpp
int hc_reduce_in_scratch(hc_ctx* ctx, int op, int dtype, const void* in, void* out, int64_t outer, int64_t reduce,
                         int64_t inner, void* scratch_base, size_t scratch_bytes);
int hc_ctx_device(const hc_ctx* ctx);
int hc_set_error(int code, const char* message);

// Device address of this device's copy of the array. The caller has made `device` current.
__attribute__((visibility("hidden"))) int hc_noalloc_setup(int device) {
  if (device < 0 || device >= kMaxDevices) return hc_set_error(HC_ERR_INVALID, "hc_noalloc_setup: device out of range");
  std::lock_guard<std::mutex> lock(g_setup_mu);
  if (g_scratch_ptr[device]) return HC_OK;
  void* ptr = nullptr;
  hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr) {
    char msg[256];
    snprintf(msg, sizeof(msg), "hipGetSymbolAddress(scratch) on device %d: %s", device, hipGetErrorString(e));
    (void)hipGetLastError();
    return hc_set_error(HC_ERR_HIP_BASE + (int)e, msg);
  }
  g_scratch_ptr[device] = ptr;
  return HC_OK;
}

extern "C" int hc_reduce_noalloc(hc_ctx* ctx, int op, int dtype, const void* in, void* out, int64_t outer,
                                 int64_t reduce, int64_t inner) {
  const int device = hc_ctx_device(ctx);
  if (device < 0 || device >= kMaxDevices) return hc_set_error(HC_ERR_INVALID, "hc_reduce_noalloc: null context");
  // Every partial result is written by the first pass before the second pass reads it, so nothing
  // in the array has to start at zero.
  std::lock_guard<std::mutex> lock(g_call_mu[device]);
  return hc_reduce_in_scratch(ctx, op, dtype, in, out, outer, reduce, inner, g_scratch_ptr[device],
                              (size_t)HC_NOALLOC_SCRATCH_BYTES);
}
