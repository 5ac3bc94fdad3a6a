// cogni_gemv_top1_noalloc_dev: the output-head arg-max (cogni_gemv_top1_dev) for callers that cannot allocate device
// memory - code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. The per-workgroup
// partial results, which cogni_gemv_top1_dev takes from caller-owned buffers, live here in a file-scope device array.
//
// This file is compiled by hipcc as host + device code (the array needs a device-side definition that the HIP runtime
// registers when the library is loaded); the kernels stay in the code object the rest of the library launches from and
// receive the array's device address as an ordinary argument.
//
// The array's name is only a host-side stand-in in host code. Its device address is asked for once per device, with
// that device current, through hipGetSymbolAddress, and every later use goes through that address.
#include "cogni_quant.h"
#include "internal.h"

#include <hip/hip_runtime.h>

#include <string>

// ids: u32[COGNI_TOP1_NOALLOC_MAX_PARTIALS], then values: f32[COGNI_TOP1_NOALLOC_MAX_PARTIALS]. Each GPU the library
// runs on holds its own copy until the process ends.
static __device__ __align__(256) unsigned char scratch[2 * 4 * COGNI_TOP1_NOALLOC_MAX_PARTIALS];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];   // device address of `scratch` on device i, null until cogni_internal_noalloc_setup(i)
}

// Called from cogni_quant_init with the device it selected current.
extern "C" int cogni_internal_noalloc_setup(int device) {
  if (device < 0 || device >= kMaxDevices)
    return cogni_internal_fail(COGNI_ERR_INVALID_ARGUMENT, "static scratch: device ordinal out of range");
  if (g_scratch_ptr[device]) return 0;
  void* ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr) return cogni_internal_hip_fail((int)e, "hipGetSymbolAddress(static top-1 scratch)");
  g_scratch_ptr[device] = ptr;
  return 0;
}

extern "C" int cogni_gemv_top1_noalloc_dev(uint64_t w_raw, uint32_t w_type, uint64_t x, uint64_t top1_ids,
                                           uint64_t top1_values, uint32_t in_dim, uint32_t out_dim, uint32_t tokens,
                                           void* stream) {
  int device = -1;
  const hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return cogni_internal_hip_fail((int)e, "hipGetDevice");
  if (device < 0 || device >= kMaxDevices || !g_scratch_ptr[device])
    return cogni_internal_fail(COGNI_ERR_NOT_INITIALIZED, "cogni_gemv_top1_noalloc_dev: cogni_quant_init has not been called on the current device");
  const uint64_t stride = cogni_gemv_top1_partials(w_type, out_dim);   // 0 for a type or shape the operator rejects below
  if (stride * tokens > COGNI_TOP1_NOALLOC_MAX_PARTIALS)
    return cogni_internal_fail(COGNI_ERR_INVALID_ARGUMENT,
                               ("cogni_gemv_top1_noalloc_dev: " + std::to_string(tokens) + " tokens x " + std::to_string(stride) +
                                " partial results per token exceed the static scratch of " +
                                std::to_string(COGNI_TOP1_NOALLOC_MAX_PARTIALS) + "; use cogni_gemv_top1_dev with caller-owned buffers").c_str());
  // Every slot the reduce kernel reads was written by the partial kernel of the same call, so nothing has to start at
  // zero; what an earlier call left in the array is never read.
  const uint64_t ids = (uint64_t)(uintptr_t)g_scratch_ptr[device];
  const uint64_t values = ids + 4ull * COGNI_TOP1_NOALLOC_MAX_PARTIALS;
  return cogni_gemv_top1_dev(w_raw, w_type, x, ids, values, top1_ids, top1_values, in_dim, out_dim, tokens, stream);
}
