// Hooks between the translation units of libcogni_hip.so. Not part of the C ABI (include/*.h).
#pragma once
#ifdef __cplusplus
extern "C" {
#endif
// Record `text` as the calling thread's last error (cogni_last_error) and return `code`.
int cogni_internal_fail(int code, const char* text);
// The same for a failed HIP call: "<what> failed with HIP error <n> (<name>)"; returns hip_error.
int cogni_internal_hip_fail(int hip_error, const char* what);
// Resolve, on the current device, the address of the static scratch array behind cogni_gemv_top1_noalloc_dev
// (top1_noalloc.hip). Called by cogni_quant_init once the device is selected.
int cogni_internal_noalloc_setup(int device);
#ifdef __cplusplus
}
#endif
