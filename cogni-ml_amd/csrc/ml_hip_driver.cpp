// ML::HIP driver layer: thin C wrappers over the HIP runtime/module API, one per function the
// reference binds from libcuda (src/ml/cuda/driver.cr:20-50). See include/ml_hip_driver.h.
#include "ml_hip_driver.h"

#include <hip/hip_runtime_api.h>
#include <cstdio>
#include <cstring>

extern "C" {

int mlhip_init(uint32_t flags) { return (int)hipInit(flags); }

int mlhip_device_get(int32_t* device, int32_t ordinal) {
  hipDevice_t d = 0;
  hipError_t e = hipDeviceGet(&d, ordinal);
  if (e == hipSuccess && device) *device = (int32_t)d;
  return (int)e;
}

int mlhip_device_get_name(char* name, int32_t len, int32_t device) {
  hipError_t e = hipDeviceGetName(name, len, (hipDevice_t)device);
  if (e == hipSuccess && name && len > 0 && name[0] == '\0') {   // some containers expose no marketing name
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess) std::snprintf(name, (size_t)len, "AMD %s", prop.gcnArchName);
  }
  return (int)e;
}

int mlhip_device_compute_capability(int32_t* major, int32_t* minor, int32_t device) {
  int a = 0, b = 0;
  hipError_t e = hipDeviceComputeCapability(&a, &b, (hipDevice_t)device);
  if (e == hipSuccess) {
    if (major) *major = a;
    if (minor) *minor = b;
  }
  return (int)e;
}

int mlhip_device_get_arch(char* name, int32_t len, int32_t device) {
  if (!name || len <= 0) return (int)hipErrorInvalidValue;
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, device);
  if (e != hipSuccess) return (int)e;
  std::strncpy(name, prop.gcnArchName, (size_t)len - 1);
  name[len - 1] = '\0';
  return 0;
}

int mlhip_device_get_cu_clock(int32_t* compute_units, int32_t* clock_khz, int32_t device) {
  int cu = 0, clk = 0;
  hipError_t e = hipDeviceGetAttribute(&cu, hipDeviceAttributeMultiprocessorCount, device);
  if (e != hipSuccess) return (int)e;
  e = hipDeviceGetAttribute(&clk, hipDeviceAttributeClockRate, device);
  if (e != hipSuccess) return (int)e;
  if (compute_units) *compute_units = cu;
  if (clock_khz) *clock_khz = clk;
  return 0;
}

int mlhip_ctx_create(mlhip_context* ctx, uint32_t /*flags*/, int32_t device) {
  hipError_t e = hipSetDevice(device);
  if (e != hipSuccess) return (int)e;
  if (ctx) *ctx = reinterpret_cast<void*>((intptr_t)device + 1);  // non-null token for the primary context
  return 0;
}

int mlhip_ctx_destroy(mlhip_context /*ctx*/) { return 0; }

int mlhip_module_load_data(mlhip_module* mod, const void* image) {
  return (int)hipModuleLoadData(reinterpret_cast<hipModule_t*>(mod), image);
}

int mlhip_module_unload(mlhip_module mod) { return (int)hipModuleUnload((hipModule_t)mod); }

int mlhip_module_get_function(mlhip_function* fn, mlhip_module mod, const char* name) {
  return (int)hipModuleGetFunction(reinterpret_cast<hipFunction_t*>(fn), (hipModule_t)mod, name);
}

int mlhip_func_get_attribute(int32_t* value, int32_t attrib, mlhip_function fn) {
  int v = 0;
  hipError_t e = hipFuncGetAttribute(&v, (hipFunction_attribute)attrib, (hipFunction_t)fn);
  if (e == hipSuccess && value) *value = v;
  return (int)e;
}

int mlhip_stream_create(mlhip_stream* stream, uint32_t flags) {
  return (int)hipStreamCreateWithFlags(reinterpret_cast<hipStream_t*>(stream), flags);
}

int mlhip_stream_destroy(mlhip_stream stream) { return (int)hipStreamDestroy((hipStream_t)stream); }

int mlhip_stream_synchronize(mlhip_stream stream) { return (int)hipStreamSynchronize((hipStream_t)stream); }

int mlhip_stream_begin_capture(mlhip_stream stream, int32_t mode) {
  return (int)hipStreamBeginCapture((hipStream_t)stream, (hipStreamCaptureMode)mode);
}

int mlhip_stream_end_capture(mlhip_stream stream, mlhip_graph* graph) {
  return (int)hipStreamEndCapture((hipStream_t)stream, reinterpret_cast<hipGraph_t*>(graph));
}

int mlhip_graph_instantiate(mlhip_graph_exec* exec, mlhip_graph graph, uint64_t flags) {
  return (int)hipGraphInstantiateWithFlags(reinterpret_cast<hipGraphExec_t*>(exec), (hipGraph_t)graph,
                                           (unsigned long long)flags);
}

int mlhip_graph_upload(mlhip_graph_exec exec, mlhip_stream stream) {
  return (int)hipGraphUpload((hipGraphExec_t)exec, (hipStream_t)stream);
}

int mlhip_graph_launch(mlhip_graph_exec exec, mlhip_stream stream) {
  return (int)hipGraphLaunch((hipGraphExec_t)exec, (hipStream_t)stream);
}

int mlhip_graph_destroy(mlhip_graph graph) { return (int)hipGraphDestroy((hipGraph_t)graph); }

int mlhip_graph_exec_destroy(mlhip_graph_exec exec) { return (int)hipGraphExecDestroy((hipGraphExec_t)exec); }

int mlhip_mem_alloc(mlhip_deviceptr* dptr, size_t bytesize) {
  void* p = nullptr;
  hipError_t e = hipMalloc(&p, bytesize);
  if (e == hipSuccess && dptr) *dptr = (mlhip_deviceptr)(uintptr_t)p;
  return (int)e;
}

int mlhip_mem_free(mlhip_deviceptr dptr) { return (int)hipFree((void*)(uintptr_t)dptr); }

int mlhip_memcpy_htod(mlhip_deviceptr dst, const void* src, size_t bytesize) {
  return (int)hipMemcpyHtoD((hipDeviceptr_t)(uintptr_t)dst, const_cast<void*>(src), bytesize);
}

int mlhip_memcpy_dtoh(void* dst, mlhip_deviceptr src, size_t bytesize) {
  return (int)hipMemcpyDtoH(dst, (hipDeviceptr_t)(uintptr_t)src, bytesize);
}

int mlhip_memcpy_dtod(mlhip_deviceptr dst, mlhip_deviceptr src, size_t bytesize) {
  return (int)hipMemcpyDtoD((hipDeviceptr_t)(uintptr_t)dst, (hipDeviceptr_t)(uintptr_t)src, bytesize);
}

int mlhip_launch_kernel(mlhip_function fn, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z, uint32_t block_x,
                        uint32_t block_y, uint32_t block_z, uint32_t shared_mem_bytes, mlhip_stream stream,
                        void** kernel_params, void** extra) {
  return (int)hipModuleLaunchKernel((hipFunction_t)fn, grid_x, grid_y, grid_z, block_x, block_y, block_z,
                                    shared_mem_bytes, (hipStream_t)stream, kernel_params, extra);
}

int mlhip_ctx_synchronize(void) { return (int)hipDeviceSynchronize(); }

int mlhip_event_create(mlhip_event* ev) { return (int)hipEventCreate(reinterpret_cast<hipEvent_t*>(ev)); }

int mlhip_event_record(mlhip_event ev, mlhip_stream stream) {
  return (int)hipEventRecord((hipEvent_t)ev, (hipStream_t)stream);
}

int mlhip_event_synchronize(mlhip_event ev) { return (int)hipEventSynchronize((hipEvent_t)ev); }

int mlhip_event_elapsed_ms(float* ms, mlhip_event start, mlhip_event stop) {
  return (int)hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop);
}

int mlhip_event_destroy(mlhip_event ev) { return (int)hipEventDestroy((hipEvent_t)ev); }

const char* mlhip_error_string(int code) { return hipGetErrorName((hipError_t)code); }

}  // extern "C"
