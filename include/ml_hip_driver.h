/*
 * ml_hip_driver.h - C ABI of the ML::HIP driver layer (libcogni_hip.so).
 *
 * One entry point per function the reference binds from the CUDA driver API in
 * `lib LibCUDADriver` (src/ml/cuda/driver.cr:1-51), with the same argument
 * order and the same convention: every call returns an int status, 0 on
 * success, otherwise the hipError_t value. The reference turns a non-zero
 * status into an exception in ML::CUDA.check! (driver.cr:57-59); a binding of
 * this header does the same (see mlhip_error_string for the text).
 *
 * Handles are opaque pointers; device addresses are 64-bit integers, as the
 * reference's `alias CUdeviceptr = UInt64` (driver.cr:10).
 *
 * Not thread safe by contract, like the reference (module-global current
 * stream, driver.cr:55,252-260). Streams keep the default priority.
 */
#ifndef ML_HIP_DRIVER_H
#define ML_HIP_DRIVER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint64_t mlhip_deviceptr;   /* driver.cr:10  CUdeviceptr */
typedef void* mlhip_context;        /* driver.cr:3   CUcontext   */
typedef void* mlhip_module;         /* driver.cr:4   CUmodule    */
typedef void* mlhip_function;       /* driver.cr:5   CUfunction  */
typedef void* mlhip_stream;         /* driver.cr:6   CUstream    */
typedef void* mlhip_graph;          /* driver.cr:7   CUgraph     */
typedef void* mlhip_graph_exec;     /* driver.cr:8   CUgraphExec */
typedef void* mlhip_event;          /* no counterpart: GPU-side timing */

/* driver.cr:20 cuInit */
int mlhip_init(uint32_t flags);
/* driver.cr:21 cuDeviceGet */
int mlhip_device_get(int32_t* device, int32_t ordinal);
/* driver.cr:22 cuDeviceGetName */
int mlhip_device_get_name(char* name, int32_t len, int32_t device);
/* driver.cr:23 cuDeviceComputeCapability. On gfx950 this reports 9.5. */
int mlhip_device_compute_capability(int32_t* major, int32_t* minor, int32_t device);
/* No counterpart: the ISA name ("gfx950:sramecc+:xnack-") the code object must match. */
int mlhip_device_get_arch(char* name, int32_t len, int32_t device);
/* No counterpart: compute units and peak engine clock (kHz), printed by the probes. */
int mlhip_device_get_cu_clock(int32_t* compute_units, int32_t* clock_khz, int32_t device);
/* driver.cr:24 cuCtxCreate_v2. HIP works on the device's primary context: this makes `device`
 * current (hipSetDevice) and returns a token for it. */
int mlhip_ctx_create(mlhip_context* ctx, uint32_t flags, int32_t device);
/* driver.cr:25 cuCtxDestroy_v2. Releases the token; the primary context stays alive. */
int mlhip_ctx_destroy(mlhip_context ctx);
/* driver.cr:26 cuModuleLoadData. `image` is a gfx950 code object (ELF or clang offload bundle),
 * not a NUL-terminated PTX string. */
int mlhip_module_load_data(mlhip_module* mod, const void* image);
/* driver.cr:27 cuModuleUnload */
int mlhip_module_unload(mlhip_module mod);
/* driver.cr:28 cuModuleGetFunction */
int mlhip_module_get_function(mlhip_function* fn, mlhip_module mod, const char* name);
/* driver.cr:29 cuFuncGetAttribute; `attrib` uses the numbering of ML::CUDA::FunctionAttribute
 * (driver.cr:154-165), which HIP's hipFunction_attribute shares. */
int mlhip_func_get_attribute(int32_t* value, int32_t attrib, mlhip_function fn);
/* driver.cr:30 cuStreamCreate (default priority) */
int mlhip_stream_create(mlhip_stream* stream, uint32_t flags);
/* driver.cr:31 cuStreamDestroy_v2 */
int mlhip_stream_destroy(mlhip_stream stream);
/* driver.cr:32 cuStreamSynchronize */
int mlhip_stream_synchronize(mlhip_stream stream);
/* driver.cr:33 cuStreamBeginCapture */
int mlhip_stream_begin_capture(mlhip_stream stream, int32_t mode);
/* driver.cr:34 cuStreamEndCapture */
int mlhip_stream_end_capture(mlhip_stream stream, mlhip_graph* graph);
/* driver.cr:35 cuGraphInstantiateWithFlags. (cuGraphInstantiateWithParams, driver.cr:36, exists only
 * for CUDA's device-side graph launch flag, which HIP does not have; it has no entry here.) */
int mlhip_graph_instantiate(mlhip_graph_exec* exec, mlhip_graph graph, uint64_t flags);
/* driver.cr:37 cuGraphUpload */
int mlhip_graph_upload(mlhip_graph_exec exec, mlhip_stream stream);
/* driver.cr:38 cuGraphLaunch */
int mlhip_graph_launch(mlhip_graph_exec exec, mlhip_stream stream);
/* driver.cr:39 cuGraphDestroy */
int mlhip_graph_destroy(mlhip_graph graph);
/* driver.cr:40 cuGraphExecDestroy */
int mlhip_graph_exec_destroy(mlhip_graph_exec exec);
/* driver.cr:41 cuMemAlloc_v2 */
int mlhip_mem_alloc(mlhip_deviceptr* dptr, size_t bytesize);
/* driver.cr:42 cuMemFree_v2 */
int mlhip_mem_free(mlhip_deviceptr dptr);
/* driver.cr:43 cuMemcpyHtoD_v2 (synchronous) */
int mlhip_memcpy_htod(mlhip_deviceptr dst, const void* src, size_t bytesize);
/* driver.cr:44 cuMemcpyDtoH_v2 (synchronous) */
int mlhip_memcpy_dtoh(void* dst, mlhip_deviceptr src, size_t bytesize);
/* driver.cr:45 cuMemcpyDtoD_v2 (synchronous) */
int mlhip_memcpy_dtod(mlhip_deviceptr dst, mlhip_deviceptr src, size_t bytesize);
/* driver.cr:46-49 cuLaunchKernel. kernel_params[i] points at the i-th argument value. */
int mlhip_launch_kernel(mlhip_function fn, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                        uint32_t block_x, uint32_t block_y, uint32_t block_z, uint32_t shared_mem_bytes,
                        mlhip_stream stream, void** kernel_params, void** extra);
/* driver.cr:50 cuCtxSynchronize */
int mlhip_ctx_synchronize(void);

/* No counterpart in the reference (it times with the host clock around cuCtxSynchronize,
 * bin/cuda_q4k_gemv_probe.cr:261-266): GPU events on a stream, for per-launch durations. */
int mlhip_event_create(mlhip_event* ev);
int mlhip_event_record(mlhip_event ev, mlhip_stream stream);
int mlhip_event_synchronize(mlhip_event ev);
int mlhip_event_elapsed_ms(float* ms, mlhip_event start, mlhip_event stop);
int mlhip_event_destroy(mlhip_event ev);

/* Name of a status value ("hipErrorInvalidValue"); static storage. */
const char* mlhip_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* ML_HIP_DRIVER_H */
