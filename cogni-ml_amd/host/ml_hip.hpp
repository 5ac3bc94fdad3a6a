// ml::hip - C++ host mirror of the reference's ML::CUDA module (src/ml/cuda/driver.cr:53-343), built on
// the C ABI of libcogni_hip.so (include/ml_hip_driver.h). Same classes, same ownership rules (one handle
// per wrapper, idempotent close(), no finalizer-driven release beyond the destructor calling close()),
// same error rule: a non-zero status throws "<what> failed with HIP error <code>" (driver.cr:57-59).
// The reference's host language is Crystal; no Crystal compiler exists where this is built, so the host
// side is C++ and the Crystal binding is shipped as source (crystal/src/ml/hip/driver.cr).
#pragma once
#include <cstdint>
#include <functional>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "ml_hip_driver.h"

namespace ml::hip {

using DevicePtr = mlhip_deviceptr;   // driver.cr:54

class Error : public std::runtime_error {
 public:
  Error(const std::string& what, int code)
      : std::runtime_error(what + " failed with HIP error " + std::to_string(code)), code_(code) {}
  int code() const { return code_; }

 private:
  int code_;
};

// ML::CUDA.check! (driver.cr:57-59)
inline void check(int code, const std::string& what) {
  if (code != 0) throw Error(what, code);
}

namespace detail {
inline mlhip_stream& current_stream() {   // @@current_stream (driver.cr:55); not thread safe, as in the reference
  static mlhip_stream s = nullptr;
  return s;
}
}  // namespace detail

// driver.cr:61-94
class Context {
 public:
  static Context create(int ordinal = 0) {
    check(mlhip_init(0), "hipInit");
    int32_t dev = 0;
    check(mlhip_device_get(&dev, ordinal), "hipDeviceGet");
    char buf[256] = {0};
    check(mlhip_device_get_name(buf, sizeof buf, dev), "hipDeviceGetName");
    std::string name(buf);
    int32_t major = 0, minor = 0;
    check(mlhip_device_compute_capability(&major, &minor, dev), "hipDeviceComputeCapability");
    check(mlhip_device_get_arch(buf, sizeof buf, dev), "hipGetDeviceProperties");
    std::string arch(buf);
    mlhip_context h = nullptr;
    check(mlhip_ctx_create(&h, 0, dev), "hipCtxCreate");
    return Context(h, name, major, minor, arch);
  }
  Context(Context&& o) noexcept { *this = std::move(o); }
  Context& operator=(Context&& o) noexcept {
    handle_ = o.handle_; name_ = std::move(o.name_); arch_ = std::move(o.arch_);
    major_ = o.major_; minor_ = o.minor_; closed_ = o.closed_; o.closed_ = true;
    return *this;
  }
  ~Context() { close(); }
  const std::string& device_name() const { return name_; }
  const std::string& arch() const { return arch_; }
  int compute_capability_major() const { return major_; }
  int compute_capability_minor() const { return minor_; }
  void close() {
    if (closed_) return;
    if (handle_) mlhip_ctx_destroy(handle_);
    closed_ = true;
  }

 private:
  Context(mlhip_context h, std::string name, int major, int minor, std::string arch)
      : handle_(h), name_(std::move(name)), arch_(std::move(arch)), major_(major), minor_(minor) {}
  mlhip_context handle_ = nullptr;
  std::string name_, arch_;
  int major_ = 0, minor_ = 0;
  bool closed_ = false;
};

// driver.cr:96-112
class DeviceBuffer {
 public:
  explicit DeviceBuffer(size_t bytesize) : bytesize_(bytesize) {
    check(mlhip_mem_alloc(&ptr_, bytesize ? bytesize : 1), "hipMalloc");
  }
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  DeviceBuffer(DeviceBuffer&& o) noexcept : ptr_(o.ptr_), bytesize_(o.bytesize_), closed_(o.closed_) { o.closed_ = true; }
  ~DeviceBuffer() { close(); }
  DevicePtr ptr() const { return ptr_; }
  size_t bytesize() const { return bytesize_; }
  void close() {
    if (closed_) return;
    if (ptr_) mlhip_mem_free(ptr_);
    closed_ = true;
  }

 private:
  DevicePtr ptr_ = 0;
  size_t bytesize_ = 0;
  bool closed_ = false;
};

// driver.cr:154-165
enum class FunctionAttribute : int {
  MaxThreadsPerBlock = 0, SharedSizeBytes = 1, ConstSizeBytes = 2, LocalSizeBytes = 3, NumRegs = 4,
  PtxVersion = 5, BinaryVersion = 6, CacheModeCa = 7, MaxDynamicSharedSizeBytes = 8,
  PreferredSharedMemoryCarveout = 9
};

// driver.cr:139-152
class KernelFunction {
 public:
  KernelFunction(mlhip_function h, std::string name) : handle_(h), name_(std::move(name)) {}
  mlhip_function handle() const { return handle_; }
  const std::string& name() const { return name_; }
  int attribute(FunctionAttribute attr) const {
    int32_t v = 0;
    check(mlhip_func_get_attribute(&v, (int)attr, handle_), "hipFuncGetAttribute(" + name_ + ")");
    return v;
  }

 private:
  mlhip_function handle_;
  std::string name_;
};

// CUDAModule (driver.cr:114-137): the image is a gfx950 code object instead of PTX text
class HIPModule {
 public:
  static HIPModule load(const void* image, const std::string& label) {
    mlhip_module h = nullptr;
    check(mlhip_module_load_data(&h, image), "hipModuleLoadData(" + label + ")");
    return HIPModule(h);
  }
  HIPModule(HIPModule&& o) noexcept : handle_(o.handle_), closed_(o.closed_) { o.closed_ = true; }
  ~HIPModule() { close(); }
  KernelFunction function(const std::string& name) const {
    mlhip_function fn = nullptr;
    check(mlhip_module_get_function(&fn, handle_, name.c_str()), "hipModuleGetFunction(" + name + ")");
    return KernelFunction(fn, name);
  }
  void close() {
    if (closed_) return;
    if (handle_) mlhip_module_unload(handle_);
    closed_ = true;
  }

 private:
  explicit HIPModule(mlhip_module h) : handle_(h) {}
  mlhip_module handle_ = nullptr;
  bool closed_ = false;
};

class HIPStream;

// driver.cr:228-250
class HIPGraphExec {
 public:
  explicit HIPGraphExec(mlhip_graph_exec h) : handle_(h) {}
  HIPGraphExec(HIPGraphExec&& o) noexcept : handle_(o.handle_), closed_(o.closed_) { o.closed_ = true; }
  ~HIPGraphExec() { close(); }
  void launch(const HIPStream& stream) const;
  void upload(const HIPStream& stream) const;
  void close() {
    if (closed_) return;
    if (handle_) mlhip_graph_exec_destroy(handle_);
    closed_ = true;
  }

 private:
  mlhip_graph_exec handle_;
  bool closed_ = false;
};

// driver.cr:195-226 (CUDA's device-launch instantiation has no HIP counterpart)
class HIPGraph {
 public:
  explicit HIPGraph(mlhip_graph h) : handle_(h) {}
  HIPGraph(HIPGraph&& o) noexcept : handle_(o.handle_), closed_(o.closed_) { o.closed_ = true; }
  ~HIPGraph() { close(); }
  HIPGraphExec instantiate() const {
    mlhip_graph_exec e = nullptr;
    check(mlhip_graph_instantiate(&e, handle_, 0), "hipGraphInstantiateWithFlags");
    return HIPGraphExec(e);
  }
  void close() {
    if (closed_) return;
    if (handle_) mlhip_graph_destroy(handle_);
    closed_ = true;
  }

 private:
  mlhip_graph handle_;
  bool closed_ = false;
};

// driver.cr:167-193; default priority only
class HIPStream {
 public:
  explicit HIPStream(uint32_t flags = 0) { check(mlhip_stream_create(&handle_, flags), "hipStreamCreate"); }
  HIPStream(const HIPStream&) = delete;
  ~HIPStream() { close(); }
  mlhip_stream handle() const { return handle_; }
  void synchronize() const { check(mlhip_stream_synchronize(handle_), "hipStreamSynchronize"); }
  void begin_capture(int mode = 1) const { check(mlhip_stream_begin_capture(handle_, mode), "hipStreamBeginCapture"); }
  HIPGraph end_capture() const {
    mlhip_graph g = nullptr;
    check(mlhip_stream_end_capture(handle_, &g), "hipStreamEndCapture");
    return HIPGraph(g);
  }
  void close() {
    if (closed_) return;
    if (handle_) mlhip_stream_destroy(handle_);
    closed_ = true;
  }

 private:
  mlhip_stream handle_ = nullptr;
  bool closed_ = false;
};

inline void HIPGraphExec::launch(const HIPStream& s) const { check(mlhip_graph_launch(handle_, s.handle()), "hipGraphLaunch"); }
inline void HIPGraphExec::upload(const HIPStream& s) const { check(mlhip_graph_upload(handle_, s.handle()), "hipGraphUpload"); }

inline mlhip_stream current_stream_handle() { return detail::current_stream(); }

// driver.cr:252-260
template <class F>
void with_stream(const HIPStream& stream, F&& body) {
  mlhip_stream previous = detail::current_stream();
  detail::current_stream() = stream.handle();
  try {
    body();
  } catch (...) {
    detail::current_stream() = previous;
    throw;
  }
  detail::current_stream() = previous;
}

// driver.cr:262-276
inline void copy_htod(DevicePtr dst, const void* src, size_t n, const std::string& what) {
  check(mlhip_memcpy_htod(dst, src, n), "hipMemcpyHtoD(" + what + ")");
}
inline void copy_dtoh(void* dst, DevicePtr src, size_t n, const std::string& what) {
  check(mlhip_memcpy_dtoh(dst, src, n), "hipMemcpyDtoH(" + what + ")");
}
inline void copy_dtod(DevicePtr dst, DevicePtr src, size_t n, const std::string& what) {
  check(mlhip_memcpy_dtod(dst, src, n), "hipMemcpyDtoD(" + what + ")");
}
inline void synchronize(const std::string& what = "hipDeviceSynchronize") { check(mlhip_ctx_synchronize(), what); }

// ML::CUDA.launch! (driver.cr:278-286): params[i] points at the i-th argument value
inline void launch(const KernelFunction& fn, uint32_t gx, uint32_t gy, uint32_t gz, uint32_t bx, uint32_t by,
                   uint32_t bz, void** params, const std::string& label, uint32_t shared_mem_bytes = 0) {
  check(mlhip_launch_kernel(fn.handle(), gx, gy, gz, bx, by, bz, shared_mem_bytes, detail::current_stream(), params,
                            nullptr),
        "hipModuleLaunchKernel(" + label + ")");
}

// driver.cr:288-342
class ResidentSequenceRunner {
 public:
  using Proc = std::function<void()>;
  using TokenProc = std::function<void(int)>;

  ResidentSequenceRunner(int tokens, Proc upload_weights, Proc reset_sequence, TokenProc run_token,
                         std::optional<Proc> read_outputs = std::nullopt,
                         std::optional<TokenProc> run_sequence_override = std::nullopt)
      : tokens_(tokens), upload_weights_(std::move(upload_weights)), reset_sequence_(std::move(reset_sequence)),
        run_token_(std::move(run_token)), read_outputs_(std::move(read_outputs)),
        run_sequence_override_(std::move(run_sequence_override)) {
    if (!(tokens_ > 0)) throw std::invalid_argument("tokens must be positive");
    active_tokens_ = tokens_;
  }
  int tokens() const { return tokens_; }
  int active_tokens() const { return active_tokens_; }
  int set_active_tokens(int n) {
    if (!(n > 0)) throw std::invalid_argument("active_tokens must be positive");
    if (!(n <= tokens_)) throw std::invalid_argument("active_tokens must be <= tokens");
    return active_tokens_ = n;
  }
  void reset_active_tokens() { active_tokens_ = tokens_; }
  void upload_weights() { upload_weights_(); }
  void reset_sequence() { reset_sequence_(); }
  void run_sequence() {
    if (run_sequence_override_) {
      (*run_sequence_override_)(active_tokens_);
    } else {
      for (int tok = 0; tok < active_tokens_; tok++) run_token_(tok);
    }
  }
  int run_repeated(int reps) {
    if (!(reps > 0)) throw std::invalid_argument("reps must be positive");
    for (int i = 0; i < reps; i++) run_sequence();
    return reps * active_tokens_;
  }
  void read_outputs() {
    if (read_outputs_) (*read_outputs_)();
  }

 private:
  int tokens_, active_tokens_;
  Proc upload_weights_, reset_sequence_;
  TokenProc run_token_;
  std::optional<Proc> read_outputs_;
  std::optional<TokenProc> run_sequence_override_;
};

}  // namespace ml::hip
