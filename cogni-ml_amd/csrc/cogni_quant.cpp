// Quantized-matmul operators over the gfx950 code object. See include/cogni_quant.h.
//
// The kernels live in a separately compiled code object that is embedded in this library
// (hsaco_blob.S) and loaded with hipModuleLoadData; every launch goes through
// hipModuleLaunchKernel with the kernel ABI the header documents. There is no host fallback.
#include "cogni_quant.h"
#include "internal.h"
#include "kernels/gemv_config.h"

#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

extern "C" const unsigned char cogni_hsaco_begin[];
extern "C" const unsigned char cogni_hsaco_end[];

namespace {

thread_local std::string g_err;

int fail(int code, const std::string& what) {
  g_err = what;
  return code;
}

int hip_fail(hipError_t e, const std::string& what) {
  char buf[64];
  std::snprintf(buf, sizeof buf, " failed with HIP error %d (", (int)e);
  g_err = what + buf + hipGetErrorName(e) + ")";
  return (int)e;
}

#define HIP_TRY(call, what)                          \
  do {                                               \
    hipError_t e__ = (call);                         \
    if (e__ != hipSuccess) return hip_fail(e__, what); \
  } while (0)

struct Runtime {
  bool ready = false;
  int ordinal = -1;
  int compute_units = 0;
  hipModule_t mod = nullptr;
  std::unordered_map<std::string, hipFunction_t> fns;
  // activation images of the one-pass multi-token GEMV for the calls that bring none: one slot per stream
  static constexpr int kImageSlots = 8;
  void* image_pool = nullptr;
  size_t image_slot_bytes = 0;
  void* image_stream[kImageSlots] = {};
  bool image_used[kImageSlots] = {};
  bool image_pinned[kImageSlots] = {};   // handed out under stream capture: a graph names it, it never changes hands
  unsigned long long calls_without_image = 0;   // multi-token calls that found every slot taken and made several passes
};
Runtime g_rt;
std::mutex g_mu;

int get_fn(const char* name, hipFunction_t* out) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (!g_rt.ready) return fail(COGNI_ERR_NOT_INITIALIZED, "cogni_quant_init has not been called");
  auto it = g_rt.fns.find(name);
  if (it != g_rt.fns.end()) {
    *out = it->second;
    return 0;
  }
  hipFunction_t fn = nullptr;
  HIP_TRY(hipModuleGetFunction(&fn, g_rt.mod, name), std::string("hipModuleGetFunction(") + name + ")");
  g_rt.fns.emplace(name, fn);
  *out = fn;
  return 0;
}

int launch(const char* name, uint32_t grid, uint32_t block, uint32_t shmem, void** params, void* stream,
           uint32_t grid_y = 1) {
  hipFunction_t fn = nullptr;
  int rc = get_fn(name, &fn);
  if (rc != 0) return rc;
  HIP_TRY(hipModuleLaunchKernel(fn, grid, grid_y, 1, block, 1, 1, shmem, (hipStream_t)stream, params, nullptr),
          std::string("hipModuleLaunchKernel(") + name + ")");
  return 0;
}

// The library-owned activation image of `stream` (0 if every slot belongs to another stream). Work on one stream is
// ordered, so a stream's slot is free again by the time its next call writes it; different streams never share one.
// A slot handed out while `stream` is capturing is baked into the graph, which may be replayed long after the stream is
// gone: such a slot is pinned, it stays with its stream key until cogni_quant_shutdown and cogni_gemv_release_stream
// leaves it alone. A call that finds no slot is counted (cogni_gemv_image_stats).
uint64_t image_for_stream(void* stream) {
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  const bool capturing = stream && hipStreamIsCapturing((hipStream_t)stream, &cs) == hipSuccess && cs == hipStreamCaptureStatusActive;
  std::lock_guard<std::mutex> lk(g_mu);
  if (!g_rt.ready || !g_rt.image_pool) return 0;
  int slot = -1;
  for (int i = 0; i < Runtime::kImageSlots && slot < 0; i++)
    if (g_rt.image_used[i] && g_rt.image_stream[i] == stream) slot = i;
  for (int i = 0; i < Runtime::kImageSlots && slot < 0; i++)
    if (!g_rt.image_used[i]) {
      g_rt.image_used[i] = true;
      g_rt.image_stream[i] = stream;
      slot = i;
    }
  if (slot < 0) {
    g_rt.calls_without_image++;
    return 0;
  }
  if (capturing) g_rt.image_pinned[slot] = true;
  return (uint64_t)(uintptr_t)g_rt.image_pool + (uint64_t)slot * g_rt.image_slot_bytes;
}

const char* type_prefix(uint32_t type) {
  switch (type) {
    case COGNI_TYPE_Q8_0: return "q8_0";
    case COGNI_TYPE_Q4_K: return "q4_k";
    case COGNI_TYPE_Q5_K: return "q5_k";
    case COGNI_TYPE_Q6_K: return "q6_k";
    case COGNI_TYPE_IQ4_NL: return "iq4_nl";
    case COGNI_TYPE_F16: return "f16";
    case COGNI_TYPE_F32: return "f32";
    default: return nullptr;
  }
}

const char* type_name(uint32_t type) {
  switch (type) {
    case COGNI_TYPE_Q8_0: return "Q8_0";
    case COGNI_TYPE_Q4_K: return "Q4_K";
    case COGNI_TYPE_Q5_K: return "Q5_K";
    case COGNI_TYPE_Q6_K: return "Q6_K";
    case COGNI_TYPE_IQ4_NL: return "IQ4_NL";
    case COGNI_TYPE_F16: return "F16";
    case COGNI_TYPE_F32: return "F32";
    case 2: return "Q4_0";
    case 3: return "Q4_1";
    case 6: return "Q5_0";
    case 7: return "Q5_1";
    case 10: return "Q2_K";
    case 11: return "Q3_K";
    case 15: return "Q8_K";
    default: return "unknown";
  }
}

bool gemv_type(uint32_t t) {
  return t == COGNI_TYPE_Q8_0 || t == COGNI_TYPE_Q4_K || t == COGNI_TYPE_Q5_K || t == COGNI_TYPE_Q6_K;
}
// F32, F16, IQ4_NL: the arms of the reference's dispatch served by the plain kernels (quant_matmul.cr:30-32)
bool plain_type(uint32_t t) { return t == COGNI_TYPE_F32 || t == COGNI_TYPE_F16 || t == COGNI_TYPE_IQ4_NL; }
bool k_quant(uint32_t t) { return t == COGNI_TYPE_Q4_K || t == COGNI_TYPE_Q5_K || t == COGNI_TYPE_Q6_K; }

// Bytes of one weight row, the reference's row_bytes (quant_matmul.cr:46-47, 241-242).
size_t row_bytes_of(uint32_t type, uint32_t in_dim) {
  const size_t be = (size_t)cogni_block_elements(type), bb = (size_t)cogni_block_bytes(type);
  return ((in_dim + be - 1) / be) * bb;
}

struct DeviceMem {  // frees on scope exit; host-buffer operators are synchronous
  void* p = nullptr;
  ~DeviceMem() {
    if (p) (void)hipFree(p);
  }
  uint64_t addr() const { return (uint64_t)(uintptr_t)p; }
};

}  // namespace

struct cogni_quant_weight {
  void* dev = nullptr;
  size_t bytes = 0;
  uint32_t type = 0;
  int32_t out_dim = 0, in_dim = 0;
};

extern "C" {

const char* cogni_last_error(void) { return g_err.c_str(); }
int cogni_internal_fail(int code, const char* text) { return fail(code, text); }
int cogni_internal_hip_fail(int hip_error, const char* what) { return hip_fail((hipError_t)hip_error, what); }

// ---- geometry (reader.cr:51-78, 119-127) -----------------------------------------------------
int32_t cogni_block_bytes(uint32_t type) {
  switch (type) {
    case 0: return 4;    case 1: return 2;    case 2: return 18;   case 3: return 20;
    case 6: return 22;   case 7: return 24;   case 8: return 34;   case 10: return 84;
    case 11: return 110; case 12: return 144; case 13: return 176; case 14: return 210;
    case 15: return 292; case 20: return 18;
    default: return -1;
  }
}

int32_t cogni_block_elements(uint32_t type) {
  switch (type) {
    case 0: case 1: return 1;
    case 2: case 3: case 6: case 7: case 8: case 20: return 32;
    case 10: case 11: case 12: case 13: case 14: case 15: return 256;
    default: return -1;
  }
}

int64_t cogni_data_bytes(uint32_t type, int64_t n_elements) {
  const int64_t bb = cogni_block_bytes(type), be = cogni_block_elements(type);
  if (bb < 0) return -1;
  if (type == COGNI_TYPE_F32 || type == COGNI_TYPE_F16) return n_elements * bb;
  return ((n_elements + be - 1) / be) * bb;
}

// ---- code object ----------------------------------------------------------------------------------
int cogni_quant_code_object(const void** image, size_t* size) {
  if (!image || !size) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_quant_code_object: null argument");
  *image = cogni_hsaco_begin;
  *size = (size_t)(cogni_hsaco_end - cogni_hsaco_begin);
  return 0;
}

const char* cogni_gemv_kernel_name(uint32_t type, uint32_t tokens, int add) {
  static thread_local char buf[64];
  if (!gemv_type(type) || tokens < 1 || tokens > COGNI_MAX_GEMV_TOKENS) return nullptr;
  if (tokens == 1)
    std::snprintf(buf, sizeof buf, "%s_gemv_%sf32", type_prefix(type), add ? "add_" : "");
  else
    std::snprintf(buf, sizeof buf, "%s_gemv_%sf32_tbatch%u", type_prefix(type), add ? "add_" : "", tokens);
  return buf;
}

int cogni_gemv_launch_dims(uint32_t type, uint32_t tokens, uint32_t in_dim, uint32_t out_dim, uint32_t* grid_x,
                           uint32_t* block_x, uint32_t* shared_mem_bytes) {
  const int rows = (tokens >= 1 && tokens <= COGNI_MAX_GEMV_TOKENS) ? gemv_rows_per_block(type, (int)tokens) : 0;
  if (!grid_x || !block_x || !shared_mem_bytes || out_dim == 0 || in_dim == 0 || rows == 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_launch_dims: bad argument");
  *grid_x = gemv_grid(type, (int)tokens, out_dim);
  *block_x = GEMV_BLOCK;
  *shared_mem_bytes = gemv_lds_bytes(type, (int)tokens, in_dim);
  return 0;
}

const char* cogni_dequantize_kernel_name(uint32_t type) {
  static thread_local char buf[64];
  const char* p = type_prefix(type);
  if (!p) return nullptr;
  std::snprintf(buf, sizeof buf, "dequantize_%s_f32", p);
  return buf;
}

// ---- initialisation -------------------------------------------------------------------------------
int cogni_quant_init(int32_t ordinal) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_rt.ready) {
    if (g_rt.ordinal == ordinal) return 0;
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_quant_init: already initialised on another device");
  }
  hipError_t e = hipInit(0);
  if (e != hipSuccess) return fail(COGNI_ERR_NO_DEVICE, std::string("hipInit failed (") + hipGetErrorName(e) + "): no GPU, and there is no CPU fallback");
  int count = 0;
  e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= ordinal || ordinal < 0)
    return fail(COGNI_ERR_NO_DEVICE, "no HIP device with the requested ordinal; there is no CPU fallback");
  HIP_TRY(hipSetDevice(ordinal), "hipSetDevice");
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, ordinal), "hipGetDeviceProperties");
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(COGNI_ERR_NO_DEVICE, std::string("device is ") + prop.gcnArchName + ", the code object is gfx950 only");
  HIP_TRY(hipModuleLoadData(&g_rt.mod, cogni_hsaco_begin), "hipModuleLoadData(cogni_quant gfx950 code object)");
  // from here on a failure leaves nothing behind: the module is unloaded, the pool freed, the table emptied, so that a
  // later call starts from scratch
  auto undo = [&](int rc) {
    (void)hipModuleUnload(g_rt.mod);
    if (g_rt.image_pool) (void)hipFree(g_rt.image_pool);
    g_rt = Runtime();
    return rc;
  };
  auto resolve = [&](const std::string& name, bool required) -> int {
    hipFunction_t fn = nullptr;
    const hipError_t he = hipModuleGetFunction(&fn, g_rt.mod, name.c_str());
    if (he == hipSuccess) g_rt.fns.emplace(name, fn);
    else if (required) return hip_fail(he, "hipModuleGetFunction(" + name + ")");
    return 0;
  };
  // the static scratch of the entry point that allocates nothing: its device address, once per device
  if (int rc = cogni_internal_noalloc_setup(ordinal)) return undo(rc);
  // its kernels are resolved now, so that a call under stream capture finds them in the table
  for (const char* t : {"q8_0", "q4_k", "q5_k", "q6_k"})
    for (const char* sfx : {"", "_tbatch2", "_tbatch3"}) (void)resolve(std::string(t) + "_gemv_top1_partial_f32" + sfx, false);
  for (const char* name : {"q4_k_gemv_mfma_top1_partial_f32_tbatch3", "q4_k_gemv_mfma_top1_partial_f32_tbatch4",
                           "q6_k_gemv_mfma_top1_partial_f32_tbatch3", "q6_k_gemv_mfma_top1_partial_f32_tbatch4", "top1_reduce_f32"})
    if (int rc = resolve(name, true)) return undo(rc);
  g_rt.image_slot_bytes = ((size_t)gemv_mt_image_bytes(COGNI_TYPE_Q6_K, GEMV_MT_MAX_IN_DIM) + 255) & ~(size_t)255;
  if (hipError_t he = hipMalloc(&g_rt.image_pool, g_rt.image_slot_bytes * Runtime::kImageSlots); he != hipSuccess) {
    g_rt.image_pool = nullptr;
    return undo(hip_fail(he, "hipMalloc(activation images)"));
  }
  for (const char* name : {"pack_x_mt_q4k_f16", "pack_x_mt_q6k_f16", "q4_k_gemv_mt_f32", "q5_k_gemv_mt_f32", "q6_k_gemv_mt_f32", "q8_0_gemv_mt_f32", "q4_k_gemv_mt_swiglu_f32",
                           "q4_k_gemv_mt_top1_partial_f32", "q6_k_gemv_mt_top1_partial_f32", "rmsnorm_pack_q4k_f32",
                           "rmsnorm_pack_q6k_f32", "add_rmsnorm_pack_q4k_f32", "add_rmsnorm_pack_q6k_f32"})
    if (int rc = resolve(name, true)) return undo(rc);
  g_rt.compute_units = prop.multiProcessorCount;
  g_rt.ordinal = ordinal;
  g_rt.ready = true;
  return 0;
}

int cogni_quant_shutdown(void) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (!g_rt.ready) return 0;
  (void)hipModuleUnload(g_rt.mod);
  if (g_rt.image_pool) (void)hipFree(g_rt.image_pool);
  g_rt = Runtime();
  return 0;
}

// ---- device-pointer operators -----------------------------------------------------------------------
int cogni_dequantize_dev(uint64_t w_raw, uint32_t w_type, uint64_t n_elements, uint64_t out, void* stream) {
  const char* name = cogni_dequantize_kernel_name(w_type);
  if (!name) return fail(COGNI_ERR_UNSUPPORTED_TYPE, "Unsupported dequantization type: " + std::to_string(w_type));
  if (n_elements == 0) return 0;
  if (!w_raw || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_dequantize_dev: null device pointer");
  // one wavefront step produces 256 floats; 4 wavefronts per workgroup; grid-stride beyond the cap
  uint64_t groups = (n_elements + 1023) / 1024;
  const uint64_t cap = 65536;
  uint32_t grid = (uint32_t)(groups < cap ? groups : cap);
  if (grid == 0) grid = 1;
  unsigned long long n = n_elements;
  void* params[] = {&w_raw, &out, &n};
  return launch(name, grid, 256, 0, params, stream);
}

// ---- several tokens in one pass over the weights: pack the activations once, then one launch per matrix list ------
size_t cogni_gemv_image_bytes(uint32_t w_type, uint32_t in_dim, uint32_t tokens) {
  return gemv_mt_supported(w_type, (int)tokens, in_dim) ? (size_t)gemv_mt_image_bytes(w_type, in_dim) : 0;
}

uint32_t cogni_gemv_one_pass_from(uint32_t w_type, uint32_t in_dim, uint32_t out_dim) { return gemv_mt_from(w_type, in_dim, out_dim); }
uint32_t cogni_gemv_one_pass_multi_from(uint32_t w_type, uint32_t in_dim) { return gemv_mt_multi_from(w_type, in_dim); }

int cogni_gemv_release_stream(void* stream) {
  int slot = -1;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    for (int i = 0; i < Runtime::kImageSlots; i++)
      if (g_rt.image_used[i] && g_rt.image_stream[i] == stream) slot = i;
  }
  if (slot < 0) return 0;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_rt.image_pinned[slot]) return 0;   // a captured graph names this slot: it stays where it is
  }
  // the slot may only change hands once everything that reads it has run
  HIP_TRY(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize(cogni_gemv_release_stream)");
  std::lock_guard<std::mutex> lk(g_mu);
  if (g_rt.image_used[slot] && g_rt.image_stream[slot] == stream) g_rt.image_used[slot] = false, g_rt.image_stream[slot] = nullptr;
  return 0;
}

int cogni_gemv_image_stats(uint32_t* slots, uint32_t* in_use, uint32_t* pinned, uint64_t* calls_without_image) {
  std::lock_guard<std::mutex> lk(g_mu);
  uint32_t used = 0, pin = 0;
  for (int i = 0; i < Runtime::kImageSlots; i++) used += g_rt.image_used[i], pin += g_rt.image_pinned[i];
  if (slots) *slots = Runtime::kImageSlots;
  if (in_use) *in_use = used;
  if (pinned) *pinned = pin;
  if (calls_without_image) *calls_without_image = g_rt.calls_without_image;
  return 0;
}

// Passes over the weights cogni_gemv_dev makes for one call (with an image slot at hand): the same rules as the call itself.
int32_t cogni_gemv_passes(uint32_t w_type, uint32_t tokens, uint32_t in_dim, uint32_t out_dim) {
  if ((!gemv_type(w_type) && !plain_type(w_type)) || tokens == 0 || in_dim == 0 || out_dim == 0) return -1;
  if (plain_type(w_type)) return 1;
  if (k_quant(w_type) && (in_dim % 256) != 0) return -1;
  const uint32_t from = gemv_mt_from(w_type, in_dim, out_dim);
  if (from && tokens >= from) return (int32_t)((tokens + GEMV_MT_MAX_TOKENS - 1) / GEMV_MT_MAX_TOKENS);
  uint32_t cap = k_quant(w_type) ? 2u : (uint32_t)COGNI_MAX_GEMV_TOKENS;
  bool pairs = k_quant(w_type);
  for (int mt = GEMV_MFMA_MAX_TOKENS; mt >= 2; mt--)
    if (gemv_mfma_supported(w_type, mt, in_dim)) {
      cap = (uint32_t)mt;
      pairs = false;
      break;
    }
  const bool walks = (uint64_t)gemv_grid(w_type, 2, out_dim) * (uint32_t)gemv_rows_per_block(w_type, 2) < out_dim;
  int32_t passes = 0;
  for (uint32_t t0 = 0, m = 0; t0 < tokens; t0 += m, passes++) {
    const uint32_t left = tokens - t0;
    m = left < cap ? left : cap;
    if (pairs && left == 3 && !walks) m = 3;
  }
  return passes;
}

int cogni_gemv_packed_launch_dims(uint32_t w_type, uint32_t in_dim, uint32_t total_rows, uint32_t* grid_x, uint32_t* block_x,
                                  uint32_t* shared_mem_bytes) {
  if (!grid_x || !block_x || !shared_mem_bytes || total_rows == 0 || !gemv_mt_supported(w_type, 2, in_dim))
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_launch_dims: bad argument");
  *grid_x = gemv_mt_grid(w_type, in_dim, total_rows);
  *block_x = GEMV_MT_WAVES * 64;
  *shared_mem_bytes = gemv_mt_lds_bytes(w_type);
  return 0;
}

int cogni_gemv_pack_dev(uint64_t x, uint32_t w_type, uint32_t in_dim, uint32_t tokens, uint64_t image, void* stream) {
  if (!gemv_mt_supported(w_type, (int)tokens, in_dim))
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_pack_dev: no one-pass kernel for this type, token count and in_dim "
                                            "(cogni_gemv_image_bytes is 0)");
  if (!x || !image) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_pack_dev: null device pointer");
  void* params[] = {&x, &image, &tokens, &in_dim};
  return launch(w_type == COGNI_TYPE_Q6_K ? "pack_x_mt_q6k_f16" : "pack_x_mt_q4k_f16", 2 * gemv_mt_padded_sb(in_dim), 256, 0, params, stream);
}

int cogni_gemv_packed_dev(const uint64_t* w_raw, uint32_t w_type, uint64_t image, uint64_t residual, const uint64_t* out,
                          const uint32_t* out_dims, uint32_t count, uint32_t in_dim, uint32_t tokens, void* stream) {
  if (!w_raw || !out || !out_dims || !image) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_dev: null argument");
  if (count == 0 || count > 8) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_dev: count must be 1..8");
  if (!gemv_mt_supported(w_type, (int)tokens, in_dim))
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_dev: no one-pass kernel for this type, token count and in_dim");
  if (residual && count != 1) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_dev: a residual goes with a single matrix");
  for (uint32_t i = 0; i < count; i++)
    if (!w_raw[i] || !out[i] || out_dims[i] == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_dev: null pointer or zero rows");
  // up to three matrices per launch, as one matrix of all their rows; a matrix whose row count is not a multiple of 16
  // ends its launch (a tile of 16 rows is of one matrix)
  for (uint32_t i0 = 0; i0 < count;) {
    uint64_t w[3] = {0, 0, 0}, o[3] = {0, 0, 0};
    uint32_t rows[3] = {0, 0, 0}, n = 0;
    uint64_t total = 0;
    while (n < 3 && i0 + n < count) {
      w[n] = w_raw[i0 + n], o[n] = out[i0 + n], rows[n] = out_dims[i0 + n];
      total += rows[n];
      n++;
      if (rows[n - 1] % 16 != 0) break;
    }
    if (total > 0x7FFFFFFFull) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_dev: too many rows");
    uint64_t res = i0 == 0 ? residual : 0;
    void* params[] = {&w[0], &w[1], &w[2], &image, &res, &o[0], &o[1], &o[2], &in_dim, &rows[0], &rows[1], &rows[2], &tokens};
    const char* kernel = w_type == COGNI_TYPE_Q6_K ? "q6_k_gemv_mt_f32" : (w_type == COGNI_TYPE_Q5_K ? "q5_k_gemv_mt_f32" : (w_type == COGNI_TYPE_Q8_0 ? "q8_0_gemv_mt_f32" : "q4_k_gemv_mt_f32"));
    const int rc = launch(kernel, gemv_mt_grid(w_type, in_dim, (uint32_t)total),
                          GEMV_MT_WAVES * 64, gemv_mt_lds_bytes(w_type), params, stream);
    if (rc != 0) return rc;
    i0 += n;
  }
  return 0;
}

// Nine to sixteen tokens in one pass over the weights: the one-pass kernels with their sixteen activation rows as sixteen
// tokens in one binary16 term each (the precision class of the prefill GEMM), Q4_K, Q5_K and Q6_K.
static bool gemv16_shape(uint32_t w_type, uint32_t in_dim, uint32_t tokens) {
  return (w_type == COGNI_TYPE_Q4_K || w_type == COGNI_TYPE_Q5_K || w_type == COGNI_TYPE_Q6_K || w_type == COGNI_TYPE_Q8_0) && tokens >= 1 &&
         tokens <= 16 && gemv_mt_supported(w_type, 2, in_dim);
}
int cogni_gemv_pack16_dev(uint64_t x, uint32_t w_type, uint32_t in_dim, uint32_t tokens, uint64_t image, void* stream) {
  if (!gemv16_shape(w_type, in_dim, tokens))
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_pack16_dev: Q4_K, Q5_K, Q6_K or Q8_0, 1..16 tokens, in_dim a multiple of 256 up to 12288");
  if (!x || !image) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_pack16_dev: null device pointer");
  void* params[] = {&x, &image, &tokens, &in_dim};
  return launch(w_type == COGNI_TYPE_Q6_K ? "pack_x_mt16_q6k_f16" : "pack_x_mt16_q4k_f16", 4 * gemv_mt_padded_sb(in_dim), 256, 0, params, stream);
}
int cogni_gemv_packed16_dev(const uint64_t* w_raw, uint32_t w_type, uint64_t image, uint64_t residual, const uint64_t* out,
                            const uint32_t* out_dims, uint32_t count, uint32_t in_dim, uint32_t tokens, void* stream) {
  const char* who = "cogni_gemv_packed16_dev";
  if (!w_raw || !out || !out_dims || !image) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": null argument");
  if (count == 0 || count > 8) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": count must be 1..8");
  if (!gemv16_shape(w_type, in_dim, tokens))
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": Q4_K, Q5_K, Q6_K or Q8_0, 1..16 tokens, in_dim a multiple of 256 up to 12288");
  if (residual && count != 1) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": a residual goes with a single matrix");
  for (uint32_t i = 0; i < count; i++)
    if (!w_raw[i] || !out[i] || out_dims[i] == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": null pointer or zero rows");
  // up to three matrices per launch, as cogni_gemv_packed_dev
  for (uint32_t i0 = 0; i0 < count;) {
    uint64_t w[3] = {0, 0, 0}, o[3] = {0, 0, 0}, none = residual;
    uint32_t rows[3] = {0, 0, 0}, n = 0;
    uint64_t total = 0;
    while (n < 3 && i0 + n < count) {
      w[n] = w_raw[i0 + n], o[n] = out[i0 + n], rows[n] = out_dims[i0 + n];
      total += rows[n];
      n++;
      if (rows[n - 1] % 16 != 0) break;
    }
    if (total > 0x7FFFFFFFull) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": too many rows");
    void* params[] = {&w[0], &w[1], &w[2], &image, &none, &o[0], &o[1], &o[2], &in_dim, &rows[0], &rows[1], &rows[2], &tokens};
    const char* kernel = w_type == COGNI_TYPE_Q6_K ? "q6_k_gemv_mt16_f32" : (w_type == COGNI_TYPE_Q5_K ? "q5_k_gemv_mt16_f32" : (w_type == COGNI_TYPE_Q8_0 ? "q8_0_gemv_mt16_f32" : "q4_k_gemv_mt16_f32"));
    const int rc = launch(kernel, gemv_mt_grid(w_type, in_dim, (uint32_t)total),
                          GEMV_MT_WAVES * 64, gemv_mt_lds_bytes(w_type) + GEMV_MT_X16_LDS_EXTRA, params, stream);
    if (rc != 0) return rc;
    i0 += n;
  }
  return 0;
}

int cogni_gemv_packed16_swiglu_dev(uint64_t w_gate, uint64_t w_up, uint32_t w_type, uint64_t image, uint64_t out, uint32_t in_dim,
                                   uint32_t out_dim, uint32_t tokens, void* stream) {
  const char* who = "cogni_gemv_packed16_swiglu_dev";
  if (!w_gate || !w_up || !image || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": null device pointer");
  if (out_dim == 0 || out_dim > 0x7FFFFFFFu) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": bad out_dim");
  if (w_type != COGNI_TYPE_Q4_K || !gemv16_shape(w_type, in_dim, tokens))
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": Q4_K, 1..16 tokens, in_dim a multiple of 256 up to 12288");
  const uint32_t groups = (out_dim + 15) / 16;
  void* params[] = {&w_gate, &w_up, &image, &out, &in_dim, &out_dim, &tokens};
  return launch("q4_k_gemv_mt16_swiglu_f32", groups < 256u ? groups : 256u, GEMV_MT_WAVES * 64,
                gemv_mt_lds_bytes(w_type) + GEMV_MT_X16_LDS_EXTRA, params, stream);
}

int cogni_gemv_packed_swiglu_dev(uint64_t w_gate, uint64_t w_up, uint32_t w_type, uint64_t image, uint64_t out, uint32_t in_dim,
                                 uint32_t out_dim, uint32_t tokens, void* stream) {
  if (!w_gate || !w_up || !image || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_swiglu_dev: null device pointer");
  if (out_dim == 0 || out_dim > 0x7FFFFFFFu) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_swiglu_dev: bad out_dim");
  if (!gemv_mt_supported(w_type, (int)tokens, in_dim) || w_type != COGNI_TYPE_Q4_K)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_swiglu_dev: no one-pass kernel for this type, token count and in_dim");
  const uint32_t groups = (out_dim + 15) / 16;
  void* params[] = {&w_gate, &w_up, &image, &out, &in_dim, &out_dim, &tokens};
  return launch("q4_k_gemv_mt_swiglu_f32", groups < 256u ? groups : 256u, GEMV_MT_WAVES * 64, gemv_mt_lds_bytes(w_type), params, stream);
}

// Token groups of up to 8 through the library's own image of `stream`: pack, then the matrices. false = not taken (no
// kernel for the shape, or every image slot belongs to another stream): the caller goes the older way.
static bool try_one_pass(const uint64_t* w_raw, uint32_t w_type, uint64_t x, uint64_t residual, const uint64_t* out,
                         const uint32_t* out_dims, uint32_t count, uint32_t in_dim, uint32_t tokens, uint32_t min_tokens,
                         void* stream, int* rc_out) {
  if (tokens < min_tokens || !gemv_mt_supported(w_type, 2, in_dim)) return false;
  const uint64_t image = image_for_stream(stream);
  if (!image) return false;
  *rc_out = 0;
  for (uint32_t t0 = 0; t0 < tokens;) {
    const uint32_t m = tokens - t0 < (uint32_t)GEMV_MT_MAX_TOKENS ? tokens - t0 : (uint32_t)GEMV_MT_MAX_TOKENS;
    uint64_t o[8];
    for (uint32_t i = 0; i < count; i++) o[i] = out[i] + (uint64_t)t0 * out_dims[i] * 4;
    const uint64_t xm = x + (uint64_t)t0 * in_dim * 4, rm = residual ? residual + (uint64_t)t0 * out_dims[0] * 4 : 0;
    if (m == 1) {   // a last single token: the one-token kernels
      for (uint32_t i = 0; i < count && *rc_out == 0; i++)
        *rc_out = cogni_gemv_dev(w_raw[i], w_type, xm, i == 0 ? rm : 0, o[i], in_dim, out_dims[i], 1, stream);
    } else {
      *rc_out = cogni_gemv_pack_dev(xm, w_type, in_dim, m, image, stream);
      if (*rc_out == 0) *rc_out = cogni_gemv_packed_dev(w_raw, w_type, image, rm, o, out_dims, count, in_dim, m, stream);
    }
    if (*rc_out != 0) return true;
    t0 += m;
  }
  return true;
}

int cogni_gemv_plan(uint32_t type, uint32_t tokens, int add, uint32_t in_dim, uint32_t out_dim, const char** kernel,
                    uint32_t* grid_x, uint32_t* block_x, uint32_t* shared_mem_bytes) {
  static thread_local char buf[64];
  if (!kernel || !grid_x || !block_x || !shared_mem_bytes || !gemv_type(type) || tokens < 1 ||
      tokens > COGNI_MAX_GEMV_TOKENS || in_dim == 0 || out_dim == 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_plan: bad argument");
  // two to four tokens of a Q4_K matrix and three or four of a Q5_K or Q6_K matrix go to the matrix-core kernels; one token
  // is faster on the vector ALU
  if (tokens >= 2 && gemv_mfma_supported(type, (int)tokens, in_dim)) {
    std::snprintf(buf, sizeof buf, "q%c_k_gemv_mfma_%sf32_tbatch%u", type == COGNI_TYPE_Q6_K ? '6' : (type == COGNI_TYPE_Q5_K ? '5' : '4'), add ? "add_" : "",
                  tokens);
    *kernel = buf;
    *grid_x = gemv_mfma_grid((int)tokens, in_dim, out_dim);
    *block_x = GEMV_MFMA_WAVES * 64;
    *shared_mem_bytes = gemv_mfma_lds_bytes(type, (int)tokens, in_dim);
    return 0;
  }
  // one token of a matrix of few rows: the variant with fewer rows per wavefront, so that 256 workgroups share the matrix
  if (tokens == 1) {
    const int r = gemv_rows_m1(type, out_dim);
    if (r * GEMV_WAVES != gemv_rows_per_block(type, 1)) {
      std::snprintf(buf, sizeof buf, "%s_gemv_%sf32_r%d", type_prefix(type), add ? "add_" : "", r);
      *kernel = buf;
      *grid_x = (out_dim + (uint32_t)(GEMV_WAVES * r) - 1) / (uint32_t)(GEMV_WAVES * r);
      *block_x = GEMV_BLOCK;
      *shared_mem_bytes = gemv_lds_bytes(type, 1, in_dim);
      return 0;
    }
  }
  *kernel = cogni_gemv_kernel_name(type, tokens, add);
  return cogni_gemv_launch_dims(type, tokens, in_dim, out_dim, grid_x, block_x, shared_mem_bytes);
}

int cogni_gemv_dev(uint64_t w_raw, uint32_t w_type, uint64_t x, uint64_t residual, uint64_t out, uint32_t in_dim,
                   uint32_t out_dim, uint32_t tokens, void* stream) {
  if (!gemv_type(w_type) && !plain_type(w_type))
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for fused matmul: ") + type_name(w_type));
  if (!w_raw || !x || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_dev: null device pointer");
  if (in_dim == 0 || out_dim == 0 || tokens == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_dev: zero dimension");
  if (plain_type(w_type)) {   // any token count in one launch: a wavefront per row, the workgroups walk the rows
    const char* name = w_type == COGNI_TYPE_F32 ? "f32_gemv_plain_f32" : (w_type == COGNI_TYPE_F16 ? "f16_gemv_plain_f32" : "iq4_nl_gemv_plain_f32");
    const uint32_t groups = (out_dim + 3) / 4;
    void* params[] = {&w_raw, &x, &residual, &out, &in_dim, &out_dim, &tokens};
    return launch(name, groups < 65536u ? groups : 65536u, 256, 0, params, stream);
  }
  if (k_quant(w_type) && (in_dim % 256) != 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(type_name(w_type)) + " GEMV requires in_dim multiple of 256, got " + std::to_string(in_dim));
  // several tokens of a matrix the one-pass kernel takes: groups of up to eight, the weights read once per group, from
  // the token count at which pack + one pass measures faster than the kernels below
  if (const uint32_t from = gemv_mt_from(w_type, in_dim, out_dim)) {
    int rc = 0;
    if (try_one_pass(&w_raw, w_type, x, residual, &out, &out_dim, 1, in_dim, tokens, from, stream, &rc)) return rc;
  }
  // tokens per launch: groups of up to 4 where the matrix-core kernel takes the shape (several passes over
  // the weights are still cheaper than one pass on the vector ALU, measured up to 8 tokens); Q8_0 up to 8; the
  // vector-ALU kernels of the K-quants hold two tokens in registers (a third costs a second pass over the staged
  // weights, a fourth as much as the first two: Q6_K 4096x12288 takes 10.6 / 14.9 / 23.6 / 43.0 us for 1 / 2 / 3 / 4
  // tokens), so they go in pairs, with one group of three when the count is odd
  uint32_t cap = k_quant(w_type) ? 2u : (uint32_t)COGNI_MAX_GEMV_TOKENS;
  bool pairs = k_quant(w_type);
  for (int mt = GEMV_MFMA_MAX_TOKENS; mt >= 2; mt--) {
    if (gemv_mfma_supported(w_type, mt, in_dim)) {   // the most tokens whose activations fit its staging buffer
      cap = (uint32_t)mt;
      pairs = false;
      break;
    }
  }
  uint32_t m = 0;
  for (uint32_t t0 = 0; t0 < tokens; t0 += m) {
    const uint32_t left = tokens - t0;
    m = left < cap ? left : cap;
    // an odd count ends in a group of three, except on a matrix long enough for the pair kernel to walk its row groups
    // (there a pair and a single token are faster: Q6_K 151936 x 4096 158 + 96 us against 283)
    const bool walks = (uint64_t)gemv_grid(w_type, 2, out_dim) * (uint32_t)gemv_rows_per_block(w_type, 2) < out_dim;
    if (pairs && left == 3 && !walks) m = 3;
    uint32_t grid = 0, block = 0, shmem = 0;
    const char* kernel = nullptr;
    int rc = cogni_gemv_plan(w_type, m, residual != 0, in_dim, out_dim, &kernel, &grid, &block, &shmem);
    if (rc != 0) return rc;
    const std::string name = kernel;
    uint64_t xm = x + (uint64_t)t0 * in_dim * 4, om = out + (uint64_t)t0 * out_dim * 4;
    uint64_t rm = residual ? residual + (uint64_t)t0 * out_dim * 4 : 0;
    if (residual) {
      void* params[] = {&w_raw, &xm, &rm, &om, &in_dim, &out_dim};
      rc = launch(name.c_str(), grid, block, shmem, params, stream);
    } else {
      void* params[] = {&w_raw, &xm, &om, &in_dim, &out_dim};
      rc = launch(name.c_str(), grid, block, shmem, params, stream);
    }
    if (rc != 0) return rc;
  }
  return 0;
}

int cogni_gemv_dual_dev(uint64_t w_raw_a, uint64_t w_raw_b, uint32_t w_type, uint64_t x, uint64_t out_a, uint64_t out_b,
                        uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream) {
  if (!gemv_type(w_type))
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for fused matmul: ") + type_name(w_type));
  if (!w_raw_a || !w_raw_b || !x || !out_a || !out_b)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_dual_dev: null device pointer");
  if (in_dim == 0 || out_dim == 0 || tokens == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_dual_dev: zero dimension");
  if (w_type == COGNI_TYPE_Q4_K && tokens == 1 && (in_dim % 256) == 0) {
    uint32_t grid = 0, block = 0, shmem = 0;
    int rc = cogni_gemv_launch_dims(w_type, 1, in_dim, out_dim, &grid, &block, &shmem);
    if (rc != 0) return rc;
    const uint32_t rows = GEMV_WAVES * GEMV_ROWS_Q4K_PAIR;
    grid = (2 * out_dim + rows - 1) / rows;
    void* params[] = {&w_raw_a, &w_raw_b, &x, &out_a, &out_b, &in_dim, &out_dim};
    return launch("q4_k_dual_gemv_f32", grid, block, shmem, params, stream);
  }
  // several tokens of a pair the one-pass kernel takes: the activations packed once, both matrices in one launch
  if (const uint32_t from = gemv_mt_multi_from(w_type, in_dim); from && tokens >= from) {
    const uint64_t ws[2] = {w_raw_a, w_raw_b}, os[2] = {out_a, out_b};
    const uint32_t dims[2] = {out_dim, out_dim};
    int rc = 0;
    if (try_one_pass(ws, w_type, x, 0, os, dims, 2, in_dim, tokens, from, stream, &rc)) return rc;
  }
  // several tokens of a Q4_K pair whose shape the matrix-core kernel takes: groups of up to four tokens, the two
  // matrices as one of 2 * out_dim rows (the activations are staged once for both); a last single token goes to the
  // one-token pair kernel
  if (w_type == COGNI_TYPE_Q4_K && tokens >= 2 && (in_dim % 256) == 0 && (out_dim % 16) == 0 && out_dim <= 0x7FFFFFFFu) {
    uint32_t cap = 0;
    for (int mt = GEMV_MFMA_MAX_TOKENS; mt >= 2 && cap == 0; mt--)
      if (gemv_mfma_supported(w_type, mt, in_dim)) cap = (uint32_t)mt;
    if (cap != 0) {
      uint32_t m = 0;
      for (uint32_t t0 = 0; t0 < tokens; t0 += m) {
        const uint32_t left = tokens - t0;
        m = left < cap ? left : cap;
        uint64_t xm = x + (uint64_t)t0 * in_dim * 4, oa = out_a + (uint64_t)t0 * out_dim * 4, ob = out_b + (uint64_t)t0 * out_dim * 4;
        int rc = 0;
        if (m == 1) {
          rc = cogni_gemv_dual_dev(w_raw_a, w_raw_b, w_type, xm, oa, ob, in_dim, out_dim, 1, stream);
        } else {
          const uint32_t grid = gemv_mfma_grid((int)m, in_dim, 2 * out_dim);
          const std::string name = "q4_k_dual_gemv_mfma_f32_tbatch" + std::to_string(m);
          void* params[] = {&w_raw_a, &w_raw_b, &xm, &oa, &ob, &in_dim, &out_dim};
          rc = launch(name.c_str(), grid, GEMV_MFMA_WAVES * 64, gemv_mfma_lds_bytes(w_type, (int)m, in_dim), params, stream);
        }
        if (rc != 0) return rc;
      }
      return 0;
    }
  }
  // other types and shapes: the pair as two launches of the kernels cogni_gemv_dev picks
  int rc = cogni_gemv_dev(w_raw_a, w_type, x, 0, out_a, in_dim, out_dim, tokens, stream);
  if (rc != 0) return rc;
  return cogni_gemv_dev(w_raw_b, w_type, x, 0, out_b, in_dim, out_dim, tokens, stream);
}

int cogni_gemv_many_dev(const uint64_t* w_raw, uint32_t w_type, uint64_t x, const uint64_t* out, const uint32_t* out_dims,
                        uint32_t count, uint32_t in_dim, uint32_t tokens, void* stream) {
  if (!gemv_type(w_type))
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for fused matmul: ") + type_name(w_type));
  if (!w_raw || !out || !out_dims || !x) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_many_dev: null argument");
  if (count == 0 || count > 8) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_many_dev: count must be 1..8");
  if (in_dim == 0 || tokens == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_many_dev: zero dimension");
  uint64_t total = 0;
  bool aligned = true;
  for (uint32_t i = 0; i < count; i++) {
    if (!w_raw[i] || !out[i] || out_dims[i] == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_many_dev: null pointer or zero rows");
    total += out_dims[i];
    aligned = aligned && (out_dims[i] % 16) == 0;
  }
  if (const uint32_t from = gemv_mt_multi_from(w_type, in_dim); from && count >= 2 && tokens >= from) {
    // the one-pass kernel: one image for all of them, up to three matrices per launch
    int rc = 0;
    if (try_one_pass(w_raw, w_type, x, 0, out, out_dims, count, in_dim, tokens, from, stream, &rc)) return rc;
  }
  if (count == 2 && out_dims[0] == out_dims[1])
    return cogni_gemv_dual_dev(w_raw[0], w_raw[1], w_type, x, out[0], out[1], in_dim, out_dims[0], tokens, stream);
  // one token of several Q4_K matrices: up to three per launch as one matrix of all their rows (q | k | v: one launch and
  // one staging of x instead of three)
  if (tokens == 1 && w_type == COGNI_TYPE_Q4_K && (in_dim % 256) == 0 && total <= 0x7FFFFFFFull) {
    for (uint32_t i0 = 0; i0 < count; i0 += 3) {
      const uint32_t n = count - i0 < 3 ? count - i0 : 3;
      int rc;
      if (n == 1) {
        rc = cogni_gemv_dev(w_raw[i0], w_type, x, 0, out[i0], in_dim, out_dims[i0], 1, stream);
      } else {
        uint64_t w[3] = {w_raw[i0], w_raw[i0 + 1], n > 2 ? w_raw[i0 + 2] : 0};
        uint64_t o[3] = {out[i0], out[i0 + 1], n > 2 ? out[i0 + 2] : 0};
        uint32_t rows[3] = {out_dims[i0], out_dims[i0 + 1], n > 2 ? out_dims[i0 + 2] : 0};
        uint32_t grid = 0, block = 0, shmem = 0;
        rc = cogni_gemv_launch_dims(w_type, 1, in_dim, rows[0] + rows[1] + rows[2], &grid, &block, &shmem);
        if (rc != 0) return rc;
        void* params[] = {&w[0], &w[1], &w[2], &x, &o[0], &o[1], &o[2], &in_dim, &rows[0], &rows[1], &rows[2]};
        rc = launch("q4_k_many_gemv_f32", grid, block, shmem, params, stream);
      }
      if (rc != 0) return rc;
    }
    return 0;
  }
  uint32_t cap = 0;
  if (w_type == COGNI_TYPE_Q4_K && (count == 2 || count == 3) && tokens >= 2 && aligned && (in_dim % 256) == 0 && total <= 0x7FFFFFFFull)
    for (int mt = GEMV_MFMA_MAX_TOKENS; mt >= 2 && cap == 0; mt--)
      if (gemv_mfma_supported(w_type, mt, in_dim)) cap = (uint32_t)mt;
  if (cap == 0) {
    for (uint32_t i = 0; i < count; i++) {
      const int rc = cogni_gemv_dev(w_raw[i], w_type, x, 0, out[i], in_dim, out_dims[i], tokens, stream);
      if (rc != 0) return rc;
    }
    return 0;
  }
  uint32_t m = 0;
  for (uint32_t t0 = 0; t0 < tokens; t0 += m) {
    const uint32_t left = tokens - t0;
    m = left < cap ? left : cap;
    uint64_t xm = x + (uint64_t)t0 * in_dim * 4;
    if (m == 1) {   // a last single token: one launch per matrix
      for (uint32_t i = 0; i < count; i++) {
        const int rc = cogni_gemv_dev(w_raw[i], w_type, xm, 0, out[i] + (uint64_t)t0 * out_dims[i] * 4, in_dim, out_dims[i], 1, stream);
        if (rc != 0) return rc;
      }
      continue;
    }
    uint64_t w[3] = {w_raw[0], w_raw[1], count > 2 ? w_raw[2] : 0};
    uint64_t o[3] = {out[0] + (uint64_t)t0 * out_dims[0] * 4, out[1] + (uint64_t)t0 * out_dims[1] * 4,
                     count > 2 ? out[2] + (uint64_t)t0 * out_dims[2] * 4 : 0};
    uint32_t rows[3] = {out_dims[0], out_dims[1], count > 2 ? out_dims[2] : 0};
    const uint32_t grid = gemv_mfma_grid((int)m, in_dim, (uint32_t)total);
    const std::string name = "q4_k_many_gemv_mfma_f32_tbatch" + std::to_string(m);
    void* params[] = {&w[0], &w[1], &w[2], &xm, &o[0], &o[1], &o[2], &in_dim, &rows[0], &rows[1], &rows[2]};
    const int rc = launch(name.c_str(), grid, GEMV_MFMA_WAVES * 64, gemv_mfma_lds_bytes(w_type, (int)m, in_dim), params, stream);
    if (rc != 0) return rc;
  }
  return 0;
}

int cogni_swiglu_dev(uint64_t gate, uint64_t up, uint64_t out, uint32_t n, void* stream) {
  if (!gate || !up || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_swiglu_dev: null device pointer");
  if (n == 0) return 0;
  void* params[] = {&gate, &up, &out, &n};
  return launch("swiglu_f32", (n + 255) / 256, 256, 0, params, stream);
}

int cogni_gemv_dual_swiglu_dev(uint64_t w_gate, uint64_t w_up, uint32_t w_type, uint64_t x, uint64_t out, uint32_t in_dim,
                               uint32_t out_dim, uint32_t tokens, void* stream) {
  if (w_type != COGNI_TYPE_Q4_K)
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for the fused gate/up SwiGLU: ") + type_name(w_type));
  if (!w_gate || !w_up || !x || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_dual_swiglu_dev: null device pointer");
  if (in_dim == 0 || out_dim == 0 || tokens == 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_dual_swiglu_dev: zero dimension");
  if ((in_dim % 256) != 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "Q4_K GEMV requires in_dim multiple of 256, got " + std::to_string(in_dim));
  // several tokens of a pair the one-pass kernel takes: the activations packed once per group of up to eight tokens, gate
  // tile and up tile side by side in a workgroup, which stores silu(gate) * up
  if (const uint32_t from = gemv_mt_multi_from(w_type, in_dim); from && tokens >= from && out_dim <= 0x7FFFFFFFu) {
    const uint64_t image = image_for_stream(stream);
    if (image) {
      for (uint32_t t0 = 0; t0 < tokens;) {
        const uint32_t m = tokens - t0 < (uint32_t)GEMV_MT_MAX_TOKENS ? tokens - t0 : (uint32_t)GEMV_MT_MAX_TOKENS;
        const uint64_t xm = x + (uint64_t)t0 * in_dim * 4, om = out + (uint64_t)t0 * out_dim * 4;
        int rc;
        if (m == 1) {
          rc = cogni_gemv_dual_swiglu_dev(w_gate, w_up, w_type, xm, om, in_dim, out_dim, 1, stream);
        } else {
          rc = cogni_gemv_pack_dev(xm, w_type, in_dim, m, image, stream);
          if (rc == 0) rc = cogni_gemv_packed_swiglu_dev(w_gate, w_up, w_type, image, om, in_dim, out_dim, m, stream);
        }
        if (rc != 0) return rc;
        t0 += m;
      }
      return 0;
    }
  }
  // several tokens, out_dim a multiple of 16 and a row length the matrix-core kernel takes: groups of up to four tokens
  // on the matrix cores (gate tile and up tile side by side in a wavefront, two tiles per wavefront, 256 workgroups at
  // most, which walk the row groups with the activations staged once); a last single token as below
  uint32_t cap = 0;
  if (tokens >= 2 && (out_dim % 16) == 0 && out_dim <= 0x7FFFFFFFu)
    for (int mt = GEMV_MFMA_MAX_TOKENS; mt >= 2 && cap == 0; mt--)
      if (gemv_mfma_supported(w_type, mt, in_dim)) cap = (uint32_t)mt;
  if (cap != 0) {
    uint32_t m = 0;
    for (uint32_t t0 = 0; t0 < tokens; t0 += m) {
      const uint32_t left = tokens - t0;
      m = left < cap ? left : cap;
      uint64_t xm = x + (uint64_t)t0 * in_dim * 4, om = out + (uint64_t)t0 * out_dim * 4;
      int rc = 0;
      if (m == 1) {
        rc = cogni_gemv_dual_swiglu_dev(w_gate, w_up, w_type, xm, om, in_dim, out_dim, 1, stream);
      } else {
        const uint32_t nwr = GEMV_MFMA_WAVES >> gemv_mfma_log2_kslices(in_dim >> 8);
        const uint32_t groups = (out_dim / 16 + nwr - 1) / nwr;   // pairs of tiles, one pair per wavefront
        const uint32_t g = gemv_mfma_chunked((int)m, in_dim) || groups <= 256u ? groups : 256u;
        const std::string name = "q4_k_dual_gemv_swiglu_mfma_f32_tbatch" + std::to_string(m);
        void* params[] = {&w_gate, &w_up, &xm, &om, &in_dim, &out_dim};
        rc = launch(name.c_str(), g, GEMV_MFMA_WAVES * 64, gemv_mfma_lds_bytes(w_type, (int)m, in_dim), params, stream);
      }
      if (rc != 0) return rc;
    }
    return 0;
  }
  uint32_t grid = 0, block = 0, shmem = 0;
  int rc = cogni_gemv_launch_dims(w_type, 1, in_dim, out_dim, &grid, &block, &shmem);
  if (rc != 0) return rc;
  const uint32_t rows = GEMV_WAVES * GEMV_ROWS_Q4K_PAIR / 2;   // gate rows per workgroup (as many of up)
  grid = (out_dim + rows - 1) / rows;
  void* params[] = {&w_gate, &w_up, &x, &out, &in_dim, &out_dim};
  return launch("q4_k_dual_gemv_swiglu_f32", grid, block, shmem, params, stream, tokens);
}

int cogni_embed_dev(uint64_t w_raw, uint32_t w_type, uint64_t token_ids, uint64_t output, uint64_t history,
                    uint32_t token_index, uint32_t hidden_dim, uint32_t vocab_size, void* stream) {
  if (w_type != COGNI_TYPE_Q4_K && w_type != COGNI_TYPE_Q6_K)
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("GPU token embedding requires Q4_K or Q6_K token embeddings, got ") + type_name(w_type));
  if (!w_raw || !token_ids || !output || !history) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_embed_dev: null device pointer");
  if (hidden_dim == 0 || (hidden_dim % 256) != 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "embedding dim " + std::to_string(hidden_dim) + " must be divisible by 256");
  const std::string name = std::string("embed_") + type_prefix(w_type) + "_f32_from_token_id";
  void* params[] = {&w_raw, &token_ids, &output, &history, &token_index, &hidden_dim, &vocab_size};
  return launch(name.c_str(), (hidden_dim + 1023) / 1024, 256, 0, params, stream);
}

// ---- output head: GEMV with the arg-max over the rows ---------------------------------------------------
// tokens per launch: two for the types that have the kernel (a pair shares one pass over the weights and, on a long
// matrix, walks the row groups with the activations staged once; a third token would be a second token group with its
// own staging: Q6_K 151936 x 4096 takes 100 / 168 / 310 us for 1 / 2 / 3 tokens)
static uint32_t top1_token_cap(uint32_t type) { return (type == COGNI_TYPE_Q4_K || type == COGNI_TYPE_Q6_K) ? 2u : 1u; }

uint32_t cogni_gemv_top1_partials(uint32_t w_type, uint32_t out_dim) {
  if (!gemv_type(w_type) || out_dim == 0) return 0;
  uint32_t most = 0;
  for (uint32_t m = 1; m <= top1_token_cap(w_type); m++) {
    const uint32_t grid = gemv_grid(w_type, (int)m, out_dim);
    if (grid > most) most = grid;
  }
  return most;
}

int cogni_gemv_top1_dev(uint64_t w_raw, uint32_t w_type, uint64_t x, uint64_t partial_ids, uint64_t partial_values,
                        uint64_t top1_ids, uint64_t top1_values, uint32_t in_dim, uint32_t out_dim, uint32_t tokens,
                        void* stream) {
  if (!gemv_type(w_type))
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for fused matmul: ") + type_name(w_type));
  if (!w_raw || !x || !partial_ids || !partial_values || !top1_ids || !top1_values)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_top1_dev: null device pointer");
  if (in_dim == 0 || out_dim == 0 || tokens == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_top1_dev: zero dimension");
  if (k_quant(w_type) && (in_dim % 256) != 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(type_name(w_type)) + " GEMV requires in_dim multiple of 256, got " + std::to_string(in_dim));
  const uint32_t cap = top1_token_cap(w_type), stride = cogni_gemv_top1_partials(w_type, out_dim);
  uint32_t m = 0;
  for (uint32_t t0 = 0; t0 < tokens; t0 += m) {
    const uint32_t left = tokens - t0;
    m = left < cap ? left : cap;
    uint32_t grid = 0, block = 0, shmem = 0;
    std::string name;
    int rc = 0;
    // the group's partial results: [token in group][workgroup], inside the group's share of the caller's buffers
    uint64_t xm = x + (uint64_t)t0 * in_dim * 4, pi = partial_ids + (uint64_t)t0 * stride * 4, pv = partial_values + (uint64_t)t0 * stride * 4;
    uint64_t oi = top1_ids + (uint64_t)t0 * 4, ov = top1_values + (uint64_t)t0 * 4;
    // up to eight tokens of a Q4_K or Q6_K matrix the one-pass kernel takes, from the token count at which pack + one
    // pass is the faster way to the logits: the weights once for the whole group, the arg-max inside
    const uint32_t from = (w_type == COGNI_TYPE_Q4_K || w_type == COGNI_TYPE_Q6_K) ? gemv_mt_from(w_type, in_dim, out_dim) : 0;
    const uint32_t m8 = left < (uint32_t)GEMV_MT_MAX_TOKENS ? left : (uint32_t)GEMV_MT_MAX_TOKENS;
    if (from && m8 >= from && gemv_mt_grid(w_type, in_dim, out_dim) <= stride) {
      if (uint64_t image = image_for_stream(stream)) {
        m = m8;
        grid = gemv_mt_grid(w_type, in_dim, out_dim);
        rc = cogni_gemv_pack_dev(xm, w_type, in_dim, m, image, stream);
        if (rc != 0) return rc;
        void* params[] = {&w_raw, &image, &pi, &pv, &in_dim, &out_dim, &m};
        rc = launch(w_type == COGNI_TYPE_Q6_K ? "q6_k_gemv_mt_top1_partial_f32" : "q4_k_gemv_mt_top1_partial_f32", grid,
                    GEMV_MT_WAVES * 64, gemv_mt_lds_bytes(w_type), params, stream);
        if (rc != 0) return rc;
        void* rparams[] = {&pi, &pv, &oi, &ov, &grid};
        rc = launch("top1_reduce_f32", m, 1024, 0, rparams, stream);
        if (rc != 0) return rc;
        continue;
      }
    }
    // three or four tokens of a Q4_K or Q6_K matrix: the matrix-core kernel with the arg-max inside, where its
    // workgroups fit the caller's partial buffers (sized for the vector-ALU kernels)
    const uint32_t mm = left < (uint32_t)GEMV_MFMA_MAX_TOKENS ? left : (uint32_t)GEMV_MFMA_MAX_TOKENS;
    if (mm >= 3 && (w_type == COGNI_TYPE_Q4_K || w_type == COGNI_TYPE_Q6_K) && gemv_mfma_supported(w_type, (int)mm, in_dim) &&
        gemv_mfma_grid((int)mm, in_dim, out_dim) <= stride) {
      m = mm;
      grid = gemv_mfma_grid((int)m, in_dim, out_dim);
      block = GEMV_MFMA_WAVES * 64;
      shmem = gemv_mfma_lds_bytes(w_type, (int)m, in_dim);
      name = std::string(type_prefix(w_type)) + "_gemv_mfma_top1_partial_f32_tbatch" + std::to_string(m);
    } else {
      rc = cogni_gemv_launch_dims(w_type, m, in_dim, out_dim, &grid, &block, &shmem);
      if (rc != 0) return rc;
      name = std::string(type_prefix(w_type)) + "_gemv_top1_partial_f32";
      if (m > 1) name += "_tbatch" + std::to_string(m);
    }
    void* params[] = {&w_raw, &xm, &pi, &pv, &in_dim, &out_dim};
    rc = launch(name.c_str(), grid, block, shmem, params, stream);
    if (rc != 0) return rc;
    void* rparams[] = {&pi, &pv, &oi, &ov, &grid};
    rc = launch("top1_reduce_f32", m, 1024, 0, rparams, stream);
    if (rc != 0) return rc;
  }
  return 0;
}

int cogni_gemv_packed_top1_dev(uint64_t w_raw, uint32_t w_type, uint64_t image, uint64_t partial_ids, uint64_t partial_values,
                               uint64_t top1_ids, uint64_t top1_values, uint32_t in_dim, uint32_t out_dim, uint32_t tokens,
                               void* stream) {
  if (!w_raw || !image || !partial_ids || !partial_values || !top1_ids || !top1_values)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_top1_dev: null device pointer");
  if (out_dim == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_top1_dev: zero dimension");
  if ((w_type != COGNI_TYPE_Q4_K && w_type != COGNI_TYPE_Q6_K) || tokens == 0 || tokens > (uint32_t)GEMV_MT_MAX_TOKENS ||
      !gemv_mt_supported(w_type, 2, in_dim))
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_top1_dev: no one-pass top-1 kernel for this type, token count and in_dim");
  uint32_t grid = gemv_mt_grid(w_type, in_dim, out_dim);
  if (grid > cogni_gemv_top1_partials(w_type, out_dim))
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemv_packed_top1_dev: the partial buffers are sized by cogni_gemv_top1_partials");
  void* params[] = {&w_raw, &image, &partial_ids, &partial_values, &in_dim, &out_dim, &tokens};
  int rc = launch(w_type == COGNI_TYPE_Q6_K ? "q6_k_gemv_mt_top1_partial_f32" : "q4_k_gemv_mt_top1_partial_f32", grid,
                  GEMV_MT_WAVES * 64, gemv_mt_lds_bytes(w_type), params, stream);
  if (rc != 0) return rc;
  void* rparams[] = {&partial_ids, &partial_values, &top1_ids, &top1_values, &grid};
  return launch("top1_reduce_f32", tokens, 1024, 0, rparams, stream);
}

int cogni_rmsnorm_dev(uint64_t x, uint64_t norm, uint64_t out, uint32_t dim, uint32_t tokens, float eps, void* stream) {
  if (!x || !norm || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_rmsnorm_dev: null device pointer");
  if (dim == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_rmsnorm_dev: zero dimension");
  if (tokens == 0) return 0;
  void* params[] = {&x, &norm, &out, &dim, &eps};
  return launch("rmsnorm_f32", tokens, 256, 0, params, stream);
}

int cogni_add_rmsnorm_dev(uint64_t x, uint64_t add, uint64_t norm, uint64_t residual_out, uint64_t normed_out, uint32_t dim,
                          uint32_t tokens, float eps, void* stream) {
  if (!x || !add || !norm || !residual_out || !normed_out)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_add_rmsnorm_dev: null device pointer");
  if (dim == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_add_rmsnorm_dev: zero dimension");
  if (tokens == 0) return 0;
  void* params[] = {&x, &add, &norm, &residual_out, &normed_out, &dim, &eps};
  return launch("add_rmsnorm_f32", tokens, 256, 0, params, stream);
}

// The norms with the activation image of the one-pass GEMV as a second output (norm.hpp): dim must be a shape those
// kernels take with rows short enough for a thread to keep its values (a multiple of 256 up to 4096).
static int norm_pack_check(const char* who, uint32_t w_type, uint32_t dim, uint32_t tokens) {
  if (!gemv_mt_supported(w_type, tokens < 2 ? 2 : (int)tokens, dim) || dim > 4096u || tokens == 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": needs 1..8 tokens of a row length the one-pass GEMV takes, up to 4096 "
                                                               "(cogni_gemv_image_bytes) - got type " + type_name(w_type) + ", dim " +
                                                std::to_string(dim) + ", " + std::to_string(tokens) + " tokens");
  return 0;
}
int cogni_rmsnorm_pack_dev(uint64_t x, uint64_t norm, uint64_t out, uint32_t w_type, uint64_t image, uint32_t dim, uint32_t tokens,
                           float eps, void* stream) {
  if (!x || !norm || !image) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_rmsnorm_pack_dev: null device pointer");
  if (int rc = norm_pack_check("cogni_rmsnorm_pack_dev", w_type, dim, tokens)) return rc;
  void* params[] = {&x, &norm, &out, &image, &dim, &tokens, &eps};
  return launch(w_type == COGNI_TYPE_Q6_K ? "rmsnorm_pack_q6k_f32" : "rmsnorm_pack_q4k_f32", GEMV_MT_MAX_TOKENS, 256, 0, params, stream);
}
int cogni_add_rmsnorm_pack_dev(uint64_t x, uint64_t add, uint64_t norm, uint64_t residual_out, uint64_t normed_out, uint32_t w_type,
                               uint64_t image, uint32_t dim, uint32_t tokens, float eps, void* stream) {
  if (!x || !add || !norm || !residual_out || !image)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_add_rmsnorm_pack_dev: null device pointer");
  if (int rc = norm_pack_check("cogni_add_rmsnorm_pack_dev", w_type, dim, tokens)) return rc;
  void* params[] = {&x, &add, &norm, &residual_out, &normed_out, &image, &dim, &tokens, &eps};
  return launch(w_type == COGNI_TYPE_Q6_K ? "add_rmsnorm_pack_q6k_f32" : "add_rmsnorm_pack_q4k_f32", GEMV_MT_MAX_TOKENS, 256, 0, params, stream);
}

// the same norms in front of the sixteen-token one-pass kernels (the image of cogni_gemv_pack16_dev)
static int norm_pack16_check(const char* who, uint32_t w_type, uint32_t dim, uint32_t tokens) {
  if (!(w_type == COGNI_TYPE_Q4_K || w_type == COGNI_TYPE_Q5_K || w_type == COGNI_TYPE_Q6_K) || tokens == 0 || tokens > 16 ||
      !gemv_mt_supported(w_type, 2, dim) || dim > 4096u)
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": needs 1..16 tokens of a Q4_K, Q5_K or Q6_K row length that is a multiple of 256 "
                                                               "up to 4096 - got type " + type_name(w_type) + ", dim " + std::to_string(dim) +
                                                ", " + std::to_string(tokens) + " tokens");
  return 0;
}
int cogni_rmsnorm_pack16_dev(uint64_t x, uint64_t norm, uint64_t out, uint32_t w_type, uint64_t image, uint32_t dim, uint32_t tokens,
                             float eps, void* stream) {
  if (!x || !norm || !image) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_rmsnorm_pack16_dev: null device pointer");
  if (int rc = norm_pack16_check("cogni_rmsnorm_pack16_dev", w_type, dim, tokens)) return rc;
  void* params[] = {&x, &norm, &out, &image, &dim, &tokens, &eps};
  return launch(w_type == COGNI_TYPE_Q6_K ? "rmsnorm_pack_x16_q6k_f32" : "rmsnorm_pack_x16_q4k_f32", 16, 256, 0, params, stream);
}
int cogni_add_rmsnorm_pack16_dev(uint64_t x, uint64_t add, uint64_t norm, uint64_t residual_out, uint64_t normed_out, uint32_t w_type,
                                 uint64_t image, uint32_t dim, uint32_t tokens, float eps, void* stream) {
  if (!x || !add || !norm || !residual_out || !image)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_add_rmsnorm_pack16_dev: null device pointer");
  if (int rc = norm_pack16_check("cogni_add_rmsnorm_pack16_dev", w_type, dim, tokens)) return rc;
  void* params[] = {&x, &add, &norm, &residual_out, &normed_out, &image, &dim, &tokens, &eps};
  return launch(w_type == COGNI_TYPE_Q6_K ? "add_rmsnorm_pack_x16_q6k_f32" : "add_rmsnorm_pack_x16_q4k_f32", 16, 256, 0, params, stream);
}

int g_gemm_threshold = -1;   // -1: not resolved yet

static bool gemm_type(uint32_t t) { return t == COGNI_TYPE_Q4_K || t == COGNI_TYPE_Q5_K || t == COGNI_TYPE_Q6_K; }

size_t cogni_gemm_workspace_bytes(uint32_t w_type, uint32_t in_dim, uint32_t tokens) {
  if (!gemm_type(w_type) || in_dim == 0 || tokens == 0) return 0;
  const size_t mtiles = ((size_t)tokens + 127) / 128;
  return mtiles * 128 * (size_t)in_dim * 2;
}

// The norms that write the packed activations of the prefill GEMMs (kernels/norm.hpp): one workgroup per token of whole
// 128-token tiles, rows of the short-row path.
static int norm_gemm_pack_check(const char* who, uint32_t w_type, uint32_t dim, uint32_t tokens, uint64_t workspace, size_t workspace_bytes) {
  if (!gemm_type(w_type))
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for the prefill GEMM: ") + type_name(w_type));
  if (dim == 0 || tokens == 0 || (dim % 256) != 0 || dim > 4096)
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": dim must be a multiple of 256 up to 4096, tokens at least 1");
  const size_t need = cogni_gemm_workspace_bytes(w_type, dim, tokens);
  if (!workspace || workspace_bytes < need)
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": workspace has " + std::to_string(workspace_bytes) + " bytes, needs " + std::to_string(need));
  return 0;
}
int cogni_rmsnorm_gemm_pack_dev(uint64_t x, uint64_t norm, uint64_t out, uint32_t w_type, uint64_t workspace, size_t workspace_bytes,
                                uint32_t dim, uint32_t tokens, float eps, void* stream) {
  if (!x || !norm) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_rmsnorm_gemm_pack_dev: null device pointer");
  if (int rc = norm_gemm_pack_check("cogni_rmsnorm_gemm_pack_dev", w_type, dim, tokens, workspace, workspace_bytes)) return rc;
  void* params[] = {&x, &norm, &out, &workspace, &dim, &tokens, &eps};
  return launch(w_type == COGNI_TYPE_Q6_K ? "rmsnorm_gemm_pack_q6k_f32" : "rmsnorm_gemm_pack_q4k_f32", 128 * ((tokens + 127) / 128), 256, 0,
                params, stream);
}
int cogni_add_rmsnorm_gemm_pack_dev(uint64_t x, uint64_t add, uint64_t norm, uint64_t residual_out, uint64_t normed_out, uint32_t w_type,
                                    uint64_t workspace, size_t workspace_bytes, uint32_t dim, uint32_t tokens, float eps, void* stream) {
  if (!x || !add || !norm || !residual_out)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_add_rmsnorm_gemm_pack_dev: null device pointer");
  if (int rc = norm_gemm_pack_check("cogni_add_rmsnorm_gemm_pack_dev", w_type, dim, tokens, workspace, workspace_bytes)) return rc;
  void* params[] = {&x, &add, &norm, &residual_out, &normed_out, &workspace, &dim, &tokens, &eps};
  return launch(w_type == COGNI_TYPE_Q6_K ? "add_rmsnorm_gemm_pack_q6k_f32" : "add_rmsnorm_gemm_pack_q4k_f32", 128 * ((tokens + 127) / 128),
                256, 0, params, stream);
}

// k splits of the prefill GEMM: a launch of fewer than half as many tiles as there are compute units (256) leaves most
// of them idle, so the super-blocks of a row are divided among up to 8 workgroups per tile, each with at least two
// super-blocks; the partial sums go through the workspace.
static uint32_t gemm_splits_of(uint32_t tiles, uint32_t in_dim) {
  const uint32_t nkb = in_dim / 256;
  uint32_t s = 256u / tiles;
  if (s > 8) s = 8;
  if (s > nkb / 2) s = nkb / 2;
  return s < 2 ? 1 : s;
}
// Rows of the workgroup tile and k splits of a launch. Every type has two tile heights, 192 and 128 rows (<type>_gemm_f16 and
// <type>_gemm_n128_f16), Q4_K also the 256-row tile of the eight-wavefront kernel (no k split). A launch runs in rounds of
// 256 workgroups and a workgroup walks ceil(super-blocks / splits) super-blocks; per super-block a 128-row tile costs
// GEMM_N128_COST_X100 per cent of a 192-row one and a 256-row tile GEMM_WIDE_ROUND_COST_X100 per cent; the cheapest plan wins
// (the 4096-row projections at 512 tokens: 88 tiles x 2 splits = 176 workgroups of 192 rows, or 128 x 2 = 256 of the
// smaller ones). `split` false: the plan for a workspace without planes. COGNI_GEMM_N128=0 | 1 and COGNI_GEMM_WIDE=0 | 1
// override the choice (measurement knobs: 1 takes that tile wherever its kernel can run).
#define GEMM_N128_COST_X100 75u
struct GemmShape {
  uint32_t bn, splits;
};
static GemmShape gemm_shape(uint32_t w_type, uint32_t in_dim, uint32_t out_dim, uint32_t tokens, bool split = true) {
  const uint32_t mtiles = (tokens + 127) / 128, nkb = in_dim / 256;
  auto eval = [&](uint32_t bn, uint32_t cost_x100, uint32_t* cost) {
    const uint32_t tiles = mtiles * ((out_dim + bn - 1) / bn), s = split && bn != 256 ? gemm_splits_of(tiles, in_dim) : 1u;
    *cost = ((tiles * s + 255u) / 256u) * ((nkb + s - 1) / s) * cost_x100;
    return s;
  };
  uint32_t cost192 = 0, cost128 = 0, cost256 = 0;
  const uint32_t s192 = eval(192, 100u, &cost192), s128 = eval(128, GEMM_N128_COST_X100, &cost128);
  bool n128 = cost128 < cost192;
  if (const char* e = std::getenv("COGNI_GEMM_N128")) {
    if (e[0] == '0') n128 = false;
    if (e[0] == '1') n128 = true;
  }
  GemmShape best = n128 ? GemmShape{128, s128} : GemmShape{192, s192};
  // the eight-wavefront kernel: Q4_K launches that are not split and fill whole rounds of its tiles
  if (w_type == COGNI_TYPE_Q4_K && best.splits == 1) {
    (void)eval(256, GEMM_WIDE_ROUND_COST_X100, &cost256);
    bool wide = gemm_q4k_use_wide(out_dim, tokens) && cost256 < (n128 ? cost128 : cost192);
    if (const char* e = std::getenv("COGNI_GEMM_WIDE")) {
      if (e[0] == '0') wide = false;
      if (e[0] == '1') wide = true;
    }
    if (wide) best = GemmShape{256, 1};
  }
  return best;
}

size_t cogni_gemm_workspace_bytes_split(uint32_t w_type, uint32_t in_dim, uint32_t out_dim, uint32_t tokens) {
  const size_t pack = cogni_gemm_workspace_bytes(w_type, in_dim, tokens);
  if (pack == 0 || out_dim == 0 || (in_dim % 256) != 0) return pack;
  const uint32_t s = gemm_shape(w_type, in_dim, out_dim, tokens).splits;
  return s == 1 ? pack : pack + (size_t)s * tokens * out_dim * sizeof(float);
}

// The two halves of cogni_gemm_dev. `who` names the entry point in messages.
static int gemm_check(const char* who, uint32_t w_type, uint32_t in_dim, uint32_t out_dim, uint32_t tokens, uint64_t workspace,
                      size_t workspace_bytes) {
  if (!gemm_type(w_type))
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for the prefill GEMM: ") + type_name(w_type));
  if (in_dim == 0 || out_dim == 0 || tokens == 0) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": zero dimension");
  if ((in_dim % 256) != 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(type_name(w_type)) + " GEMM requires in_dim multiple of 256, got " + std::to_string(in_dim));
  if ((uint64_t)tokens * out_dim > 0xFFFFFFFFull)
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": tokens * out_dim exceeds 2^32 - 1");
  const size_t need = cogni_gemm_workspace_bytes(w_type, in_dim, tokens);
  if (!workspace || workspace_bytes < need)
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": workspace has " + std::to_string(workspace_bytes) + " bytes, needs " + std::to_string(need));
  return 0;
}

int cogni_gemm_pack_dev(uint64_t x, uint32_t w_type, uint32_t in_dim, uint32_t tokens, uint64_t workspace, size_t workspace_bytes,
                        void* stream) {
  if (!x) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemm_pack_dev: null device pointer");
  if (int rc = gemm_check("cogni_gemm_pack_dev", w_type, in_dim, 1, tokens, workspace, workspace_bytes)) return rc;
  const uint32_t mtiles = (tokens + 127) / 128;
  void* params[] = {&x, &workspace, &tokens, &in_dim};
  // 8 tokens x one super-block per workgroup
  return launch(w_type == COGNI_TYPE_Q6_K ? "pack_x_f16_q6k" : "pack_x_f16_q4k", mtiles * 16 * (in_dim / 256), 256, 0, params, stream);
}

int cogni_gemm_dev(uint64_t w_raw, uint32_t w_type, uint64_t x, uint64_t bias, uint64_t out, uint32_t in_dim,
                   uint32_t out_dim, uint32_t tokens, uint64_t workspace, size_t workspace_bytes, void* stream) {
  if (!w_raw || !x || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemm_dev: null device pointer");
  if (int rc = gemm_check("cogni_gemm_dev", w_type, in_dim, out_dim, tokens, workspace, workspace_bytes)) return rc;
  if (int rc = cogni_gemm_pack_dev(x, w_type, in_dim, tokens, workspace, workspace_bytes, stream)) return rc;
  return cogni_gemm_packed_dev(w_raw, w_type, workspace, workspace_bytes, bias, out, in_dim, out_dim, tokens, stream);
}

// The launch cogni_gemm_packed_dev makes for a shape and a workspace size: kernel, grid (x = tiles rounded up to a multiple
// of 8, y = k splits), block.
struct GemmPlan {
  const char* kernel;
  uint32_t grid_x, splits, block;
};
static GemmPlan gemm_plan(uint32_t w_type, uint32_t in_dim, uint32_t out_dim, uint32_t tokens, size_t workspace_bytes) {
  const uint32_t mtiles = (tokens + 127) / 128;
  GemmPlan p;
  // a workspace that holds the packed activations only: one workgroup per tile walks the whole row
  GemmShape shape = gemm_shape(w_type, in_dim, out_dim, tokens);
  if (workspace_bytes < cogni_gemm_workspace_bytes_split(w_type, in_dim, out_dim, tokens)) shape = gemm_shape(w_type, in_dim, out_dim, tokens, false);
  p.splits = shape.splits;
  const bool wide = shape.bn == 256, n128 = shape.bn == 128;
  // up to 64 tokens: the kernels that work on the first 64 tokens of the (one) token tile (COGNI_GEMM_M64=0 keeps the
  // 128-token tiles, a measurement knob)
  bool m64 = tokens <= 64 && !wide;
  if (const char* e = std::getenv("COGNI_GEMM_M64"))
    if (e[0] == '0') m64 = false;
  static const char* const names[3][2][2] = {
      {{"q4_k_gemm_f16", "q4_k_gemm_n128_f16"}, {"q4_k_gemm_m64_f16", "q4_k_gemm_m64_n128_f16"}},
      {{"q5_k_gemm_f16", "q5_k_gemm_n128_f16"}, {"q5_k_gemm_m64_f16", "q5_k_gemm_m64_n128_f16"}},
      {{"q6_k_gemm_f16", "q6_k_gemm_n128_f16"}, {"q6_k_gemm_m64_f16", "q6_k_gemm_m64_n128_f16"}}};
  p.kernel = wide ? "q4_k_gemm_wide_f16" : names[w_type == COGNI_TYPE_Q6_K ? 2 : (w_type == COGNI_TYPE_Q5_K ? 1 : 0)][m64][n128];
  const uint32_t ntiles = (out_dim + shape.bn - 1) / shape.bn;
  p.grid_x = gemm_grid_x(mtiles, ntiles);
  p.block = wide ? 512 : 256;
  return p;
}

int cogni_gemm_plan(uint32_t w_type, uint32_t in_dim, uint32_t out_dim, uint32_t tokens, size_t workspace_bytes, const char** kernel,
                    uint32_t* grid_x, uint32_t* grid_y, uint32_t* block_x) {
  if (!gemm_type(w_type))
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for the prefill GEMM: ") + type_name(w_type));
  if (in_dim == 0 || out_dim == 0 || tokens == 0 || (in_dim % 256) != 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemm_plan: zero dimension or in_dim not a multiple of 256");
  const GemmPlan p = gemm_plan(w_type, in_dim, out_dim, tokens, workspace_bytes);
  if (kernel) *kernel = p.kernel;
  if (grid_x) *grid_x = p.grid_x;
  if (grid_y) *grid_y = p.splits;
  if (block_x) *block_x = p.block;
  return 0;
}

// One matrix against packed activations; `add` is a [out_dim] bias (add_stride 0) or a [tokens][out_dim] residual (add_stride out_dim).
static int gemm_packed_launch(const char* who, uint64_t w_raw, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, uint64_t add,
                              uint32_t add_stride, uint64_t out, uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream) {
  if (!w_raw || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": null device pointer");
  if (int rc = gemm_check(who, w_type, in_dim, out_dim, tokens, workspace, workspace_bytes)) return rc;
  const size_t need = cogni_gemm_workspace_bytes(w_type, in_dim, tokens);
  const GemmPlan p = gemm_plan(w_type, in_dim, out_dim, tokens, workspace_bytes);
  uint32_t splits = p.splits;
  if (splits == 1) {
    void* params[] = {&w_raw, &workspace, &add, &out, &in_dim, &out_dim, &tokens, &add_stride};
    return launch(p.kernel, p.grid_x, p.block, 0, params, stream);
  }
  uint64_t planes = workspace + need, none = 0;
  uint32_t total = tokens * out_dim, zero = 0;
  {
    void* params[] = {&w_raw, &workspace, &none, &planes, &in_dim, &out_dim, &tokens, &zero};
    int rc = launch(p.kernel, p.grid_x, p.block, 0, params, stream, splits);
    if (rc != 0) return rc;
  }
  void* params[] = {&planes, &add, &out, &total, &out_dim, &splits, &add_stride};
  return launch("gemm_sum_splits_f32", (total + 1023) / 1024, 256, 0, params, stream);
}

int cogni_gemm_packed_dev(uint64_t w_raw, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, uint64_t bias, uint64_t out,
                          uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream) {
  return gemm_packed_launch("cogni_gemm_packed_dev", w_raw, w_type, workspace, workspace_bytes, bias, 0, out, in_dim, out_dim, tokens, stream);
}

int cogni_gemm_packed_add_dev(uint64_t w_raw, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, uint64_t residual, uint64_t out,
                              uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream) {
  if (!residual) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemm_packed_add_dev: null device pointer");
  return gemm_packed_launch("cogni_gemm_packed_add_dev", w_raw, w_type, workspace, workspace_bytes, residual, out_dim, out, in_dim, out_dim,
                            tokens, stream);
}

int cogni_gemm_packed_swiglu_dev(uint64_t w_gate, uint64_t w_up, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, uint64_t out,
                                 uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream) {
  if (w_type != COGNI_TYPE_Q4_K)
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for the fused gate/up SwiGLU GEMM: ") + type_name(w_type));
  if (!w_gate || !w_up || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_gemm_packed_swiglu_dev: null device pointer");
  if (int rc = gemm_check("cogni_gemm_packed_swiglu_dev", w_type, in_dim, out_dim, tokens, workspace, workspace_bytes)) return rc;
  // a tile is 128 tokens x 96 rows of each matrix
  const uint32_t mtiles = (tokens + 127) / 128, ntiles = (out_dim + 95) / 96;
  void* params[] = {&w_gate, &w_up, &workspace, &out, &in_dim, &out_dim, &tokens};
  return launch(tokens <= 64 ? "q4_k_gemm_swiglu_m64_f16" : "q4_k_gemm_swiglu_f16", gemm_grid_x(mtiles, ntiles), 256, 0, params, stream);
}

// Several matrices of one type and row length against one block of packed activations, as one launch: no k split (the list
// is what fills the chip), the tile height that needs fewer rounds of 256 workgroups (a 128-row tile costs
// GEMM_N128_COST_X100 per cent of a 192-row one), the 64-token kernels for up to 64 tokens.
namespace {
struct GemmManyArgs {   // the kernels' first parameter (kernels/gemm_q4k.hpp)
  uint64_t w[6];
  uint64_t out[6];
  uint32_t out_dim[6];
  uint32_t tile_end[6];
  uint32_t count;
};
}   // namespace
int cogni_gemm_packed_many_dev(const uint64_t* w_raw, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, const uint64_t* outs,
                               const uint32_t* out_dims, uint32_t count, uint32_t in_dim, uint32_t tokens, void* stream) {
  const char* who = "cogni_gemm_packed_many_dev";
  if (w_type != COGNI_TYPE_Q4_K && w_type != COGNI_TYPE_Q5_K)
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for the list GEMM: ") + type_name(w_type));
  if (!w_raw || !outs || !out_dims || count == 0 || count > 6) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": one to six matrices");
  for (uint32_t i = 0; i < count; i++) {
    if (!w_raw[i] || !outs[i]) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": null device pointer");
    if (int rc = gemm_check(who, w_type, in_dim, out_dims[i], tokens, workspace, workspace_bytes)) return rc;
  }
  const uint32_t mtiles = (tokens + 127) / 128, nkb = in_dim / 256;
  const size_t packed_bytes = cogni_gemm_workspace_bytes(w_type, in_dim, tokens);
  // a matrix that alone gets the 256-row tiles of the eight-wavefront kernel (many tokens, many rows) keeps them: it is
  // launched by itself, unsplit as the list is; the others form the list
  uint32_t listed[6], nlisted = 0;
  for (uint32_t i = 0; i < count; i++) {
    if (gemm_shape(w_type, in_dim, out_dims[i], tokens, false).bn == 256) {
      if (int rc = gemm_packed_launch(who, w_raw[i], w_type, workspace, packed_bytes, 0, 0, outs[i], in_dim, out_dims[i], tokens, stream)) return rc;
    } else {
      listed[nlisted++] = i;
    }
  }
  if (nlisted == 0) return 0;
  if (nlisted == 1) {
    const uint32_t i = listed[0];
    return gemm_packed_launch(who, w_raw[i], w_type, workspace, packed_bytes, 0, 0, outs[i], in_dim, out_dims[i], tokens, stream);
  }
  uint64_t tiles[2] = {0, 0};   // 192-row, 128-row
  for (uint32_t k = 0; k < nlisted; k++) {
    tiles[0] += (out_dims[listed[k]] + 191) / 192;
    tiles[1] += (out_dims[listed[k]] + 127) / 128;
  }
  const uint64_t cost192 = ((mtiles * tiles[0] + 255) / 256) * nkb * 100, cost128 = ((mtiles * tiles[1] + 255) / 256) * nkb * GEMM_N128_COST_X100;
  const bool n128 = cost128 < cost192, m64 = tokens <= 64;
  const uint32_t bn = n128 ? 128 : 192;
  GemmManyArgs list{};
  uint32_t end = 0;
  for (uint32_t k = 0; k < nlisted; k++) {
    const uint32_t i = listed[k];
    list.w[k] = w_raw[i];
    list.out[k] = outs[i];
    list.out_dim[k] = out_dims[i];
    list.tile_end[k] = end += (out_dims[i] + bn - 1) / bn;
  }
  list.count = nlisted;
  static const char* const names[2][2][2] = {
      {{"q4_k_gemm_many_f16", "q4_k_gemm_many_n128_f16"}, {"q4_k_gemm_many_m64_f16", "q4_k_gemm_many_m64_n128_f16"}},
      {{"q5_k_gemm_many_f16", "q5_k_gemm_many_n128_f16"}, {"q5_k_gemm_many_m64_f16", "q5_k_gemm_many_m64_n128_f16"}}};
  void* params[] = {&list, &workspace, &in_dim, &tokens};
  return launch(names[w_type == COGNI_TYPE_Q5_K][m64][n128], gemm_grid_x(mtiles, end), 256, 0, params, stream);
}

int cogni_gemm_packed_swiglu_pack_dev(uint64_t w_gate, uint64_t w_up, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, uint64_t out,
                                      uint32_t next_type, uint64_t next_workspace, size_t next_workspace_bytes, uint32_t in_dim,
                                      uint32_t out_dim, uint32_t tokens, void* stream) {
  const char* who = "cogni_gemm_packed_swiglu_pack_dev";
  if (w_type != COGNI_TYPE_Q4_K)
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for the fused gate/up SwiGLU GEMM: ") + type_name(w_type));
  if (!gemm_type(next_type))
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for the prefill GEMM: ") + type_name(next_type));
  if (!w_gate || !w_up || !next_workspace) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": null device pointer");
  if (int rc = gemm_check(who, w_type, in_dim, out_dim, tokens, workspace, workspace_bytes)) return rc;
  // the products are the activations of a matrix with rows of out_dim values
  if ((out_dim % 256) != 0) return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": out_dim must be a multiple of 256");
  if (next_workspace_bytes < cogni_gemm_workspace_bytes(next_type, out_dim, tokens))
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(who) + ": next_workspace too small (cogni_gemm_workspace_bytes)");
  const uint32_t mtiles = (tokens + 127) / 128, ntiles = (out_dim + 95) / 96;
  void* params[] = {&w_gate, &w_up, &workspace, &out, &next_workspace, &in_dim, &out_dim, &tokens};
  static const char* const names[2][2] = {{"q4_k_gemm_swiglu_pack_q4k_f16", "q4_k_gemm_swiglu_pack_q4k_m64_f16"},
                                          {"q4_k_gemm_swiglu_pack_q6k_f16", "q4_k_gemm_swiglu_pack_q6k_m64_f16"}};
  return launch(names[next_type == COGNI_TYPE_Q6_K][tokens <= 64], gemm_grid_x(mtiles, ntiles), 256, 0, params, stream);
}

int cogni_set_gemm_threshold(int32_t tokens) {
  if (tokens < 1) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_set_gemm_threshold: threshold must be >= 1");
  g_gemm_threshold = tokens;
  return 0;
}

int32_t cogni_get_gemm_threshold(void) {
  if (g_gemm_threshold < 0) {
    g_gemm_threshold = 8;
    if (const char* e = std::getenv("QWEN35_GEMM_BATCH_THRESHOLD")) {
      const int v = std::atoi(e);
      if (v >= 1) g_gemm_threshold = v;
    }
  }
  return g_gemm_threshold;
}

int cogni_matmul_dev(uint64_t w_raw, uint32_t w_type, uint64_t x, uint64_t bias, uint64_t out, uint32_t in_dim,
                     uint32_t out_dim, uint32_t tokens, uint64_t workspace, size_t workspace_bytes, void* stream) {
  if (gemm_type(w_type) && tokens > (uint32_t)cogni_get_gemm_threshold()) {
    // up to sixteen tokens of a Q4_K, Q5_K or Q6_K matrix without a bias: one pass over the weights on the decode kernels with
    // sixteen single-term tokens (the GEMM's precision class) costs about half of pack + GEMM + plane sum; the image goes
    // where the GEMM's packed activations would (COGNI_MATMUL_X16=0 keeps the GEMM: a measurement knob)
    bool x16 = tokens <= 16 && !bias && gemv16_shape(w_type, in_dim, tokens) && workspace &&
               workspace_bytes >= (size_t)gemv_mt_image_bytes(w_type, in_dim);
    if (const char* e = std::getenv("COGNI_MATMUL_X16"))
      if (e[0] == '0') x16 = false;
    if (x16) {
      if (!w_raw || !x || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_matmul_dev: null device pointer");
      if (int rc = cogni_gemv_pack16_dev(x, w_type, in_dim, tokens, workspace, stream)) return rc;
      return cogni_gemv_packed16_dev(&w_raw, w_type, workspace, 0, &out, &out_dim, 1, in_dim, tokens, stream);
    }
    return cogni_gemm_dev(w_raw, w_type, x, bias, out, in_dim, out_dim, tokens, workspace, workspace_bytes, stream);
  }
  if (bias && tokens != 1)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_matmul_dev: a [out_dim] bias is only accepted with one token or on the GEMM path; "
                                            "pass a [tokens][out_dim] residual to cogni_gemv_dev");
  return cogni_gemv_dev(w_raw, w_type, x, bias, out, in_dim, out_dim, tokens, stream);
}

// ---- host-buffer operators --------------------------------------------------------------------------
int cogni_dequantize(const void* data, size_t data_bytes, uint32_t type, int64_t n_elements, float* out) {
  if (!cogni_dequantize_kernel_name(type))
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, "Unsupported dequantization type: " + std::to_string(type));
  if (n_elements < 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_dequantize: negative n_elements");
  if (n_elements == 0) return 0;
  if (!data || !out) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_dequantize: null buffer");
  // K-quants read floor(n/256) blocks (dequant.cr:107,147,198); the 32-element formats ceil(n/32).
  const size_t need = k_quant(type) ? (size_t)(n_elements / 256) * (size_t)cogni_block_bytes(type)
                                    : (size_t)cogni_data_bytes(type, n_elements);
  if (data_bytes < need)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_dequantize: data has " + std::to_string(data_bytes) + " bytes, needs " + std::to_string(need));
  {
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_rt.ready) return fail(COGNI_ERR_NOT_INITIALIZED, "cogni_quant_init has not been called");
  }
  DeviceMem dw, dout;
  HIP_TRY(hipMalloc(&dw.p, need ? need : 16), "hipMalloc(dequantize input)");
  HIP_TRY(hipMalloc(&dout.p, (size_t)n_elements * 4), "hipMalloc(dequantize output)");
  if (need) HIP_TRY(hipMemcpyHtoD(dw.p, const_cast<void*>(data), need), "hipMemcpyHtoD(dequantize input)");
  int rc = cogni_dequantize_dev(dw.addr(), type, (uint64_t)n_elements, dout.addr(), nullptr);
  if (rc != 0) return rc;
  HIP_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize(dequantize)");
  HIP_TRY(hipMemcpyDtoH(out, dout.p, (size_t)n_elements * 4), "hipMemcpyDtoH(dequantize output)");
  return 0;
}

int cogni_weight_create(cogni_quant_weight** qw, const void* raw, size_t raw_bytes, uint32_t type, int32_t out_dim,
                        int32_t in_dim) {
  if (!qw || !raw) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_weight_create: null argument");
  if (!gemv_type(type) && !plain_type(type))
    return fail(COGNI_ERR_UNSUPPORTED_TYPE, std::string("Unsupported quant type for fused matmul: ") + type_name(type));
  if (out_dim <= 0 || in_dim <= 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_weight_create: dimensions must be positive");
  if (k_quant(type) && in_dim % 256 != 0)
    return fail(COGNI_ERR_INVALID_ARGUMENT, std::string(type_name(type)) + " requires in_dim multiple of 256, got " + std::to_string(in_dim));
  const size_t need = (size_t)out_dim * row_bytes_of(type, (uint32_t)in_dim);
  if (raw_bytes < need)
    return fail(COGNI_ERR_INVALID_ARGUMENT, "weight has " + std::to_string(raw_bytes) + " bytes, shape needs " + std::to_string(need));
  {
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_rt.ready) return fail(COGNI_ERR_NOT_INITIALIZED, "cogni_quant_init has not been called");
  }
  cogni_quant_weight* w = new cogni_quant_weight();
  hipError_t e = hipMalloc(&w->dev, need);
  if (e == hipSuccess) e = hipMemcpyHtoD(w->dev, const_cast<void*>(raw), need);
  if (e != hipSuccess) {
    if (w->dev) (void)hipFree(w->dev);
    delete w;
    return hip_fail(e, "upload of quantized weight");
  }
  w->bytes = need;
  w->type = type;
  w->out_dim = out_dim;
  w->in_dim = in_dim;
  *qw = w;
  return 0;
}

uint64_t cogni_weight_device_ptr(const cogni_quant_weight* qw) { return qw ? (uint64_t)(uintptr_t)qw->dev : 0; }

int cogni_weight_destroy(cogni_quant_weight* qw) {
  if (!qw) return 0;
  if (qw->dev) (void)hipFree(qw->dev);
  delete qw;
  return 0;
}

int cogni_weight_matmul(const cogni_quant_weight* qw, const float* x, int32_t rows, const float* bias, float* result) {
  if (!qw || !x || !result) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_weight_matmul: null argument");
  if (rows <= 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_weight_matmul: rows must be positive");
  const size_t xin = (size_t)rows * qw->in_dim * 4, xout = (size_t)rows * qw->out_dim * 4;
  DeviceMem dx, dres, dout;
  HIP_TRY(hipMalloc(&dx.p, xin), "hipMalloc(x)");
  HIP_TRY(hipMalloc(&dout.p, xout), "hipMalloc(result)");
  HIP_TRY(hipMemcpyHtoD(dx.p, const_cast<float*>(x), xin), "hipMemcpyHtoD(x)");
  const bool gemm_path = gemm_type(qw->type) && rows > cogni_get_gemm_threshold();
  if (bias && !gemm_path) {  // bias[o] is added to every row: stage it as a [rows][out_dim] residual
    std::vector<float> tiled((size_t)rows * qw->out_dim);
    for (int32_t r = 0; r < rows; r++) std::memcpy(&tiled[(size_t)r * qw->out_dim], bias, (size_t)qw->out_dim * 4);
    HIP_TRY(hipMalloc(&dres.p, xout), "hipMalloc(bias)");
    HIP_TRY(hipMemcpyHtoD(dres.p, tiled.data(), xout), "hipMemcpyHtoD(bias)");
  }
  int rc;
  if (gemm_path) {
    DeviceMem dws, dbias;
    const size_t wsb = cogni_gemm_workspace_bytes_split(qw->type, (uint32_t)qw->in_dim, (uint32_t)qw->out_dim, (uint32_t)rows);
    HIP_TRY(hipMalloc(&dws.p, wsb), "hipMalloc(gemm workspace)");
    if (bias) {
      HIP_TRY(hipMalloc(&dbias.p, (size_t)qw->out_dim * 4), "hipMalloc(bias)");
      HIP_TRY(hipMemcpyHtoD(dbias.p, const_cast<float*>(bias), (size_t)qw->out_dim * 4), "hipMemcpyHtoD(bias)");
    }
    rc = cogni_gemm_dev((uint64_t)(uintptr_t)qw->dev, qw->type, dx.addr(), dbias.addr(), dout.addr(),
                        (uint32_t)qw->in_dim, (uint32_t)qw->out_dim, (uint32_t)rows, dws.addr(), wsb, nullptr);
    if (rc != 0) return rc;
    HIP_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize(matmul)");
    HIP_TRY(hipMemcpyDtoH(result, dout.p, xout), "hipMemcpyDtoH(result)");
    return 0;
  }
  rc = cogni_gemv_dev((uint64_t)(uintptr_t)qw->dev, qw->type, dx.addr(), dres.addr(), dout.addr(),
                      (uint32_t)qw->in_dim, (uint32_t)qw->out_dim, (uint32_t)rows, nullptr);
  if (rc != 0) return rc;
  HIP_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize(matmul)");
  HIP_TRY(hipMemcpyDtoH(result, dout.p, xout), "hipMemcpyDtoH(result)");
  return 0;
}

int cogni_weight_matvec_many(const cogni_quant_weight* const* qws, int32_t count, const float* x, float* const* results) {
  if (count < 0) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_weight_matvec_many: count must not be negative");
  if (count == 0) return 0;
  if (!qws || !x || !results) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_weight_matvec_many: null argument");
  size_t total_out = 0;
  for (int32_t i = 0; i < count; i++) {
    if (!qws[i] || !results[i]) return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_weight_matvec_many: null weight or result");
    if (qws[i]->in_dim != qws[0]->in_dim)
      return fail(COGNI_ERR_INVALID_ARGUMENT, "cogni_weight_matvec_many: weight " + std::to_string(i) + " has in_dim " +
                                                  std::to_string(qws[i]->in_dim) + ", the first one " + std::to_string(qws[0]->in_dim));
    total_out += (size_t)qws[i]->out_dim;
  }
  // one upload of x, every GEMV on the default stream, one wait, then the outputs (they share one allocation)
  DeviceMem dx, dout;
  HIP_TRY(hipMalloc(&dx.p, (size_t)qws[0]->in_dim * 4), "hipMalloc(x)");
  HIP_TRY(hipMalloc(&dout.p, total_out * 4), "hipMalloc(results)");
  HIP_TRY(hipMemcpyHtoD(dx.p, const_cast<float*>(x), (size_t)qws[0]->in_dim * 4), "hipMemcpyHtoD(x)");
  size_t at = 0;
  for (int32_t i = 0; i < count; i++) {
    const int rc = cogni_gemv_dev((uint64_t)(uintptr_t)qws[i]->dev, qws[i]->type, dx.addr(), 0, dout.addr() + at * 4,
                                  (uint32_t)qws[i]->in_dim, (uint32_t)qws[i]->out_dim, 1, nullptr);
    if (rc != 0) return rc;
    at += (size_t)qws[i]->out_dim;
  }
  HIP_TRY(hipDeviceSynchronize(), "hipDeviceSynchronize(matvec_many)");
  at = 0;
  for (int32_t i = 0; i < count; i++) {
    HIP_TRY(hipMemcpyDtoH(results[i], static_cast<char*>(dout.p) + at * 4, (size_t)qws[i]->out_dim * 4), "hipMemcpyDtoH(result)");
    at += (size_t)qws[i]->out_dim;
  }
  return 0;
}

int cogni_matmul_add(const float* x, int32_t rows, int32_t in_dim, const void* w_raw, size_t w_bytes, uint32_t w_type,
                     int32_t out_dim, const float* bias, float* result) {
  cogni_quant_weight* qw = nullptr;
  int rc = cogni_weight_create(&qw, w_raw, w_bytes, w_type, out_dim, in_dim);
  if (rc != 0) return rc;
  rc = cogni_weight_matmul(qw, x, rows, bias, result);
  cogni_weight_destroy(qw);
  return rc;
}

}  // extern "C"
