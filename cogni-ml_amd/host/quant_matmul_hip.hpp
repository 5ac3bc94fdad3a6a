// ml::gguf - C++ host mirror of the reference's QuantMatmul / Dequant / QuantWeight / TensorType for the
// HIP path, on the C ABI of libcogni_hip.so (include/cogni_quant.h). Signatures follow the reference so a
// caller changes the namespace, not the call:
//   QuantMatmul.matmul_add(x, rows, in_dim, w_raw, w_type, out_dim, bias)   src/ml/gguf/quant_matmul.cr:20
//   Dequant.dequantize(data, type, n_elements)                              src/ml/gguf/dequant.cr:19
//   QuantWeight {raw, type, out_dim, in_dim, route_tag}                     src/ml/gguf/compute.cr:20-30
// Errors throw std::runtime_error with the library's message (the reference raises, quant_matmul.cr:33-34).
#pragma once
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "cogni_quant.h"

namespace ml::gguf {

// src/ml/gguf/reader.cr:34-98
enum class TensorType : uint32_t {
  F32 = 0, F16 = 1, Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8, Q2_K = 10, Q3_K = 11, Q4_K = 12,
  Q5_K = 13, Q6_K = 14, Q8_K = 15, IQ4_NL = 20
};
inline int block_bytes(TensorType t) { return cogni_block_bytes((uint32_t)t); }
inline int block_elements(TensorType t) { return cogni_block_elements((uint32_t)t); }
inline int64_t data_bytes(TensorType t, int64_t n_elements) { return cogni_data_bytes((uint32_t)t, n_elements); }

class QuantError : public std::runtime_error {
 public:
  explicit QuantError(int code) : std::runtime_error(cogni_last_error()), code_(code) {}
  int code() const { return code_; }

 private:
  int code_;
};
inline void qcheck(int code) {
  if (code != 0) throw QuantError(code);
}

inline void init(int ordinal = 0) { qcheck(cogni_quant_init(ordinal)); }

struct Dequant {
  static std::vector<float> dequantize(const uint8_t* data, size_t data_bytes, TensorType type, int64_t n_elements) {
    std::vector<float> out((size_t)n_elements);
    qcheck(cogni_dequantize(data, data_bytes, (uint32_t)type, n_elements, out.data()));
    return out;
  }
};

struct QuantMatmul {
  static std::vector<float> matmul_add(const std::vector<float>& x, int rows, int in_dim, const uint8_t* w_raw,
                                       size_t w_bytes, TensorType w_type, int out_dim,
                                       const std::vector<float>& bias) {
    if (x.size() < (size_t)rows * in_dim) throw std::invalid_argument("x is smaller than rows*in_dim");
    if (bias.size() < (size_t)out_dim) throw std::invalid_argument("bias is smaller than out_dim");
    std::vector<float> result((size_t)rows * out_dim);
    qcheck(cogni_matmul_add(x.data(), rows, in_dim, w_raw, w_bytes, (uint32_t)w_type, out_dim, bias.data(), result.data()));
    return result;
  }
};

// compute.cr:20-45: the raw bytes stay with the caller; the device copy is made once and kept.
class QuantWeight {
 public:
  QuantWeight(const uint8_t* raw, size_t raw_bytes, TensorType type, int out_dim, int in_dim, std::string route_tag = "")
      : raw_(raw), raw_bytes_(raw_bytes), type_(type), out_dim_(out_dim), in_dim_(in_dim), route_tag_(std::move(route_tag)) {
    qcheck(cogni_weight_create(&handle_, raw, raw_bytes, (uint32_t)type, out_dim, in_dim));
  }
  QuantWeight(const QuantWeight&) = delete;
  ~QuantWeight() { close(); }
  const uint8_t* raw() const { return raw_; }
  size_t raw_bytes() const { return raw_bytes_; }
  TensorType type() const { return type_; }
  int out_dim() const { return out_dim_; }
  int in_dim() const { return in_dim_; }
  const std::string& route_tag() const { return route_tag_; }
  uint64_t device_ptr() const { return cogni_weight_device_ptr(handle_); }
  // ComputeBackend#matmul(x, rows, qw, bias) (compute.cr:50); bias may be null (qmatvec_nobias)
  std::vector<float> matmul(const std::vector<float>& x, int rows, const std::vector<float>* bias = nullptr) const {
    if (rows <= 0) throw std::invalid_argument("matmul: rows must be positive");
    if (x.size() < (size_t)rows * (size_t)in_dim_)   // the library copies rows*in_dim floats from this buffer
      throw std::invalid_argument("matmul: x has " + std::to_string(x.size()) + " elements, rows*in_dim is " +
                                  std::to_string((size_t)rows * (size_t)in_dim_));
    if (bias && bias->size() < (size_t)out_dim_)
      throw std::invalid_argument("matmul: bias has " + std::to_string(bias->size()) + " elements, out_dim is " + std::to_string(out_dim_));
    std::vector<float> result((size_t)rows * out_dim_);
    qcheck(cogni_weight_matmul(handle_, x.data(), rows, bias ? bias->data() : nullptr, result.data()));
    return result;
  }
  void close() {
    if (handle_) cogni_weight_destroy(handle_);
    handle_ = nullptr;
  }
  // qmatvec_many(qws, x) (qwen35_cpu.cr:1419-1445): every weight against the same one-token x in one call
  static std::vector<std::vector<float>> matvec_many(const std::vector<const QuantWeight*>& qws, const std::vector<float>& x) {
    std::vector<std::vector<float>> results(qws.size());
    if (qws.empty()) return results;
    if (x.size() != (size_t)qws[0]->in_dim_) throw std::invalid_argument("matvec_many x size mismatch");
    std::vector<const cogni_quant_weight*> handles(qws.size());
    std::vector<float*> outs(qws.size());
    for (size_t i = 0; i < qws.size(); i++) {
      results[i].resize((size_t)qws[i]->out_dim_);
      handles[i] = qws[i]->handle_;
      outs[i] = results[i].data();
    }
    qcheck(cogni_weight_matvec_many(handles.data(), (int32_t)qws.size(), x.data(), outs.data()));
    return results;
  }

 private:
  const uint8_t* raw_;
  size_t raw_bytes_;
  TensorType type_;
  int out_dim_, in_dim_;
  std::string route_tag_;
  cogni_quant_weight* handle_ = nullptr;
};

}  // namespace ml::gguf
