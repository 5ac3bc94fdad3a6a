// Exercises the C++ host mirror (cogni-ml_amd/host/*.hpp).
//   no arguments: host-only checks, the three examples of spec/cuda_resident_sequence_runner_spec.cr:5-50
//                 and the argument errors that need no GPU;
//   --gpu:        additionally the probe sequence of bin/gemma4_cuda_primitive_probe.cr:49-132 through the
//                 C++ classes (Context -> HIPModule -> function by name -> DeviceBuffer x3 -> copy_htod ->
//                 launch with boxed params -> synchronize -> copy_dtoh), checked against the CPU oracle
//                 (oracle/quant_oracle.c, linked only into this test), printing the probe's key=value lines.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "ml_hip.hpp"
#include "quant_matmul_hip.hpp"
#include "../../cogni-ml_amd/csrc/kernels/gemv_config.h"

extern "C" int oracle_matmul_add(const float* x, int rows, int in_dim, const uint8_t* w_raw, uint32_t w_type,
                                 int out_dim, const float* bias, float* result);
extern "C" int oracle_dequantize(const uint8_t* data, uint32_t type, int n, float* out);

static int failures = 0;
#define EXPECT(cond)                                                        \
  do {                                                                      \
    if (!(cond)) { std::printf("FAILED %s:%d %s\n", __FILE__, __LINE__, #cond); failures++; } \
  } while (0)

template <class E, class F>
static bool throws_with(F&& f, const char* needle) {
  try { f(); } catch (const E& e) { return std::strstr(e.what(), needle) != nullptr; } catch (...) { return false; }
  return false;
}

static void runner_spec() {
  using ml::hip::ResidentSequenceRunner;
  {  // runs only the configured active token prefix on the token-local path
    std::vector<int> seen;
    ResidentSequenceRunner r(4, [] {}, [] {}, [&](int tok) { seen.push_back(tok); });
    r.set_active_tokens(2);
    r.run_sequence();
    EXPECT((seen == std::vector<int>{0, 1}));
    EXPECT(r.run_repeated(3) == 6);
  }
  {  // passes active token count to sequence overrides
    std::vector<int> seen;
    ResidentSequenceRunner r(8, [] {}, [] {}, [](int) {}, std::nullopt, [&](int n) { seen.push_back(n); });
    r.set_active_tokens(4);
    r.run_sequence();
    EXPECT((seen == std::vector<int>{4}));
  }
  {  // rejects invalid active token counts
    ResidentSequenceRunner r(4, [] {}, [] {}, [](int) {});
    EXPECT(throws_with<std::invalid_argument>([&] { r.set_active_tokens(0); }, "active_tokens must be positive"));
    EXPECT(throws_with<std::invalid_argument>([&] { r.set_active_tokens(5); }, "active_tokens must be <= tokens"));
    EXPECT(throws_with<std::invalid_argument>([&] { ResidentSequenceRunner bad(0, [] {}, [] {}, [](int) {}); }, "tokens must be positive"));
  }
}

static void host_errors() {
  using namespace ml::gguf;
  EXPECT(block_bytes(TensorType::Q4_K) == 144 && block_elements(TensorType::Q6_K) == 256);
  EXPECT(data_bytes(TensorType::Q6_K, 151936LL * 4096) == 510504960LL);
  std::vector<float> x(256), bias(1);
  std::vector<uint8_t> w(144);
  EXPECT(throws_with<QuantError>([&] { QuantMatmul::matmul_add(x, 1, 256, w.data(), w.size(), TensorType::Q4_0, 1, bias); },
                                 "Unsupported quant type for fused matmul: Q4_0"));
  EXPECT(throws_with<QuantError>([&] { QuantMatmul::matmul_add(x, 1, 100, w.data(), w.size(), TensorType::Q4_K, 1, bias); },
                                 "in_dim multiple of 256"));
  EXPECT(throws_with<QuantError>([&] { Dequant::dequantize(w.data(), w.size(), TensorType::Q2_K, 256); },
                                 "Unsupported dequantization type"));
}

static uint16_t f32_to_f16_bits(float f) {   // good enough for positive scales well inside the normal range
  uint32_t u; std::memcpy(&u, &f, 4);
  int e = (int)((u >> 23) & 0xFF) - 127 + 15;
  uint32_t m = (u >> 13) & 0x3FF;
  if (e <= 0) return 0;
  return (uint16_t)((e << 10) | m);
}

static int gpu_probe() {
  using namespace ml::hip;
  using namespace ml::gguf;
  const int in_dim = 4096, out_dim = 1024, reps = 20, warmup = 3;
  std::mt19937_64 rng(23);
  std::vector<uint8_t> w((size_t)out_dim * (in_dim / 256) * 144);
  for (auto& b : w) b = (uint8_t)(rng() & 0xFF);
  std::normal_distribution<float> nd(0.f, 1.f);
  for (size_t b = 0; b < w.size() / 144; b++) {
    uint16_t d = f32_to_f16_bits(std::fabs(nd(rng)) * 0.005f + 1e-4f), dm = f32_to_f16_bits(std::fabs(nd(rng)) * 0.002f + 1e-4f);
    std::memcpy(&w[b * 144], &d, 2);
    std::memcpy(&w[b * 144 + 2], &dm, 2);
  }
  std::vector<float> x(in_dim), zero(out_dim, 0.f), cpu(out_dim), gpu(out_dim);
  for (auto& v : x) v = nd(rng);
  oracle_matmul_add(x.data(), 1, in_dim, w.data(), 12, out_dim, zero.data(), cpu.data());

  Context ctx = Context::create(0);
  const void* image; size_t image_size;
  qcheck(cogni_quant_code_object(&image, &image_size));
  HIPModule mod = HIPModule::load(image, "cogni_quant_gfx950");
  KernelFunction fn = mod.function(cogni_gemv_kernel_name(12, 1, 0));
  DeviceBuffer wb(w.size()), xb(4 * in_dim), ob(4 * out_dim);
  copy_htod(wb.ptr(), w.data(), w.size(), "weights");
  copy_htod(xb.ptr(), x.data(), 4 * in_dim, "input");
  DevicePtr d_w = wb.ptr(), d_x = xb.ptr(), d_out = ob.ptr();
  uint32_t in_u = in_dim, out_u = out_dim, grid, block, shmem;
  qcheck(cogni_gemv_launch_dims(12, 1, in_u, out_u, &grid, &block, &shmem));
  void* params[] = {&d_w, &d_x, &d_out, &in_u, &out_u};
  HIPStream stream;
  float ms = 0;
  with_stream(stream, [&] {
    for (int i = 0; i < warmup; i++) launch(fn, grid, 1, 1, block, 1, 1, params, fn.name(), shmem);
    stream.synchronize();
    mlhip_event e0, e1;
    check(mlhip_event_create(&e0), "hipEventCreate");
    check(mlhip_event_create(&e1), "hipEventCreate");
    check(mlhip_event_record(e0, stream.handle()), "hipEventRecord");
    for (int i = 0; i < reps; i++) launch(fn, grid, 1, 1, block, 1, 1, params, fn.name(), shmem);
    check(mlhip_event_record(e1, stream.handle()), "hipEventRecord");
    check(mlhip_event_synchronize(e1), "hipEventSynchronize");
    check(mlhip_event_elapsed_ms(&ms, e0, e1), "hipEventElapsedTime");
    mlhip_event_destroy(e0);
    mlhip_event_destroy(e1);
  });
  synchronize("timed");
  copy_dtoh(gpu.data(), ob.ptr(), 4 * out_dim, "output");
  double dot = 0, na = 0, nb = 0, max_diff = 0;
  for (int i = 0; i < out_dim; i++) {
    dot += (double)gpu[i] * cpu[i]; na += (double)gpu[i] * gpu[i]; nb += (double)cpu[i] * cpu[i];
    max_diff = std::fmax(max_diff, std::fabs((double)gpu[i] - cpu[i]));
  }
  const double cos = dot / std::sqrt(na * nb);
  const bool ok = cos >= 0.99999 && max_diff <= 1e-3;
  std::printf("device=%s\narch=%s\ncompute_capability=%d.%d\ncase=synthetic.q4_k\ntype=Q4_K\nshape=%dx%d\nraw_bytes=%zu\n"
              "reps=%d\nwarmup=%d\nhip_ms=%.4f\ncos=%.8f\nmax_diff=%g\nok=%s\n",
              ctx.device_name().c_str(), ctx.arch().c_str(), ctx.compute_capability_major(), ctx.compute_capability_minor(),
              in_dim, out_dim, w.size(), reps, warmup, ms / reps, cos, max_diff, ok ? "true" : "false");
  EXPECT(ok);
  EXPECT(fn.attribute(FunctionAttribute::NumRegs) > 0);

  // the same product through the host-buffer operator and through a resident QuantWeight
  init(0);
  std::vector<float> via_op = QuantMatmul::matmul_add(x, 1, in_dim, w.data(), w.size(), TensorType::Q4_K, out_dim, zero);
  EXPECT(std::memcmp(via_op.data(), gpu.data(), 4 * out_dim) == 0);
  QuantWeight qw(w.data(), w.size(), TensorType::Q4_K, out_dim, in_dim, "probe");
  EXPECT(qw.device_ptr() != 0);
  std::vector<float> via_qw = qw.matmul(x, 1);
  EXPECT(std::memcmp(via_qw.data(), gpu.data(), 4 * out_dim) == 0);
  // a buffer shorter than the shape says is refused before the library reads from it
  std::vector<float> short_x(in_dim - 1), short_bias(out_dim - 1);
  EXPECT(throws_with<std::invalid_argument>([&] { qw.matmul(short_x, 1); }, "rows*in_dim is 4096"));
  EXPECT(throws_with<std::invalid_argument>([&] { qw.matmul(x, 2); }, "rows*in_dim is 8192"));
  EXPECT(throws_with<std::invalid_argument>([&] { qw.matmul(x, 1, &short_bias); }, "out_dim is 1024"));
  // qmatvec_many: the same weight twice against one x, and no weights at all
  std::vector<std::vector<float>> many = QuantWeight::matvec_many({&qw, &qw}, x);
  EXPECT(many.size() == 2 && std::memcmp(many[0].data(), gpu.data(), 4 * out_dim) == 0 &&
         std::memcmp(many[1].data(), gpu.data(), 4 * out_dim) == 0);
  EXPECT(QuantWeight::matvec_many({}, x).empty());
  // bit-exact dequantize of the first rows
  std::vector<float> deq = Dequant::dequantize(w.data(), w.size(), TensorType::Q4_K, 8 * in_dim), ref(8 * in_dim);
  oracle_dequantize(w.data(), 12, 8 * in_dim, ref.data());
  EXPECT(std::memcmp(deq.data(), ref.data(), 4 * 8 * in_dim) == 0);
  EXPECT(throws_with<Error>([&] { mod.function("no_such_kernel"); }, "hipModuleGetFunction(no_such_kernel) failed with HIP error"));
  std::printf("summary_ok=%s\n", failures == 0 ? "true" : "false");
  return 0;
}

// The vmcnt values of the one-pass kernel's streamed path (mt_stream_wait, gemv_config.h) against a list of what the
// kernel issues, in its order: up front set u (u < NS) and unit u for u < NSLOT; behind unit i's arithmetic set i + NS and
// unit i + NSLOT. A unit may start when the youngest load of operand set i and of unit i has landed, i.e. when at most the
// loads issued after it are outstanding. Every (super-blocks per k-slice, slots, register sets) the kernels are built with,
// and the neighbouring ones.
static void stream_wait_spec() {
  struct Fmt { int slots, nc; };
  for (int S = 3; S <= 6; S++)
    for (Fmt f : {Fmt{6, 3}, Fmt{4, 4}, Fmt{4, 5}})   // Q4_K | Q5_K, Q6_K, Q8_0
      for (int NS = 2; NS <= 3; NS++)
        for (int NA : {9, 13}) {
          const int NSLOT = f.slots < S ? f.slots : S, NC = f.nc;
          std::vector<std::pair<char, int>> issued;
          auto issue = [&](char kind, int index, int n) { for (int k = 0; k < n; k++) issued.push_back({kind, index}); };
          for (int u = 0; u < NSLOT; u++) {
            if (u < NS) issue('s', u, NA);
            issue('u', u, NC);
          }
          for (int i = 0; i < S; i++) {
            int last = -1, nset = 0, nunit = 0;
            for (int k = 0; k < (int)issued.size(); k++)
              if (issued[k].second == i) {
                last = k;
                (issued[k].first == 's' ? nset : nunit)++;
              }
            EXPECT(nset == NA && nunit == NC);   // both were requested before their wait
            const int behind = (int)issued.size() - 1 - last;
            EXPECT(mt_stream_wait(S, NSLOT, NS, NA, NC, i) == behind);
            EXPECT(behind >= 0 && behind < 64);  // vmcnt has six bits
            if (i + NS < S) issue('s', i + NS, NA);
            if (i + NSLOT < S) issue('u', i + NSLOT, NC);
          }
        }
  // a known point: Q4_K at 12288 columns (S = 6, six slots, two sets): unit 0 waits with everything behind unit 0 outstanding
  EXPECT(mt_stream_wait(6, 6, 2, 9, 3, 0) == 9 + 3 + 4 * 3);
  EXPECT(mt_stream_wait(6, 6, 2, 9, 3, 5) == 0);
}

int main(int argc, char** argv) {
  runner_spec();
  stream_wait_spec();
  host_errors();
  if (argc > 1 && std::string(argv[1]) == "--gpu") gpu_probe();
  std::printf("%s (%d failures)\n", failures == 0 ? "PASSED" : "FAILED", failures);
  return failures == 0 ? 0 : 1;
}
