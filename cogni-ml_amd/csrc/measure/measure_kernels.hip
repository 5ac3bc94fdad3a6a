// Measurement-only kernels, built into a code object of their own (lib/measure_kernels_gfx950.hsaco) that only
// bench.py loads; nothing in here is part of libcogni_hip.so. A plain copy (calibrates the profiler's byte counters),
// a read-only stream (what a launch that only reads a buffer of a given size achieves) and a loop of nothing but matrix-core instructions (the rate the matrix cores sustain on this machine).
#include "../kernels/common.hpp"

// (src, dst, n_bytes): n_bytes must be a multiple of 16. block = 256, any grid.
extern "C" __global__ __launch_bounds__(256) void copy_bytes_16(const uint4* __restrict__ src,
                                                                 uint4* __restrict__ dst, u64 n_bytes) {
  const u64 n = n_bytes >> 4;
  const u64 tid = (u64)blockIdx.x * blockDim.x + threadIdx.x, step = (u64)gridDim.x * blockDim.x;
  for (u64 i = tid; i < n; i += step) dst[i] = src[i];
}

// (src, out, n_bytes): every thread XORs the 16-byte words it reads; the result is stored only if it has one
// particular value, which keeps the loads alive and the kernel free of any epilogue. block = 256, any grid
// (about 8 workgroups per compute unit reads a 28 MB buffer fastest).
extern "C" __global__ __launch_bounds__(256) void read_bytes_16(const uint4* __restrict__ src,
                                                                 u32* __restrict__ out, u64 n_bytes) {
  const u64 n = n_bytes >> 4;
  const u64 tid = (u64)blockIdx.x * blockDim.x + threadIdx.x, step = (u64)gridDim.x * blockDim.x;
  u32 a = 0;
  for (u64 i = tid; i < n; i += step) {
    const uint4 v = src[i];
    a ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (a == 0x12345678u) out[tid & 1023] = a;
}

// What the matrix cores give a loop of nothing but v_mfma_f32_32x32x16_f16: every wavefront holds twelve 32x32
// accumulator tiles (4 A operands x 3 B operands read once from `src`, 7 x 64 x 16 bytes of fp16 per wavefront pattern)
// and issues `iters` rounds of the twelve MFMAs, flipping operand bits between rounds so that the inputs toggle as real
// data does. (src, out, iters): out gets one float per thread. 2 * 32*32*16 * 12 * iters flops per wavefront.
// _w4: block 256, one wavefront per SIMD (what the prefill GEMM runs at); _w8: block 512, two per SIMD.
typedef _Float16 util_half8 __attribute__((ext_vector_type(8)));
typedef float util_float16 __attribute__((ext_vector_type(16)));
__device__ __forceinline__ void mfma_ceiling_core(const uint4* src, float* out, u32 iters) {
  const u32 lane = threadIdx.x & 63;
  uint4 a[4], b[3];
#pragma unroll
  for (int i = 0; i < 4; i++) a[i] = src[i * 64 + lane];
#pragma unroll
  for (int i = 0; i < 3; i++) b[i] = src[(4 + i) * 64 + lane];
  util_float16 acc[4][3];
#pragma unroll
  for (int r = 0; r < 4; r++)
#pragma unroll
    for (int c = 0; c < 3; c++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[r][c][v] = 0.0f;
  for (u32 it = 0; it < iters; it++) {
#pragma unroll
    for (int r = 0; r < 4; r++)
#pragma unroll
      for (int c = 0; c < 3; c++)
        acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(*reinterpret_cast<const util_half8*>(&a[r]),
                                                           *reinterpret_cast<const util_half8*>(&b[c]), acc[r][c], 0, 0, 0);
    // sign and low mantissa bits flip: values stay finite and of the same size
#pragma unroll
    for (int i = 0; i < 4; i++) a[i].x ^= 0x80038003u, a[i].z ^= 0x00058005u;
#pragma unroll
    for (int i = 0; i < 3; i++) b[i].y ^= 0x80038003u, b[i].w ^= 0x00058005u;
  }
  float sum = 0.0f;
#pragma unroll
  for (int r = 0; r < 4; r++)
#pragma unroll
    for (int c = 0; c < 3; c++)
#pragma unroll
      for (int v = 0; v < 16; v++) sum += acc[r][c][v];
  out[blockIdx.x * blockDim.x + threadIdx.x] = sum;
}
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mfma_f16_ceiling_w4(
    const uint4* src, float* out, u32 iters) {
  mfma_ceiling_core(src, out, iters);
}
extern "C" __global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void mfma_f16_ceiling_w8(
    const uint4* src, float* out, u32 iters) {
  mfma_ceiling_core(src, out, iters);
}

// What the other work of the prefill GEMM's k-step costs a wavefront that is issuing its twelve MFMAs (one wavefront per
// SIMD, four ds_read_b128 of token tiles per k-step, as in q4_k_gemm_f16). COPIES: global -> LDS copies of 1 KiB per
// wavefront and k-step (global_load_lds_dwordx4 out of a 1 MiB region that 32 workgroups share, so they hit in L2);
// DECODE: the 54 vector instructions that turn twelve 4-bit words into fp16 weight operands. (src, out, iters): `src`
// holds at least 1 MiB + 64 KiB; one iteration is eight k-steps, 2 * 32*32*16 * 12 * 8 flops per wavefront.
typedef const __attribute__((address_space(1))) void probe_gbl_void;
typedef __attribute__((address_space(3))) void probe_lds_void;
__shared__ uint4 probe_tokens[4096];
__shared__ uint4 probe_landing[4096];
__device__ __forceinline__ u32 probe_q4_pair(u32 t, u32 scale, u32 negmin) {
  const u32 off = 0xE400E400u;   // -1024 twice: takes the 0x6400 exponent trick's offset out again
  const __half2 q = __hadd2(*reinterpret_cast<const __half2*>(&t), *reinterpret_cast<const __half2*>(&off));
  const __half2 w = __hfma2(q, *reinterpret_cast<const __half2*>(&scale), *reinterpret_cast<const __half2*>(&negmin));
  return *reinterpret_cast<const u32*>(&w);
}
template <int COPIES, bool DECODE>
__device__ __forceinline__ void mfma_step_probe_core(const uint4* src, float* out, u32 iters) {
  const u32 tid = threadIdx.x, lane = tid & 63;
  const u32 wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const u32 j = lane & 31, kg = lane >> 5, kh = wave >> 1;
  const uint4* region = src + (size_t)(blockIdx.x & 7) * 8192;   // 8 x 128 KiB windows of the first MiB
  util_float16 acc[4][3];
#pragma unroll
  for (int r = 0; r < 4; r++)
#pragma unroll
    for (int c = 0; c < 3; c++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[r][c][v] = 0.0f;
  util_half8 B[3], Bnext[3];
  uint4 raw[3];
  u32 sc[3], nm[3];
#pragma unroll
  for (int c = 0; c < 3; c++) {
    uint4 v = src[tid + 256 * c];
    B[c] = *reinterpret_cast<util_half8*>(&v);
    Bnext[c] = B[c];
    raw[c] = src[tid + 256 * c + 2048];
    sc[c] = src[tid + 3000 + c].x;
    nm[c] = src[tid + 3000 + c].y;
  }
  for (u32 i = tid; i < 4096; i += 256) {
    probe_tokens[i] = src[i];
    probe_landing[i] = src[i + 4096];
  }
  __syncthreads();
  uint4 A[2][4];
#pragma unroll
  for (int r = 0; r < 4; r++) A[0][r] = probe_tokens[(16 * kh + kg) * 128 + j + r * 32];
  for (u32 it = 0; it < iters; it++) {
    const uint4* xsrc = region + (size_t)(it & 1) * 4096;
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const uint4* arow = probe_tokens + (16 * kh + kg) * 128 + j;
#pragma unroll
      for (int r = 0; r < 4; r++) A[(t + 1) & 1][r] = arow[((t + 1) & 7) * 256 + r * 32];
#pragma unroll
      for (int i = 0; i < COPIES; i++) {
        const int ci = (t * COPIES + i) & 15;
        __builtin_amdgcn_global_load_lds((probe_gbl_void*)(xsrc + 256 * ci + tid),
                                         (probe_lds_void*)(probe_landing + 256 * ci + wave * 64), 16, 0, 0);
      }
      if (DECODE) {
#pragma unroll
        for (int c = 0; c < 3; c++) {
          uint4 q = raw[c];
          asm volatile("" : "+v"(q.x), "+v"(q.y), "+v"(q.z), "+v"(q.w));
          uint4 bw;
          bw.x = probe_q4_pair((q.x & 0x000F000Fu) | 0x64006400u, sc[c], nm[c]);
          bw.y = probe_q4_pair(((q.x >> 8) & 0x000F000Fu) | 0x64006400u, sc[c], nm[c]);
          bw.z = probe_q4_pair((q.y & 0x000F000Fu) | 0x64006400u, sc[c], nm[c]);
          bw.w = probe_q4_pair(((q.y >> 8) & 0x000F000Fu) | 0x64006400u, sc[c], nm[c]);
          Bnext[c] = *reinterpret_cast<util_half8*>(&bw);
        }
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const util_half8 Ar = *reinterpret_cast<const util_half8*>(&A[t & 1][r]);
#pragma unroll
        for (int c = 0; c < 3; c++) acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(B[c], Ar, acc[r][c], 0, 0, 0);
      }
      if (DECODE) {
#pragma unroll
        for (int c = 0; c < 3; c++) {
          asm volatile("" : "+v"(Bnext[c]));
          B[c] = Bnext[c];
        }
      }
      // one MFMA, the four LDS reads, then a copy behind every second MFMA: the placement the GEMM kernel uses
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
      for (int i = 0; i < COPIES; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (COPIES > 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
  }
  __syncthreads();
  float s = __uint_as_float(probe_landing[tid].x);
#pragma unroll
  for (int r = 0; r < 4; r++)
#pragma unroll
    for (int c = 0; c < 3; c++)
#pragma unroll
      for (int v = 0; v < 16; v++) s += acc[r][c][v];
  out[blockIdx.x * 256 + tid] = s;
}
#define MFMA_STEP_PROBE(name, copies, decode)                                                                        \
  extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void name(                 \
      const uint4* src, float* out, u32 iters) {                                                                     \
    mfma_step_probe_core<copies, decode>(src, out, iters);                                                           \
  }
MFMA_STEP_PROBE(mfma_step_probe_bare, 0, false)
MFMA_STEP_PROBE(mfma_step_probe_decode, 0, true)
MFMA_STEP_PROBE(mfma_step_probe_copy1, 1, false)
MFMA_STEP_PROBE(mfma_step_probe_copy2, 2, false)
MFMA_STEP_PROBE(mfma_step_probe_copy3, 3, false)
MFMA_STEP_PROBE(mfma_step_probe_copy2_decode, 2, true)
MFMA_STEP_PROBE(mfma_step_probe_copy3_decode, 3, true)
