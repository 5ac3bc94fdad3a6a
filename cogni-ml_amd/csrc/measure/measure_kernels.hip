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
