// Small utility kernels: a plain copy (bandwidth calibration for profiler counters), a read-only
// stream (practical HBM read ceiling for a buffer of a given size) and fp32 -> fp16 conversion of
// the activations ahead of the prefill GEMM.
#pragma once
#include "common.cuh"

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

// (src f32, dst f16, n): round-to-nearest-even; n multiple of 4 is the fast path. block = 256, any grid.
extern "C" __global__ __launch_bounds__(256) void convert_f32_to_f16(const float* __restrict__ src,
                                                                      __half* __restrict__ dst, u64 n) {
  const u64 tid = (u64)blockIdx.x * blockDim.x + threadIdx.x, step = (u64)gridDim.x * blockDim.x;
  for (u64 e = tid * 4; e < n; e += step * 4) {
    if (e + 4 <= n) {
      float4 v;
      __builtin_memcpy(&v, src + e, 16);
      __half2 a = __floats2half2_rn(v.x, v.y), b = __floats2half2_rn(v.z, v.w);
      uint2 o;
      o.x = *reinterpret_cast<u32*>(&a);
      o.y = *reinterpret_cast<u32*>(&b);
      __builtin_memcpy(dst + e, &o, 8);
    } else {
      for (u64 c = e; c < n; c++) dst[c] = __float2half_rn(src[c]);
    }
  }
}
