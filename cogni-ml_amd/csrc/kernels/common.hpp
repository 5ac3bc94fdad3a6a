// Shared device helpers for the gfx950 (CDNA4, wave64) quantized-matmul kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#define WAVE 64

typedef unsigned int u32;
typedef unsigned long long u64;

// 16-byte load that tolerates any byte alignment (Q6_K / Q8_0 blocks are only 2-byte aligned).
__device__ __forceinline__ uint4 ld16(const uint8_t* p) {
  uint4 v;
  __builtin_memcpy(&v, p, 16);
  return v;
}
__device__ __forceinline__ uint2 ld8(const uint8_t* p) {
  uint2 v;
  __builtin_memcpy(&v, p, 8);
  return v;
}
__device__ __forceinline__ u32 ld4(const uint8_t* p) {
  u32 v;
  __builtin_memcpy(&v, p, 4);
  return v;
}
__device__ __forceinline__ u32 ld2(const uint8_t* p) {
  unsigned short v;
  __builtin_memcpy(&v, p, 2);
  return v;
}

// IEEE binary16 -> binary32, exact for every finite input including subnormals (v_cvt_f32_f16).
__device__ __forceinline__ float h2f(u32 bits16) {
  return __half2float(__ushort_as_half((unsigned short)(bits16 & 0xFFFFu)));
}
// As the reference's fp16_to_f32 (src/ml/gguf/dequant.cr:257-283): any NaN becomes the canonical quiet NaN.
__device__ __forceinline__ float h2f_canonical(u32 bits16) {
  float f = h2f(bits16);
  return (f != f) ? __uint_as_float(0x7FC00000u) : f;
}

// unsigned byte k (0..3) of a dword -> float (v_cvt_f32_ubyteK)
template <int K>
__device__ __forceinline__ float ubyte_f(u32 v) {
  return (float)((v >> (8 * K)) & 0xFFu);
}

// Sum over the 64 lanes of a wavefront. In-row steps use DPP (quad_perm, row_ror); the four
// 16-lane row sums are combined through v_readlane. Every lane returns the total.
__device__ __forceinline__ float wave_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));   // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, false));  // row_ror:4
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, false));  // row_ror:8
  int iv = __builtin_bit_cast(int, v);
  float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));
  float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
  float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));
  float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
  return (r0 + r1) + (r2 + r3);
}

// K-quant 6-bit (scale, min) pair j of a 12-byte packed field held as three little-endian dwords
// (src/ml/gguf/dequant.cr:240-249).
__device__ __forceinline__ u32 k4_byte(u32 s0, u32 s1, u32 s2, int k) {
  u32 w = (k < 4) ? s0 : ((k < 8) ? s1 : s2);
  return (w >> (8 * (k & 3))) & 0xFFu;
}
__device__ __forceinline__ void get_scale_min_k4(int j, u32 s0, u32 s1, u32 s2, u32& sc, u32& m) {
  if (j < 4) {
    sc = k4_byte(s0, s1, s2, j) & 63u;
    m = k4_byte(s0, s1, s2, j + 4) & 63u;
  } else {
    sc = (k4_byte(s0, s1, s2, j + 4) & 0x0Fu) | ((k4_byte(s0, s1, s2, j - 4) >> 6) << 4);
    m = (k4_byte(s0, s1, s2, j + 4) >> 4) | ((k4_byte(s0, s1, s2, j) >> 6) << 4);
  }
}

// (scale, min) of the two sub-blocks 2g and 2g+1 at once, as 16-bit pairs (low byte = sub-block 2g).
// sh = 16*(g&1), upper = (g >= 2) are per-lane constants.
__device__ __forceinline__ void k4_pair(u32 s0, u32 s1, u32 s2, u32 sh, bool upper, u32& sc_pair, u32& m_pair) {
  u32 a0 = (s0 >> sh) & 0xFFFFu, a1 = (s1 >> sh) & 0xFFFFu, a2 = (s2 >> sh) & 0xFFFFu;
  u32 sc_lo = a0 & 0x3F3Fu, m_lo = a1 & 0x3F3Fu;
  u32 sc_up = (a2 & 0x0F0Fu) | ((a0 & 0xC0C0u) >> 2);
  u32 m_up = ((a2 >> 4) & 0x0F0Fu) | ((a1 & 0xC0C0u) >> 2);
  sc_pair = upper ? sc_up : sc_lo;
  m_pair = upper ? m_up : m_lo;
}

// silu(g) * u in fp32: g / (1 + exp(-g)), then times u (bin/cuda_ffn_sequence_probe.cr:189-191)
__device__ __forceinline__ float swiglu_one(float g, float u) {
  const float s = g / (1.0f + expf(-g));
  return s * u;
}
