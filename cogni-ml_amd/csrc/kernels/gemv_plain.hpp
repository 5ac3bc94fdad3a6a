// Matrix-vector / small matmul over the three weight types of the reference's fused matmul that are not block-quantized
// K- or Q8 formats: F32, F16 and IQ4_NL (src/ml/gguf/quant_matmul.cr:30-32, 272-368):
//   out[m][o] = (residual ? residual[m][o] : 0) + sum_j x[m][j] * w(o, j)
// with w(o, j) the float itself, the binary16 value widened, or d * table[q] of an 18-byte IQ4_NL block (d: f16, then 16
// bytes: element e < 16 of the block is the low nibble of byte e, element 16 + e its high nibble; the last block of a row
// is clipped to in_dim, quant_matmul.cr:296-312). These types hold embeddings, norms and small projections in the
// reference's models; the kernels are plain: fp32 accumulation, no staging.
//
// Kernel ABI: (w_raw, x, residual, out, in_dim:u32, out_dim:u32, tokens:u32); residual may be null. Block 256 = four
// wavefronts, one output row per wavefront at a time, any grid (the workgroups walk the rows); tokens go in groups of up to
// four whose sums a lane holds in registers, the row is re-read per group. Rows of any in_dim: the 16-byte loads are taken
// only where in_dim is a multiple of 4 (rows and x rows are then aligned), single elements otherwise.
#pragma once
#include "common.hpp"
#include "dequant.hpp"

#define GEMV_PLAIN_BLOCK 256
#define GEMV_PLAIN_TOKENS 4

struct PlainF32 {
  static __device__ __forceinline__ size_t row_bytes(u32 in_dim) { return (size_t)in_dim * 4; }
  static __device__ __forceinline__ float at(const uint8_t* row, u32 j) { return reinterpret_cast<const float*>(row)[j]; }
  static __device__ __forceinline__ float4 at4(const uint8_t* row, u32 j) { return *reinterpret_cast<const float4*>(row + (size_t)j * 4); }
};
struct PlainF16 {
  static __device__ __forceinline__ size_t row_bytes(u32 in_dim) { return (size_t)in_dim * 2; }
  static __device__ __forceinline__ float at(const uint8_t* row, u32 j) { return h2f(ld2(row + (size_t)j * 2)); }
  static __device__ __forceinline__ float4 at4(const uint8_t* row, u32 j) {
    const uint2 v = *reinterpret_cast<const uint2*>(row + (size_t)j * 2);
    return make_float4(h2f(v.x), h2f(v.x >> 16), h2f(v.y), h2f(v.y >> 16));
  }
};

template <class T>
__device__ __forceinline__ void gemv_plain_core(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                const float* __restrict__ residual, float* __restrict__ out, u32 in_dim,
                                                u32 out_dim, u32 tokens) {
  const u32 lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool vec = (in_dim & 3u) == 0;
  for (u32 row = blockIdx.x * 4 + wave; row < out_dim; row += gridDim.x * 4) {
    const uint8_t* rp = w + (size_t)row * T::row_bytes(in_dim);
    for (u32 m0 = 0; m0 < tokens; m0 += GEMV_PLAIN_TOKENS) {
      const u32 nm = min(tokens - m0, (u32)GEMV_PLAIN_TOKENS);
      float acc[GEMV_PLAIN_TOKENS] = {0.f, 0.f, 0.f, 0.f};
      if (vec) {
        for (u32 j = lane * 4; j < in_dim; j += 256) {
          const float4 wv = T::at4(rp, j);
#pragma unroll
          for (u32 m = 0; m < GEMV_PLAIN_TOKENS; m++) {
            if (m < nm) {
              const float4 xv = *reinterpret_cast<const float4*>(x + (size_t)(m0 + m) * in_dim + j);
              acc[m] = fmaf(xv.x, wv.x, acc[m]);
              acc[m] = fmaf(xv.y, wv.y, acc[m]);
              acc[m] = fmaf(xv.z, wv.z, acc[m]);
              acc[m] = fmaf(xv.w, wv.w, acc[m]);
            }
          }
        }
      } else {
        for (u32 j = lane; j < in_dim; j += 64) {
          const float wv = T::at(rp, j);
#pragma unroll
          for (u32 m = 0; m < GEMV_PLAIN_TOKENS; m++)
            if (m < nm) acc[m] = fmaf(x[(size_t)(m0 + m) * in_dim + j], wv, acc[m]);
        }
      }
#pragma unroll
      for (u32 m = 0; m < GEMV_PLAIN_TOKENS; m++) {
        const float s = wave_sum(acc[m]);
        if (lane == 0 && m < nm) {
          const size_t oi = (size_t)(m0 + m) * out_dim + row;
          out[oi] = residual ? residual[oi] + s : s;
        }
      }
    }
  }
}

extern "C" __global__ __launch_bounds__(GEMV_PLAIN_BLOCK) void f32_gemv_plain_f32(const uint8_t* w, const float* x, const float* residual,
                                                                                 float* out, u32 in_dim, u32 out_dim, u32 tokens) {
  gemv_plain_core<PlainF32>(w, x, residual, out, in_dim, out_dim, tokens);
}
extern "C" __global__ __launch_bounds__(GEMV_PLAIN_BLOCK) void f16_gemv_plain_f32(const uint8_t* w, const float* x, const float* residual,
                                                                                 float* out, u32 in_dim, u32 out_dim, u32 tokens) {
  gemv_plain_core<PlainF16>(w, x, residual, out, in_dim, out_dim, tokens);
}

// IQ4_NL: two lanes per 32-element block, lane parity = half of the block (low nibbles: elements 0..15, high nibbles:
// 16..31), 32 blocks per step of a wavefront. The block scale is applied once per block half: d * sum(x * table[q]).
extern "C" __global__ __launch_bounds__(GEMV_PLAIN_BLOCK) void iq4_nl_gemv_plain_f32(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                                                    const float* __restrict__ residual, float* __restrict__ out,
                                                                                    u32 in_dim, u32 out_dim, u32 tokens) {
  const u32 lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const u32 nb = (in_dim + 31) >> 5, half = lane & 1;
  for (u32 row = blockIdx.x * 4 + wave; row < out_dim; row += gridDim.x * 4) {
    const uint8_t* rp = w + (size_t)row * nb * 18;
    for (u32 m0 = 0; m0 < tokens; m0 += GEMV_PLAIN_TOKENS) {
      const u32 nm = min(tokens - m0, (u32)GEMV_PLAIN_TOKENS);
      float acc[GEMV_PLAIN_TOKENS] = {0.f, 0.f, 0.f, 0.f};
      for (u32 b = lane >> 1; b < nb; b += 32) {
        const uint8_t* bp = rp + (size_t)b * 18;
        const float d = h2f(ld2(bp));
        const uint4 q = ld16(bp + 2);
        const u32 qs[4] = {q.x, q.y, q.z, q.w};
        const u32 base = b * 32 + 16 * half;
        const u32 count = base < in_dim ? min(16u, in_dim - base) : 0u;
        float part[GEMV_PLAIN_TOKENS] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (u32 e = 0; e < 16; e++) {
          const u32 byte = (qs[e >> 2] >> (8 * (e & 3))) & 0xFFu;
          const float tv = kIq4nlValues[half ? byte >> 4 : byte & 15u];
          if (e < count) {
#pragma unroll
            for (u32 m = 0; m < GEMV_PLAIN_TOKENS; m++)
              if (m < nm) part[m] = fmaf(x[(size_t)(m0 + m) * in_dim + base + e], tv, part[m]);
          }
        }
#pragma unroll
        for (u32 m = 0; m < GEMV_PLAIN_TOKENS; m++)
          if (count) acc[m] = fmaf(d, part[m], acc[m]);   // (a half beyond in_dim adds nothing, whatever its d)
      }
#pragma unroll
      for (u32 m = 0; m < GEMV_PLAIN_TOKENS; m++) {
        const float s = wave_sum(acc[m]);
        if (lane == 0 && m < nm) {
          const size_t oi = (size_t)(m0 + m) * out_dim + row;
          out[oi] = residual ? residual[oi] + s : s;
        }
      }
    }
  }
}
