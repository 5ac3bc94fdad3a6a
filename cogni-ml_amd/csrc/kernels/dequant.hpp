// Bulk dequantize kernels: raw GGUF blocks -> float32, bit-exact with the reference's
// Dequant.dequantize_* (src/ml/gguf/dequant.cr). Every product and difference is rounded on its
// own (the translation unit is built with -ffp-contract=off), in the reference's association:
//   Q4_K/Q5_K  y = (d*sc)*q - (dmin*m)        dequant.cr:122-133, 167-184
//   Q6_K       y = (d*sc)*q                   dequant.cr:223-226
//   Q8_0       y = d*q                        dequant.cr:66
//   IQ4_NL     y = d*table[q]                 dequant.cr:88-97
//
// These kernels are write bound (4 bytes out per 4.5..8.5 bits in). One wavefront produces 256
// consecutive floats per step: lane l owns elements 4l..4l+3 and issues one 16-byte store, so
// each store instruction writes 1 KiB of contiguous memory. Signature of every kernel:
//   (const uint8_t* w_raw, float* out, uint64 n_elements), block = 256 threads, any grid size.
#pragma once
#include "common.hpp"

#define DEQ_BLOCK 256
#define DEQ_WAVES (DEQ_BLOCK / WAVE)

// The output of a bulk dequantize is written once and not read again by the kernel: a streaming (non-temporal) store.
#ifndef DEQ_STREAM_STORES
#define DEQ_STREAM_STORES 1
#endif
typedef float deq_f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void deq_store4(float* p, float4 y) {
  const deq_f32x4 v = {y.x, y.y, y.z, y.w};
  if (DEQ_STREAM_STORES) __builtin_nontemporal_store(v, reinterpret_cast<deq_f32x4*>(p));
  else *reinterpret_cast<deq_f32x4*>(p) = v;
}

// Elements past the last whole block stay zero, as in the reference's zero-initialised result.
__device__ __forceinline__ void zero_tail(float* out, u64 from, u64 n) {
  u64 tid = (u64)blockIdx.x * blockDim.x + threadIdx.x;
  u64 step = (u64)gridDim.x * blockDim.x;
  for (u64 e = from + tid; e < n; e += step) out[e] = 0.0f;
}

// Elements 4 lane .. 4 lane + 3 of the 256-element super-block at bp.
__device__ __forceinline__ float4 deq4_q4_k(const uint8_t* bp, int lane) {
  const int g = lane >> 4, li = lane & 15, hi = li >> 3;
  const uint4 hdr = ld16(bp);
  u32 q = ld4(bp + 16 + 32 * g + 4 * (li & 7));
  u32 sc, m;
  get_scale_min_k4(2 * g + hi, hdr.y, hdr.z, hdr.w, sc, m);
  const float d = h2f_canonical(hdr.x), dmin = h2f_canonical(hdr.x >> 16);
  const float d1 = d * (float)sc;
  const float m1 = dmin * (float)m;
  q = (hi ? (q >> 4) : q) & 0x0F0F0F0Fu;
  float4 y;
  y.x = d1 * ubyte_f<0>(q) - m1;
  y.y = d1 * ubyte_f<1>(q) - m1;
  y.z = d1 * ubyte_f<2>(q) - m1;
  y.w = d1 * ubyte_f<3>(q) - m1;
  return y;
}

extern "C" __global__ __launch_bounds__(DEQ_BLOCK) void dequantize_q4_k_f32(const uint8_t* __restrict__ w,
                                                                              float* __restrict__ out, u64 n) {
  const u64 nb = n >> 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (u64 b = (u64)blockIdx.x * DEQ_WAVES + wave; b < nb; b += (u64)gridDim.x * DEQ_WAVES)
    deq_store4(out + b * 256 + 4 * lane, deq4_q4_k(w + b * 144, lane));
  zero_tail(out, nb << 8, n);
}

extern "C" __global__ __launch_bounds__(DEQ_BLOCK) void dequantize_q5_k_f32(const uint8_t* __restrict__ w,
                                                                              float* __restrict__ out, u64 n) {
  const u64 nb = n >> 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane >> 4, li = lane & 15, hi = li >> 3, l0 = 4 * (li & 7);
  for (u64 b = (u64)blockIdx.x * DEQ_WAVES + wave; b < nb; b += (u64)gridDim.x * DEQ_WAVES) {
    const uint8_t* bp = w + b * 176;
    const uint4 hdr = ld16(bp);
    const u32 qh = ld4(bp + 16 + l0);
    u32 q = ld4(bp + 48 + 32 * g + l0);
    u32 sc, m;
    get_scale_min_k4(2 * g + hi, hdr.y, hdr.z, hdr.w, sc, m);
    const float d = h2f_canonical(hdr.x), dmin = h2f_canonical(hdr.x >> 16);
    const float d1 = d * (float)sc;
    const float m1 = dmin * (float)m;
    q = (hi ? (q >> 4) : q) & 0x0F0F0F0Fu;
    q |= ((qh >> (2 * g + hi)) & 0x01010101u) << 4;
    float4 y;
    y.x = d1 * ubyte_f<0>(q) - m1;
    y.y = d1 * ubyte_f<1>(q) - m1;
    y.z = d1 * ubyte_f<2>(q) - m1;
    y.w = d1 * ubyte_f<3>(q) - m1;
    deq_store4(out + b * 256 + 4 * lane, y);
  }
  zero_tail(out, nb << 8, n);
}

__device__ __forceinline__ float4 deq4_q6_k(const uint8_t* bp, int lane) {   // bp is 2-byte aligned only
  const int half = lane >> 5, k = (lane & 31) >> 3, l0 = 4 * (lane & 7);
  u32 ql = ld4(bp + 64 * half + 32 * (k & 1) + l0);
  const u32 qh = ld4(bp + 128 + 32 * half + l0);
  const int sc = (int)(signed char)bp[192 + 8 * half + 2 * k + (l0 >> 4)];
  const float d = h2f_canonical(ld2(bp + 208));
  const float ds = d * (float)sc;
  ql = ((k < 2) ? ql : (ql >> 4)) & 0x0F0F0F0Fu;
  const u32 q = ql | (((qh >> (2 * k)) & 0x03030303u) << 4);
  float4 y;
  y.x = ds * (float)((int)((q >> 0) & 0xFFu) - 32);
  y.y = ds * (float)((int)((q >> 8) & 0xFFu) - 32);
  y.z = ds * (float)((int)((q >> 16) & 0xFFu) - 32);
  y.w = ds * (float)((int)((q >> 24) & 0xFFu) - 32);
  return y;
}

extern "C" __global__ __launch_bounds__(DEQ_BLOCK) void dequantize_q6_k_f32(const uint8_t* __restrict__ w,
                                                                              float* __restrict__ out, u64 n) {
  const u64 nb = n >> 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (u64 b = (u64)blockIdx.x * DEQ_WAVES + wave; b < nb; b += (u64)gridDim.x * DEQ_WAVES)
    deq_store4(out + b * 256 + 4 * lane, deq4_q6_k(w + b * 210, lane));
  zero_tail(out, nb << 8, n);
}

// One row of a Q4_K / Q6_K embedding matrix, picked by a token id that lives on the device - the reference's
// embed_q4k_f32_from_token_id_cuda (src/ml/cuda/kernels/embed_q4k_probe.ptx:5-13; host side
// bin/cuda_mixed_stack_probe.cr:900-947), same parameters:
//   (w_raw, token_ids:u32*, output:f32*, history:u32*, token_index:u32, hidden_dim:u32, vocab_size:u32)
// output[0..hidden_dim) = dequantized row token_ids[0] (zeros if the id is not below vocab_size), and
// history[token_index] = token_ids[0]. hidden_dim is a multiple of 256; block 256, grid ceil(hidden_dim / 1024)
// (a wavefront per super-block; the reference uses a thread per element, grid hidden_dim / 256).
#define EMBED_KERNEL(NAME, DEQ4, BB)                                                                              \
  extern "C" __global__ __launch_bounds__(DEQ_BLOCK) void NAME(const uint8_t* w, const u32* token_ids, float* output, \
                                                               u32* history, u32 token_index, u32 hidden_dim,     \
                                                               u32 vocab_size) {                                  \
    const u32 id = token_ids[0];                                                                                  \
    if (blockIdx.x == 0 && threadIdx.x == 0) history[token_index] = id;                                           \
    const int lane = threadIdx.x & 63;                                                                            \
    const u32 b = blockIdx.x * DEQ_WAVES + (threadIdx.x >> 6), nb = hidden_dim >> 8;                              \
    if (b >= nb) return;                                                                                          \
    float4 y = make_float4(0.f, 0.f, 0.f, 0.f);                                                                   \
    if (id < vocab_size) y = DEQ4(w + ((size_t)id * nb + b) * BB, lane);                                          \
    *reinterpret_cast<float4*>(output + b * 256 + 4 * lane) = y;                                                  \
  }
EMBED_KERNEL(embed_q4_k_f32_from_token_id, deq4_q4_k, 144)
EMBED_KERNEL(embed_q6_k_f32_from_token_id, deq4_q6_k, 210)

// Q8_0 and IQ4_NL: 32-element blocks, ceil(n/32) of them, the last one clipped to n.
extern "C" __global__ __launch_bounds__(DEQ_BLOCK) void dequantize_q8_0_f32(const uint8_t* __restrict__ w,
                                                                              float* __restrict__ out, u64 n) {
  const u64 ngroups = (n + 255) >> 8;  // 8 blocks per wavefront step
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (u64 gi = (u64)blockIdx.x * DEQ_WAVES + wave; gi < ngroups; gi += (u64)gridDim.x * DEQ_WAVES) {
    const u64 e = gi * 256 + 4 * lane;
    if (e >= n) continue;
    const uint8_t* bp = w + (e >> 5) * 34;
    const float d = h2f_canonical(ld2(bp));
    const u32 q = ld4(bp + 2 + (e & 31));
    float y[4];
    y[0] = d * (float)(int)(signed char)(q & 0xFFu);
    y[1] = d * (float)(int)(signed char)((q >> 8) & 0xFFu);
    y[2] = d * (float)(int)(signed char)((q >> 16) & 0xFFu);
    y[3] = d * (float)(int)(signed char)((q >> 24) & 0xFFu);
    if (e + 4 <= n) {
      deq_store4(out + e, make_float4(y[0], y[1], y[2], y[3]));
    } else {
      for (int c = 0; c < 4; c++)
        if (e + c < n) out[e + c] = y[c];
    }
  }
}

__constant__ float kIq4nlValues[16] = {-127.f, -104.f, -83.f, -65.f, -49.f, -35.f, -22.f, -10.f,
                                       1.f,    13.f,   25.f,  38.f,  53.f,  69.f,  89.f,  113.f};

extern "C" __global__ __launch_bounds__(DEQ_BLOCK) void dequantize_iq4_nl_f32(const uint8_t* __restrict__ w,
                                                                                float* __restrict__ out, u64 n) {
  const u64 ngroups = (n + 255) >> 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (u64 gi = (u64)blockIdx.x * DEQ_WAVES + wave; gi < ngroups; gi += (u64)gridDim.x * DEQ_WAVES) {
    const u64 e = gi * 256 + 4 * lane;
    if (e >= n) continue;
    const uint8_t* bp = w + (e >> 5) * 18;
    const float d = h2f_canonical(ld2(bp));
    const int idx = (int)(e & 31);             // low nibbles -> elements 0..15, high nibbles -> 16..31
    u32 q = ld4(bp + 2 + (idx & 15));
    q = ((idx < 16) ? q : (q >> 4)) & 0x0F0F0F0Fu;
    float y[4];
    y[0] = d * kIq4nlValues[q & 0xFFu];
    y[1] = d * kIq4nlValues[(q >> 8) & 0xFFu];
    y[2] = d * kIq4nlValues[(q >> 16) & 0xFFu];
    y[3] = d * kIq4nlValues[(q >> 24) & 0xFFu];
    if (e + 4 <= n) {
      deq_store4(out + e, make_float4(y[0], y[1], y[2], y[3]));
    } else {
      for (int c = 0; c < 4; c++)
        if (e + c < n) out[e + c] = y[c];
    }
  }
}

extern "C" __global__ __launch_bounds__(DEQ_BLOCK) void dequantize_f16_f32(const uint8_t* __restrict__ w,
                                                                             float* __restrict__ out, u64 n) {
  const u64 tid = (u64)blockIdx.x * blockDim.x + threadIdx.x, step = (u64)gridDim.x * blockDim.x;
  for (u64 e = tid * 4; e < n; e += step * 4) {
    if (e + 4 <= n) {
      const uint2 h = ld8(w + 2 * e);
      deq_store4(out + e, make_float4(h2f_canonical(h.x), h2f_canonical(h.x >> 16), h2f_canonical(h.y), h2f_canonical(h.y >> 16)));
    } else {
      for (u64 c = e; c < n; c++) out[c] = h2f_canonical(ld2(w + 2 * c));
    }
  }
}

extern "C" __global__ __launch_bounds__(DEQ_BLOCK) void dequantize_f32_f32(const uint8_t* __restrict__ w,
                                                                             float* __restrict__ out, u64 n) {
  const u64 tid = (u64)blockIdx.x * blockDim.x + threadIdx.x, step = (u64)gridDim.x * blockDim.x;
  for (u64 e = tid; e < n; e += step) out[e] = __uint_as_float(ld4(w + 4 * e));
}
