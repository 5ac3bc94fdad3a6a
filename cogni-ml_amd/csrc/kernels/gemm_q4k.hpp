// Prefill GEMM over raw Q4_K (and, as the same template, Q5_K) weights: out[m][n] = (bias[n] +) sum_k x[m][k] * deq(W[n][k]), M >= 9.
// fp16 operands, v_mfma_f32_32x32x16_f16, fp32 accumulation (the precision of the reference's Metal
// prefill kernels, which round both x and the dequantized weights to half:
// src/ml/gguf/kernels/gemm_q4k.metal:97-105,678-686). On gfx950 the 32x32x16 instruction sustains twice
// the rate of 16x16x32 (about 32 vs 2 x 32 clocks for the same 32768 flops per SIMD), hence the tile shape.
//
// Kernels:
//   pack_x_f16_q4k  (x:f32 [m][in_dim], xp:f16, m:u32, in_dim:u32)           block 256, grid ceil(m/128) * 16 * in_dim/256
//   q4_k_gemm_f16, q5_k_gemm_f16
//                   (w_raw, xp, bias|null, out:f32 [m][out_dim], in_dim:u32, out_dim:u32, m:u32, bias_stride:u32)
//                   block 256, grid (gemm_grid_x(ceil(m/128), ceil(out_dim/192)) from gemv_config.h, k splits), no dynamic LDS
//                   (156 / 160 KiB static); with k splits > 1 `out` is `splits` planes of [m][out_dim] and bias is null.
//                   bias_stride 0: a [out_dim] bias added to every token; out_dim: a [m][out_dim] residual (it may be
//                   `out` itself) - the reference's f32out_add prefill pipelines (gemm_mm.metal:651)
//   q4_k_gemm_swiglu_f16
//                   (w_gate, w_up, xp, out:f32 [m][out_dim], in_dim:u32, out_dim:u32, m:u32): out = silu(x W_gate^T) * (x W_up^T),
//                   the reference's simd_mm_q4k_h16_b64_swiglu (gemm_q4k.metal:1233). A tile is 128 tokens x 96 rows of each
//                   matrix; block 256, grid gemm_grid_x(ceil(m/128), ceil(out_dim/96)), no k split
//   q4_k_gemm_swiglu_pack_q4k_f16, q4_k_gemm_swiglu_pack_q6k_f16
//                   (w_gate, w_up, xp, out | null, xq, in_dim, out_dim, m): the same, and the products written as the packed
//                   activations of the next GEMM (the down projection) as pack_x_f16_q4k | pack_x_f16_q6k would write them
//   gemm_sum_splits_f32 (planes, bias|null, out, m*out_dim:u32, out_dim:u32, splits:u32, bias_stride:u32)   block 256, grid ceil(m*out_dim/1024)
//
// Tiling. A workgroup (4 wavefronts) owns 128 tokens x 192 weight rows, so 512 x 12288 gives 256
// workgroups, one per CU. K is walked one 256-value super-block at a time = 16 MFMA k-steps of 16.
// The four wavefronts split the tile as (row half nh) x (k-step half kh): a wavefront accumulates
// 128 tokens x 96 rows (4 x 3 tiles of 32 x 32, 192 accumulator registers) over 8 of the 16 k-steps of
// every super-block; the two k halves are added through LDS once, at the end. Every weight is
// dequantized by exactly one wavefront and reused for 128 tokens.
//
// The weights pass through LDS as raw bytes only (27 KiB per super-block, copied global -> LDS 16 bytes per lane
// along the rows and picked up once per super-block by the lanes that decode them); they are never stored
// dequantized. In MFMA terms a lane is (weight row j = lane % 32, k-group kg = lane / 32)
// and supplies 8 k values per k-step. Lane (j, kg) of a kh wavefront owns the 64-value group
// g = 2*kh + kg of its row's super-block: the 32 bytes qs[32g, 32g+32) as two 16-byte LDS reads, one
// (scale, min) pair decode. Eight consecutive bytes give two k-steps: their low nibbles (sub-block 2g)
// and their high nibbles (sub-block 2g+1). A masked dword (q & 0x000F000F) | 0x64006400 is the half2
// (1024 + n0, 1024 + n4); subtracting 1024 and one packed fma give fp16(d*sc*n - dmin*m) for two
// weights. The 8 k values of a lane therefore come in nibble order (bytes 0,2,1,3,4,6,5,7);
// pack_x_f16_q4k writes x in exactly that order, already laid out as the LDS image
// [k-step][k-group][token][8 halves] of each (128-token tile, super-block), so staging x is a straight
// 64 KiB copy (global_load_lds_dwordx4, no registers) and an A operand is one conflict-free ds_read_b128.
//
// LDS traffic in the loop: the activations, 4 KiB read per wavefront and k-step for 12 MFMAs, and the raw weights,
// 9 x 16 bytes per lane and super-block. The x tile of the next super-block is copied while the current one is
// consumed (two 64 KiB buffers); the raw weight bytes of the next super-block are copied into the one 28 KiB
// buffer as soon as every wavefront has taken the current ones into registers.
#pragma once
#include <type_traits>
#include "common.hpp"
#include "gemv_config.h"

#define GEMM_BM 128
#define GEMM_BN 192
#define GEMM_XCDS 8

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

// Element (0..255) of a super-block that k-slot (ks, kg, e) of the MFMA stands for. ks = 8*kh + 4*h + op:
// kh = k half (which wavefront), h = 16-byte half of the lane's group, op & 1 = upper 8 bytes of that
// half, op >> 1 = high nibbles. The group is g = 2*kh + kg: the two k-groups of a wavefront read 64 adjacent
// bytes of a row, so a wavefront touches one or two cache lines per row rather than two or three.
__device__ __forceinline__ u32 gemm_k_element(u32 ks, u32 kg, u32 e) {
  const u32 kh = ks >> 3, h = (ks >> 2) & 1, op = ks & 3;
  const u32 g = 2 * kh + kg;
  const u32 perm = ((e & 1) << 1) | ((e >> 1) & 1) | (e & 4);   // 0,2,1,3,4,6,5,7
  return 64 * g + 32 * (op >> 1) + 16 * h + 8 * (op & 1) + perm;
}

// One workgroup packs 8 tokens x one super-block (256 k): the fp32 rows are read 1 KiB at a time (a wavefront
// per row), converted, transposed through LDS into the [k-step][k-group][token][8 halves] image and written out
// as 32 runs of 128 contiguous bytes. Grid: ceil(m/128) * 16 * (in_dim/256) workgroups, x fastest (1024 workgroups at
// 512 tokens x 4096: with 32 tokens per workgroup there were 256, one per compute unit, and the kernel was all latency).
#ifndef PACK_TOK
#define PACK_TOK 8
#endif
// Q6: the element order of the Q6_K kernel (gemm_q6k.hpp) instead of the Q4_K one.
template <bool Q6>
__device__ __forceinline__ void pack_x_core(const float* __restrict__ x, uint4* __restrict__ xp, u32 m, u32 in_dim) {
  // [32 (k-step, k-group)][32 tokens] uint4, each (k-step, k-group) row padded by one uint4 so that the
  // transposing 8-byte writes of a wavefront (same token, 32 different rows) spread over the banks
  __shared__ uint2 img[32 * (PACK_TOK + 1) * 2];
  const u32 nkb = in_dim >> 8;
  const u32 tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr u32 NQ = GEMM_BM / PACK_TOK;
  const u32 kb = blockIdx.x % nkb, tq = (blockIdx.x / nkb) % NQ, mt = blockIdx.x / (NQ * nkb);
  // lane -> 4 consecutive k = 4 lane .. 4 lane + 3 of the super-block; their place in the image (inverse of
  // gemm_k_element): Q4_K: group g = k / 64, high-nibble half, 16-byte half h, upper-8-bytes bit, slot 0 or 4;
  // Q6_K: 128-half n, quadrant qd, 16-run u, upper-8 bit, slot 0 or 4 (gemm_k_element_q6k)
  const u32 k0 = 4 * lane, slot4 = (k0 >> 2) & 1;
  u32 ks, kg;
  if (Q6) {
    const u32 n = k0 >> 7, qd = (k0 >> 5) & 3, u = (k0 >> 4) & 1, h8 = (k0 >> 3) & 1;
    ks = 8 * n + 2 * qd + h8;
    kg = u;
  } else {
    const u32 g = k0 >> 6, hi = (k0 >> 5) & 1, h = (k0 >> 4) & 1, up = (k0 >> 3) & 1;
    ks = 8 * (g >> 1) + 4 * h + 2 * hi + up;
    kg = g & 1;
  }
  const u32 cell = (ks * 2 + kg) * (PACK_TOK + 1);
#pragma unroll
  for (int p = 0; p < PACK_TOK / 4; p++) {
    const u32 tl = 4 * p + wave;
    const u32 row = mt * GEMM_BM + tq * PACK_TOK + tl;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row < m) __builtin_memcpy(&v, x + (size_t)row * in_dim + kb * 256 + k0, 16);
    const __half2 p0 = __floats2half2_rn(v.x, v.z), p1 = __floats2half2_rn(v.y, v.w);   // slot order 0,2,1,3
    uint2 o;
    o.x = *reinterpret_cast<const u32*>(&p0);
    o.y = *reinterpret_cast<const u32*>(&p1);
    img[(cell + tl) * 2 + slot4] = o;
  }
  __syncthreads();
  uint4* dst = xp + ((size_t)mt * nkb + kb) * 4096 + tq * PACK_TOK;
  for (u32 i = tid; i < 32 * PACK_TOK; i += 256) {
    const u32 c = i / PACK_TOK, tl = i % PACK_TOK;
    dst[c * 128 + tl] = *reinterpret_cast<const uint4*>(&img[(c * (PACK_TOK + 1) + tl) * 2]);
  }
}
extern "C" __global__ __launch_bounds__(256) void pack_x_f16_q4k(const float* x, uint4* xp, u32 m, u32 in_dim) {
  pack_x_core<false>(x, xp, m, in_dim);
}

__device__ __forceinline__ u32 h2_dup(float v) {
  const __half2 h = __float2half2_rn(v);
  return *reinterpret_cast<const u32*>(&h);
}
__device__ __forceinline__ u32 h2_fma_off(u32 t, u32 off, u32 scale, u32 negmin) {
  const __half2 q = __hadd2(*reinterpret_cast<const __half2*>(&t), *reinterpret_cast<const __half2*>(&off));
  const __half2 w = __hfma2(q, *reinterpret_cast<const __half2*>(&scale), *reinterpret_cast<const __half2*>(&negmin));
  return *reinterpret_cast<const u32*>(&w);
}

// The two x-tile buffers are separate objects so the compiler can tell the LDS-direct loads into one from
// the operand reads out of the other (otherwise every read would first wait for all loads in flight).
__shared__ uint4 gemm_xbuf0[4096];   // [16 k-steps][2 k-groups][128 tokens] uint4
__shared__ uint4 gemm_xbuf1[4096];
// Raw bytes of one super-block of the workgroup's 192 weight rows, [row][144 B] = 1728 pieces of 16 bytes. Copied
// global -> LDS 16 bytes per lane with consecutive lanes on consecutive pieces of a row (a 64-lane copy touches 7 or 8
// rows = 14 to 16 cache lines; the same bytes fetched straight into the MFMA lane layout, one row per lane, touch 64).
__shared__ uint4 gemm_wbuf[28 * 64];   // 27 copies of 64 pieces, and a 28th that keeps the four wavefronts in step
// Q5_K: the 160 bytes behind the 16-byte header of each row (qh[32], qs[128]) = 1920 pieces, 30 copies of 64 and two more
// for the same reason; with the two x buffers this is all of the 160 KiB a workgroup can have. The header (d, dmin,
// 12 scale bytes) goes from global memory straight to the lane that decodes it.
__shared__ uint4 gemm_wbuf5[32 * 64];

// Epilogue shared by the GEMM kernels. The MFMAs are issued as (weights, x), so an accumulator tile is laid out with the
// weight rows along the register index: acc[r][c][v] of lane (j, kg) belongs to token 32 r + j and weight row
// nh * 32 NT + 32 c + 8 (v / 4) + 4 kg + v % 4 (NT = 3 tiles of 32 rows per wavefront, two with the 128-row workgroup tile) - four
// consecutive output floats per register quad, which leave as one
// 16-byte store without passing through LDS. What does pass through LDS is the other k half: a kh wavefront finishes the
// token tiles r = 2 kh, 2 kh + 1 (r = kh with the 64-token tile, MT = 2) and hands the others to its partner (same nh) as 24 float4 per lane in the lane
// layout both share (kh = 0 writes into x buffer 0, kh = 1 into x buffer 1: 2 x 24 KiB each). Sum first, bias second.
template <int KH, int NT = 3, int MT = 4>
__device__ __forceinline__ void gemm_epilogue_half(float16_t (&acc)[MT][NT], const float* bias, float* out, u32 out_dim, u32 m,
                                                   u32 mt, u32 nt, u32 nh, u32 j, u32 kg, u32 lane, u32 bias_stride) {
  constexpr u32 BN = 64 * NT;   // weight rows of the workgroup tile: NT tiles of 32 rows per wavefront, two row halves
  constexpr int RH = MT / 2;    // token tiles of 32 a wavefront finishes (MT = 4: tokens 0..127 of the tile; 2: 0..63)
  float4* mine = reinterpret_cast<float4*>(KH ? gemm_xbuf1 : gemm_xbuf0) + nh * (8 * NT) * 64 + lane;
  const float4* theirs = reinterpret_cast<const float4*>(KH ? gemm_xbuf0 : gemm_xbuf1) + nh * (8 * NT) * 64 + lane;
#pragma unroll
  for (int rr = 0; rr < RH; rr++)
#pragma unroll
    for (int c = 0; c < NT; c++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const float16_t& t = acc[RH * (1 - KH) + rr][c];
        mine[((rr * NT + c) * 4 + g4) * 64] = make_float4(t[4 * g4], t[4 * g4 + 1], t[4 * g4 + 2], t[4 * g4 + 3]);
      }
  __syncthreads();
  const bool vec = (out_dim & 3u) == 0;
  if (vec && mt * GEMM_BM + 32 * MT <= m && nt * BN + BN <= out_dim) {
    // a whole tile: one address per token row, the 12 stores of a row at constant offsets from it, 16 bytes each (kept
    // apart from the general path below so that the compiler cannot merge the two into single-float stores)
#pragma unroll
    for (int rr = 0; rr < RH; rr++) {
      const size_t token = mt * GEMM_BM + 32 * (RH * KH + rr) + j;
      const u32 col = nt * BN + nh * (32 * NT) + 4 * kg;
      float* base = out + token * out_dim + col;
      // what is added: a [out_dim] bias, or row `token` of a residual (which may be `out`: a thread reads the values it
      // is about to overwrite, nobody else's)
      const float* bbase = bias ? bias + token * bias_stride + col : nullptr;
#pragma unroll
      for (int c = 0; c < NT; c++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const float16_t& t = acc[RH * KH + rr][c];
          const float4 p = theirs[((rr * NT + c) * 4 + g4) * 64];
          float4 o = KH ? make_float4(p.x + t[4 * g4], p.y + t[4 * g4 + 1], p.z + t[4 * g4 + 2], p.w + t[4 * g4 + 3])
                        : make_float4(t[4 * g4] + p.x, t[4 * g4 + 1] + p.y, t[4 * g4 + 2] + p.z, t[4 * g4 + 3] + p.w);
          if (bbase) {
            const float* b = bbase + 32 * c + 8 * g4;
            o.x += b[0]; o.y += b[1]; o.z += b[2]; o.w += b[3];
          }
          *reinterpret_cast<float4*>(base + 32 * c + 8 * g4) = o;
        }
    }
    return;
  }
  // a clipped tile: a lane's four values go out as 16 bytes where the row allows it and they all exist, else one by one.
  // (Two copies of the loop, chosen once, rather than one loop with the choice inside: there the compiler merges the
  // two kinds of store into single floats for every tile.)
  auto tail = [&](auto vec16) {
#pragma unroll
    for (int rr = 0; rr < RH; rr++) {
      const u32 token = mt * GEMM_BM + 32 * (RH * KH + rr) + j;
#pragma unroll
      for (int c = 0; c < NT; c++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const float16_t& t = acc[RH * KH + rr][c];
          const float4 p = theirs[((rr * NT + c) * 4 + g4) * 64];
          // (k half 0) + (k half 1) whichever of the two this wavefront holds
          float4 o = KH ? make_float4(p.x + t[4 * g4], p.y + t[4 * g4 + 1], p.z + t[4 * g4 + 2], p.w + t[4 * g4 + 3])
                        : make_float4(t[4 * g4] + p.x, t[4 * g4 + 1] + p.y, t[4 * g4 + 2] + p.z, t[4 * g4 + 3] + p.w);
          const u32 n = nt * BN + nh * (32 * NT) + 32 * c + 8 * g4 + 4 * kg;
          if (token >= m || n >= out_dim) continue;
          float* dst = out + (size_t)token * out_dim + n;
          const float* b = bias ? bias + (size_t)token * bias_stride + n : nullptr;   // bias, or a residual (stride out_dim)
          if (decltype(vec16)::value && n + 4 <= out_dim) {
            if (b) {
              o.x += b[0]; o.y += b[1]; o.z += b[2]; o.w += b[3];
            }
            *reinterpret_cast<float4*>(dst) = o;
          } else {
            const float ov[4] = {o.x, o.y, o.z, o.w};
            for (u32 e = 0; e < 4 && n + e < out_dim; e++) dst[e] = ov[e] + (b ? b[e] : 0.0f);
          }
        }
    }
  };
  if (vec) tail(std::true_type{});
  else tail(std::false_type{});
}
template <int NT, int MT>
__device__ __forceinline__ void gemm_epilogue(float16_t (&acc)[MT][NT], const float* bias, float* out, u32 out_dim, u32 m,
                                              u32 mt, u32 nt, u32 nh, u32 kh, u32 j, u32 kg, u32 tid, u32 bias_stride = 0) {
  if (kh == 0) gemm_epilogue_half<0, NT, MT>(acc, bias, out, out_dim, m, mt, nt, nh, j, kg, tid & 63, bias_stride);
  else gemm_epilogue_half<1, NT, MT>(acc, bias, out, out_dim, m, mt, nt, nh, j, kg, tid & 63, bias_stride);
}

// Epilogue of the gate | up kernel: the nh = 0 wavefronts hold 96 gate rows, the nh = 1 wavefronts the same 96 rows of up,
// in the same lane layout. First the two k halves are added as above, each wavefront finishing its two token tiles in
// place; then the gate and the up wavefront of the same kh exchange half of their sums through LDS and each stores
// silu(gate) * up for its half of the column quads: 128 tokens x 96 outputs per workgroup, four consecutive floats per
// register quad.
// PACK (12: the Q4_K / Q5_K order, 14: the Q6_K order): the products also leave as fp16 in the packed layout the GEMM
// kernels read their activations from (what pack_x_f16_q4k | pack_x_f16_q6k would make of `out`, bit for bit), so that the
// GEMM behind this one - the down projection - needs no pack launch and `out` may be null. A lane's four consecutive
// products are one 8-byte half of a 16-byte cell of that layout, and the lane pair (kg = 0, 1) fills the cell: a wavefront
// stores 512 contiguous bytes. out_dim is a multiple of 256 then (it is the row length of the next matrix).
template <int KH, int PACK = 0, int MT = 4>
__device__ __forceinline__ void gemm_epilogue_swiglu_half(float16_t (&acc)[MT][3], float* out, u32 out_dim, u32 m, u32 mt, u32 nt,
                                                          u32 nh, u32 j, u32 kg, u32 lane, uint2* xq = nullptr) {
  constexpr int RH = MT / 2;   // token tiles of 32 a wavefront finishes (MT = 2: the 64-token kernels)
  float4* mine = reinterpret_cast<float4*>(KH ? gemm_xbuf1 : gemm_xbuf0) + nh * (12 * RH) * 64 + lane;
  const float4* theirs = reinterpret_cast<const float4*>(KH ? gemm_xbuf0 : gemm_xbuf1) + nh * (12 * RH) * 64 + lane;
#pragma unroll
  for (int rr = 0; rr < RH; rr++)
#pragma unroll
    for (int c = 0; c < 3; c++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const float16_t& t = acc[RH * (1 - KH) + rr][c];
        mine[((rr * 3 + c) * 4 + g4) * 64] = make_float4(t[4 * g4], t[4 * g4 + 1], t[4 * g4 + 2], t[4 * g4 + 3]);
      }
  __syncthreads();
#pragma unroll
  for (int rr = 0; rr < RH; rr++)
#pragma unroll
    for (int c = 0; c < 3; c++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        float16_t& t = acc[RH * KH + rr][c];
        const float4 p = theirs[((rr * 3 + c) * 4 + g4) * 64];
        // (k half 0) + (k half 1), in that order whichever of the two this wavefront holds
        t[4 * g4] = KH ? p.x + t[4 * g4] : t[4 * g4] + p.x;
        t[4 * g4 + 1] = KH ? p.y + t[4 * g4 + 1] : t[4 * g4 + 1] + p.y;
        t[4 * g4 + 2] = KH ? p.z + t[4 * g4 + 2] : t[4 * g4 + 2] + p.z;
        t[4 * g4 + 3] = KH ? p.w + t[4 * g4 + 3] : t[4 * g4 + 3] + p.w;
      }
  __syncthreads();   // the hand-over regions have been read: they carry the exchanged sums next
  // silu(gate) * up costs some thirty instructions a value, so both wavefronts of a pair finish half of the cells each:
  // the gate wavefront keeps column quads g4 = 0, 1 of every (token tile, column group) and gives 2, 3 to the up
  // wavefront, which gives its 0, 1 in return. Region nh of the buffer holds what wavefront nh gives.
  float4* xch = reinterpret_cast<float4*>(KH ? gemm_xbuf1 : gemm_xbuf0) + lane;
  const bool vec = (out_dim & 3u) == 0;
  auto give = [&](auto nhc) {
    constexpr int NH = decltype(nhc)::value;
#pragma unroll
    for (int rr = 0; rr < RH; rr++)
#pragma unroll
      for (int c = 0; c < 3; c++)
#pragma unroll
        for (int gg = 0; gg < 2; gg++) {
          const int g4 = NH == 0 ? 2 + gg : gg;   // the quad given away
          const float16_t& t = acc[RH * KH + rr][c];
          xch[(NH * (RH * 6) + (rr * 3 + c) * 2 + gg) * 64] = make_float4(t[4 * g4], t[4 * g4 + 1], t[4 * g4 + 2], t[4 * g4 + 3]);
        }
  };
  auto finish = [&](auto nhc) {
    constexpr int NH = decltype(nhc)::value;
#pragma unroll
    for (int rr = 0; rr < RH; rr++) {
      const u32 token = mt * GEMM_BM + 32 * (RH * KH + rr) + j;
#pragma unroll
      for (int c = 0; c < 3; c++)
#pragma unroll
        for (int gg = 0; gg < 2; gg++) {
          const int g4 = NH == 0 ? gg : 2 + gg;   // the quad finished here
          const float16_t& t = acc[RH * KH + rr][c];
          const float4 other = xch[((1 - NH) * (RH * 6) + (rr * 3 + c) * 2 + gg) * 64];
          const float4 mine4 = make_float4(t[4 * g4], t[4 * g4 + 1], t[4 * g4 + 2], t[4 * g4 + 3]);
          const float4 g = NH == 0 ? mine4 : other, u = NH == 0 ? other : mine4;
          const float4 o = make_float4(swiglu_one(g.x, u.x), swiglu_one(g.y, u.y), swiglu_one(g.z, u.z), swiglu_one(g.w, u.w));
          const u32 n = nt * (GEMM_BN / 2) + 32 * c + 8 * g4 + 4 * kg;
          if ((PACK == 0 || out) && token < m && n < out_dim) {
            float* dst = out + (size_t)token * out_dim + n;
            if (vec && n + 4 <= out_dim) {
              *reinterpret_cast<float4*>(dst) = o;
            } else {
              const float ov[4] = {o.x, o.y, o.z, o.w};
              for (u32 e = 0; e < 4 && n + e < out_dim; e++) dst[e] = ov[e];
            }
          }
          if constexpr (PACK != 0) {
            // the eight consecutive rows n8 .. n8 + 7 of the lane pair are k values of the next GEMM: super-block n8 / 256,
            // cell (k-step, k-group) by the inverse of gemm_k_element | gemm_k_element_q6k (as in pack_x_core), all
            // uniform over the wavefront; the absent tokens of the last tile are zeros, as the pack kernel writes them
            const u32 n8 = nt * (GEMM_BN / 2) + 32 * c + 8 * g4;
            if (n8 < out_dim) {
              const u32 kb = n8 >> 8, k = n8 & 255u;
              u32 ks, kgr;
              if (PACK == 14) {
                ks = 8 * (k >> 7) + 2 * ((k >> 5) & 3) + ((k >> 3) & 1);
                kgr = (k >> 4) & 1;
              } else {
                const u32 g6 = k >> 6;
                ks = 8 * (g6 >> 1) + 4 * ((k >> 4) & 1) + 2 * ((k >> 5) & 1) + ((k >> 3) & 1);
                kgr = g6 & 1;
              }
              const float4 z = token < m ? o : make_float4(0.f, 0.f, 0.f, 0.f);
              const __half2 p0 = __floats2half2_rn(z.x, z.z), p1 = __floats2half2_rn(z.y, z.w);   // slot order 0,2,1,3
              uint2 q;
              q.x = *reinterpret_cast<const u32*>(&p0);
              q.y = *reinterpret_cast<const u32*>(&p1);
              uint2* cell = xq + (((size_t)mt * (out_dim >> 8) + kb) * 4096 + (ks * 2 + kgr) * 128 + 32 * (RH * KH + rr) + j) * 2 + kg;
              *cell = q;
              // (64 tokens: the upper half of the token tile is nobody's; it gets the zeros the pack kernel writes there)
              if constexpr (MT == 2) cell[2 * 64] = make_uint2(0u, 0u);
            }
          }
        }
    }
  };
  if (nh == 0) give(std::integral_constant<int, 0>{});
  else give(std::integral_constant<int, 1>{});
  __syncthreads();
  if (nh == 0) finish(std::integral_constant<int, 0>{});
  else finish(std::integral_constant<int, 1>{});
}

// Up to GEMM_MANY_MAX matrices of one type and row length against the same packed activations, as one launch: the tiles of
// the launch are the tiles of matrix 0, then of matrix 1, ... (tile_end[i]: tiles of matrices 0..i), every matrix with its
// own output [m][out_dim[i]]. A workgroup looks its matrix up once; everything behind that is the single-matrix kernel.
#define GEMM_MANY_MAX 6
struct GemmManyArgs {
  const uint8_t* w[GEMM_MANY_MAX];
  float* out[GEMM_MANY_MAX];
  u32 out_dim[GEMM_MANY_MAX];
  u32 tile_end[GEMM_MANY_MAX];
  u32 count;
};

// raw bytes of one group of one super-block of one weight row, as a lane sees them
template <bool Q5>
struct GemmRawT {
  uint4 hdr, qa, qb;
};
template <>
struct GemmRawT<true> {   // Q5_K: plus the 32 bytes of fifth bits (bit 2g + hi of qh[l] belongs to value 64g + 32hi + l)
  uint4 hdr, qa, qb, qh0, qh1;
};

// Q5 = false: Q4_K (144-byte super-blocks, everything through gemm_wbuf); true: Q5_K (176 bytes; same nibbles, groups and
// x order, one more bit per value).
// SWIGLU (Q4_K): rows 0..95 of the tile are rows [96 nt, 96 nt + 96) of `w` (gate), rows 96..191 the same rows of `w_b` (up);
// the epilogue stores silu(gate) * up. No k split and no bias then.
// NT: tiles of 32 weight rows per wavefront - 3 (workgroup tile 128 tokens x 192 rows) or 2 (128 x 128, for launches whose
// 192-row tiles, times the k split, leave compute units idle: q4_k_gemm_n128_f16, q5_k_gemm_n128_f16).
// MT: tiles of 32 tokens - 4 (128 tokens) or 2: launches of up to 64 tokens, where the upper half of a 128-token tile would
// be MFMAs on padding and copies of nothing (<type>_gemm_m64[_n128]_f16; the packed x is the same, its first 64 tokens are used).
// PACK (SWIGLU only): the epilogue also writes the products as the packed fp16 activations of the next GEMM, to `xq`.
template <bool Q5, bool SWIGLU = false, int NT = 3, int MT = 4, int PACK = 0>
__device__ __forceinline__ void gemm_k45_core(const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim,
                                              u32 out_dim, u32 m, u32 bias_stride = 0, const uint8_t* w_b = nullptr,
                                              uint4* xq = nullptr, const GemmManyArgs* many = nullptr) {
  static_assert(PACK == 0 || SWIGLU, "only the gate | up kernel writes packed activations");
  static_assert(!(Q5 && SWIGLU), "the gate | up kernel is built for Q4_K");
  static_assert(NT == 3 || (NT == 2 && !SWIGLU), "tile heights");
  static_assert(MT == 4 || MT == 2, "tokens per tile");
  constexpr int NX = 4 * MT;              // copies of x per thread and super-block: 32 chunks of 128 tokens x 16 bytes, or of the first 64 tokens of each
  constexpr u32 BN = 64 * NT;             // weight rows of the workgroup tile
  constexpr u32 BS = Q5 ? 176 : 144;      // bytes of a super-block
  constexpr u32 PPR = Q5 ? 10 : 9;        // 16-byte pieces of a row that go through LDS
  constexpr int NCOPY = (int)((BN * PPR + 255) / 256);   // copies of 64 pieces a wavefront issues per super-block (192 rows: 7, Q5_K 8)
  uint4* const wbuf = Q5 ? gemm_wbuf5 : gemm_wbuf;
  // (no __restrict__ on w / xp: loads the compiler knows to be invariant are rematerialised next to
  // their use, which would undo the prefetch distance set up below)
  const u32 tid = threadIdx.x, lane = tid & 63;
  const u32 wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const u32 nh = wave & 1, kh = wave >> 1;
  const u32 j = lane & 31, kg = lane >> 5;
  const u32 g = 2 * kh + kg;
  // k split: workgroups of blockIdx.y = s take super-blocks [kb0, kb0 + nkb) of the nkb_all a row has and write their
  // sums to the s-th [m][out_dim] plane behind `out` (the host passes the partial planes and no bias, then sums them)
  const u32 nkb_all = in_dim >> 8;
  const u32 kb0 = blockIdx.y * nkb_all / gridDim.y, nkb = (blockIdx.y + 1) * nkb_all / gridDim.y - kb0;
  out += (size_t)blockIdx.y * m * out_dim;
  constexpr u32 TILE_ROWS = SWIGLU ? BN / 2 : BN;   // rows of a matrix a tile covers
  const u32 mtiles = (m + GEMM_BM - 1) / GEMM_BM;
  const u32 ntiles = many ? many->tile_end[many->count - 1] : (out_dim + TILE_ROWS - 1) / TILE_ROWS;
  // Workgroup -> tile, XCD-aware (gemm_tile_of, gemv_config.h): the 32 workgroups that run side by side on an XCD take
  // a block of neighbouring tiles, so that its L2 fills with a weight tile once for several token tiles and with an x
  // tile once for several weight tiles. The grid is rounded up to whole blocks; the surplus workgroups leave.
  u32 mt, nt;
  if (!gemm_tile_of(blockIdx.x, mtiles, ntiles, &mt, &nt)) return;
  if (many) {
    // a list of matrices: the tile's matrix (uniform over the workgroup), its weights, output and row count
    u32 i = 0, first = 0;
    while (i + 1 < many->count && nt >= many->tile_end[i]) first = many->tile_end[i++];
    nt -= first;
    w = many->w[i];
    out = many->out[i];
    out_dim = many->out_dim[i];
  }
  const size_t row_bytes = (size_t)nkb_all * BS;
  const u32 sh = 16u * kg;
  // Unpacking the 6-bit (scale, min) pairs takes one of two forms by g >= 2, i.e. by kh, which is the same for a whole
  // wavefront: written as a select it becomes a scalar branch that cuts the last k-step's scheduling region into
  // pieces, so the two forms are folded into one through masks the compiler cannot see through.
  u32 um = kh ? 0xFFFFFFFFu : 0u, mA = kh ? 0x0F0Fu : 0x3F3Fu, mB = kh ? 0x3030u : 0u, shM = kh ? 4u : 0u;
  um = __builtin_amdgcn_readfirstlane(um);
  mA = __builtin_amdgcn_readfirstlane(mA);
  mB = __builtin_amdgcn_readfirstlane(mB);
  shM = __builtin_amdgcn_readfirstlane(shM);
  asm volatile("" : "+s"(um), "+s"(mA), "+s"(mB), "+s"(shM));
  // the fp16 offsets live in registers so that (q & mask) | magic is one v_and_or_b32 (two literals would be two instructions)
  u32 magic_lo = 0x64006400u, magic_hi = 0x54005400u;
  asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));

  // Weight copies: piece p = 64 i + lane of the tile's super-block, i = wave, wave + 4, ... (27 copies of 64 pieces per
  // workgroup and super-block; every wavefront issues 7, the 28th repeats the last piece into spare LDS so that no
  // copy is conditional). Piece p is bytes [16 (p % 9), +16) of row p / 9.
  const u32 tile_row0 = min(nt * TILE_ROWS, out_dim - 1);
  const uint8_t* wbase = w + (size_t)tile_row0 * row_bytes + (size_t)kb0 * BS;   // uniform
  u32 woff[NCOPY];
  const uint8_t* wsrc[SWIGLU ? NCOPY : 1];   // gate | up: the two matrices are separate allocations, a piece has a full address
#pragma unroll
  for (int i = 0; i < NCOPY; i++) {
    const u32 p = min((4u * i + wave) * 64u + lane, BN * PPR - 1u);
    const u32 r = p / PPR, part = p - PPR * r;
    if constexpr (SWIGLU) {
      const u32 row = min(nt * TILE_ROWS + (r < TILE_ROWS ? r : r - TILE_ROWS), out_dim - 1);
      wsrc[i] = (r < TILE_ROWS ? w : w_b) + (size_t)row * row_bytes + 16u * part;
      woff[i] = 0;
    } else {
      woff[i] = (min(nt * BN + r, out_dim - 1) - tile_row0) * (u32)row_bytes + 16u * part + (Q5 ? 16u : 0u);
    }
  }
  // where this lane finds the raw bytes of its three rows in gemm_wbuf (in uint4 units): header, then the 32 bytes of
  // its group
  u32 wrow[NT];
#pragma unroll
  for (int c = 0; c < NT; c++) wrow[c] = (nh * (32 * NT) + 32 * c + j) * PPR;
  // Q5_K: where this lane's three rows start relative to wbase (their headers are read from there)
  u32 hoff[NT];
#pragma unroll
  for (int c = 0; c < NT; c++) hoff[c] = (min(nt * BN + nh * (32 * NT) + 32 * c + j, out_dim - 1) - tile_row0) * (u32)row_bytes;
  const uint4* xtile = xp + ((size_t)mt * nkb_all + kb0) * 4096;

  float16_t acc[MT][NT];
#pragma unroll
  for (int r = 0; r < MT; r++)
#pragma unroll
    for (int c = 0; c < NT; c++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[r][c][v] = 0.0f;

  // copy i of a super-block's x tile: 128 tokens - 4 KiB of the image per instruction and workgroup; 64 tokens - the
  // wavefront takes the first KiB (tokens 0..63) of the 2 KiB chunk 4 i + wave
  auto x_copy = [&](const uint4* src, uint4* dst, int i) {
    if constexpr (MT == 4)
      __builtin_amdgcn_global_load_lds((gbl_void*)(src + 256 * i + tid), (lds_void*)(dst + 256 * i + wave * 64), 16, 0, 0);
    else
      __builtin_amdgcn_global_load_lds((gbl_void*)(src + (4 * i + wave) * 128 + lane), (lds_void*)(dst + (4 * i + wave) * 128), 16, 0, 0);
  };
  auto copy_w = [&](u32 kb, int i) {   // copy i of this wavefront for super-block kb
    if constexpr (SWIGLU)
      __builtin_amdgcn_global_load_lds((gbl_void*)(wsrc[i] + (size_t)kb * BS), (lds_void*)(wbuf + (4 * i + wave) * 64), 16, 0, 0);
    else
      __builtin_amdgcn_global_load_lds((gbl_void*)(wbase + (size_t)kb * BS + woff[i]),
                                       (lds_void*)(wbuf + (4 * i + wave) * 64), 16, 0, 0);
  };
  uint4 nhdr[NT];   // Q5_K: headers of the super-block being copied
  auto load_hdr = [&](u32 kb, int c) {
    if constexpr (Q5) nhdr[c] = ld16(wbase + (size_t)kb * BS + hoff[c]);
  };

  // Stage super-block 0 of x and of the weights. The main loop below takes super-blocks in pairs with fixed x buffers
  // (0 then 1) and no branch in its body; with an odd number of super-blocks the first one is taken alone out of
  // buffer 1.
  const bool odd = nkb & 1;
#pragma unroll
  for (int i = 0; i < NCOPY; i++) copy_w(0, i);
#pragma unroll
  for (int c = 0; c < NT; c++) load_hdr(0, c);
  if (odd) {
#pragma unroll
    for (int i = 0; i < NX; i++) x_copy(xtile, gemm_xbuf1, i);
  } else {
#pragma unroll
    for (int i = 0; i < NX; i++) x_copy(xtile, gemm_xbuf0, i);
  }
  __syncthreads();

  // State that lives across super-blocks: the raw bytes and the decoded (scale, -min) pairs of the current one, and
  // the two operand sets of the k-step pipeline.
  GemmRawT<Q5> cur[NT];
  u32 S[NT][4];
  uint4 A[2][MT];
  half8_t B[2][NT];
  // The raw bytes of a super-block, out of gemm_wbuf into the registers of the lanes that decode them.
  auto take_raw = [&]() {
#pragma unroll
    for (int c = 0; c < NT; c++) {
      if constexpr (Q5) {
        cur[c].hdr = nhdr[c];
        cur[c].qh0 = wbuf[wrow[c]];
        cur[c].qh1 = wbuf[wrow[c] + 1];
        cur[c].qa = wbuf[wrow[c] + 2 + 2 * g];
        cur[c].qb = wbuf[wrow[c] + 3 + 2 * g];
      } else {
        cur[c].hdr = wbuf[wrow[c]];
        cur[c].qa = wbuf[wrow[c] + 1 + 2 * g];
        cur[c].qb = wbuf[wrow[c] + 2 + 2 * g];
      }
    }
  };
  // (scale, -min) of sub-blocks 2g (low nibbles) and 2g+1 (high nibbles) as duplicated half2
  auto decode_scales = [&]() {
#pragma unroll
    for (int c = 0; c < NT; c++) {
      const float d = h2f(cur[c].hdr.x), dm = h2f(cur[c].hdr.x >> 16);
      const u32 a0 = cur[c].hdr.y >> sh, a1 = cur[c].hdr.z >> sh, a2 = cur[c].hdr.w >> sh;
      // kh = 0: a0 & 0x3F3F, a1 & 0x3F3F; kh = 1: (a2 & 0x0F0F) | ((a0 >> 2) & 0x3030), ((a2 >> 4) & 0x0F0F) | ((a1 >> 2) & 0x3030)
      const u32 aS = (um & a2) | (~um & a0), aM = (um & a2) | (~um & a1);
      const u32 scp = (aS & mA) | ((a0 >> 2) & mB);
      const u32 mp = ((aM >> shM) & mA) | ((a1 >> 2) & mB);
      S[c][0] = h2_dup(d * ubyte_f<0>(scp));
      S[c][1] = h2_dup(-(dm * ubyte_f<0>(mp)));
      S[c][2] = h2_dup(d * ubyte_f<1>(scp));
      S[c][3] = h2_dup(-(dm * ubyte_f<1>(mp)));
    }
  };
  auto build_b = [&](half8_t (&Bd)[NT], int t) {
    const int h = t >> 2, op = t & 3, hi = op >> 1;
#pragma unroll
    for (int c = 0; c < NT; c++) {
      const uint4 Q = h ? cur[c].qb : cur[c].qa;
      const u32 qa = (op & 1) ? Q.z : Q.x, qb = (op & 1) ? Q.w : Q.y;
      const u32 mask = hi ? 0x00F000F0u : 0x000F000Fu;
      const u32 magic = hi ? magic_hi : magic_lo;           // 64 + n (n sits 4 bits up) : 1024 + n
      const u32 off = hi ? 0xD400D400u : 0xE400E400u;       // half2(-64) : half2(-1024)
      const u32 sc = S[c][2 * hi], nm = S[c][2 * hi + 1];
      uint4 bw;
      if constexpr (Q5) {
        // the fifth bit is worth 16: bit 4 beside a low nibble (1024 + q, one unit per mantissa step), bit 8 beside a
        // high nibble (64 + q with the nibble 4 bits up, 1/16 per step)
        const uint4 QH = h ? cur[c].qh1 : cur[c].qh0;
        const u32 ha = ((op & 1) ? QH.z : QH.x) >> (2 * g + hi), hb = ((op & 1) ? QH.w : QH.y) >> (2 * g + hi);
        const int up = hi ? 8 : 4;
        bw.x = h2_fma_off((qa & mask) | magic | ((ha & 0x00010001u) << up), off, sc, nm);
        bw.y = h2_fma_off(((qa >> 8) & mask) | magic | (((ha >> 8) & 0x00010001u) << up), off, sc, nm);
        bw.z = h2_fma_off((qb & mask) | magic | ((hb & 0x00010001u) << up), off, sc, nm);
        bw.w = h2_fma_off(((qb >> 8) & mask) | magic | (((hb >> 8) & 0x00010001u) << up), off, sc, nm);
      } else {
        bw.x = h2_fma_off((qa & mask) | magic, off, sc, nm);
        bw.y = h2_fma_off(((qa >> 8) & mask) | magic, off, sc, nm);
        bw.z = h2_fma_off((qb & mask) | magic, off, sc, nm);
        bw.w = h2_fma_off(((qb >> 8) & mask) | magic, off, sc, nm);
      }
      Bd[c] = *reinterpret_cast<const half8_t*>(&bw);
    }
  };
  // A operands of k-step t of the wavefront (k-steps 8*kh .. 8*kh+7 of the tile; 32 lanes read 512 contiguous bytes)
  auto read_a = [&](uint4 (&Ad)[MT], const uint4* xbuf, int t) {
    const uint4* arow = xbuf + (16 * kh + kg) * 128 + j;
#pragma unroll
    for (int r = 0; r < MT; r++) Ad[r] = arow[t * 256 + r * 32];
  };

  // Operands of k-step 0 of the first super-block; after that every super-block prepares the first k-step of the
  // next one in the shadow of its own last k-step.
  take_raw();
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();   // gemm_wbuf is free for the copies of the next super-block
  asm volatile("" ::: "memory");
  decode_scales();
  read_a(A[0], odd ? gemm_xbuf1 : gemm_xbuf0, 0);
  build_b(B[0], 0);

  auto iteration = [&](u32 kb, const uint4* xcur, uint4* xnxt) {
    const u32 kn = min(kb + 1, nkb - 1);   // the last iteration re-reads its own tile; the copy is not used
    const uint4* xnext = xtile + (size_t)kn * 4096;   // uniform
    auto copy_x = [&](int i) { x_copy(xnext, xnxt, i); };
    // software pipeline over the wavefront's eight k-steps: while the MFMAs of step t run, the A operands
    // of step t+1 are read from LDS and its B operands are built
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const int p = t & 1;
      // Copies for the next super-block, a few per k-step rather than all up front: a wavefront issues in order and
      // a vector memory instruction costs it some 50 clocks, so 23 of them in a row stall the (only) wavefront of the
      // SIMD with nothing to overlap. All of them are out by k-step 5; they are waited for behind k-step 6.
      // (copy 2 t and 2 t + 1 in k-steps 0..2, the seventh in k-step 3, the eighth in k-step 4, as far as the tile has them)
      if (t < 3) {
        if (2 * t < NCOPY) copy_w(kn, 2 * t);
        if (2 * t + 1 < NCOPY) copy_w(kn, 2 * t + 1);
        if (t < NT) load_hdr(kn, t);
      }
      if (t == 3 && NCOPY > 6) copy_w(kn, 6);
      if (t == 4 && NCOPY > 7) copy_w(kn, 7);
      if (t < 6) {
#pragma unroll
        for (int i = (t < 2 ? 2 * t : 3 * t - 2); i < (t < 2 ? 2 * t + 2 : 3 * t + 1); i++)
          if (i < NX) copy_x(i);   // (64 tokens: eight copies, out by k-step 3)
      }
      if (t < 7) {
        read_a(A[p ^ 1], xcur, t + 1);
        build_b(B[p ^ 1], t + 1);
      } else {
        // last k-step: the next super-block is in LDS (wait and barrier behind k-step 6); its raw bytes, scales and
        // the operands of its first k-step are prepared while this step's MFMAs run (the current raw bytes and
        // scales are no longer needed: the operands of this step were built in the previous one)
        take_raw();
        read_a(A[0], xnxt, 0);
        decode_scales();
        build_b(B[0], 0);
      }
#pragma unroll
      for (int r = 0; r < MT; r++) {
        const half8_t Ar = *reinterpret_cast<const half8_t*>(&A[p][r]);
#pragma unroll
        for (int c = 0; c < NT; c++) acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(B[p][c], Ar, acc[r][c], 0, 0, 0);
      }
      // Scheduling window = one k-step. Left alone the scheduler emits the twelve MFMAs back to back and the
      // operand preparation of the next step behind them, so the matrix pipe and the vector ALU take turns;
      // the group barriers below ask for the interleaving instead: the loads first, then one MFMA followed
      // by a few vector instructions, twelve times (an MFMA occupies the matrix pipe for 32 clocks, five
      // vector instructions issue in 20 to 35).
      // keep the operands built above inside this window (otherwise they sink next to their first use,
      // behind the window's MFMAs)
#pragma unroll
      for (int c = 0; c < NT; c++) asm volatile("" : "+v"(B[p ^ 1][c]));
      if (t < 7) {
        __builtin_amdgcn_sched_group_barrier(0x020, 8, 0);   // VMEM reads (LDS-direct copies) of this step
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);   // LDS reads: A operands of the next step
#pragma unroll
        for (int i = 0; i < MT * NT; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);            // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x002, Q5 ? 8 : 5, 0);   // five VALU (eight with the fifth bits)
        }
      } else {
        __builtin_amdgcn_sched_group_barrier(0x100, Q5 ? 16 : 13, 0);  // LDS reads: raw bytes and first A operands of the next super-block
#pragma unroll
        for (int i = 0; i < NT; i++) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // a few MFMAs while they arrive
#pragma unroll
        for (int i = 0; i < (MT - 1) * NT; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 16, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if (t == 6) {
        // everything this wavefront requested for the next super-block has to be there, then everybody meets
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // End of the iteration: every wavefront has taken the next raw bytes out of gemm_wbuf and is done reading xcur;
    // both are free for the copies of the super-block after next.
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  if (odd) iteration(0, gemm_xbuf1, gemm_xbuf0);
  for (u32 kb = odd; kb < nkb; kb += 2) {
    iteration(kb, gemm_xbuf0, gemm_xbuf1);
    iteration(kb + 1, gemm_xbuf1, gemm_xbuf0);
  }
  __syncthreads();   // drains the last (unused) prefetches before the buffers are reused below

  if constexpr (SWIGLU) {
    if (kh == 0) gemm_epilogue_swiglu_half<0, PACK, MT>(acc, out, out_dim, m, mt, nt, nh, j, kg, lane, reinterpret_cast<uint2*>(xq));
    else gemm_epilogue_swiglu_half<1, PACK, MT>(acc, out, out_dim, m, mt, nt, nh, j, kg, lane, reinterpret_cast<uint2*>(xq));
  } else {
    gemm_epilogue<NT, MT>(acc, bias, out, out_dim, m, mt, nt, nh, kh, j, kg, tid, bias_stride);
  }
}

extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q4_k_gemm_f16(
    const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim, u32 m, u32 bias_stride) {
  gemm_k45_core<false>(w, xp, bias, out, in_dim, out_dim, m, bias_stride);
}
// the same with a workgroup tile of 128 tokens x 128 rows; grid from gemm_grid_x(ceil(m/128), ceil(out_dim/128))
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q4_k_gemm_n128_f16(
    const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim, u32 m, u32 bias_stride) {
  gemm_k45_core<false, false, 2>(w, xp, bias, out, in_dim, out_dim, m, bias_stride);
}
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q5_k_gemm_n128_f16(
    const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim, u32 m, u32 bias_stride) {
  gemm_k45_core<true, false, 2>(w, xp, bias, out, in_dim, out_dim, m, bias_stride);
}
// up to 64 tokens: the first 64 tokens of the (one) token tile only; grid from gemm_grid_x(1, ceil(out_dim / 192 | 128))
#define GEMM_K45_M64_ENTRY(NAME, Q5, NT)                                                                                  \
  extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void NAME(                       \
      const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim, u32 m, u32 bias_stride) { \
    gemm_k45_core<Q5, false, NT, 2>(w, xp, bias, out, in_dim, out_dim, m, bias_stride);                                   \
  }
GEMM_K45_M64_ENTRY(q4_k_gemm_m64_f16, false, 3)
GEMM_K45_M64_ENTRY(q4_k_gemm_m64_n128_f16, false, 2)
GEMM_K45_M64_ENTRY(q5_k_gemm_m64_f16, true, 3)
GEMM_K45_M64_ENTRY(q5_k_gemm_m64_n128_f16, true, 2)
// Q5_K: x is packed by pack_x_f16_q4k (the values of a super-block sit where the Q4_K ones do).
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q5_k_gemm_f16(
    const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim, u32 m, u32 bias_stride) {
  gemm_k45_core<true>(w, xp, bias, out, in_dim, out_dim, m, bias_stride);
}
// Lists of matrices (q | k | v | gate | up of a prefill layer against one packed x): (list: GemmManyArgs by value, xp, in_dim, m),
// block 256, grid gemm_grid_x(ceil(m/128), sum of the matrices' tiles), no k split, no bias; 192- and 128-row tiles, 128 and
// up to 64 tokens, as the single-matrix kernels of the same suffixes, and every output bit for bit theirs.
#define GEMM_K45_MANY_ENTRY(NAME, Q5, NT, MT)                                                                                \
  extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void NAME(                       \
      const GemmManyArgs list, const uint4* xp, u32 in_dim, u32 m) {                                                         \
    gemm_k45_core<Q5, false, NT, MT>(nullptr, xp, nullptr, nullptr, in_dim, 0, m, 0, nullptr, nullptr, &list);              \
  }
GEMM_K45_MANY_ENTRY(q4_k_gemm_many_f16, false, 3, 4)
GEMM_K45_MANY_ENTRY(q4_k_gemm_many_n128_f16, false, 2, 4)
GEMM_K45_MANY_ENTRY(q4_k_gemm_many_m64_f16, false, 3, 2)
GEMM_K45_MANY_ENTRY(q4_k_gemm_many_m64_n128_f16, false, 2, 2)
GEMM_K45_MANY_ENTRY(q5_k_gemm_many_f16, true, 3, 4)
GEMM_K45_MANY_ENTRY(q5_k_gemm_many_n128_f16, true, 2, 4)
GEMM_K45_MANY_ENTRY(q5_k_gemm_many_m64_f16, true, 3, 2)
GEMM_K45_MANY_ENTRY(q5_k_gemm_many_m64_n128_f16, true, 2, 2)

// gate | up of a feed-forward block against one packed x, silu(gate) * up stored: no gate and up matrices in memory.
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q4_k_gemm_swiglu_f16(
    const uint8_t* w_gate, const uint8_t* w_up, const uint4* xp, float* out, u32 in_dim, u32 out_dim, u32 m) {
  gemm_k45_core<false, true>(w_gate, xp, nullptr, out, in_dim, out_dim, m, 0, w_up);
}
// The same with silu(gate) * up also (out null: only) written as the packed fp16 activations of the GEMM that follows, in
// the order of its weight type - q4k: Q4_K and Q5_K, q6k: Q6_K; (w_gate, w_up, xp, out | null, xq, in_dim, out_dim, m),
// out_dim a multiple of 256, xq as large as pack_x_f16_* needs for [m][out_dim].
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q4_k_gemm_swiglu_pack_q4k_f16(
    const uint8_t* w_gate, const uint8_t* w_up, const uint4* xp, float* out, uint4* xq, u32 in_dim, u32 out_dim, u32 m) {
  gemm_k45_core<false, true, 3, 4, 12>(w_gate, xp, nullptr, out, in_dim, out_dim, m, 0, w_up, xq);
}
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q4_k_gemm_swiglu_pack_q6k_f16(
    const uint8_t* w_gate, const uint8_t* w_up, const uint4* xp, float* out, uint4* xq, u32 in_dim, u32 out_dim, u32 m) {
  gemm_k45_core<false, true, 3, 4, 14>(w_gate, xp, nullptr, out, in_dim, out_dim, m, 0, w_up, xq);
}
// the three for up to 64 tokens (two tiles of 32 tokens per wavefront, as <type>_gemm_m64_f16)
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q4_k_gemm_swiglu_m64_f16(
    const uint8_t* w_gate, const uint8_t* w_up, const uint4* xp, float* out, u32 in_dim, u32 out_dim, u32 m) {
  gemm_k45_core<false, true, 3, 2>(w_gate, xp, nullptr, out, in_dim, out_dim, m, 0, w_up);
}
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q4_k_gemm_swiglu_pack_q4k_m64_f16(
    const uint8_t* w_gate, const uint8_t* w_up, const uint4* xp, float* out, uint4* xq, u32 in_dim, u32 out_dim, u32 m) {
  gemm_k45_core<false, true, 3, 2, 12>(w_gate, xp, nullptr, out, in_dim, out_dim, m, 0, w_up, xq);
}
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q4_k_gemm_swiglu_pack_q6k_m64_f16(
    const uint8_t* w_gate, const uint8_t* w_up, const uint4* xp, float* out, uint4* xq, u32 in_dim, u32 out_dim, u32 m) {
  gemm_k45_core<false, true, 3, 2, 14>(w_gate, xp, nullptr, out, in_dim, out_dim, m, 0, w_up, xq);
}

// Sum of the k-split planes: out[i] = (bias ? bias[bias_stride ? i : i % out_dim] : 0) + partials[0][i] + partials[1][i] + ... in that order
// (the result does not depend on which workgroup finished first). block 256, grid ceil(total / 1024); 4 elements per lane.
// (bias and out are not __restrict__: a residual may be `out` itself; a thread reads only the elements it writes)
extern "C" __global__ __launch_bounds__(256) void gemm_sum_splits_f32(const float* __restrict__ partials, const float* bias,
                                                                       float* out, u32 total, u32 out_dim, u32 splits, u32 bias_stride) {
  const u32 i = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= total) return;
  if (i + 4 <= total && (total & 3u) == 0) {
    float4 a = *reinterpret_cast<const float4*>(partials + i);
    for (u32 s = 1; s < splits; s++) {
      const float4 b = *reinterpret_cast<const float4*>(partials + (size_t)s * total + i);
      a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
    }
    if (bias) {
      if (bias_stride) {   // a [m][out_dim] residual: element for element
        a.x += bias[i]; a.y += bias[i + 1]; a.z += bias[i + 2]; a.w += bias[i + 3];
      } else {
        a.x += bias[i % out_dim]; a.y += bias[(i + 1) % out_dim]; a.z += bias[(i + 2) % out_dim]; a.w += bias[(i + 3) % out_dim];
      }
    }
    *reinterpret_cast<float4*>(out + i) = a;
  } else {
    for (u32 e = i; e < total && e < i + 4; e++) {
      float a = partials[e];
      for (u32 s = 1; s < splits; s++) a += partials[(size_t)s * total + e];
      out[e] = a + (bias ? bias[bias_stride ? e : e % out_dim] : 0.0f);
    }
  }
}
