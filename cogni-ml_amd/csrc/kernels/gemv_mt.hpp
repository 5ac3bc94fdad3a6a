// Decode GEMV for 2..8 tokens in ONE pass over the weights, Q4_K, Q5_K, Q6_K and Q8_0, on the matrix cores:
//   out_i[m][o] = (residual[m][o] +) sum_j x[m][j] * deq(W_i[o][j])      for up to three matrices W_i of one in_dim.
//
// Kernels.
//   pack_x_mt_q4k_f16 | pack_x_mt_q6k_f16 (x, image, tokens, in_dim)            block 256, grid 2 * gemv_mt_padded_sb(in_dim)
//     turn the activations x[tokens][in_dim] (fp32) into the image the GEMV kernel of that weight type reads: per
//     super-block of 256 values the matrix-core operands of its instructions, laid out lane by lane, followed by the
//     scale and the sub-block sums of every (token, super-block). Written once per activation block, whatever the number
//     of matrices that block then meets (q | k | v | gate | up of a decoder layer share one).
//   q4_k_gemv_mt_f32 | q5_k_gemv_mt_f32 | q6_k_gemv_mt_f32 | q8_0_gemv_mt_f32 (w0, w1, w2, image, residual, out0, out1, out2, in_dim, rows0, rows1, rows2, tokens)
//     (Q5_K and Q8_0 read the image pack_x_mt_q4k_f16 writes)
//     block 512 (8 wavefronts), grid and dynamic shared memory from gemv_config.h (gemv_mt_grid, gemv_mt_lds_bytes).
//   pack_x_mt16_q4k_f16 | pack_x_mt16_q6k_f16 and q4_k_gemv_mt16_f32 | q5_k_ | q6_k_ | q8_0_gemv_mt16_f32 (same parameters)
//     the same for up to sixteen tokens, each as ONE binary16 term (x rounded to half: the precision class of the prefill GEMM,
//     which these kernels stand in for between 9 and 16 tokens); grid 4 * gemv_mt_padded_sb(in_dim) for the pack, shared memory
//     gemv_mt_lds_bytes + GEMV_MT_X16_LDS_EXTRA for the GEMV.
//     rows1 / rows2 may be 0 (then w1 / w2 / out1 / out2 are not read); residual (may be null) belongs to the first
//     matrix. Row counts of all but the last matrix present must be multiples of 16. in_dim must be a multiple of 256
//     up to 12288 (8 k-slices of 1..6 super-blocks; see "Rows that are not a multiple of 2048 values" below). out_i rows at stride rows_i (the reference's multi-token kernel
//     contract, src/ml/cuda/kernels/q4k_gemv_probe.ptx:437-768, q5k_gemv_probe.ptx:237 and q6k_gemv_probe.ptx:977: x rows at stride in_dim, outs
//     at stride out_dim; these kernels handle eight tokens where those handle four).
//   q4_k_gemv_mt_swiglu_f32 (w_gate, w_up, image, out, in_dim, out_dim, tokens)
//
// Arithmetic. The matrix cores multiply 16 activation rows x K values by K x 16 weight rows. The weights stay exact: a
// masked pair of codes read as two binary16 numbers is code * 2^-24 (code * 2^-20 for codes left four bits up), the
// matrix cores honour subnormals, accumulation is fp32. The activations are fed as two binary16 terms, x * 2^e = hi + lo
// (22 bits; e per token and super-block, so any fp32 range fits), which makes the 16 rows (token 0..7) x (hi, lo). One
// instruction covers exactly one sub-block - Q4_K and Q5_K: v_mfma_f32_16x16x32_f16 on a 32-weight sub-block (a lane supplies
// the low or the high nibbles of 8 bytes, Q5_K with the fifth bit of each from qh), Q6_K: v_mfma_f32_16x16x16_f16 on a 16-weight sub-block (4 bytes) - so the integer
// scale of that sub-block is applied to the instruction's result, and the terms that do not depend on the codes (Q4_K, Q5_K:
// dmin * m * sum(x), Q6_K: 32 * d * sc * sum(x)) come from the sub-block sums of the image. A result lane holds two
// tokens x (hi, lo) of one weight row, the row whose header the same lane reads: the scales never change lanes.
//
// Work split. The eight wavefronts of a workgroup are eight k-slices (super-blocks wave, wave + 8, ...); a wavefront
// takes T tiles of 16 rows at a time. Nobody waits for anybody until the k-slices' sums meet in LDS, where they are added
// in a fixed order (bit-reproducible). A workgroup walks the row groups blockIdx.x, blockIdx.x + gridDim.x, ...
// With one or two super-blocks per k-slice the activation operands stay in registers for the whole kernel and the next
// row group's weights are requested while the current one is worked on; with three to six (rows of 6144..12288 values)
// a wavefront carries one tile and streams the operands of its super-blocks through two register sets.
//
// Rows that are not a multiple of 2048 values. The eight k-slices take ceil(nsb / 8) super-blocks each, as if the row had
// nsbp = 8 * ceil(nsb / 8) of them. The image has nsbp super-blocks, the ones past the row's end all zeros (operands, sums
// and the tokens' scales), and a k-slice whose super-block does not exist copies the row's last block in its place: a
// finite weight times zero, so such a unit adds exactly 0 to every sum and every wavefront issues the same loads and
// waits as for a full row. (A 1024-value row keeps four of the eight wavefronts busy with zeros: still one pass over the
// weights where the per-token-group kernels take two from five tokens on.)
//
// Memory. A tile's share of a super-block is 16 rows x one block at a stride of a whole row: fetched by the lanes that
// use it (a few bytes each, 16 rows per instruction) it comes in at a third of the rate of a plain stream. So the weights
// are copied global -> LDS 16 bytes per lane with the lanes along the rows (lane p of a unit takes piece p % P of row
// p / P), which lands them in a wavefront-private slot as [row][P x 16 bytes], and each lane then picks its bytes out of
// LDS. Every copy of a row group is issued up front behind the activation operands; all loads are written in assembly and
// counted by hand (s_waitcnt vmcnt), unit after unit as they land.
#pragma once
#include <type_traits>
#include "common.hpp"
#include "gemv_config.h"

// Register sets the streamed activation operands go through (rows above 4096 values). Three measure 2-4 % slower than two
// at every such shape (Q6_K 4096x12288 15.66 -> 16.00 us, Q4_K 11.84 -> 12.04): the third set's loads stand in front of
// weight copies.
#ifndef GEMV_MT_STREAM_SETS
#define GEMV_MT_STREAM_SETS 2
#endif

// Which super-blocks a k-slice takes: wave, wave + 8, ... (0) or the SBW consecutive ones from wave * SBW on (1), where a
// row contributes SBW blocks in one piece to a wavefront's copies instead of one block each. Measured with 1: 2-5 % slower
// at every shape (Q4_K 12288x4096 M=8 9.31 -> 9.81 us, 5120x5120 11.0 -> 11.3, Q6_K 4096x12288 15.6 -> 15.9).
#ifndef GEMV_MT_CONTIGUOUS_SLICES
#define GEMV_MT_CONTIGUOUS_SLICES 0
#endif

typedef _Float16 mt_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 mt_half4 __attribute__((ext_vector_type(4)));
typedef float mt_float4 __attribute__((ext_vector_type(4)));
typedef u32 mt_u32x4 __attribute__((ext_vector_type(4)));
typedef u32 mt_u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void mt_lds_void;

#define MT_DPP(v, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), (ctrl), 0xF, 0xF, false))
#define MT_DPP_U(v, ctrl) ((u32)__builtin_amdgcn_update_dpp(0, (int)(v), (ctrl), 0xF, 0xF, false))
#define MT_QUAD_1032 0xB1
#define MT_QUAD_2301 0x4E
#define MT_ROW_ROR4 0x124
#define MT_ROW_ROR8 0x128
#define MT_ROW_HALF_MIRROR 0x141
#define MT_TWO_P24 16777216.0f
#define MT_TWO_P20 1048576.0f

// ---- the images ----------------------------------------------------------------------------------------------------------
// One wavefront per (token slot 0..7, super-block); lane l holds elements 4 l .. 4 l + 3 of the super-block. Returns the
// four values as (hi, lo) binary16 pairs of x * 2^e in the half order (0, 2, 1, 3) in which the nibble masks deliver the
// weights, and 2^-e.
struct MtPacked {
  mt_half4 hv, lv;
  float inv, scale;   // 2^-e and 2^e
};
__device__ __forceinline__ MtPacked mt_pack4(float4 v) {
  // power of two that brings the largest magnitude of the super-block to [2^12, 2^13) (unsigned maximum of the bit
  // patterns without sign: orders magnitudes like the floats)
  u32 ab = __builtin_bit_cast(u32, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
  ab = max(ab, MT_DPP_U(ab, MT_QUAD_1032));
  ab = max(ab, MT_DPP_U(ab, MT_QUAD_2301));
  ab = max(ab, MT_DPP_U(ab, MT_ROW_ROR4));
  ab = max(ab, MT_DPP_U(ab, MT_ROW_ROR8));
  const u32 ab4 = max(max((u32)__builtin_amdgcn_readlane((int)ab, 0), (u32)__builtin_amdgcn_readlane((int)ab, 16)),
                      max((u32)__builtin_amdgcn_readlane((int)ab, 32), (u32)__builtin_amdgcn_readlane((int)ab, 48)));
  const int e = (int)((ab4 >> 23) & 0xFFu);
  int sh = 139 - e;            // scale = 2^sh
  sh = sh > 126 ? 126 : sh;    // zeros and subnormal values: 2^sh and 2^-sh stay normal numbers (every normal input keeps its 22 bits)
  // (the largest finite magnitudes give sh = -115, infinities and NaN -116: 2^sh and 2^-sh are normal numbers for every
  // input, so any finite activation lands in the binary16 range and non-finite ones stay what they are)
  const float scale = __builtin_bit_cast(float, (u32)(127 + sh) << 23);
  MtPacked r;
  r.scale = scale;
  r.inv = __builtin_bit_cast(float, (u32)(127 - sh) << 23);
  const _Float16 h0 = (_Float16)(v.x * scale), h1 = (_Float16)(v.y * scale), h2 = (_Float16)(v.z * scale), h3 = (_Float16)(v.w * scale);
  // (x * scale is exact, so fma(x, scale, -hi) is (x * scale) - hi in one instruction)
  const _Float16 l0 = (_Float16)fmaf(v.x, scale, -(float)h0), l1 = (_Float16)fmaf(v.y, scale, -(float)h1),
                 l2 = (_Float16)fmaf(v.z, scale, -(float)h2), l3 = (_Float16)fmaf(v.w, scale, -(float)h3);
  r.hv = (mt_half4){h0, h2, h1, h3};
  r.lv = (mt_half4){l0, l2, l1, l3};
  return r;
}

// Q4_K image: [super-block][instruction j = 2 g + par][lane = 16 kg + row][8 halves]: the halves of lane (kg, row = 2 token
// + part) are part (0 = hi, 1 = lo) of x[token][256 sb + 64 g + 32 par + 8 kg + (0,2,1,3,4,6,5,7)] * 2^e. Behind the
// in_dim / 256 * 8 KiB of operands: [super-block][lane = 16 kg + row][16 bytes]: four halves, part of sum(x[token] over
// sub-block 4 kg + (0,2,1,3)) * 2^(e-5) for kg < 2 and zeros for kg >= 2 (the eight sub-block sums as one more matrix-core
// operand, in the order in which a masked dword of min bytes delivers them), then 2^-e of tokens 2 kg and 2 kg + 1 (what
// result lane 16 kg + n needs). Tokens at and above `tokens` are zero.
// One wavefront's share of the Q4_K image: (token slot tok, super-block sb) from the lane's four values v (elements
// 4 lane .. 4 lane + 3 of the super-block; zeros and present = false for a token that is not there).
__device__ __forceinline__ void mt_pack_store_q4k(uint8_t* __restrict__ image, u32 nsb, u32 sb, u32 tok, u32 lane, float4 v, bool present) {
  const MtPacked pk = mt_pack4(v);
  // element 4 l sits in instruction j = l / 8, k-group (l / 2) % 4, upper half of the lane's eight if l is odd
  const u32 j = lane >> 3, kg = (lane >> 1) & 3;
  uint8_t* op = image + ((size_t)(sb * 8 + j) * 64 + kg * 16 + 2 * tok) * 16 + 8 * (lane & 1);
  *reinterpret_cast<mt_half4*>(op) = pk.hv;
  *reinterpret_cast<mt_half4*>(op + 16) = pk.lv;
  // sums of the eight sub-blocks (eight lanes each) for the min term
  // (summed after the scaling, which is exact: the same bits as scaling the sum, and no overflow for activations near
  // the top of the fp32 range)
  float sm = (v.x * pk.scale + v.y * pk.scale) + (v.z * pk.scale + v.w * pk.scale);
  sm += MT_DPP(sm, MT_QUAD_1032);
  sm += MT_DPP(sm, MT_QUAD_2301);
  sm += MT_DPP(sm, MT_ROW_HALF_MIRROR);
  const float s32 = 0.03125f;
  const _Float16 sh = (_Float16)(sm * s32), sl = (_Float16)fmaf(sm, s32, -(float)sh);
  uint8_t* aux = image + (size_t)nsb * 8192 + (size_t)sb * 1024;
  if ((lane & 3) == 0) {
    // lanes 8 j hold sub-block j: k-group j / 4, slot (0,2,1,3)[j % 4]; lanes 8 j + 4 write the zeros of k-groups 2, 3
    const u32 sj = lane >> 3, zero = (lane >> 2) & 1;
    const u32 slot = ((sj & 1) << 1) | ((sj >> 1) & 1);
    _Float16* ap = reinterpret_cast<_Float16*>(aux + (((sj >> 2) + 2 * zero) * 16 + 2 * tok) * 16) + slot;
    ap[0] = zero ? (_Float16)0.0f : sh;   // row 2 tok (hi)
    ap[8] = zero ? (_Float16)0.0f : sl;   // row 2 tok + 1 (lo): the next lane's 16 bytes
  }
  if (lane < 16) reinterpret_cast<float*>(aux + ((tok >> 1) * 16 + lane) * 16)[2 + (tok & 1)] = present ? pk.inv : 0.0f;
}
extern "C" __global__ __launch_bounds__(256) void pack_x_mt_q4k_f16(const float* __restrict__ x, uint8_t* __restrict__ image,
                                                                    u32 tokens, u32 in_dim) {
  const u32 lane = threadIdx.x & 63;
  const u32 unit = blockIdx.x * 4 + (threadIdx.x >> 6);
  const u32 nsb = in_dim >> 8, nsbp = gemv_mt_padded_sb(in_dim);
  const u32 sb = unit >> 3, tok = unit & 7;
  if (sb >= nsbp) return;
  const bool present = tok < tokens && sb < nsb;   // (super-blocks past the row's end: zeros, as for an absent token)
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (present) __builtin_memcpy(&v, x + (size_t)tok * in_dim + (size_t)sb * 256 + 4 * lane, 16);
  mt_pack_store_q4k(image, nsbp, sb, tok, lane, v, present);
}

// The image for sixteen single-term tokens (MtK45<Q5, true>): the same bytes per super-block with row = token, the halves
// binary16(x) as they are; behind the operands, per (super-block, lane = 16 kg + token), the sums of sub-blocks
// 4 kg + (0,2,1,3) of the rounded values / 32 as hi (halves 0..3) and lo (halves 4..7) binary16 terms, zeros for kg >= 2.
// (x, image, tokens <= 16, in_dim): block 256, grid 4 * gemv_mt_padded_sb(in_dim). |x| has to stay inside the binary16
// range, as for the prefill GEMM.
// One wavefront's share of that image: (token slot tok < 16, super-block sb) from the lane's four values v (zeros for a token or
// super-block that is not there).
__device__ __forceinline__ void mt_pack16_store_q4k(uint8_t* __restrict__ image, u32 nsbp, u32 sb, u32 tok, u32 lane, float4 v) {
  const _Float16 h0 = (_Float16)v.x, h1 = (_Float16)v.y, h2 = (_Float16)v.z, h3 = (_Float16)v.w;
  // element 4 l sits in instruction j = l / 8, k-group (l / 2) % 4, upper half of the lane's eight if l is odd (mt_pack_store_q4k)
  const u32 j = lane >> 3, kg = (lane >> 1) & 3;
  *reinterpret_cast<mt_half4*>(image + ((size_t)(sb * 8 + j) * 64 + kg * 16 + tok) * 16 + 8 * (lane & 1)) = (mt_half4){h0, h2, h1, h3};
  float sm = ((float)h0 + (float)h1) + ((float)h2 + (float)h3);
  sm += MT_DPP(sm, MT_QUAD_1032);
  sm += MT_DPP(sm, MT_QUAD_2301);
  sm += MT_DPP(sm, MT_ROW_HALF_MIRROR);
  const float s32 = 0.03125f;
  const _Float16 sh = (_Float16)(sm * s32), sl = (_Float16)fmaf(sm, s32, -(float)sh);
  uint8_t* aux = image + (size_t)nsbp * 8192 + (size_t)sb * 1024;
  if ((lane & 3) == 0) {
    const u32 sj = lane >> 3, zero = (lane >> 2) & 1;
    const u32 slot = ((sj & 1) << 1) | ((sj >> 1) & 1);
    _Float16* ap = reinterpret_cast<_Float16*>(aux + (((sj >> 2) + 2 * zero) * 16 + tok) * 16) + slot;
    ap[0] = zero ? (_Float16)0.0f : sh;
    ap[4] = zero ? (_Float16)0.0f : sl;
  }
}
extern "C" __global__ __launch_bounds__(256) void pack_x_mt16_q4k_f16(const float* __restrict__ x, uint8_t* __restrict__ image,
                                                                      u32 tokens, u32 in_dim) {
  const u32 lane = threadIdx.x & 63;
  const u32 unit = blockIdx.x * 4 + (threadIdx.x >> 6);
  const u32 nsb = in_dim >> 8, nsbp = gemv_mt_padded_sb(in_dim);
  const u32 sb = unit >> 4, tok = unit & 15;
  if (sb >= nsbp) return;
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (tok < tokens && sb < nsb) __builtin_memcpy(&v, x + (size_t)tok * in_dim + (size_t)sb * 256 + 4 * lane, 16);
  mt_pack16_store_q4k(image, nsbp, sb, tok, lane, v);
}

// The same for the Q6_K order: sums of sub-blocks 4 kg .. 4 kg + 3 / 16 as hi (halves 0..3) and lo (halves 4..7).
__device__ __forceinline__ void mt_pack16_store_q6k(uint8_t* __restrict__ image, u32 nsbp, u32 sb, u32 tok, u32 lane, float4 v) {
  const _Float16 h0 = (_Float16)v.x, h1 = (_Float16)v.y, h2 = (_Float16)v.z, h3 = (_Float16)v.w;
  // element 4 l sits in sub-block s = l / 4, k-group l % 4 (mt_pack_store_q6k)
  const u32 s = lane >> 2, kg = lane & 3;
  *reinterpret_cast<mt_half4*>(image + ((size_t)(sb * 8 + (s >> 1)) * 64 + kg * 16 + tok) * 16 + 8 * (s & 1)) = (mt_half4){h0, h2, h1, h3};
  float sm = ((float)h0 + (float)h1) + ((float)h2 + (float)h3);
  sm += MT_DPP(sm, MT_QUAD_1032);
  sm += MT_DPP(sm, MT_QUAD_2301);
  const float s16 = 0.0625f;
  const _Float16 sh = (_Float16)(sm * s16), sl = (_Float16)fmaf(sm, s16, -(float)sh);
  uint8_t* aux = image + (size_t)nsbp * 8192 + (size_t)sb * 1024;
  if ((lane & 3) == 0) {
    _Float16* ap = reinterpret_cast<_Float16*>(aux + ((s >> 2) * 16 + tok) * 16) + (s & 3);
    ap[0] = sh;
    ap[4] = sl;
  }
}
extern "C" __global__ __launch_bounds__(256) void pack_x_mt16_q6k_f16(const float* __restrict__ x, uint8_t* __restrict__ image,
                                                                      u32 tokens, u32 in_dim) {
  const u32 lane = threadIdx.x & 63;
  const u32 unit = blockIdx.x * 4 + (threadIdx.x >> 6);
  const u32 nsb = in_dim >> 8, nsbp = gemv_mt_padded_sb(in_dim);
  const u32 sb = unit >> 4, tok = unit & 15;
  if (sb >= nsbp) return;
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (tok < tokens && sb < nsb) __builtin_memcpy(&v, x + (size_t)tok * in_dim + (size_t)sb * 256 + 4 * lane, 16);
  mt_pack16_store_q6k(image, nsbp, sb, tok, lane, v);
}

// Q6_K image: [super-block][sub-block pair p][lane = 16 kg + row][2 x 4 halves]: the halves of lane (kg, row = 2 token +
// part) for sub-block s = 2 p + (0 | 1) are part of x[token][256 sb + 16 s + 4 kg + (0,2,1,3)] * 2^e. Behind the operands:
// [super-block][lane = 16 kg + row][16 bytes]: four halves, part of sum(x[token] over sub-block 4 kg + (0,1,2,3)) * 2^(e-4)
// (the sixteen sub-block sums as one more matrix-core operand: sixteen values of magnitude below 2^e-13 each stay in
// binary16 range at 2^(e-4)), then 2^-e of tokens 2 kg and 2 kg + 1 (what result lane 16 kg + n needs).
__device__ __forceinline__ void mt_pack_store_q6k(uint8_t* __restrict__ image, u32 nsb, u32 sb, u32 tok, u32 lane, float4 v, bool present) {
  const MtPacked pk = mt_pack4(v);
  // element 4 l sits in sub-block s = l / 4, k-group l % 4
  const u32 s = lane >> 2, kg = lane & 3;
  uint8_t* op = image + ((size_t)(sb * 8 + (s >> 1)) * 64 + kg * 16 + 2 * tok) * 16 + 8 * (s & 1);
  *reinterpret_cast<mt_half4*>(op) = pk.hv;
  *reinterpret_cast<mt_half4*>(op + 16) = pk.lv;
  // sums of the sixteen sub-blocks (four lanes each), of the scaled values (exact, and safe near the top of the fp32 range)
  float sm = (v.x * pk.scale + v.y * pk.scale) + (v.z * pk.scale + v.w * pk.scale);
  sm += MT_DPP(sm, MT_QUAD_1032);
  sm += MT_DPP(sm, MT_QUAD_2301);
  const float s16 = 0.0625f;
  const _Float16 sh = (_Float16)(sm * s16), sl = (_Float16)fmaf(sm, s16, -(float)sh);
  uint8_t* aux = image + (size_t)nsb * 8192 + (size_t)sb * 1024;
  if ((lane & 3) == 0) {
    _Float16* ap = reinterpret_cast<_Float16*>(aux + ((s >> 2) * 16 + 2 * tok) * 16) + (s & 3);
    ap[0] = sh;   // row 2 tok (hi)
    ap[8] = sl;   // row 2 tok + 1 (lo): the next lane's 16 bytes
  }
  if (lane < 16) reinterpret_cast<float*>(aux + ((tok >> 1) * 16 + lane) * 16)[2 + (tok & 1)] = present ? pk.inv : 0.0f;
}
extern "C" __global__ __launch_bounds__(256) void pack_x_mt_q6k_f16(const float* __restrict__ x, uint8_t* __restrict__ image,
                                                                    u32 tokens, u32 in_dim) {
  const u32 lane = threadIdx.x & 63;
  const u32 unit = blockIdx.x * 4 + (threadIdx.x >> 6);
  const u32 nsb = in_dim >> 8, nsbp = gemv_mt_padded_sb(in_dim);
  const u32 sb = unit >> 3, tok = unit & 7;
  if (sb >= nsbp) return;
  const bool present = tok < tokens && sb < nsb;   // (super-blocks past the row's end: zeros, as for an absent token)
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (present) __builtin_memcpy(&v, x + (size_t)tok * in_dim + (size_t)sb * 256 + 4 * lane, 16);
  mt_pack_store_q6k(image, nsbp, sb, tok, lane, v, present);
}

// ---- loads in assembly ---------------------------------------------------------------------------------------------------
// The compiler knows neither that these are loads nor when they land. A value loaded this way must not be touched before
// mt_wait<N> has said that it is there and mt_pin has tied it to that wait.
// A uniform address as a scalar base. When the compiler keeps the value in a vector register (it does under scalar
// register pressure), the readfirstlane that brings it back is a vector instruction that writes scalar registers, and a
// memory instruction may read such registers only five wait states later. The compiler spaces the instructions it
// emits itself, but not the ones inside an asm statement: mt_settle provides the wait states, and because the bases pass
// through it, every readfirstlane lies before it and every load behind it.
__device__ __forceinline__ u64 mt_sbase(const void* p) {
  const u64 b = (u64)(uintptr_t)p;
  return (u64)(u32)__builtin_amdgcn_readfirstlane((int)(u32)b) | ((u64)(u32)__builtin_amdgcn_readfirstlane((int)(u32)(b >> 32)) << 32);
}
__device__ __forceinline__ void mt_settle(u64& a, u64& b, u64& c) { asm volatile("s_nop 4" : "+s"(a), "+s"(b), "+s"(c)); }
// 16 bytes from sb (mt_sbase, settled) + voff + IMM
template <int IMM>
__device__ __forceinline__ void mt_load16(mt_u32x4& dst, u64 sb, u32 voff) {
  static_assert(IMM >= 0 && IMM < 4096, "the instruction's offset field");
  asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(dst) : "v"(voff), "s"(sb), "n"(IMM) : "memory");
}
// 16 bytes per active lane from addr to LDS byte address lds_base (uniform) + 16 * lane
__device__ __forceinline__ void mt_copy16(u32 lds_base, const void* addr) {
  const u32 m0 = (u32)__builtin_amdgcn_readfirstlane((int)lds_base);
  // (M0 cannot be named as clobbered - it is a reserved register and the compiler says it may ignore such a clobber -
  // so nothing the compiler emits in these kernels may rely on a value of M0: the build checks that every reader of M0
  // in them sits directly behind a write of M0, check_hazards.py)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m0), "v"(addr) : "memory");
}
template <int N>
__device__ __forceinline__ void mt_wait() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __forceinline__ void mt_pin(mt_u32x4& v) { asm volatile("" : "+v"(v)); }

// ---- the weight formats --------------------------------------------------------------------------------------------------
// A format says how a tile's share of a super-block (a unit: 16 rows x one block) is copied to LDS and what a lane does
// with it. P = 16-byte pieces per row in LDS, NCOPY = copy instructions per unit (the last with LAST lanes), NAUX = 16-byte
// loads of scales and sums per (super-block, token pair), NSLOT = units a wavefront has room for in LDS, TYPE = the GGUF
// type number (what gemv_config.h's rules are asked with).
//
// Q4_K (144 B: d, dmin, scales[12], qs[128]) and Q5_K (176 B: d, dmin, scales[12], qh[32], qs[128]): byte l of qs[32 g ..
// 32 g + 32) holds element 64 g + l (low nibble, sub-block 2 g) and element 64 g + 32 + l (high nibble, sub-block 2 g + 1);
// Q5_K adds bit 2 g / 2 g + 1 of qh[l] as the fifth bit of the two. Both read the same activation image (the Q4_K one).
// X16: the sixteen rows of the activation operand are sixteen tokens in one binary16 term each (the precision of the prefill
// GEMM: x rounded to half, no scaling) instead of eight tokens x (hi, lo) - the kernel for 9..16 tokens (image from
// pack_x_mt16_q4k_f16: no token scales, the sub-block sums as hi and lo operands).
template <bool Q5, bool X16 = false>
struct MtK45 {
  static constexpr unsigned TYPE = Q5 ? 13 : 12;
  static constexpr int NTOK = X16 ? 16 : 8;   // tokens a launch covers
  static constexpr int BB = Q5 ? 176 : 144, P = BB / 16, NCOPY = 3, LAST = 16 * P - 128, NAUX = 1, NSLOT = 6, TMAX = 3;
  static constexpr int QOFF = Q5 ? 48 : 16;   // where qs starts in the block
  static constexpr u32 UNIT_BYTES = 16 * P * 16, AUX_SB_BYTES = 64 * 16;
  // byte offset, inside the row's block, of the piece that goes to place `piece` of the row in LDS
  static __device__ __forceinline__ u32 piece_offset(u32 piece) { return piece * 16; }
  // where a lane's scales and sums sit inside a super-block's share of the image: 16 bytes of its own per lane
  static __device__ __forceinline__ u32 aux_offset(u32 lane) { return lane * 16; }

  // the scales of the lane's two tokens and, as the matrix-core operand of lane (kg, row), the sums of sub-blocks
  // 4 kg + (0,2,1,3) of that row's (token, part) (zeros for kg >= 2)
  // (X16: no scales; the second half of the 16 bytes is the low term of the sums, a second operand)
  struct Aux { float fsc[2]; mt_u32x2 sums, sums_lo; };
  static __device__ __forceinline__ Aux aux(const mt_u32x4 (&r)[NAUX]) {
    Aux a;
    a.sums = (mt_u32x2){r[0].x, r[0].y};
    a.sums_lo = (mt_u32x2){r[0].z, r[0].w};
    a.fsc[0] = __uint_as_float(r[0].z), a.fsc[1] = __uint_as_float(r[0].w);
    return a;
  }
  // what a lane takes out of its row's block in LDS
  struct Raw { uint4 hdr; uint2 q[4], h; u32 kg; };   // (h: the lane's eight qh bytes, Q5_K only; kg: the lane's k-group)
  static __device__ __forceinline__ Raw read(const char* row, u32 kg) {
    Raw w;
    w.kg = kg;
    w.hdr = *reinterpret_cast<const uint4*>(row);
#pragma unroll
    for (int g = 0; g < 4; g++) w.q[g] = *reinterpret_cast<const uint2*>(row + QOFF + 32 * g + 8 * kg);
    w.h = Q5 ? *reinterpret_cast<const uint2*>(row + 16 + 8 * kg) : make_uint2(0u, 0u);
    return w;
  }
  // acc[0..3] += this unit's share for tokens (2 rg, 2 rg + 1) x (hi, lo)
  static __device__ __forceinline__ void unit(const Raw& w, const mt_u32x4 (&b)[8], const Aux& ax, float (&acc)[4]) {
    // (a) eight instructions, one per sub-block, each into an accumulator of its own
    mt_float4 dacc[8];
#pragma unroll
    for (int g = 0; g < 4; g++) {
      // Q5_K: per byte of t, bit 0 is the fifth bit of the low-nibble element and bit 1 that of the high-nibble element
      const u32 tx = w.h.x >> (2 * g), ty = w.h.y >> (2 * g);
#pragma unroll
      for (int par = 0; par < 2; par++) {
        const u32 mask = par ? 0x00F000F0u : 0x000F000Fu;
        uint4 a4;
        a4.x = w.q[g].x & mask;
        a4.y = (w.q[g].x >> 8) & mask;
        a4.z = w.q[g].y & mask;
        a4.w = (w.q[g].y >> 8) & mask;
        if constexpr (Q5) {
          // a code is nibble | fifth bit << 4: bit 4 of a half for the low nibbles (x 2^-24), bit 8 for the high ones (x 2^-20)
          if (par == 0) {
            a4.x |= (tx << 4) & 0x00100010u;   // bytes 0, 2
            a4.y |= (tx >> 4) & 0x00100010u;   // bytes 1, 3
            a4.z |= (ty << 4) & 0x00100010u;
            a4.w |= (ty >> 4) & 0x00100010u;
          } else {
            a4.x |= (tx << 7) & 0x01000100u;
            a4.y |= (tx >> 1) & 0x01000100u;
            a4.z |= (ty << 7) & 0x01000100u;
            a4.w |= (ty >> 1) & 0x01000100u;
          }
        }
        dacc[2 * g + par] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(mt_half8, b[2 * g + par]),
                                                                   __builtin_bit_cast(mt_half8, a4),
                                                                   (mt_float4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
      }
    }
    // (b) the eight (scale, min) pairs of this lane's weight row as bytes (dequant.cr:240-249, four at a time):
    //     scA = sc 0..3, scB = sc 4..7, mA = m 0..3, mB = m 4..7
    const u32 s0 = w.hdr.y, s1 = w.hdr.z, s2 = w.hdr.w;
    const u32 scA = s0 & 0x3F3F3F3Fu, mA = s1 & 0x3F3F3F3Fu;
    const u32 scB = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
    const u32 mB = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
    const float sc[8] = {ubyte_f<0>(scA), ubyte_f<1>(scA), ubyte_f<2>(scA), ubyte_f<3>(scA),
                         ubyte_f<0>(scB), ubyte_f<1>(scB), ubyte_f<2>(scB), ubyte_f<3>(scB)};
    const float dd = h2f(w.hdr.x), dmin = h2f(w.hdr.x >> 16);
    // (c) sum_j sc_j * result_j, even sub-blocks (low nibbles, 2^-24) and odd ones (high nibbles, 2^-20) apart
    float ev[4] = {0.f, 0.f, 0.f, 0.f}, od[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 8; j++) {
#pragma unroll
      for (int k = 0; k < 4; k++) {
        if (j & 1) od[k] = fmaf(sc[j], dacc[j][k], od[k]);
        else ev[k] = fmaf(sc[j], dacc[j][k], ev[k]);
      }
    }
    // (d) sum_j m_j * sum(x_j): one more instruction, the eight sub-block sums (times 2^(e-5), hi and lo) against the min
    //     bytes of k-groups 0 and 1 read as binary16 (m * 2^-24, in the order bytes 0, 2, 1, 3 of the masked dword)
    const u32 msel = w.kg == 0 ? mA : (w.kg == 1 ? mB : 0u);
    const mt_u32x2 mb = {msel & 0x00FF00FFu, (msel >> 8) & 0x00FF00FFu};
    mt_float4 off = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(mt_half4, ax.sums), __builtin_bit_cast(mt_half4, mb),
                                                          (mt_float4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    if constexpr (X16)
      off = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(mt_half4, ax.sums_lo), __builtin_bit_cast(mt_half4, mb), off, 0, 0, 0);
    const float d24 = dd * MT_TWO_P24, d20 = dd * MT_TWO_P20, dm29 = dmin * -536870912.0f;   // 2^24 * 2^5
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const float in = fmaf(d24, ev[k], fmaf(dm29, off[k], d20 * od[k]));
      if constexpr (X16) acc[k] += in;   // (rows 4 rg .. 4 rg + 3 are four tokens)
      else acc[k] = fmaf(ax.fsc[k >> 1], in, acc[k]);
    }
  }
};
typedef MtK45<false> MtQ4K;
typedef MtK45<true> MtQ5K;
typedef MtK45<false, true> MtQ4Kx16;
typedef MtK45<true, true> MtQ5Kx16;

// Q8_0 (34 B per 32 values: d, qs:i8[32]). Eight blocks are taken together as one 272-byte "super-block" of 256 values
// (17 pieces of 16 bytes; in_dim a multiple of 256 makes every row a whole number of them, 16-byte aligned when the matrix
// is). Block j of the eight is instruction j: a lane supplies bytes 8 kg .. 8 kg + 7 of its 32 codes, which the masks
// deliver in the order (0, 2, 1, 3, 4, 6, 5, 7) - the order of the Q4_K image, so Q8_0 reads the image pack_x_mt_q4k_f16
// writes. A code goes in as the unsigned byte q + 128 (q ^ 0x80 read as a binary16 subnormal, (q + 128) * 2^-24); the 128
// comes out again through the sub-block sums: sum_j d_j * (sum(x u) - 128 sum(x)), with sum_j d_j * sum_j(x) as one more
// instruction (the image's sums operand against the eight d as they are: binary16 numbers).
// In LDS a row is its 272 bytes as they are: d of block j at 34 j, its codes at 34 j + 2. The codes of the odd blocks start
// on a multiple of 4 (two dword reads); the even blocks' are 2 bytes off and come out of three dwords through
// v_alignbyte_b32.
template <bool X16 = false>   // (X16: sixteen single-term tokens, as MtK45's; the image of pack_x_mt16_q4k_f16)
struct MtQ80T {
  static constexpr unsigned TYPE = 8;
  static constexpr int NTOK = X16 ? 16 : 8;
  static constexpr int BB = 272, P = 17, NCOPY = 5, LAST = 16, NAUX = 1, NSLOT = 4, TMAX = 2;
  static constexpr u32 UNIT_BYTES = 16 * P * 16, AUX_SB_BYTES = 64 * 16;
  static __device__ __forceinline__ u32 piece_offset(u32 piece) { return piece * 16; }
  static __device__ __forceinline__ u32 aux_offset(u32 lane) { return lane * 16; }
  typedef MtK45<false>::Aux Aux;
  static __device__ __forceinline__ Aux aux(const mt_u32x4 (&r)[NAUX]) { return MtK45<false>::aux(r); }
  struct Raw { u32 q[8][2]; u32 d[8]; u32 kg; };   // (d: binary16 bits)
  static __device__ __forceinline__ Raw read(const char* row, u32 kg) {
    Raw w;
    w.kg = kg;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      w.d[j] = *reinterpret_cast<const unsigned short*>(row + 34 * j);
      const char* c = row + 34 * j + 2 + 8 * kg;
      if (j & 1) {
        w.q[j][0] = *reinterpret_cast<const u32*>(c);
        w.q[j][1] = *reinterpret_cast<const u32*>(c + 4);
      } else {
        const u32 a = *reinterpret_cast<const u32*>(c - 2), b = *reinterpret_cast<const u32*>(c + 2), e = *reinterpret_cast<const u32*>(c + 6);
        w.q[j][0] = __builtin_amdgcn_alignbyte(b, a, 2);
        w.q[j][1] = __builtin_amdgcn_alignbyte(e, b, 2);
      }
    }
    return w;
  }
  static __device__ __forceinline__ void unit(const Raw& w, const mt_u32x4 (&b)[8], const Aux& ax, float (&acc)[4]) {
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const u32 u0 = w.q[j][0] ^ 0x80808080u, u1 = w.q[j][1] ^ 0x80808080u;
      uint4 a4;
      a4.x = u0 & 0x00FF00FFu;          // bytes 0, 2
      a4.y = (u0 >> 8) & 0x00FF00FFu;   // bytes 1, 3
      a4.z = u1 & 0x00FF00FFu;
      a4.w = (u1 >> 8) & 0x00FF00FFu;
      const mt_float4 r = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(mt_half8, b[j]), __builtin_bit_cast(mt_half8, a4),
                                                                 (mt_float4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
      const float dj = h2f(w.d[j]);
#pragma unroll
      for (int k = 0; k < 4; k++) sum[k] = fmaf(dj, r[k], sum[k]);
    }
    // sum_j d_j * sum_j(x): the image's sums (times 2^(e-5), hi and lo; sub-blocks 4 kg + (0, 2, 1, 3) for kg < 2) against d
    const u32 dA = w.kg == 0 ? (w.d[0] | (w.d[2] << 16)) : (w.d[4] | (w.d[6] << 16));
    const u32 dB = w.kg == 0 ? (w.d[1] | (w.d[3] << 16)) : (w.d[5] | (w.d[7] << 16));
    const mt_u32x2 db = w.kg < 2 ? (mt_u32x2){dA, dB} : (mt_u32x2){0u, 0u};
    mt_float4 off = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(mt_half4, ax.sums), __builtin_bit_cast(mt_half4, db),
                                                          (mt_float4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    if constexpr (X16)
      off = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(mt_half4, ax.sums_lo), __builtin_bit_cast(mt_half4, db), off, 0, 0, 0);
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const float in = fmaf(MT_TWO_P24, sum[k], -4096.0f * off[k]);   // 128 * 2^5
      if constexpr (X16) acc[k] += in;
      else acc[k] = fmaf(ax.fsc[k >> 1], in, acc[k]);
    }
  }
};
typedef MtQ80T<false> MtQ80;
typedef MtQ80T<true> MtQ80x16;


// Q6_K (210 B: ql[128], qh[64], scales:i8[16], d). Element 128 n + 32 k + l (half n, quarter k, l < 32) has its low four bits
// in nibble k / 2 of ql[64 n + 32 (k % 2) + l] and its high two in bits 2 k, 2 k + 1 of qh[32 n + l]; sub-block
// s = 8 n + 2 k + l / 16. A row's block starts at a multiple of 2 bytes only; it is copied from exactly its start (the
// memory pipeline takes unaligned 16-byte loads), so inside LDS every field sits at its natural alignment. A row in LDS
// is 15 pieces (240 bytes: rows 60 dwords apart hit 16 different bank groups): pieces 0..12 are bytes 0..207 of the block,
// piece 13 is bytes 194..209 (shifted back so that nothing past the end of the matrix is read: d sits at byte 222 of
// the row) and piece 14 repeats piece 13.
// (X16: sixteen single-term tokens, as MtK45's)
template <bool X16 = false>
struct MtQ6KT {
  static constexpr int NTOK = X16 ? 16 : 8;
  static constexpr unsigned TYPE = 14;
  static constexpr int BB = 210, P = 15, NCOPY = 4, LAST = 48, NAUX = 1, NSLOT = 4, TMAX = 2;
  static constexpr u32 UNIT_BYTES = 16 * P * 16, AUX_SB_BYTES = 64 * 16;
  static __device__ __forceinline__ u32 piece_offset(u32 piece) { return piece < 13 ? piece * 16 : 194u; }
  static __device__ __forceinline__ u32 aux_offset(u32 lane) { return lane * 16; }   // 16 bytes of its own per lane

  // the scales of the lane's two tokens and, as the matrix-core operand of lane (kg, row), the sums of sub-blocks
  // 4 kg .. 4 kg + 3 of that row's (token, part)
  struct Aux { float fsc[2]; mt_u32x2 sums, sums_lo; };
  static __device__ __forceinline__ Aux aux(const mt_u32x4 (&r)[NAUX]) {
    Aux a;
    a.sums = (mt_u32x2){r[0].x, r[0].y};
    a.sums_lo = (mt_u32x2){r[0].z, r[0].w};
    a.fsc[0] = __uint_as_float(r[0].z), a.fsc[1] = __uint_as_float(r[0].w);
    return a;
  }
  // [2 n + hh]: ql dword of quarters 0/2, of quarters 1/3, qh dword; sck: the scale bytes of sub-blocks 4 kg .. 4 kg + 3
  struct Raw { u32 a[4], b[4], h[4]; uint4 sc; u32 d, sck; };
  static __device__ __forceinline__ Raw read(const char* row, u32 kg) {
    Raw w;
#pragma unroll
    for (int n = 0; n < 2; n++)
#pragma unroll
      for (int hh = 0; hh < 2; hh++) {
        w.a[2 * n + hh] = *reinterpret_cast<const u32*>(row + 64 * n + 16 * hh + 4 * kg);
        w.b[2 * n + hh] = *reinterpret_cast<const u32*>(row + 64 * n + 32 + 16 * hh + 4 * kg);
        w.h[2 * n + hh] = *reinterpret_cast<const u32*>(row + 128 + 32 * n + 16 * hh + 4 * kg);
      }
    w.sc = *reinterpret_cast<const uint4*>(row + 192);
    w.sck = *reinterpret_cast<const u32*>(row + 192 + 4 * kg);
    w.d = *reinterpret_cast<const unsigned short*>(row + 222);
    return w;
  }
  static __device__ __forceinline__ float sbyte_f(u32 v, int k) { return (float)(int)(signed char)((v >> (8 * k)) & 0xFFu); }
  static __device__ __forceinline__ void unit(const Raw& w, const mt_u32x4 (&b)[8], const Aux& ax, float (&acc)[4]) {
    const u32 scw[4] = {w.sc.x, w.sc.y, w.sc.z, w.sc.w};
    float lo[4] = {0.f, 0.f, 0.f, 0.f}, hi[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int n = 0; n < 2; n++) {
#pragma unroll
      for (int hh = 0; hh < 2; hh++) {
        const u32 A = w.a[2 * n + hh], B = w.b[2 * n + hh], H = w.h[2 * n + hh];
        const u32 A8 = A >> 8, B8 = B >> 8, Hl4 = H << 4, Hr4 = H >> 4, Hl2 = H << 2, Hr6 = H >> 6;
        // 6-bit codes of quarters 0..3 as pairs of binary16 subnormals: .x = bytes 0, 2, .y = bytes 1, 3 of the dword
        mt_u32x2 q[4];
        q[0] = (mt_u32x2){(A & 0x000F000Fu) | (Hl4 & 0x00300030u), (A8 & 0x000F000Fu) | (Hr4 & 0x00300030u)};
        q[1] = (mt_u32x2){(B & 0x000F000Fu) | (Hl2 & 0x00300030u), (B8 & 0x000F000Fu) | (Hr6 & 0x00300030u)};
        q[2] = (mt_u32x2){(A & 0x00F000F0u) | (Hl4 & 0x03000300u), (A8 & 0x00F000F0u) | (Hr4 & 0x03000300u)};
        q[3] = (mt_u32x2){(B & 0x00F000F0u) | (Hl2 & 0x03000300u), (B8 & 0x00F000F0u) | (Hr6 & 0x03000300u)};
#pragma unroll
        for (int k = 0; k < 4; k++) {
          const int s = 8 * n + 2 * k + hh;   // the sub-block these sixteen weights are
          const mt_u32x4 bp = b[s >> 1];
          const mt_u32x2 xop = (s & 1) ? (mt_u32x2){bp.z, bp.w} : (mt_u32x2){bp.x, bp.y};
          const mt_float4 r = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(mt_half4, xop), __builtin_bit_cast(mt_half4, q[k]),
                                                                    (mt_float4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
          const float sc = sbyte_f(scw[s >> 2], s & 3);
#pragma unroll
          for (int e = 0; e < 4; e++) {
            if (k >= 2) hi[e] = fmaf(sc, r[e], hi[e]);
            else lo[e] = fmaf(sc, r[e], lo[e]);
          }
        }
      }
    }
    // sum (q - 32) x = sum q x - 32 sum x: per sub-block that is sc * sum(x), sixteen of them: one more instruction, the
    // sums (times 2^(e-4), hi and lo) against the scales as exact binary16 integers
    const mt_half4 scb = {(_Float16)sbyte_f(w.sck, 0), (_Float16)sbyte_f(w.sck, 1), (_Float16)sbyte_f(w.sck, 2), (_Float16)sbyte_f(w.sck, 3)};
    mt_float4 off = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(mt_half4, ax.sums), scb,
                                                          (mt_float4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
    if constexpr (X16) off = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(mt_half4, ax.sums_lo), scb, off, 0, 0, 0);
    const float dd = h2f(w.d), d24 = dd * MT_TWO_P24, d20 = dd * MT_TWO_P20, d512 = dd * -512.0f;   // 32 * 2^4
#pragma unroll
    for (int k = 0; k < 4; k++) {
      const float in = fmaf(d24, lo[k], fmaf(d512, off[k], d20 * hi[k]));
      if constexpr (X16) acc[k] += in;
      else acc[k] = fmaf(ax.fsc[k >> 1], in, acc[k]);
    }
  }
};
typedef MtQ6KT<false> MtQ6K;
typedef MtQ6KT<true> MtQ6Kx16;

// ---- the GEMV ------------------------------------------------------------------------------------------------------------
struct MtArgs {
  const uint8_t* w[3];
  float* out[3];
  u32 rows[3];
};

// (mt_stream_wait, the number a streamed unit waits with, lives in gemv_config.h: host code can test it there)

// SBW: super-blocks per k-slice (ceil(in_dim / 2048)). SBW <= 2: operands resident in registers, T tiles per wavefront, the next
// row group requested while this one is worked on. SBW >= 3: T = 1, operands streamed through two register sets.
// SWIGLU (T = 2, or T = 1 with streamed operands: gate tile, then up tile): the two tiles of a row group are tile grp of
// w[0] (gate) and tile grp of w[1] (up), rows[0] = rows[1] = out_dim, and the workgroup stores out[0][m][o] = silu(gate . x) * (up . x) (swiglu_one, the function of
// swiglu_f32): the values of the pair launch followed by swiglu_f32, bit for bit, without the gate and up vectors in memory.
// TOP1 (one matrix): instead of the row values the workgroup stores, per token, the largest of the rows it walked and
// that row's index (out[0][m * gridDim.x + blockIdx.x], top_ids[same]; of equal values the lowest row wins): the partial
// results top1_reduce_f32 finishes, as q6_k_gemv_top1_partial_f32 writes them for one token.
template <class F, int SBW, int T, bool SWIGLU = false, bool TOP1 = false>
__device__ __forceinline__ void gemv_mt_core(const MtArgs& a, const uint8_t* __restrict__ image,
                                             const float* __restrict__ residual, u32 in_dim, u32 tokens,
                                             u32* __restrict__ top_ids = nullptr) {
  constexpr bool STREAM = SBW > 2;
  constexpr int NTOK = F::NTOK;   // token rows of the partial sums: 8, or 16 single-term tokens
  static_assert(NTOK == 8 || (NTOK == 16 && !TOP1), "sixteen tokens: rows or SwiGLU, no top-1");
  static_assert(!TOP1 || (!SWIGLU && T * 16 * GEMV_MT_MAX_TOKENS <= GEMV_MT_WAVES * 64), "TOP1: a thread owns one (tile, token, row) of a row group");
  static_assert(!SWIGLU || T == (STREAM ? 1 : 2), "SWIGLU pairs a gate tile with an up tile");
  static_assert(!STREAM || T == 1, "streamed operands: one tile per wavefront");
  static_assert(STREAM || SBW * T <= F::NSLOT, "every unit of a row group has a slot");
  constexpr int NS = GEMV_MT_STREAM_SETS;   // register sets the streamed operands go through
  constexpr int NSETS = STREAM ? NS : SBW, NU = SBW * T, NA = 8 + F::NAUX, NC = F::NCOPY;
  extern __shared__ uint4 mt_lds4[];
  char* lds = reinterpret_cast<char*>(mt_lds4);
  const int tid = threadIdx.x, lane = tid & 63;
  const u32 wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const u32 nsb = in_dim >> 8, nsbp = gemv_mt_padded_sb(in_dim);   // super-blocks of a row, and of the image
  const u32 total_rows = a.rows[0] + a.rows[1] + a.rows[2];
  const u32 ntiles = (total_rows + 15) >> 4;
  const u32 ngroups = SWIGLU ? (a.rows[0] + 15) >> 4 : (ntiles + T - 1) / T;
  // LDS: partial[wave][GEMV_MT_TMAX][NTOK tokens][16 rows] f32 | slots[wave][NSLOT units]
  float* part = reinterpret_cast<float*>(lds);
  constexpr u32 SLOTS_OFF = GEMV_MT_WAVES * GEMV_MT_TMAX * NTOK * 16 * 4;
  const char* slots = lds + SLOTS_OFF + wave * (F::NSLOT * F::UNIT_BYTES);
  const u32 slots_lds = (u32)(size_t)(mt_lds_void*)mt_lds4 + SLOTS_OFF + wave * (F::NSLOT * F::UNIT_BYTES);

  // Lane roles. The activations are the A operand (16 rows = (token, part), k-group kg) and the weights the B operand
  // (16 columns = weight rows of the tile, k-group kg), so a result lane (column n = lane % 16, row group rg = lane / 16)
  // holds rows 4 rg .. 4 rg + 3 = tokens 2 rg, 2 rg + 1 x (hi, lo) of weight row n.
  const u32 ar = lane & 15, kg = lane >> 4;
  const u32 rg = lane >> 4;

  u32 grp = blockIdx.x;
  if (grp >= ngroups) return;
  float top_v = -__builtin_inff();   // TOP1: the best row this thread has seen in its place of the row groups
  u32 top_i = 0xFFFFFFFFu;

  // ---- operand sets: the A operands of a super-block and its scales and sub-block sums ----
  mt_u32x4 breg[NSETS][8], auxr[NSETS][F::NAUX];
  const uint8_t* aux = image + (size_t)nsbp * 8192;
  // (uniform bases and two lane offsets: no address registers per load)
  const u32 lane16 = lane * 16u, rg_off = F::aux_offset(lane);
  auto slice_sb = [&](int i) -> u32 { return GEMV_MT_CONTIGUOUS_SLICES ? wave * (u32)SBW + (u32)i : wave + 8u * (u32)i; };
  auto issue_set = [&](int i, int set) {
    const u32 sb = slice_sb(i);
    u64 ob = mt_sbase(image + (size_t)sb * 8192), ob2 = mt_sbase(image + (size_t)sb * 8192 + 4096);
    u64 ab = mt_sbase(aux + (size_t)sb * F::AUX_SB_BYTES);
    mt_settle(ob, ob2, ab);
    mt_load16<0>(breg[set][0], ob, lane16);
    mt_load16<1024>(breg[set][1], ob, lane16);
    mt_load16<2048>(breg[set][2], ob, lane16);
    mt_load16<3072>(breg[set][3], ob, lane16);
    mt_load16<0>(breg[set][4], ob2, lane16);
    mt_load16<1024>(breg[set][5], ob2, lane16);
    mt_load16<2048>(breg[set][6], ob2, lane16);
    mt_load16<3072>(breg[set][7], ob2, lane16);
    mt_load16<0>(auxr[set][0], ab, rg_off);
    if constexpr (F::NAUX > 1) {
      mt_load16<16>(auxr[set][1], ab, rg_off);
      mt_load16<32>(auxr[set][2], ab, rg_off);
      mt_load16<48>(auxr[set][3], ab, rg_off);
      mt_load16<64>(auxr[set][4], ab, rg_off);
    }
    static_assert(F::NAUX == 1 || F::NAUX == 5, "scale and sum loads per operand set");
  };
  auto pin_set = [&](int set) {
#pragma unroll
    for (int j = 0; j < 8; j++) mt_pin(breg[set][j]);
#pragma unroll
    for (int q = 0; q < F::NAUX; q++) mt_pin(auxr[set][q]);
  };

  // ---- the copies of a row group's units. Copy m of a unit: piece p = 64 m + lane (< 16 P), row p / P of the tile.
  const size_t row_bytes = (size_t)nsb * F::BB;
  const uint8_t* cptr[T][NC];   // where this lane's piece of copy m of tile t starts, without the super-block offset
  auto set_rows = [&](u32 g, int mat = 0) {   // (mat: with SWIGLU and streamed operands, gate (0) and up (1) take turns)
#pragma unroll
    for (int t = 0; t < T; t++) {
#pragma unroll
      for (int m = 0; m < NC; m++) {
        const u32 p = 64u * m + lane;
        const u32 pr = min(p / (u32)F::P, 15u), piece = p - (u32)F::P * (p / (u32)F::P);
        const u32 vr = SWIGLU ? min(g * 16 + pr, a.rows[0] - 1) : min((g * T + (u32)t) * 16 + pr, total_rows - 1);
        const uint8_t* rp;
        if constexpr (SWIGLU) rp = a.w[STREAM ? mat : t] + (size_t)vr * row_bytes;
        else if (vr < a.rows[0]) rp = a.w[0] + (size_t)vr * row_bytes;
        else if (vr < a.rows[0] + a.rows[1]) rp = a.w[1] + (size_t)(vr - a.rows[0]) * row_bytes;
        else rp = a.w[2] + (size_t)(vr - a.rows[0] - a.rows[1]) * row_bytes;
        cptr[t][m] = rp + F::piece_offset(piece);
      }
    }
  };
  auto issue_unit = [&](int i, int t, int slot) {
    // (a super-block past the row's end: the row's last block stands in; its operands in the image are zeros)
    const u32 off = min(slice_sb(i), nsb - 1u) * F::BB, dst = slots_lds + (u32)slot * F::UNIT_BYTES;
#pragma unroll
    for (int m = 0; m + 1 < NC; m++) mt_copy16(dst + 1024u * m, cptr[t][m] + off);
    if (lane < F::LAST) mt_copy16(dst + 1024u * (NC - 1), cptr[t][NC - 1] + off);
  };

  // k-slices through LDS in wavefront order: partial[wave][tile][token][row]; hi + lo of a token first
  auto store_part = [&](int t, const float (&acc)[4]) {
    if constexpr (NTOK == 16) {
#pragma unroll
      for (int k = 0; k < 4; k++) part[((wave * GEMV_MT_TMAX + t) * 16 + 4 * rg + k) * 16 + ar] = acc[k];
    } else {
      part[((wave * GEMV_MT_TMAX + t) * 8 + 2 * rg) * 16 + ar] = acc[0] + acc[1];
      part[((wave * GEMV_MT_TMAX + t) * 8 + 2 * rg + 1) * 16 + ar] = acc[2] + acc[3];
    }
  };
  auto finish = [&]() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if constexpr (SWIGLU) {
      for (u32 o = tid; o < 16u * tokens; o += GEMV_MT_WAVES * 64) {
        const u32 r = o & 15, m = o >> 4;
        float g = 0.f, u = 0.f;
#pragma unroll
        for (u32 k = 0; k < GEMV_MT_WAVES; k++) {
          g += part[((k * GEMV_MT_TMAX + 0) * NTOK + m) * 16 + r];
          u += part[((k * GEMV_MT_TMAX + 1) * NTOK + m) * 16 + r];
        }
        const u32 row = grp * 16 + r;
        if (row < a.rows[0]) a.out[0][(size_t)m * a.rows[0] + row] = swiglu_one(g, u);
      }
    } else {
      for (u32 o = tid; o < (u32)T * 16u * tokens; o += GEMV_MT_WAVES * 64) {
        const u32 r = o & 15, m = (o >> 4) % tokens, t = o / (16 * tokens);
        float v = 0.f;
#pragma unroll
        for (u32 k = 0; k < GEMV_MT_WAVES; k++) v += part[((k * GEMV_MT_TMAX + t) * NTOK + m) * 16 + r];
        const u32 row = (grp * T + t) * 16 + r;
        if constexpr (TOP1) {
          // (the groups a thread walks ascend, so do its rows: among equal values the first one stays; a row past the end
          // competes as minus infinity under the highest index)
          const bool real = row < a.rows[0];
          top1_take(top_v, top_i, real ? v : -__builtin_inff(), real ? row : 0xFFFFFFFFu);
        } else if (row < a.rows[0]) {
          const size_t oi = (size_t)m * a.rows[0] + row;
          if (residual) v += residual[oi];
          a.out[0][oi] = v;
        } else if (row < a.rows[0] + a.rows[1]) {
          a.out[1][(size_t)m * a.rows[1] + (row - a.rows[0])] = v;
        } else if (row < total_rows) {
          a.out[2][(size_t)m * a.rows[2] + (row - a.rows[0] - a.rows[1])] = v;
        }
      }
    }
  };
  auto between_groups = [&]() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();   // every partial sum has been read
    asm volatile("" ::: "memory");
  };

  if constexpr (!STREAM) {
    // ---- operands resident -------------------------------------------------------------------------------------------
#pragma unroll
    for (int i = 0; i < SBW; i++) issue_set(i, i);
    set_rows(grp);
#pragma unroll
    for (int i = 0; i < SBW; i++)
#pragma unroll
      for (int t = 0; t < T; t++) issue_unit(i, t, i * T + t);
    mt_wait<NC * NU>();   // the operands are older than the copies
    typename F::Aux ax[SBW];
#pragma unroll
    for (int i = 0; i < SBW; i++) {
      pin_set(i);
      ax[i] = F::aux(auxr[i]);
    }
    // One row group. `prefetch` (a compile-time tag) says that another group follows: a unit's slot is refilled with that
    // group's unit as soon as it has been read. The body has no branch of its own (one basic block for the scheduler).
    auto group = [&](auto prefetch) {
      constexpr bool walk = decltype(prefetch)::value;
      float acc[T][4];
#pragma unroll
      for (int t = 0; t < T; t++) acc[t][0] = acc[t][1] = acc[t][2] = acc[t][3] = 0.f;
      if constexpr (walk) set_rows(grp + gridDim.x);
      auto unit = [&](auto utag) {
        constexpr int u = decltype(utag)::value, i = u / T, t = u % T;
        __builtin_amdgcn_sched_barrier(0);   // (unit after unit: interleaved, their operands do not fit the register file)
        // the unit has landed when at most the copies behind it are outstanding: all NU - 1 other units while slots are
        // being refilled, else the ones after it in this group (other loads or stores in between only make the wait longer)
        mt_wait<walk ? NC * (NU - 1) : NC * (NU - 1 - u)>();
        const typename F::Raw w = F::read(slots + u * F::UNIT_BYTES + ar * (F::P * 16), kg);
        if constexpr (walk) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slot has been read
          issue_unit(i, t, u);
        }
        F::unit(w, breg[i], ax[i], acc[t]);
        // (pins the sums here: otherwise the compiler sinks this arithmetic towards its use behind the last unit, and the
        // results it reads stay live, or are spilled, until then)
        asm volatile("" : "+v"(acc[t][0]), "+v"(acc[t][1]), "+v"(acc[t][2]), "+v"(acc[t][3]));
      };
      unit(std::integral_constant<int, 0>{});
      if constexpr (NU > 1) unit(std::integral_constant<int, 1>{});
      if constexpr (NU > 2) unit(std::integral_constant<int, 2>{});
      if constexpr (NU > 3) unit(std::integral_constant<int, 3>{});
      if constexpr (NU > 4) unit(std::integral_constant<int, 4>{});
      if constexpr (NU > 5) unit(std::integral_constant<int, 5>{});
      static_assert(NU <= 6, "units per row group");
#pragma unroll
      for (int t = 0; t < T; t++) store_part(t, acc[t]);
      finish();
    };
    while (grp + gridDim.x < ngroups) {
      group(std::true_type{});
      grp += gridDim.x;
      between_groups();
    }
    group(std::false_type{});
  } else {
    // ---- operands streamed through two register sets, one tile per wavefront -----------------------------------------
    constexpr int S = SBW, NSLOT = F::NSLOT < S ? F::NSLOT : S;
    for (;;) {
#pragma unroll 1
     for (int mat = 0; mat < (SWIGLU ? 2 : 1); mat++) {
      set_rows(grp, mat);
#pragma unroll
      for (int u = 0; u < NSLOT; u++) {
        if (u < NS) issue_set(u, u);
        issue_unit(u, 0, u);
      }
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
      auto unit = [&](auto utag) {
        constexpr int i = decltype(utag)::value;
        __builtin_amdgcn_sched_barrier(0);
        mt_wait<mt_stream_wait(S, NSLOT, NS, NA, NC, i)>();
        pin_set(i % NS);
        const typename F::Aux ax = F::aux(auxr[i % NS]);
        const typename F::Raw w = F::read(slots + (i % NSLOT) * F::UNIT_BYTES + ar * (F::P * 16), kg);
        F::unit(w, breg[i % NS], ax, acc);
        asm volatile("" : "+v"(acc[0]), "+v"(acc[1]), "+v"(acc[2]), "+v"(acc[3]));
        __builtin_amdgcn_sched_barrier(0);
        // the set and the slot are free: the operands NS super-blocks on, and the unit NSLOT on
        if constexpr (i + NS < S) issue_set(i + NS, i % NS);
        if constexpr (i + NSLOT < S) {
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          issue_unit(i + NSLOT, 0, i % NSLOT);
        }
      };
      unit(std::integral_constant<int, 0>{});
      unit(std::integral_constant<int, 1>{});
      unit(std::integral_constant<int, 2>{});
      if constexpr (S > 3) unit(std::integral_constant<int, 3>{});
      if constexpr (S > 4) unit(std::integral_constant<int, 4>{});
      if constexpr (S > 5) unit(std::integral_constant<int, 5>{});
      static_assert(S <= 6, "super-blocks per k-slice");
      store_part(mat, acc);
     }
      finish();
      if (grp + gridDim.x >= ngroups) break;
      grp += gridDim.x;
      between_groups();
    }
  }
  if constexpr (TOP1) {
    // the threads' winners meet where the partial sums were: thread o held (tile o / (16 tokens), token (o / 16) % tokens,
    // row o % 16), so token m's candidates are the T runs of 16 threads from 16 (t tokens + m) on
    between_groups();
    u32* const cand_i = reinterpret_cast<u32*>(part + GEMV_MT_WAVES * 64);
    part[tid] = top_v;
    cand_i[tid] = top_i;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if ((u32)tid < tokens) {
      float best = -__builtin_inff();
      u32 best_id = 0xFFFFFFFFu;
      for (u32 t = 0; t < (u32)T; t++)
        for (u32 r = 0; r < 16; r++) {
          const u32 o = (t * tokens + (u32)tid) * 16 + r;
          top1_take(best, best_id, part[o], cand_i[o]);
        }
      a.out[0][(size_t)tid * gridDim.x + blockIdx.x] = best;
      top_ids[(size_t)tid * gridDim.x + blockIdx.x] = best_id;
    }
  }
}

// The tile count per wavefront follows from the row count (gemv_mt_tiles, the rule the host sizes the grid with); tile
// count and super-blocks per k-slice are template parameters so that register use and loads in flight are compile-time
// constants. Shapes outside gemv_mt_supported() must not be launched.
template <class F, bool TOP1 = false>
__device__ __forceinline__ void gemv_mt_dispatch(const MtArgs& a, const uint8_t* image, const float* residual, u32 in_dim, u32 tokens,
                                                 u32* top_ids = nullptr) {
  const u32 ntiles = (a.rows[0] + a.rows[1] + a.rows[2] + 15) >> 4;
  const u32 t = gemv_mt_tiles(F::TYPE, in_dim, ntiles);
  switch (gemv_mt_padded_sb(in_dim) >> 3) {
    case 1:
      if (t <= 1) gemv_mt_core<F, 1, 1, false, TOP1>(a, image, residual, in_dim, tokens, top_ids);
      else if (t == 2) gemv_mt_core<F, 1, 2, false, TOP1>(a, image, residual, in_dim, tokens, top_ids);
      else if constexpr (F::TMAX >= 3) gemv_mt_core<F, 1, 3, false, TOP1>(a, image, residual, in_dim, tokens, top_ids);
      break;
    case 2:
      if (t <= 1) gemv_mt_core<F, 2, 1, false, TOP1>(a, image, residual, in_dim, tokens, top_ids);
      else if (t == 2) gemv_mt_core<F, 2, 2, false, TOP1>(a, image, residual, in_dim, tokens, top_ids);
      else if constexpr (F::TMAX >= 3) gemv_mt_core<F, 2, 3, false, TOP1>(a, image, residual, in_dim, tokens, top_ids);
      break;
    case 3: gemv_mt_core<F, 3, 1, false, TOP1>(a, image, residual, in_dim, tokens, top_ids); break;
    case 4: gemv_mt_core<F, 4, 1, false, TOP1>(a, image, residual, in_dim, tokens, top_ids); break;
    case 5: gemv_mt_core<F, 5, 1, false, TOP1>(a, image, residual, in_dim, tokens, top_ids); break;
    default: gemv_mt_core<F, 6, 1, false, TOP1>(a, image, residual, in_dim, tokens, top_ids); break;
  }
}

#define GEMV_MT_ENTRY(NAME, FMT)                                                                                         \
  extern "C" __global__ __launch_bounds__(GEMV_MT_WAVES * 64) void NAME(                                                 \
      const uint8_t* w0, const uint8_t* w1, const uint8_t* w2, const uint8_t* image, const float* residual, float* out0, \
      float* out1, float* out2, u32 in_dim, u32 rows0, u32 rows1, u32 rows2, u32 tokens) {                               \
    const MtArgs a = {{w0, w1, w2}, {out0, out1, out2}, {rows0, rows1, rows2}};                                          \
    gemv_mt_dispatch<FMT>(a, image, residual, in_dim, tokens);                                                           \
  }
GEMV_MT_ENTRY(q4_k_gemv_mt_f32, MtQ4K)
GEMV_MT_ENTRY(q5_k_gemv_mt_f32, MtQ5K)
GEMV_MT_ENTRY(q6_k_gemv_mt_f32, MtQ6K)
GEMV_MT_ENTRY(q8_0_gemv_mt_f32, MtQ80)
// 9..16 tokens against the image of pack_x_mt16_q4k_f16 (activations as one binary16 term per token); same parameters,
// grid and block, dynamic shared memory gemv_mt_lds_bytes(type) + GEMV_MT_X16_LDS_EXTRA
GEMV_MT_ENTRY(q4_k_gemv_mt16_f32, MtQ4Kx16)
GEMV_MT_ENTRY(q5_k_gemv_mt16_f32, MtQ5Kx16)
GEMV_MT_ENTRY(q6_k_gemv_mt16_f32, MtQ6Kx16)
GEMV_MT_ENTRY(q8_0_gemv_mt16_f32, MtQ80x16)

// (w, image, partial_ids, partial_values, in_dim, out_dim, tokens): the output head's arg-max for 2..8 tokens in one pass
// over the weights. Grid, block and dynamic shared memory as q4_k_gemv_mt_f32 | q6_k_gemv_mt_f32 for out_dim rows;
// partial_*[token * gridDim.x + workgroup], finished by top1_reduce_f32 with count = gridDim.x. The one-token kernel's
// parameter order (src/ml/cuda/kernels/q6k_gemv_probe.ptx:1331-1338) with the image in the place of x and the token count
// behind.
#define GEMV_MT_TOP1_ENTRY(NAME, FMT)                                                                                    \
  extern "C" __global__ __launch_bounds__(GEMV_MT_WAVES * 64) void NAME(const uint8_t* w, const uint8_t* image,          \
                                                                        u32* partial_ids, float* partial_values,         \
                                                                        u32 in_dim, u32 out_dim, u32 tokens) {           \
    /* the absent matrices' row counts: a zero the optimizer cannot see through (with literal zeros it folds the lookup */ \
    /* of a row's matrix away, and this release of the compiler crashes in its control-flow simplification doing so)    */ \
    u32 none;                                                                                                            \
    asm volatile("s_mov_b32 %0, 0" : "=s"(none));                                                                        \
    const MtArgs a = {{w, w, w}, {partial_values, partial_values, partial_values}, {out_dim, none, none}};               \
    gemv_mt_dispatch<FMT, true>(a, image, nullptr, in_dim, tokens, partial_ids);                                         \
  }
GEMV_MT_TOP1_ENTRY(q4_k_gemv_mt_top1_partial_f32, MtQ4K)
GEMV_MT_TOP1_ENTRY(q6_k_gemv_mt_top1_partial_f32, MtQ6K)

// (w_gate, w_up, image, out, in_dim, out_dim, tokens): out[m][o] = silu(gate . x) * (up . x); block 512, grid = min(256,
// ceil(out_dim / 16)), dynamic shared memory as q4_k_gemv_mt_f32. The parameter list of q4_k_dual_gemv_swiglu_f32 with the
// image in the place of x and the token count behind.
template <class F>
__device__ __forceinline__ void gemv_mt_swiglu_dispatch(const uint8_t* w_gate, const uint8_t* w_up, const uint8_t* image, float* out,
                                                        u32 in_dim, u32 out_dim, u32 tokens) {
  const MtArgs a = {{w_gate, w_up, nullptr}, {out, nullptr, nullptr}, {out_dim, out_dim, 0u}};
  switch (gemv_mt_padded_sb(in_dim) >> 3) {
    case 1: gemv_mt_core<F, 1, 2, true>(a, image, nullptr, in_dim, tokens); break;
    case 2: gemv_mt_core<F, 2, 2, true>(a, image, nullptr, in_dim, tokens); break;
    case 3: gemv_mt_core<F, 3, 1, true>(a, image, nullptr, in_dim, tokens); break;
    case 4: gemv_mt_core<F, 4, 1, true>(a, image, nullptr, in_dim, tokens); break;
    case 5: gemv_mt_core<F, 5, 1, true>(a, image, nullptr, in_dim, tokens); break;
    default: gemv_mt_core<F, 6, 1, true>(a, image, nullptr, in_dim, tokens); break;
  }
}
extern "C" __global__ __launch_bounds__(GEMV_MT_WAVES * 64) void q4_k_gemv_mt_swiglu_f32(
    const uint8_t* w_gate, const uint8_t* w_up, const uint8_t* image, float* out, u32 in_dim, u32 out_dim, u32 tokens) {
  gemv_mt_swiglu_dispatch<MtQ4K>(w_gate, w_up, image, out, in_dim, out_dim, tokens);
}
// the same against the image of pack_x_mt16_q4k_f16, up to sixteen tokens (shared memory + GEMV_MT_X16_LDS_EXTRA)
extern "C" __global__ __launch_bounds__(GEMV_MT_WAVES * 64) void q4_k_gemv_mt16_swiglu_f32(
    const uint8_t* w_gate, const uint8_t* w_up, const uint8_t* image, float* out, u32 in_dim, u32 out_dim, u32 tokens) {
  gemv_mt_swiglu_dispatch<MtQ4Kx16>(w_gate, w_up, image, out, in_dim, out_dim, tokens);
}
