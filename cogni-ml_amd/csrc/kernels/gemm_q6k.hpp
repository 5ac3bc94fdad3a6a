// Prefill GEMM over raw Q6_K weights: out[m][n] = (bias[n] +) sum_k x[m][k] * deq(W[n][k]), M >= 9.
// Same tiling, operand layouts, x workspace format and epilogue as the Q4_K kernel (gemm_q4k.hpp): 128 tokens x 192
// rows per workgroup, 4 wavefronts = 2 row halves x 2 k-step halves, v_mfma_f32_32x32x16_f16 with fp32 accumulation,
// x as fp16 in LDS (two 64 KiB buffers filled by global_load_lds_dwordx4). What differs is the weight side:
//
//   pack_x_f16_q6k  (x:f32 [m][in_dim], xp:f16, m:u32, in_dim:u32)           block 256, grid ceil(m/128) * 16 * in_dim/256
//   q6_k_gemm_f16   (w_raw, xp, bias|null, out:f32 [m][out_dim], in_dim:u32, out_dim:u32, m:u32, bias_stride:u32; as q4_k_gemm_f16)
//                   block 256, grid 8 * ceil(ceil(m/128) * ceil(out_dim/192) / 8), no dynamic LDS (128 KiB static)
//
// A Q6_K super-block (210 bytes, 2-byte aligned: ql[128], qh[64], scales:i8[16], d:f16; src/ml/gguf/dequant.cr:197-236)
// is walked in the reference as two halves n of 128 values, each l in [0, 32) giving four values l, l+32, l+64, l+96
// ("quadrants") from the low / high nibbles of ql[l], ql[l+32] and two bits of qh[l]. Lane (j, kg) of a kh wavefront
// owns the 64-value group (n = kh, u = kg): l in [16u, 16u+16) of half n, i.e. the three 16-byte pieces
// ql[64n + 16u ..], ql[64n + 32 + 16u ..], qh[32n + 16u ..], the eight scale bytes of the half and d. All 39 KiB of raw
// bytes of 192 rows do not fit beside the two x buffers (160 KiB of LDS in all), so only ql does (128 of the 210 bytes:
// gemm_wbuf6, loaded one super-block ahead with consecutive lanes on consecutive pieces of a row, stored to LDS behind
// k-step 6 and picked up during k-step 7) and the 18 bytes of scales and d (gemm_wsc6, one row per thread); qh is read
// from global memory straight into the registers of the lane that decodes it, also one super-block ahead. Rows are only 2-byte aligned, and a 16-byte load
// from an odd multiple of 2 costs about twice an aligned one; the one-row-per-lane loads cost more again because a
// wavefront instruction touches 32 rows. The raw blocks of the 128-row tile (q6_k_gemm_n128_f16, q6_k_gemm_m64_n128_f16) do
// fit, and there they are copied whole, global -> LDS, without passing through registers (template parameter DMA below).
// k-step t of the wavefront is quadrant
// t / 2, bytes 8 (t % 2) .. +8 of the pieces: 8 values with one scale. A code is put together in the low bits of a
// half, (ql nibble) | (qh bits << 4) | 0x6400 = 1024 + q as binary16 (high nibbles are left in place, four bits up, beside
// 0x5400: 64 + q); subtracting 1056 (96) gives q - 32 exactly and one
// packed multiply gives fp16((q - 32) * (d * sc)). The 8 values come in byte order 0,2,1,3,4,6,5,7;
// pack_x_f16_q6k writes x accordingly (gemm_k_element_q6k).
#pragma once
#include "gemm_q4k.hpp"

// Element (0..255) of a super-block that k-slot (ks, kg, e) of the MFMA stands for: ks = 8 n + 2 qd + h8.
__device__ __forceinline__ u32 gemm_k_element_q6k(u32 ks, u32 kg, u32 e) {
  const u32 n = ks >> 3, qd = (ks >> 1) & 3, h8 = ks & 1;
  const u32 perm = ((e & 1) << 1) | ((e >> 1) & 1) | (e & 4);   // 0,2,1,3,4,6,5,7
  return 128 * n + 32 * qd + 16 * kg + 8 * h8 + perm;
}

extern "C" __global__ __launch_bounds__(256) void pack_x_f16_q6k(const float* x, uint4* xp, u32 m, u32 in_dim) {
  pack_x_core<true>(x, xp, m, in_dim);
}

struct GemmRaw6 {   // raw bytes of one group of one super-block of one weight row, as a lane sees them
  uint4 qa, qb, qh;
  uint2 sc;
  u32 d;
};

__device__ __forceinline__ u32 h2_sub_mul(u32 t, u32 off, u32 scale) {
  const __half2 q = __hadd2(*reinterpret_cast<const __half2*>(&t), *reinterpret_cast<const __half2*>(&off));
  const __half2 w = __hmul2(q, *reinterpret_cast<const __half2*>(&scale));
  return *reinterpret_cast<const u32*>(&w);
}

// ql of one super-block of the workgroup's 192 rows, [row][128 B + 16 B of padding]: staged by all lanes with consecutive
// lanes on consecutive 16-byte pieces of a row (8 rows per wavefront instruction), picked up by the lanes that decode it.
__shared__ uint4 gemm_wbuf6[GEMM_BN * 9];
// the 16 scale bytes and d of the same rows, [row][6 dwords]: staged one row per thread by the first three wavefronts
__shared__ u32 gemm_wsc6[GEMM_BN * 6];

// NT: tiles of 32 weight rows per wavefront - 3 (a workgroup tile of 128 tokens x 192 rows) or 2 (128 x 128: a third less
// work per workgroup for shapes whose 192-row tiles, times the k split, leave compute units idle - 4096 rows at 512 tokens
// are 88 tiles x 2 splits = 176 workgroups, but 128 x 2 = 256 of the smaller ones).
// MT: tiles of 32 tokens, 4 or 2 (launches of up to 64 tokens: q6_k_gemm_m64[_n128]_f16), as in gemm_k45_core.
// DMA (NT = 2 only): the whole 210-byte blocks of the 128 rows go global -> LDS without passing through registers, as the
// Q4_K kernel's do (global_load_lds_dwordx4 from the blocks' 2-byte-aligned addresses): a row is 15 pieces of 16 bytes in
// gemm_wbuf5 - bytes [16 p, 16 p + 16) for p < 13 (ql, qh, scales), bytes [194, 210) as piece 13 (d is its last two bytes)
// and a 15th that repeats piece 12, there so that a row is 60 dwords and the 16-byte reads of 16 consecutive rows fall on
// different banks. 1920 pieces = 30 copies of 64; every wavefront issues 8 (the last two repeat the tile's last piece into
// spare LDS), which with the two x buffers is all of the 160 KiB. With three row tiles (2880 pieces) this does not fit.
template <int NT, int MT = 4, bool DMA = false>
__device__ __forceinline__ void gemm_q6k_core(const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim,
                                              u32 m, u32 bias_stride) {
  static_assert(!DMA || NT == 2, "the raw blocks of 128 rows are what fits beside the x buffers");
  constexpr int NX = 4 * MT;   // copies of x per thread and super-block
  constexpr u32 BN = 64 * NT, NSTG = DMA ? 8 : 2 * NT;   // rows of the workgroup tile; 16-byte pieces a thread stages (DMA: copies) per super-block
  const u32 tid = threadIdx.x, lane = tid & 63;
  const u32 wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const u32 nh = wave & 1, kh = wave >> 1;
  const u32 j = lane & 31, kg = lane >> 5;
  // k split as in q4_k_gemm_f16: super-blocks [kb0, kb0 + nkb) into plane blockIdx.y behind `out`
  const u32 nkb_all = in_dim >> 8;
  const u32 kb0 = blockIdx.y * nkb_all / gridDim.y, nkb = (blockIdx.y + 1) * nkb_all / gridDim.y - kb0;
  out += (size_t)blockIdx.y * m * out_dim;
  const u32 mtiles = (m + GEMM_BM - 1) / GEMM_BM, ntiles = (out_dim + BN - 1) / BN;
  // workgroup -> tile as in q4_k_gemm_f16: XCD x takes a contiguous run of token-tile-major tiles
  u32 mt, nt;
  if (!gemm_tile_of(blockIdx.x, mtiles, ntiles, &mt, &nt)) return;
  const u32 n0 = nt * BN + nh * (32 * NT);           // first weight row of this wavefront
  const size_t row_bytes = (size_t)nkb_all * 210;

  // uniform base of the wavefront's rows + a 32-bit per-lane offset (96 rows are far below 4 GiB) to the lane's
  // piece of qh at 128 + 32 kh + 16 kg
  const u32 base_row = min(n0, out_dim - 1);
  const uint8_t* wbase = w + (size_t)base_row * row_bytes + (size_t)kb0 * 210;
  u32 rowoff[NT];
#pragma unroll
  for (int c = 0; c < NT; c++) rowoff[c] = (min(n0 + 32 * c + j, out_dim - 1) - base_row) * (u32)row_bytes;
  const u32 o_qh = 128 + 32 * kh + 16 * kg;
  // constants of the code assembly, kept in registers (as literals each (a & mask) | b would be two instructions)
  u32 mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x64006400u, magic_hi = 0x54005400u, m3_lo = 0x00300030u, m3_hi = 0x03000300u;
  asm volatile("" : "+v"(mask_lo), "+v"(mask_hi), "+v"(magic_lo), "+v"(magic_hi), "+v"(m3_lo), "+v"(m3_hi));
  const uint4* xtile = xp + ((size_t)mt * nkb_all + kb0) * 4096;

  float16_t acc[MT][NT];
#pragma unroll
  for (int r = 0; r < MT; r++)
#pragma unroll
    for (int c = 0; c < NT; c++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[r][c][v] = 0.0f;

  // staging of ql: piece p = 64 (4 i + wave) + lane, i < NSTG, is bytes [16 (p % 8), +16) of row p / 8 of the tile
  const u32 tile_row0 = min(nt * BN, out_dim - 1);
  const uint8_t* tbase = w + (size_t)tile_row0 * row_bytes + (size_t)kb0 * 210;   // uniform
  u32 soff[NSTG], sdst[NSTG];
#pragma unroll
  for (int i = 0; i < (int)NSTG; i++) {
    if constexpr (DMA) {
      const u32 p = min((4u * i + wave) * 64u + lane, BN * 15u - 1u), r = p / 15u, part = p - 15u * r;
      soff[i] = (min(nt * BN + r, out_dim - 1) - tile_row0) * (u32)row_bytes + (part < 13u ? 16u * part : (part == 13u ? 194u : 192u));
      sdst[i] = (4u * i + wave) * 64u;   // (the copy's LDS address is uniform: lane l lands 16 l bytes further)
    } else {
      const u32 p = (4u * i + wave) * 64u + lane, r = p >> 3, part = p & 7u;
      soff[i] = (min(nt * BN + r, out_dim - 1) - tile_row0) * (u32)row_bytes + 16u * part;
      sdst[i] = r * 9u + part;
    }
  }
  // DMA: piece 0 of the lane's row c = 0 in gemm_wbuf5 (row c is 32 * 15 pieces further)
  const u32 dbase = (nh * (32 * NT) + j) * 15;
  auto copy_w = [&](const uint8_t* kbase, int i) {
    __builtin_amdgcn_global_load_lds((gbl_void*)(kbase + soff[i]), (lds_void*)(gemm_wbuf5 + sdst[i]), 16, 0, 0);
  };
  auto take_raw = [&](GemmRaw6 (&raw)[NT]) {
#pragma unroll
    for (int c = 0; c < NT; c++) {
      const u32 b = dbase + 480 * c;
      raw[c].qa = gemm_wbuf5[b + 4 * kh + kg];
      raw[c].qb = gemm_wbuf5[b + 4 * kh + 2 + kg];
      raw[c].qh = gemm_wbuf5[b + 8 + 2 * kh + kg];
      raw[c].sc = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint8_t*>(gemm_wbuf5 + b + 12) + 8 * kh);
      raw[c].d = *reinterpret_cast<const uint16_t*>(reinterpret_cast<const uint8_t*>(gemm_wbuf5 + b + 13) + 14);
    }
  };
  const u32 take0 = (nh * (32 * NT) + j) * 9 + 4 * kh + kg;   // the lane's first ql piece of its row c = 0; the second is 2 further
  const u32 srow = (min(nt * BN + min(tid, BN - 1), out_dim - 1) - tile_row0) * (u32)row_bytes + 192u;
  const u32 tsc = (nh * (32 * NT) + j) * 6;                   // the lane's row c = 0 in gemm_wsc6
  uint4 stg[NSTG], stg_sc;
  u32 stg_d;
  auto stage_load = [&](const uint8_t* kbase, int i) { stg[i] = ld16(kbase + soff[i]); };
  auto stage_load_sc = [&](const uint8_t* kbase) {
    if (wave < (u32)NT) {   // one row per thread: the first BN threads
      stg_sc = ld16(kbase + srow);
      stg_d = ld2(kbase + (srow + 16));
    }
  };
  auto stage_store = [&]() {
#pragma unroll
    for (int i = 0; i < (int)NSTG; i++) gemm_wbuf6[sdst[i]] = stg[i];
    if (wave < (u32)NT) {
      *reinterpret_cast<uint2*>(&gemm_wsc6[tid * 6]) = make_uint2(stg_sc.x, stg_sc.y);
      *reinterpret_cast<uint2*>(&gemm_wsc6[tid * 6 + 2]) = make_uint2(stg_sc.z, stg_sc.w);
      gemm_wsc6[tid * 6 + 4] = stg_d;
    }
  };
  auto take_ql = [&](GemmRaw6 (&raw)[NT]) {
#pragma unroll
    for (int c = 0; c < NT; c++) {
      raw[c].qa = gemm_wbuf6[take0 + 288 * c];
      raw[c].qb = gemm_wbuf6[take0 + 288 * c + 2];
      raw[c].sc = *reinterpret_cast<const uint2*>(&gemm_wsc6[tsc + 192 * c + 2 * kh]);
      raw[c].d = gemm_wsc6[tsc + 192 * c + 4];
    }
  };

  // copy i of a super-block's x tile (as in gemm_k45_core: 128 tokens, or the first 64 of every chunk)
  auto x_copy = [&](const uint4* src, uint4* dst, int i) {
    if constexpr (MT == 4)
      __builtin_amdgcn_global_load_lds((gbl_void*)(src + 256 * i + tid), (lds_void*)(dst + 256 * i + wave * 64), 16, 0, 0);
    else
      __builtin_amdgcn_global_load_lds((gbl_void*)(src + (4 * i + wave) * 128 + lane), (lds_void*)(dst + (4 * i + wave) * 128), 16, 0, 0);
  };
  auto load_row = [&](GemmRaw6& raw, const uint8_t* kbase, int c) {
    raw.qh = ld16(kbase + (rowoff[c] + o_qh));
  };

  // Stage super-block 0 of x and the first weights. The main loop takes super-blocks in pairs with fixed roles (x
  // buffer 0 then 1, weight registers A then B); with an odd number of super-blocks the first one is taken alone
  // out of buffer 1 / registers B.
  const bool odd = nkb & 1;
  GemmRaw6 rawA[NT], rawB[NT];
  if constexpr (DMA) {
#pragma unroll
    for (int i = 0; i < (int)NSTG; i++) copy_w(tbase, i);
  } else {
#pragma unroll
    for (int i = 0; i < (int)NSTG; i++) stage_load(tbase, i);
    stage_load_sc(tbase);
  }
  if (odd) {
    if constexpr (!DMA) {
#pragma unroll
      for (int c = 0; c < NT; c++) load_row(rawB[c], wbase, c);
    }
#pragma unroll
    for (int i = 0; i < NX; i++) x_copy(xtile, gemm_xbuf1, i);
  } else {
    if constexpr (!DMA) {
#pragma unroll
      for (int c = 0; c < NT; c++) load_row(rawA[c], wbase, c);
    }
#pragma unroll
    for (int i = 0; i < NX; i++) x_copy(xtile, gemm_xbuf0, i);
  }
  if constexpr (!DMA) stage_store();
  __syncthreads();
  if constexpr (DMA) {
    if (odd) take_raw(rawB); else take_raw(rawA);
  } else {
    if (odd) take_ql(rawB); else take_ql(rawA);
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();   // gemm_wbuf6 is free for the next super-block
  asm volatile("" ::: "memory");

  auto iteration = [&](u32 kb, const uint4* xcur, uint4* xnxt, const GemmRaw6 (&cur)[NT], GemmRaw6 (&nxt)[NT]) {
    // d * sc of the four 16-value sub-blocks of the lane's group (scale bytes kg, kg + 2, kg + 4, kg + 6 of the
    // half's eight), as duplicated half2
    u32 S[NT][4];
#pragma unroll
    for (int c = 0; c < NT; c++) {
      const float d = h2f(cur[c].d);
      const u32 lo = cur[c].sc.x >> (8 * kg), hi = cur[c].sc.y >> (8 * kg);
      S[c][0] = h2_dup(d * (float)(int)(signed char)(lo & 0xFFu));
      S[c][1] = h2_dup(d * (float)(int)(signed char)((lo >> 16) & 0xFFu));
      S[c][2] = h2_dup(d * (float)(int)(signed char)(hi & 0xFFu));
      S[c][3] = h2_dup(d * (float)(int)(signed char)((hi >> 16) & 0xFFu));
    }
    const u32 kn = min(kb + 1, nkb - 1);   // the last iteration re-reads its own tile; the copy is not used
    const uint4* xnext = xtile + (size_t)kn * 4096;   // uniform
    const uint8_t* knbase = wbase + (size_t)kn * 210; // uniform
    const uint8_t* tnext = tbase + (size_t)kn * 210;  // uniform

    const uint4* arow = xcur + (16 * kh + kg) * 128 + j;   // k-steps 8*kh .. 8*kh+7; 32 lanes read 512 contiguous bytes
    auto build_b = [&](half8_t (&B)[NT], int t) {
      const int qd = t >> 1, h8 = t & 1, hi = qd >> 1;
#pragma unroll
      for (int c = 0; c < NT; c++) {
        const uint4 Q = (qd & 1) ? cur[c].qb : cur[c].qa;
        const u32 qa = h8 ? Q.z : Q.x, qb = h8 ? Q.w : Q.y;
        const u32 ha = h8 ? cur[c].qh.z : cur[c].qh.x, hb = h8 ? cur[c].qh.w : cur[c].qh.y;
        // low nibbles: 1024 + q with the code in mantissa bits 0..5, minus 1056; high nibbles stay where they are: 64 + q with
        // the code in mantissa bits 4..9 (one step is 1/16 there), minus 96 - q - 32 exactly either way. The two bits of qh
        // go beside the nibble (bits 4..5, or 8..9): for bytes 0 and 2 of a dword a left shift by 4 (quadrants 0, 2) or 2
        // (1, 3) puts them there, for bytes 1 and 3 a right shift by 4 or 6 - four shifted forms of a qh dword, each used by
        // two quadrants. Masks and offsets sit in registers so that (a & mask) | b is one v_and_or_b32.
        const u32 mask = hi ? mask_hi : mask_lo, magic = hi ? magic_hi : magic_lo, m3 = hi ? m3_hi : m3_lo;
        const u32 off = hi ? 0xD600D600u : 0xE420E420u;   // half2(-96) : half2(-1056)
        const int sl = (qd & 1) ? 2 : 4, sr = (qd & 1) ? 6 : 4;
        const u32 sc = S[c][qd];
        uint4 bw;
        // (the nibble halves are held as values of their own: left to itself the compiler merges the two steps into two
        // ands and a three-way or)
        u32 n0 = (qa & mask) | magic, n1 = ((qa >> 8) & mask) | magic, n2 = (qb & mask) | magic, n3 = ((qb >> 8) & mask) | magic;
        asm("" : "+v"(n0), "+v"(n1), "+v"(n2), "+v"(n3));
        bw.x = h2_sub_mul(((ha << sl) & m3) | n0, off, sc);
        bw.y = h2_sub_mul(((ha >> sr) & m3) | n1, off, sc);
        bw.z = h2_sub_mul(((hb << sl) & m3) | n2, off, sc);
        bw.w = h2_sub_mul(((hb >> sr) & m3) | n3, off, sc);
        B[c] = *reinterpret_cast<const half8_t*>(&bw);
      }
    };

    // software pipeline over the wavefront's eight k-steps: while the MFMAs of step t run, the A operands
    // of step t+1 are read from LDS and its B operands are built
    uint4 A[2][MT];
    half8_t B[2][NT];
#pragma unroll
    for (int r = 0; r < MT; r++) A[0][r] = arow[r * 32];
    build_b(B[0], 0);
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const int p = t & 1;
      // prefetches for the next super-block, a few per k-step: the raw weights of one row tile (5 loads) in each of
      // the first NT steps, the x tile global -> LDS spread over the first six
      if constexpr (DMA) {
        // the eight copies of the next super-block's raw blocks, two per k-step; they and the x copies are waited for
        // behind k-step 6, the lanes that decode them pick them up during k-step 7
        if (t < 4) {
          copy_w(tnext, 2 * t);
          copy_w(tnext, 2 * t + 1);
        }
        if (t == 7) take_raw(nxt);
      } else {
        if (t < NT) {
          stage_load(tnext, 2 * t);
          stage_load(tnext, 2 * t + 1);
          load_row(nxt[t], knbase, t);
        }
        if (t == 3) stage_load_sc(tnext);
        if (t == 6) stage_store();
        if (t == 7) take_ql(nxt);
      }
      if (t < 6) {
#pragma unroll
        for (int i = (t < 3 ? 2 * t : 3 * t - 3); i < (t < 3 ? 2 * t + 2 : (t < 5 ? 3 * t : 16)); i++)
          if (i < NX) x_copy(xnext, xnxt, i);
      }
      if (t < 7) {
#pragma unroll
        for (int r = 0; r < MT; r++) A[p ^ 1][r] = arow[(t + 1) * 256 + r * 32];
        build_b(B[p ^ 1], t + 1);
      }
#pragma unroll
      for (int r = 0; r < MT; r++) {
        const half8_t Ar = *reinterpret_cast<const half8_t*>(&A[p][r]);
#pragma unroll
        for (int c = 0; c < NT; c++) acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(B[p][c], Ar, acc[r][c], 0, 0, 0);
      }
      if (t < 7) {
#pragma unroll
        for (int c = 0; c < NT; c++) asm volatile("" : "+v"(B[p ^ 1][c]));
      }
      __builtin_amdgcn_sched_group_barrier(0x020, 10, 0);  // VMEM reads (weights, LDS-direct x) of this step
      __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);   // LDS reads: A operands of the next step
#pragma unroll
      for (int i = 0; i < MT * NT; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);   // eight VALU (a Q6_K operand takes more than a Q4_K one)
      }
      __builtin_amdgcn_sched_barrier(0);
      if (t == 6) {
        // the staged ql of the next super-block is complete once every wavefront's stores have landed (DMA: once every
        // wavefront's copies have)
        if constexpr (DMA) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // End of the iteration: everything this wavefront requested has to be there (the x tile for everybody, the
    // weights for its own next iteration) and its reads of the raw-weight buffer have to be done, then everybody meets.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  if (odd) iteration(0, gemm_xbuf1, gemm_xbuf0, rawB, rawA);
  for (u32 kb = odd; kb < nkb; kb += 2) {
    iteration(kb, gemm_xbuf0, gemm_xbuf1, rawA, rawB);
    iteration(kb + 1, gemm_xbuf1, gemm_xbuf0, rawB, rawA);
  }
  __syncthreads();   // drains the last (unused) prefetches before the buffers are reused below
  gemm_epilogue<NT, MT>(acc, bias, out, out_dim, m, mt, nt, nh, kh, j, kg, tid, bias_stride);
}

extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q6_k_gemm_f16(
    const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim, u32 m, u32 bias_stride) {
  gemm_q6k_core<3>(w, xp, bias, out, in_dim, out_dim, m, bias_stride);
}
// up to 64 tokens, tiles of 64 x 192 and 64 x 128
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q6_k_gemm_m64_f16(
    const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim, u32 m, u32 bias_stride) {
  gemm_q6k_core<3, 2>(w, xp, bias, out, in_dim, out_dim, m, bias_stride);
}
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q6_k_gemm_m64_n128_f16(
    const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim, u32 m, u32 bias_stride) {
  gemm_q6k_core<2, 2, true>(w, xp, bias, out, in_dim, out_dim, m, bias_stride);
}
// the same with a workgroup tile of 128 tokens x 128 rows (whole blocks copied global -> LDS); grid from
// gemm_grid_x(ceil(m/128), ceil(out_dim/128))
extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q6_k_gemm_n128_f16(
    const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim, u32 m, u32 bias_stride) {
  gemm_q6k_core<2, 4, true>(w, xp, bias, out, in_dim, out_dim, m, bias_stride);
}
