// Decode GEMV on the matrix cores for M = 3, 4 tokens, Q6_K: out[m][o] = (residual[m][o] +) sum_j x[m][j] * deq(W[o][j]).
//
// Same kernel ABI, launch geometry and work split as the Q4_K kernel in gemv_mfma.hpp (block = 8 wavefronts = k-slices x
// row groups, 16-row tiles, activations as binary16 hi + lo pairs in LDS, partial sums added in a fixed order); dynamic
// shared memory from gemv_mfma_lds_bytes(14, ...). What differs is the block format (210 B: ql[128], qh[64],
// scales:i8[16], d:f16 - src/ml/gguf/dequant.cr:195-236):
//
// * A value is (ql nibble | qh two bits << 4) - 32 times d * sc, one int8 scale per 16 values. Sixteen consecutive ql
//   bytes hold one 16-value sub-block in their low nibbles and another in their high nibbles, so the lanes kg = 0, 1
//   of a row take the two 8-byte halves of one such run and kg = 2, 3 those of the run 32 bytes further on (the
//   other two quadrants of the same l range): an MFMA of 32 k values then meets two sub-blocks, one per lane pair,
//   and the 16 columns are (slot = lane pair, token, hi/lo) - two slots, up to four tokens.
// * Codes stay exact: (ql & 0x000F000F) | (qh bits << 4) read as two binary16 numbers is code * 2^-24; the high
//   nibbles are left where they are, (ql & 0x00F000F0) | (qh bits << 8) = code * 2^-20. About 15 vector
//   instructions per ql dword (four operand dwords).
// * Every MFMA has its own pair of scales, so each of the 8 per super-block and tile gets its own accumulator tile,
//   folded into the row sums with d * sc and the -32 * sum(x) term right away. The lanes that hold the scale bytes
//   (A layout: row, four scales each) hand d * sc to the accumulator layout through a wave-private LDS buffer.
//
// Rows are only 2-byte aligned (210-byte blocks): all weight loads are 8, 4 or 2 bytes at any alignment.
#pragma once
#include "common.hpp"
#include "gemv_config.h"
#include "gemv_mfma.hpp"

// TOP1: instead of the row values a workgroup stores, per token, the largest of all its rows and that row's index
// (out[token * gridDim.x + blockIdx.x], top_ids[...]: the layout of the vector-ALU top-1 kernels, finished by
// top1_reduce_f32); of equal values the lowest row wins.
template <int M, bool ADD, int T, bool CHUNK = false, bool TOP1 = false>
__device__ __forceinline__ void q6k_gemv_mfma_core(const uint8_t* w, const float* x, const float* residual,
                                                   float* out, u32 in_dim, u32 out_dim, u32* top_ids = nullptr) {
  static_assert(!TOP1 || !ADD, "TOP1 is a mode of the plain GEMV");
  constexpr int MP = 4;                               // token slots in the column index: (slot 2, token 4, hi/lo 2)
  constexpr int BB = 210;
  constexpr int NPRE = GEMV_MFMA_MAX_UNITS(M) / GEMV_MFMA_WAVES;   // staging units (token, super-block) per wavefront
  constexpr int C = NPRE / M;                                      // CHUNK: super-blocks of a k-slice staged at a time
  extern __shared__ uint4 mf_lds4[];
  char* lds = reinterpret_cast<char*>(mf_lds4);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const u32 nsb = in_dim >> 8;
  const u32 lg_nwk = gemv_mfma_log2_kslices(nsb);
  const u32 NWK = 1u << lg_nwk, NWR = GEMV_MFMA_WAVES >> lg_nwk;
  const u32 kslice = wave & (NWK - 1), rgrp = wave >> lg_nwk;
  const u32 ntiles = (out_dim + 15) >> 4;
  // A workgroup takes the row groups (NWR * T tiles each) blockIdx.x, blockIdx.x + gridDim.x, ... with the activations
  // staged once: a matrix with more groups than compute units (an output head) is launched as one workgroup per unit.
  const u32 ngroups = (ntiles + NWR * T - 1) / (NWR * T);
  u32 grp = blockIdx.x;

  // LDS map (gemv_mfma_lds_bytes): zero[64] | handover[waves][TMAX][16 sub-blocks][16 rows] f32
  //                                | partial[waves][TMAX][MP][16] f32 | fs[units] f32 | sx[units][16] f32
  //                                | ximg[units][2][256] f16
  const u32 off_tb = 64 + (u32)wave * (GEMV_MFMA_TMAX * 1024);
  const u32 off_part = 64 + GEMV_MFMA_WAVES * GEMV_MFMA_TMAX * 1024;
  const u32 off_fs = off_part + GEMV_MFMA_WAVES * GEMV_MFMA_TMAX * MP * 64;
  const u32 units_lds = CHUNK ? (u32)(GEMV_MFMA_WAVES * C * M) : (u32)M * nsb;
  const u32 off_sx = off_fs + units_lds * 4;
  const u32 off_x = off_sx + units_lds * 64;
  auto xslot = [&](u32 sb) -> u32 { return CHUNK ? (u32)wave * C + ((sb >> 3) % (u32)C) : sb; };
  auto uidx = [&](u32 m, u32 sb) -> u32 { return CHUNK ? xslot(sb) * M + m : m * nsb + sb; };
  if (tid < 16) reinterpret_cast<u32*>(lds)[tid] = 0u;

  // ---- lane roles -------------------------------------------------------------------------------
  // A layout: row ar of the tile; kg & 1 = which 8 bytes of a 16-byte run, kg >> 1 = which pair of quadrants
  const u32 ar = lane & 15, kg = lane >> 4;
  const u32 qp = kg >> 1, hb = kg & 1;
  const u32 hshift = 2 * qp;   // quadrants 0 / 2 sit in qh bits 0-1 / 4-5, quadrants 1 / 3 two bits higher
  // D / B layout: column c = (slot, token, hi/lo)
  const u32 c = lane & 15, rg = lane >> 4;
  const u32 hl = c & 1, tok = (c >> 1) & (MP - 1), slot = c / (2 * MP);
  const bool col_live = tok < (u32)M;

  const size_t row_bytes = (size_t)nsb * BB;
  const uint8_t* rowp[T];
  auto set_rows = [&](u32 g) {
    const u32 tile0 = (g * NWR + rgrp) * T;
#pragma unroll
    for (int t = 0; t < T; t++) {
      const u32 tile = min(tile0 + (u32)t, ntiles - 1);
      rowp[t] = w + (size_t)min(tile * 16 + ar, out_dim - 1) * row_bytes;
    }
  };
  set_rows(grp);

  // per tile and super-block: four 8-byte pieces of ql and of qh (half n, l range a), the lane's four scale bytes, d
  struct Stage { uint2 ql[4], qh[4]; u32 sc, d; };
  Stage stA[T];
  auto load_sb = [&](Stage* st, u32 sb) {
    const u32 off = sb * BB;
#pragma unroll
    for (int t = 0; t < T; t++) {
#pragma unroll
      for (int na = 0; na < 4; na++) {
        const u32 n = na >> 1, a = na & 1;
        st[t].ql[na] = ld8(rowp[t] + (off + 64 * n + 32 * qp + 16 * a + 8 * hb));
        st[t].qh[na] = ld8(rowp[t] + (off + 128 + 32 * n + 16 * a + 8 * hb));
      }
      st[t].sc = ld4(rowp[t] + (off + 192 + 4 * kg));
      st[t].d = ld2(rowp[t] + (off + 208));
    }
  };

  const u32 nunits = (u32)M * nsb;
  auto unit_of = [&](int i, u32 i0, u32& m, u32& sb) -> bool {
    if constexpr (CHUNK) {
      const u32 j = (u32)(i % C);
      m = (u32)(i / C);
      sb = kslice + 8u * (i0 + j);
      return i < C * M && i0 + j < (nsb >> 3);
    } else {
      const u32 p = (u32)wave + (u32)i * GEMV_MFMA_WAVES;
      m = p / nsb;
      sb = p - m * nsb;
      return p < nunits;
    }
  };
  float4 xv[NPRE];
  auto load_xv = [&](u32 i0) {
#pragma unroll
    for (int i = 0; i < NPRE; i++) {
      u32 m, sb;
      if (unit_of(i, i0, m, sb)) __builtin_memcpy(&xv[i], x + (size_t)m * in_dim + (size_t)sb * 256 + 4 * lane, 16);
    }
  };
  // activations first, by every wavefront, then the weights: the memory pipeline returns loads in order
  load_xv(0);
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
  load_sb(stA, kslice);

  mf_float4 acc[T];
  float run_best = -__builtin_inff();   // TOP1: wavefront m keeps token m's best over the row groups it has seen
  u32 run_id = 0xFFFFFFFFu;

  // ---- stage the activations: one wavefront per (token, super-block) -----------------------------------
  auto stage_xv = [&](u32 i0) {
#pragma unroll
    for (int i = 0; i < NPRE; i++) {
      u32 m, sb;
      if (unit_of(i, i0, m, sb)) {
        const float4 v = xv[i];
        // power of two that brings the largest magnitude of the super-block to [2^12, 2^13)
        // (unsigned maximum of the bit patterns without sign: orders magnitudes like the floats, and its DPP steps are
        // single instructions)
        u32 ab = __builtin_bit_cast(u32, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        ab = max(ab, MF_DPP_U(ab, MF_DPP_QUAD_1032));
        ab = max(ab, MF_DPP_U(ab, MF_DPP_QUAD_2301));
        ab = max(ab, MF_DPP_U(ab, MF_DPP_ROW_ROR4));
        ab = max(ab, MF_DPP_U(ab, MF_DPP_ROW_ROR8));
        const u32 ab4 = max(max((u32)__builtin_amdgcn_readlane((int)ab, 0), (u32)__builtin_amdgcn_readlane((int)ab, 16)),
                            max((u32)__builtin_amdgcn_readlane((int)ab, 32), (u32)__builtin_amdgcn_readlane((int)ab, 48)));
        const int e = (int)((ab4 >> 23) & 0xFFu);
        int sh = 139 - e;                      // scale = 2^sh
        sh = sh > 126 ? 126 : sh;              // zeros / subnormal values: 2^sh and 2^-sh stay normal numbers
        const float scale = __builtin_bit_cast(float, (u32)(127 + sh) << 23);
        const float inv = __builtin_bit_cast(float, (u32)(127 - sh) << 23);
        const float s0 = v.x * scale, s1 = v.y * scale, s2 = v.z * scale, s3 = v.w * scale;
        const _Float16 h0 = (_Float16)s0, h1 = (_Float16)s1, h2 = (_Float16)s2, h3 = (_Float16)s3;
        // (x * scale is exact, so fma(x, scale, -hi) is the same value as (x * scale) - hi, in one mixed-precision instruction)
        const _Float16 l0 = (_Float16)fmaf(v.x, scale, -(float)h0), l1 = (_Float16)fmaf(v.y, scale, -(float)h1),
                       l2 = (_Float16)fmaf(v.z, scale, -(float)h2), l3 = (_Float16)fmaf(v.w, scale, -(float)h3);
        // k-slot order inside a run of 8 weights is 0,2,1,3,4,6,5,7 (how the nibble masks deliver them)
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        const h4 hv = {h0, h2, h1, h3}, lv = {l0, l2, l1, l3};
        char* img = lds + off_x + ((size_t)(xslot(sb) * M + m) * 2) * 512 + 8 * lane;
        *reinterpret_cast<h4*>(img) = hv;
        *reinterpret_cast<h4*>(img + 512) = lv;
        // sums of the 16 sub-blocks (4 lanes each) for the -32 term, unscaled
        float sm = (v.x + v.y) + (v.z + v.w);
        sm += MF_DPP(sm, MF_DPP_QUAD_1032);
        sm += MF_DPP(sm, MF_DPP_QUAD_2301);
        // (every lane of a quad holds the quad's sum, every lane the scale: stored by all of them, no lane masks)
        reinterpret_cast<float*>(lds + off_sx)[uidx(m, sb) * 16 + (lane >> 2)] = sm;
        reinterpret_cast<float*>(lds + off_fs)[uidx(m, sb)] = inv;
      }
    }
  };
  stage_xv(0);
  if (CHUNK || (NWR == 1 && (nsb & 7u) == 0)) {
    // every wavefront reads only what it staged itself; the zero words are wavefront 0's: rewrite them here
    if (wave != 0) {
      if (lane < 16) reinterpret_cast<u32*>(lds)[lane] = 0u;
    }
    wave_lds_fence();
  } else {
    __syncthreads();
  }

  // one super-block of the k-slice; with refill a tile's stage is reloaded with super-block refill_sb as soon as
  // its MFMAs are issued
  auto process = [&](Stage* st, u32 sb, u32 refill_sb, auto refill) {
    // B operands of the 8 MFMAs q = (n, a, lohi): the lane's 8 k values are elements
    // 128 n + 32 (qp + 2 lohi) + 16 a + 8 hb + (0..7) of the super-block; live iff the column's slot is the lane pair qp
    uint4 breg[8];
    const u32 ximg = off_x + ((xslot(sb) * M + tok) * 2 + hl) * 512;
    const bool live = col_live && slot == qp;
#pragma unroll
    for (int q = 0; q < 8; q++) {
      const u32 n = q >> 2, a = (q >> 1) & 1, lohi = q & 1;
      const u32 e0 = 128 * n + 32 * (qp + 2 * lohi) + 16 * a + 8 * hb;
      breg[q] = *reinterpret_cast<const uint4*>(lds + (live ? ximg + 2 * e0 : 0u));
    }
    // what the lane's column needs of the activations: 2^-e and -32 * sum(x) of the 8 sub-blocks it meets,
    // s = 8 n + 4 lohi + 2 slot + a
    float fsc = 0.f, m32sx[8];
#pragma unroll
    for (int q = 0; q < 8; q++) m32sx[q] = 0.f;
    if (col_live) {
      fsc = reinterpret_cast<const float*>(lds + off_fs)[uidx(tok, sb)];
      if (hl == 0) {
        const float* sxp = reinterpret_cast<const float*>(lds + off_sx) + uidx(tok, sb) * 16 + 2 * slot;
#pragma unroll
        for (int q = 0; q < 8; q++) {
          const u32 n = q >> 2, a = (q >> 1) & 1, lohi = q & 1;
          m32sx[q] = -32.0f * sxp[8 * n + 4 * lohi + a];
        }
      }
    }
    const float fsc24 = fsc * TWO_P24, fsc20 = fsc * TWO_P20;
    float* tb = reinterpret_cast<float*>(lds + off_tb);
    // (a) d * sc of sub-blocks 4 kg .. 4 kg + 3 of row ar into the handover buffer [tile][sub-block][row]
#pragma unroll
    for (int t = 0; t < T; t++) {
      const float dd = h2f(st[t].d);
      const u32 s4 = st[t].sc;
      tb[t * 256 + (4 * kg + 0) * 16 + ar] = dd * (float)(int)(signed char)(s4 & 0xFFu);
      tb[t * 256 + (4 * kg + 1) * 16 + ar] = dd * (float)(int)(signed char)((s4 >> 8) & 0xFFu);
      tb[t * 256 + (4 * kg + 2) * 16 + ar] = dd * (float)(int)(signed char)((s4 >> 16) & 0xFFu);
      tb[t * 256 + (4 * kg + 3) * 16 + ar] = dd * (float)(int)(signed char)(s4 >> 24);
    }
    wave_lds_fence();
#pragma unroll
    for (int t = 0; t < T; t++) {
      // (b) the 8 MFMAs of the tile, each into its own accumulator tile; (c) a pair is folded into the row sums while
      // the next pair is in the matrix cores (two pairs of accumulator tiles live, not four): rows 4 rg .. 4 rg + 3 of
      // the column's sub-block s = 8 n + 4 lohi + 2 slot + a
      auto fold = [&](int q, const mf_float4& dq) {
        const u32 n = q >> 2, a = (q >> 1) & 1, lohi = q & 1;
        const u32 s = 8 * n + 4 * lohi + 2 * slot + a;
        const float4 sv = *reinterpret_cast<const float4*>(tb + t * 256 + s * 16 + 4 * rg);
        const float f = lohi ? fsc20 : fsc24;
        acc[t][0] = fmaf(sv.x, fmaf(f, dq[0], m32sx[q]), acc[t][0]);   // d sc (2^-e sum(code x) - 32 sum(x))
        acc[t][1] = fmaf(sv.y, fmaf(f, dq[1], m32sx[q]), acc[t][1]);
        acc[t][2] = fmaf(sv.z, fmaf(f, dq[2], m32sx[q]), acc[t][2]);
        acc[t][3] = fmaf(sv.w, fmaf(f, dq[3], m32sx[q]), acc[t][3]);
      };
      mf_float4 dp0 = (mf_float4){0.f, 0.f, 0.f, 0.f}, dp1 = dp0;
#pragma unroll
      for (int na = 0; na < 4; na++) {
        // The two qh bits of a code go to bits 4, 5 of its 16-bit half (beside a low nibble) or 8, 9 (above a high
        // nibble left in place). For bytes 0 and 2 of a dword that is one left shift by 4 - hshift, for bytes 1 and 3
        // one right shift by 4 + hshift; the masks pick the quadrant's pair out of either.
        const uint2 q = st[t].ql[na];
        const u32 hax = st[t].qh[na].x << (4 - hshift), hay = st[t].qh[na].x >> (4 + hshift);
        const u32 hbx = st[t].qh[na].y << (4 - hshift), hby = st[t].qh[na].y >> (4 + hshift);
        const u32 qa8 = q.x >> 8, qb8 = q.y >> 8;
        uint4 lo, hi;
        lo.x = (q.x & 0x000F000Fu) | (hax & 0x00300030u);
        lo.y = (qa8 & 0x000F000Fu) | (hay & 0x00300030u);
        lo.z = (q.y & 0x000F000Fu) | (hbx & 0x00300030u);
        lo.w = (qb8 & 0x000F000Fu) | (hby & 0x00300030u);
        hi.x = (q.x & 0x00F000F0u) | (hax & 0x03000300u);
        hi.y = (qa8 & 0x00F000F0u) | (hay & 0x03000300u);
        hi.z = (q.y & 0x00F000F0u) | (hbx & 0x03000300u);
        hi.w = (qb8 & 0x00F000F0u) | (hby & 0x03000300u);
        const mf_float4 zero = (mf_float4){0.f, 0.f, 0.f, 0.f};
        const mf_float4 d0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(mf_half8, lo),
                                                                    __builtin_bit_cast(mf_half8, breg[2 * na]), zero, 0, 0, 0);
        const mf_float4 d1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(mf_half8, hi),
                                                                    __builtin_bit_cast(mf_half8, breg[2 * na + 1]), zero, 0, 0, 0);
        if (na > 0) {
          fold(2 * na - 2, dp0);
          fold(2 * na - 1, dp1);
        }
        dp0 = d0;
        dp1 = d1;
      }
      if constexpr (decltype(refill)::value) {
        // this tile's stage is free: request its next super-block
        const u32 off = refill_sb * BB;
#pragma unroll
        for (int na = 0; na < 4; na++) {
          const u32 n = na >> 1, a = na & 1;
          st[t].ql[na] = ld8(rowp[t] + (off + 64 * n + 32 * qp + 16 * a + 8 * hb));
          st[t].qh[na] = ld8(rowp[t] + (off + 128 + 32 * n + 16 * a + 8 * hb));
        }
        st[t].sc = ld4(rowp[t] + (off + 192 + 4 * kg));
        st[t].d = ld2(rowp[t] + (off + 208));
      }
      fold(6, dp0);
      fold(7, dp1);
    }
    wave_lds_fence();
  };

  for (;;) {
#pragma unroll
  for (int t = 0; t < T; t++) acc[t] = (mf_float4){0.f, 0.f, 0.f, 0.f};
  if constexpr (!CHUNK) {
    u32 sb = kslice;
    for (; sb + NWK < nsb; sb += NWK) process(stA, sb, sb + NWK, mf_true{});
    process(stA, sb, 0, mf_false{});
  } else {
    const u32 nslice = nsb >> 3;   // super-blocks of a k-slice: kslice, kslice + 8, ...
    for (u32 i0 = 0;;) {
      const bool more = i0 + C < nslice;
      if (more) load_xv(i0 + C);   // behind the weights in flight, ahead of the ones process() requests
      const u32 iend = min(i0 + (u32)C, nslice);
      for (u32 i = i0; i < iend; i++) {
        const u32 sb = kslice + 8u * i;
        if (i + 1 < nslice) process(stA, sb, sb + 8u, mf_true{});
        else process(stA, sb, 0, mf_false{});
      }
      if (!more) break;
      i0 += C;
      stage_xv(i0);
      wave_lds_fence();
    }
  }

  const u32 next = grp + gridDim.x;
  const bool walk = !CHUNK && next < ngroups;   // (rows staged in chunks: one group per workgroup)
  // ---- add up the columns of a token inside the wavefront, then the k-slices through LDS ------------
#pragma unroll
  for (int t = 0; t < T; t++) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      float v = acc[t][i];
      v += MF_DPP(v, MF_DPP_QUAD_1032);                   // hi + lo
      v += MF_DPP(v, MF_DPP_ROW_ROR8);                    // the two slots: column bit 3
      acc[t][i] = v;
    }
  }
  float* part = reinterpret_cast<float*>(lds + off_part);
  if (slot == 0 && hl == 0 && col_live) {
#pragma unroll
    for (int t = 0; t < T; t++)
      *reinterpret_cast<mf_float4*>(part + ((wave * GEMV_MFMA_TMAX + t) * MP + tok) * 16 + 4 * rg) = acc[t];
  }
  __syncthreads();
  const u32 nout = NWR * T * 16 * M;
  const u32 group_rows = NWR * T * 16;
  float* tv = reinterpret_cast<float*>(lds + 64);   // TOP1: the group's row values [token][row in group], in the handover space
  for (u32 o = tid; o < nout; o += GEMV_MFMA_WAVES * 64) {
    const u32 r = o & 15, m = (o >> 4) % M, tt = (o / (16 * M)) % T, rgp = o / (16 * M * T);
    float v = 0.f;
    for (u32 k = 0; k < NWK; k++) v += part[(((rgp << lg_nwk) + k) * GEMV_MFMA_TMAX + tt) * MP * 16 + m * 16 + r];
    const u32 row = ((grp * NWR + rgp) * T + tt) * 16 + r;
    if constexpr (TOP1) {
      tv[m * group_rows + (rgp * T + tt) * 16 + r] = v;
    } else if (row < out_dim) {
      const size_t oi = (size_t)m * out_dim + row;
      if (ADD) v += residual[oi];
      out[oi] = v;
    }
  }
  if constexpr (TOP1) {
    __syncthreads();
    if (wave < M) {
      const u32 row_base = grp * group_rows;
      float best = -__builtin_inff();
      u32 best_id = 0xFFFFFFFFu;
      for (u32 i = lane; i < group_rows; i += 64)
        if (row_base + i < out_dim) top1_take(best, best_id, tv[(u32)wave * group_rows + i], row_base + i);
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const float ov = __shfl_xor(best, d, 64);
        const u32 oi = (u32)__shfl_xor((int)best_id, d, 64);
        top1_take(best, best_id, ov, oi);
      }
      top1_take(run_best, run_id, best, best_id);
    }
  }
  if (!walk) break;
  grp = next;
  set_rows(grp);
  load_sb(stA, kslice);
  __syncthreads();   // every partial sum has been read
  }
  if constexpr (TOP1) {
    if (wave < M && lane == 0) {
      out[(size_t)wave * gridDim.x + blockIdx.x] = run_best;
      top_ids[(size_t)wave * gridDim.x + blockIdx.x] = run_id == 0xFFFFFFFFu ? 0u : run_id;
    }
  }
}

template <int M, bool ADD, bool TOP1 = false>
__device__ __forceinline__ void q6k_gemv_mfma_dispatch(const uint8_t* w, const float* x, const float* residual,
                                                       float* out, u32 in_dim, u32 out_dim, u32* top_ids = nullptr) {
  const u32 nsb = in_dim >> 8;
  const u32 lg = gemv_mfma_log2_kslices(nsb);
  const u32 nwr = GEMV_MFMA_WAVES >> lg;
  const u32 ntiles = (out_dim + 15) >> 4;
  const u32 t = (ntiles + gridDim.x * nwr - 1) / (gridDim.x * nwr);
  if (gemv_mfma_chunked(M, in_dim)) {
    if (t <= 1) q6k_gemv_mfma_core<M, ADD, 1, true, TOP1>(w, x, residual, out, in_dim, out_dim, top_ids);
    else if (t == 2) q6k_gemv_mfma_core<M, ADD, 2, true, TOP1>(w, x, residual, out, in_dim, out_dim, top_ids);
    else q6k_gemv_mfma_core<M, ADD, 3, true, TOP1>(w, x, residual, out, in_dim, out_dim, top_ids);
    return;
  }
  if (t <= 1) q6k_gemv_mfma_core<M, ADD, 1, false, TOP1>(w, x, residual, out, in_dim, out_dim, top_ids);
  else if (t == 2) q6k_gemv_mfma_core<M, ADD, 2, false, TOP1>(w, x, residual, out, in_dim, out_dim, top_ids);
  else q6k_gemv_mfma_core<M, ADD, 3, false, TOP1>(w, x, residual, out, in_dim, out_dim, top_ids);
}

#define GEMV_MFMA_Q6K_ENTRY(NAME, M)                                                                          \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(const uint8_t* w, const float* x,   \
                                                                         float* out, u32 in_dim, u32 out_dim) { \
    q6k_gemv_mfma_dispatch<M, false>(w, x, nullptr, out, in_dim, out_dim);                                    \
  }
#define GEMV_MFMA_Q6K_ADD_ENTRY(NAME, M)                                                                      \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(const uint8_t* w, const float* x,   \
                                                                         const float* residual, float* out,   \
                                                                         u32 in_dim, u32 out_dim) {           \
    q6k_gemv_mfma_dispatch<M, true>(w, x, residual, out, in_dim, out_dim);                                    \
  }
#define GEMV_MFMA_Q6K_TOP1_ENTRY(NAME, M)                                                                      \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(const uint8_t* w, const float* x,    \
                                                                         u32* partial_ids, float* partial_values, \
                                                                         u32 in_dim, u32 out_dim) {            \
    q6k_gemv_mfma_dispatch<M, false, true>(w, x, nullptr, partial_values, in_dim, out_dim, partial_ids);       \
  }
