// Decode GEMV on the matrix cores for M = 1..4 tokens, Q4_K: out[m][o] = (residual[m][o] +) sum_j x[m][j] * deq(W[o][j]).
//
// Same kernel ABI as the vector-ALU GEMV (gemv.hpp): (w_raw, x, [residual,] out, in_dim, out_dim), x rows at
// stride in_dim, out/residual rows at stride out_dim. Launch: block = 512 threads (8 wavefronts), grid and
// dynamic shared memory from gemv_config.h (gemv_mfma_grid, gemv_mfma_lds_bytes).
//
// Why the matrix cores for a matrix-vector product: the vector ALU needs one fused multiply-add per weight
// on top of the unpacking, and at one wavefront instruction per four clocks that, not HBM, bounds the
// kernel. v_mfma_f32_16x16x32_f16 takes the multiply-adds away: 16 weight rows x 32 weights per
// instruction, with the weights still exact - a masked pair of 4-bit codes read as two binary16 numbers is
// code * 2^-24 (or code * 2^-20 for the high nibbles, left in place), subnormals are honoured by the
// matrix cores, and the accumulator is fp32.
//
// Operands. A (16 rows x 32 k): lane (r = lane % 16, kg = lane / 16) supplies 8 weights of row r. The lane
// loads 16 bytes qs[16 (kg + 4 j)) .. +16) of its row and super-block (j = 0, 1): four MFMAs per load
// (low / high nibbles of bytes 0-7 and of bytes 8-15), no cross-lane movement, 5 VALU per dword.
// B (32 k x 16 columns): the activations as binary16, split hi + lo (x * 2^e = hi + lo to 22 bits, e per
// token and super-block so that any fp32 range fits binary16), staged once per workgroup in LDS.
// With 16-byte loads lanes kg = 0,1 and kg = 2,3 hold different 32-weight sub-blocks (different scales), so
// the sub-blocks must not meet in one accumulator entry: the 16 columns are used as (slot, token, hi/lo)
// and a lane's B operand is the activations only where its column's slot matches the sub-block the lane's
// kg feeds, zero elsewhere. M = 1: 8 slots, one accumulator tile holds all 8 sub-blocks of a super-block;
// M = 2: 4 slots, 2 tiles; M = 3, 4: 2 slots, 4 tiles. The MFMA count (8 per 16 rows x 256 weights) does
// not depend on M.
// D (16 x 16 fp32): lane (c = lane % 16, rg = lane / 16) holds rows 4 rg .. 4 rg + 3 of column c. Each entry
// belongs to one sub-block, so the fp32 scale d * sc and the min term dmin * m * sum(x) are applied here:
// the lanes that decoded the 6-bit fields (A layout) hand them over through a wave-private LDS buffer.
//
// Work split: a workgroup owns 16 * T * NWR rows at a time (and walks such row groups blockIdx.x, blockIdx.x + gridDim.x,
// ... with the activations staged once where the host launches fewer workgroups than groups); its 8 wavefronts are NWK k-slices (super-blocks kslice,
// kslice + NWK, ...) times NWR row groups, NWK = min(8, largest power of two <= in_dim / 256). Partial sums meet in LDS
// and are added in a fixed order, so results are reproducible.
#pragma once
#include "common.hpp"
#include "gemv_config.h"

typedef _Float16 mf_half8 __attribute__((ext_vector_type(8)));
typedef float mf_float4 __attribute__((ext_vector_type(4)));
struct mf_true { static constexpr bool value = true; };
struct mf_false { static constexpr bool value = false; };

#define MF_DPP(v, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), (ctrl), 0xF, 0xF, false))
#define MF_DPP_U(v, ctrl) ((u32)__builtin_amdgcn_update_dpp(0, (int)(v), (ctrl), 0xF, 0xF, false))
#define MF_DPP_QUAD_1032 0xB1
#define MF_DPP_QUAD_2301 0x4E
#define MF_DPP_ROW_ROR4 0x124
#define MF_DPP_ROW_ROR8 0x128
#define MF_DPP_ROW_HALF_MIRROR 0x141

// the compiler must not move LDS accesses of one lane across this point: other lanes of the wavefront
// read what this lane wrote (the LDS itself executes a wavefront's accesses in order)
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// T: 16-row tiles per wavefront, compile-time so that the number of weight loads in flight is a constant and
// a wait for the (older) activation loads never has to drain them.
//
// CHUNK: rows whose activations do not fit the staging buffer at once. With in_dim a multiple of 2048 the eight
// wavefronts are eight k-slices and each stages and reads the activations of its own super-blocks only, so a wavefront
// stages them C super-blocks at a time into a region of its own (no workgroup barrier), with the next chunk's
// activations requested while the current one is consumed.
// TOP1: instead of the row values a workgroup stores, per token, the largest of all its rows and that row's index
// (out[token * gridDim.x + blockIdx.x], top_ids[...]: the layout of the vector-ALU top-1 kernels, finished by
// top1_reduce_f32); of equal values the lowest row wins.
// Further matrices of the same in_dim behind the first (w, out, out_dim = rows0): rows [0, rows0) are the first's,
// [rows0, rows0 + rows1) the second's, then the third's. Every row count a multiple of 16 (a tile is of one matrix).
struct MfMany {
  const uint8_t* w1;
  const uint8_t* w2;
  float* out1;
  float* out2;
  u32 rows1, rows2;
};
// SWIGLU (gate = w, up = many->w1, many->rows1 = out_dim, a multiple of 16): the tiles alternate gate tile p, up tile p,
// so a wavefront with an even tile count holds both and the workgroup stores out[m][o] = silu(gate . x) * (up . x)
// (swiglu_one, the function of swiglu_f32) - no gate or up vectors in memory.
// Q5: Q5_K blocks (176 B: the Q4_K header, qh[32], qs[128]): bit 2g / 2g + 1 of qh[l] is the fifth bit of the low /
// high nibble of qs[32 g + l]; it is or-ed in beside the nibble (bit 4, or bit 8 next to a high nibble left in place),
// so the codes 0..31 stay exact binary16 subnormals. One more 16-byte load per lane and super-block.
template <int M, bool ADD, int T, bool CHUNK = false, bool TOP1 = false, bool SWIGLU = false, bool Q5 = false>
__device__ __forceinline__ void q4k_gemv_mfma_core(const uint8_t* w, const float* x, const float* residual,
                                                   float* out, u32 in_dim, u32 out_dim, u32* top_ids = nullptr,
                                                   const MfMany* many = nullptr) {
  static_assert(!TOP1 || !ADD, "TOP1 is a mode of the plain GEMV");
  static_assert(!SWIGLU || (T % 2 == 0 && !ADD && !TOP1), "SWIGLU pairs a gate tile with an up tile");
  // several matrices against the same activations (q | k | v, gate | up) as one matrix of all their rows
  const u32 rows1 = many ? many->rows1 : 0u, rows2 = many ? many->rows2 : 0u;
  const u32 total_rows = out_dim + rows1 + rows2;
  constexpr int MP = M <= 1 ? 1 : (M <= 2 ? 2 : 4);   // token slots in the column index
  constexpr int ND = MP;                              // accumulator tiles per 16 rows and super-block
  constexpr int BB = Q5 ? 176 : 144, QOFF = Q5 ? 48 : 16;
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
  const u32 ntiles = (total_rows + 15) >> 4;
  // A workgroup takes the row groups (NWR * T tiles each) blockIdx.x, blockIdx.x + gridDim.x, ... with the activations
  // staged once: a matrix with more groups than compute units (an output head) is launched as one workgroup per unit.
  const u32 ngroups = (ntiles + NWR * T - 1) / (NWR * T);
  u32 grp = blockIdx.x;

  // LDS map (gemv_mfma_lds_bytes): zero[64] | handover[waves][TMAX][2][8][16] f32 | partial[waves][TMAX][MP][16] f32
  //                                | fs[M][nsb] f32 | sx[M][nsb][8] f32 | ximg[nsb][M][2][256] f16
  const u32 off_tb = 64 + (u32)wave * (GEMV_MFMA_TMAX * 1024);
  const u32 off_part = 64 + GEMV_MFMA_WAVES * GEMV_MFMA_TMAX * 1024;
  const u32 off_fs = off_part + GEMV_MFMA_WAVES * GEMV_MFMA_TMAX * MP * 64;
  const u32 units_lds = CHUNK ? (u32)(GEMV_MFMA_WAVES * C * M) : (u32)M * nsb;   // units the LDS image has room for
  const u32 off_sx = off_fs + units_lds * 4;
  const u32 off_x = off_sx + units_lds * 32;
  // place of super-block sb in the activation image, and of (token, super-block) in fs / sx: by super-block, or
  // (CHUNK) by wavefront and position in the chunk
  auto xslot = [&](u32 sb) -> u32 { return CHUNK ? (u32)wave * C + ((sb >> 3) % (u32)C) : sb; };
  auto uidx = [&](u32 m, u32 sb) -> u32 { return CHUNK ? xslot(sb) * M + m : m * nsb + sb; };
  if (tid < 16) reinterpret_cast<u32*>(lds)[tid] = 0u;

  // ---- lane roles -------------------------------------------------------------------------------
  // A layout
  const u32 ar = lane & 15, kg = lane >> 4;
  const u32 k4_sh = 16u * (kg & 1);
  const bool k4_upper = kg >= 2;
  // D / B layout: column c = (slot, token, hi/lo)
  const u32 c = lane & 15, rg = lane >> 4;
  const u32 hl = c & 1, tok = (c >> 1) & (MP - 1), slot = c / (2 * MP);
  const bool col_live = tok < (u32)M;

  // weight rows of this lane, one per tile
  const size_t row_bytes = (size_t)nsb * BB;
  const uint8_t* rowp[T];
  auto set_rows = [&](u32 g) {
    const u32 tile0 = (g * NWR + rgrp) * T;
#pragma unroll
    for (int t = 0; t < T; t++) {
      const u32 tile = min(tile0 + (u32)t, ntiles - 1);
      const u32 vr = min(tile * 16 + ar, total_rows - 1);
      if constexpr (SWIGLU) rowp[t] = ((tile & 1) ? many->w1 : w) + (size_t)min((tile >> 1) * 16 + ar, out_dim - 1) * row_bytes;
      else if (!many || vr < out_dim) rowp[t] = w + (size_t)vr * row_bytes;
      else if (vr < out_dim + rows1) rowp[t] = many->w1 + (size_t)(vr - out_dim) * row_bytes;
      else rowp[t] = many->w2 + (size_t)(vr - out_dim - rows1) * row_bytes;
    }
  };
  set_rows(grp);

  struct Stage { uint4 hdr, q0, q1, hq; };
  Stage stA[T];
  auto load_sb = [&](Stage* st, u32 sb) {
    const u32 off = sb * BB;
#pragma unroll
    for (int t = 0; t < T; t++) {
      st[t].hdr = ld16(rowp[t] + off);
      st[t].q0 = ld16(rowp[t] + (off + QOFF + 16 * kg));
      st[t].q1 = ld16(rowp[t] + (off + QOFF + 64 + 16 * kg));
      if constexpr (Q5) st[t].hq = ld16(rowp[t] + (off + 16 + 16 * (kg & 1)));
    }
  };
  // The activations are requested ahead of the weights, by every wavefront of the workgroup (hence the
  // barrier): the compute unit's memory pipeline returns loads in order, and the staging below, with the
  // barrier behind it, must not wait for weight bytes.
  const u32 nunits = (u32)M * nsb;
  // unit i of this wavefront (wave-uniform): whole rows: unit wave + 8 i of the M * nsb; CHUNK: token i / C,
  // super-block i0 + i % C of the wavefront's k-slice
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
      // sums of the 8 sub-blocks (8 lanes each) for the min term, unscaled
      float sm = (v.x + v.y) + (v.z + v.w);
      sm += MF_DPP(sm, MF_DPP_QUAD_1032);
      sm += MF_DPP(sm, MF_DPP_QUAD_2301);
      sm += MF_DPP(sm, MF_DPP_ROW_HALF_MIRROR);
      // (every lane of a group holds the group's sum, every lane the scale: stored by all of them, no lane masks)
      reinterpret_cast<float*>(lds + off_sx)[uidx(m, sb) * 8 + (lane >> 3)] = sm;
      reinterpret_cast<float*>(lds + off_fs)[uidx(m, sb)] = inv;
    }
  }
  };
  stage_xv(0);
  // With all eight wavefronts in one row group and in_dim a multiple of 2048 the units a wavefront staged
  // are exactly the super-blocks of its own k-slice (unit p sits on wavefront p % 8 and covers super-block
  // p % nsb), so nobody has to wait for anybody; only the zeroed LDS words need the workgroup.
  if (NWR == 1 && (nsb & 7u) == 0) {
    if (wave != 0) {
      // the zero words are written by wavefront 0: rewrite them here instead of waiting for it
      if (lane < 16) reinterpret_cast<u32*>(lds)[lane] = 0u;
    }
    wave_lds_fence();
  } else {
    __syncthreads();
  }

  // one super-block of the k-slice: stage st holds its weights; with refill the stage is reloaded with the
  // super-block two rounds ahead as soon as the MFMAs have read it
  auto process = [&](Stage* st, u32 sb, u32 refill_sb, auto refill) {
    // B operands: 8 MFMAs (j, t); element run e0 = 64 g + 32 par + 16 hh + 8 half with g = 2 j + kg / 2,
    // hh = kg % 2, par = t % 2, half = t / 2. Live iff the column's slot is the one of sub-block
    // s = 4 j + 2 (kg / 2) + par.
    uint4 breg[8];
    const u32 ximg = off_x + ((xslot(sb) * M + tok) * 2 + hl) * 512;
#pragma unroll
    for (int j = 0; j < 2; j++) {
#pragma unroll
      for (int t = 0; t < 4; t++) {
        const u32 par = t & 1, half = t >> 1, h = kg >> 1;
        const u32 s = 4 * j + 2 * h + par;
        const u32 sl = MP == 1 ? s : (MP == 2 ? 2 * j + h : h);
        const u32 e0 = 64 * (2 * j + h) + 32 * par + 16 * (kg & 1) + 8 * half;
        const u32 a = (col_live && sl == slot) ? ximg + 2 * e0 : 0u;
        breg[j * 4 + t] = *reinterpret_cast<const uint4*>(lds + a);
      }
    }
    // per accumulator tile: the sub-block this lane's column holds, its activation sum and 2^-e
    float fsc = 0.f, sxl[ND];
    u32 sd[ND];
#pragma unroll
    for (int d = 0; d < ND; d++) {
      sd[d] = MP == 1 ? slot : (MP == 2 ? 2 * slot + d : 4 * (d >> 1) + 2 * slot + (d & 1));
      sxl[d] = 0.f;
    }
    if (col_live) {
      fsc = reinterpret_cast<const float*>(lds + off_fs)[uidx(tok, sb)];
      if (hl == 0) {
#pragma unroll
        for (int d = 0; d < ND; d++) sxl[d] = reinterpret_cast<const float*>(lds + off_sx)[uidx(tok, sb) * 8 + sd[d]];
      }
    }
    float* tb = reinterpret_cast<float*>(lds + off_tb);
    // (a) per tile: decode the (scale, min) of sub-blocks 2 kg, 2 kg + 1 of row ar into the handover
    //     buffer [tile][which][s][row]
#pragma unroll
    for (int t = 0; t < T; t++) {
      u32 sc_pair, m_pair;
      k4_pair(st[t].hdr.y, st[t].hdr.z, st[t].hdr.w, k4_sh, k4_upper, sc_pair, m_pair);
      const float dd = h2f(st[t].hdr.x), dmin = h2f(st[t].hdr.x >> 16);
      tb[t * 256 + (2 * kg) * 16 + ar] = (dd * TWO_P24) * ubyte_f<0>(sc_pair);
      tb[t * 256 + (2 * kg + 1) * 16 + ar] = (dd * TWO_P20) * ubyte_f<1>(sc_pair);
      tb[t * 256 + 128 + (2 * kg) * 16 + ar] = dmin * ubyte_f<0>(m_pair);
      tb[t * 256 + 128 + (2 * kg + 1) * 16 + ar] = dmin * ubyte_f<1>(m_pair);
    }
    // (b) the MFMAs. With one accumulator tile per 16 rows (M = 1) or two (M = 2) the tiles are interleaved
    //     so that consecutive instructions are independent; with four (M = 3, 4) the four chains of a tile
    //     are independent already and the tiles go one after the other, which keeps the registers down.
    constexpr int TI = MP >= 4 ? 1 : T;   // tiles interleaved at a time
#pragma unroll
    for (int tb0 = 0; tb0 < T; tb0 += TI) {
      mf_float4 dacc[TI][ND];
#pragma unroll
      for (int t = 0; t < TI; t++)
#pragma unroll
        for (int d = 0; d < ND; d++) dacc[t][d] = (mf_float4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 2; j++) {
#pragma unroll
        for (int t4 = 0; t4 < 4; t4++) {
#pragma unroll
          for (int t = 0; t < TI; t++) {
            const uint4 q = j == 0 ? st[tb0 + t].q0 : st[tb0 + t].q1;
            const u32 wa = (t4 & 2) ? q.z : q.x, wb = (t4 & 2) ? q.w : q.y;
            const u32 mask = (t4 & 1) ? 0x00F000F0u : 0x000F000Fu;
            uint4 a4;
            a4.x = wa & mask;
            a4.y = (wa >> 8) & mask;
            a4.z = wb & mask;
            a4.w = (wb >> 8) & mask;
            if constexpr (Q5) {
              const uint4 hq = st[tb0 + t].hq;
              const u32 sh = 2 * (kg >> 1) + 4 * j + (t4 & 1);   // bit 2 g + (high nibble) of every qh byte, g = kg / 2 + 2 j
              const u32 ba = (((t4 & 2) ? hq.z : hq.x) >> sh) & 0x01010101u, bb = (((t4 & 2) ? hq.w : hq.y) >> sh) & 0x01010101u;
              const int up = (t4 & 1) ? 8 : 4;
              a4.x |= (ba & 0x00010001u) << up;
              a4.y |= ((ba >> 8) & 0x00010001u) << up;
              a4.z |= (bb & 0x00010001u) << up;
              a4.w |= ((bb >> 8) & 0x00010001u) << up;
            }
            const int d = MP == 1 ? 0 : (MP == 2 ? (t4 & 1) : 2 * j + (t4 & 1));
            dacc[t][d] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(mf_half8, a4),
                                                                __builtin_bit_cast(mf_half8, breg[j * 4 + t4]),
                                                                dacc[t][d], 0, 0, 0);
          }
        }
      }
      if (tb0 + TI >= T) {
        if constexpr (decltype(refill)::value) load_sb(st, refill_sb);
      }
      if (tb0 == 0) wave_lds_fence();
      // (c) scales and min terms on the accumulator entries
#pragma unroll
      for (int t = 0; t < TI; t++) {
#pragma unroll
        for (int d = 0; d < ND; d++) {
          const float4 sv = *reinterpret_cast<const float4*>(tb + (tb0 + t) * 256 + sd[d] * 16 + 4 * rg);
          const float4 mv = *reinterpret_cast<const float4*>(tb + (tb0 + t) * 256 + 128 + sd[d] * 16 + 4 * rg);
          acc[tb0 + t][0] = fmaf(fsc, sv.x * dacc[t][d][0], acc[tb0 + t][0]);
          acc[tb0 + t][1] = fmaf(fsc, sv.y * dacc[t][d][1], acc[tb0 + t][1]);
          acc[tb0 + t][2] = fmaf(fsc, sv.z * dacc[t][d][2], acc[tb0 + t][2]);
          acc[tb0 + t][3] = fmaf(fsc, sv.w * dacc[t][d][3], acc[tb0 + t][3]);
          acc[tb0 + t][0] = fmaf(-mv.x, sxl[d], acc[tb0 + t][0]);
          acc[tb0 + t][1] = fmaf(-mv.y, sxl[d], acc[tb0 + t][1]);
          acc[tb0 + t][2] = fmaf(-mv.z, sxl[d], acc[tb0 + t][2]);
          acc[tb0 + t][3] = fmaf(-mv.w, sxl[d], acc[tb0 + t][3]);
        }
      }
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
      stage_xv(i0);   // (process ends with a wavefront fence: the old chunk has been read)
      wave_lds_fence();
    }
  }

  // the first super-block of the next row group is requested ahead of the reduction (the stage is free)
  const u32 next = grp + gridDim.x;
  const bool walk = !CHUNK && next < ngroups;   // (rows staged in chunks: one group per workgroup)
  if (walk) {
    set_rows(next);
    load_sb(stA, kslice);
  }
  // ---- add up the columns of a token inside the wavefront, then the k-slices through LDS ------------
#pragma unroll
  for (int t = 0; t < T; t++) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      float v = acc[t][i];
      v += MF_DPP(v, MF_DPP_QUAD_1032);                   // hi + lo
      if (MP == 1) v += MF_DPP(v, MF_DPP_QUAD_2301);      // slots: column bits 1..3
      if (MP <= 2) v += MF_DPP(v, MF_DPP_ROW_ROR4);       // column bit 2
      v += MF_DPP(v, MF_DPP_ROW_ROR8);                    // column bit 3
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
  if constexpr (SWIGLU) {
    for (u32 o = tid; o < nout / 2; o += GEMV_MFMA_WAVES * 64) {
      const u32 r = o & 15, m = (o >> 4) % M, pp = (o / (16 * M)) % (T / 2), rgp = o / (16 * M * (T / 2));
      float g = 0.f, u = 0.f;
      for (u32 k = 0; k < NWK; k++) {
        const u32 base = (((rgp << lg_nwk) + k) * GEMV_MFMA_TMAX + 2 * pp) * MP * 16 + m * 16 + r;
        g += part[base];
        u += part[base + MP * 16];
      }
      const u32 row = ((((grp * NWR + rgp) * T) >> 1) + pp) * 16 + r;
      if (row < out_dim) out[(size_t)m * out_dim + row] = swiglu_one(g, u);
    }
  } else
  for (u32 o = tid; o < nout; o += GEMV_MFMA_WAVES * 64) {
    const u32 r = o & 15, m = (o >> 4) % M, tt = (o / (16 * M)) % T, rgp = o / (16 * M * T);
    float v = 0.f;
    for (u32 k = 0; k < NWK; k++) v += part[(((rgp << lg_nwk) + k) * GEMV_MFMA_TMAX + tt) * MP * 16 + m * 16 + r];
    const u32 row = ((grp * NWR + rgp) * T + tt) * 16 + r;
    if constexpr (TOP1) {
      tv[m * group_rows + (rgp * T + tt) * 16 + r] = v;
    } else if (row >= out_dim) {
      if (row < out_dim + rows1) many->out1[(size_t)m * rows1 + (row - out_dim)] = v;
      else if (row < total_rows) many->out2[(size_t)m * rows2 + (row - out_dim - rows1)] = v;
    } else {
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
  __syncthreads();   // every partial sum has been read
  }
  if constexpr (TOP1) {
    if (wave < M && lane == 0) {
      out[(size_t)wave * gridDim.x + blockIdx.x] = run_best;
      top_ids[(size_t)wave * gridDim.x + blockIdx.x] = run_id == 0xFFFFFFFFu ? 0u : run_id;
    }
  }
}

// The tile count per wavefront follows from the grid the host chose (gemv_mfma_grid); tile count and
// round structure are template parameters so that register use and loads in flight are compile-time constants.
// Shapes outside gemv_mfma_supported() must not be launched.
template <int M, bool ADD, bool TOP1 = false, bool Q5 = false>
__device__ __forceinline__ void q4k_gemv_mfma_dispatch(const uint8_t* w, const float* x, const float* residual,
                                                       float* out, u32 in_dim, u32 out_dim, u32* top_ids = nullptr,
                                                       const MfMany* many = nullptr) {
  const u32 nsb = in_dim >> 8;
  const u32 lg = gemv_mfma_log2_kslices(nsb);
  const u32 nwr = GEMV_MFMA_WAVES >> lg;
  const u32 ntiles = (out_dim + (many ? many->rows1 + many->rows2 : 0u) + 15) >> 4;
  const u32 t = (ntiles + gridDim.x * nwr - 1) / (gridDim.x * nwr);
  if (gemv_mfma_chunked(M, in_dim)) {
    if (t <= 1) q4k_gemv_mfma_core<M, ADD, 1, true, TOP1, false, Q5>(w, x, residual, out, in_dim, out_dim, top_ids, many);
    else if (t == 2) q4k_gemv_mfma_core<M, ADD, 2, true, TOP1, false, Q5>(w, x, residual, out, in_dim, out_dim, top_ids, many);
    else q4k_gemv_mfma_core<M, ADD, 3, true, TOP1, false, Q5>(w, x, residual, out, in_dim, out_dim, top_ids, many);
    return;
  }
  if (t <= 1) q4k_gemv_mfma_core<M, ADD, 1, false, TOP1, false, Q5>(w, x, residual, out, in_dim, out_dim, top_ids, many);
  else if (t == 2) q4k_gemv_mfma_core<M, ADD, 2, false, TOP1, false, Q5>(w, x, residual, out, in_dim, out_dim, top_ids, many);
  else q4k_gemv_mfma_core<M, ADD, 3, false, TOP1, false, Q5>(w, x, residual, out, in_dim, out_dim, top_ids, many);
}

#define GEMV_MFMA_ENTRY(NAME, M)                                                                              \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(const uint8_t* w, const float* x,   \
                                                                         float* out, u32 in_dim, u32 out_dim) { \
    q4k_gemv_mfma_dispatch<M, false>(w, x, nullptr, out, in_dim, out_dim);                                    \
  }
#define GEMV_MFMA_ADD_ENTRY(NAME, M)                                                                          \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(const uint8_t* w, const float* x,   \
                                                                         const float* residual, float* out,   \
                                                                         u32 in_dim, u32 out_dim) {           \
    q4k_gemv_mfma_dispatch<M, true>(w, x, residual, out, in_dim, out_dim);                                    \
  }
// (w_raw, x, partial_ids, partial_values, in_dim, out_dim): the parameter list of the vector-ALU top-1 kernels
#define GEMV_MFMA_TOP1_ENTRY(NAME, M)                                                                          \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(const uint8_t* w, const float* x,    \
                                                                         u32* partial_ids, float* partial_values, \
                                                                         u32 in_dim, u32 out_dim) {            \
    q4k_gemv_mfma_dispatch<M, false, true>(w, x, nullptr, partial_values, in_dim, out_dim, partial_ids);       \
  }
// (w_raw_a, w_raw_b, x, out_a, out_b, in_dim, out_dim): the matrix pair, parameters of q4_k_dual_gemv_f32; M tokens at
// strides in_dim / out_dim; out_dim a multiple of 16; grid and shared memory of the single matrix with 2 * out_dim rows
#define GEMV_MFMA_DUAL_ENTRY(NAME, M)                                                                          \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(const uint8_t* w_a, const uint8_t* w_b, \
                                                                         const float* x, float* out_a, float* out_b, \
                                                                         u32 in_dim, u32 out_dim) {            \
    const MfMany many = {w_b, nullptr, out_b, nullptr, out_dim, 0u};                                           \
    q4k_gemv_mfma_dispatch<M, false>(w_a, x, nullptr, out_a, in_dim, out_dim, nullptr, &many);                 \
  }
// (w0, w1, w2, x, out0, out1, out2, in_dim, rows0, rows1, rows2): up to three matrices of one in_dim against the same
// activations (q | k | v); rows2 may be 0; every row count a multiple of 16; out_i rows at stride rows_i; grid and shared
// memory of a single matrix with rows0 + rows1 + rows2 rows
#define GEMV_MFMA_MANY_ENTRY(NAME, M)                                                                          \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(                                     \
      const uint8_t* w0, const uint8_t* w1, const uint8_t* w2, const float* x, float* out0, float* out1, float* out2, \
      u32 in_dim, u32 rows0, u32 rows1, u32 rows2) {                                                           \
    const MfMany many = {w1, w2, out1, out2, rows1, rows2};                                                    \
    q4k_gemv_mfma_dispatch<M, false>(w0, x, nullptr, out0, in_dim, rows0, nullptr, &many);                     \
  }
// (w_gate, w_up, x, out, in_dim, out_dim): the parameters of q4_k_dual_gemv_swiglu_f32; M tokens at strides in_dim /
// out_dim; out_dim a multiple of 16; two tiles per wavefront: grid = min(256, ceil(out_dim / 16 / row groups per workgroup))
#define GEMV_MFMA_SWIGLU_ENTRY(NAME, M)                                                                        \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(const uint8_t* w_gate, const uint8_t* w_up, \
                                                                         const float* x, float* out, u32 in_dim, \
                                                                         u32 out_dim) {                        \
    const MfMany many = {w_up, nullptr, nullptr, nullptr, out_dim, 0u};                                        \
    if (gemv_mfma_chunked(M, in_dim))                                                                          \
      q4k_gemv_mfma_core<M, false, 2, true, false, true>(w_gate, x, nullptr, out, in_dim, out_dim, nullptr, &many); \
    else                                                                                                       \
      q4k_gemv_mfma_core<M, false, 2, false, false, true>(w_gate, x, nullptr, out, in_dim, out_dim, nullptr, &many); \
  }
// Q5_K: the same parameter lists as GEMV_MFMA_ENTRY / GEMV_MFMA_ADD_ENTRY
#define GEMV_MFMA_Q5K_ENTRY(NAME, M)                                                                          \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(const uint8_t* w, const float* x,   \
                                                                         float* out, u32 in_dim, u32 out_dim) { \
    q4k_gemv_mfma_dispatch<M, false, false, true>(w, x, nullptr, out, in_dim, out_dim);                       \
  }
#define GEMV_MFMA_Q5K_ADD_ENTRY(NAME, M)                                                                      \
  extern "C" __global__ __launch_bounds__(GEMV_MFMA_WAVES * 64) void NAME(const uint8_t* w, const float* x,   \
                                                                         const float* residual, float* out,   \
                                                                         u32 in_dim, u32 out_dim) {           \
    q4k_gemv_mfma_dispatch<M, true, false, true>(w, x, residual, out, in_dim, out_dim);                       \
  }
