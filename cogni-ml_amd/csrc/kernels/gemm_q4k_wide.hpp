// Prefill GEMM over raw Q4_K weights with eight wavefronts per workgroup, two per SIMD: the second formulation of
// out[m][n] = (bias[n] +) sum_k x[m][k] * deq(W[n][k]) (src/ml/gguf/kernels/gemm_q4k.metal:615-776 is the reference's
// prefill kernel; precision as there: x and the dequantized weights rounded to half, fp32 accumulation).
//
//   q4_k_gemm_wide_f16 (w_raw, xp, bias|null, out:f32 [m][out_dim], in_dim:u32, out_dim:u32, m:u32, bias_stride:u32)
//                      block 512, grid gemm_grid_x(ceil(m/128), ceil(out_dim/256)) from gemv_config.h, no dynamic LDS (136 KiB static)
//   xp is the image pack_x_f16_q4k writes (gemm_q4k.hpp); bias as for q4_k_gemm_f16; no k split.
//
// Tiling. A workgroup owns 128 tokens x 256 weight rows. Its eight wavefronts are (row quarter nh) x (k-step half kh):
// a wavefront accumulates 128 tokens x 64 rows (4 x 2 tiles of v_mfma_f32_32x32x16_f16, 128 accumulator registers) over
// 8 of the 16 k-steps of every super-block, so two wavefronts fit a SIMD and one's operand preparation and copies run
// under the other's MFMAs. No two wavefronts decode the same weights (a wavefront's tile spans all 128 tokens), so the
// dequantized values never need to be shared: they go from the raw bytes to the matrix cores through registers, and
// LDS carries only the 4.5-bit bytes.
//
// Against q4_k_gemm_f16 (128 x 192, four wavefronts): the x tile is reused by a third more rows (25 % fewer bytes
// copied per flop) and a SIMD always has a second wavefront to issue from; a tile is a third larger, so a launch
// needs ceil(m/128) * ceil(out_dim/256) tiles to fill the 256 compute units in whole rounds to gain from it (the
// host picks, gemm_q4k_use_wide in gemv_config.h).
//
// Staging. x: as in q4_k_gemm_f16 (two 64 KiB buffers, global_load_lds_dwordx4, eight copies per wavefront and
// super-block). Weights: a wavefront copies what it decodes itself - bytes [16 + 64 kh, +64) of the super-block of
// its 64 rows, 4 KiB = four copies - into a region of its own, so the only workgroup barrier of an iteration is the
// one that hands the next x tile over; the 16-byte headers go from global memory straight to the lanes that decode
// them. A lane (row j of a 32-row tile, k-group kg) reads pieces 2 kg and 2 kg + 1 of its row; piece q of
// wave-local row r sits in slot r * 4 + (q ^ ((r >> 2) & 3)), which spreads the 16 lanes served together over all banks.
#pragma once
#include "gemm_q4k.hpp"

#define GEMM_WIDE_BN 256

__shared__ uint4 gemm_wide_wbuf[8 * 256];   // [wavefront][64 rows][4 pieces]

// Epilogue of the wide kernel: as gemm_epilogue_half, with 4 x 2 tiles per wavefront. A kh wavefront finishes the
// token tiles r = 2 kh, 2 kh + 1 and hands the other two to its partner (same nh) as 16 float4 per lane (kh = 0 writes
// into x buffer 0, kh = 1 into x buffer 1: 4 x 16 KiB each). Sum first, bias second.
template <int KH>
__device__ __forceinline__ void gemm_wide_epilogue_half(float16_t (&acc)[4][2], const float* bias, float* out, u32 out_dim, u32 m,
                                                        u32 mt, u32 nt, u32 nh, u32 j, u32 kg, u32 lane, u32 bias_stride) {
  float4* mine = reinterpret_cast<float4*>(KH ? gemm_xbuf1 : gemm_xbuf0) + nh * 16 * 64 + lane;
  const float4* theirs = reinterpret_cast<const float4*>(KH ? gemm_xbuf0 : gemm_xbuf1) + nh * 16 * 64 + lane;
#pragma unroll
  for (int rr = 0; rr < 2; rr++)
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
      for (int g4 = 0; g4 < 4; g4++) {
        const float16_t& t = acc[2 * (1 - KH) + rr][c];
        mine[((rr * 2 + c) * 4 + g4) * 64] = make_float4(t[4 * g4], t[4 * g4 + 1], t[4 * g4 + 2], t[4 * g4 + 3]);
      }
  __syncthreads();
  const bool vec = (out_dim & 3u) == 0;
  if (vec && mt * GEMM_BM + GEMM_BM <= m && nt * GEMM_WIDE_BN + GEMM_WIDE_BN <= out_dim) {
    // a whole tile: one address per token row, the 8 stores of a row at constant offsets from it, 16 bytes each (kept
    // apart from the general path below so that the compiler cannot merge the two into single-float stores)
#pragma unroll
    for (int rr = 0; rr < 2; rr++) {
      const size_t token = mt * GEMM_BM + 32 * (2 * KH + rr) + j;
      const u32 col = nt * GEMM_WIDE_BN + nh * 64 + 4 * kg;
      float* base = out + token * out_dim + col;
      const float* bbase = bias ? bias + token * bias_stride + col : nullptr;
#pragma unroll
      for (int c = 0; c < 2; c++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const float16_t& t = acc[2 * KH + rr][c];
          const float4 p = theirs[((rr * 2 + c) * 4 + g4) * 64];
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
    for (int rr = 0; rr < 2; rr++) {
      const u32 token = mt * GEMM_BM + 32 * (2 * KH + rr) + j;
#pragma unroll
      for (int c = 0; c < 2; c++)
#pragma unroll
        for (int g4 = 0; g4 < 4; g4++) {
          const float16_t& t = acc[2 * KH + rr][c];
          const float4 p = theirs[((rr * 2 + c) * 4 + g4) * 64];
          // (k half 0) + (k half 1) whichever of the two this wavefront holds
          float4 o = KH ? make_float4(p.x + t[4 * g4], p.y + t[4 * g4 + 1], p.z + t[4 * g4 + 2], p.w + t[4 * g4 + 3])
                        : make_float4(t[4 * g4] + p.x, t[4 * g4 + 1] + p.y, t[4 * g4 + 2] + p.z, t[4 * g4 + 3] + p.w);
          const u32 n = nt * GEMM_WIDE_BN + nh * 64 + 32 * c + 8 * g4 + 4 * kg;
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

extern "C" __global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void q4_k_gemm_wide_f16(
    const uint8_t* w, const uint4* xp, const float* bias, float* out, u32 in_dim, u32 out_dim, u32 m, u32 bias_stride) {
  constexpr u32 BS = 144;
  const u32 tid = threadIdx.x, lane = tid & 63;
  const u32 wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const u32 nh = wave & 3, kh = wave >> 2;
  const u32 j = lane & 31, kg = lane >> 5;
  const u32 nkb = in_dim >> 8;   // (no k split: the host takes this kernel only for launches of whole rounds of tiles)
  const u32 mtiles = (m + GEMM_BM - 1) / GEMM_BM, ntiles = (out_dim + GEMM_WIDE_BN - 1) / GEMM_WIDE_BN;
  // workgroup -> tile, XCD-aware (see q4_k_gemm_f16)
  u32 mt, nt;
  if (!gemm_tile_of(blockIdx.x, mtiles, ntiles, &mt, &nt)) return;
  const size_t row_bytes = (size_t)nkb * BS;
  const u32 sh = 16u * kg;
  // the two forms of the 6-bit unpacking folded into one through opaque masks (see gemm_k45_core)
  u32 um = kh ? 0xFFFFFFFFu : 0u, mA = kh ? 0x0F0Fu : 0x3F3Fu, mB = kh ? 0x3030u : 0u, shM = kh ? 4u : 0u;
  um = __builtin_amdgcn_readfirstlane(um);
  mA = __builtin_amdgcn_readfirstlane(mA);
  mB = __builtin_amdgcn_readfirstlane(mB);
  shM = __builtin_amdgcn_readfirstlane(shM);
  asm volatile("" : "+s"(um), "+s"(mA), "+s"(mB), "+s"(shM));
  u32 magic_lo = 0x64006400u, magic_hi = 0x54005400u;
  asm volatile("" : "+v"(magic_lo), "+v"(magic_hi));

  const u32 tile_row0 = min(nt * GEMM_WIDE_BN, out_dim - 1);
  const uint8_t* wbase = w + (size_t)tile_row0 * row_bytes;   // uniform
  // copy i of this wavefront: lane -> (wave-local row 16 i + lane / 4, the piece that belongs in slot lane % 4 of that row)
  u32 woff[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const u32 r = 16u * i + (lane >> 2), q = (lane & 3u) ^ ((r >> 2) & 3u);
    woff[i] = (min(nt * GEMM_WIDE_BN + nh * 64 + r, out_dim - 1) - tile_row0) * (u32)row_bytes + 16u + 64u * kh + 16u * q;
  }
  // where this lane finds the two pieces of its k-group for its two rows, and where its rows' headers are
  u32 wslot[2][2], hoff[2];
#pragma unroll
  for (int c = 0; c < 2; c++) {
    const u32 r = 32 * c + j;
    wslot[c][0] = wave * 256 + r * 4 + ((2 * kg) ^ ((r >> 2) & 3));
    wslot[c][1] = wave * 256 + r * 4 + ((2 * kg + 1) ^ ((r >> 2) & 3));
    hoff[c] = (min(nt * GEMM_WIDE_BN + nh * 64 + r, out_dim - 1) - tile_row0) * (u32)row_bytes;
  }
  const uint4* xtile = xp + (size_t)mt * nkb * 4096;

  float16_t acc[4][2];
#pragma unroll
  for (int r = 0; r < 4; r++)
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[r][c][v] = 0.0f;

  auto copy_w = [&](u32 kb, int i) {
    __builtin_amdgcn_global_load_lds((gbl_void*)(wbase + (size_t)kb * BS + woff[i]),
                                     (lds_void*)(gemm_wide_wbuf + wave * 256 + i * 64), 16, 0, 0);
  };
  uint4 nhdr[2];   // headers of the super-block being copied
  auto load_hdr = [&](u32 kb, int c) { nhdr[c] = ld16(wbase + (size_t)kb * BS + hoff[c]); };

  // Super-block 0. The main loop takes super-blocks in pairs with fixed x buffers (0 then 1); with an odd number the
  // first one is taken alone out of buffer 1.
  const bool odd = nkb & 1;
#pragma unroll
  for (int i = 0; i < 4; i++) copy_w(0, i);
#pragma unroll
  for (int c = 0; c < 2; c++) load_hdr(0, c);
  if (odd) {
#pragma unroll
    for (int i = 0; i < 8; i++)
      __builtin_amdgcn_global_load_lds((gbl_void*)(xtile + 512 * i + tid), (lds_void*)(gemm_xbuf1 + 512 * i + wave * 64), 16, 0, 0);
  } else {
#pragma unroll
    for (int i = 0; i < 8; i++)
      __builtin_amdgcn_global_load_lds((gbl_void*)(xtile + 512 * i + tid), (lds_void*)(gemm_xbuf0 + 512 * i + wave * 64), 16, 0, 0);
  }
  __syncthreads();

  GemmRawT<false> cur[2];
  u32 S[2][4];
  uint4 A[2][4];
  half8_t B[2][2];
  auto take_raw = [&]() {
#pragma unroll
    for (int c = 0; c < 2; c++) {
      cur[c].hdr = nhdr[c];
      cur[c].qa = gemm_wide_wbuf[wslot[c][0]];
      cur[c].qb = gemm_wide_wbuf[wslot[c][1]];
    }
  };
  auto decode_scales = [&]() {
#pragma unroll
    for (int c = 0; c < 2; c++) {
      const float d = h2f(cur[c].hdr.x), dm = h2f(cur[c].hdr.x >> 16);
      const u32 a0 = cur[c].hdr.y >> sh, a1 = cur[c].hdr.z >> sh, a2 = cur[c].hdr.w >> sh;
      const u32 aS = (um & a2) | (~um & a0), aM = (um & a2) | (~um & a1);
      const u32 scp = (aS & mA) | ((a0 >> 2) & mB);
      const u32 mp = ((aM >> shM) & mA) | ((a1 >> 2) & mB);
      S[c][0] = h2_dup(d * ubyte_f<0>(scp));
      S[c][1] = h2_dup(-(dm * ubyte_f<0>(mp)));
      S[c][2] = h2_dup(d * ubyte_f<1>(scp));
      S[c][3] = h2_dup(-(dm * ubyte_f<1>(mp)));
    }
  };
  auto build_b = [&](half8_t (&Bd)[2], int t) {
    const int h = t >> 2, op = t & 3, hi = op >> 1;
#pragma unroll
    for (int c = 0; c < 2; c++) {
      const uint4 Q = h ? cur[c].qb : cur[c].qa;
      const u32 qa = (op & 1) ? Q.z : Q.x, qb = (op & 1) ? Q.w : Q.y;
      const u32 mask = hi ? 0x00F000F0u : 0x000F000Fu;
      const u32 magic = hi ? magic_hi : magic_lo;
      const u32 off = hi ? 0xD400D400u : 0xE400E400u;
      const u32 sc = S[c][2 * hi], nm = S[c][2 * hi + 1];
      uint4 bw;
      bw.x = h2_fma_off((qa & mask) | magic, off, sc, nm);
      bw.y = h2_fma_off(((qa >> 8) & mask) | magic, off, sc, nm);
      bw.z = h2_fma_off((qb & mask) | magic, off, sc, nm);
      bw.w = h2_fma_off(((qb >> 8) & mask) | magic, off, sc, nm);
      Bd[c] = *reinterpret_cast<const half8_t*>(&bw);
    }
  };
  auto read_a = [&](uint4 (&Ad)[4], const uint4* xbuf, int t) {
    const uint4* arow = xbuf + (16 * kh + kg) * 128 + j;
#pragma unroll
    for (int r = 0; r < 4; r++) Ad[r] = arow[t * 256 + r * 32];
  };

  take_raw();
  decode_scales();
  read_a(A[0], odd ? gemm_xbuf1 : gemm_xbuf0, 0);
  build_b(B[0], 0);

  auto iteration = [&](u32 kb, const uint4* xcur, uint4* xnxt) {
    const u32 kn = min(kb + 1, nkb - 1);   // the last iteration re-reads its own tile; the copy is not used
    const uint4* xnext = xtile + (size_t)kn * 4096;   // uniform
    auto copy_x = [&](int i) {
      __builtin_amdgcn_global_load_lds((gbl_void*)(xnext + 512 * i + tid), (lds_void*)(xnxt + 512 * i + wave * 64), 16, 0, 0);
    };
#pragma unroll
    for (int t = 0; t < 8; t++) {
      const int p = t & 1;
      // the wavefront's own raw bytes were taken into registers in the previous iteration's last k-step (and waited
      // for by the arithmetic that used them), so its region is free again
      if (t < 2) {
        copy_w(kn, 2 * t);
        copy_w(kn, 2 * t + 1);
        load_hdr(kn, t);
      }
      if (t >= 2 && t < 6) {
        copy_x(2 * (t - 2));
        copy_x(2 * (t - 2) + 1);
      }
      if (t < 7) {
        read_a(A[p ^ 1], xcur, t + 1);
        build_b(B[p ^ 1], t + 1);
      } else {
        // the next super-block is in LDS (wait and barrier behind k-step 6): its raw bytes, scales and first operands
        take_raw();
        read_a(A[0], xnxt, 0);
        decode_scales();
        build_b(B[0], 0);
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const half8_t Ar = *reinterpret_cast<const half8_t*>(&A[p][r]);
#pragma unroll
        for (int c = 0; c < 2; c++) acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(B[p][c], Ar, acc[r][c], 0, 0, 0);
      }
#pragma unroll
      for (int c = 0; c < 2; c++) asm volatile("" : "+v"(B[p ^ 1][c]));
      // one MFMA, then a few of the vector instructions that prepare the next step (see q4_k_gemm_f16)
      if (t < 7) {
        __builtin_amdgcn_sched_group_barrier(0x020, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
        for (int i = 0; i < 8; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        }
      } else {
        __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
        for (int i = 0; i < 8; i++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, 10, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if (t == 6) {
        // this wavefront's copies (its weights, its share of the next x tile) have landed and its reads of xcur are
        // done; behind the barrier that holds for every wavefront
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // the raw bytes taken in the last k-step are in registers before the next iteration's copies overwrite the region
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  if (odd) iteration(0, gemm_xbuf1, gemm_xbuf0);
  for (u32 kb = odd; kb < nkb; kb += 2) {
    iteration(kb, gemm_xbuf0, gemm_xbuf1);
    iteration(kb + 1, gemm_xbuf1, gemm_xbuf0);
  }
  __syncthreads();   // drains the last (unused) prefetches before the buffers are reused below

  if (kh == 0) gemm_wide_epilogue_half<0>(acc, bias, out, out_dim, m, mt, nt, nh, j, kg, lane, bias_stride);
  else gemm_wide_epilogue_half<1>(acc, bias, out, out_dim, m, mt, nt, nh, j, kg, lane, bias_stride);
}
