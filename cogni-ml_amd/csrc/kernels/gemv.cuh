// Decode GEMV over raw GGUF blocks: out[m][o] = (residual[m][o] +) sum_j x[m][j] * deq(W[o][j]),
// for M = 1..8 tokens in one launch with the weights read once (weight-stationary).
//
// Kernel ABI (kept from the reference's CUDA kernels, src/ml/cuda/kernels/q4k_gemv_probe.ptx:5-11):
//   *_gemv_f32            (w_raw, x, out, in_dim:u32, out_dim:u32)
//   *_gemv_add_f32        (w_raw, x, residual, out, in_dim, out_dim)           (q4k_gemv_probe.ptx:1572-1578)
//   *_gemv_f32_tbatchM    same, M tokens: x rows at stride in_dim, out/residual rows at stride out_dim
//   *_gemv_add_f32_tbatchM
// Launch: block = 256 threads (4 wavefronts), grid = ceil(out_dim / 16), no dynamic shared memory.
// w_raw is row-major [out_dim][in_dim/QK][block_bytes]; in_dim must be a multiple of the block size
// (256 for the K-quants, 32 for Q8_0). Accumulation is fp32.
//
// Work split. A wavefront owns GEMV_ROWS consecutive output rows and walks the row in "column sets":
// the span of blocks one 16-byte-per-lane load instruction covers (Q4_K/Q5_K: 8 lanes per 256-value
// super-block -> 8 blocks; Q6_K: 4 lanes per block -> 16 blocks; Q8_0: 2 lanes per 32-value block ->
// 32 blocks). A lane always sits at the same position inside a block, so the activations it needs
// for a column set are fixed: they are staged once per workgroup into LDS in lane order
// ([float4 index][lane], conflict-free 16-byte reads), pulled into registers, and reused for all rows
// of the wavefront. Each weight byte is loaded exactly once, 16 bytes per lane, and the 6-bit
// scale/min fields are unpacked in registers.
//
// Arithmetic per 32-value sub-block uses sum_j x_j*(d*sc*q_j - dmin*m) = d*sc*sum(q_j x_j) - dmin*m*sum(x_j):
// the integer codes are converted with v_cvt_f32_ubyte and multiplied into fp32 accumulators; the
// per-lane sum(x_j) is computed once per column set.
#pragma once
#include "common.cuh"

#define GEMV_BLOCK 256
#define GEMV_WAVES (GEMV_BLOCK / WAVE)
#define GEMV_ROWS 4                           // rows per wavefront
#define GEMV_ROWS_PER_BLOCK (GEMV_WAVES * GEMV_ROWS)

__device__ __forceinline__ float4 ldx4(const float* p) {
  float4 v;
  __builtin_memcpy(&v, p, 16);
  return v;
}
__device__ __forceinline__ float hsum4(float4 v) { return (v.x + v.y) + (v.z + v.w); }

template <int B>
__device__ __forceinline__ float f4c(const float4& v) {
  return B == 0 ? v.x : (B == 1 ? v.y : (B == 2 ? v.z : v.w));
}

// acc[mm] += sum_b byte_b(q) * xv[mm].b
template <int MG, int NF4, int IDX>
__device__ __forceinline__ void dot4_bytes(u32 q, const float4 (&xr)[MG][NF4], float (&acc)[MG]) {
  const float f0 = ubyte_f<0>(q), f1 = ubyte_f<1>(q), f2 = ubyte_f<2>(q), f3 = ubyte_f<3>(q);
#pragma unroll
  for (int mm = 0; mm < MG; mm++) {
    acc[mm] = fmaf(f0, xr[mm][IDX].x, acc[mm]);
    acc[mm] = fmaf(f1, xr[mm][IDX].y, acc[mm]);
    acc[mm] = fmaf(f2, xr[mm][IDX].z, acc[mm]);
    acc[mm] = fmaf(f3, xr[mm][IDX].w, acc[mm]);
  }
}

template <int R, int M, bool ADD>
__device__ __forceinline__ void gemv_epilogue(float (&acc)[R][M], const float* residual, float* out, u32 row0,
                                              u32 out_dim, int lane) {
#pragma unroll
  for (int r = 0; r < R; r++) {
#pragma unroll
    for (int m = 0; m < M; m++) {
      float v = wave_sum(acc[r][m]);
      const u32 row = row0 + r;
      if (lane == 0 && row < out_dim) {
        const size_t o = (size_t)m * out_dim + row;
        if (ADD) v += residual[o];
        out[o] = v;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Q4_K (144 B: d, dmin, scales[12], qs[128]) and Q5_K (176 B: d, dmin, scales[12], qh[32], ql[128]).
// Lane = (jb, t): block jb of the column set, 16-byte chunk t of its nibble array. Chunk t = 2g+h
// holds bytes [16h,16h+16) of group g: low nibbles are elements 64g+16h+i (sub-block 2g), high
// nibbles are elements 64g+32+16h+i (sub-block 2g+1). Q5_K adds bit 2g / 2g+1 of qh[16h+i].
// ---------------------------------------------------------------------------------------------
template <int M, bool Q5, bool ADD>
__device__ __forceinline__ void k45_gemv(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                         const float* __restrict__ residual, float* __restrict__ out, u32 in_dim,
                                         u32 out_dim) {
  constexpr int R = GEMV_ROWS;
  constexpr int BB = Q5 ? 176 : 144;
  constexpr int QOFF = Q5 ? 48 : 16;
  constexpr int MG = M < 4 ? M : 4;          // tokens held in registers at a time
  constexpr int NG = (M + MG - 1) / MG;
  __shared__ float4 xs[MG * 8 * 64];          // [token][float4 index][lane]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int t = lane & 7, jb = lane >> 3, g = t >> 1, h = t & 1;
  const u32 nb = in_dim >> 8;
  const u32 ncs = (nb + 7) >> 3;
  const size_t row_bytes = (size_t)nb * BB;
  const u32 row0 = (blockIdx.x * GEMV_WAVES + wave) * R;
  const u32 sh = 16u * (g & 1);
  const bool upper = g >= 2;

  float acc[R][M];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < M; m++) acc[r][m] = 0.0f;

  for (u32 cs = 0; cs < ncs; cs++) {
    const u32 blk = cs * 8 + jb;
    const bool valid = blk < nb;
    const u32 blkc = valid ? blk : nb - 1;
    uint4 hdr[R], qs[R], qh[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      const u32 row = min(row0 + r, out_dim - 1);
      const uint8_t* bp = w + (size_t)row * row_bytes + (size_t)blkc * BB;
      hdr[r] = ld16(bp);
      qs[r] = ld16(bp + QOFF + 16 * t);
      qh[r] = Q5 ? ld16(bp + 16 + 16 * h) : make_uint4(0u, 0u, 0u, 0u);
    }

#pragma unroll
    for (int mg = 0; mg < NG; mg++) {
      __syncthreads();
      // stage x of tokens [mg*MG, mg*MG+MG) for this column set, already in lane order
      for (u32 idx = tid; idx < (u32)(MG * 8 * 64); idx += GEMV_BLOCK) {
        const u32 l = idx & 63, i = (idx >> 6) & 7, mm = idx >> 9;
        const u32 m = mg * MG + mm;
        const u32 b = cs * 8 + (l >> 3);
        const u32 e = b * 256 + ((l & 7) >> 1) * 64 + (i >> 2) * 32 + (l & 1) * 16 + (i & 3) * 4;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (b < nb && m < (u32)M) v = ldx4(x + (size_t)m * in_dim + e);
        xs[idx] = v;
      }
      __syncthreads();

      float4 xr[MG][8];
      float sxl[MG], sxh[MG];
#pragma unroll
      for (int mm = 0; mm < MG; mm++) {
#pragma unroll
        for (int i = 0; i < 8; i++) xr[mm][i] = xs[(mm * 8 + i) * 64 + lane];
        sxl[mm] = (hsum4(xr[mm][0]) + hsum4(xr[mm][1])) + (hsum4(xr[mm][2]) + hsum4(xr[mm][3]));
        sxh[mm] = (hsum4(xr[mm][4]) + hsum4(xr[mm][5])) + (hsum4(xr[mm][6]) + hsum4(xr[mm][7]));
      }

#pragma unroll
      for (int r = 0; r < R; r++) {
        const float d = h2f(hdr[r].x), dmin = h2f(hdr[r].x >> 16);
        u32 scp, mp;
        k4_pair(hdr[r].y, hdr[r].z, hdr[r].w, sh, upper, scp, mp);
        const float dsl = d * (float)(scp & 0xFFu), dsh = d * (float)(scp >> 8);
        const float dml = dmin * (float)(mp & 0xFFu), dmh = dmin * (float)(mp >> 8);
        float dl[MG], dh[MG];
#pragma unroll
        for (int mm = 0; mm < MG; mm++) dl[mm] = dh[mm] = 0.0f;
        const u32 qd[4] = {qs[r].x, qs[r].y, qs[r].z, qs[r].w};
        const u32 hd[4] = {qh[r].x, qh[r].y, qh[r].z, qh[r].w};
        u32 lo[4], hi[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
          lo[i] = qd[i] & 0x0F0F0F0Fu;
          hi[i] = (qd[i] >> 4) & 0x0F0F0F0Fu;
          if (Q5) {
            const u32 tq = hd[i] >> (2 * g);
            lo[i] |= (tq << 4) & 0x10101010u;
            hi[i] |= (tq << 3) & 0x10101010u;
          }
        }
        dot4_bytes<MG, 8, 0>(lo[0], xr, dl);
        dot4_bytes<MG, 8, 1>(lo[1], xr, dl);
        dot4_bytes<MG, 8, 2>(lo[2], xr, dl);
        dot4_bytes<MG, 8, 3>(lo[3], xr, dl);
        dot4_bytes<MG, 8, 4>(hi[0], xr, dh);
        dot4_bytes<MG, 8, 5>(hi[1], xr, dh);
        dot4_bytes<MG, 8, 6>(hi[2], xr, dh);
        dot4_bytes<MG, 8, 7>(hi[3], xr, dh);
#pragma unroll
        for (int mm = 0; mm < MG; mm++) {
          if (mg * MG + mm < M) {
            float c = fmaf(dsl, dl[mm], -(dml * sxl[mm]));
            c = fmaf(dsh, dh[mm], c);
            c = fmaf(-dmh, sxh[mm], c);
            acc[r][mg * MG + mm] += valid ? c : 0.0f;
          }
        }
      }
    }
  }
  gemv_epilogue<R, M, ADD>(acc, residual, out, row0, out_dim, lane);
}

// ---------------------------------------------------------------------------------------------
// Q6_K (210 B: ql[128], qh[64], scales:i8[16], d). Lane = (jb, n, v): block jb of the column set,
// 128-value half n, 16-byte slice v of the half's 32 "l" positions. With l = 16v+i:
//   A = ql[64n+l], B = ql[64n+32+l], H = qh[32n+l]
//   elements 128n + {0,32,64,96} + l  <-  (A&15|H<<4&48, B&15|H<<2&48, A>>4|H&48, B>>4|H>>2&48) - 32
//   scales sc[8n + v + {0,2,4,6}]
// Blocks are 2-byte aligned only; the 16-byte loads are issued at their natural addresses.
// ---------------------------------------------------------------------------------------------
template <int M, bool ADD>
__device__ __forceinline__ void q6k_gemv(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                         const float* __restrict__ residual, float* __restrict__ out, u32 in_dim,
                                         u32 out_dim) {
  constexpr int R = GEMV_ROWS;
  constexpr int MG = M < 2 ? M : 2;
  constexpr int NG = (M + MG - 1) / MG;
  __shared__ float4 xs[MG * 16 * 64];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int s = lane & 3, jb = lane >> 2, n = s >> 1, v = s & 1;
  const u32 nb = in_dim >> 8;
  const u32 ncs = (nb + 15) >> 4;
  const size_t row_bytes = (size_t)nb * 210;
  const u32 row0 = (blockIdx.x * GEMV_WAVES + wave) * R;

  float acc[R][M];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < M; m++) acc[r][m] = 0.0f;

  for (u32 cs = 0; cs < ncs; cs++) {
    const u32 blk = cs * 16 + jb;
    const bool valid = blk < nb;
    const u32 blkc = valid ? blk : nb - 1;
    uint4 qa[R], qb[R], qh[R];
    uint2 scb[R];
    u32 db[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      const u32 row = min(row0 + r, out_dim - 1);
      const uint8_t* bp = w + (size_t)row * row_bytes + (size_t)blkc * 210;
      qa[r] = ld16(bp + 64 * n + 16 * v);
      qb[r] = ld16(bp + 64 * n + 32 + 16 * v);
      qh[r] = ld16(bp + 128 + 32 * n + 16 * v);
      scb[r] = ld8(bp + 192 + 8 * n);
      db[r] = ld2(bp + 208);
    }

#pragma unroll
    for (int mg = 0; mg < NG; mg++) {
      __syncthreads();
      // float4 index i = 4*quarter + c: elements 128n + 32*quarter + 16v + 4c .. +3
      for (u32 idx = tid; idx < (u32)(MG * 16 * 64); idx += GEMV_BLOCK) {
        const u32 l = idx & 63, i = (idx >> 6) & 15, mm = idx >> 10;
        const u32 m = mg * MG + mm;
        const u32 b = cs * 16 + (l >> 2);
        const u32 e = b * 256 + ((l & 3) >> 1) * 128 + (i >> 2) * 32 + (l & 1) * 16 + (i & 3) * 4;
        float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
        if (b < nb && m < (u32)M) val = ldx4(x + (size_t)m * in_dim + e);
        xs[idx] = val;
      }
      __syncthreads();

      float4 xr[MG][16];
      float sx[MG][4];
#pragma unroll
      for (int mm = 0; mm < MG; mm++) {
#pragma unroll
        for (int i = 0; i < 16; i++) xr[mm][i] = xs[(mm * 16 + i) * 64 + lane];
#pragma unroll
        for (int k = 0; k < 4; k++)
          sx[mm][k] = (hsum4(xr[mm][4 * k]) + hsum4(xr[mm][4 * k + 1])) +
                      (hsum4(xr[mm][4 * k + 2]) + hsum4(xr[mm][4 * k + 3]));
      }

#pragma unroll
      for (int r = 0; r < R; r++) {
        const float d = h2f(db[r]);
        // scale bytes v, v+2, v+4, v+6 of the half's 8
        const u32 s01 = scb[r].x >> (8 * v), s23 = scb[r].y >> (8 * v);
        const float sc0 = d * (float)(int)(signed char)(s01 & 0xFFu);
        const float sc1 = d * (float)(int)(signed char)((s01 >> 16) & 0xFFu);
        const float sc2 = d * (float)(int)(signed char)(s23 & 0xFFu);
        const float sc3 = d * (float)(int)(signed char)((s23 >> 16) & 0xFFu);
        const u32 a4[4] = {qa[r].x, qa[r].y, qa[r].z, qa[r].w};
        const u32 b4[4] = {qb[r].x, qb[r].y, qb[r].z, qb[r].w};
        const u32 h4[4] = {qh[r].x, qh[r].y, qh[r].z, qh[r].w};
        float d0[MG], d1[MG], d2[MG], d3[MG];
#pragma unroll
        for (int mm = 0; mm < MG; mm++) d0[mm] = d1[mm] = d2[mm] = d3[mm] = 0.0f;
        u32 q0[4], q1[4], q2[4], q3[4];
#pragma unroll
        for (int c = 0; c < 4; c++) {
          q0[c] = (a4[c] & 0x0F0F0F0Fu) | ((h4[c] << 4) & 0x30303030u);
          q1[c] = (b4[c] & 0x0F0F0F0Fu) | ((h4[c] << 2) & 0x30303030u);
          q2[c] = ((a4[c] >> 4) & 0x0F0F0F0Fu) | (h4[c] & 0x30303030u);
          q3[c] = ((b4[c] >> 4) & 0x0F0F0F0Fu) | ((h4[c] >> 2) & 0x30303030u);
        }
        dot4_bytes<MG, 16, 0>(q0[0], xr, d0);
        dot4_bytes<MG, 16, 1>(q0[1], xr, d0);
        dot4_bytes<MG, 16, 2>(q0[2], xr, d0);
        dot4_bytes<MG, 16, 3>(q0[3], xr, d0);
        dot4_bytes<MG, 16, 4>(q1[0], xr, d1);
        dot4_bytes<MG, 16, 5>(q1[1], xr, d1);
        dot4_bytes<MG, 16, 6>(q1[2], xr, d1);
        dot4_bytes<MG, 16, 7>(q1[3], xr, d1);
        dot4_bytes<MG, 16, 8>(q2[0], xr, d2);
        dot4_bytes<MG, 16, 9>(q2[1], xr, d2);
        dot4_bytes<MG, 16, 10>(q2[2], xr, d2);
        dot4_bytes<MG, 16, 11>(q2[3], xr, d2);
        dot4_bytes<MG, 16, 12>(q3[0], xr, d3);
        dot4_bytes<MG, 16, 13>(q3[1], xr, d3);
        dot4_bytes<MG, 16, 14>(q3[2], xr, d3);
        dot4_bytes<MG, 16, 15>(q3[3], xr, d3);
#pragma unroll
        for (int mm = 0; mm < MG; mm++) {
          if (mg * MG + mm < M) {
            // sum (q-32) x = sum q x - 32 sum x
            float c = sc0 * fmaf(-32.0f, sx[mm][0], d0[mm]);
            c = fmaf(sc1, fmaf(-32.0f, sx[mm][1], d1[mm]), c);
            c = fmaf(sc2, fmaf(-32.0f, sx[mm][2], d2[mm]), c);
            c = fmaf(sc3, fmaf(-32.0f, sx[mm][3], d3[mm]), c);
            acc[r][mg * MG + mm] += valid ? c : 0.0f;
          }
        }
      }
    }
  }
  gemv_epilogue<R, M, ADD>(acc, residual, out, row0, out_dim, lane);
}

// ---------------------------------------------------------------------------------------------
// Q8_0 (34 B: d, qs:i8[32]). Lane = (jb, hf): block jb of the column set (32 blocks = 1024 values),
// 16-byte half hf of its codes. Signed codes are read as unsigned with the top bit flipped:
// sum q x = sum (q^0x80) x - 128 sum x. in_dim may end inside a block (the tail is clipped).
// ---------------------------------------------------------------------------------------------
template <int M, bool ADD>
__device__ __forceinline__ void q80_gemv(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                         const float* __restrict__ residual, float* __restrict__ out, u32 in_dim,
                                         u32 out_dim) {
  constexpr int R = GEMV_ROWS;
  constexpr int MG = M < 4 ? M : 4;
  constexpr int NG = (M + MG - 1) / MG;
  __shared__ float4 xs[MG * 4 * 64];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hf = lane & 1, jb = lane >> 1;
  const u32 nb = (in_dim + 31) >> 5;
  const u32 ncs = (nb + 31) >> 5;
  const size_t row_bytes = (size_t)nb * 34;
  const u32 row0 = (blockIdx.x * GEMV_WAVES + wave) * R;

  float acc[R][M];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < M; m++) acc[r][m] = 0.0f;

  for (u32 cs = 0; cs < ncs; cs++) {
    const u32 blk = cs * 32 + jb;
    const bool valid = blk < nb;
    const u32 blkc = valid ? blk : nb - 1;
    uint4 qs[R];
    u32 db[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
      const u32 row = min(row0 + r, out_dim - 1);
      const uint8_t* bp = w + (size_t)row * row_bytes + (size_t)blkc * 34;
      qs[r] = ld16(bp + 2 + 16 * hf);
      db[r] = ld2(bp);
    }

#pragma unroll
    for (int mg = 0; mg < NG; mg++) {
      __syncthreads();
      for (u32 idx = tid; idx < (u32)(MG * 4 * 64); idx += GEMV_BLOCK) {
        const u32 l = idx & 63, i = (idx >> 6) & 3, mm = idx >> 8;
        const u32 m = mg * MG + mm;
        const u32 e = (cs * 32 + (l >> 1)) * 32 + (l & 1) * 16 + i * 4;
        float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
        if (m < (u32)M) {
          const float* xp = x + (size_t)m * in_dim;
          if (e + 4 <= in_dim) {
            val = ldx4(xp + e);
          } else {                      // clipped tail of the last block
            if (e + 0 < in_dim) val.x = xp[e + 0];
            if (e + 1 < in_dim) val.y = xp[e + 1];
            if (e + 2 < in_dim) val.z = xp[e + 2];
          }
        }
        xs[idx] = val;
      }
      __syncthreads();

      float4 xr[MG][4];
      float sx[MG];
#pragma unroll
      for (int mm = 0; mm < MG; mm++) {
#pragma unroll
        for (int i = 0; i < 4; i++) xr[mm][i] = xs[(mm * 4 + i) * 64 + lane];
        sx[mm] = (hsum4(xr[mm][0]) + hsum4(xr[mm][1])) + (hsum4(xr[mm][2]) + hsum4(xr[mm][3]));
      }

#pragma unroll
      for (int r = 0; r < R; r++) {
        const float d = h2f(db[r]);
        float dt[MG];
#pragma unroll
        for (int mm = 0; mm < MG; mm++) dt[mm] = 0.0f;
        dot4_bytes<MG, 4, 0>(qs[r].x ^ 0x80808080u, xr, dt);
        dot4_bytes<MG, 4, 1>(qs[r].y ^ 0x80808080u, xr, dt);
        dot4_bytes<MG, 4, 2>(qs[r].z ^ 0x80808080u, xr, dt);
        dot4_bytes<MG, 4, 3>(qs[r].w ^ 0x80808080u, xr, dt);
#pragma unroll
        for (int mm = 0; mm < MG; mm++) {
          if (mg * MG + mm < M) {
            const float c = d * fmaf(-128.0f, sx[mm], dt[mm]);
            acc[r][mg * MG + mm] += valid ? c : 0.0f;
          }
        }
      }
    }
  }
  gemv_epilogue<R, M, ADD>(acc, residual, out, row0, out_dim, lane);
}

// ---- entry points ---------------------------------------------------------------------------
#define GEMV_ENTRY(NAME, BODY, M)                                                                                  \
  extern "C" __global__ __launch_bounds__(GEMV_BLOCK) void NAME(const uint8_t* w, const float* x, float* out,      \
                                                                 u32 in_dim, u32 out_dim) {                        \
    BODY(M, false)(w, x, nullptr, out, in_dim, out_dim);                                                          \
  }
#define GEMV_ADD_ENTRY(NAME, BODY, M)                                                                              \
  extern "C" __global__ __launch_bounds__(GEMV_BLOCK) void NAME(const uint8_t* w, const float* x,                  \
                                                                 const float* residual, float* out, u32 in_dim,    \
                                                                 u32 out_dim) {                                    \
    BODY(M, true)(w, x, residual, out, in_dim, out_dim);                                                          \
  }
#define BODY_Q4K(M, ADD) k45_gemv<M, false, ADD>
#define BODY_Q5K(M, ADD) k45_gemv<M, true, ADD>
#define BODY_Q6K(M, ADD) q6k_gemv<M, ADD>
#define BODY_Q80(M, ADD) q80_gemv<M, ADD>

#define GEMV_FAMILY(PFX, BODY)                        \
  GEMV_ENTRY(PFX##_gemv_f32, BODY, 1)                 \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch2, BODY, 2)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch3, BODY, 3)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch4, BODY, 4)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch5, BODY, 5)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch6, BODY, 6)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch7, BODY, 7)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch8, BODY, 8)         \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32, BODY, 1)         \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch2, BODY, 2) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch3, BODY, 3) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch4, BODY, 4) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch5, BODY, 5) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch6, BODY, 6) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch7, BODY, 7) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch8, BODY, 8)

GEMV_FAMILY(q4_k, BODY_Q4K)
GEMV_FAMILY(q5_k, BODY_Q5K)
GEMV_FAMILY(q6_k, BODY_Q6K)
GEMV_FAMILY(q8_0, BODY_Q80)
