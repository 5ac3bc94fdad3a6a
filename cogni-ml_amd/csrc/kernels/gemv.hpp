// Decode GEMV over raw GGUF blocks: out[m][o] = (residual[m][o] +) sum_j x[m][j] * deq(W[o][j]),
// for M = 1..8 tokens in one launch with the weights read once (weight-stationary).
//
// Kernel ABI (kept from the reference's CUDA kernels, src/ml/cuda/kernels/q4k_gemv_probe.ptx:5-11):
//   *_gemv_f32            (w_raw, x, out, in_dim:u32, out_dim:u32)
//   *_gemv_add_f32        (w_raw, x, residual, out, in_dim, out_dim)           (q4k_gemv_probe.ptx:1572-1578)
//   *_gemv_f32_tbatchM    same, M tokens: x rows at stride in_dim, out/residual rows at stride out_dim
//   *_gemv_add_f32_tbatchM
// Launch: block = 256 threads (4 wavefronts), grid = any number of workgroups up to ceil(out_dim / rows_per_block)
// (a workgroup walks the row groups blockIdx.x, blockIdx.x + gridDim.x, ...; gemv_grid in gemv_config.h gives the
// grid the library uses), dynamic shared memory = gemv_lds_bytes(type, tokens, in_dim), also from gemv_config.h.
// w_raw is row-major [out_dim][in_dim/QK][block_bytes];
// in_dim must be a multiple of 256 for the K-quants (Q8_0 takes any in_dim). Accumulation is fp32.
//
// Work split. A wavefront owns R consecutive output rows and walks them in "column sets": the span
// of blocks the 64 lanes cover side by side (Q4_K/Q5_K/Q6_K: 4 lanes per 256-value super-block ->
// 16 blocks; Q8_0: 2 lanes per 32-value block -> 32 blocks), all loads 16 bytes per lane. A lane always sits at
// the same position inside a block, so the activations it needs for a column set are fixed: the workgroup stages
// x into LDS once (K-quants with one or two tokens: in natural order with a bank swizzle, see stage_rounds;
// otherwise already in lane order, [float4 index][lane]), each lane pulls its share into registers and reuses it
// for all R rows. Every weight byte is loaded exactly once, 16 bytes per lane. One token of a K-quant matrix takes
// its rows through a rolling pipeline (a row or two in flight while one is consumed); the other kernels request
// the R rows of a column set together.
//
// Arithmetic. Per 32-value sub-block sum_j x_j*(d*sc*q_j - dmin*m) = d*sc*sum(q_j x_j) - dmin*m*sum(x_j);
// sum(x_j) is per lane and computed once per column set. The integer codes are not converted to
// float one by one: a masked pair of codes (two 16-bit halves of a dword, values < 1024) read as two
// binary16 numbers is exactly code * 2^-24 (a subnormal) or, for codes sitting 4 bits up, code * 2^-20.
// v_fma_mix_f32 multiplies such a half by an fp32 activation into an fp32 accumulator, subnormals
// honoured, so a code costs one mask per pair plus one fused multiply-add; the power of two is folded
// into the block scale.
#pragma once
#include <type_traits>
#include "common.hpp"
#include "gemv_config.h"


__device__ __forceinline__ float4 ldx4(const float* p) {
  float4 v;
  __builtin_memcpy(&v, p, 16);
  return v;
}
__device__ __forceinline__ float hsum4(float4 v) { return (v.x + v.y) + (v.z + v.w); }

// acc + lo16(t) * a + hi16(t) * b with the halves of t read as binary16 (two v_fma_mix_f32)
__device__ __forceinline__ float mix2(u32 t, float a, float b, float acc) {
  const __half2 h = *reinterpret_cast<const __half2*>(&t);
  acc = fmaf(__low2float(h), a, acc);
  acc = fmaf(__high2float(h), b, acc);
  return acc;
}

struct gemv_true { static constexpr bool value = true; };
struct gemv_false { static constexpr bool value = false; };
#define TWO_P24 16777216.0f
#define TWO_P20 1048576.0f

// ---------------------------------------------------------------------------------------------
// Q4_K (144 B: d, dmin, scales[12], qs[128]) and Q5_K (176 B: d, dmin, scales[12], qh[32], ql[128]).
// Lane = (jb, g): block jb of the column set (16 blocks), 64-value group g of the block: the 32 bytes
// qs[32g, 32g+32) as two 16-byte loads. Byte l holds element 64g+l (low nibble, sub-block 2g) and
// element 64g+32+l (high nibble, sub-block 2g+1); Q5_K adds bit 2g / 2g+1 of qh[l]. One (scale, min)
// pair decode per lane and row serves 64 weights.
// x registers: float4 i<8 -> low elements 4i..4i+3, i>=8 -> high elements 4(i-8)..
// ---------------------------------------------------------------------------------------------
template <bool Q5>
struct FmtK45 {
  static constexpr int BB = Q5 ? 176 : 144;
  static constexpr int QOFF = Q5 ? 48 : 16;
  static constexpr int BPS = 16;   // blocks per column set
  static constexpr int NF4 = 16;   // float4 of x per lane per column set and token
  static constexpr int NSUM = 2;
  static constexpr int MG_MAX = 2;
  static constexpr int SPI = 1;   // sets per iteration: a column set is 4096 values
  static constexpr unsigned TYPE = Q5 ? 13 : 12;
  static constexpr int rows(int m) { return Q5 ? GEMV_ROWS_Q5K(m) : GEMV_ROWS_Q4K(m); }

  struct Lane {
    int jb, g;
    u32 sh, sh2, shm, m1, m2;   // constants of the branch-free 6-bit field decode below
    bool upper;
    __device__ __forceinline__ explicit Lane(int lane) : jb(lane >> 2), g(lane & 3) {
      upper = g >= 2;
      sh = 16u * (g & 1);
      sh2 = sh + 2;
      shm = upper ? sh + 4 : sh;
      m1 = upper ? 0x0F0Fu : 0x3F3Fu;
      m2 = upper ? 0x3030u : 0u;
    }
  };
  template <int R>
  struct Stage {
    uint4 hdr[R], q0[R], q1[R], h0[R], h1[R];
  };

  static __device__ __forceinline__ u32 nblocks(u32 in_dim) { return in_dim >> 8; }
  static __device__ __forceinline__ size_t row_bytes(u32 nb) { return (size_t)nb * BB; }
  // first element (in the row) of float4 i of lane l in column set `set`
  static __device__ __forceinline__ u32 x_elem(u32 set, u32 l, u32 i) {
    return (set * 16 + (l >> 2)) * 256 + (l & 3) * 64 + (i >> 3) * 32 + (i & 7) * 4;
  }
  static __device__ __forceinline__ float4 load_x(const float* xrow, u32 e, u32 in_dim) {
    return e < in_dim ? ldx4(xrow + e) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  // Place of 16-byte piece p (0..1023) of a column set in the directly staged LDS image: the natural order with the
  // low four bits of the index XORed by a function of the higher ones. A lane reads the 16 consecutive pieces
  // 16 l .. 16 l + 15, so without this the 16 lanes served together would all hit the same four banks; with it
  // they hit 16 different groups of four. An involution: it also gives the piece that belongs at place p.
  static __device__ __forceinline__ u32 swz(u32 p) {
    const u32 grp = p >> 4;
    return p ^ (((grp & 3u) << 2) | ((grp >> 2) & 3u));
  }

  template <int R>
  static __device__ __forceinline__ void load(Stage<R>& st, const uint8_t* const (&rowp)[R], const Lane& ln,
                                              u32 set, u32 nb) {
#pragma unroll
    for (int r = 0; r < R; r++) load_row<R>(st, r, rowp[r], ln, set, nb);
  }
  template <int R>
  static __device__ __forceinline__ void load_row(Stage<R>& st, int r, const uint8_t* rp, const Lane& ln, u32 set,
                                                  u32 nb) {
    const u32 off = min(set * 16 + ln.jb, nb - 1) * BB;   // a row is far below 4 GiB
    st.hdr[r] = ld16(rp + off);
    st.q0[r] = ld16(rp + (off + QOFF + 32 * ln.g));
    st.q1[r] = ld16(rp + (off + QOFF + 32 * ln.g + 16));
    st.h0[r] = Q5 ? ld16(rp + (off + 16)) : make_uint4(0u, 0u, 0u, 0u);
    st.h1[r] = Q5 ? ld16(rp + (off + 32)) : make_uint4(0u, 0u, 0u, 0u);
  }

  // contribution of this lane's 64 weights of row r to MG tokens
  template <int R, int MG>
  static __device__ __forceinline__ void compute(const Stage<R>& st, int r, const Lane& ln,
                                                 const float4 (&xr)[MG][NF4], const float (&sx)[MG][NSUM],
                                                 float (&c)[MG]) {
    const float d = h2f(st.hdr[r].x), dmin = h2f(st.hdr[r].x >> 16);
    const float d24 = d * TWO_P24, d20 = d * TWO_P20;
    // (scale, min) of sub-blocks 2g and 2g+1 as byte pairs (dequant.cr:240-249 for j = 2g, 2g+1 at once):
    //   g < 2 : sc = s[2g..] & 63,                         m = s[2g+4..] & 63
    //   g >= 2: sc = (s[2g+4..] & 15) | (s[2g-4..] >> 6 << 4), m = (s[2g+4..] >> 4) | (s[2g..] >> 6 << 4)
    // with s0/s1/s2 the three dwords of the field, both cases are
    //   sc = ((P >> sh) & m1) | ((s0 >> (sh+2)) & m2),  m = ((Q >> shm) & m1) | ((s1 >> (sh+2)) & m2)
    const u32 s0 = st.hdr[r].y, s1 = st.hdr[r].z, s2 = st.hdr[r].w;
    const u32 P = ln.upper ? s2 : s0, Q = ln.upper ? s2 : s1;
    const u32 scp = ((P >> ln.sh) & ln.m1) | ((s0 >> ln.sh2) & ln.m2);
    const u32 mp = ((Q >> ln.shm) & ln.m1) | ((s1 >> ln.sh2) & ln.m2);
    const float dsl = d24 * ubyte_f<0>(scp), dsh = d20 * ubyte_f<1>(scp);
    const float dml = dmin * ubyte_f<0>(mp), dmh = dmin * ubyte_f<1>(mp);
    const u32 qd[8] = {st.q0[r].x, st.q0[r].y, st.q0[r].z, st.q0[r].w, st.q1[r].x, st.q1[r].y, st.q1[r].z, st.q1[r].w};
    const u32 hd[8] = {st.h0[r].x, st.h0[r].y, st.h0[r].z, st.h0[r].w, st.h1[r].x, st.h1[r].y, st.h1[r].z, st.h1[r].w};
    float dl[MG][2], dh[MG][2];   // two chains each to shorten the dependency
#pragma unroll
    for (int mm = 0; mm < MG; mm++) dl[mm][0] = dl[mm][1] = dh[mm][0] = dh[mm][1] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const u32 q = qd[i], q8 = q >> 8;
      u32 t0 = q & 0x000F000Fu;    // low nibbles of bytes 0,2   (x 2^-24)
      u32 t1 = q & 0x00F000F0u;    // high nibbles of bytes 0,2  (x 2^-20)
      u32 t2 = q8 & 0x000F000Fu;   // low nibbles of bytes 1,3
      u32 t3 = q8 & 0x00F000F0u;   // high nibbles of bytes 1,3
      if (Q5) {
        const u32 tq = hd[i] >> (2 * ln.g);  // per byte: bit 0 -> 5th bit of the low element, bit 1 -> high element
        t0 |= (tq << 4) & 0x00100010u;
        t2 |= (tq >> 4) & 0x00100010u;
        t1 |= (tq << 7) & 0x01000100u;
        t3 |= (tq >> 1) & 0x01000100u;
      }
#pragma unroll
      for (int mm = 0; mm < MG; mm++) {
        dl[mm][i & 1] = mix2(t0, xr[mm][i].x, xr[mm][i].z, dl[mm][i & 1]);
        dl[mm][i & 1] = mix2(t2, xr[mm][i].y, xr[mm][i].w, dl[mm][i & 1]);
        dh[mm][i & 1] = mix2(t1, xr[mm][8 + i].x, xr[mm][8 + i].z, dh[mm][i & 1]);
        dh[mm][i & 1] = mix2(t3, xr[mm][8 + i].y, xr[mm][8 + i].w, dh[mm][i & 1]);
      }
    }
#pragma unroll
    for (int mm = 0; mm < MG; mm++) {
      const float dl0 = dl[mm][0], dl1 = dl[mm][1], dh0 = dh[mm][0], dh1 = dh[mm][1];
      float v = fmaf(dsl, dl0 + dl1, -(dml * sx[mm][0]));
      v = fmaf(dsh, dh0 + dh1, v);
      c[mm] = fmaf(-dmh, sx[mm][1], v);
    }
  }
};

// ---------------------------------------------------------------------------------------------
// Q6_K (210 B: ql[128], qh[64], scales:i8[16], d). Lane = (jb, n, v): block jb of the column set,
// 128-value half n, 16-byte slice v of the half's 32 "l" positions. With l = 16v+i:
//   A = ql[64n+l], B = ql[64n+32+l], H = qh[32n+l]
//   quarter k element 128n + 32k + l  <-  (A&15|H<<4&48, B&15|H<<2&48, A>>4|H&48, B>>4|H>>2&48)[k] - 32
//   scales sc[8n + v + 2k]
// x registers: float4 4k+c -> quarter k, l = 16v+4c..+3. Blocks are 2-byte aligned only; the
// 16-byte loads are issued at their natural addresses.
// ---------------------------------------------------------------------------------------------
struct FmtQ6K {
  static constexpr int BB = 210;
  static constexpr int BPS = 16;
  static constexpr int NF4 = 16;
  static constexpr int NSUM = 4;
  static constexpr int MG_MAX = 2;
  static constexpr int SPI = 1;
  static constexpr unsigned TYPE = 14;
  static constexpr int rows(int m) { return GEMV_ROWS_Q6K(m); }

  struct Lane {
    int jb, n, v;
    __device__ __forceinline__ explicit Lane(int lane) : jb(lane >> 2), n((lane & 3) >> 1), v(lane & 1) {}
  };
  template <int R>
  struct Stage {
    uint4 qa[R], qb[R], qh[R];
    uint2 sc[R];
    u32 d[R];
  };

  static __device__ __forceinline__ u32 nblocks(u32 in_dim) { return in_dim >> 8; }
  static __device__ __forceinline__ size_t row_bytes(u32 nb) { return (size_t)nb * BB; }
  static __device__ __forceinline__ u32 x_elem(u32 set, u32 l, u32 i) {
    return (set * 16 + (l >> 2)) * 256 + ((l & 3) >> 1) * 128 + (i >> 2) * 32 + (l & 1) * 16 + (i & 3) * 4;
  }
  static __device__ __forceinline__ float4 load_x(const float* xrow, u32 e, u32 in_dim) {
    return e < in_dim ? ldx4(xrow + e) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  // As FmtK45::swz for this lane mapping: piece index = jb * 64 + n * 32 + (i >> 2) * 8 + v * 4 + (i & 3), so the
  // 16 lanes served together differ in jb & 3, n and v; v already selects bit 2, n goes to bit 3, jb & 3 to bits 0-1.
  static __device__ __forceinline__ u32 swz(u32 p) { return p ^ ((((p >> 5) & 1u) << 3) | ((p >> 6) & 3u)); }

  template <int R>
  static __device__ __forceinline__ void load(Stage<R>& st, const uint8_t* const (&rowp)[R], const Lane& ln,
                                              u32 set, u32 nb) {
#pragma unroll
    for (int r = 0; r < R; r++) load_row<R>(st, r, rowp[r], ln, set, nb);
  }
  template <int R>
  static __device__ __forceinline__ void load_row(Stage<R>& st, int r, const uint8_t* rp, const Lane& ln, u32 set,
                                                  u32 nb) {
    const u32 off = min(set * 16 + ln.jb, nb - 1) * BB;
    st.qa[r] = ld16(rp + (off + 64 * ln.n + 16 * ln.v));
    st.qb[r] = ld16(rp + (off + 64 * ln.n + 32 + 16 * ln.v));
    st.qh[r] = ld16(rp + (off + 128 + 32 * ln.n + 16 * ln.v));
    st.sc[r] = ld8(rp + (off + 192 + 8 * ln.n));
    st.d[r] = ld2(rp + (off + 208));
  }

  template <int R, int MG>
  static __device__ __forceinline__ void compute(const Stage<R>& st, int r, const Lane& ln,
                                                 const float4 (&xr)[MG][NF4], const float (&sx)[MG][NSUM],
                                                 float (&c)[MG]) {
    const float d = h2f(st.d[r]);
    // scale bytes v, v+2, v+4, v+6 of the half's eight
    const u32 s01 = st.sc[r].x >> (8 * ln.v), s23 = st.sc[r].y >> (8 * ln.v);
    const float sc0 = d * (float)(int)(signed char)(s01 & 0xFFu);
    const float sc1 = d * (float)(int)(signed char)((s01 >> 16) & 0xFFu);
    const float sc2 = d * (float)(int)(signed char)(s23 & 0xFFu);
    const float sc3 = d * (float)(int)(signed char)((s23 >> 16) & 0xFFu);
    const u32 a4[4] = {st.qa[r].x, st.qa[r].y, st.qa[r].z, st.qa[r].w};
    const u32 b4[4] = {st.qb[r].x, st.qb[r].y, st.qb[r].z, st.qb[r].w};
    const u32 h4[4] = {st.qh[r].x, st.qh[r].y, st.qh[r].z, st.qh[r].w};
    // 6-bit codes as pairs of binary16 subnormals: [k][c][0] = bytes 0,2, [k][c][1] = bytes 1,3 of dword c
    u32 q[4][4][2];
#pragma unroll
    for (int cc = 0; cc < 4; cc++) {
      const u32 A = a4[cc], B = b4[cc], H = h4[cc];
      const u32 A8 = A >> 8, B8 = B >> 8, Hl4 = H << 4, Hr4 = H >> 4, Hl2 = H << 2, Hr6 = H >> 6;
      q[0][cc][0] = (A & 0x000F000Fu) | (Hl4 & 0x00300030u);
      q[0][cc][1] = (A8 & 0x000F000Fu) | (Hr4 & 0x00300030u);
      q[1][cc][0] = (B & 0x000F000Fu) | (Hl2 & 0x00300030u);
      q[1][cc][1] = (B8 & 0x000F000Fu) | (Hr6 & 0x00300030u);
      q[2][cc][0] = (A & 0x00F000F0u) | (Hl4 & 0x03000300u);
      q[2][cc][1] = (A8 & 0x00F000F0u) | (Hr4 & 0x03000300u);
      q[3][cc][0] = (B & 0x00F000F0u) | (Hl2 & 0x03000300u);
      q[3][cc][1] = (B8 & 0x00F000F0u) | (Hr6 & 0x03000300u);
    }
#pragma unroll
    for (int mm = 0; mm < MG; mm++) {
      float dk[4];
#pragma unroll
      for (int k = 0; k < 4; k++) {
        float a = 0.0f;
#pragma unroll
        for (int cc = 0; cc < 4; cc++) {
          a = mix2(q[k][cc][0], xr[mm][4 * k + cc].x, xr[mm][4 * k + cc].z, a);
          a = mix2(q[k][cc][1], xr[mm][4 * k + cc].y, xr[mm][4 * k + cc].w, a);
        }
        dk[k] = a;
      }
      // sum (q-32) x = sum q x - 32 sum x; quarters 0,1 carry 2^-24, quarters 2,3 carry 2^-20
      float v = sc0 * fmaf(TWO_P24, dk[0], -32.0f * sx[mm][0]);
      v = fmaf(sc1, fmaf(TWO_P24, dk[1], -32.0f * sx[mm][1]), v);
      v = fmaf(sc2, fmaf(TWO_P20, dk[2], -32.0f * sx[mm][2]), v);
      c[mm] = fmaf(sc3, fmaf(TWO_P20, dk[3], -32.0f * sx[mm][3]), v);
    }
  }
};

// ---------------------------------------------------------------------------------------------
// Q8_0 (34 B: d, qs:i8[32]). Lane = (jb, hf): block jb of the column set (32 blocks = 1024 values),
// 16-byte half hf of its codes. Signed codes are read as unsigned with the top bit flipped:
// sum q x = sum (q^0x80) x - 128 sum x. in_dim may end inside a block (the tail is clipped).
// ---------------------------------------------------------------------------------------------
struct FmtQ80 {
  static constexpr int BB = 34;
  static constexpr int BPS = 32;
  static constexpr int NF4 = 4;
  static constexpr int NSUM = 1;
  static constexpr int MG_MAX = 4;
  static constexpr int SPI = 2;   // sets per iteration: a column set is 1024 values
  static constexpr unsigned TYPE = 8;
  static constexpr int rows(int m) { return GEMV_ROWS_Q80(m); }

  struct Lane {
    int jb, hf;
    __device__ __forceinline__ explicit Lane(int lane) : jb(lane >> 1), hf(lane & 1) {}
  };
  template <int R>
  struct Stage {
    uint4 qs[R];
    u32 d[R];
  };
  static __device__ __forceinline__ u32 swz(u32 p) { return p; }   // (no direct staging for this format)

  static __device__ __forceinline__ u32 nblocks(u32 in_dim) { return (in_dim + 31) >> 5; }
  static __device__ __forceinline__ size_t row_bytes(u32 nb) { return (size_t)nb * BB; }
  static __device__ __forceinline__ u32 x_elem(u32 set, u32 l, u32 i) {
    return (set * 32 + (l >> 1)) * 32 + (l & 1) * 16 + i * 4;
  }
  static __device__ __forceinline__ float4 load_x(const float* xrow, u32 e, u32 in_dim) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (e + 4 <= in_dim) {
      v = ldx4(xrow + e);
    } else {  // clipped tail of the last block
      if (e + 0 < in_dim) v.x = xrow[e + 0];
      if (e + 1 < in_dim) v.y = xrow[e + 1];
      if (e + 2 < in_dim) v.z = xrow[e + 2];
    }
    return v;
  }

  template <int R>
  static __device__ __forceinline__ void load(Stage<R>& st, const uint8_t* const (&rowp)[R], const Lane& ln,
                                              u32 set, u32 nb) {
#pragma unroll
    for (int r = 0; r < R; r++) load_row<R>(st, r, rowp[r], ln, set, nb);
  }
  template <int R>
  static __device__ __forceinline__ void load_row(Stage<R>& st, int r, const uint8_t* rp, const Lane& ln, u32 set,
                                                  u32 nb) {
    const u32 off = min(set * 32 + ln.jb, nb - 1) * BB;
    st.qs[r] = ld16(rp + (off + 2 + 16 * ln.hf));
    st.d[r] = ld2(rp + off);
  }

  template <int R, int MG>
  static __device__ __forceinline__ void compute(const Stage<R>& st, int r, const Lane&,
                                                 const float4 (&xr)[MG][NF4], const float (&sx)[MG][NSUM],
                                                 float (&c)[MG]) {
    const float d24 = h2f(st.d[r]) * TWO_P24, d = h2f(st.d[r]);
    const u32 qd[4] = {st.qs[r].x ^ 0x80808080u, st.qs[r].y ^ 0x80808080u, st.qs[r].z ^ 0x80808080u,
                       st.qs[r].w ^ 0x80808080u};
#pragma unroll
    for (int mm = 0; mm < MG; mm++) {
      float a = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; i++) {
        a = mix2(qd[i] & 0x00FF00FFu, xr[mm][i].x, xr[mm][i].z, a);         // bytes 0,2 as code * 2^-24
        a = mix2((qd[i] >> 8) & 0x00FF00FFu, xr[mm][i].y, xr[mm][i].w, a);  // bytes 1,3
      }
      c[mm] = fmaf(d24, a, -128.0f * (d * sx[mm][0]));
    }
  }
};

// ---------------------------------------------------------------------------------------------
// silu(g) * u in fp32: g / (1 + exp(-g)), then times u (bin/cuda_ffn_sequence_probe.cr:189-191)
__device__ __forceinline__ float swiglu_one(float g, float u) {
  const float s = g / (1.0f + expf(-g));
  return s * u;
}

// DUAL: two matrices of the same shape share the activations in one launch; output row r of the launch is
// row r of w / out for r < out_dim and row r - out_dim of w_b / out_b above (the reference's
// q4_k_dual_gemv_warp4_f32, src/ml/cuda/kernels/q4k_dual_gemv_probe.ptx:5-52, used for the gate | up and
// similar projection pairs, src/ml/cuda/qwen_recurrent_layer_runner.cr:519-520).
// SWIGLU (with DUAL, M = 1): a wavefront takes R/2 rows of w (gate) and the same R/2 rows of w_b (up) and stores
// silu(gate) * up into out - the reference's gate/up GEMVs followed by its swiglu_f32 kernel
// (bin/cuda_ffn_sequence_probe.cr:46-84) in one launch.
// TOP1: instead of the row values the workgroup stores, per token, the largest of its rows and that row's index
// (out[m * gridDim.x + blockIdx.x], top_ids[same]); of equal values the lowest row wins. The reference's
// q6_k_gemv_top1_partial_f32 (src/ml/cuda/kernels/q6k_gemv_probe.ptx:1331-1580) for the output head.
template <class F, int M, bool ADD, bool DUAL = false, bool SWIGLU = false, bool TOP1 = false>
__device__ __forceinline__ void gemv_core(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                          const float* __restrict__ residual, float* __restrict__ out,
                                          u32 in_dim, u32 out_dim, const uint8_t* __restrict__ w_b = nullptr,
                                          float* __restrict__ out_b = nullptr, u32* __restrict__ top_ids = nullptr) {
  constexpr int R = F::rows(M);
  constexpr int MG = M < F::MG_MAX ? M : F::MG_MAX;   // tokens held in registers at a time
  constexpr int NG = (M + MG - 1) / MG;
  constexpr int NF4 = F::NF4, NSUM = F::NSUM;
  constexpr int SET_F4 = NF4 * 64;                     // float4 per token and column set
  extern __shared__ float4 xs[];                       // [token][set in chunk][float4 index][lane]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const typename F::Lane ln(lane);
  const u32 nb = F::nblocks(in_dim);
  const u32 ncs = (nb + F::BPS - 1) / F::BPS;
  // K-quants with one token group: the activations go global -> LDS directly (no registers), sums from registers
  constexpr bool DIRECT = gemv_direct_x(F::TYPE, NG);
  // column sets staged in LDS at a time (the host sizes the dynamic LDS with the same formula);
  // with several token groups each set is staged per group
  const u32 CH = NG > 1 ? 1u : (u32)(DIRECT ? gemv_chunk_sets_direct(MG * SET_F4, ncs) : gemv_chunk_sets(MG * SET_F4, ncs));
  const size_t row_bytes = F::row_bytes(nb);
  static_assert(!SWIGLU || (DUAL && M == 1 && !ADD && R % 2 == 0), "SWIGLU is a one-token mode of the matrix pair");
  static_assert(!TOP1 || (!DUAL && !ADD), "TOP1 is a mode of the plain GEMV");
  const u32 total_rows = DUAL ? 2 * out_dim : out_dim;
  // A workgroup takes the row groups blockIdx.x, blockIdx.x + gridDim.x, ... (GEMV_WAVES * R rows each; with SWIGLU
  // half as many rows of each matrix); a grid of one workgroup per group is the plain case.
  const u32 group_rows = SWIGLU ? GEMV_WAVES * R / 2 : GEMV_WAVES * R;
  const u32 ngroups = ((SWIGLU ? out_dim : total_rows) + group_rows - 1) / group_rows;
  u32 row0 = (blockIdx.x * GEMV_WAVES + wave) * R;
  const uint8_t* rowp[R];
  auto set_group = [&](u32 grp) {
    row0 = (grp * GEMV_WAVES + wave) * R;
#pragma unroll
    for (int r = 0; r < R; r++) {
      if (SWIGLU) {   // slots 0 .. R/2-1: gate rows, slots R/2 .. R-1: the same rows of up
        const u32 row = min(row0 / 2 + (u32)(r % (R / 2)), out_dim - 1);
        rowp[r] = (r < R / 2 ? w : w_b) + (size_t)row * row_bytes;
      } else {
        const u32 row = min(row0 + r, total_rows - 1);
        rowp[r] = (DUAL && row >= out_dim) ? w_b + (size_t)(row - out_dim) * row_bytes : w + (size_t)row * row_bytes;
      }
    }
  };
  set_group(blockIdx.x);

  float acc[R][M];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int m = 0; m < M; m++) acc[r][m] = 0.0f;

  float* xsum = reinterpret_cast<float*>(xs + (size_t)(MG * SET_F4) * CH);   // [token][set in chunk][k][lane]
  constexpr int FU = 4;                                 // float4 a thread keeps in flight while staging
  const u32 stage_n = (u32)(MG * SET_F4) * CH;          // float4 staged per chunk and token group

  // Staging of the activations of column sets [s0, s0+CH), token group mg, is split in two so that
  // the global loads of x can be issued ahead of the weight loads (loads return in order, and x is
  // needed first): stage_begin issues the first FU loads per thread, stage_end stores them, handles the
  // rest, and builds the per-lane sums.
  auto stage_addr = [&](u32 idx, u32 s0, int mg, const float*& xrow, u32& e) -> bool {
    const u32 l = idx & 63, i = (idx >> 6) % NF4, cm = idx / SET_F4;
    const u32 cset = s0 + cm % CH, m = mg * MG + cm / CH;
    xrow = x + (size_t)m * in_dim;
    e = F::x_elem(cset, l, i);
    return cset < ncs && m < (u32)M;
  };
  auto stage_begin = [&](u32 s0, int mg, float4 (&buf)[FU]) {
#pragma unroll
    for (int k = 0; k < FU; k++) {
      const u32 idx = tid + k * GEMV_BLOCK;
      const float* xrow;
      u32 e;
      buf[k] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (idx < stage_n && stage_addr(idx, s0, mg, xrow, e)) buf[k] = F::load_x(xrow, e, in_dim);
    }
  };
  auto stage_end = [&](u32 s0, int mg, const float4 (&buf)[FU]) {
    __syncthreads();   // every wavefront is done with the previous contents
#pragma unroll
    for (int k = 0; k < FU; k++) {
      const u32 idx = tid + k * GEMV_BLOCK;
      if (idx < stage_n) xs[idx] = buf[k];
    }
    for (u32 idx = tid + FU * GEMV_BLOCK; idx < stage_n; idx += GEMV_BLOCK) {
      const float* xrow;
      u32 e;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (stage_addr(idx, s0, mg, xrow, e)) v = F::load_x(xrow, e, in_dim);
      xs[idx] = v;
    }
    __syncthreads();
    // per-lane sums of the staged activations, one per scale group of the lane
    for (u32 idx = tid; idx < (u32)(MG * NSUM * 64) * CH; idx += GEMV_BLOCK) {
      const u32 l = idx & 63, k = (idx >> 6) % NSUM, cm = idx / (NSUM * 64);
      float a = 0.0f;
#pragma unroll
      for (int i = 0; i < NF4 / NSUM; i++) a += hsum4(xs[(cm * NF4 + k * (NF4 / NSUM) + i) * 64 + l]);
      xsum[idx] = a;
    }
    __syncthreads();
  };

  // Staging of the chunk of column sets that starts at s0 for the kernels with one token group (DIRECT): the LDS image
  // of a (token, set) is its 16 KiB in natural order up to F::swz, 1024 float4 = 4 per thread, read from global memory
  // 1 KiB per wavefront and instruction. Every float4 of the chunk is requested before anything else happens (up to 12
  // per thread, in registers that are free this early), `between` then requests the first weight rows, and the values
  // are stored to LDS: the wait in front of the stores is a register dependency, so the compiler counts the younger
  // loads and the weight rows stay in flight across the barrier. Sets past the end of the row are replaced by the
  // row's last float4; the lanes that would use them are masked out of the sums by `valid`.
  constexpr int CHC = gemv_chunk_sets_direct(MG * SET_F4, 2);   // sets per chunk of a row longer than one set
  auto stage_rounds = [&](u32 s0, auto rounds, auto&& between) {
    constexpr int NR = decltype(rounds)::value, PER_TOKEN = NR / MG;
    float4 buf[NR * 4];
#pragma unroll
    for (int q = 0; q < NR; q++) {
      const u32 cset = min(s0 + (u32)(q % PER_TOKEN), ncs - 1);
      const float* xrow = x + (size_t)(q / PER_TOKEN) * in_dim;
#pragma unroll
      for (int k = 0; k < 4; k++)
        buf[q * 4 + k] = ldx4(xrow + min((cset * 1024u + F::swz(k * GEMV_BLOCK + tid)) * 4u, in_dim - 4));
    }
    between();
#pragma unroll
    for (int q = 0; q < NR; q++)
#pragma unroll
      for (int k = 0; k < 4; k++) xs[q * 1024 + k * GEMV_BLOCK + tid] = buf[q * 4 + k];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  auto stage_chunk = [&](u32 s0, auto&& between) {
    if (ncs == 1) stage_rounds(s0, std::integral_constant<int, MG>{}, between);
    else stage_rounds(s0, std::integral_constant<int, MG * CHC>{}, between);
  };
  // The same chunk one (token, set) at a time, for the places where many registers are live: the later chunks of a
  // row that is longer than one chunk.
  auto stage_chunk_serial = [&](u32 s0) {
    for (u32 q = 0; q < (u32)MG * CH; q++) {
      const u32 cset = min(s0 + q % CH, ncs - 1);
      const float* xrow = x + (size_t)(q / CH) * in_dim;
#pragma unroll 1
      for (u32 k = 0; k < 4; k++)   // (one float4 at a time: this runs with most registers taken)
        xs[q * 1024 + k * GEMV_BLOCK + tid] = ldx4(xrow + min((cset * 1024u + F::swz(k * GEMV_BLOCK + tid)) * 4u, in_dim - 4));
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  const u32 lane_byte = F::swz(F::x_elem(0, lane, 0) >> 2) << 4;   // byte offset of the lane's first piece in the image
  auto read_x = [&](u32 s, float4 (&xr)[MG][NF4], float (&sx)[MG][NSUM]) {
    // (one XOR per address, formed here every time: left to itself the compiler keeps the 16 addresses in registers
    // for the whole kernel, which the pipeline below cannot spare)
    u32 lb = lane_byte;
    asm volatile("" : "+v"(lb));
    const char* xsb = reinterpret_cast<const char*>(xs);
#pragma unroll
    for (int mm = 0; mm < MG; mm++) {
      const u32 cm = mm * CH + (s % CH);
#pragma unroll
      for (int i = 0; i < NF4; i++) {
        // direct image: the lane's pieces differ from its first in bits the swizzle neither reads nor writes
        if constexpr (DIRECT) xr[mm][i] = *reinterpret_cast<const float4*>(xsb + ((lb + cm * 16384u) ^ ((F::x_elem(0, 0, i) >> 2) << 4)));
        else xr[mm][i] = xs[(cm * NF4 + i) * 64 + lane];
      }
#pragma unroll
      for (int k = 0; k < NSUM; k++) {
        if constexpr (DIRECT) {
          float a = 0.0f;
#pragma unroll
          for (int i = 0; i < NF4 / NSUM; i++) a += hsum4(xr[mm][k * (NF4 / NSUM) + i]);
          sx[mm][k] = a;
        } else {
          sx[mm][k] = xsum[(cm * NSUM + k) * 64 + lane];
        }
      }
    }
  };

  auto step = [&](const typename F::template Stage<R>& st, u32 s) {
    const bool valid = s * F::BPS + ln.jb < nb;
#pragma unroll
    for (int mg = 0; mg < NG; mg++) {
      if (NG > 1) {   // several token groups share the weight registers: stage each group in turn
        float4 buf[FU];
        stage_begin(s, mg, buf);
        stage_end(s, mg, buf);
      }
      float4 xr[MG][NF4];
      float sx[MG][NSUM];
      read_x(s, xr, sx);
#pragma unroll
      for (int r = 0; r < R; r++) {
        float c[MG];
        F::template compute<R, MG>(st, r, ln, xr, sx, c);
#pragma unroll
        for (int mm = 0; mm < MG; mm++)
          if (mg * MG + mm < M) acc[r][mg * MG + mm] += valid ? c[mm] : 0.0f;
      }
    }
  };

  // end of a row group: the lanes' partial sums become row values, which are stored (or, with TOP1, compared)
  float top_best[M];
  u32 top_best_id[M];
#pragma unroll
  for (int m = 0; m < M; m++) top_best[m] = -__builtin_inff(), top_best_id[m] = 0;
  auto finish = [&](u32 row0) {
    if constexpr (SWIGLU) {
      float v[R];
#pragma unroll
      for (int r = 0; r < R; r++) v[r] = wave_sum(acc[r][0]);
#pragma unroll
      for (int r = 0; r < R / 2; r++) {
        const u32 row = row0 / 2 + r;
        if (lane == 0 && row < out_dim) out[row] = swiglu_one(v[r], v[r + R / 2]);
      }
    } else if constexpr (TOP1) {
#pragma unroll
      for (int m = 0; m < M; m++) {
#pragma unroll
        for (int r = 0; r < R; r++) {
          const float v = wave_sum(acc[r][m]);
          if (row0 + r < out_dim && v > top_best[m]) top_best[m] = v, top_best_id[m] = row0 + r;   // rows ascend
        }
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; r++) {
#pragma unroll
        for (int m = 0; m < M; m++) {
          float v = wave_sum(acc[r][m]);
          const u32 row = row0 + r;
          if (lane == 0 && row < total_rows) {
            if (DUAL && row >= out_dim) {
              out_b[(size_t)m * out_dim + (row - out_dim)] = v;
            } else {
              const size_t o = (size_t)m * out_dim + row;
              if (ADD) v += residual[o];
              out[o] = v;
            }
          }
        }
      }
    }
  };
  // TOP1: the wavefronts' winners meet in LDS; within a wavefront and from wavefront to wavefront the rows ascend,
  // so "greater than" keeps the lowest row among equal values
  auto top1_store = [&]() {
    __shared__ float top_v[M][GEMV_WAVES];
    __shared__ u32 top_i[M][GEMV_WAVES];
    if (lane == 0) {
#pragma unroll
      for (int m = 0; m < M; m++) top_v[m][wave] = top_best[m], top_i[m][wave] = top_best_id[m];
    }
    __syncthreads();
    if (tid < M) {
      float best = top_v[tid][0];
      u32 best_id = top_i[tid][0];
#pragma unroll
      for (int wv = 1; wv < GEMV_WAVES; wv++)
        if (top_v[tid][wv] > best || (top_v[tid][wv] == best && top_i[tid][wv] < best_id)) best = top_v[tid][wv], best_id = top_i[tid][wv];
      out[(size_t)tid * gridDim.x + blockIdx.x] = best;
      top_ids[(size_t)tid * gridDim.x + blockIdx.x] = best_id;
    }
  };

  // (one token only: with two the registers no longer allow it)
  constexpr bool PIPE = M == 1 && NG == 1 && F::SPI == 1 && DIRECT;
  if constexpr (PIPE) {
    // Rolling pipeline over (column set, row): PF rows are in flight while one is consumed. A compute unit
    // accepts only so many loads at a time and serves its oldest wavefronts first, so a wavefront that
    // queues all its loads up front sits in the issue of them, and the ones served last still have all
    // their arithmetic to do when the last byte arrives. Here the arithmetic of a row starts as soon as
    // that row is there, and what is left after the last byte is one row's worth.
    constexpr int PF = R >= 3 ? 2 : 1;
    typename F::template Stage<R> st;
    // The first rows are requested only once the activations are staged: a compute unit returns loads in order, and
    // weight loads (HBM misses) issued ahead of the barrier hold up the activation loads (L2 hits) of the wavefronts
    // that issue theirs a little later - measured 8.05-8.25 us with the rows requested before the barrier, 7.75 after.
    stage_chunk(0, [&]() {});
#pragma unroll
    for (int r = 0; r < PF; r++) F::template load_row<R>(st, r, rowp[r], ln, 0, nb);
    // one column set; `last` (a compile-time tag) says that no column set follows, so the prefetches that
    // would wrap into the next set are left out and the number of loads in flight stays a constant
    auto column_set = [&](u32 s, auto last) {
      if (s > 0 && (s % CH) == 0) {
        __builtin_amdgcn_s_barrier();   // every wavefront has read the previous chunk into registers
        stage_chunk_serial(s);
      }
      const bool valid = s * F::BPS + ln.jb < nb;
      float4 xr[MG][NF4];
      float sx[MG][NSUM];
      read_x(s, xr, sx);
#pragma unroll
      for (int r = 0; r < R; r++) {
        const int rr = (r + PF) % R;
        if (r + PF < R) F::template load_row<R>(st, rr, rowp[rr], ln, s, nb);
        else if constexpr (!decltype(last)::value) F::template load_row<R>(st, rr, rowp[rr], ln, s + 1, nb);
        __builtin_amdgcn_sched_barrier(0);
        float c[MG];
        F::template compute<R, MG>(st, r, ln, xr, sx, c);
#pragma unroll
        for (int mm = 0; mm < MG; mm++) acc[r][mm] += valid ? c[mm] : 0.0f;
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // The row groups of this workgroup. The first rows of the first group are in flight already (requested above,
    // between the request for the activations and their way into LDS); a later group requests them at the top of the
    // loop, after staging its first chunk of activations again if the row is longer than one chunk (otherwise the
    // activations stay where they are).
    for (u32 grp = blockIdx.x;;) {
      if (grp != blockIdx.x) {
        if (ncs > CH) {
          __builtin_amdgcn_s_barrier();   // every wavefront has read the last chunk into registers
          stage_chunk_serial(0);
        }
#pragma unroll
        for (int r = 0; r < PF; r++) F::template load_row<R>(st, r, rowp[r], ln, 0, nb);
      }
      for (u32 s = 0; s + 1 < ncs; s++) column_set(s, gemv_false{});
      column_set(ncs - 1, gemv_true{});
      grp += gridDim.x;
      if (grp >= ngroups) break;
      finish(row0);
#pragma unroll
      for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < M; m++) acc[r][m] = 0.0f;
      set_group(grp);
    }
  }
  // Column sets are taken F::SPI at a time: all their weight loads are issued before the first is consumed. Directly
  // staged activations of one token group (two tokens of a K-quant): the workgroup walks the row groups blockIdx.x,
  // blockIdx.x + gridDim.x, ... and stages the activations again only if the row is longer than one chunk.
  if constexpr (!PIPE) {
    constexpr bool WALK = DIRECT && NG == 1;
    for (u32 grp = blockIdx.x;;) {
      const bool first = grp == blockIdx.x;
      for (u32 s = 0; s < ncs; s += F::SPI) {
        const bool restage = NG == 1 && (s % CH) == 0 && (first || ncs > CH);   // CH is a multiple of SPI or covers the whole row
        typename F::template Stage<R> stA, stB;
        const bool two = F::SPI == 2 && s + 1 < ncs;
        if constexpr (DIRECT) {
          auto rows = [&]() { F::template load<R>(stA, rowp, ln, s, nb); };   // (SPI is 1 for these formats)
          if (restage) {
            if (s > 0 || !first) __builtin_amdgcn_s_barrier();   // every wavefront has read the previous chunk into registers
            stage_chunk(s, [&]() {});   // (rows after the barrier, as in the one-token pipeline)
            rows();
          } else {
            rows();
          }
        } else {
          float4 buf[FU];
          if (restage) stage_begin(s, 0, buf);
          F::template load<R>(stA, rowp, ln, s, nb);
          if (two) F::template load<R>(stB, rowp, ln, s + 1, nb);
          if (restage) stage_end(s, 0, buf);
        }
        step(stA, s);
        if (two) step(stB, s + 1);
      }
      if (!WALK) break;
      grp += gridDim.x;
      if (grp >= ngroups) break;
      finish(row0);
#pragma unroll
      for (int r = 0; r < R; r++)
#pragma unroll
        for (int m = 0; m < M; m++) acc[r][m] = 0.0f;
      set_group(grp);
    }
  }
  finish(row0);
  if constexpr (TOP1) top1_store();
}

// ---- entry points ---------------------------------------------------------------------------
// M = 1, 2: ask for at least 3 wavefronts per SIMD so a 12288-row matrix is resident in one round
#define GEMV_OCC(M) __attribute__((amdgpu_waves_per_eu((M) <= 1 ? 3 : 1)))
#define GEMV_ENTRY(NAME, FMT, M)                                                                                \
  extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(M) void NAME(const uint8_t* w, const float* x, float* out,   \
                                                                 u32 in_dim, u32 out_dim) {                     \
    gemv_core<FMT, M, false>(w, x, nullptr, out, in_dim, out_dim);                                              \
  }
#define GEMV_ADD_ENTRY(NAME, FMT, M)                                                                            \
  extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(M) void NAME(const uint8_t* w, const float* x,               \
                                                                 const float* residual, float* out, u32 in_dim, \
                                                                 u32 out_dim) {                                 \
    gemv_core<FMT, M, true>(w, x, residual, out, in_dim, out_dim);                                              \
  }

#define GEMV_FAMILY(PFX, FMT)                        \
  GEMV_ENTRY(PFX##_gemv_f32, FMT, 1)                 \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch2, FMT, 2)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch3, FMT, 3)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch4, FMT, 4)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch5, FMT, 5)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch6, FMT, 6)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch7, FMT, 7)         \
  GEMV_ENTRY(PFX##_gemv_f32_tbatch8, FMT, 8)         \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32, FMT, 1)         \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch2, FMT, 2) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch3, FMT, 3) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch4, FMT, 4) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch5, FMT, 5) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch6, FMT, 6) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch7, FMT, 7) \
  GEMV_ADD_ENTRY(PFX##_gemv_add_f32_tbatch8, FMT, 8)

// (w_raw, x, partial_ids, partial_values, in_dim, out_dim): the reference's parameter order
// (src/ml/cuda/kernels/q6k_gemv_probe.ptx:1331-1338); same grid, block and dynamic shared memory as the GEMV of the
// same type and token count, partial_*[token * grid + workgroup].
#define GEMV_TOP1_ENTRY(NAME, FMT, M)                                                                            \
  extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(M) void NAME(const uint8_t* w, const float* x, u32* partial_ids, \
                                                                 float* partial_values, u32 in_dim, u32 out_dim) { \
    gemv_core<FMT, M, false, false, false, true>(w, x, nullptr, partial_values, in_dim, out_dim, nullptr, nullptr, \
                                                 partial_ids);                                                   \
  }

typedef FmtK45<false> FmtQ4K;
typedef FmtK45<true> FmtQ5K;
GEMV_FAMILY(q4_k, FmtQ4K)
GEMV_FAMILY(q5_k, FmtQ5K)
GEMV_FAMILY(q6_k, FmtQ6K)
GEMV_FAMILY(q8_0, FmtQ80)
GEMV_TOP1_ENTRY(q4_k_gemv_top1_partial_f32, FmtQ4K, 1)
GEMV_TOP1_ENTRY(q4_k_gemv_top1_partial_f32_tbatch2, FmtQ4K, 2)
GEMV_TOP1_ENTRY(q4_k_gemv_top1_partial_f32_tbatch3, FmtQ4K, 3)
GEMV_TOP1_ENTRY(q5_k_gemv_top1_partial_f32, FmtQ5K, 1)
GEMV_TOP1_ENTRY(q6_k_gemv_top1_partial_f32, FmtQ6K, 1)
GEMV_TOP1_ENTRY(q6_k_gemv_top1_partial_f32_tbatch2, FmtQ6K, 2)
GEMV_TOP1_ENTRY(q6_k_gemv_top1_partial_f32_tbatch3, FmtQ6K, 3)
GEMV_TOP1_ENTRY(q8_0_gemv_top1_partial_f32, FmtQ80, 1)

// (partial_ids, partial_values, out_ids, out_values, count): the largest of `count` partial values and its id, per
// token (grid.x = tokens; partial_* + token * count, out_* + token). Of equal values the lowest id wins, which is
// what the reference's CPU scan gives (bin/cuda_mixed_stack_probe.cr:1485-1497); its device reduce is
// output_top1_values_reduce_probe (src/ml/cuda/qwen_output_head_runner.cr:530-612). block = 1024.
#define TOP1_REDUCE_BLOCK 1024
__device__ __forceinline__ void top1_take(float& best, u32& best_id, float v, u32 id) {
  if (v > best || (v == best && id < best_id)) best = v, best_id = id;
}
extern "C" __global__ __launch_bounds__(TOP1_REDUCE_BLOCK) void top1_reduce_f32(const u32* partial_ids,
                                                                                const float* partial_values, u32* out_ids,
                                                                                float* out_values, u32 count) {
  __shared__ float sv[TOP1_REDUCE_BLOCK / WAVE];
  __shared__ u32 si[TOP1_REDUCE_BLOCK / WAVE];
  const u32* ids = partial_ids + (size_t)blockIdx.x * count;
  const float* vals = partial_values + (size_t)blockIdx.x * count;
  float best = -__builtin_inff();
  u32 best_id = 0xFFFFFFFFu;
  for (u32 i = threadIdx.x; i < count; i += TOP1_REDUCE_BLOCK) top1_take(best, best_id, vals[i], ids[i]);
#pragma unroll
  for (int d = 1; d < WAVE; d <<= 1) {
    const float ov = __shfl_xor(best, d, WAVE);
    const u32 oi = (u32)__shfl_xor((int)best_id, d, WAVE);
    top1_take(best, best_id, ov, oi);
  }
  if ((threadIdx.x & (WAVE - 1)) == 0) sv[threadIdx.x / WAVE] = best, si[threadIdx.x / WAVE] = best_id;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int wv = 1; wv < TOP1_REDUCE_BLOCK / WAVE; wv++) top1_take(best, best_id, sv[wv], si[wv]);
    out_ids[blockIdx.x] = best_id == 0xFFFFFFFFu ? 0u : best_id;   // nothing above -inf: id 0, as the CPU scan
    out_values[blockIdx.x] = best;
  }
}

// (w_raw_a, w_raw_b, x, out_a, out_b, in_dim, out_dim): one token per grid.y slice (x + y * in_dim, out_* + y * out_dim),
// grid.x = ceil(2 * out_dim / rows per workgroup), same block and dynamic shared memory as q4_k_gemv_f32.
// The reference has this pair as q4_k_dual_gemv_warp4_f32 and ..._batched (q4k_dual_gemv_probe.ptx:5, 233).
extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(1) void q4_k_dual_gemv_f32(
    const uint8_t* w_a, const uint8_t* w_b, const float* x, float* out_a, float* out_b, u32 in_dim, u32 out_dim) {
  const size_t tok = blockIdx.y;
  gemv_core<FmtQ4K, 1, false, true>(w_a, x + tok * in_dim, nullptr, out_a + tok * out_dim, in_dim, out_dim, w_b,
                                    out_b + tok * out_dim);
}

// (w_gate, w_up, x, out, in_dim, out_dim): out[o] = silu(gate[o]) * up[o] for one token per grid.y slice; block and
// dynamic shared memory as q4_k_gemv_f32, grid.x = ceil(out_dim / (rows per workgroup / 2)).
extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(1) void q4_k_dual_gemv_swiglu_f32(
    const uint8_t* w_gate, const uint8_t* w_up, const float* x, float* out, u32 in_dim, u32 out_dim) {
  const size_t tok = blockIdx.y;
  gemv_core<FmtQ4K, 1, false, true, true>(w_gate, x + tok * in_dim, nullptr, out + tok * out_dim, in_dim, out_dim, w_up,
                                          nullptr);
}

// (gate, up, out, n): out[i] = silu(gate[i]) * up[i], the reference's swiglu_f32 (bin/cuda_ffn_sequence_probe.cr:46-84).
// block = 256, grid = ceil(n / 256).
extern "C" __global__ __launch_bounds__(256) void swiglu_f32(const float* gate, const float* up, float* out, u32 n) {
  const u32 i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = swiglu_one(gate[i], up[i]);
}
