// Block formats of the decode GEMV kernels: for each GGUF type the lane mapping inside a column set, the loads of a
// lane's share of a row, and the arithmetic on it. Shared by the kernels of gemv.hpp and gemv_stream.hpp.
//
// A wavefront walks a row in "column sets": the span of blocks the 64 lanes cover side by side (Q4_K/Q5_K/Q6_K: 4 lanes
// per 256-value super-block -> 16 blocks; Q8_0: 2 lanes per 32-value block -> 32 blocks), all loads 16 bytes per lane.
// A lane always sits at the same position inside a block, so the activations it needs for a column set are fixed.
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

