// Prefill GEMM over raw Q4_K weights: out[m][n] = (bias[n] +) sum_k x[m][k] * deq(W[n][k]), M >= 9.
// fp16 operands, v_mfma_f32_16x16x32_f16, fp32 accumulation (the precision of the reference's Metal
// prefill kernels, which round both x and the dequantized weights to half:
// src/ml/gguf/kernels/gemm_q4k.metal:97-105,678-686).
//
// Two kernels:
//   pack_x_f16_q4k  (x:f32 [m][in_dim], xp:f16, m:u32, in_dim:u32)           block 256, any grid
//   q4_k_gemm_f16   (w_raw, xp, bias|null, out:f32 [m][out_dim], in_dim:u32, out_dim:u32, m:u32)
//                   block 256, grid ceil(m/128) * ceil(out_dim/192), dynamic LDS 131072 bytes
//
// Tiling. A workgroup (4 wavefronts) owns 128 tokens x 192 weight rows; a wavefront owns all 128 tokens
// x 48 rows, so every weight is dequantized by exactly one wavefront of the workgroup and reused for
// 128 tokens, and 512 x 12288 gives 256 workgroups, one per CU. K is walked one 256-value super-block
// at a time, eight MFMA k-steps of 32.
//
// Weights never touch LDS: a lane holds 16-byte chunks of "its" weight row (row = lane % 16, k-group
// = lane / 16) and turns their nibbles into the MFMA B operand in registers. A masked dword
// (q & 0x000F000F) | 0x64006400 is the half2 (1024 + n0, 1024 + n4); subtracting 1024 and one packed
// fma give fp16(d*sc*n - dmin*m) for two weights. The eight k values a lane contributes to one k-step
// therefore come in nibble order (bytes 0,2,1,3,4,6,5,7 of eight consecutive bytes); pack_x_f16_q4k
// writes x in exactly that order, already laid out as the LDS image [k-step][token][k-group][8 halves]
// of each (128-token tile, super-block), so staging x is a straight 64 KiB copy and the A operand
// is one conflict-free ds_read_b128 per lane.
//
// The only LDS traffic is the activations: 8 KiB read per wavefront and k-step for 24 MFMAs.
// The x tile of the next super-block is copied global -> LDS while the current one is consumed
// (two 64 KiB buffers), and the raw weight chunks of the next super-block are prefetched into
// registers.
#pragma once
#include "common.cuh"

#define GEMM_BM 128
#define GEMM_BN 192
#define GEMM_WN 48          // weight rows per wavefront (3 column tiles of 16)
#define GEMM_LDS_BYTES 131072

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// Element (0..255) of a super-block that k-slot (kstep, kg, e) of the MFMA stands for.
// kstep = 4u + op: u = 64-byte half of the nibble array, op&1 = upper 8 bytes of the lane's chunk,
// op>>1 = high nibbles.
__device__ __forceinline__ u32 gemm_k_element(u32 kstep, u32 kg, u32 e) {
  const u32 u = kstep >> 2, op = kstep & 3;
  const u32 chunk = 4 * u + kg, g = chunk >> 1, h = chunk & 1;
  const u32 perm = ((e & 1) << 1) | ((e >> 1) & 1) | (e & 4);   // 0,2,1,3,4,6,5,7
  return 64 * g + 32 * (op >> 1) + 16 * h + 8 * (op & 1) + perm;
}

extern "C" __global__ __launch_bounds__(256) void pack_x_f16_q4k(const float* __restrict__ x, uint4* __restrict__ xp,
                                                                  u32 m, u32 in_dim) {
  const u32 nkb = in_dim >> 8;
  const u32 mtiles = (m + GEMM_BM - 1) / GEMM_BM;
  const u64 total = (u64)mtiles * nkb * 4096;   // 16-byte pieces
  const u64 step = (u64)gridDim.x * blockDim.x;
  for (u64 idx = (u64)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += step) {
    const u32 kg = idx & 3, tok = (idx >> 2) & 127, kstep = (idx >> 9) & 7;
    const u64 tile = idx >> 12;
    const u32 kb = (u32)(tile % nkb), mt = (u32)(tile / nkb);
    const u32 row = mt * GEMM_BM + tok;
    uint4 o = make_uint4(0u, 0u, 0u, 0u);
    if (row < m) {
      const float* src = x + (size_t)row * in_dim + kb * 256 + gemm_k_element(kstep, kg, 0);   // e = 0 is the base
      float4 a, b;
      __builtin_memcpy(&a, src, 16);
      __builtin_memcpy(&b, src + 4, 16);
      const __half2 p0 = __floats2half2_rn(a.x, a.z), p1 = __floats2half2_rn(a.y, a.w);
      const __half2 p2 = __floats2half2_rn(b.x, b.z), p3 = __floats2half2_rn(b.y, b.w);
      o.x = *reinterpret_cast<const u32*>(&p0);
      o.y = *reinterpret_cast<const u32*>(&p1);
      o.z = *reinterpret_cast<const u32*>(&p2);
      o.w = *reinterpret_cast<const u32*>(&p3);
    }
    xp[idx] = o;
  }
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

struct GemmRaw {   // raw bytes of one super-block of one weight row, as a lane sees them
  uint4 hdr, q0, q1;
};

extern "C" __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void q4_k_gemm_f16(const uint8_t* __restrict__ w,
                                                                 const uint4* __restrict__ xp,
                                                                 const float* __restrict__ bias,
                                                                 float* __restrict__ out, u32 in_dim, u32 out_dim,
                                                                 u32 m) {
  extern __shared__ uint4 lds[];   // 2 x [8 k-steps][128 tokens][4 k-groups] uint4
  const u32 tid = threadIdx.x, lane = tid & 63;
  const u32 wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const u32 j = lane & 15, kg = lane >> 4;
  const u32 nkb = in_dim >> 8;
  const u32 mtiles = (m + GEMM_BM - 1) / GEMM_BM;
  const u32 mt = blockIdx.x % mtiles, nt = blockIdx.x / mtiles;
  const u32 n0 = nt * GEMM_BN + wave * GEMM_WN;      // first weight row of this wavefront
  const size_t row_bytes = (size_t)nkb * 144;
  const u32 sh = 16u * (kg >> 1);

  // uniform base of the wavefront's rows + a 32-bit per-lane offset (48 rows are far below 4 GiB)
  const u32 base_row = min(n0, out_dim - 1);
  const uint8_t* wbase = w + (size_t)base_row * row_bytes;
  u32 rowoff[3];
#pragma unroll
  for (int c = 0; c < 3; c++) rowoff[c] = (min(n0 + 16 * c + j, out_dim - 1) - base_row) * (u32)row_bytes + 16 * kg;
  const uint4* xtile = xp + (size_t)mt * nkb * 4096;

  float4_t acc[8][3];
#pragma unroll
  for (int r = 0; r < 8; r++)
#pragma unroll
    for (int c = 0; c < 3; c++) acc[r][c] = (float4_t){0.f, 0.f, 0.f, 0.f};

  auto load_raw = [&](GemmRaw (&raw)[3], u32 kb) {
    const uint8_t* kbase = wbase + (size_t)kb * 144;   // uniform
#pragma unroll
    for (int c = 0; c < 3; c++) {
      raw[c].hdr = ld16(kbase + (rowoff[c] - 16 * kg));
      raw[c].q0 = ld16(kbase + (rowoff[c] + 16));
      raw[c].q1 = ld16(kbase + (rowoff[c] + 80));
    }
  };

  // stage super-block 0 of x and the first weights
  GemmRaw cur[3];
  load_raw(cur, 0);
#pragma unroll
  for (int i = 0; i < 16; i++) lds[tid + 256 * i] = (xtile + 256 * i)[tid];
  __syncthreads();

  for (u32 kb = 0; kb < nkb; kb++) {
    const u32 cb = (kb & 1) * 4096, nb_ = 4096 - cb;
    const u32 kn = min(kb + 1, nkb - 1);   // the last iteration re-reads its own tile; the copy is not used
    GemmRaw nxt[3];
    load_raw(nxt, kn);
    const uint4* xnext = xtile + (size_t)kn * 4096;   // uniform
    uint4 xbuf[16];
#pragma unroll
    for (int i = 0; i < 16; i++) xbuf[i] = (xnext + 256 * i)[tid];

    // per-row scales of this super-block as duplicated half2: [c][u][lo scale, lo -min, hi scale, hi -min]
    u32 S[3][2][4];
#pragma unroll
    for (int c = 0; c < 3; c++) {
      const float d = h2f(cur[c].hdr.x), dm = h2f(cur[c].hdr.x >> 16);
      const u32 a0 = cur[c].hdr.y >> sh, a1 = cur[c].hdr.z >> sh, a2 = cur[c].hdr.w >> sh;
      const u32 scL = a0 & 0x3F3Fu, mL = a1 & 0x3F3Fu;                       // sub-blocks 2g, 2g+1, g = kg>>1
      const u32 scU = (a2 & 0x0F0Fu) | ((a0 >> 2) & 0x3030u);                // sub-blocks 2g+4, 2g+5
      const u32 mU = ((a2 >> 4) & 0x0F0Fu) | ((a1 >> 2) & 0x3030u);
      S[c][0][0] = h2_dup(d * ubyte_f<0>(scL));
      S[c][0][1] = h2_dup(-(dm * ubyte_f<0>(mL)));
      S[c][0][2] = h2_dup(d * ubyte_f<1>(scL));
      S[c][0][3] = h2_dup(-(dm * ubyte_f<1>(mL)));
      S[c][1][0] = h2_dup(d * ubyte_f<0>(scU));
      S[c][1][1] = h2_dup(-(dm * ubyte_f<0>(mU)));
      S[c][1][2] = h2_dup(d * ubyte_f<1>(scU));
      S[c][1][3] = h2_dup(-(dm * ubyte_f<1>(mU)));
    }

    const uint4* arow = lds + cb + j * 4 + kg;
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
      const int u = ks >> 2, op = ks & 3, hi = op >> 1;
      half8_t B[3];
#pragma unroll
      for (int c = 0; c < 3; c++) {
        const uint4 Q = u ? cur[c].q1 : cur[c].q0;
        const u32 qa = (op & 1) ? Q.z : Q.x, qb = (op & 1) ? Q.w : Q.y;
        const u32 mask = hi ? 0x00F000F0u : 0x000F000Fu;
        const u32 magic = hi ? 0x54005400u : 0x64006400u;     // 64 + n (n sits 4 bits up) : 1024 + n
        const u32 off = hi ? 0xD400D400u : 0xE400E400u;       // half2(-64) : half2(-1024)
        const u32 sc = S[c][u][2 * hi], nm = S[c][u][2 * hi + 1];
        uint4 bw;
        bw.x = h2_fma_off((qa & mask) | magic, off, sc, nm);
        bw.y = h2_fma_off(((qa >> 8) & mask) | magic, off, sc, nm);
        bw.z = h2_fma_off((qb & mask) | magic, off, sc, nm);
        bw.w = h2_fma_off(((qb >> 8) & mask) | magic, off, sc, nm);
        B[c] = *reinterpret_cast<const half8_t*>(&bw);
      }
#pragma unroll
      for (int r = 0; r < 8; r++) {
        const uint4 av = arow[(ks * 128 + r * 16) * 4];
        const half8_t A = *reinterpret_cast<const half8_t*>(&av);
#pragma unroll
        for (int c = 0; c < 3; c++) acc[r][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B[c], acc[r][c], 0, 0, 0);
      }
    }
    // the other buffer was last read in the previous iteration, which ended with a barrier
#pragma unroll
    for (int i = 0; i < 16; i++) lds[nb_ + tid + 256 * i] = xbuf[i];
    __syncthreads();
#pragma unroll
    for (int c = 0; c < 3; c++) cur[c] = nxt[c];
  }

  // D layout: lane holds column j (weight row) and rows 4*kg + v (tokens) of each 16x16 tile
#pragma unroll
  for (int c = 0; c < 3; c++) {
    const u32 n = n0 + 16 * c + j;
    if (n < out_dim) {
      const float b = bias ? bias[n] : 0.0f;
#pragma unroll
      for (int r = 0; r < 8; r++) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
          const u32 row = mt * GEMM_BM + 16 * r + 4 * kg + v;
          if (row < m) out[(size_t)row * out_dim + n] = acc[r][c][v] + b;
        }
      }
    }
  }
}
