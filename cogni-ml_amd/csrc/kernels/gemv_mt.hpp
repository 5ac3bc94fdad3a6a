// Decode GEMV for 2..8 tokens in ONE pass over the weights, Q4_K, on the matrix cores:
//   out_i[m][o] = (residual[m][o] +) sum_j x[m][j] * deq(W_i[o][j])      for up to three matrices W_i of one in_dim.
//
// Two kernels.
//   pack_x_mt_f16 (x, image, tokens, in_dim)            block 256, grid 2 * in_dim / 256
//     turns the activations x[tokens][in_dim] (fp32) into the image the GEMV kernel reads: per super-block of 256
//     values the B operands of its eight matrix-core instructions, laid out lane by lane, followed by the scale and
//     the sub-block sums of every (token, super-block). Written once per activation block, whatever the number of
//     matrices that block then meets (q | k | v | gate | up of a decoder layer share one).
//   q4_k_gemv_mt_f32 (w0, w1, w2, image, residual, out0, out1, out2, in_dim, rows0, rows1, rows2, tokens)
//     block 512 (8 wavefronts), grid and dynamic shared memory from gemv_mt_plan (gemv_config.h). rows1 / rows2 may be
//     0 (then w1 / w2 / out1 / out2 are not read); residual (may be null) belongs to the first matrix. Row counts of all
//     but the last matrix present must be multiples of 16. in_dim must be 2048 or 4096 (8 or 16 super-blocks: one or
//     two per wavefront). out_i rows at stride rows_i (the reference's multi-token kernel contract,
//     src/ml/cuda/kernels/q4k_gemv_probe.ptx:437-768: x rows at stride in_dim, outs at stride out_dim; this kernel
//     handles eight tokens where that one handles four).
//
// Arithmetic. v_mfma_f32_16x16x32_f16 multiplies 16 weight rows x 32 weights by 32 x 16 columns. The weights stay exact:
// a masked pair of 4-bit codes read as two binary16 numbers is code * 2^-24 (code * 2^-20 for high nibbles left in
// place), the matrix cores honour subnormals, accumulation is fp32. The activations are fed as two binary16 terms,
// x * 2^e = hi + lo (22 bits; e per token and super-block, so any fp32 range fits), which makes the 16 columns
// (token 0..7) x (hi, lo). One instruction covers exactly one 32-weight sub-block (its lanes load 8 bytes each:
// lane (row r, k-group kg) takes bytes 32 g + 8 kg .. + 8 of the super-block's quants for g = 0..3, whose low nibbles
// are sub-block 2 g and whose high nibbles are sub-block 2 g + 1), so the fp32 scale d * sc of that sub-block is applied
// to the instruction's result, and the min term dmin * m * sum(x) is added from the sub-block sums of the image.
//
// Work split. The eight wavefronts of a workgroup are eight k-slices (super-blocks wave, wave + 8); each keeps the
// activation operands of its own super-blocks in registers for the whole kernel and takes T tiles of 16 rows at a time.
// Nobody waits for anybody until the k-slices' sums meet in LDS, where they are added in a fixed order
// (bit-reproducible). A workgroup walks the row groups blockIdx.x, blockIdx.x + gridDim.x, ...
//
// Memory. A tile's share of a super-block is 16 rows x 144 bytes at a stride of a whole row: fetched by the lanes that
// use it (8 bytes each, 16 rows per instruction) it comes in at a third of the rate of a plain stream. So the weights are
// copied global -> LDS 16 bytes per lane with the lanes along the rows (lane p of a unit takes 16-byte piece p % 9 of row
// p / 9: 144 pieces = three copy instructions, the third with 16 lanes), which lands them in a wavefront-private slot
// as [row][144 bytes], and each lane then picks its 8-byte pieces out of LDS. Every copy of a row group is issued up
// front behind the activation operands; all loads are written in assembly and counted by hand (s_waitcnt vmcnt), unit
// after unit as they land, and with another row group to come a unit's slot is refilled as soon as it has been read.
#pragma once
#include <type_traits>
#include "common.hpp"
#include "gemv_config.h"

typedef _Float16 mt_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 mt_half4 __attribute__((ext_vector_type(4)));
typedef float mt_float4 __attribute__((ext_vector_type(4)));
typedef u32 mt_u32x4 __attribute__((ext_vector_type(4)));

#define MT_DPP(v, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (v)), (ctrl), 0xF, 0xF, false))
#define MT_DPP_U(v, ctrl) ((u32)__builtin_amdgcn_update_dpp(0, (int)(v), (ctrl), 0xF, 0xF, false))
#define MT_QUAD_1032 0xB1
#define MT_QUAD_2301 0x4E
#define MT_ROW_ROR4 0x124
#define MT_ROW_ROR8 0x128
#define MT_ROW_HALF_MIRROR 0x141
#define MT_TWO_P24 16777216.0f
#define MT_TWO_P20 1048576.0f

// The compiler must not move LDS accesses of one lane across this point: other lanes of the wavefront read what this
// lane wrote (the LDS itself executes a wavefront's accesses in order).
__device__ __forceinline__ void mt_wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---- the image ---------------------------------------------------------------------------------------------------------
// [super-block][instruction j = 2 g + par][lane = 16 kg + column][8 halves]: the halves of lane (kg, column = 2 token +
// part) are part (0 = hi, 1 = lo) of x[token][256 sb + 64 g + 32 par + 8 kg + (0,2,1,3,4,6,5,7)] * 2^e, the order in which
// the nibble masks deliver the weights. Behind the in_dim / 256 * 8 KiB of operands: [super-block][token pair][20 floats]:
// 2^-e of the pair's two tokens, two unused, the eight sub-block sums of x (unscaled) of the first token, those of the
// second. Tokens at and above `tokens` are zero.
// One wavefront per (token slot 0..7, super-block); lane l holds elements 4 l .. 4 l + 3 of the super-block.
extern "C" __global__ __launch_bounds__(256) void pack_x_mt_f16(const float* __restrict__ x, uint8_t* __restrict__ image,
                                                                u32 tokens, u32 in_dim) {
  const u32 lane = threadIdx.x & 63;
  const u32 unit = blockIdx.x * 4 + (threadIdx.x >> 6);
  const u32 nsb = in_dim >> 8;
  const u32 sb = unit >> 3, tok = unit & 7;
  if (sb >= nsb) return;
  float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
  if (tok < tokens) __builtin_memcpy(&v, x + (size_t)tok * in_dim + (size_t)sb * 256 + 4 * lane, 16);
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
  int sh = 139 - e;           // scale = 2^sh
  sh = sh > 100 ? 100 : sh;   // zeros and tiny values: keep 2^-sh a normal number
  sh = sh < -100 ? -100 : sh; // infinities and NaN: they stay what they are
  const float scale = __builtin_bit_cast(float, (u32)(127 + sh) << 23);
  const float inv = __builtin_bit_cast(float, (u32)(127 - sh) << 23);
  const _Float16 h0 = (_Float16)(v.x * scale), h1 = (_Float16)(v.y * scale), h2 = (_Float16)(v.z * scale), h3 = (_Float16)(v.w * scale);
  // (x * scale is exact, so fma(x, scale, -hi) is (x * scale) - hi in one instruction)
  const _Float16 l0 = (_Float16)fmaf(v.x, scale, -(float)h0), l1 = (_Float16)fmaf(v.y, scale, -(float)h1),
                 l2 = (_Float16)fmaf(v.z, scale, -(float)h2), l3 = (_Float16)fmaf(v.w, scale, -(float)h3);
  const mt_half4 hv = {h0, h2, h1, h3}, lv = {l0, l2, l1, l3};
  // element 4 l sits in instruction j = l / 8, k-group (l / 2) % 4, upper half of the lane's eight if l is odd
  const u32 j = lane >> 3, kg = (lane >> 1) & 3;
  uint8_t* op = image + ((size_t)(sb * 8 + j) * 64 + kg * 16 + 2 * tok) * 16 + 8 * (lane & 1);
  *reinterpret_cast<mt_half4*>(op) = hv;
  *reinterpret_cast<mt_half4*>(op + 16) = lv;
  // sums of the eight sub-blocks (eight lanes each), unscaled, for the min term
  float sm = (v.x + v.y) + (v.z + v.w);
  sm += MT_DPP(sm, MT_QUAD_1032);
  sm += MT_DPP(sm, MT_QUAD_2301);
  sm += MT_DPP(sm, MT_ROW_HALF_MIRROR);
  float* aux = reinterpret_cast<float*>(image + (size_t)nsb * 8192) + (size_t)(sb * 4 + (tok >> 1)) * 20;
  if ((lane & 7) == 0) aux[4 + 8 * (tok & 1) + (lane >> 3)] = sm;
  if (lane == 0) aux[tok & 1] = tok < tokens ? inv : 0.0f;
}

// ---- the GEMV ------------------------------------------------------------------------------------------------------------
struct MtArgs {
  const uint8_t* w[3];
  float* out[3];
  u32 rows[3];
};

// Loads in assembly: the compiler knows neither that they are loads nor when they land. A value loaded this way must
// not be touched before mt_wait<N> has said that it is there and mt_pin has tied it to that wait.
__device__ __forceinline__ void mt_load16(mt_u32x4& dst, const void* addr) {
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(dst) : "v"(addr) : "memory");
}
// 16 bytes per active lane from addr to LDS byte address lds_base (uniform) + 16 * lane
__device__ __forceinline__ void mt_copy16(u32 lds_base, const void* addr) {
  const u32 m0 = (u32)__builtin_amdgcn_readfirstlane((int)lds_base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(m0), "v"(addr) : "memory");
}
template <int N>
__device__ __forceinline__ void mt_wait() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __forceinline__ void mt_pin(mt_u32x4& v) { asm volatile("" : "+v"(v)); }

typedef __attribute__((address_space(3))) void mt_lds_void;

// SWIGLU (T = 2): the two tiles of a row group are tile grp of w[0] (gate) and tile grp of w[1] (up), rows[0] = rows[1] =
// out_dim, and the workgroup stores out[0][m][o] = silu(gate . x) * (up . x) (swiglu_one, the function of swiglu_f32): the
// values of the pair launch followed by swiglu_f32, bit for bit, without the gate and up vectors in memory.
template <int SBW, int T, bool SWIGLU = false>
__device__ __forceinline__ void q4k_gemv_mt_core(const MtArgs& a, const uint8_t* __restrict__ image,
                                                 const float* __restrict__ residual, u32 in_dim, u32 tokens) {
  static_assert(!SWIGLU || T == 2, "SWIGLU pairs a gate tile with an up tile");
  constexpr int BB = 144, NU = SBW * T;          // units (super-block of the k-slice, tile) of a row group, 3 copies each
  constexpr u32 UNIT_BYTES = 16 * BB;            // 2304
  extern __shared__ uint4 mt_lds4[];
  char* lds = reinterpret_cast<char*>(mt_lds4);
  const int tid = threadIdx.x, lane = tid & 63;
  const u32 wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const u32 nsb = in_dim >> 8;
  const u32 total_rows = a.rows[0] + a.rows[1] + a.rows[2];
  const u32 ntiles = (total_rows + 15) >> 4;
  const u32 ngroups = SWIGLU ? (a.rows[0] + 15) >> 4 : (ntiles + T - 1) / T;
  // LDS: partial[wave][TMAX][8 tokens][16 rows] f32 | slots[wave][SBW * TMAX units][2304 B]
  float* part = reinterpret_cast<float*>(lds);
  constexpr u32 SLOTS_OFF = GEMV_MT_WAVES * GEMV_MT_TMAX * 8 * 16 * 4;
  const char* slots = lds + SLOTS_OFF + wave * (2 * GEMV_MT_TMAX * UNIT_BYTES);
  const u32 slots_lds = (u32)(size_t)(mt_lds_void*)mt_lds4 + SLOTS_OFF + wave * (2 * GEMV_MT_TMAX * UNIT_BYTES);

  // Lane roles. The activations are the A operand (16 rows = (token, part), k-group kg) and the weights the B operand
  // (16 columns = weight rows of the tile, k-group kg), so a result lane (column n = lane % 16, row group rg = lane / 16)
  // holds rows 4 rg .. 4 rg + 3 = tokens 2 rg, 2 rg + 1 x (hi, lo) of weight row n - the row whose header this very lane
  // reads: the scales never change lanes.
  const u32 ar = lane & 15, kg = lane >> 4;
  const u32 rg = lane >> 4;

  u32 grp = blockIdx.x;
  if (grp >= ngroups) return;

  // ---- this wavefront's A operands, scales and sub-block sums: registers, for the whole kernel ----
  mt_u32x4 breg[SBW][8], auxr[SBW][5];
  const uint8_t* aux = image + (size_t)nsb * 8192;
#pragma unroll
  for (int i = 0; i < SBW; i++) {
    const u32 sb = wave + 8u * i;
#pragma unroll
    for (int j = 0; j < 8; j++) mt_load16(breg[i][j], image + ((size_t)(sb * 8 + j) * 64 + lane) * 16);
#pragma unroll
    for (int q = 0; q < 5; q++) mt_load16(auxr[i][q], aux + (size_t)(sb * 4 + rg) * 80 + 16 * q);
  }

  // ---- the copies of a row group's units. Copy m of a unit: piece p = 64 m + lane (< 144), row p / 9 of the tile.
  const size_t row_bytes = (size_t)nsb * BB;
  const uint8_t* cptr[T][3];   // where this lane's piece of copy m of tile t starts, without the super-block offset
  auto set_rows = [&](u32 g) {
#pragma unroll
    for (int t = 0; t < T; t++) {
#pragma unroll
      for (int m = 0; m < 3; m++) {
        const u32 p = 64u * m + lane;
        const u32 pr = min(p / 9u, 15u), piece = p - 9u * (p / 9u);
        const u32 vr = SWIGLU ? min(g * 16 + pr, a.rows[0] - 1) : min((g * T + (u32)t) * 16 + pr, total_rows - 1);
        const uint8_t* rp;
        if constexpr (SWIGLU) rp = a.w[t] + (size_t)vr * row_bytes;
        else if (vr < a.rows[0]) rp = a.w[0] + (size_t)vr * row_bytes;
        else if (vr < a.rows[0] + a.rows[1]) rp = a.w[1] + (size_t)(vr - a.rows[0]) * row_bytes;
        else rp = a.w[2] + (size_t)(vr - a.rows[0] - a.rows[1]) * row_bytes;
        cptr[t][m] = rp + piece * 16;
      }
    }
  };
  auto issue_unit = [&](int i, int t) {
    const u32 off = (wave + 8u * i) * BB, dst = slots_lds + (u32)(i * T + t) * UNIT_BYTES;
    mt_copy16(dst, cptr[t][0] + off);
    mt_copy16(dst + 1024, cptr[t][1] + off);
    if (lane < 16) mt_copy16(dst + 2048, cptr[t][2] + off);
  };
  set_rows(grp);
#pragma unroll
  for (int i = 0; i < SBW; i++)
#pragma unroll
    for (int t = 0; t < T; t++) issue_unit(i, t);
  mt_wait<3 * NU>();   // the operands are older than the copies
  float fsc[SBW][2], sxl[SBW][2][8];
#pragma unroll
  for (int i = 0; i < SBW; i++) {
#pragma unroll
    for (int j = 0; j < 8; j++) mt_pin(breg[i][j]);
#pragma unroll
    for (int q = 0; q < 5; q++) mt_pin(auxr[i][q]);
    fsc[i][0] = __uint_as_float(auxr[i][0].x), fsc[i][1] = __uint_as_float(auxr[i][0].y);
#pragma unroll
    for (int tt = 0; tt < 2; tt++) {
      const mt_u32x4 lo = auxr[i][1 + 2 * tt], hi = auxr[i][2 + 2 * tt];
      sxl[i][tt][0] = __uint_as_float(lo.x), sxl[i][tt][1] = __uint_as_float(lo.y), sxl[i][tt][2] = __uint_as_float(lo.z);
      sxl[i][tt][3] = __uint_as_float(lo.w), sxl[i][tt][4] = __uint_as_float(hi.x), sxl[i][tt][5] = __uint_as_float(hi.y);
      sxl[i][tt][6] = __uint_as_float(hi.z), sxl[i][tt][7] = __uint_as_float(hi.w);
    }
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
      mt_wait<walk ? 3 * (NU - 1) : 3 * (NU - 1 - u)>();
      const char* up = slots + u * UNIT_BYTES + ar * BB;
      const uint4 hdr = *reinterpret_cast<const uint4*>(up);
      uint2 q[4];
#pragma unroll
      for (int g = 0; g < 4; g++) q[g] = *reinterpret_cast<const uint2*>(up + 16 + 32 * g + 8 * kg);
      if constexpr (walk) {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the slot has been read
        issue_unit(i, t);
      }
      // (a) eight instructions, one per sub-block, each into an accumulator of its own
      mt_float4 dacc[8];
#pragma unroll
      for (int g = 0; g < 4; g++) {
#pragma unroll
        for (int par = 0; par < 2; par++) {
          const u32 mask = par ? 0x00F000F0u : 0x000F000Fu;
          uint4 a4;
          a4.x = q[g].x & mask;
          a4.y = (q[g].x >> 8) & mask;
          a4.z = q[g].y & mask;
          a4.w = (q[g].y >> 8) & mask;
          dacc[2 * g + par] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(mt_half8, breg[i][2 * g + par]),
                                                                     __builtin_bit_cast(mt_half8, a4),
                                                                     (mt_float4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
        }
      }
      // (b) the eight (scale, min) pairs of this lane's weight row as bytes (dequant.cr:240-249, four at a time):
      //     scA = sc 0..3, scB = sc 4..7, mA = m 0..3, mB = m 4..7
      const u32 s0 = hdr.y, s1 = hdr.z, s2 = hdr.w;
      const u32 scA = s0 & 0x3F3F3F3Fu, mA = s1 & 0x3F3F3F3Fu;
      const u32 scB = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
      const u32 mB = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
      const float sc[8] = {ubyte_f<0>(scA), ubyte_f<1>(scA), ubyte_f<2>(scA), ubyte_f<3>(scA),
                           ubyte_f<0>(scB), ubyte_f<1>(scB), ubyte_f<2>(scB), ubyte_f<3>(scB)};
      const float mn[8] = {ubyte_f<0>(mA), ubyte_f<1>(mA), ubyte_f<2>(mA), ubyte_f<3>(mA),
                           ubyte_f<0>(mB), ubyte_f<1>(mB), ubyte_f<2>(mB), ubyte_f<3>(mB)};
      const float dd = h2f(hdr.x), dmin = h2f(hdr.x >> 16);
      // (c) sum_j sc_j * result_j, even sub-blocks (low nibbles, 2^-24) and odd ones (high nibbles, 2^-20) apart;
      //     sum_j m_j * sum(x_j) for the two tokens of this lane
      float ev[4] = {0.f, 0.f, 0.f, 0.f}, od[4] = {0.f, 0.f, 0.f, 0.f}, mt0 = 0.f, mt1 = 0.f;
#pragma unroll
      for (int j = 0; j < 8; j++) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
          if (j & 1) od[k] = fmaf(sc[j], dacc[j][k], od[k]);
          else ev[k] = fmaf(sc[j], dacc[j][k], ev[k]);
        }
        mt0 = fmaf(mn[j], sxl[i][0][j], mt0);
        mt1 = fmaf(mn[j], sxl[i][1][j], mt1);
      }
      const float d24 = dd * MT_TWO_P24, d20 = dd * MT_TWO_P20;
#pragma unroll
      for (int k = 0; k < 4; k++) {
        const float in = fmaf(d24, ev[k], d20 * od[k]);
        acc[t][k] = fmaf(fsc[i][k >> 1], in, acc[t][k]);
      }
      acc[t][0] = fmaf(-dmin, mt0, acc[t][0]);   // the min term goes to the hi part only
      acc[t][2] = fmaf(-dmin, mt1, acc[t][2]);
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

    // hi + lo of a token, then the k-slices through LDS in wavefront order: partial[wave][tile][token][row]
#pragma unroll
    for (int t = 0; t < T; t++) {
      part[((wave * GEMV_MT_TMAX + t) * 8 + 2 * rg) * 16 + ar] = acc[t][0] + acc[t][1];
      part[((wave * GEMV_MT_TMAX + t) * 8 + 2 * rg + 1) * 16 + ar] = acc[t][2] + acc[t][3];
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if constexpr (SWIGLU) {
      for (u32 o = tid; o < 16u * tokens; o += GEMV_MT_WAVES * 64) {
        const u32 r = o & 15, m = o >> 4;
        float g = 0.f, u = 0.f;
#pragma unroll
        for (u32 k = 0; k < GEMV_MT_WAVES; k++) {
          g += part[((k * GEMV_MT_TMAX + 0) * 8 + m) * 16 + r];
          u += part[((k * GEMV_MT_TMAX + 1) * 8 + m) * 16 + r];
        }
        const u32 row = grp * 16 + r;
        if (row < a.rows[0]) a.out[0][(size_t)m * a.rows[0] + row] = swiglu_one(g, u);
      }
      return;
    }
    for (u32 o = tid; o < (u32)T * 16u * tokens; o += GEMV_MT_WAVES * 64) {
      const u32 r = o & 15, m = (o >> 4) % tokens, t = o / (16 * tokens);
      float v = 0.f;
#pragma unroll
      for (u32 k = 0; k < GEMV_MT_WAVES; k++) v += part[((k * GEMV_MT_TMAX + t) * 8 + m) * 16 + r];
      const u32 row = (grp * T + t) * 16 + r;
      if (row < a.rows[0]) {
        const size_t oi = (size_t)m * a.rows[0] + row;
        if (residual) v += residual[oi];
        a.out[0][oi] = v;
      } else if (row < a.rows[0] + a.rows[1]) {
        a.out[1][(size_t)m * a.rows[1] + (row - a.rows[0])] = v;
      } else if (row < total_rows) {
        a.out[2][(size_t)m * a.rows[2] + (row - a.rows[0] - a.rows[1])] = v;
      }
    }
  };
  while (grp + gridDim.x < ngroups) {
    group(std::true_type{});
    grp += gridDim.x;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();   // every partial sum has been read
    asm volatile("" ::: "memory");
  }
  group(std::false_type{});
}

// The tile count per wavefront follows from the grid the host chose (gemv_mt_plan); tile count and super-blocks per
// wavefront are template parameters so that register use and loads in flight are compile-time constants.
extern "C" __global__ __launch_bounds__(GEMV_MT_WAVES * 64) void q4_k_gemv_mt_f32(
    const uint8_t* w0, const uint8_t* w1, const uint8_t* w2, const uint8_t* image, const float* residual, float* out0,
    float* out1, float* out2, u32 in_dim, u32 rows0, u32 rows1, u32 rows2, u32 tokens) {
  const MtArgs a = {{w0, w1, w2}, {out0, out1, out2}, {rows0, rows1, rows2}};
  const u32 ntiles = (rows0 + rows1 + rows2 + 15) >> 4;
  const u32 t = gemv_mt_tiles(ntiles, gridDim.x);
  if (in_dim == 2048) {
    if (t <= 1) q4k_gemv_mt_core<1, 1>(a, image, residual, in_dim, tokens);
    else if (t == 2) q4k_gemv_mt_core<1, 2>(a, image, residual, in_dim, tokens);
    else q4k_gemv_mt_core<1, 3>(a, image, residual, in_dim, tokens);
  } else {
    if (t <= 1) q4k_gemv_mt_core<2, 1>(a, image, residual, in_dim, tokens);
    else if (t == 2) q4k_gemv_mt_core<2, 2>(a, image, residual, in_dim, tokens);
    else q4k_gemv_mt_core<2, 3>(a, image, residual, in_dim, tokens);
  }
}

// (w_gate, w_up, image, out, in_dim, out_dim, tokens): out[m][o] = silu(gate . x) * (up . x); block 512, grid = min(256,
// ceil(out_dim / 16)), dynamic shared memory as q4_k_gemv_mt_f32. The parameter list of q4_k_dual_gemv_swiglu_f32 with the
// image in the place of x and the token count behind.
extern "C" __global__ __launch_bounds__(GEMV_MT_WAVES * 64) void q4_k_gemv_mt_swiglu_f32(
    const uint8_t* w_gate, const uint8_t* w_up, const uint8_t* image, float* out, u32 in_dim, u32 out_dim, u32 tokens) {
  const MtArgs a = {{w_gate, w_up, nullptr}, {out, nullptr, nullptr}, {out_dim, out_dim, 0u}};
  if (in_dim == 2048) q4k_gemv_mt_core<1, 2, true>(a, image, nullptr, in_dim, tokens);
  else q4k_gemv_mt_core<2, 2, true>(a, image, nullptr, in_dim, tokens);
}
