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
#include "gemv_formats.hpp"


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
// LIST (with DUAL, M = 1): up to three matrices of one row length and any row counts as one matrix of all their rows
// (q | k | v of a decoder layer: the reference's qmatvec_many seam, src/ml/gguf/qwen35_cpu.cr:1419-1445); `list` names
// them, w / w_b / out / out_b / out_dim are not used.
struct GemvList {
  const uint8_t* w[3];
  float* out[3];
  u32 rows[3];
};
// RO (one token, plain kernels): rows per wavefront where they differ from F::rows(M) - the variants for matrices of few
// rows (gemv_rows_m1 in gemv_config.h), 0 = F::rows(M).
template <class F, int M, bool ADD, bool DUAL = false, bool SWIGLU = false, bool TOP1 = false, bool LIST = false, int RO = 0>
__device__ __forceinline__ void gemv_core(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                          const float* __restrict__ residual, float* __restrict__ out,
                                          u32 in_dim, u32 out_dim, const uint8_t* __restrict__ w_b = nullptr,
                                          float* __restrict__ out_b = nullptr, u32* __restrict__ top_ids = nullptr,
                                          const GemvList* list = nullptr) {
  constexpr int R = RO ? RO : F::rows(M);
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
  static_assert(!LIST || (DUAL && M == 1 && !ADD && !SWIGLU), "LIST is a one-token mode of several matrices");
  const u32 total_rows = LIST ? list->rows[0] + list->rows[1] + list->rows[2] : (DUAL ? 2 * out_dim : out_dim);
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
        if constexpr (LIST) {
          const u32 r0 = list->rows[0], r01 = r0 + list->rows[1];
          rowp[r] = row < r0 ? list->w[0] + (size_t)row * row_bytes
                             : (row < r01 ? list->w[1] + (size_t)(row - r0) * row_bytes : list->w[2] + (size_t)(row - r01) * row_bytes);
        } else {
          rowp[r] = (DUAL && row >= out_dim) ? w_b + (size_t)(row - out_dim) * row_bytes : w + (size_t)row * row_bytes;
        }
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
            if constexpr (LIST) {   // (one token: m = 0)
              const u32 r0 = list->rows[0], r01 = r0 + list->rows[1];
              if (row < r0) list->out[0][row] = v;
              else if (row < r01) list->out[1][row - r0] = v;
              else list->out[2][row - r01] = v;
            } else if (DUAL && row >= out_dim) {
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
        // (one row per wavefront: the slot the next request lands in is the one being consumed, so the request follows
        // the arithmetic instead of preceding it)
        constexpr bool AHEAD = R > PF;
        if constexpr (AHEAD) {
          if (r + PF < R) F::template load_row<R>(st, rr, rowp[rr], ln, s, nb);
          else if constexpr (!decltype(last)::value) F::template load_row<R>(st, rr, rowp[rr], ln, s + 1, nb);
        }
        __builtin_amdgcn_sched_barrier(0);
        float c[MG];
        F::template compute<R, MG>(st, r, ln, xr, sx, c);
#pragma unroll
        for (int mm = 0; mm < MG; mm++) acc[r][mm] += valid ? c[mm] : 0.0f;
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!AHEAD && !decltype(last)::value) F::template load_row<R>(st, rr, rowp[rr], ln, s + 1, nb);
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

// ---- one token of a small Q8_0 matrix -----------------------------------------------------------
// A matrix of a few megabytes is over before the memory system is busy: its launch is a chain of latencies (dispatch,
// activations, barrier, first rows, reduction) and the staging above spends two of them one after the other. Where a row is
// one column set, every workgroup has one row group, the weights are at most GEMV_SMALL_BYTES and a lane's share of x is
// small (Q8_0: 16 values; the 64 values of a K-quant lane cost more to fetch per wavefront than the staging they would
// replace - Q5_K 4096x4096 7.8 us this way against 4.9), a lane takes its share of x straight from global memory into
// registers (the wavefronts of a compute unit hit the same lines), requests its R rows at once behind it, and nothing waits
// for another wavefront: no LDS, no barrier. The arithmetic and its order are those of gemv_core (F::compute on the same
// operands, the same sums, wave_sum), so the values are the same bit for bit.
#define GEMV_SMALL_BYTES (16u << 20)
template <class F, int RO = 0>
__device__ __forceinline__ bool gemv_small_shape(u32 in_dim, u32 out_dim) {
  const u32 nb = F::nblocks(in_dim);
  const u32 group_rows = GEMV_WAVES * (RO ? RO : F::rows(1));
  return F::NF4 <= 4 && nb <= (u32)F::BPS && (size_t)out_dim * F::row_bytes(nb) <= GEMV_SMALL_BYTES &&
         (size_t)gridDim.x * group_rows >= out_dim;
}
template <class F, bool ADD, int RO = 0>
__device__ __forceinline__ void gemv_small_core(const uint8_t* __restrict__ w, const float* __restrict__ x,
                                                const float* __restrict__ residual, float* __restrict__ out, u32 in_dim,
                                                u32 out_dim) {
  constexpr int R = RO ? RO : F::rows(1), NF4 = F::NF4, NSUM = F::NSUM;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const typename F::Lane ln(lane);
  const u32 nb = F::nblocks(in_dim);
  const size_t row_bytes = F::row_bytes(nb);
  const u32 row0 = (blockIdx.x * GEMV_WAVES + wave) * R;
  if (row0 >= out_dim) return;   // (whole wavefronts; nothing below meets another wavefront)
  float4 xr[1][NF4];
#pragma unroll
  for (int i = 0; i < NF4; i++) xr[0][i] = F::load_x(x, F::x_elem(0, lane, i), in_dim);
  const uint8_t* rowp[R];
#pragma unroll
  for (int r = 0; r < R; r++) rowp[r] = w + (size_t)min(row0 + r, out_dim - 1) * row_bytes;
  typename F::template Stage<R> st;
  F::template load<R>(st, rowp, ln, 0, nb);
  float sx[1][NSUM];
#pragma unroll
  for (int k = 0; k < NSUM; k++) {
    float a = 0.0f;
#pragma unroll
    for (int i = 0; i < NF4 / NSUM; i++) a += hsum4(xr[0][k * (NF4 / NSUM) + i]);
    sx[0][k] = a;
  }
  const bool valid = (u32)ln.jb < nb;
#pragma unroll
  for (int r = 0; r < R; r++) {
    float c[1];
    F::template compute<R, 1>(st, r, ln, xr, sx, c);
    float v = wave_sum(0.0f + (valid ? c[0] : 0.0f));
    const u32 row = row0 + r;
    if (lane == 0 && row < out_dim) {
      if (ADD) v += residual[row];
      out[row] = v;
    }
  }
}
template <class F, int M, bool ADD, int RO = 0>
__device__ __forceinline__ void gemv_entry(const uint8_t* w, const float* x, const float* residual, float* out, u32 in_dim, u32 out_dim) {
  if constexpr (M == 1) {
    if (gemv_small_shape<F, RO>(in_dim, out_dim)) {
      gemv_small_core<F, ADD, RO>(w, x, residual, out, in_dim, out_dim);
      return;
    }
  }
  gemv_core<F, M, ADD, false, false, false, false, RO>(w, x, residual, out, in_dim, out_dim);
}

// ---- entry points ---------------------------------------------------------------------------
// M = 1, 2: ask for at least 3 wavefronts per SIMD so a 12288-row matrix is resident in one round
#ifndef GEMV_OCC_M1
#define GEMV_OCC_M1 3
#endif
#define GEMV_OCC(M) __attribute__((amdgpu_waves_per_eu((M) <= 1 ? GEMV_OCC_M1 : 1)))
#define GEMV_ENTRY(NAME, FMT, M)                                                                                \
  extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(M) void NAME(const uint8_t* w, const float* x, float* out,   \
                                                                 u32 in_dim, u32 out_dim) {                     \
    gemv_entry<FMT, M, false>(w, x, nullptr, out, in_dim, out_dim);                                             \
  }
#define GEMV_ADD_ENTRY(NAME, FMT, M)                                                                            \
  extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(M) void NAME(const uint8_t* w, const float* x,               \
                                                                 const float* residual, float* out, u32 in_dim, \
                                                                 u32 out_dim) {                                 \
    gemv_entry<FMT, M, true>(w, x, residual, out, in_dim, out_dim);                                             \
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
// One token of a matrix of few rows: the same kernels with fewer rows per wavefront (NAME_rR: R rows), so that at least
// 256 workgroups share the matrix. Same parameters; grid ceil(out_dim / (4 R)). Q4_K 1024x4096 3.18 -> 2.90 us, Q6_K
// 3.72 -> 3.40, Q5_K 3.51 -> 3.21, Q8_0 1024 rows of 3584 values 7.16 -> 4.81, 3584 rows of 1024 values 3.66 -> 3.53 (two rows).
#define GEMV_SHORT_ENTRIES(PFX, FMT, R)                                                                                       \
  extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(1) void PFX##_gemv_f32_r##R(const uint8_t* w, const float* x,  \
                                                                                          float* out, u32 in_dim, u32 out_dim) { \
    gemv_entry<FMT, 1, false, R>(w, x, nullptr, out, in_dim, out_dim);                                                       \
  }                                                                                                                          \
  extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(1) void PFX##_gemv_add_f32_r##R(                               \
      const uint8_t* w, const float* x, const float* residual, float* out, u32 in_dim, u32 out_dim) {                        \
    gemv_entry<FMT, 1, true, R>(w, x, residual, out, in_dim, out_dim);                                                       \
  }
GEMV_SHORT_ENTRIES(q4_k, FmtQ4K, 1)
GEMV_SHORT_ENTRIES(q5_k, FmtQ5K, 1)
GEMV_SHORT_ENTRIES(q6_k, FmtQ6K, 1)
GEMV_SHORT_ENTRIES(q8_0, FmtQ80, 1)
GEMV_SHORT_ENTRIES(q8_0, FmtQ80, 2)
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
// grid.x = ceil(2 * out_dim / (GEMV_WAVES * GEMV_ROWS_Q4K_PAIR)), same block and dynamic shared memory as q4_k_gemv_f32.
// The reference has this pair as q4_k_dual_gemv_warp4_f32 and ..._batched (q4k_dual_gemv_probe.ptx:5, 233).
// (the pair kernels keep four rows per wavefront: GEMV_ROWS_Q4K_PAIR)
struct FmtQ4KPair : FmtQ4K {
  static constexpr int rows(int) { return GEMV_ROWS_Q4K_PAIR; }
};
extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(1) void q4_k_dual_gemv_f32(
    const uint8_t* w_a, const uint8_t* w_b, const float* x, float* out_a, float* out_b, u32 in_dim, u32 out_dim) {
  const size_t tok = blockIdx.y;
  gemv_core<FmtQ4KPair, 1, false, true>(w_a, x + tok * in_dim, nullptr, out_a + tok * out_dim, in_dim, out_dim, w_b,
                                        out_b + tok * out_dim);
}

// (w_gate, w_up, x, out, in_dim, out_dim): out[o] = silu(gate[o]) * up[o] for one token per grid.y slice; block and
// dynamic shared memory as q4_k_gemv_f32, grid.x = ceil(out_dim / (GEMV_WAVES * GEMV_ROWS_Q4K_PAIR / 2)).
extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(1) void q4_k_dual_gemv_swiglu_f32(
    const uint8_t* w_gate, const uint8_t* w_up, const float* x, float* out, u32 in_dim, u32 out_dim) {
  const size_t tok = blockIdx.y;
  gemv_core<FmtQ4KPair, 1, false, true, true>(w_gate, x + tok * in_dim, nullptr, out + tok * out_dim, in_dim, out_dim,
                                              w_up, nullptr);
}

// (w0, w1, w2, x, out0, out1, out2, in_dim, rows0, rows1, rows2): one token against up to three Q4_K matrices of one row
// length (rows1 / rows2 may be 0), the parameter list of q4_k_many_gemv_mfma_f32_tbatchM. Block, dynamic shared memory and
// grid as q4_k_gemv_f32 for a matrix of rows0 + rows1 + rows2 rows. Every row is computed exactly as q4_k_gemv_f32 does it.
extern "C" __global__ __launch_bounds__(GEMV_BLOCK) GEMV_OCC(1) void q4_k_many_gemv_f32(
    const uint8_t* w0, const uint8_t* w1, const uint8_t* w2, const float* x, float* out0, float* out1, float* out2, u32 in_dim,
    u32 rows0, u32 rows1, u32 rows2) {
  const GemvList list = {{w0, w1, w2}, {out0, out1, out2}, {rows0, rows1, rows2}};
  gemv_core<FmtQ4K, 1, false, true, false, false, true>(nullptr, x, nullptr, nullptr, in_dim, 0, nullptr, nullptr, nullptr, &list);
}

// (gate, up, out, n): out[i] = silu(gate[i]) * up[i], the reference's swiglu_f32 (bin/cuda_ffn_sequence_probe.cr:46-84).
// block = 256, grid = ceil(n / 256).
extern "C" __global__ __launch_bounds__(256) void swiglu_f32(const float* gate, const float* up, float* out, u32 n) {
  const u32 i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = swiglu_one(gate[i], up[i]);
}
