// Launch geometry shared by the GEMV kernels and the host code that sizes their grids.
// A workgroup is 4 wavefronts; each wavefront owns GEMV_ROWS_*(tokens) consecutive output rows.
#pragma once

#ifndef GEMV_WAVES
#define GEMV_WAVES 4
#endif
#define GEMV_BLOCK (64 * GEMV_WAVES)

// rows per wavefront. One token of a Q4_K matrix: two rows and four workgroups per compute unit (1024 resident workgroups
// that walk the row groups) measured 7.55 us against 7.9-8.0 for four rows and three workgroups at 12288 x 4096, interleaved
// runs; 896, 960 or 1088 workgroups lose that again. The one-token matrix-pair kernels keep four rows (no gain there).
#ifndef GEMV_ROWS_Q4K
#define GEMV_ROWS_Q4K(M) ((M) == 1 ? 2 : ((M) == 2 ? 4 : 2))
#endif
#define GEMV_ROWS_Q4K_PAIR 4
#ifndef GEMV_ROWS_Q5K
#define GEMV_ROWS_Q5K(M) 2
#endif
#ifndef GEMV_ROWS_Q6K
#define GEMV_ROWS_Q6K(M) 2
#endif
#ifndef GEMV_ROWS_Q80
#define GEMV_ROWS_Q80(M) 4
#endif

// rows of the weight matrix one workgroup produces
static inline int gemv_rows_per_block(unsigned type, int tokens) {
  switch (type) {
    case 12: return GEMV_WAVES * GEMV_ROWS_Q4K(tokens);
    case 13: return GEMV_WAVES * GEMV_ROWS_Q5K(tokens);
    case 14: return GEMV_WAVES * GEMV_ROWS_Q6K(tokens);
    case 8: return GEMV_WAVES * GEMV_ROWS_Q80(tokens);
    default: return 0;
  }
}

// One token of a matrix of few rows: halve the rows per wavefront until at least 256 workgroups share the matrix
// (kernels NAME_r1, Q8_0 also NAME_r2). Returns rows per wavefront; the value for many rows is the kernel's own.
#define GEMV_SHORT_MIN_GROUPS 256u
static inline int gemv_rows_m1(unsigned type, unsigned out_dim) {
  int r = gemv_rows_per_block(type, 1) / GEMV_WAVES;
  while (r > 1 && (out_dim + (unsigned)(GEMV_WAVES * r) - 1) / (unsigned)(GEMV_WAVES * r) < GEMV_SHORT_MIN_GROUPS) r >>= 1;
  return r;
}

// ---- staged activations ------------------------------------------------------------------------
// A workgroup keeps the activations of up to GEMV_LDS_BYTES in LDS: `chunk` whole column sets for the
// token group it is working on. per_set_f4 = float4 count of one column set for that token group.
#define GEMV_LDS_BYTES 49152

#if defined(__HIPCC__)
#define GEMV_HD __host__ __device__
#else
#define GEMV_HD
#endif

static inline GEMV_HD int gemv_chunk_sets(int per_set_f4, unsigned ncs) {
  // 17/16: the per-lane activation sums kept beside the staged activations never exceed 1/16 of them
  int ch = GEMV_LDS_BYTES / 17 / per_set_f4;
  if (ch < 1) ch = 1;
  if ((unsigned)ch >= ncs) return (int)ncs;
  if (ch > 1) ch &= ~1;   // a chunk boundary never splits a pair of column sets taken together
  return ch;
}

// K-quant kernels whose tokens all fit the registers at once (one token group) keep the activations in LDS in natural
// order (16 KiB per token and column set) and form the per-lane sums from the registers they are read into: no sums
// in LDS. A row of one column set is staged as just that; longer rows in chunks of as many sets as fit the budget
// (3 for one token, 1 for two), whole chunks even where the row ends inside one.
static constexpr inline GEMV_HD int gemv_chunk_sets_direct(int per_set_f4, unsigned ncs) {
  int ch = GEMV_LDS_BYTES / 16 / per_set_f4;
  if (ch < 1) ch = 1;
  return ncs <= 1 ? 1 : ch;
}
static constexpr inline GEMV_HD bool gemv_direct_x(unsigned type, int token_groups) {
  return (type == 12 || type == 13 || type == 14) && token_groups == 1;
}

// One or two tokens of a K-quant matrix (one token group): the kernel walks row groups blockIdx.x, blockIdx.x +
// gridDim.x, ... with the activations staged once, so a long matrix is launched as the workgroups that are resident
// together (256 compute units x 3 per unit at 3 wavefronts per SIMD for one token, x 2 for two), each with the same
// number of groups up to one.
#define GEMV_RESIDENT_WGS 768u
#define GEMV_RESIDENT_WGS_2 512u
// (one token of Q4_K: every resident slot is launched, 4 per compute unit, and the workgroups' group counts differ by at
// most one)
#define GEMV_RESIDENT_WGS_Q4K 1024u
// (one token of a Q6_K matrix of many groups: 5 per compute unit. The 151936 x 4096 head, interleaved runs: 93.6 us on 760,
// 768 or 1024 workgroups, 90.2 on 1280, 91.1 on 1536, 90.8 on 2048; 92.4 - 97.2 on counts that are not multiples of the 256
// compute units. With only a few groups per workgroup the even split over 768 stays: 12288 rows 10.35 us against 11.1 on
// 1280, 24576 rows 17.4 against 18.65)
#define GEMV_RESIDENT_WGS_Q6K 1280u
#define GEMV_RESIDENT_Q6K_MIN_GROUPS (8u * GEMV_RESIDENT_WGS_Q6K)
static inline unsigned gemv_grid(unsigned type, int tokens, unsigned out_dim) {
  const unsigned rows = (unsigned)gemv_rows_per_block(type, tokens);
  const unsigned groups = (out_dim + rows - 1) / rows;
  if (type == 12 && tokens == 1) return groups < GEMV_RESIDENT_WGS_Q4K ? groups : GEMV_RESIDENT_WGS_Q4K;
  if (type == 14 && tokens == 1 && groups >= GEMV_RESIDENT_Q6K_MIN_GROUPS) return GEMV_RESIDENT_WGS_Q6K;
  const unsigned resident = tokens == 1 ? GEMV_RESIDENT_WGS : GEMV_RESIDENT_WGS_2;
  if (tokens > 2 || !gemv_direct_x(type, 1) || groups <= resident) return groups;
  const unsigned per_wg = (groups + resident - 1) / resident;
  return (groups + per_wg - 1) / per_wg;
}

// column-set geometry per type: blocks per set, float4 of x per lane and set, tokens per register group
// (nsum = scale groups per lane whose activation sums are kept in LDS)
static inline void gemv_set_geometry(unsigned type, int* bps, int* nf4, int* nsum, int* mg_max, int* block_elems) {
  switch (type) {
    case 12: case 13: *bps = 16; *nf4 = 16; *nsum = 2; *mg_max = 2; *block_elems = 256; break;
    case 14: *bps = 16; *nf4 = 16; *nsum = 4; *mg_max = 2; *block_elems = 256; break;
    default: *bps = 32; *nf4 = 4; *nsum = 1; *mg_max = 4; *block_elems = 32; break;
  }
}

// dynamic shared memory (bytes) the GEMV kernel for (type, tokens) needs at this in_dim
static inline unsigned gemv_lds_bytes(unsigned type, int tokens, unsigned in_dim) {
  int bps, nf4, nsum, mg_max, be;
  gemv_set_geometry(type, &bps, &nf4, &nsum, &mg_max, &be);
  const int mg = tokens < mg_max ? tokens : mg_max;
  const int ng = (tokens + mg - 1) / mg;
  const unsigned nb = (in_dim + (unsigned)be - 1) / (unsigned)be;
  const unsigned ncs = (nb + (unsigned)bps - 1) / (unsigned)bps;
  const int per_set_f4 = mg * nf4 * 64;
  if (gemv_direct_x(type, ng)) return (unsigned)(per_set_f4 * gemv_chunk_sets_direct(per_set_f4, ncs)) * 16u;
  const int ch = ng > 1 ? 1 : gemv_chunk_sets(per_set_f4, ncs);
  return (unsigned)(per_set_f4 * ch) * 16u + (unsigned)(mg * nsum * 64 * ch) * 4u;
}

// ---- matrix-core GEMV (gemv_mfma.hpp): 8 wavefronts per workgroup ------------------------------------
#define GEMV_MFMA_WAVES 8
#define GEMV_MFMA_TMAX 3            // 16-row tiles a wavefront carries at most
#define GEMV_MFMA_MAX_TOKENS 4
// (token, super-block) pairs of activations a workgroup stages (tokens * in_dim / 256) at most
#define GEMV_MFMA_MAX_UNITS(M) ((M) >= 3 ? 64 : 96)

// log2 of the k-slices a workgroup's wavefronts form: the largest power of two <= min(8, super-blocks)
static inline GEMV_HD unsigned gemv_mfma_log2_kslices(unsigned nsb) {
  unsigned lg = 0;
  while (lg < 3 && (2u << lg) <= nsb) lg++;
  return lg;
}
// Rows too long for all their activations to be staged at once are staged a chunk at a time, which needs every
// wavefront to be a k-slice of its own: in_dim a multiple of 2048.
static inline GEMV_HD int gemv_mfma_chunked(int tokens, unsigned in_dim) {
  return (unsigned)tokens * (in_dim >> 8) > (unsigned)GEMV_MFMA_MAX_UNITS(tokens) && (in_dim & 2047u) == 0;
}
// Shapes the matrix-core kernels take: Q4_K with 1..4 tokens, Q5_K and Q6_K with 3 or 4 (its columns are laid out for four
// tokens, and two are as fast on the vector ALU); in_dim a multiple of 256, all activations staged at once or in_dim a
// multiple of 2048.
static inline int gemv_mfma_supported(unsigned type, int tokens, unsigned in_dim) {
  if ((type != 12 && type != 13 && type != 14) || tokens < (type == 12 ? 1 : 3) || tokens > GEMV_MFMA_MAX_TOKENS || in_dim == 0 ||
      (in_dim & 255u))
    return 0;
  return (unsigned)tokens * (in_dim >> 8) <= (unsigned)GEMV_MFMA_MAX_UNITS(tokens) || (in_dim & 2047u) == 0;
}
// 16-row tiles per row group and the grid: aim at one workgroup per compute unit (256 of them)
static inline unsigned gemv_mfma_tiles(int tokens, unsigned in_dim, unsigned out_dim) {
  (void)tokens;
  const unsigned nwr = GEMV_MFMA_WAVES >> gemv_mfma_log2_kslices(in_dim >> 8);
  const unsigned ntiles = (out_dim + 15) / 16, tmax = (unsigned)GEMV_MFMA_TMAX;
  unsigned t = ntiles / (nwr * 256u);
  if (t < 1) t = 1;
  if (t > tmax) t = tmax;
  return t;
}
static inline unsigned gemv_mfma_grid(int tokens, unsigned in_dim, unsigned out_dim) {
  const unsigned nwr = GEMV_MFMA_WAVES >> gemv_mfma_log2_kslices(in_dim >> 8);
  const unsigned ntiles = (out_dim + 15) / 16, per_wg = nwr * gemv_mfma_tiles(tokens, in_dim, out_dim);
  const unsigned groups = (ntiles + per_wg - 1) / per_wg;
  // more row groups of the largest size than compute units: one workgroup per unit walks them with the activations
  // staged once (not where the activations are staged in chunks)
  if (groups > 256u && per_wg == nwr * (unsigned)GEMV_MFMA_TMAX && !gemv_mfma_chunked(tokens, in_dim)) return 256u;
  return groups;
}
static inline unsigned gemv_mfma_lds_bytes(unsigned type, int tokens, unsigned in_dim) {
  const int mp = type == 14 ? 4 : (tokens <= 1 ? 1 : (tokens <= 2 ? 2 : 4));
  const unsigned nsums = type == 14 ? 16u : 8u;   // sub-block sums of the activations kept per (token, super-block)
  // (token, super-block) units the activation image holds: all of them, or one chunk per wavefront
  const unsigned per_wave = (unsigned)(GEMV_MFMA_MAX_UNITS(tokens) / GEMV_MFMA_WAVES / tokens * tokens);
  const unsigned units = gemv_mfma_chunked(tokens, in_dim) ? GEMV_MFMA_WAVES * per_wave : (unsigned)tokens * (in_dim >> 8);
  return 64u + GEMV_MFMA_WAVES * GEMV_MFMA_TMAX * 1024u + GEMV_MFMA_WAVES * GEMV_MFMA_TMAX * (unsigned)mp * 64u +
         units * (4u + 4u * nsums + 1024u);
}

// ---- several tokens in one pass over a Q4_K, Q5_K or Q6_K matrix (gemv_mt.hpp): 8 wavefronts = 8 k-slices, activations packed once
#define GEMV_MT_WAVES 8
#define GEMV_MT_TMAX 3              // 16-row tiles a wavefront carries at most (Q4_K, Q5_K; Q6_K two)
#define GEMV_MT_MAX_TOKENS 8
#define GEMV_MT_MAX_IN_DIM 12288u
// Shapes the kernels take: Q4_K, Q5_K, Q6_K or Q8_0 (eight blocks at a time), 2..8 tokens, in_dim a multiple of 256 up to 12288 (1..6 super-blocks per
// k-slice; a row whose super-blocks do not divide by 8 is worked on as if zeros filled it up, gemv_mt_padded_sb).
static inline GEMV_HD int gemv_mt_supported(unsigned type, int tokens, unsigned in_dim) {
  return (type == 12 || type == 13 || type == 14 || type == 8) && tokens >= 2 && tokens <= GEMV_MT_MAX_TOKENS && in_dim != 0 &&
         (in_dim & 255u) == 0 && in_dim <= GEMV_MT_MAX_IN_DIM;
}
// super-blocks of the activation image: the row's, rounded up to a multiple of the 8 k-slices
static inline GEMV_HD unsigned gemv_mt_padded_sb(unsigned in_dim) { return ((in_dim >> 8) + 7u) & ~7u; }
// Token count from which one matrix goes through pack + one pass rather than the per-token-group kernels (0: never): where
// the pair measures faster. Q6_K from three tokens; Q4_K and Q5_K from four on rows of 4096 values and more, else from five.
// Tall matrices of up to 4096 columns (an output head): the workgroups walk many row groups and pay their start once, which
// puts the kernel ahead earlier - Q6_K from two tokens at GEMV_MT_TALL_ROWS rows, Q4_K and Q5_K from three there and from
// two at GEMV_MT_VERY_TALL_ROWS. Q8_0 (the other way is one launch on the vector ALU for up to eight tokens, whose time
// grows with every token: 3584 -> 1024 takes 9.0 / 13.6 / 21.3 us at 2 / 4 / 8 tokens against 7.3 in one pass): from two
// tokens on rows of 3584 values and more and on tall matrices, else from three; half-filled rows (1024 values) from five.
#define GEMV_MT_TALL_ROWS 40960u
#define GEMV_MT_VERY_TALL_ROWS 98304u
static inline unsigned gemv_mt_from(unsigned type, unsigned in_dim, unsigned out_dim) {
  if (!gemv_mt_supported(type, 2, in_dim)) return 0;
  // rows that fill less than three quarters of their eight k-slices (1024 values: half of them): from five tokens, where
  // the per-token-group kernels start to read the weights twice
  const int sparse = 4u * (in_dim >> 8) < 3u * gemv_mt_padded_sb(in_dim);
  if (type == 8) {
    if (out_dim >= GEMV_MT_TALL_ROWS) return 2u;
    return sparse ? 5u : (in_dim >= 3584u ? 2u : 3u);
  }
  if (sparse) return 5u;
  if (in_dim <= 4096u && out_dim >= GEMV_MT_TALL_ROWS) return (type == 14 || out_dim >= GEMV_MT_VERY_TALL_ROWS) ? 2u : 3u;
  return type == 14 ? 3u : (in_dim >= 4096u ? 4u : 5u);
}
// The same for a pair, a list of matrices or the fused gate | up | SwiGLU: from two tokens (one pack serves all of them and
// the weights are read once), from five on rows that fill less than three quarters of their k-slices.
static inline unsigned gemv_mt_multi_from(unsigned type, unsigned in_dim) {
  if (!gemv_mt_supported(type, 2, in_dim)) return 0;
  return 4u * (in_dim >> 8) < 3u * gemv_mt_padded_sb(in_dim) ? 5u : 2u;
}
// tiles per wavefront: rows of more than 4096 values one (the operands are streamed); else as many as keep 256 workgroups
// busy, at most three (Q4_K, Q5_K) or two (Q6_K, Q8_0: their units are larger). Host and kernel use the same rule.
static inline GEMV_HD unsigned gemv_mt_tiles(unsigned type, unsigned in_dim, unsigned ntiles) {
  if (in_dim > 4096u) return 1;
  const unsigned tmax = (type == 14 || type == 8) ? 2u : (unsigned)GEMV_MT_TMAX;
  unsigned t = ntiles / 256u;
  if (t < 1) t = 1;
  if (t > tmax) t = tmax;
  return t;
}
static inline unsigned gemv_mt_grid(unsigned type, unsigned in_dim, unsigned total_rows) {
  const unsigned ntiles = (total_rows + 15) / 16, t = gemv_mt_tiles(type, in_dim, ntiles);
  const unsigned groups = (ntiles + t - 1) / t;
  return groups < 256u ? groups : 256u;   // more groups than compute units: the workgroups walk them
}
// the k-slices' partial sums, then per wavefront the slots of its units: 6 x (16 rows x 144 B) for Q4_K, 6 x (16 rows x
// 176 B) for Q5_K, 4 x (16 rows x 240 B) for Q6_K, 4 x (16 rows x 272 B) for Q8_0
// (the sixteen-token kernels keep twice the partial sums)
#define GEMV_MT_X16_LDS_EXTRA (GEMV_MT_WAVES * GEMV_MT_TMAX * 8u * 16u * 4u)
static inline unsigned gemv_mt_lds_bytes(unsigned type) {
  return GEMV_MT_WAVES * GEMV_MT_TMAX * 8u * 16u * 4u +
         GEMV_MT_WAVES * (type == 14 ? 4u * 3840u : (type == 8 ? 4u * 4352u : (type == 13 ? 6u * 2816u : 6u * 2304u)));
}
// bytes of the activation image: per super-block (of the padded count) 8 KiB of operands, then 16 bytes per (super-block, lane) for the scales and
// the sub-block sums (one more matrix-core operand). Q4_K and Q5_K share one image, Q6_K has its own.
static inline unsigned long long gemv_mt_image_bytes(unsigned type, unsigned in_dim) {
  (void)type;
  return (unsigned long long)gemv_mt_padded_sb(in_dim) * (8192u + 1024u);
}

// ---- prefill GEMM: which Q4_K kernel an unsplit launch takes (gemm_q4k.hpp: 128 x 192 tiles, four wavefronts;
// gemm_q4k_wide.hpp: 128 x 256 tiles, eight wavefronts). One workgroup per compute unit either way, so a launch runs in
// rounds of 256 tiles. A round of wide tiles measures 1.24 times a round of the narrower ones (a third more work, done
// with 25 % fewer activation bytes copied per flop and two wavefronts per SIMD), so the wide kernel is taken where it
// saves enough whole rounds: 2048 x 12288 is 3 rounds instead of 4, 512 x 12288 (192 wide tiles: a quarter of the
// compute units idle) and 1024 x 12288 (2 rounds either way) stay with the narrow tiles.
#define GEMM_ROUND_TILES 256u
#define GEMM_WIDE_ROUND_COST_X100 124u
static inline int gemm_q4k_use_wide(unsigned out_dim, unsigned tokens) {
  const unsigned mtiles = (tokens + 127u) / 128u;
  const unsigned narrow = mtiles * ((out_dim + 191u) / 192u), wide = mtiles * ((out_dim + 255u) / 256u);
  if (wide < GEMM_ROUND_TILES) return 0;
  const unsigned rn = (narrow + GEMM_ROUND_TILES - 1) / GEMM_ROUND_TILES, rw = (wide + GEMM_ROUND_TILES - 1) / GEMM_ROUND_TILES;
  return rw * GEMM_WIDE_ROUND_COST_X100 < rn * 100u;
}

// ---- prefill GEMM: which tile a workgroup takes. Workgroups go to the 8 XCDs round-robin (id % 8), each XCD has its own
// L2 and 32 compute units, and a GEMM workgroup has a compute unit to itself, so the workgroups id = 8 l + x with the
// same l / 32 run side by side on XCD x. They are given a block of bnt x bmt = 32 neighbouring tiles (bmt token tiles of
// bnt weight tiles each): a weight tile is then fetched into that L2 once for bmt workgroups and an x tile once for bnt,
// where one token tile per XCD (every workgroup of an XCD on the same x, each on weights of its own) made every L2 fill
// with all the weights. One token tile: the blocks degenerate to that older numbering, which is kept as it is.
#define GEMM_XCD_COUNT 8u
#define GEMM_XCD_UNITS 32u
static inline GEMV_HD unsigned gemm_block_mt(unsigned mtiles) { return mtiles >= 4u ? 4u : (mtiles >= 2u ? 2u : 1u); }
// A block is bnt weight tiles x bmt token tiles: 32 tiles where there are enough of them, fewer when the launch has
// fewer than 256 tiles, so that the blocks still go round all 8 XCDs.
static inline GEMV_HD void gemm_block_shape(unsigned mtiles, unsigned ntiles, unsigned* bmt, unsigned* bnt) {
  *bmt = gemm_block_mt(mtiles);
  const unsigned per_xcd = (mtiles * ntiles + GEMM_XCD_COUNT - 1u) / GEMM_XCD_COUNT;   // tiles an XCD gets when they are dealt evenly
  const unsigned want = (per_xcd + *bmt - 1u) / *bmt, cap = GEMM_XCD_UNITS / *bmt;
  *bnt = want < 1u ? 1u : (want > cap ? cap : want);
}
static inline GEMV_HD unsigned gemm_grid_x(unsigned mtiles, unsigned ntiles) {
  if (mtiles < 2u) return GEMM_XCD_COUNT * ((mtiles * ntiles + GEMM_XCD_COUNT - 1u) / GEMM_XCD_COUNT);
  unsigned bmt, bnt;
  gemm_block_shape(mtiles, ntiles, &bmt, &bnt);
  const unsigned nb = ((ntiles + bnt - 1u) / bnt) * ((mtiles + bmt - 1u) / bmt);
  return GEMM_XCD_COUNT * bmt * bnt * ((nb + GEMM_XCD_COUNT - 1u) / GEMM_XCD_COUNT);
}
// false: this workgroup has no tile (the grid is rounded up to whole blocks)
static inline GEMV_HD bool gemm_tile_of(unsigned id, unsigned mtiles, unsigned ntiles, unsigned* mt, unsigned* nt) {
  const unsigned x = id % GEMM_XCD_COUNT, l = id / GEMM_XCD_COUNT;
  if (mtiles < 2u) {
    const unsigned per = (mtiles * ntiles + GEMM_XCD_COUNT - 1u) / GEMM_XCD_COUNT, vt = x * per + l;
    *mt = vt / ntiles;
    *nt = vt - *mt * ntiles;
    return vt < mtiles * ntiles;
  }
  unsigned bmt, bnt;
  gemm_block_shape(mtiles, ntiles, &bmt, &bnt);
  const unsigned units = bmt * bnt, nbn = (ntiles + bnt - 1u) / bnt, nb = nbn * ((mtiles + bmt - 1u) / bmt);
  const unsigned b = (l / units) * GEMM_XCD_COUNT + x, i = l % units;
  *nt = (b % nbn) * bnt + i / bmt;
  *mt = (b / nbn) * bmt + i % bmt;
  return b < nb && *nt < ntiles && *mt < mtiles;
}

// ---- one-pass kernel, rows above 4096 values: what a streamed unit waits for (gemv_mt.hpp)
// vmcnt value that says "operand set i and unit i of a streamed row group have landed" (T = 1, S super-blocks per
// k-slice, NSLOT units in LDS). Issue order: set 0, unit 0, set 1, unit 1, units 2 .. min(S, NSLOT) - 1 up front; behind unit
// i's arithmetic: set i + 2, then unit i + NSLOT. NA loads per set, NC copies per unit. The answer is the number of loads
// issued, by the time of the wait, behind the later of the two.
static inline GEMV_HD constexpr int mt_stream_wait(int S, int NSLOT, int NS, int NA, int NC, int i) {
  int pos = 0, end_set[8] = {}, end_unit[8] = {};
  const int up = S < NSLOT ? S : NSLOT;
  for (int u = 0; u < up; u++) {
    if (u < NS) end_set[u] = (pos += NA);
    end_unit[u] = (pos += NC);
  }
  for (int j = 0; j < i; j++) {   // what was issued behind the units before i
    if (j + NS < S) end_set[j + NS] = (pos += NA);
    if (j + NSLOT < S) end_unit[j + NSLOT] = (pos += NC);
  }
  const int need = end_set[i] > end_unit[i] ? end_set[i] : end_unit[i];
  return pos - need;
}
