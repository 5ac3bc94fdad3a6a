// Launch geometry shared by the GEMV kernels and the host code that sizes their grids.
// A workgroup is 4 wavefronts; each wavefront owns GEMV_ROWS_*(tokens) consecutive output rows.
#pragma once

#define GEMV_BLOCK 256
#define GEMV_WAVES 4

#define GEMV_ROWS_Q4K(M) ((M) <= 2 ? 4 : 2)
#define GEMV_ROWS_Q5K(M) 2
#define GEMV_ROWS_Q6K(M) 2
#define GEMV_ROWS_Q80(M) 4

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

// ---- staged activations ------------------------------------------------------------------------
// A workgroup keeps the activations of up to GEMV_LDS_BYTES in LDS: `chunk` whole column sets for the
// token group it is working on. per_set_f4 = float4 count of one column set for that token group.
#define GEMV_LDS_BYTES 49152

#if defined(__HIPCC__) || defined(__CUDACC__)
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
  const int ch = ng > 1 ? 1 : gemv_chunk_sets(per_set_f4, ncs);
  return (unsigned)(per_set_f4 * ch) * 16u + (unsigned)(mg * nsum * 64 * ch) * 4u;
}
