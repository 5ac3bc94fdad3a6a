/*
 * cogni_quant.h - C ABI of the quantized-matmul operators (libcogni_hip.so).
 *
 * Replaces, for one MI355X (gfx950), the reference's CPU operators
 *   ML::GGUF::QuantMatmul.matmul_add   src/ml/gguf/quant_matmul.cr:20-36
 *   ML::GGUF::Dequant.dequantize       src/ml/gguf/dequant.cr:19-31
 * and the GPU kernels its CUDA probes launch (src/ml/cuda/kernels/q{4,5,6}k_gemv_probe.ptx,
 * bin/cuda_q8_gemv_probe.cr:39-227). Weights are the raw GGUF bytes, row-major
 * [out_dim][in_dim / block_elements][block_bytes]; nothing is repacked on the host.
 *
 * Three levels, lowest first:
 *   1. the code object: kernels are unmangled symbols, launched by name through
 *      ml_hip_driver.h exactly as the reference launches PTX entries
 *      (cogni_quant_code_object, cogni_gemv_kernel_name, cogni_gemv_launch_dims);
 *   2. device-pointer operators, asynchronous on a stream (cogni_*_dev);
 *   3. host-buffer operators with the reference's CPU signatures (cogni_dequantize,
 *      cogni_matmul_add) and the QuantWeight handle that keeps weights resident.
 *
 * Every function returns 0 on success, a positive hipError_t value when a HIP call failed, or one
 * of the negative COGNI_ERR_* codes. cogni_last_error() gives the text for the calling thread.
 * There is no CPU fallback: without a gfx950 device every operator fails with an error.
 */
#ifndef COGNI_QUANT_H
#define COGNI_QUANT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ggml tensor type ids, src/ml/gguf/reader.cr:34-49 */
enum {
  COGNI_TYPE_F32 = 0,
  COGNI_TYPE_F16 = 1,
  COGNI_TYPE_Q8_0 = 8,
  COGNI_TYPE_Q4_K = 12,
  COGNI_TYPE_Q5_K = 13,
  COGNI_TYPE_Q6_K = 14,
  COGNI_TYPE_IQ4_NL = 20
};

enum {
  COGNI_ERR_INVALID_ARGUMENT = -1, /* the reference raises ArgumentError / a size check fails */
  COGNI_ERR_UNSUPPORTED_TYPE = -2, /* "Unsupported ... type", quant_matmul.cr:33-34, dequant.cr:29-30 */
  COGNI_ERR_NOT_INITIALIZED = -3,  /* cogni_quant_init has not succeeded in this process */
  COGNI_ERR_NO_DEVICE = -4         /* no gfx950 device: there is no fallback path */
};

enum { COGNI_MAX_GEMV_TOKENS = 8 }; /* tokens one weight-stationary GEMV launch handles */

/* ---- geometry: TensorType#block_bytes / #block_elements / TensorInfo#data_bytes,
 *      src/ml/gguf/reader.cr:51-78,119-127. Return -1 for an unknown type id. No GPU needed. */
int32_t cogni_block_bytes(uint32_t type);
int32_t cogni_block_elements(uint32_t type);
int64_t cogni_data_bytes(uint32_t type, int64_t n_elements);

/* ---- level 1: the code object ---------------------------------------------------------------- */

/* The embedded gfx950 code object, suitable for hipModuleLoadData / mlhip_module_load_data. Takes the
 * place of the PTX text the reference embeds (bin/cuda_q4k_gemv_probe.cr:39, driver.cr:115-119).
 * No GPU needed. */
int cogni_quant_code_object(const void** image, size_t* size);

/* Kernel symbol for (type, tokens, add): "q4_k_gemv_f32", "q6_k_gemv_add_f32_tbatch4", ...
 * tokens in 1..COGNI_MAX_GEMV_TOKENS. Parameters of the kernel, in order:
 *   (w_raw:u64, x:u64, out:u64, in_dim:u32, out_dim:u32)              q4k_gemv_probe.ptx:5-11
 *   (w_raw, x, residual, out, in_dim, out_dim) for the *_add_* kernels  q4k_gemv_probe.ptx:1572-1578
 * x rows at stride in_dim floats, out/residual rows at stride out_dim floats (q4k_gemv_probe.ptx:747-768).
 * Returns NULL for an unsupported combination. No GPU needed. */
const char* cogni_gemv_kernel_name(uint32_t type, uint32_t tokens, int add);
/* Launch geometry of the GEMV kernel for (type, tokens) at this shape: block_x = 256 threads, grid_x =
 * ceil(out_dim / rows_per_block) where rows_per_block depends on the type and token count - except that one token
 * of a K-quant matrix with more such row groups than workgroups are resident together (Q4_K: 1024 of 8 rows; Q5_K and Q6_K:
 * 768, Q6_K 1280 from 10240 row groups) is launched as that many workgroups at most, each walking several groups (the kernels accept any grid_x
 * up to the number of row groups) - all other
 * grid/block extents 1, and shared_mem_bytes of dynamic shared memory (the staged activations), which
 * goes into the shared_mem_bytes argument of the launch (driver.cr:278-286). (The reference's kernels
 * use grid ceil(out_dim/4) x block 128 and no dynamic shared memory, bin/cuda_q4k_gemv_probe.cr:225-230.)
 * No GPU needed. */
int cogni_gemv_launch_dims(uint32_t type, uint32_t tokens, uint32_t in_dim, uint32_t out_dim, uint32_t* grid_x,
                           uint32_t* block_x, uint32_t* shared_mem_bytes);
/* The kernel the library itself launches for this shape where the call does not go through pack + one pass (see
 * cogni_gemv_one_pass_from), with its geometry: for 2..4 tokens of a Q4_K matrix and
 * 3 or 4 tokens of a Q5_K or Q6_K matrix whose activations fit the staging buffer (tokens * in_dim / 256 <= 96, or 64 from
 * 3 tokens) or whose in_dim is a multiple of 2048 (staged a chunk at a time) that is the matrix-core variant
 * "q4_k_gemv_mfma_[add_]f32_tbatchM" / "q5_k_..." / "q6_k_gemv_mfma_[add_]f32_tbatchM" (same parameter list, block 512); for one
 * token of a matrix with so few rows that the plain kernel would run on fewer than 256 workgroups (Q4_K, Q5_K, Q6_K below
 * 2048 rows, Q8_0 below 4096) the variant of the plain kernel with fewer rows per wavefront, "<type>_gemv_[add_]f32_r1" (Q8_0
 * from 2048 rows: "_r2"; same parameter list and block, grid ceil(out_dim / (4 R))); otherwise the kernel
 * cogni_gemv_kernel_name / cogni_gemv_launch_dims describe. *kernel points at thread-local storage that the
 * next call on the thread overwrites. tokens in 1..COGNI_MAX_GEMV_TOKENS. No GPU needed. */
int cogni_gemv_plan(uint32_t type, uint32_t tokens, int add, uint32_t in_dim, uint32_t out_dim, const char** kernel,
                    uint32_t* grid_x, uint32_t* block_x, uint32_t* shared_mem_bytes);
/* Kernel symbol "dequantize_<type>_f32"; parameters (w_raw:u64, out:u64, n_elements:u64); block = 256
 * threads, any grid (grid-stride). NULL for an unsupported type. No GPU needed. */
const char* cogni_dequantize_kernel_name(uint32_t type);

/* ---- initialisation --------------------------------------------------------------------------- */

/* Select device `ordinal`, check that it is gfx950, load the code object and resolve the kernels.
 * Idempotent per process for the same ordinal. */
int cogni_quant_init(int32_t ordinal);
/* Unload the module and free cached scratch buffers. */
int cogni_quant_shutdown(void);

/* ---- level 2: device-pointer operators (asynchronous on `stream`; NULL = the null stream) ----- */

/* Dequant.dequantize on device memory: out[0..n_elements) float32. dequant.cr:19-31. */
int cogni_dequantize_dev(uint64_t w_raw, uint32_t w_type, uint64_t n_elements, uint64_t out, void* stream);

/* Decode GEMV, weights read once for all tokens:
 *   out[m*out_dim + o] = (residual ? residual[m*out_dim + o] : 0) + sum_j x[m*in_dim + j] * deq(W[o][j])
 * fp32 accumulation. tokens >= 1; several tokens of a matrix the one-pass kernel takes (see cogni_gemv_pack_dev below;
 * cogni_gemv_one_pass_from: Q6_K from three tokens, Q4_K and Q5_K from four on rows of 4096 values and more, else from
 * five, tall matrices earlier) go in groups of up to 8 with
 * the weights read once per group; otherwise they are issued as consecutive launches of the token count that measures
 * fastest for the type and shape: up to 4 where cogni_gemv_plan picks the matrix-core kernel, else pairs for the
 * K-quants (one group of three when the count is odd and the matrix is short enough for one workgroup per row group)
 * and up to 8 for Q8_0. in_dim must be a multiple of 256 for Q4_K/Q5_K/Q6_K (the reference requires the same,
 * bin/cuda_q4k_gemv_probe.cr:125); Q8_0 accepts any in_dim >= 1 (its last block is clipped, quant_matmul.cr:241,259).
 * Types: Q8_0, Q4_K, Q5_K, Q6_K on the kernels above; F32, F16 and IQ4_NL (the remaining arms of
 * QuantMatmul.matmul_add, quant_matmul.cr:30-32, 272-368) on plain row kernels "f32_gemv_plain_f32" |
 * "f16_gemv_plain_f32" | "iq4_nl_gemv_plain_f32" (w_raw, x, residual, out, in_dim:u32, out_dim:u32, tokens:u32), block 256
 * (a wavefront per output row), any in_dim >= 1 and any token count in one launch. Every other ggml type is refused with
 * COGNI_ERR_UNSUPPORTED_TYPE and the reference's message. */
int cogni_gemv_dev(uint64_t w_raw, uint32_t w_type, uint64_t x, uint64_t residual, uint64_t out,
                   uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream);

/* Several tokens in ONE pass over the weights (Q4_K, Q5_K, Q6_K and Q8_0, in_dim a multiple of 256 up to 12288, 2..8 tokens): the
 * activations are packed once into an image - per 256-value super-block the matrix-core operands of its instructions (x as
 * two binary16 terms, scaled per token and super-block), then the scales and sub-block sums - and every matrix that meets
 * those activations (q | k | v | gate | up of a layer) is one launch that reads its weights once for all the tokens. The
 * reference's multi-token kernels stop at four tokens per pass (tbatch4, src/ml/cuda/kernels/q4k_gemv_probe.ptx:437-768,
 * q6k_gemv_probe.ptx:977; q5k_gemv_probe.ptx:237). The image depends on the weight type (Q4_K and Q6_K order their
 * sub-blocks differently; Q5_K and Q8_0 - eight of its blocks at a time - read the Q4_K image, so one pack serves matrices
 * of the three types).
 *   cogni_gemv_image_bytes  size of the image for (type, in_dim, tokens); 0 = no one-pass kernel for that combination.
 *   cogni_gemv_pack_dev     kernel "pack_x_mt_q4k_f16" | "pack_x_mt_q6k_f16" (x, image, tokens:u32, in_dim:u32), block 256,
 *                           grid 2 * S with S = in_dim / 256 rounded up to a multiple of 8 (the image holds S super-blocks:
 *                           the eight k-slices of the GEMV take S / 8 each, the ones past the row's end are zeros).
 *   cogni_gemv_packed_dev   `count` (1..8) matrices of one type and in_dim against the image:
 *                           out[i][m*out_dims[i] + o] = (residual ? residual[m*out_dims[0] + o] : 0) + sum_j x[m][j] deq(W_i[o][j])
 *                           (a residual only with count == 1). Kernel "q4_k_gemv_mt_f32" | "q5_k_gemv_mt_f32" |
 *                           "q6_k_gemv_mt_f32" | "q8_0_gemv_mt_f32" (w0, w1, w2,
 *                           image, residual, out0, out1, out2, in_dim, rows0, rows1, rows2, tokens), block 512, up to three
 *                           matrices per launch as one matrix of all their rows (a matrix whose row count is not a multiple
 *                           of 16 ends its launch), geometry from cogni_gemv_packed_launch_dims.
 * The image is caller-owned device memory; pack and GEMV are ordered by the stream. Accuracy: about 5e-7 of max|out|
 * (22-bit activations, exact weights, fp32 accumulation).
 * cogni_gemv_dev (from 3 to 5 tokens on, by type and row length), cogni_gemv_dual_dev and cogni_gemv_many_dev (2 tokens
 * and more) take this path by
 * themselves with an image the library keeps per stream (8 streams at most; a ninth falls back to the kernels
 * cogni_gemv_plan describes, which is counted: cogni_gemv_image_stats). A graph captured from one stream carries that
 * stream's image: replay it on one stream at a time, and not beside eager calls on the capture stream. An image handed
 * out while its stream is capturing is pinned: it keeps its stream key until cogni_quant_shutdown, so that a graph
 * replayed after its capture stream was released or destroyed never shares the image with another stream. */
size_t cogni_gemv_image_bytes(uint32_t w_type, uint32_t in_dim, uint32_t tokens);
/* The token count from which cogni_gemv_dev and cogni_gemv_top1_dev take this path for one matrix (Q6_K 3; Q4_K and Q5_K 4
 * on rows of 4096 values and more, else 5; a tall matrix of up to 4096 columns - 40960 rows and more, an output head -
 * earlier: Q6_K 2, Q4_K and Q5_K 3, and 2 from 98304 rows; Q8_0 2 on rows of 3584 values and more and on tall matrices,
 * else 3), 0 where they never do; below it the call runs the kernel cogni_gemv_plan names. No GPU needed. */
uint32_t cogni_gemv_one_pass_from(uint32_t w_type, uint32_t in_dim, uint32_t out_dim);
/* The same for the calls that take several matrices of one input (cogni_gemv_dual_dev, cogni_gemv_many_dev,
 * cogni_gemv_dual_swiglu_dev): 2, or 5 where a row fills less than three quarters of the eight k-slices the kernel
 * divides it into (in_dim / 256 rounded up to a multiple of 8: rows of 256..1280, 2304, 2560 values ...); 0 = never.
 * Rows that are not a multiple of 2048 values also wait for 5 tokens in cogni_gemv_one_pass_from when they fill less
 * than that. No GPU needed. */
uint32_t cogni_gemv_one_pass_multi_from(uint32_t w_type, uint32_t in_dim);
/* Gives back the image the library keeps for `stream` (waits for the stream's work first; nothing to do and no error if it
 * has none). Call it before destroying a stream that ran multi-token GEMVs: the eight slots are otherwise used up by the
 * first eight streams of the process, and later streams run the per-token-group kernels. A graph captured on the stream
 * recorded while the stream was capturing keeps the image pinned: the call then changes nothing (see above). */
int cogni_gemv_release_stream(void* stream);
/* What became of the library's images: how many slots there are, how many belong to a stream, how many of those are
 * pinned by a capture, and how many multi-token calls found no slot and ran the per-token-group kernels instead (two or
 * four passes over the weights where one was possible: slower, same results to the bar). Any pointer may be null. */
int cogni_gemv_image_stats(uint32_t* slots, uint32_t* in_use, uint32_t* pinned, uint64_t* calls_without_image);
/* Passes over the weights that cogni_gemv_dev makes for a call of `tokens` tokens when an image slot is at hand: 1 where
 * the one-pass kernel takes the shape (ceil(tokens / 8) beyond eight tokens), else one per token group of the kernels
 * cogni_gemv_plan names (groups of up to four on the matrix cores, pairs on the vector ALU, eight for Q8_0). -1 for a
 * type or shape the call refuses. No GPU needed. */
int32_t cogni_gemv_passes(uint32_t w_type, uint32_t tokens, uint32_t in_dim, uint32_t out_dim);
/* Launch geometry of the one-pass kernel for a launch of total_rows rows (all its matrices together): a workgroup's eight
 * wavefronts carry t tiles of 16 rows at a time (in_dim above 4096: t = 1; else t = clamp(tiles / 256, 1, 3), Q6_K at most 2),
 * a row group is t tiles, grid_x = min(256, row groups) and the workgroups walk the groups blockIdx.x, blockIdx.x +
 * grid_x, ...; block_x = 512; shared_mem_bytes 122880 (Q4_K) or 135168 (Q6_K). No GPU needed. */
int cogni_gemv_packed_launch_dims(uint32_t w_type, uint32_t in_dim, uint32_t total_rows, uint32_t* grid_x, uint32_t* block_x,
                                  uint32_t* shared_mem_bytes);
int cogni_gemv_pack_dev(uint64_t x, uint32_t w_type, uint32_t in_dim, uint32_t tokens, uint64_t image, void* stream);
int cogni_gemv_packed_dev(const uint64_t* w_raw, uint32_t w_type, uint64_t image, uint64_t residual, const uint64_t* out,
                          const uint32_t* out_dims, uint32_t count, uint32_t in_dim, uint32_t tokens, void* stream);
/* Nine to sixteen tokens in one pass over the weights (Q4_K, Q5_K, Q6_K, Q8_0): the one-pass kernels with their sixteen activation rows
 * as sixteen tokens in ONE binary16 term each instead of eight tokens x (hi, lo) - the precision class of the prefill GEMM (x
 * rounded to half, |x| < 65504; fp32 sums), at the cost of a decode launch where pack + GEMM + plane sum take twice as long.
 * cogni_gemv_pack16_dev writes the image (cogni_gemv_image_bytes(type, in_dim, 8) bytes: the same size; Q4_K and Q5_K
 * share one, Q6_K has its own; kernels "pack_x_mt16_q4k_f16" | "pack_x_mt16_q6k_f16" (x, image, tokens:u32, in_dim:u32), block
 * 256, grid 4 * ceil(in_dim / 2048) * 8); cogni_gemv_packed16_dev runs up to eight matrices of one type and row length
 * against it, three per launch, a [tokens][out_dim] residual (may be 0) with a single matrix (kernels "q4_k_gemv_mt16_f32" |
 * "q5_k_gemv_mt16_f32" | "q6_k_gemv_mt16_f32" | "q8_0_gemv_mt16_f32" - Q8_0 reads the Q4_K image -, parameters, grid and block of "<type>_gemv_mt_f32", 12 KiB more dynamic
 * shared memory). The reference has no counterpart: its router sends every M > 8 to the prefill GEMM
 * (src/ml/gguf/qwen35_cpu.cr:1478-1490); cogni_matmul_dev takes this path by itself for 9..16 tokens of a K-quant matrix without a bias (Q8_0, whose reference path stays in
 * fp32 at every token count, only on request). */
int cogni_gemv_pack16_dev(uint64_t x, uint32_t w_type, uint32_t in_dim, uint32_t tokens, uint64_t image, void* stream);
/* (cogni_gemv_packed16_swiglu_dev, below: gate | up | SwiGLU against the same image, as cogni_gemv_packed_swiglu_dev does for up
 * to eight tokens - kernel "q4_k_gemv_mt16_swiglu_f32", the parameters of "q4_k_gemv_mt_swiglu_f32"; the bits of
 * cogni_gemv_packed16_dev on the pair followed by cogni_swiglu_dev) */
/* (cogni_rmsnorm_pack16_dev, cogni_add_rmsnorm_pack16_dev: the norms that write this image themselves, as cogni_rmsnorm_pack_dev /
 * cogni_add_rmsnorm_pack_dev write the eight-token one - 1..16 tokens, rows of a multiple of 256 up to 4096 values, byte for byte
 * what cogni_gemv_pack16_dev makes of the normalised rows; kernels "rmsnorm_pack_x16_q4k_f32" | "rmsnorm_pack_x16_q6k_f32" and
 * "add_rmsnorm_pack_x16_q4k_f32" | "add_rmsnorm_pack_x16_q6k_f32", the parameters of the eight-token ones, grid 16) */
int cogni_rmsnorm_pack16_dev(uint64_t x, uint64_t norm, uint64_t out, uint32_t w_type, uint64_t image, uint32_t dim, uint32_t tokens,
                             float eps, void* stream);
int cogni_add_rmsnorm_pack16_dev(uint64_t x, uint64_t add, uint64_t norm, uint64_t residual_out, uint64_t normed_out, uint32_t w_type,
                                 uint64_t image, uint32_t dim, uint32_t tokens, float eps, void* stream);
int cogni_gemv_packed16_swiglu_dev(uint64_t w_gate, uint64_t w_up, uint32_t w_type, uint64_t image, uint64_t out, uint32_t in_dim,
                                   uint32_t out_dim, uint32_t tokens, void* stream);
int cogni_gemv_packed16_dev(const uint64_t* w_raw, uint32_t w_type, uint64_t image, uint64_t residual, const uint64_t* out,
                            const uint32_t* out_dims, uint32_t count, uint32_t in_dim, uint32_t tokens, void* stream);
/* The gate and up projections and the SwiGLU against an image, one launch:
 *   out[m*out_dim + o] = silu(sum_j x[m][j] deq(W_gate[o][j])) * sum_j x[m][j] deq(W_up[o][j])
 * Kernel "q4_k_gemv_mt_swiglu_f32" (w_gate, w_up, image, out, in_dim, out_dim, tokens), block 512, grid = min(256,
 * ceil(out_dim / 16)), dynamic shared memory as q4_k_gemv_mt_f32. Q4_K only. The values of
 * cogni_gemv_packed_dev on the pair followed by cogni_swiglu_dev, bit for bit. cogni_gemv_dual_swiglu_dev takes this path
 * for 2 tokens and more. */
int cogni_gemv_packed_swiglu_dev(uint64_t w_gate, uint64_t w_up, uint32_t w_type, uint64_t image, uint64_t out, uint32_t in_dim,
                                 uint32_t out_dim, uint32_t tokens, void* stream);

/* Two matrices of one shape against the same activations (the gate | up, k | v pairs):
 *   out_a[m*out_dim + o] = sum_j x[m*in_dim + j] * deq(W_a[o][j]),  out_b likewise with W_b.
 * One token of a Q4_K pair is one launch of "q4_k_dual_gemv_f32" (w_raw_a, w_raw_b, x, out_a, out_b, in_dim, out_dim),
 * the parameter list of the reference's q4_k_dual_gemv_warp4_f32 (src/ml/cuda/kernels/q4k_dual_gemv_probe.ptx:5-13,
 * used by src/ml/cuda/qwen_recurrent_layer_runner.cr:519-520): output row r of the launch is row r of W_a for
 * r < out_dim and row r - out_dim of W_b above; block and dynamic shared memory as cogni_gemv_launch_dims gives for
 * one token, grid_x = ceil(2*out_dim / 16), grid_y = tokens (one token per slice, x + y*in_dim,
 * out_* + y*out_dim, the reference's ..._batched entry). Several tokens of a Q4_K pair with out_dim a multiple of 16
 * and a row length the matrix-core kernel takes: "q4_k_dual_gemv_mfma_f32_tbatchM", same parameters, block 512, grid and
 * shared memory of one matrix with 2*out_dim rows (cogni_gemv_plan), per group of up to four tokens. Every other case is
 * issued as two cogni_gemv_dev calls. */
int cogni_gemv_dual_dev(uint64_t w_raw_a, uint64_t w_raw_b, uint32_t w_type, uint64_t x, uint64_t out_a, uint64_t out_b,
                        uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream);

/* Several matrices of one type and in_dim against the same activations (q | k | v, gate | up) on device pointers: the
 * reference's qmatvec_many seam (src/ml/gguf/qwen35_cpu.cr:1419-1445), which hands a list of weights and one x to the
 * GPU arm.  out[i][m*out_dims[i] + o] = sum_j x[m*in_dim + j] * deq(W_i[o][j]).
 * Two or three Q4_K matrices, two or more tokens, every out_dims[i] a multiple of 16 and a row length the matrix-core
 * kernel takes: one launch per group of up to four tokens of "q4_k_many_gemv_mfma_f32_tbatchM"
 * (w0, w1, w2, x, out0, out1, out2, in_dim, rows0, rows1, rows2), block 512, grid and shared memory of one matrix with
 * the sum of the rows (cogni_gemv_plan), the activations staged once for all of them. Two matrices of one shape: as
 * cogni_gemv_dual_dev. One token of Q4_K matrices: up to three per launch of "q4_k_many_gemv_f32" (the same parameter
 * list), block, shared memory and grid as cogni_gemv_launch_dims gives one token of a matrix with the sum of the rows; each
 * row comes out bit for bit as from cogni_gemv_dev. Everything else: one cogni_gemv_dev per matrix. count in 1..8. */
int cogni_gemv_many_dev(const uint64_t* w_raw, uint32_t w_type, uint64_t x, const uint64_t* out, const uint32_t* out_dims,
                        uint32_t count, uint32_t in_dim, uint32_t tokens, void* stream);

/* out[i] = silu(gate[i]) * up[i], silu(g) = g / (1 + exp(-g)) in fp32: kernel "swiglu_f32" (gate, up, out, n:u32),
 * block 256, grid ceil(n/256) - the reference's swiglu_f32 (bin/cuda_ffn_sequence_probe.cr:46-84, CPU form :189-191). */
int cogni_swiglu_dev(uint64_t gate, uint64_t up, uint64_t out, uint32_t n, void* stream);

/* The gate and up projections and the SwiGLU in one launch (Q4_K):
 *   out[m*out_dim + o] = silu(sum_j x[m][j] deq(W_gate[o][j])) * sum_j x[m][j] deq(W_up[o][j])
 * i.e. the reference's gate/up GEMVs followed by swiglu_f32 (bin/cuda_ffn_sequence_probe.cr: FFN sequence) without
 * the intermediate vectors. Kernel "q4_k_dual_gemv_swiglu_f32" (w_gate, w_up, x, out, in_dim, out_dim): block and
 * dynamic shared memory as for one token of cogni_gemv_launch_dims, grid_x = ceil(out_dim / 8),
 * grid_y = tokens (one token per slice). Several tokens with out_dim a multiple of 16 and a row length the matrix-core
 * kernel takes: "q4_k_dual_gemv_swiglu_mfma_f32_tbatchM", same parameters, per group of up to four tokens, block 512,
 * shared memory as cogni_gemv_plan gives for the token count, grid = min(256, out_dim / 16 / row groups per workgroup).
 * Other types return COGNI_ERR_UNSUPPORTED_TYPE: compose
 * cogni_gemv_dual_dev and cogni_swiglu_dev. */
int cogni_gemv_dual_swiglu_dev(uint64_t w_gate, uint64_t w_up, uint32_t w_type, uint64_t x, uint64_t out, uint32_t in_dim,
                               uint32_t out_dim, uint32_t tokens, void* stream);

/* RMSNorm of `tokens` rows of `dim` floats: inv = 1 / sqrt(sum(x^2) / dim + eps), out[i] = (x[i] * inv) * norm[i], all
 * in fp32. Kernel "rmsnorm_f32" (x, norm, out, dim:u32, eps:f32), block 256, grid = tokens - the reference's
 * rmsnorm_vec_parallel_probe and its batched form (src/ml/cuda/kernels/deltanet_step_probe.ptx:744, :1157; CPU form
 * src/ml/gguf/qwen35_cpu.cr:484-490, which sums the squares in Float64). */
int cogni_rmsnorm_dev(uint64_t x, uint64_t norm, uint64_t out, uint32_t dim, uint32_t tokens, float eps, void* stream);

/* residual_out = x + add, normed_out = rmsnorm(residual_out): the step between attention and the FFN of a decoder layer
 * (src/ml/gguf/qwen35_cpu.cr:1705-1708). Kernel "add_rmsnorm_f32" (x, add, norm, residual_out, normed_out, dim:u32,
 * eps:f32), block 256, grid = tokens - the reference's add_rmsnorm_vec_parallel_probe and its batched form
 * (src/ml/cuda/kernels/deltanet_step_probe.ptx:906, :1324). residual_out may alias x. */
int cogni_add_rmsnorm_dev(uint64_t x, uint64_t add, uint64_t norm, uint64_t residual_out, uint64_t normed_out, uint32_t dim,
                          uint32_t tokens, float eps, void* stream);

/* The two norms with a second output: the normalised rows as the activation image of the one-pass multi-token GEMV
 * (cogni_gemv_pack_dev below), so that the projections behind a norm (q | k | v, gate | up of a decoder layer) go straight
 * to cogni_gemv_packed_dev / cogni_gemv_packed_swiglu_dev without a pack launch. `image` holds cogni_gemv_image_bytes(w_type,
 * dim, tokens) bytes and comes out bit for bit as cogni_gemv_pack_dev writes it from the normalised rows; out / normed_out
 * may be 0 (the normalised rows then exist only as the image). tokens in 1..8; dim a row length the one-pass kernels take,
 * up to 4096 (2048 or 4096); w_type names the image (Q4_K and Q5_K share one, Q6_K has its own). Kernels
 * "rmsnorm_pack_q4k_f32" | "rmsnorm_pack_q6k_f32" (x, norm, out, image, dim:u32, tokens:u32, eps:f32) and
 * "add_rmsnorm_pack_q4k_f32" | "add_rmsnorm_pack_q6k_f32" (x, add, norm, residual_out, normed_out, image, dim:u32, tokens:u32,
 * eps:f32), block 256, grid 8 (the image's token slots). No counterpart in the reference, whose multi-token kernels read
 * fp32 activations (src/ml/cuda/kernels/q4k_gemv_probe.ptx:437-768). */
int cogni_rmsnorm_pack_dev(uint64_t x, uint64_t norm, uint64_t out, uint32_t w_type, uint64_t image, uint32_t dim, uint32_t tokens,
                           float eps, void* stream);
int cogni_add_rmsnorm_pack_dev(uint64_t x, uint64_t add, uint64_t norm, uint64_t residual_out, uint64_t normed_out, uint32_t w_type,
                               uint64_t image, uint32_t dim, uint32_t tokens, float eps, void* stream);
/* The norms in front of the prefill GEMMs (src/ml/gguf/qwen35_cpu.cr:1705-1722: the rms_norm that feeds the
 * qmatmul_nobias calls of a prefill layer): the normalised rows leave as the packed fp16 activations cogni_gemm_pack_dev
 * would make of them, bit for bit, in the layout of `w_type` (Q4_K and Q5_K share one, Q6_K has its own), so that
 * cogni_gemm_packed_dev and its siblings follow with no pack launch. `out` / `normed_out` may be 0 (the normalised rows then
 * exist only packed). dim a multiple of 256 up to 4096; workspace_bytes >= cogni_gemm_workspace_bytes(w_type, dim, tokens).
 * Kernels "rmsnorm_gemm_pack_q4k_f32" | "rmsnorm_gemm_pack_q6k_f32" (x, norm, out, workspace, dim:u32, tokens:u32, eps:f32)
 * and "add_rmsnorm_gemm_pack_q4k_f32" | "add_rmsnorm_gemm_pack_q6k_f32" (x, add, norm, residual_out, normed_out, workspace,
 * dim:u32, tokens:u32, eps:f32), block 256, grid 128 * ceil(tokens / 128). */
int cogni_rmsnorm_gemm_pack_dev(uint64_t x, uint64_t norm, uint64_t out, uint32_t w_type, uint64_t workspace, size_t workspace_bytes,
                                uint32_t dim, uint32_t tokens, float eps, void* stream);
int cogni_add_rmsnorm_gemm_pack_dev(uint64_t x, uint64_t add, uint64_t norm, uint64_t residual_out, uint64_t normed_out, uint32_t w_type,
                                    uint64_t workspace, size_t workspace_bytes, uint32_t dim, uint32_t tokens, float eps, void* stream);

/* One row of a Q4_K or Q6_K embedding matrix chosen by a token id that lives on the device: output[0..hidden_dim) =
 * dequantized row token_ids[0] (zeros if the id is not below vocab_size) and history[token_index] = token_ids[0].
 * Kernel "embed_<prefix>_f32_from_token_id" (w_raw, token_ids:u32*, output, history:u32*, token_index:u32,
 * hidden_dim:u32, vocab_size:u32), block 256, grid ceil(hidden_dim / 1024) - the reference's
 * embed_q4k_f32_from_token_id_cuda (src/ml/cuda/kernels/embed_q4k_probe.ptx:5-13, launched from
 * bin/cuda_mixed_stack_probe.cr:935-941 with grid hidden_dim / 256). hidden_dim must be a multiple of 256. */
int cogni_embed_dev(uint64_t w_raw, uint32_t w_type, uint64_t token_ids, uint64_t output, uint64_t history,
                    uint32_t token_index, uint32_t hidden_dim, uint32_t vocab_size, void* stream);

/* Output head without the logits: for each token the index of the largest element of W x and that value
 * (top1_ids: u32[tokens], top1_values: f32[tokens]); of equal values the lowest index wins, as in the reference's CPU scan
 * (bin/cuda_mixed_stack_probe.cr:1485-1497). Groups of up to 8 tokens of a Q4_K or Q6_K matrix the one-pass kernel takes
 * (from cogni_gemv_one_pass_from(w_type, in_dim, out_dim) tokens, with the library's image of `stream`) are three launches: the
 * pack, "q4_k_gemv_mt_top1_partial_f32" | "q6_k_gemv_mt_top1_partial_f32" (w_raw, image, partial_ids, partial_values,
 * in_dim, out_dim, tokens; the geometry of cogni_gemv_packed_launch_dims) - the weights once for the group, the arg-max
 * inside - and the reduce below. Otherwise two launches per group of tokens: groups of 3 or 4 tokens of a Q4_K or Q6_K
 * matrix take the matrix-core kernel "<prefix>_gemv_mfma_top1_partial_f32_tbatchM" (same parameters, the geometry of
 * cogni_gemv_plan) where that kernel takes the shape and its grid fits the partial buffers; otherwise groups of up to
 * 2 tokens (Q4_K, Q6_K; one token for the other types):
 * kernel "<prefix>_gemv_top1_partial_f32[_tbatchM]" (w_raw, x, partial_ids, partial_values, in_dim, out_dim) -
 * the reference's q6_k_gemv_top1_partial_f32 (src/ml/cuda/kernels/q6k_gemv_probe.ptx:1331), with the grid, block and
 * shared memory of the GEMV of that type and token count and one (id, value) per workgroup and token - then
 * "top1_reduce_f32" (partial_ids, partial_values, out_ids, out_values, count:u32), block 1024, grid = tokens of the group -
 * the reference's output_top1_values_reduce_probe (src/ml/cuda/qwen_output_head_runner.cr:530, launched :939-940).
 * partial_ids / partial_values are caller-owned scratch of tokens * cogni_gemv_top1_partials(w_type, out_dim) elements. */
uint32_t cogni_gemv_top1_partials(uint32_t w_type, uint32_t out_dim);
int cogni_gemv_top1_dev(uint64_t w_raw, uint32_t w_type, uint64_t x, uint64_t partial_ids, uint64_t partial_values,
                        uint64_t top1_ids, uint64_t top1_values, uint32_t in_dim, uint32_t out_dim, uint32_t tokens,
                        void* stream);

/* The top-1 of up to 8 tokens against a caller-owned activation image (cogni_gemv_pack_dev, or the norms that write it:
 * cogni_rmsnorm_pack_dev): what cogni_gemv_top1_dev launches behind its own pack - "q4_k_gemv_mt_top1_partial_f32" |
 * "q6_k_gemv_mt_top1_partial_f32", then "top1_reduce_f32". Q4_K and Q6_K, in_dim a row length the one-pass kernels take,
 * tokens in 1..8 (an image packed for one token is that token and seven zero slots). partial_ids / partial_values as for
 * cogni_gemv_top1_dev. */
int cogni_gemv_packed_top1_dev(uint64_t w_raw, uint32_t w_type, uint64_t image, uint64_t partial_ids, uint64_t partial_values,
                               uint64_t top1_ids, uint64_t top1_values, uint32_t in_dim, uint32_t out_dim, uint32_t tokens,
                               void* stream);

/* cogni_gemv_top1_dev for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the same launches and the same results, with the per-workgroup partial
 * results in a static device array inside the library instead of caller-owned buffers. No counterpart in the
 * reference. Allocates nothing and frees nothing. Limit: tokens * cogni_gemv_top1_partials(w_type, out_dim) must not
 * exceed COGNI_TOP1_NOALLOC_MAX_PARTIALS (512 KiB of device memory per GPU, held until the process ends); beyond it the
 * call fails with COGNI_ERR_INVALID_ARGUMENT and launches nothing. Every call on a GPU uses that GPU's one array: calls
 * that overlap on one GPU (two streams, two threads) race; calls on one stream are ordered and safe. Nothing in the
 * array needs clearing between calls (every slot read was written by the same call). Needs cogni_quant_init on the
 * current device. Groups of tokens that go through the one-pass kernel use the library's activation image of `stream`
 * (allocated by cogni_quant_init, not by the call); recorded under stream capture that image is pinned to the stream
 * for the life of the library, as described at cogni_gemv_image_bytes. */
enum { COGNI_TOP1_NOALLOC_MAX_PARTIALS = 65536 };
int cogni_gemv_top1_noalloc_dev(uint64_t w_raw, uint32_t w_type, uint64_t x, uint64_t top1_ids, uint64_t top1_values,
                                uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream);

/* Prefill GEMM for `tokens` > 8 (Q4_K, Q5_K, Q6_K): out[m*out_dim + o] = (bias ? bias[o] : 0) + sum_j x[m*in_dim + j] * deq(W[o][j]).
 * x and the dequantized weights are rounded to fp16 and multiplied on the matrix cores with fp32
 * accumulation, the precision of the reference's Metal prefill kernels (src/ml/gguf/kernels/gemm_q4k.metal:
 * 97-105,678-686; Q5_K and Q6_K: gemm_q56k.metal, pipelines mm5 / mm6 src/ml/gguf/qwen35_metal.cr:11035); expect about 5e-4 of
 * max|out| where the GEMV path gives 1e-6. The conversion of x is the reference's plain `(half)y[i]` (gemm_q4k.metal:678-684):
 * an activation beyond the binary16 range (|x| > 65504) becomes infinite and its token's outputs Inf or NaN, where the GEMV
 * kernels (any token count up to 8: they scale every token and super-block by its own power of two) follow fp32. Callers whose
 * activations can be that large keep to the GEMV path: cogni_set_gemm_threshold(1 << 30). A non-finite activation gives
 * non-finite outputs for its token on every path (the multi-token GEMV kernels NaN where the reference's sum is +-Inf); the
 * other tokens of the call are not affected. `workspace` is caller-owned device memory of at least
 * cogni_gemm_workspace_bytes(...) bytes (x repacked as fp16, in the k order of the weight type); nothing is allocated.
 * Kernels: pack_x_f16_q4k (Q4_K and Q5_K) | pack_x_f16_q6k (x, workspace, tokens, in_dim) then
 *          q4_k_gemm_f16 | q5_k_gemm_f16 | q6_k_gemm_f16 (w_raw, workspace, bias, out, in_dim, out_dim, tokens,
 *          bias_stride: 0 for a [out_dim] bias, out_dim for a [tokens][out_dim] residual), block 256,
 *          grid from cogni_gemm_plan (whole blocks of 32 tiles of 128 x 192, 8 XCDs at a time), no dynamic shared memory; or, where
 *          tiles of 128 x 192 times the k split would leave compute units idle (the 4096-row projections at 512 tokens),
 *          q4_k_gemm_n128_f16 | q5_k_gemm_n128_f16 | q6_k_gemm_n128_f16 (same arguments and block, tiles of 128 x 128); or,
 *          for Q4_K launches that fill whole rounds of 128 x 256 tiles, q4_k_gemm_wide_f16 (same arguments), block 512.
 *          Launches of up to 64 tokens take the forms of the 192- and 128-row kernels that work on the first 64 tokens of
 *          the token tile, <type>_gemm_m64_f16 | <type>_gemm_m64_n128_f16 (same arguments and block).
 *          cogni_gemm_plan says which, with the grid; all of them give the same bits for the same k split.
 * (pack_x_f16_*: block 256, grid ceil(tokens/128)*16*(in_dim/256).) Other types: COGNI_ERR_UNSUPPORTED_TYPE. */
size_t cogni_gemm_workspace_bytes(uint32_t w_type, uint32_t in_dim, uint32_t tokens);
/* The workspace size with which cogni_gemm_dev may also split the k range: a launch with fewer than 128 tiles of
 * 128 tokens x 192 rows (few tokens, or a short out_dim such as the 12288 -> 4096 down projection) would leave most
 * compute units idle, so up to 8 workgroups per tile each take a run of super-blocks (at least two), write their sums
 * to planes behind the packed activations, and gemm_sum_splits_f32 (planes, bias, out, tokens*out_dim, out_dim, splits, bias_stride;
 * block 256, grid ceil(tokens*out_dim/1024)) adds the planes in a fixed order, so results repeat from run to run.
 * The GEMM kernels take the split as gridDim.y. Equal to cogni_gemm_workspace_bytes(...) where no split applies; with a
 * workspace smaller than this, cogni_gemm_dev runs unsplit. No counterpart in the reference (its Metal GEMM does not
 * split k). */
size_t cogni_gemm_workspace_bytes_split(uint32_t w_type, uint32_t in_dim, uint32_t out_dim, uint32_t tokens);
/* The two halves of cogni_gemm_dev for callers whose projections share their activations (q | k | v, gate | up of a layer:
 * one pack, several GEMMs): cogni_gemm_pack_dev writes the packed fp16 activations to the head of the workspace
 * (cogni_gemm_workspace_bytes; Q4_K and Q5_K share one layout, Q6_K has its own), cogni_gemm_packed_dev runs the GEMM of one
 * matrix against them (the k-split planes, when the workspace has room for them, live behind the packed activations and
 * are reused by every call - calls on one stream are ordered). cogni_gemm_dev is the two in a row. The counterpart of the
 * packed activation image of the decode kernels (cogni_gemv_pack_dev); no counterpart in the reference, whose Metal GEMM
 * converts x inside the kernel (gemm_q4k.metal:678-686). */
int cogni_gemm_pack_dev(uint64_t x, uint32_t w_type, uint32_t in_dim, uint32_t tokens, uint64_t workspace, size_t workspace_bytes,
                        void* stream);
int cogni_gemm_packed_dev(uint64_t w_raw, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, uint64_t bias, uint64_t out,
                          uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream);
int cogni_gemm_dev(uint64_t w_raw, uint32_t w_type, uint64_t x, uint64_t bias, uint64_t out, uint32_t in_dim,
                   uint32_t out_dim, uint32_t tokens, uint64_t workspace, size_t workspace_bytes, void* stream);
/* The prefill forms of the fused decode operators, for a feed-forward block at more tokens than the GEMV path takes
 * (src/ml/gguf/qwen35_cpu.cr:1711-1722 is the sequence, src/ml/gguf/kernels/gemm_mm.metal:651 `simd_mm_q6k_f32out_add`
 * and gemm_q4k.metal:1233 `simd_mm_q4k_h16_b64_swiglu` the reference's kernels), both against activations
 * cogni_gemm_pack_dev has packed:
 *   cogni_gemm_packed_add_dev     out[m][o] = residual[m][o] + sum_j x[m][j] * deq(W[o][j]); residual is [tokens][out_dim]
 *                                 fp32 and may be `out` itself. The same kernels as cogni_gemm_packed_dev with their
 *                                 last argument (bias_stride) set to out_dim instead of 0.
 *   cogni_gemm_packed_swiglu_dev  out[m][o] = silu(g) * u, g = x[m] . W_gate[o], u = x[m] . W_up[o] (Q4_K; two matrices of
 *                                 out_dim rows; the sums as cogni_gemm_packed_dev gives them, silu as swiglu_f32): the
 *                                 gate and up matrices never exist in memory. Kernel q4_k_gemm_swiglu_f16 (w_gate, w_up,
 *                                 workspace, out, in_dim, out_dim, tokens), block 256, grid as cogni_gemm_plan gives it
 *                                 for a matrix of 2 * out_dim rows. Other types: COGNI_ERR_UNSUPPORTED_TYPE. */
int cogni_gemm_packed_add_dev(uint64_t w_raw, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, uint64_t residual, uint64_t out,
                              uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream);
int cogni_gemm_packed_swiglu_dev(uint64_t w_gate, uint64_t w_up, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, uint64_t out,
                                 uint32_t in_dim, uint32_t out_dim, uint32_t tokens, void* stream);
/* Several matrices of one type and row length against the same packed activations in one launch - q | k | v | gate | up of
 * a prefill layer, the counterpart for M > 8 of cogni_gemv_many_dev (the reference issues one qmatmul_nobias per weight,
 * src/ml/gguf/qwen35_cpu.cr:1478-1490): out_i[m][o] = sum_j x[m][j] * deq(W_i[o][j]), every output bit for bit what
 * cogni_gemm_packed_dev gives for that matrix with a workspace that holds the packed activations only (no k split). One to
 * six matrices, Q4_K or Q5_K, no bias. A matrix that alone gets the 256-row tiles of q4_k_gemm_wide_f16 (cogni_gemm_plan)
 * keeps them and is launched by itself; the others form the list. Kernels "<type>_gemm_many[_m64][_n128]_f16" (list by value: six weight pointers, six
 * output pointers, six row counts, six cumulative tile counts, the count; workspace; in_dim:u32; tokens:u32), block 256,
 * grid as cogni_gemm_plan gives it for a matrix of all the tiles. */
int cogni_gemm_packed_many_dev(const uint64_t* w_raw, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, const uint64_t* outs,
                               const uint32_t* out_dims, uint32_t count, uint32_t in_dim, uint32_t tokens, void* stream);
/* cogni_gemm_packed_swiglu_dev that also hands its products on as the packed activations of the GEMM behind it - the down
 * projection of the same feed-forward block (qwen35_cpu.cr:1711-1722: `act` goes nowhere else): the epilogue writes
 * silu(g) * u as fp16 into `next_workspace` in the layout cogni_gemm_pack_dev gives a [tokens][out_dim] input of a matrix of
 * `next_type` (Q4_K, Q5_K or Q6_K), bit for bit what that call would write from `out`, so cogni_gemm_packed_dev /
 * cogni_gemm_packed_add_dev can follow with in_dim = out_dim and no pack launch. `out` may be 0: the fp32 products are then
 * not stored at all. out_dim a multiple of 256; next_workspace_bytes >= cogni_gemm_workspace_bytes(next_type, out_dim,
 * tokens) (with the k-split planes behind it if the next GEMM is to split: cogni_gemm_workspace_bytes_split); the two
 * workspaces must not overlap. Kernels q4_k_gemm_swiglu_pack_q4k_f16 | q4_k_gemm_swiglu_pack_q6k_f16 (w_gate, w_up,
 * workspace, out | 0, next_workspace, in_dim, out_dim, tokens), launched as q4_k_gemm_swiglu_f16. Up to 64 tokens go to the
 * kernels of the same names with `_m64` in front of `_f16` (q4_k_gemm_swiglu_m64_f16, q4_k_gemm_swiglu_pack_q4k_m64_f16, ...:
 * two tiles of 32 tokens per wavefront, the same parameters and bits). */
int cogni_gemm_packed_swiglu_pack_dev(uint64_t w_gate, uint64_t w_up, uint32_t w_type, uint64_t workspace, size_t workspace_bytes, uint64_t out,
                                      uint32_t next_type, uint64_t next_workspace, size_t next_workspace_bytes, uint32_t in_dim,
                                      uint32_t out_dim, uint32_t tokens, void* stream);
/* The launch cogni_gemm_packed_dev makes for a shape and a workspace of `workspace_bytes`: kernel name, grid (x: tiles,
 * y: k splits; with y > 1 gemm_sum_splits_f32 follows) and block, for hosts that launch by name (level 1) and for
 * callers who want to know which of the two Q4_K tilings a shape gets. Any out pointer may be null. The counterpart of
 * cogni_gemv_plan; the reference picks its Metal prefill pipeline by type only (qwen35_metal.cr:11035). */
int cogni_gemm_plan(uint32_t w_type, uint32_t in_dim, uint32_t out_dim, uint32_t tokens, size_t workspace_bytes, const char** kernel,
                    uint32_t* grid_x, uint32_t* grid_y, uint32_t* block_x);

/* The router of the reference's GPU arm (Qwen35Metal.matmul, src/ml/gguf/qwen35_metal.cr:11404-11449):
 * tokens > threshold and a type with a GEMM kernel -> cogni_gemm_dev, else cogni_gemv_dev. The threshold
 * defaults to 8 (GEMM_BATCH_THRESHOLD, qwen35_metal.cr:70-75) and can be changed with
 * cogni_set_gemm_threshold or the QWEN35_GEMM_BATCH_THRESHOLD environment variable the reference reads.
 * `bias` ([out_dim], may be 0) is only accepted with tokens == 1 or on the GEMM path. `workspace` may be 0
 * when the call stays on the GEMV path. Between the threshold and sixteen tokens a Q4_K, Q5_K or Q6_K matrix without a bias takes
 * cogni_gemv_pack16_dev + cogni_gemv_packed16_dev instead of the GEMM (same precision class, about half the time; the
 * workspace holds the image). */
int cogni_matmul_dev(uint64_t w_raw, uint32_t w_type, uint64_t x, uint64_t bias, uint64_t out, uint32_t in_dim,
                     uint32_t out_dim, uint32_t tokens, uint64_t workspace, size_t workspace_bytes, void* stream);
int cogni_set_gemm_threshold(int32_t tokens);
int32_t cogni_get_gemm_threshold(void);

/* ---- level 3: host-buffer operators with the reference's CPU signatures (synchronous) -------- */

/* Dequant.dequantize(data, type, n_elements) : Array(Float32)   dequant.cr:19
 * `out` receives n_elements floats. data_bytes is checked against the type's geometry. */
int cogni_dequantize(const void* data, size_t data_bytes, uint32_t type, int64_t n_elements, float* out);

/* QuantMatmul.matmul_add(x, rows, in_dim, w_raw, w_type, out_dim, bias) : Array(Float32)   quant_matmul.cr:20
 * result[r*out_dim + o] = bias[o] + sum_j x[r*in_dim + j] * deq(W[o][j]); `result` receives rows*out_dim floats. */
int cogni_matmul_add(const float* x, int32_t rows, int32_t in_dim, const void* w_raw, size_t w_bytes,
                     uint32_t w_type, int32_t out_dim, const float* bias, float* result);

/* QuantWeight {raw, type, out_dim, in_dim} (src/ml/gguf/compute.cr:20-30) with its bytes uploaded once
 * and kept resident, the role of fallback_metal_buffer (compute.cr:36-43). */
typedef struct cogni_quant_weight cogni_quant_weight;
int cogni_weight_create(cogni_quant_weight** qw, const void* raw, size_t raw_bytes, uint32_t type,
                        int32_t out_dim, int32_t in_dim);
uint64_t cogni_weight_device_ptr(const cogni_quant_weight* qw);
/* matmul(x, rows, qw, bias): ComputeBackend#matmul, compute.cr:50; bias may be NULL (qmatvec_nobias,
 * src/ml/gguf/qwen35_cpu.cr:1462-1468). */
int cogni_weight_matmul(const cogni_quant_weight* qw, const float* x, int32_t rows, const float* bias,
                        float* result);
/* qmatvec_many(qws, x) (src/ml/gguf/qwen35_cpu.cr:1419-1445, Qwen35Metal.matmul_many): `count` resident weights of one
 * in_dim against the same x (one token) with one upload of x, one wait and results[i] receiving qws[i].out_dim floats.
 * count == 0 does nothing (the reference returns an empty array). */
int cogni_weight_matvec_many(const cogni_quant_weight* const* qws, int32_t count, const float* x, float* const* results);
int cogni_weight_destroy(cogni_quant_weight* qw);

/* Text of the last failure on the calling thread ("hipModuleLoadData failed with HIP error 209 (...)"). */
const char* cogni_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* COGNI_QUANT_H */
