// RMSNorm over fp32 activation rows, one workgroup per token: the kernels that sit between the projections of a
// decoder layer in the reference's runners (src/ml/cuda/kernels/deltanet_step_probe.ptx:744 rmsnorm_vec_parallel_probe,
// :906 add_rmsnorm_vec_parallel_probe, :1157 and :1324 their batched forms; CPU form src/ml/gguf/qwen35_cpu.cr:484-490).
//   inv = 1 / sqrt(sum(x^2) / dim + eps);  out[i] = (x[i] * inv) * norm[i]
// The add form first forms r = x + add, stores r (the residual stream) and normalises r.
// The pack forms also write the normalised rows as the activation image of the one-pass multi-token GEMV (gemv_mt.hpp), so
// that the projections behind a norm (q | k | v, gate | up) need no pack launch of their own: a thread of the short-row
// path holds elements 4 (tid % 64) .. + 3 of super-block 4 k + tid / 64, which is exactly one wavefront per (token,
// super-block) with the lane order of pack_x_mt_*, and the image comes out bit for bit as from that kernel.
// The gemm-pack forms write the normalised rows as the packed fp16 activations of the prefill GEMMs instead (the block
// pack_x_f16_q4k | pack_x_f16_q6k makes of them, bit for bit): the same thread holds the four consecutive values that are
// one 8-byte half of a 16-byte cell of that layout. Eight consecutive tokens share a 128-byte line of it, so the workgroups
// of such a run are numbered onto one XCD (workgroups go to the eight XCDs round-robin) and its L2 sees the whole line.
#pragma once
#include "common.hpp"
#include "gemv_mt.hpp"

#define NORM_BLOCK 256
#define NORM_KEEP 4   // float4 a thread keeps across the reduction on the short-row path

// IMG: 0 = no image, 12 = the Q4_K (and Q5_K) image, 14 = the Q6_K image, 112 / 114 = the images for sixteen single-term tokens
// (pack_x_mt16_q4k_f16 / pack_x_mt16_q6k_f16). With an image the grid is the image's eight (sixteen) token
// slots, the workgroups of slots at and above `tokens` write the zeros of an absent token, dim is a multiple of 256 up to
// 4096 (the short-row path), and `out` may be null (the normalised rows then exist only as the image).
// GP: 0, or the packed GEMM activations in the Q4_K / Q5_K order (12) or the Q6_K order (14) behind `image`: the grid is the
// token count rounded up to whole tiles of 128, the workgroups of absent tokens write the zeros of the last tile, dim is a
// multiple of 256 up to 4096, `out` may be null.
template <int GP>
__device__ __forceinline__ void gemm_pack_store(uint8_t* xq, u32 nkb, u32 tok, u32 kb, u32 lane, float4 o) {
  // the lane's values are k0 .. k0 + 3 of super-block kb; their cell by the inverse of gemm_k_element | gemm_k_element_q6k
  // (gemm_q4k.hpp, gemm_q6k.hpp), as in pack_x_core
  const u32 k0 = 4 * lane;
  u32 ks, kg;
  if (GP == 14) {
    ks = 8 * (k0 >> 7) + 2 * ((k0 >> 5) & 3) + ((k0 >> 3) & 1);
    kg = (k0 >> 4) & 1;
  } else {
    const u32 g = k0 >> 6;
    ks = 8 * (g >> 1) + 4 * ((k0 >> 4) & 1) + 2 * ((k0 >> 5) & 1) + ((k0 >> 3) & 1);
    kg = g & 1;
  }
  const __half2 p0 = __floats2half2_rn(o.x, o.z), p1 = __floats2half2_rn(o.y, o.w);   // slot order 0,2,1,3
  uint2 q;
  q.x = *reinterpret_cast<const u32*>(&p0);
  q.y = *reinterpret_cast<const u32*>(&p1);
  reinterpret_cast<uint2*>(xq)[((((size_t)(tok >> 7) * nkb + kb) * 4096) + (ks * 2 + kg) * 128 + (tok & 127u)) * 2 + (lane & 1u)] = q;
}

template <bool ADD, int IMG = 0, int GP = 0>
__device__ __forceinline__ void rmsnorm_core(const float* x, const float* __restrict__ add,
                                             const float* __restrict__ norm, float* residual_out,
                                             float* __restrict__ out, u32 dim, float eps, uint8_t* __restrict__ image = nullptr,
                                             u32 tokens = 0) {
  static_assert(IMG == 0 || GP == 0, "one image per launch");
  __shared__ float part[NORM_BLOCK / WAVE];
  // the row of this workgroup; with the packed GEMM activations, workgroups b, b + 8, .., b + 56 (one XCD) take tokens
  // 8 b .. 8 b + 7 of every run of 64
  const u32 row = GP ? 64u * (blockIdx.x >> 6) + 8u * (blockIdx.x & 7u) + ((blockIdx.x >> 3) & 7u) : blockIdx.x;
  if constexpr (GP != 0) {
    if (row >= tokens) {
      for (u32 i = threadIdx.x * 4; i < dim; i += NORM_BLOCK * 4)
        gemm_pack_store<GP>(image, dim >> 8, row, i >> 8, threadIdx.x & 63, make_float4(0.f, 0.f, 0.f, 0.f));
      return;
    }
  }
  // this token slot's share of the image from super-block `from` on: zeros (an absent token; the super-blocks past the
  // row's end that fill the image up to a multiple of 8)
  [[maybe_unused]] auto zero_image = [&](u32 from) {
    if constexpr (IMG != 0) {
      const u32 lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
      for (u32 sb = from + wave; sb < gemv_mt_padded_sb(dim); sb += NORM_BLOCK / WAVE) {
        if constexpr (IMG == 14) mt_pack_store_q6k(image, gemv_mt_padded_sb(dim), sb, blockIdx.x, lane, make_float4(0.f, 0.f, 0.f, 0.f), false);
        else if constexpr (IMG == 12) mt_pack_store_q4k(image, gemv_mt_padded_sb(dim), sb, blockIdx.x, lane, make_float4(0.f, 0.f, 0.f, 0.f), false);
        else if constexpr (IMG == 114) mt_pack16_store_q6k(image, gemv_mt_padded_sb(dim), sb, blockIdx.x, lane, make_float4(0.f, 0.f, 0.f, 0.f));
        else mt_pack16_store_q4k(image, gemv_mt_padded_sb(dim), sb, blockIdx.x, lane, make_float4(0.f, 0.f, 0.f, 0.f));
      }
    }
  };
  if constexpr (IMG != 0) {
    if (blockIdx.x >= tokens) {
      zero_image(0);
      return;
    }
  }
  const u64 base = (u64)row * dim;
  const float* xt = x + base;
  const float* at = ADD ? add + base : nullptr;
  float* rt = ADD ? residual_out + base : nullptr;
  float* ot = out ? out + base : nullptr;
  const float* st = ADD ? rt : xt;   // second pass: the sum this thread stored (residual_out may be x itself)
  const u32 tid = threadIdx.x;
  const bool vec = (dim & 3u) == 0;   // rows then start 16-byte aligned when the buffers do
  float ss = 0.0f;
  if (vec && dim <= NORM_BLOCK * 4 * NORM_KEEP) {
    // rows of up to 4096 values: a thread's values and norm weights stay in registers across the reduction (no second
    // read of what was just written, the weights are on their way before the barrier); same sums in the same order
    float4 v[NORM_KEEP], w[NORM_KEEP];
#pragma unroll
    for (int k = 0; k < NORM_KEEP; k++) {
      const u32 i = ((u32)k * NORM_BLOCK + tid) * 4;
      v[k] = w[k] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < dim) {
        v[k] = *reinterpret_cast<const float4*>(xt + i);
        w[k] = *reinterpret_cast<const float4*>(norm + i);
        if (ADD) {
          const float4 a = *reinterpret_cast<const float4*>(at + i);
          v[k].x += a.x, v[k].y += a.y, v[k].z += a.z, v[k].w += a.w;
          *reinterpret_cast<float4*>(rt + i) = v[k];
        }
        ss += v[k].x * v[k].x;
        ss += v[k].y * v[k].y;
        ss += v[k].z * v[k].z;
        ss += v[k].w * v[k].w;
      }
    }
    ss = wave_sum(ss);
    if ((tid & (WAVE - 1)) == 0) part[tid / WAVE] = ss;
    __syncthreads();
    const float total = (part[0] + part[1]) + (part[2] + part[3]);
    const float inv = 1.0f / sqrtf(total / (float)dim + eps);
#pragma unroll
    for (int k = 0; k < NORM_KEEP; k++) {
      const u32 i = ((u32)k * NORM_BLOCK + tid) * 4;
      if (i < dim) {
        float4 o;
        o.x = (v[k].x * inv) * w[k].x, o.y = (v[k].y * inv) * w[k].y, o.z = (v[k].z * inv) * w[k].z, o.w = (v[k].w * inv) * w[k].w;
        if ((IMG == 0 && GP == 0) || out) *reinterpret_cast<float4*>(ot + i) = o;
        if constexpr (GP != 0) gemm_pack_store<GP>(image, dim >> 8, row, 4u * (u32)k + (tid >> 6), tid & 63, o);
        if constexpr (IMG != 0) {
          // (i < dim holds for whole wavefronts: dim is a multiple of 256)
          const u32 sb = 4u * (u32)k + (tid >> 6);
          if constexpr (IMG == 14) mt_pack_store_q6k(image, gemv_mt_padded_sb(dim), sb, blockIdx.x, tid & 63, o, true);
          else if constexpr (IMG == 12) mt_pack_store_q4k(image, gemv_mt_padded_sb(dim), sb, blockIdx.x, tid & 63, o, true);
          else if constexpr (IMG == 114) mt_pack16_store_q6k(image, gemv_mt_padded_sb(dim), sb, blockIdx.x, tid & 63, o);
          else mt_pack16_store_q4k(image, gemv_mt_padded_sb(dim), sb, blockIdx.x, tid & 63, o);
        }
      }
    }
    zero_image(dim >> 8);
    return;
  }
  static_assert(IMG == 0 || IMG == 12 || IMG == 14 || IMG == 112 || IMG == 114, "image kinds");
  static_assert(GP == 0 || GP == 12 || GP == 14, "packed layouts");
  if constexpr (IMG != 0 || GP != 0) return;   // (the host launches the pack forms for the short-row shapes only)
  if (vec) {
    for (u32 i = tid * 4; i < dim; i += NORM_BLOCK * 4) {
      float4 v = *reinterpret_cast<const float4*>(xt + i);
      if (ADD) {
        const float4 a = *reinterpret_cast<const float4*>(at + i);
        v.x += a.x, v.y += a.y, v.z += a.z, v.w += a.w;
        *reinterpret_cast<float4*>(rt + i) = v;
      }
      ss += v.x * v.x;
      ss += v.y * v.y;
      ss += v.z * v.z;
      ss += v.w * v.w;
    }
  } else {
    for (u32 i = tid; i < dim; i += NORM_BLOCK) {
      float v = xt[i];
      if (ADD) {
        v += at[i];
        rt[i] = v;
      }
      ss += v * v;
    }
  }
  ss = wave_sum(ss);
  if ((tid & (WAVE - 1)) == 0) part[tid / WAVE] = ss;
  __syncthreads();
  const float total = (part[0] + part[1]) + (part[2] + part[3]);
  const float inv = 1.0f / sqrtf(total / (float)dim + eps);
  if (vec) {
    for (u32 i = tid * 4; i < dim; i += NORM_BLOCK * 4) {
      const float4 v = *reinterpret_cast<const float4*>(st + i);
      const float4 w = *reinterpret_cast<const float4*>(norm + i);
      float4 o;
      o.x = (v.x * inv) * w.x, o.y = (v.y * inv) * w.y, o.z = (v.z * inv) * w.z, o.w = (v.w * inv) * w.w;
      *reinterpret_cast<float4*>(ot + i) = o;
    }
  } else {
    for (u32 i = tid; i < dim; i += NORM_BLOCK) {
      ot[i] = (st[i] * inv) * norm[i];
    }
  }
}

// (x, norm, out, dim, eps): grid.x = tokens (rows at stride dim), block 256.
extern "C" __global__ __launch_bounds__(NORM_BLOCK) void rmsnorm_f32(const float* x, const float* norm, float* out, u32 dim,
                                                                     float eps) {
  rmsnorm_core<false>(x, nullptr, norm, nullptr, out, dim, eps);
}

// (x, add, norm, residual_out, normed_out, dim, eps): residual_out = x + add, normed_out = rmsnorm(residual_out).
// residual_out may be x itself (every element is read and written by the same thread); grid.x = tokens, block 256.
extern "C" __global__ __launch_bounds__(NORM_BLOCK) void add_rmsnorm_f32(const float* x, const float* add, const float* norm,
                                                                         float* residual_out, float* normed_out, u32 dim,
                                                                         float eps) {
  rmsnorm_core<true>(x, add, norm, residual_out, normed_out, dim, eps);
}

// The same with the normalised rows written as the activation image of the one-pass GEMV as well:
//   rmsnorm_pack_q4k_f32 | rmsnorm_pack_q6k_f32 (x, norm, out | null, image, dim, tokens, eps)
//   add_rmsnorm_pack_q4k_f32 | add_rmsnorm_pack_q6k_f32 (x, add, norm, residual_out, normed_out | null, image, dim, tokens, eps)
// grid.x = 8 (the image's token slots; x, add and the outputs hold `tokens` rows), block 256, dim a multiple of 256 up
// to 4096. The image is that of pack_x_mt_q4k_f16 | pack_x_mt_q6k_f16 on the normalised rows, bit for bit.
#define NORM_PACK_ENTRIES(SFX, IMG)                                                                                          \
  extern "C" __global__ __launch_bounds__(NORM_BLOCK) void rmsnorm_pack_##SFX##_f32(                                         \
      const float* x, const float* norm, float* out, uint8_t* image, u32 dim, u32 tokens, float eps) {                       \
    rmsnorm_core<false, IMG>(x, nullptr, norm, nullptr, out, dim, eps, image, tokens);                                       \
  }                                                                                                                          \
  extern "C" __global__ __launch_bounds__(NORM_BLOCK) void add_rmsnorm_pack_##SFX##_f32(                                     \
      const float* x, const float* add, const float* norm, float* residual_out, float* normed_out, uint8_t* image, u32 dim,  \
      u32 tokens, float eps) {                                                                                               \
    rmsnorm_core<true, IMG>(x, add, norm, residual_out, normed_out, dim, eps, image, tokens);                                \
  }
NORM_PACK_ENTRIES(q4k, 12)
NORM_PACK_ENTRIES(q6k, 14)
// the images of the sixteen-token kernels: rmsnorm_pack_x16_q4k_f32 | ..._x16_q6k_f32, add_rmsnorm_pack_x16_q4k_f32 | ..._x16_q6k_f32,
// the same parameters, grid.x = 16
NORM_PACK_ENTRIES(x16_q4k, 112)
NORM_PACK_ENTRIES(x16_q6k, 114)

// The same with the normalised rows written as the packed fp16 activations of the prefill GEMMs:
//   rmsnorm_gemm_pack_q4k_f32 | rmsnorm_gemm_pack_q6k_f32 (x, norm, out | null, xp, dim, tokens, eps)
//   add_rmsnorm_gemm_pack_q4k_f32 | add_rmsnorm_gemm_pack_q6k_f32 (x, add, norm, residual_out, normed_out | null, xp, dim, tokens, eps)
// grid.x = 128 * ceil(tokens / 128), block 256, dim a multiple of 256 up to 4096. xp is what pack_x_f16_q4k | pack_x_f16_q6k
// writes from the normalised rows, bit for bit.
#define NORM_GEMM_PACK_ENTRIES(SFX, GP)                                                                                      \
  extern "C" __global__ __launch_bounds__(NORM_BLOCK) void rmsnorm_gemm_pack_##SFX##_f32(                                    \
      const float* x, const float* norm, float* out, uint8_t* xp, u32 dim, u32 tokens, float eps) {                          \
    rmsnorm_core<false, 0, GP>(x, nullptr, norm, nullptr, out, dim, eps, xp, tokens);                                        \
  }                                                                                                                          \
  extern "C" __global__ __launch_bounds__(NORM_BLOCK) void add_rmsnorm_gemm_pack_##SFX##_f32(                                \
      const float* x, const float* add, const float* norm, float* residual_out, float* normed_out, uint8_t* xp, u32 dim,     \
      u32 tokens, float eps) {                                                                                               \
    rmsnorm_core<true, 0, GP>(x, add, norm, residual_out, normed_out, dim, eps, xp, tokens);                                 \
  }
NORM_GEMM_PACK_ENTRIES(q4k, 12)
NORM_GEMM_PACK_ENTRIES(q6k, 14)
