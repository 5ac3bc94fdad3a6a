// The gfx950 code object: every kernel is an unmangled extern "C" __global__ symbol so a host can
// fetch it by name with hipModuleGetFunction after hipModuleLoadData, the way the reference loads
// its PTX modules (src/ml/cuda/driver.cr:115-127).
#include "kernels/dequant.hpp"
#include "kernels/gemv.hpp"
#include "kernels/gemv_plain.hpp"
#include "kernels/gemv_mfma.hpp"
#include "kernels/gemv_mfma_q6k.hpp"
#include "kernels/gemv_mt.hpp"
#include "kernels/gemm_q4k.hpp"
#include "kernels/gemm_q4k_wide.hpp"
#include "kernels/gemm_q6k.hpp"
#include "kernels/norm.hpp"

GEMV_MFMA_ENTRY(q4_k_gemv_mfma_f32_tbatch2, 2)
GEMV_MFMA_ENTRY(q4_k_gemv_mfma_f32_tbatch3, 3)
GEMV_MFMA_ENTRY(q4_k_gemv_mfma_f32_tbatch4, 4)
GEMV_MFMA_ADD_ENTRY(q4_k_gemv_mfma_add_f32_tbatch2, 2)
GEMV_MFMA_ADD_ENTRY(q4_k_gemv_mfma_add_f32_tbatch3, 3)
GEMV_MFMA_ADD_ENTRY(q4_k_gemv_mfma_add_f32_tbatch4, 4)
GEMV_MFMA_Q6K_ENTRY(q6_k_gemv_mfma_f32_tbatch3, 3)
GEMV_MFMA_Q6K_ENTRY(q6_k_gemv_mfma_f32_tbatch4, 4)
GEMV_MFMA_Q6K_ADD_ENTRY(q6_k_gemv_mfma_add_f32_tbatch3, 3)
GEMV_MFMA_Q6K_ADD_ENTRY(q6_k_gemv_mfma_add_f32_tbatch4, 4)
GEMV_MFMA_TOP1_ENTRY(q4_k_gemv_mfma_top1_partial_f32_tbatch3, 3)
GEMV_MFMA_TOP1_ENTRY(q4_k_gemv_mfma_top1_partial_f32_tbatch4, 4)
GEMV_MFMA_Q6K_TOP1_ENTRY(q6_k_gemv_mfma_top1_partial_f32_tbatch3, 3)
GEMV_MFMA_Q6K_TOP1_ENTRY(q6_k_gemv_mfma_top1_partial_f32_tbatch4, 4)
GEMV_MFMA_DUAL_ENTRY(q4_k_dual_gemv_mfma_f32_tbatch2, 2)
GEMV_MFMA_DUAL_ENTRY(q4_k_dual_gemv_mfma_f32_tbatch3, 3)
GEMV_MFMA_DUAL_ENTRY(q4_k_dual_gemv_mfma_f32_tbatch4, 4)
GEMV_MFMA_MANY_ENTRY(q4_k_many_gemv_mfma_f32_tbatch2, 2)
GEMV_MFMA_MANY_ENTRY(q4_k_many_gemv_mfma_f32_tbatch3, 3)
GEMV_MFMA_MANY_ENTRY(q4_k_many_gemv_mfma_f32_tbatch4, 4)
GEMV_MFMA_SWIGLU_ENTRY(q4_k_dual_gemv_swiglu_mfma_f32_tbatch2, 2)
GEMV_MFMA_SWIGLU_ENTRY(q4_k_dual_gemv_swiglu_mfma_f32_tbatch3, 3)
GEMV_MFMA_SWIGLU_ENTRY(q4_k_dual_gemv_swiglu_mfma_f32_tbatch4, 4)
GEMV_MFMA_Q5K_ENTRY(q5_k_gemv_mfma_f32_tbatch3, 3)
GEMV_MFMA_Q5K_ENTRY(q5_k_gemv_mfma_f32_tbatch4, 4)
GEMV_MFMA_Q5K_ADD_ENTRY(q5_k_gemv_mfma_add_f32_tbatch3, 3)
GEMV_MFMA_Q5K_ADD_ENTRY(q5_k_gemv_mfma_add_f32_tbatch4, 4)
