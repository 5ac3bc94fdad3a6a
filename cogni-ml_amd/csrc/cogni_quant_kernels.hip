// The gfx950 code object: every kernel is an unmangled extern "C" __global__ symbol so a host can
// fetch it by name with hipModuleGetFunction after hipModuleLoadData, the way the reference loads
// its PTX modules (src/ml/cuda/driver.cr:115-127).
#include "kernels/dequant.cuh"
#include "kernels/gemv.cuh"
#include "kernels/gemm_q4k.cuh"
#include "kernels/util.cuh"
