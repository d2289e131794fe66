// Instantiates the tiled GEMM template: int8 kernels (dequant and dequant + SwiGLU epilogues), B stored [N, K].
#include "gemm_tile_kernel.h"

namespace cch {
template int launch_tile_t<KIND_I8, EPI_DEQUANT, 0, 1>(const GemmProblem &, hipStream_t);
template int launch_tile_t<KIND_I8, EPI_DEQUANT_SWIGLU, 0, 1>(const GemmProblem &, hipStream_t);
}  // namespace cch
