// Instantiates the tiled GEMM template: int8 kernels (dequant and dequant + SwiGLU epilogues), B stored [K, N].
#include "gemm_tile_kernel.h"

namespace cch {
template int launch_tile_t<KIND_I8, EPI_DEQUANT, 0, 0>(const GemmProblem &, hipStream_t);
template int launch_tile_t<KIND_I8, EPI_DEQUANT_SWIGLU, 0, 0>(const GemmProblem &, hipStream_t);
}  // namespace cch
