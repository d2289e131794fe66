// Instantiates the tiled GEMM template: MXFP4 kernels (plain and SwiGLU epilogues), B stored [K, N].
#include "gemm_tile_kernel.h"

namespace cch {
template int launch_tile_t<KIND_F4, EPI_PLAIN, CCH_FMT_E2M1, 0>(const GemmProblem &, hipStream_t);
template int launch_tile_t<KIND_F4, EPI_SWIGLU, CCH_FMT_E2M1, 0>(const GemmProblem &, hipStream_t);
}  // namespace cch
