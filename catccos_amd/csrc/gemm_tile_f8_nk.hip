// Instantiates the tiled GEMM template: MXFP8 kernels (E4M3 and E5M2 payload, plain epilogue), B stored [N, K].
#include "gemm_tile_kernel.h"

namespace cch {
template int launch_tile_t<KIND_F8, EPI_PLAIN, CCH_FMT_E4M3, 1>(const GemmProblem &, hipStream_t);
template int launch_tile_t<KIND_F8, EPI_PLAIN, CCH_FMT_E5M2, 1>(const GemmProblem &, hipStream_t);
}  // namespace cch
