// Tile shape of the tiled MFMA GEMM kernels (shared by the kernel template and the host-side checks).
#pragma once

namespace cch {

constexpr int BM = 256, BN = 256;        // output tile
constexpr int BKB = 128;                 // bytes of K per step (per row) = one L2 line

}  // namespace cch
