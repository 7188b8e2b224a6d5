// Work decomposition constants shared by the host planners and the kernels.
#pragma once

namespace fp8gmm {

// ---- element-wise kernels (quantize, scale_mul) ----
constexpr int kPwThreads = 256;                  // 4 wavefronts
constexpr int kPwVec = 8;                        // elements per thread per step (one 16-byte bf16 load)
constexpr int kPwSteps = 8;                      // steps per workgroup
constexpr int kPwBlockElems = kPwThreads * kPwVec * kPwSteps;  // 16384 elements per workgroup

// ---- pad / cast / transpose kernels ----
constexpr int kPtThreads = 256;
constexpr int kPtTileRows = 128;                 // tile extent along the token (row) dimension
constexpr int kPtTileCols = 128;                 // tile extent along the feature (column) dimension

// ---- grouped GEMM ----
constexpr int kGemmTileM = 256;                  // rows of c per workgroup tile
constexpr int kGemmTileN = 256;                  // columns of c per workgroup tile
constexpr int kGemmTileK = 128;                  // bytes of K consumed per main-loop step
constexpr int BM = kGemmTileM;
constexpr int BN = kGemmTileN;
constexpr int kNumXcd = 8;                       // workgroup i of a launch runs on XCD i % 8

}  // namespace fp8gmm
