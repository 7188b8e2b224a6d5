// One instantiation of the grouped-GEMM kernel and its launcher: compiled once per entry of
// FP8GMM_FOR_EACH_GEMM_VARIANT with -DFP8GMM_VARIANT_INDEX=0..20 (see the Makefile), so that the variants build in
// parallel.  0..6: the 256 x 256 tile, 7..13: the same operand formats and layouts with the 128 x 128 tile, 14..20:
// with the 128 x 256 tile and two sets of accumulators.
#ifndef FP8GMM_VARIANT_INDEX
#error "compile with -DFP8GMM_VARIANT_INDEX=<0..20>"
#endif
#include "grouped_gemm_kernel.h"

namespace fp8gmm {

#define FP8GMM_CAT_(a, b) a##b
#define FP8GMM_CAT(a, b) FP8GMM_CAT_(a, b)
#define FP8GMM_INSTANTIATE(AF, BF, AT, BT, TL)                                                                     \
  template int prepare_variant<AF, BF, AT, BT, TL>(int);                                                           \
  template int launch_variant<AF, BF, AT, BT, TL>(const fp8gmm_gemm_problem*, const fp8gmm_gemm_item*, int, int, int, \
                                                  uint8_t*, const fp8gmm_tensor_desc*, int, hipStream_t);

#define FP8GMM_V0 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, false, false, 256)
#define FP8GMM_V1 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, false, false, 256)
#define FP8GMM_V2 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E5M2, false, false, 256)
#define FP8GMM_V3 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, false, true, 256)
#define FP8GMM_V4 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, false, true, 256)
#define FP8GMM_V5 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, true, true, 256)
#define FP8GMM_V6 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, true, true, 256)
#define FP8GMM_V7 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, false, false, 128)
#define FP8GMM_V8 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, false, false, 128)
#define FP8GMM_V9 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E5M2, false, false, 128)
#define FP8GMM_V10 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, false, true, 128)
#define FP8GMM_V11 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, false, true, 128)
#define FP8GMM_V12 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, true, true, 128)
#define FP8GMM_V13 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, true, true, 128)
#define FP8GMM_V14 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, false, false, kTileDual)
#define FP8GMM_V15 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, false, false, kTileDual)
#define FP8GMM_V16 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E5M2, false, false, kTileDual)
#define FP8GMM_V17 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, false, true, kTileDual)
#define FP8GMM_V18 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, false, true, kTileDual)
#define FP8GMM_V19 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, true, true, kTileDual)
#define FP8GMM_V20 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, true, true, kTileDual)

FP8GMM_CAT(FP8GMM_V, FP8GMM_VARIANT_INDEX)

}  // namespace fp8gmm
