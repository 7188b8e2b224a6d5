// One instantiation of the grouped-GEMM kernel and its launcher: compiled once per entry of
// FP8GMM_FOR_EACH_GEMM_VARIANT with -DFP8GMM_VARIANT_INDEX=0..6 (see the Makefile), so that the variants build in
// parallel.
#ifndef FP8GMM_VARIANT_INDEX
#error "compile with -DFP8GMM_VARIANT_INDEX=<0..6>"
#endif
#include "grouped_gemm_kernel.h"

namespace fp8gmm {

#define FP8GMM_CAT_(a, b) a##b
#define FP8GMM_CAT(a, b) FP8GMM_CAT_(a, b)
#define FP8GMM_INSTANTIATE(AF, BF, AT, BT)                                                                     \
  template int prepare_variant<AF, BF, AT, BT>(int);                                                           \
  template int launch_variant<AF, BF, AT, BT>(const fp8gmm_gemm_problem*, const fp8gmm_gemm_item*, int, int, int, \
                                              uint8_t*, uint64_t*, hipStream_t);

#define FP8GMM_V0 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, false, false)
#define FP8GMM_V1 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, false, false)
#define FP8GMM_V2 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E5M2, false, false)
#define FP8GMM_V3 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, false, true)
#define FP8GMM_V4 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, false, true)
#define FP8GMM_V5 FP8GMM_INSTANTIATE(FP8GMM_E4M3, FP8GMM_E4M3, true, true)
#define FP8GMM_V6 FP8GMM_INSTANTIATE(FP8GMM_E5M2, FP8GMM_E4M3, true, true)

FP8GMM_CAT(FP8GMM_V, FP8GMM_VARIANT_INDEX)

}  // namespace fp8gmm
