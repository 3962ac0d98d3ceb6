// Host stand-in for the part of hipblaslt_ext that the GEMM seam uses (test infrastructure): the "all kernels" list
// holds the one kernel of the stand-in.
#pragma once

#include <hipblaslt/hipblaslt.h>

#include <vector>

namespace hipblaslt_ext {
enum class GemmType { HIPBLASLT_GEMM = 1 };
inline hipblasStatus_t getAllAlgos(hipblasLtHandle_t, GemmType, hipblasOperation_t, hipblasOperation_t, hipDataType, hipDataType,
                                   hipDataType, hipDataType, hipblasComputeType_t,
                                   std::vector<hipblasLtMatmulHeuristicResult_t>& out) {
    hipblasLtMatmulHeuristicResult_t r;
    memset(&r, 0, sizeof r);
    out.assign(1, r);
    return HIPBLAS_STATUS_SUCCESS;
}
inline hipblasStatus_t matmulIsAlgoSupported(hipblasLtHandle_t, hipblasLtMatmulDesc_t d, const void*, hipblasLtMatrixLayout_t a,
                                             hipblasLtMatrixLayout_t b, const void*, hipblasLtMatrixLayout_t c,
                                             hipblasLtMatrixLayout_t dd, hipblasLtMatmulAlgo_t&, size_t& workspace) {
    workspace = 0;
    return emu_lt_supported(d, a, b, c, dd) ? HIPBLAS_STATUS_SUCCESS : HIPBLAS_STATUS_NOT_SUPPORTED;
}
}  // namespace hipblaslt_ext
