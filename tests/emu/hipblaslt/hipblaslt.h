// Host stand-in for the part of hipBLASLt that the GEMM seam uses (test infrastructure): column-major
// D = act(alpha op(A) op(B) + beta C + bias), bias one value per row of D, fp32 accumulation, fp32 or bf16 operands
// and result.  One kernel "candidate" per problem; the Swish epilogue takes its slope argument.
#pragma once

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <vector>

typedef enum { HIPBLAS_STATUS_SUCCESS = 0, HIPBLAS_STATUS_INVALID_VALUE = 3, HIPBLAS_STATUS_NOT_SUPPORTED = 7 } hipblasStatus_t;
typedef enum { HIP_R_32F = 0, HIP_R_16BF = 14 } hipDataType;
typedef enum { HIPBLAS_COMPUTE_32F = 2 } hipblasComputeType_t;
typedef enum { HIPBLAS_OP_N = 111, HIPBLAS_OP_T = 112 } hipblasOperation_t;
typedef enum {
    HIPBLASLT_EPILOGUE_DEFAULT = 1,
    HIPBLASLT_EPILOGUE_BIAS = 4,
    HIPBLASLT_EPILOGUE_SWISH_BIAS_EXT = 65540
} hipblasLtEpilogue_t;
typedef enum {
    HIPBLASLT_MATMUL_DESC_TRANSA = 0,
    HIPBLASLT_MATMUL_DESC_TRANSB,
    HIPBLASLT_MATMUL_DESC_EPILOGUE,
    HIPBLASLT_MATMUL_DESC_BIAS_POINTER,
    HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE,
    HIPBLASLT_MATMUL_DESC_EPILOGUE_ACT_ARG0_EXT
} hipblasLtMatmulDescAttributes_t;
typedef enum { HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES = 1 } hipblasLtMatmulPreferenceAttributes_t;

struct emu_lt_desc {
    hipblasOperation_t transa = HIPBLAS_OP_N, transb = HIPBLAS_OP_N;
    hipblasLtEpilogue_t epilogue = HIPBLASLT_EPILOGUE_DEFAULT;
    const void* bias = nullptr;
    hipDataType bias_type = HIP_R_32F;
    float act_arg0 = 1.0f;
};
struct emu_lt_layout {
    hipDataType type;
    uint64_t rows, cols;
    int64_t ld;
};
struct emu_lt_pref {
    uint64_t max_workspace = 0;
};
typedef void* hipblasLtHandle_t;
typedef emu_lt_desc* hipblasLtMatmulDesc_t;
typedef emu_lt_layout* hipblasLtMatrixLayout_t;
typedef emu_lt_pref* hipblasLtMatmulPreference_t;
struct hipblasLtMatmulAlgo_t {
    uint8_t data[16];
    size_t max_workspace_bytes;
};
struct hipblasLtMatmulHeuristicResult_t {
    hipblasLtMatmulAlgo_t algo;
    size_t workspaceSize;
    hipblasStatus_t state;
    float wavesCount;
    int reserved[4];
};

inline hipblasStatus_t hipblasLtCreate(hipblasLtHandle_t* h) { *h = (void*)1; return HIPBLAS_STATUS_SUCCESS; }
inline hipblasStatus_t hipblasLtDestroy(hipblasLtHandle_t) { return HIPBLAS_STATUS_SUCCESS; }
inline hipblasStatus_t hipblasLtMatmulDescCreate(hipblasLtMatmulDesc_t* d, hipblasComputeType_t, hipDataType scale_type) {
    if (scale_type != HIP_R_32F) return HIPBLAS_STATUS_NOT_SUPPORTED;
    *d = new emu_lt_desc;
    return HIPBLAS_STATUS_SUCCESS;
}
inline hipblasStatus_t hipblasLtMatmulDescDestroy(hipblasLtMatmulDesc_t d) { delete d; return HIPBLAS_STATUS_SUCCESS; }
inline hipblasStatus_t hipblasLtMatmulDescSetAttribute(hipblasLtMatmulDesc_t d, hipblasLtMatmulDescAttributes_t attr,
                                                       const void* value, size_t bytes) {
    if (!d || !value) return HIPBLAS_STATUS_INVALID_VALUE;
    switch (attr) {
    case HIPBLASLT_MATMUL_DESC_TRANSA: if (bytes != sizeof(d->transa)) return HIPBLAS_STATUS_INVALID_VALUE; memcpy(&d->transa, value, bytes); break;
    case HIPBLASLT_MATMUL_DESC_TRANSB: if (bytes != sizeof(d->transb)) return HIPBLAS_STATUS_INVALID_VALUE; memcpy(&d->transb, value, bytes); break;
    case HIPBLASLT_MATMUL_DESC_EPILOGUE: if (bytes != sizeof(d->epilogue)) return HIPBLAS_STATUS_INVALID_VALUE; memcpy(&d->epilogue, value, bytes); break;
    case HIPBLASLT_MATMUL_DESC_BIAS_POINTER: if (bytes != sizeof(void*)) return HIPBLAS_STATUS_INVALID_VALUE; memcpy(&d->bias, value, bytes); break;
    case HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE: if (bytes != sizeof(d->bias_type)) return HIPBLAS_STATUS_INVALID_VALUE; memcpy(&d->bias_type, value, bytes); break;
    case HIPBLASLT_MATMUL_DESC_EPILOGUE_ACT_ARG0_EXT: if (bytes != sizeof(float)) return HIPBLAS_STATUS_INVALID_VALUE; memcpy(&d->act_arg0, value, bytes); break;
    default: return HIPBLAS_STATUS_NOT_SUPPORTED;
    }
    return HIPBLAS_STATUS_SUCCESS;
}
inline hipblasStatus_t hipblasLtMatrixLayoutCreate(hipblasLtMatrixLayout_t* l, hipDataType type, uint64_t rows, uint64_t cols,
                                                   int64_t ld) {
    if (ld < (int64_t)rows) return HIPBLAS_STATUS_INVALID_VALUE;
    *l = new emu_lt_layout{type, rows, cols, ld};
    return HIPBLAS_STATUS_SUCCESS;
}
inline hipblasStatus_t hipblasLtMatrixLayoutDestroy(hipblasLtMatrixLayout_t l) { delete l; return HIPBLAS_STATUS_SUCCESS; }
inline hipblasStatus_t hipblasLtMatmulPreferenceCreate(hipblasLtMatmulPreference_t* p) { *p = new emu_lt_pref; return HIPBLAS_STATUS_SUCCESS; }
inline hipblasStatus_t hipblasLtMatmulPreferenceDestroy(hipblasLtMatmulPreference_t p) { delete p; return HIPBLAS_STATUS_SUCCESS; }
inline hipblasStatus_t hipblasLtMatmulPreferenceSetAttribute(hipblasLtMatmulPreference_t p, hipblasLtMatmulPreferenceAttributes_t,
                                                             const void* value, size_t bytes) {
    if (bytes != sizeof(uint64_t)) return HIPBLAS_STATUS_INVALID_VALUE;
    memcpy(&p->max_workspace, value, bytes);
    return HIPBLAS_STATUS_SUCCESS;
}

inline bool emu_lt_supported(const emu_lt_desc* d, const emu_lt_layout* a, const emu_lt_layout* b, const emu_lt_layout* c,
                             const emu_lt_layout* dd) {
    if (d->transa != HIPBLAS_OP_N || d->transb != HIPBLAS_OP_N || d->bias_type != HIP_R_32F) return false;
    if (a->cols != b->rows || a->rows != dd->rows || b->cols != dd->cols || c->rows != dd->rows || c->cols != dd->cols) return false;
    if (a->type != b->type) return false;
    if (d->epilogue != HIPBLASLT_EPILOGUE_DEFAULT && d->bias == nullptr) return false;
    return true;
}
inline hipblasStatus_t hipblasLtMatmulAlgoGetHeuristic(hipblasLtHandle_t, hipblasLtMatmulDesc_t d, hipblasLtMatrixLayout_t a,
                                                       hipblasLtMatrixLayout_t b, hipblasLtMatrixLayout_t c,
                                                       hipblasLtMatrixLayout_t dd, hipblasLtMatmulPreference_t,
                                                       int requested, hipblasLtMatmulHeuristicResult_t* results, int* found) {
    *found = 0;
    if (requested < 1 || !emu_lt_supported(d, a, b, c, dd)) return HIPBLAS_STATUS_SUCCESS;
    memset(&results[0], 0, sizeof(results[0]));
    results[0].state = HIPBLAS_STATUS_SUCCESS;
    *found = 1;
    return HIPBLAS_STATUS_SUCCESS;
}

inline float emu_lt_load(const void* p, hipDataType type, size_t i) {
    if (type == HIP_R_32F) return ((const float*)p)[i];
    return __builtin_bit_cast(float, (uint32_t)((const uint16_t*)p)[i] << 16);
}
inline void emu_lt_store(void* p, hipDataType type, size_t i, float v) {
    if (type == HIP_R_32F) {
        ((float*)p)[i] = v;
        return;
    }
    uint32_t bits = __builtin_bit_cast(uint32_t, v);
    if ((bits & 0x7fffffffu) > 0x7f800000u) bits |= 0x00400000u;           // NaN stays NaN
    else bits += 0x7fffu + ((bits >> 16) & 1u);                             // round to nearest even
    ((uint16_t*)p)[i] = (uint16_t)(bits >> 16);
}
inline hipblasStatus_t hipblasLtMatmul(hipblasLtHandle_t, hipblasLtMatmulDesc_t d, const void* alpha, const void* A,
                                       hipblasLtMatrixLayout_t a, const void* B, hipblasLtMatrixLayout_t b, const void* beta,
                                       const void* C, hipblasLtMatrixLayout_t c, void* D, hipblasLtMatrixLayout_t dd,
                                       const hipblasLtMatmulAlgo_t*, void*, size_t, hipStream_t) {
    if (!emu_lt_supported(d, a, b, c, dd)) return HIPBLAS_STATUS_NOT_SUPPORTED;
    const float al = *(const float*)alpha, be = *(const float*)beta;
    const size_t M = a->rows, N = b->cols, K = a->cols;
    std::vector<float> column(M);
    for (size_t j = 0; j < N; ++j) {
        for (size_t i = 0; i < M; ++i) column[i] = 0.f;
        for (size_t l = 0; l < K; ++l) {
            const float x = emu_lt_load(B, b->type, j * b->ld + l);
            if (a->type == HIP_R_32F) {
                const float* col = (const float*)A + l * a->ld;
                for (size_t i = 0; i < M; ++i) column[i] += col[i] * x;
            } else {
                const uint16_t* col = (const uint16_t*)A + l * a->ld;
                for (size_t i = 0; i < M; ++i) column[i] += __builtin_bit_cast(float, (uint32_t)col[i] << 16) * x;
            }
        }
        for (size_t i = 0; i < M; ++i) {
            float v = al * column[i];
            if (be != 0.f) v += be * emu_lt_load(C, c->type, j * c->ld + i);
            if (d->epilogue != HIPBLASLT_EPILOGUE_DEFAULT) v += ((const float*)d->bias)[i];
            if (d->epilogue == HIPBLASLT_EPILOGUE_SWISH_BIAS_EXT) v = v / (1.0f + expf(-d->act_arg0 * v));
            emu_lt_store(D, dd->type, j * dd->ld + i, v);
        }
    }
    return HIPBLAS_STATUS_SUCCESS;
}
