// Host stand-in for the part of rocBLAS that the GEMM seam uses (test infrastructure): column-major
// D = alpha op(A) op(B) + beta C with fp32 or bf16 operands and fp32 result.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <vector>

typedef void* rocblas_handle;
typedef enum { rocblas_status_success = 0, rocblas_status_not_implemented = 2 } rocblas_status;
typedef enum { rocblas_operation_none = 111, rocblas_operation_transpose = 112 } rocblas_operation;
typedef enum { rocblas_datatype_f32_r = 151, rocblas_datatype_bf16_r = 168 } rocblas_datatype;
typedef enum { rocblas_gemm_algo_standard = 0 } rocblas_gemm_algo;

inline rocblas_status rocblas_create_handle(rocblas_handle* h) { *h = (void*)1; return rocblas_status_success; }
inline rocblas_status rocblas_destroy_handle(rocblas_handle) { return rocblas_status_success; }
inline rocblas_status rocblas_set_stream(rocblas_handle, hipStream_t) { return rocblas_status_success; }

inline float emu_blas_load(const void* p, rocblas_datatype type, size_t i) {
    if (type == rocblas_datatype_f32_r) return ((const float*)p)[i];
    return __builtin_bit_cast(float, (uint32_t)((const uint16_t*)p)[i] << 16);
}
inline rocblas_status rocblas_gemm_ex(rocblas_handle, rocblas_operation ta, rocblas_operation tb, int m, int n, int k,
                                      const void* alpha, const void* a, rocblas_datatype a_type, int lda, const void* b,
                                      rocblas_datatype b_type, int ldb, const void* beta, const void* c, rocblas_datatype c_type,
                                      int ldc, void* d, rocblas_datatype d_type, int ldd, rocblas_datatype compute_type,
                                      rocblas_gemm_algo, int32_t, uint32_t) {
    if (c_type != rocblas_datatype_f32_r || d_type != rocblas_datatype_f32_r || compute_type != rocblas_datatype_f32_r)
        return rocblas_status_not_implemented;
    const float al = *(const float*)alpha, be = *(const float*)beta;
    std::vector<float> column((size_t)m);
    for (int j = 0; j < n; ++j) {
        for (int i = 0; i < m; ++i) column[i] = 0.f;
        for (int l = 0; l < k; ++l) {
            const float x = tb == rocblas_operation_none ? emu_blas_load(b, b_type, (size_t)j * ldb + l)
                                                         : emu_blas_load(b, b_type, (size_t)l * ldb + j);
            for (int i = 0; i < m; ++i)
                column[i] += (ta == rocblas_operation_none ? emu_blas_load(a, a_type, (size_t)l * lda + i)
                                                           : emu_blas_load(a, a_type, (size_t)i * lda + l)) * x;
        }
        for (int i = 0; i < m; ++i) {
            float v = al * column[i];
            if (be != 0.f) v += be * ((const float*)c)[(size_t)j * ldc + i];
            ((float*)d)[(size_t)j * ldd + i] = v;
        }
    }
    return rocblas_status_success;
}
