// Dense GEMM seam (rocBLAS) and the forward pass of one BERT encoder layer with block-sparse
// attention inside.  Op order is that of the reference's CPU layer (transformer.cpp:513-580: GEMM,
// bias, attention, out-projection, bias, residual, LayerNorm, FFN GEMM, bias, GELU, GEMM, bias,
// residual) arranged post-LN and without dropout:
//     x1 = LN1(x + Attn(x Wq + bq, x Wk + bk, x Wv + bv) Wo + bo)
//     y  = LN2(x1 + gelu(x1 W1 + b1) W2 + b2)
// Weights are [in][out] row-major as in the reference (cblas_sgemm(RowMajor, N, N, m, n, k, A, k, W, n,
// C, n), transformer.cpp:516); the GEMM is issued column-major as C^T = W^T A^T, the same trick as the
// reference's cuBLAS calls (transformer_attention_optimize.cu:693-716).
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt-ext.hpp>
#include <hipblaslt/hipblaslt.h>
#include <rocblas/rocblas.h>

#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "../../include/sfbert_hip.h"

namespace {

std::mutex g_mutex;
rocblas_handle g_handle = nullptr;

rocblas_handle blas_handle() {
    if (!g_handle) {
        if (rocblas_create_handle(&g_handle) != rocblas_status_success) g_handle = nullptr;
    }
    return g_handle;
}

inline size_t align256(size_t n) { return (n + 255) / 256 * 256; }
constexpr size_t kGemmWorkspaceBytes = 32u << 20;

// GEMM with, optionally, the bias add, the activation and the output conversion in its epilogue (hipBLASLt).  One
// plan per problem (shape, element types, epilogue, whether a workspace is on offer), made on first use and kept
// until sfb_gemm_release().  Making a plan asks the library for up to kCandidates kernels that fit the offered
// workspace and -- unless the stream is being captured into a graph -- times each of them once on the caller's own
// operands (the products all write the same result) and keeps the fastest; under capture the library's first
// choice is taken.  The activation is the reference's sigmoid form of GELU, x / (1 + exp(-1.702 x))
// (ewops.h:32-43), which is the library's Swish epilogue with its argument set to 1.702.
struct LtPlan {
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t w = nullptr, a = nullptr, c = nullptr;
    hipblasLtMatmulAlgo_t algo;
    size_t workspace = 0;     // bytes the chosen kernel wants
    bool usable = false;
    bool slope_set = false;   // activation plans: the library took the GELU slope as the Swish argument
    bool tuned = false;       // candidates were timed (false: first choice taken under graph capture)
};
hipblasLtHandle_t g_lt = nullptr;
typedef std::tuple<uint32_t, uint32_t, uint32_t, int, int, int, int, int> PlanKey;
std::map<PlanKey, LtPlan> g_plans;
constexpr float kGeluSigmoidSlope = 1.702f;
constexpr int kCandidates = 16;
// sfb_gemm_tuning(): 0 = time the library's own short list of candidates, 1 = time every kernel of the library that
// supports the problem (the short list is what a heuristic expects to be fast; at the layer's shapes its best entry
// runs at about a third of the matrix peak, so the long list is worth a second or two per problem at first use)
int g_tuning_level = 0;
constexpr size_t kMostCandidates = 1024;

void destroy_plan(LtPlan& p) {
    if (p.w) hipblasLtMatrixLayoutDestroy(p.w);
    if (p.a) hipblasLtMatrixLayoutDestroy(p.a);
    if (p.c) hipblasLtMatrixLayoutDestroy(p.c);
    if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
    p = LtPlan();
}

bool stream_is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) { (void)hipGetLastError(); return true; }
    return status != hipStreamCaptureStatusNone;
}

// Operands of the call that makes a plan: the candidates are timed on them.
struct LtOperands {
    hipStream_t stream;
    void* c;
    const void* a;
    const void* w;
    const float* bias;
    void* workspace;
    size_t workspace_bytes;
};

// row-major C[m][n] = A[m][k] W[k][n] (+ bias[n])  ==  column-major D[n][m] = W'[n][k] A'[k][m] (+ bias per row of D)
// act: 0 none, 1 sigmoid-GELU (needs a bias); epilogue without bias when ops.bias is null
LtPlan& lt_plan(uint32_t m, uint32_t n, uint32_t k, int dtype, int out_dtype, int act, const LtOperands& ops) {
    const int with_bias = ops.bias != nullptr, with_ws = ops.workspace != nullptr && ops.workspace_bytes > 0;
    const PlanKey key = std::make_tuple(m, n, k, dtype, out_dtype, act, with_bias, with_ws);
    auto it = g_plans.find(key);
    if (it != g_plans.end()) return it->second;
    LtPlan& p = g_plans[key];
    if (!g_lt && hipblasLtCreate(&g_lt) != HIPBLAS_STATUS_SUCCESS) { g_lt = nullptr; return p; }
    if (act && !with_bias) return p;
    const hipDataType in = dtype == SFB_BF16 ? HIP_R_16BF : HIP_R_32F;
    const hipDataType out = out_dtype == SFB_BF16 ? HIP_R_16BF : HIP_R_32F;
    const hipblasOperation_t none = HIPBLAS_OP_N;
    const hipblasLtEpilogue_t epilogue = act ? HIPBLASLT_EPILOGUE_SWISH_BIAS_EXT
                                             : (with_bias ? HIPBLASLT_EPILOGUE_BIAS : HIPBLASLT_EPILOGUE_DEFAULT);
    const hipDataType bias_type = HIP_R_32F;
    bool ok = hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &none, sizeof(none)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &none, sizeof(none)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue)) == HIPBLAS_STATUS_SUCCESS;
    if (with_bias)
        ok = ok && hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type)) == HIPBLAS_STATUS_SUCCESS;
    // older builds of the library have the Swish epilogue but not its slope argument: there the slope stays 1 and
    // the caller scales the operands instead (see gemm_bias_gelu_scaled)
    if (ok && act)
        p.slope_set = hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE_ACT_ARG0_EXT, &kGeluSigmoidSlope,
                                                      sizeof(kGeluSigmoidSlope)) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.w, in, n, k, n) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.a, in, k, m, k) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipblasLtMatrixLayoutCreate(&p.c, out, n, m, n) == HIPBLAS_STATUS_SUCCESS;
    if (!ok) return p;
    // the heuristic needs the bias pointer to be present in the descriptor; it is set again on every call
    if (with_bias) {
        const void* bias_ptr = ops.bias;
        hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias_ptr, sizeof(bias_ptr));
    }
    hipblasLtMatmulPreference_t pref = nullptr;
    if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return p;
    const uint64_t max_ws = with_ws ? ops.workspace_bytes : 0;
    hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws, sizeof(max_ws));
    std::vector<hipblasLtMatmulHeuristicResult_t> results(kCandidates);
    int found = 0;
    const bool got = hipblasLtMatmulAlgoGetHeuristic(g_lt, p.desc, p.w, p.a, p.c, p.c, pref, kCandidates, results.data(),
                                                     &found) == HIPBLAS_STATUS_SUCCESS;
    hipblasLtMatmulPreferenceDestroy(pref);
    if (!got || found <= 0) return p;
    results.resize((size_t)found);
    const bool can_time = !stream_is_capturing(ops.stream) && ops.c && ops.a && ops.w;
    if (g_tuning_level >= 1 && can_time) {
        // every kernel the library has for these types, kept if it supports this problem within the workspace
        std::vector<hipblasLtMatmulHeuristicResult_t> all;
        if (hipblaslt_ext::getAllAlgos(g_lt, hipblaslt_ext::GemmType::HIPBLASLT_GEMM, none, none, in, in, out, out,
                                       HIPBLAS_COMPUTE_32F, all) == HIPBLAS_STATUS_SUCCESS) {
            const float one = 1.0f, zero = 0.0f;
            for (auto& r : all) {
                if (results.size() >= kMostCandidates) break;
                size_t need = 0;
                if (hipblaslt_ext::matmulIsAlgoSupported(g_lt, p.desc, &one, p.w, p.a, &zero, p.c, p.c, r.algo, need) !=
                        HIPBLAS_STATUS_SUCCESS || need > max_ws)
                    continue;
                r.workspaceSize = need;
                r.state = HIPBLAS_STATUS_SUCCESS;
                results.push_back(r);
            }
        }
        found = (int)results.size();
    }
    int best = -1;
    if (can_time) {
        // time every candidate on the caller's operands: 1 untimed + 3 timed launches each
        hipEvent_t e0 = nullptr, e1 = nullptr;
        if (hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess) {
            const float alpha = 1.0f, beta = 0.0f;
            float best_ms = 0.f;
            for (int i = 0; i < found; ++i) {
                if (results[i].state != HIPBLAS_STATUS_SUCCESS || results[i].workspaceSize > max_ws) continue;
                bool ran = true;
                for (int rep = 0; rep < 4 && ran; ++rep) {
                    if (rep == 1) ran = hipEventRecord(e0, ops.stream) == hipSuccess;
                    ran = ran && hipblasLtMatmul(g_lt, p.desc, &alpha, ops.w, p.w, ops.a, p.a, &beta, ops.c, p.c, ops.c, p.c,
                                                 &results[i].algo, ops.workspace, results[i].workspaceSize,
                                                 ops.stream) == HIPBLAS_STATUS_SUCCESS;
                }
                float ms = 0.f;
                ran = ran && hipEventRecord(e1, ops.stream) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
                      hipEventElapsedTime(&ms, e0, e1) == hipSuccess;
                if (!ran) { (void)hipGetLastError(); continue; }
                if (best < 0 || ms < best_ms) { best = i; best_ms = ms; }
            }
            p.tuned = best >= 0;
        }
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
    }
    if (best < 0)
        for (int i = 0; i < found && best < 0; ++i)
            if (results[i].state == HIPBLAS_STATUS_SUCCESS && results[i].workspaceSize <= max_ws) best = i;
    if (best < 0) return p;
    p.algo = results[best].algo;
    p.workspace = results[best].workspaceSize;
    p.usable = true;
    return p;
}

}  // namespace

// c = alpha (a w), rocBLAS
static int gemm_alpha(sfb_stream_t stream, float* c, const void* a, const void* w, int dtype, uint32_t m, uint32_t n,
                      uint32_t k, float alpha) {
    if (!c || !a || !w) return SFB_ERR_NULL_POINTER;
    if (dtype != SFB_F32 && dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (!m || !n || !k) return SFB_ERR_SHAPE;
    std::lock_guard<std::mutex> lock(g_mutex);
    rocblas_handle h = blas_handle();
    if (!h) return SFB_ERR_LAUNCH;
    if (rocblas_set_stream(h, (hipStream_t)stream) != rocblas_status_success) return SFB_ERR_LAUNCH;
    const float beta = 0.0f;
    const rocblas_datatype in = dtype == SFB_BF16 ? rocblas_datatype_bf16_r : rocblas_datatype_f32_r;
    // row-major C[m][n] = A[m][k] W[k][n]  ==  column-major C^T[n][m] = W^T[n][k] A^T[k][m]
    const rocblas_status st = rocblas_gemm_ex(h, rocblas_operation_none, rocblas_operation_none, (int)n, (int)m,
                                              (int)k, &alpha, w, in, (int)n, a, in, (int)k, &beta, c,
                                              rocblas_datatype_f32_r, (int)n, c, rocblas_datatype_f32_r, (int)n,
                                              rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
    return st == rocblas_status_success ? SFB_OK : SFB_ERR_LAUNCH;
}

// C = act(alpha A W (+ bias)) through one library GEMM; SFB_ERR_LAUNCH when the library has no kernel for it.
// act = 1 without the slope argument (*slope_set false) computes Swish with slope 1.  workspace (may be null):
// device memory the library's kernels may use.
static int lt_gemm(sfb_stream_t stream, void* c, int out_dtype, const void* a, const void* w, const float* bias,
                   int dtype, uint32_t m, uint32_t n, uint32_t k, int act, float alpha, void* workspace,
                   size_t workspace_bytes, bool* slope_set = nullptr, bool scale_unless_slope_set = false) {
    std::lock_guard<std::mutex> lock(g_mutex);
    const LtOperands ops = {(hipStream_t)stream, c, a, w, bias, workspace, workspace_bytes};
    LtPlan& p = lt_plan(m, n, k, dtype, out_dtype, act, ops);
    if (!p.usable) return SFB_ERR_LAUNCH;
    if (slope_set) *slope_set = p.slope_set;
    if (scale_unless_slope_set && p.slope_set) alpha = 1.0f;
    const float beta = 0.0f;
    const void* bias_ptr = bias;
    if ((bias == nullptr ||
         hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias_ptr, sizeof(bias_ptr)) ==
             HIPBLAS_STATUS_SUCCESS) &&
        hipblasLtMatmul(g_lt, p.desc, &alpha, w, p.w, a, p.a, &beta, c, p.c, c, p.c, &p.algo, workspace, p.workspace,
                        (hipStream_t)stream) == HIPBLAS_STATUS_SUCCESS)
        return SFB_OK;
    p.usable = false;   // do not try this plan again
    return SFB_ERR_LAUNCH;
}

extern "C" int sfb_gemm_tuning(int level) {
    if (level < 0 || level > 1) return SFB_ERR_ARGUMENT;
    std::lock_guard<std::mutex> lock(g_mutex);
    g_tuning_level = level;   // plans already made keep their kernel until sfb_gemm_release()
    return SFB_OK;
}

extern "C" void sfb_gemm_release(void) {
    std::lock_guard<std::mutex> lock(g_mutex);
    for (auto& kv : g_plans) destroy_plan(kv.second);
    g_plans.clear();
    if (g_lt) { hipblasLtDestroy(g_lt); g_lt = nullptr; }
    if (g_handle) { rocblas_destroy_handle(g_handle); g_handle = nullptr; }
}

// whether the activation plan of this shape exists and has its slope set (made on first use, on these operands)
static bool gelu_plan_state(sfb_stream_t stream, void* c, const void* a, const void* w, const float* bias, uint32_t m,
                            uint32_t n, uint32_t k, int dtype, int out_dtype, void* workspace, size_t workspace_bytes,
                            bool* slope_set) {
    std::lock_guard<std::mutex> lock(g_mutex);
    const LtOperands ops = {(hipStream_t)stream, c, a, w, bias, workspace, workspace_bytes};
    const LtPlan& p = lt_plan(m, n, k, dtype, out_dtype, 1, ops);
    *slope_set = p.slope_set;
    return p.usable;
}

__global__ __launch_bounds__(256) void scale_vector_kernel(float* out, const float* in, float factor, uint32_t n) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = in[i] * factor;
}

// c = alpha (a w): the tuned library kernel where there is one, else rocBLAS
static int gemm_ws(sfb_stream_t stream, float* c, const void* a, const void* w, int dtype, uint32_t m, uint32_t n,
                   uint32_t k, float alpha, void* ws, size_t ws_bytes) {
    if (!c || !a || !w) return SFB_ERR_NULL_POINTER;
    if (dtype != SFB_F32 && dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (!m || !n || !k) return SFB_ERR_SHAPE;
    if (lt_gemm(stream, c, SFB_F32, a, w, nullptr, dtype, m, n, k, 0, alpha, ws, ws_bytes) == SFB_OK) return SFB_OK;
    return gemm_alpha(stream, c, a, w, dtype, m, n, k, alpha);
}

extern "C" int sfb_gemm(sfb_stream_t stream, float* c, const void* a, const void* w, int dtype, uint32_t m,
                        uint32_t n, uint32_t k) {
    return gemm_ws(stream, c, a, w, dtype, m, n, k, 1.0f, nullptr, 0);
}

static int gemm_bias_ws(sfb_stream_t stream, void* c, int out_dtype, const void* a, const void* w, const float* bias,
                        int dtype, uint32_t m, uint32_t n, uint32_t k, void* ws, size_t ws_bytes) {
    if (!c || !a || !w || !bias) return SFB_ERR_NULL_POINTER;
    if ((dtype != SFB_F32 && dtype != SFB_BF16) || (out_dtype != SFB_F32 && out_dtype != SFB_BF16)) return SFB_ERR_DTYPE;
    if (!m || !n || !k || (n & 3u)) return SFB_ERR_SHAPE;
    if (lt_gemm(stream, c, out_dtype, a, w, bias, dtype, m, n, k, 0, 1.0f, ws, ws_bytes) == SFB_OK) return SFB_OK;
    // no fused kernel for this shape: plain GEMM, then the bias pass.  The fp32 product needs room: in place for
    // fp32 output, otherwise there is none here
    if (out_dtype != SFB_F32) return SFB_ERR_LAUNCH;
    const int rc = gemm_ws(stream, (float*)c, a, w, dtype, m, n, k, 1.0f, ws, ws_bytes);
    return rc != SFB_OK ? rc : sfb_bias_act(stream, c, SFB_F32, (const float*)c, bias, nullptr, 0, m, n);
}

extern "C" int sfb_gemm_bias(sfb_stream_t stream, void* c, int out_dtype, const void* a, const void* w,
                             const float* bias, int dtype, uint32_t m, uint32_t n, uint32_t k) {
    return gemm_bias_ws(stream, c, out_dtype, a, w, bias, dtype, m, n, k, nullptr, 0);
}

extern "C" int sfb_gemm_bias_gelu(sfb_stream_t stream, void* c, int out_dtype, const void* a, const void* w,
                                  const float* bias, int dtype, uint32_t m, uint32_t n, uint32_t k) {
    if (!c || !a || !w || !bias) return SFB_ERR_NULL_POINTER;
    if ((dtype != SFB_F32 && dtype != SFB_BF16) || (out_dtype != SFB_F32 && out_dtype != SFB_BF16)) return SFB_ERR_DTYPE;
    if (!m || !n || !k || (n & 3u)) return SFB_ERR_SHAPE;
    if (c == a) return SFB_ERR_ARGUMENT;
    bool slope_set = false;
    if (gelu_plan_state(stream, c, a, w, bias, m, n, k, dtype, out_dtype, nullptr, 0, &slope_set) && slope_set &&
        lt_gemm(stream, c, out_dtype, a, w, bias, dtype, m, n, k, 1, 1.0f, nullptr, 0) == SFB_OK)
        return SFB_OK;
    if (out_dtype != SFB_F32) return SFB_ERR_LAUNCH;
    const int rc = sfb_gemm(stream, (float*)c, a, w, dtype, m, n, k);
    return rc != SFB_OK ? rc : sfb_bias_act(stream, c, SFB_F32, (const float*)c, bias, nullptr, 1, m, n);
}

static int gemm_bias_gelu_scaled_ws(sfb_stream_t stream, void* c, int out_dtype, float* scale, float* bias_scratch,
                                    const void* a, const void* w, const float* bias, int dtype, uint32_t m, uint32_t n,
                                    uint32_t k, void* ws, size_t ws_bytes) {
    if (!c || !a || !w || !bias || !scale || !bias_scratch) return SFB_ERR_NULL_POINTER;
    if ((dtype != SFB_F32 && dtype != SFB_BF16) || (out_dtype != SFB_F32 && out_dtype != SFB_BF16)) return SFB_ERR_DTYPE;
    if (!m || !n || !k || (n & 3u)) return SFB_ERR_SHAPE;
    if (c == a) return SFB_ERR_ARGUMENT;
    bool slope_set = false;
    if (!gelu_plan_state(stream, c, a, w, bias, m, n, k, dtype, out_dtype, ws, ws_bytes, &slope_set)) return SFB_ERR_LAUNCH;
    *scale = 1.0f;
    if (slope_set) return lt_gemm(stream, c, out_dtype, a, w, bias, dtype, m, n, k, 1, 1.0f, ws, ws_bytes);
    // x / (1 + exp(-s x)) = Swish_1(s x) / s: the product and the bias are scaled by s going in, and the result is
    // left s times too large for the caller to fold into what it does next
    (void)hipGetLastError();   // only this launch is reported
    scale_vector_kernel<<<dim3((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(bias_scratch, bias, kGeluSigmoidSlope, n);
    if (hipGetLastError() != hipSuccess) return SFB_ERR_LAUNCH;
    *scale = kGeluSigmoidSlope;
    return lt_gemm(stream, c, out_dtype, a, w, bias_scratch, dtype, m, n, k, 1, kGeluSigmoidSlope, ws, ws_bytes);
}

extern "C" int sfb_gemm_bias_gelu_scaled(sfb_stream_t stream, void* c, int out_dtype, float* scale,
                                         float* bias_scratch, const void* a, const void* w, const float* bias,
                                         int dtype, uint32_t m, uint32_t n, uint32_t k) {
    return gemm_bias_gelu_scaled_ws(stream, c, out_dtype, scale, bias_scratch, a, w, bias, dtype, m, n, k, nullptr, 0);
}

extern "C" int sfb_gemm_nt(sfb_stream_t stream, float* c, const void* a, const void* w, int dtype, uint32_t m,
                           uint32_t n, uint32_t k) {
    if (!c || !a || !w) return SFB_ERR_NULL_POINTER;
    if (dtype != SFB_F32 && dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (!m || !n || !k) return SFB_ERR_SHAPE;
    std::lock_guard<std::mutex> lock(g_mutex);
    rocblas_handle h = blas_handle();
    if (!h) return SFB_ERR_LAUNCH;
    if (rocblas_set_stream(h, (hipStream_t)stream) != rocblas_status_success) return SFB_ERR_LAUNCH;
    const float alpha = 1.0f, beta = 0.0f;
    const rocblas_datatype in = dtype == SFB_BF16 ? rocblas_datatype_bf16_r : rocblas_datatype_f32_r;
    // row-major C[m][n] = A[m][k] W[n][k]^T  ==  column-major C^T[n][m] = (W^T[k][n])^T A^T[k][m]
    const rocblas_status st = rocblas_gemm_ex(h, rocblas_operation_transpose, rocblas_operation_none, (int)n, (int)m,
                                              (int)k, &alpha, w, in, (int)k, a, in, (int)k, &beta, c,
                                              rocblas_datatype_f32_r, (int)n, c, rocblas_datatype_f32_r, (int)n,
                                              rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
    return st == rocblas_status_success ? SFB_OK : SFB_ERR_LAUNCH;
}

extern "C" int sfb_pack_qkv(sfb_stream_t stream, void* wqkv, float* bqkv, const sfb_layer_weights* wt, int dtype,
                            uint32_t n) {
    if (!wqkv || !bqkv || !wt || !wt->wq || !wt->wk || !wt->wv || !wt->bq || !wt->bk || !wt->bv)
        return SFB_ERR_NULL_POINTER;
    if (dtype != SFB_F32 && dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (n == 0) return SFB_ERR_SHAPE;
    const size_t esz = dtype == SFB_BF16 ? 2 : 4;
    const void* w[3] = {wt->wq, wt->wk, wt->wv};
    const float* b[3] = {wt->bq, wt->bk, wt->bv};
    hipStream_t s = (hipStream_t)stream;
    for (int i = 0; i < 3; ++i) {
        // row r of W_i becomes columns [i n, (i + 1) n) of row r
        if (hipMemcpy2DAsync((uint8_t*)wqkv + (size_t)i * n * esz, (size_t)3 * n * esz, w[i], (size_t)n * esz,
                             (size_t)n * esz, n, hipMemcpyDeviceToDevice, s) != hipSuccess)
            return SFB_ERR_LAUNCH;
        if (hipMemcpyAsync(bqkv + (size_t)i * n, b[i], (size_t)n * sizeof(float), hipMemcpyDeviceToDevice, s) != hipSuccess)
            return SFB_ERR_LAUNCH;
    }
    return SFB_OK;
}

extern "C" size_t sfb_encoder_layer_workspace_bytes(uint32_t batch_dim, uint32_t ctx, uint32_t head_dim,
                                                    uint32_t state_dim, uint32_t ffn, int dtype) {
    const size_t m = (size_t)batch_dim * ctx, n = (size_t)head_dim * state_dim;
    const size_t f32 = sizeof(float), act = dtype == SFB_BF16 ? 2 : 4;
    // t (fp32 GEMM output, m x max(n, ffn)); q, k, v (compute dtype); attn (fp32); x1 (fp32);
    // bf16 path only: xa (activation in compute dtype, m x max(n, ffn)); ffn floats of bias scratch
    size_t bytes = align256(m * (ffn > n ? ffn : n) * f32) + 3 * align256(m * n * act) + 2 * align256(m * n * f32);
    if (dtype == SFB_BF16) bytes += align256(m * (ffn > n ? ffn : n) * act);
    bytes += align256(ffn * f32);   // scaled copy of the first FFN bias (sfb_gemm_bias_gelu_scaled)
    return bytes + kGemmWorkspaceBytes;   // scratch for the GEMM library's kernels
}

// Scratch offered to the GEMM library's kernels at the end of a layer's workspace
static void* gemm_scratch(const float* bias_scratch, uint32_t ffn) {
    return (uint8_t*)bias_scratch + align256((size_t)ffn * sizeof(float));
}

// Everything a layer needs besides its input, output and weights
struct LayerArgs {
    int dtype;
    const sfb_uint2* nn_lut;
    const void* mask;
    const int32_t* valid_len;
    const sfb_work_item* items;
    uint32_t n_items, n_heavy, n_slots, n_parts;
    void* attn_workspace;
    size_t attn_workspace_bytes;
    uint32_t block_size, blocks, batch_dim, ctx_blks, head_dim, state_dim, ffn;
    void* workspace;
    size_t workspace_bytes;
    // streamed attention launch instead of a scheduled one (takes per-head look-up tables and masks)
    const sfb_stream_plan* st_plan = nullptr;
    const void* st_blob = nullptr;
    uint32_t lut_heads = 1, lut_dim = 0, mask_heads = 1;
};

// out = a W + bias in the compute dtype: one GEMM with the bias in its epilogue, or, where that is not available,
// GEMM into the fp32 scratch t followed by the bias pass
static int project(sfb_stream_t stream, void* out, int out_dtype, float* t, const void* a, const void* w,
                   const float* bias, int dtype, size_t m, uint32_t n, uint32_t k, void* ws) {
    if (gemm_bias_ws(stream, out, out_dtype, a, w, bias, dtype, (uint32_t)m, n, k, ws, kGemmWorkspaceBytes) == SFB_OK)
        return SFB_OK;
    const int rc = gemm_ws(stream, t, a, w, dtype, (uint32_t)m, n, k, 1.0f, ws, kGemmWorkspaceBytes);
    return rc != SFB_OK ? rc : sfb_bias_act(stream, out, out_dtype, t, bias, nullptr, 0, m, n);
}

// Attention output as the operand of the output projection: *ain points at it.  A scheduled bf16 launch writes
// bf16 straight into lp; otherwise the fp32 result in attn is used (fp32 path) or cast into lp (bf16 path).
static int attention_call(sfb_stream_t stream, const LayerArgs& g, const void* q, const void* k, const void* v,
                          float* attn);
static int attention_operand(sfb_stream_t stream, const LayerArgs& g, const void* q, const void* k, const void* v,
                             float* attn, void* lp, size_t elements, const void** ain) {
    const float scale = 1.0f / sqrtf((float)g.state_dim);
    if (g.st_plan) {
        // bf16 activations: bf16 straight into lp; fp32: into attn
        void* const out = g.dtype == SFB_BF16 ? lp : (void*)attn;
        *ain = out;
        return sfb_fused_attention_streamed(stream, q, k, v, out, nullptr, g.dtype, g.dtype, g.nn_lut, g.mask, g.valid_len,
                                            g.st_plan, g.st_blob, g.attn_workspace, g.attn_workspace_bytes, g.block_size,
                                            g.blocks, g.batch_dim, g.ctx_blks, g.head_dim, g.state_dim, g.lut_heads,
                                            g.lut_dim, g.mask_heads, scale);
    }
    if (g.dtype == SFB_BF16 && g.items) {
        *ain = lp;
        return sfb_fused_attention_scheduled_to(stream, q, k, v, lp, g.dtype, SFB_BF16, g.nn_lut, g.mask, g.valid_len,
                                                g.items, g.n_items, g.n_heavy, g.n_slots, g.n_parts, g.attn_workspace,
                                                g.attn_workspace_bytes, g.block_size, g.blocks, g.batch_dim, g.ctx_blks,
                                                g.head_dim, g.state_dim, 1, scale);
    }
    int rc = attention_call(stream, g, q, k, v, attn);
    if (rc != SFB_OK) return rc;
    *ain = attn;
    if (g.dtype == SFB_BF16) {
        rc = sfb_cast_f32_bf16(stream, lp, attn, elements);
        *ain = lp;
    }
    return rc;
}

static int attention_call(sfb_stream_t stream, const LayerArgs& g, const void* q, const void* k, const void* v,
                          float* attn) {
    const float scale = 1.0f / sqrtf((float)g.state_dim);
    if (g.items)
        return sfb_fused_attention_scheduled(stream, q, k, v, attn, g.dtype, g.nn_lut, g.mask, g.valid_len, g.items,
                                             g.n_items, g.n_heavy, g.n_slots, g.n_parts, g.attn_workspace,
                                             g.attn_workspace_bytes, g.block_size, g.blocks, g.batch_dim, g.ctx_blks,
                                             g.head_dim, g.state_dim, 1, scale);
    return sfb_fused_attention(stream, q, k, v, attn, g.dtype, g.nn_lut, g.mask, g.valid_len, nullptr, g.block_size,
                               g.blocks, g.batch_dim, g.ctx_blks, g.head_dim, g.state_dim, 1, g.ctx_blks + g.blocks, 1,
                               scale);
}

// Q, K and V as one product when the caller supplies the merged matrix (sfb_pack_qkv) and the attention is a
// scheduled launch on the compute dtype: C [m][3n] = a [Wq | Wk | Wv] + [bq | bk | bv] into the q, k, v buffers (which
// are consecutive), then the attention reads its three operands as column slices, 3n elements per token.  Returns
// false when the conditions are not met and the three separate products are to be made.
static bool merged_projection(sfb_stream_t stream, const LayerArgs& g, const sfb_layer_weights* wt, const void* a,
                              void* q, void* k, void* v, float* t, void* lp, float* attn, size_t m, size_t n, void* gws,
                              const void** ain, int* rc) {
    const size_t act = g.dtype == SFB_BF16 ? 2 : 4;
    if (!wt->wqkv || !wt->bqkv || !g.items || g.st_plan) return false;
    if ((uint8_t*)k != (uint8_t*)q + m * n * act || (uint8_t*)v != (uint8_t*)k + m * n * act) return false;
    if ((3 * n) % (g.dtype == SFB_BF16 ? 8 : 4) != 0) return false;
    // without a library kernel for this shape the separate products (which have a fallback) are made instead
    if (gemm_bias_ws(stream, q, g.dtype, a, wt->wqkv, wt->bqkv, g.dtype, (uint32_t)m, (uint32_t)(3 * n), (uint32_t)n, gws,
                     kGemmWorkspaceBytes) != SFB_OK)
        return false;
    const float scale = 1.0f / sqrtf((float)g.state_dim);
    void* const out = g.dtype == SFB_BF16 ? lp : (void*)attn;
    *ain = out;
    *rc = sfb_fused_attention_scheduled_strided(stream, q, (const uint8_t*)q + n * act, (const uint8_t*)q + 2 * n * act, out,
                                                g.dtype, g.dtype, g.nn_lut, g.mask, g.valid_len, g.items, g.n_items,
                                                g.n_heavy, g.n_slots, g.n_parts, g.attn_workspace,
                                                g.attn_workspace_bytes, g.block_size, g.blocks, g.batch_dim, g.ctx_blks,
                                                g.head_dim, g.state_dim, (uint32_t)(3 * n), 1, scale);
    return true;
}

// The reference's own wiring (transformer.cpp:513-580, transformer_inference_part.cpp:209-232), dropout omitted:
//     a = LN1(x);  x1 = x + (Attn(a Wq + bq, a Wk + bk, a Wv + bv) Wo + bo);  y = x1 + (gelu(LN2(x1) W1 + b1) W2 + b2)
static int layer_forward_pre_ln(sfb_stream_t stream, float* y, const float* x, const sfb_layer_weights* wt,
                                const LayerArgs& g) {
    const uint32_t ctx = g.ctx_blks * g.block_size, ffn = g.ffn;
    const size_t m = (size_t)g.batch_dim * ctx, n = (size_t)g.head_dim * g.state_dim;
    const int dtype = g.dtype;
    const bool bf = dtype == SFB_BF16;
    const size_t act = bf ? 2 : 4, wide = ffn > n ? ffn : n;
    uint8_t* p = (uint8_t*)g.workspace;
    float* t = (float*)p;            p += align256(m * wide * sizeof(float));
    void* q = p;                     p += align256(m * n * act);
    void* k = p;                     p += align256(m * n * act);
    void* v = p;                     p += align256(m * n * act);
    float* attn = (float*)p;         p += align256(m * n * sizeof(float));
    float* x1 = (float*)p;           p += align256(m * n * sizeof(float));
    void* xa = bf ? (void*)p : nullptr;
    if (bf) p += align256(m * wide * act);
    float* bias_scratch = (float*)p;
    void* const gws = gemm_scratch(bias_scratch, ffn);
    int rc;
#define SFB_TRY(call) do { rc = (call); if (rc != SFB_OK) return rc; } while (0)
    // LN1 straight into the compute dtype; the fp32 path borrows the attention output buffer, which is free
    // until the attention runs
    void* a = bf ? xa : (void*)attn;
    SFB_TRY(sfb_layernorm(stream, a, dtype, nullptr, nullptr, x, wt->ln1_g, wt->ln1_b, (uint32_t)m, (uint32_t)n));
    const void* ain = nullptr;
    if (merged_projection(stream, g, wt, a, q, k, v, t, xa, attn, m, n, gws, &ain, &rc)) {
        if (rc != SFB_OK) return rc;
    } else {
        SFB_TRY(project(stream, q, dtype, t, a, wt->wq, wt->bq, dtype, m, (uint32_t)n, (uint32_t)n, gws));
        SFB_TRY(project(stream, k, dtype, t, a, wt->wk, wt->bk, dtype, m, (uint32_t)n, (uint32_t)n, gws));
        SFB_TRY(project(stream, v, dtype, t, a, wt->wv, wt->bv, dtype, m, (uint32_t)n, (uint32_t)n, gws));
        SFB_TRY(attention_operand(stream, g, q, k, v, attn, xa, m * n, &ain));
    }
    SFB_TRY(project(stream, t, SFB_F32, t, ain, wt->wo, wt->bo, dtype, m, (uint32_t)n, (uint32_t)n, gws));
    SFB_TRY(sfb_bias_act(stream, x1, SFB_F32, t, nullptr, x, 0, m, (uint32_t)n));
    // LN2 into the compute dtype (fp32: the attention output buffer again, consumed by the GEMM above)
    void* a2 = bf ? xa : (void*)attn;
    SFB_TRY(sfb_layernorm(stream, a2, dtype, nullptr, nullptr, x1, wt->ln2_g, wt->ln2_b, (uint32_t)m, (uint32_t)n));
    void* gl = t;
    float* t2 = attn;
    float g_scale = 1.0f;
    if (gemm_bias_gelu_scaled_ws(stream, t, dtype, &g_scale, bias_scratch, a2, wt->w1, wt->b1, dtype, (uint32_t)m, ffn,
                                 (uint32_t)n, gws, kGemmWorkspaceBytes) != SFB_OK) {
        SFB_TRY(gemm_ws(stream, t, a2, wt->w1, dtype, (uint32_t)m, ffn, (uint32_t)n, 1.0f, gws, kGemmWorkspaceBytes));
        gl = bf ? xa : (void*)t;
        SFB_TRY(sfb_bias_act(stream, gl, dtype, t, wt->b1, nullptr, 1, m, ffn));
        t2 = bf ? t : attn;
        g_scale = 1.0f;
    }
    SFB_TRY(gemm_ws(stream, t2, gl, wt->w2, dtype, (uint32_t)m, (uint32_t)n, ffn, 1.0f / g_scale, gws, kGemmWorkspaceBytes));
    SFB_TRY(sfb_bias_act(stream, y, SFB_F32, t2, wt->b2, x1, 0, m, (uint32_t)n));
#undef SFB_TRY
    return SFB_OK;
}

static int check_layer_args(const float* y, const float* x, const sfb_layer_weights* wt, const LayerArgs& g) {
    if (!y || !x || !wt || !g.nn_lut || !g.workspace) return SFB_ERR_NULL_POINTER;
    if (g.dtype != SFB_F32 && g.dtype != SFB_BF16) return SFB_ERR_DTYPE;
    const uint32_t ctx = g.ctx_blks * g.block_size;
    const size_t m = (size_t)g.batch_dim * ctx, n = (size_t)g.head_dim * g.state_dim;
    if (!m || !n || !g.ffn || (n & 3u) || (g.ffn & 3u)) return SFB_ERR_SHAPE;
    if (g.workspace_bytes <
            sfb_encoder_layer_workspace_bytes(g.batch_dim, ctx, g.head_dim, g.state_dim, g.ffn, g.dtype) ||
        ((uintptr_t)g.workspace & 255u))
        return SFB_ERR_WORKSPACE;
    return SFB_OK;
}

extern "C" int sfb_encoder_layer_forward_pre_ln(sfb_stream_t stream, float* y, const float* x,
                                                const sfb_layer_weights* wt, int dtype, const sfb_uint2* nn_lut,
                                                const void* mask, const int32_t* valid_len,
                                                const sfb_work_item* items, uint32_t n_items, uint32_t n_heavy,
                                                uint32_t n_slots, uint32_t n_parts, void* attn_workspace,
                                                size_t attn_workspace_bytes, uint32_t block_size, uint32_t blocks,
                                                uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                                                uint32_t state_dim, uint32_t ffn, void* workspace,
                                                size_t workspace_bytes) {
    const LayerArgs g = {dtype, nn_lut, mask, valid_len, items, n_items, n_heavy, n_slots, n_parts, attn_workspace,
                         attn_workspace_bytes, block_size, blocks, batch_dim, ctx_blks, head_dim, state_dim, ffn,
                         workspace, workspace_bytes};
    const int rc = check_layer_args(y, x, wt, g);
    return rc != SFB_OK ? rc : layer_forward_pre_ln(stream, y, x, wt, g);
}

// Post-LN layer: x1 = LN1(x + Attn(xWq+bq, xWk+bk, xWv+bv) Wo + bo), y = LN2(x1 + gelu(x1 W1 + b1) W2 + b2)
static int layer_forward_post_ln(sfb_stream_t stream, float* y, const float* x, const sfb_layer_weights* wt,
                                 const LayerArgs& la) {
    const int dtype = la.dtype;
    const sfb_uint2* const nn_lut = la.nn_lut;
    void* const workspace = la.workspace;
    const size_t workspace_bytes = la.workspace_bytes;
    const uint32_t block_size = la.block_size, batch_dim = la.batch_dim, ctx_blks = la.ctx_blks, head_dim = la.head_dim,
                   state_dim = la.state_dim, ffn = la.ffn;
    if (!y || !x || !wt || !nn_lut || !workspace) return SFB_ERR_NULL_POINTER;
    if (dtype != SFB_F32 && dtype != SFB_BF16) return SFB_ERR_DTYPE;
    const uint32_t ctx = ctx_blks * block_size;
    const size_t m = (size_t)batch_dim * ctx, n = (size_t)head_dim * state_dim;
    if (!m || !n || !ffn || (n & 3u) || (ffn & 3u)) return SFB_ERR_SHAPE;
    if (workspace_bytes < sfb_encoder_layer_workspace_bytes(batch_dim, ctx, head_dim, state_dim, ffn, dtype) ||
        ((uintptr_t)workspace & 255u))
        return SFB_ERR_WORKSPACE;
    const bool bf = dtype == SFB_BF16;
    const size_t act = bf ? 2 : 4, wide = ffn > n ? ffn : n;
    uint8_t* p = (uint8_t*)workspace;
    float* t = (float*)p;            p += align256(m * wide * sizeof(float));
    void* q = p;                     p += align256(m * n * act);
    void* k = p;                     p += align256(m * n * act);
    void* v = p;                     p += align256(m * n * act);
    float* attn = (float*)p;         p += align256(m * n * sizeof(float));
    float* x1 = (float*)p;           p += align256(m * n * sizeof(float));
    void* xa = bf ? (void*)p : nullptr;
    if (bf) p += align256(m * wide * act);
    float* bias_scratch = (float*)p;
    void* const gws = gemm_scratch(bias_scratch, ffn);
    const float scale = 1.0f / sqrtf((float)state_dim);
    int rc;
#define SFB_TRY(call) do { rc = (call); if (rc != SFB_OK) return rc; } while (0)

    // Q, K, V projections (+ bias), stored in the compute dtype for the attention kernel
    const void* xin = x;
    if (bf) { SFB_TRY(sfb_cast_f32_bf16(stream, xa, x, m * n)); xin = xa; }
    // attention, [B, L, H, d] is the token-major activation layout itself: no transposes
    const void* ain = nullptr;
    if (merged_projection(stream, la, wt, xin, q, k, v, t, xa, attn, m, n, gws, &ain, &rc)) {
        if (rc != SFB_OK) return rc;
    } else {
        SFB_TRY(project(stream, q, dtype, t, xin, wt->wq, wt->bq, dtype, m, (uint32_t)n, (uint32_t)n, gws));
        SFB_TRY(project(stream, k, dtype, t, xin, wt->wk, wt->bk, dtype, m, (uint32_t)n, (uint32_t)n, gws));
        SFB_TRY(project(stream, v, dtype, t, xin, wt->wv, wt->bv, dtype, m, (uint32_t)n, (uint32_t)n, gws));
        SFB_TRY(attention_operand(stream, la, q, k, v, attn, xa, m * n, &ain));
    }

    // output projection + bias, residual, LayerNorm 1
    SFB_TRY(project(stream, t, SFB_F32, t, ain, wt->wo, wt->bo, dtype, m, (uint32_t)n, (uint32_t)n, gws));
    // residual + LayerNorm 1 in one pass when the row fits in registers; the bf16 path gets its copy of x1
    // for the next GEMM from the same kernel
    const bool fused_ln = n <= 2048;
    if (fused_ln) {
        SFB_TRY(sfb_bias_residual_layernorm(stream, x1, bf ? xa : nullptr, t, nullptr, x, wt->ln1_g, wt->ln1_b,
                                            (uint32_t)m, (uint32_t)n));
    } else {
        SFB_TRY(sfb_bias_act(stream, t, SFB_F32, t, nullptr, x, 0, m, (uint32_t)n));
        SFB_TRY(sfb_layernorm(stream, x1, SFB_F32, nullptr, nullptr, t, wt->ln1_g, wt->ln1_b, (uint32_t)m, (uint32_t)n));
    }

    // FFN: GEMM, bias + sigmoid-GELU, GEMM, bias + residual, LayerNorm 2
    const void* fin = x1;
    if (bf) {
        if (!fused_ln) SFB_TRY(sfb_cast_f32_bf16(stream, xa, x1, m * n));
        fin = xa;
    }
    // bias and GELU ride in the first GEMM's epilogue where the library has such a kernel (its result goes into t,
    // which nothing else uses at this point); otherwise GEMM into t, then one bias + GELU pass
    void* g = t;                    // activation after GELU (times g_scale), in the compute dtype
    float* t2 = attn;               // the second FFN GEMM reads g and must not write over it
    float g_scale = 1.0f;
    if (gemm_bias_gelu_scaled_ws(stream, t, dtype, &g_scale, bias_scratch, fin, wt->w1, wt->b1, dtype, (uint32_t)m, ffn,
                                 (uint32_t)n, gws, kGemmWorkspaceBytes) != SFB_OK) {
        SFB_TRY(gemm_ws(stream, t, fin, wt->w1, dtype, (uint32_t)m, ffn, (uint32_t)n, 1.0f, gws, kGemmWorkspaceBytes));
        g = bf ? xa : (void*)t;     // in place for fp32
        SFB_TRY(sfb_bias_act(stream, g, dtype, t, wt->b1, nullptr, 1, m, ffn));
        t2 = bf ? t : attn;
        g_scale = 1.0f;
    }
    SFB_TRY(gemm_ws(stream, t2, g, wt->w2, dtype, (uint32_t)m, (uint32_t)n, ffn, 1.0f / g_scale, gws, kGemmWorkspaceBytes));
    if (fused_ln) {
        SFB_TRY(sfb_bias_residual_layernorm(stream, y, nullptr, t2, wt->b2, x1, wt->ln2_g, wt->ln2_b, (uint32_t)m,
                                            (uint32_t)n));
    } else {
        SFB_TRY(sfb_bias_act(stream, t2, SFB_F32, t2, wt->b2, x1, 0, m, (uint32_t)n));
        SFB_TRY(sfb_layernorm(stream, y, SFB_F32, nullptr, nullptr, t2, wt->ln2_g, wt->ln2_b, (uint32_t)m, (uint32_t)n));
    }
#undef SFB_TRY
    return SFB_OK;
}

extern "C" int sfb_encoder_layer_forward(sfb_stream_t stream, float* y, const float* x,
                                         const sfb_layer_weights* wt, int dtype, const sfb_uint2* nn_lut,
                                         const void* mask, const int32_t* valid_len,
                                         const sfb_work_item* items, uint32_t n_items, uint32_t n_heavy,
                                         uint32_t n_slots, uint32_t n_parts, void* attn_workspace, size_t attn_workspace_bytes,
                                         uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                         uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim, uint32_t ffn,
                                         void* workspace, size_t workspace_bytes) {
    const LayerArgs g = {dtype, nn_lut, mask, valid_len, items, n_items, n_heavy, n_slots, n_parts, attn_workspace,
                         attn_workspace_bytes, block_size, blocks, batch_dim, ctx_blks, head_dim, state_dim, ffn,
                         workspace, workspace_bytes};
    return layer_forward_post_ln(stream, y, x, wt, g);
}

extern "C" int sfb_encoder_layer_forward_streamed(sfb_stream_t stream, float* y, const float* x,
                                                  const sfb_layer_weights* wt, int dtype, int pre_ln,
                                                  const sfb_uint2* nn_lut, const void* mask, const int32_t* valid_len,
                                                  const sfb_stream_plan* plan, const void* blob, void* attn_workspace,
                                                  size_t attn_workspace_bytes, uint32_t block_size, uint32_t blocks,
                                                  uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                                                  uint32_t state_dim, uint32_t lut_heads, uint32_t lut_dim,
                                                  uint32_t mask_heads, uint32_t ffn, void* workspace,
                                                  size_t workspace_bytes) {
    if (!plan || !blob) return SFB_ERR_NULL_POINTER;
    LayerArgs g = {dtype, nn_lut, mask, valid_len, nullptr, 0, 0, 0, 0, attn_workspace,
                   attn_workspace_bytes, block_size, blocks, batch_dim, ctx_blks, head_dim, state_dim, ffn,
                   workspace, workspace_bytes};
    g.st_plan = plan;
    g.st_blob = blob;
    g.lut_heads = lut_heads;
    g.lut_dim = lut_dim;
    g.mask_heads = mask_heads;
    if (pre_ln) {
        const int rc = check_layer_args(y, x, wt, g);
        return rc != SFB_OK ? rc : layer_forward_pre_ln(stream, y, x, wt, g);
    }
    return layer_forward_post_ln(stream, y, x, wt, g);
}

// ------------------------------------------------------------------------------------------------
// Whole-model forward in the shape of transformer_inference_part.cpp:190-256 (dropout omitted):
// embedding gather + position add, n_layers encoder layers, tied-embedding logits, cross-entropy loss.
// ------------------------------------------------------------------------------------------------
extern "C" size_t sfb_model_workspace_bytes(uint32_t batch_dim, uint32_t ctx, uint32_t head_dim, uint32_t state_dim,
                                            uint32_t ffn, uint32_t vocab, int dtype) {
    const size_t m = (size_t)batch_dim * ctx, n = (size_t)head_dim * state_dim;
    // layer workspace; two activation buffers (fp32); logits (fp32); row losses; bf16 copy of the last hidden state
    size_t bytes = align256(sfb_encoder_layer_workspace_bytes(batch_dim, ctx, head_dim, state_dim, ffn, dtype)) +
                   2 * align256(m * n * sizeof(float)) + align256(m * (size_t)vocab * sizeof(float)) +
                   align256(m * sizeof(float));
    if (dtype == SFB_BF16) bytes += align256(m * n * 2);
    return bytes;
}

extern "C" int sfb_model_forward(sfb_stream_t stream, float* loss, float* logits, float* hidden, const int32_t* ids,
                                 const int32_t* labels, const sfb_model_weights* w, int dtype, int pre_ln,
                                 const sfb_uint2* nn_lut, const void* mask, const int32_t* valid_len,
                                 const sfb_work_item* items, uint32_t n_items, uint32_t n_heavy, uint32_t n_slots,
                                 uint32_t n_parts, void* attn_workspace, size_t attn_workspace_bytes,
                                 uint32_t block_size, uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks,
                                 uint32_t head_dim, uint32_t state_dim, uint32_t ffn, uint32_t vocab, void* workspace,
                                 size_t workspace_bytes) {
    if (!ids || !w || !w->tok_embed || !w->pos_embed || (w->n_layers && !w->layers) || !nn_lut || !workspace)
        return SFB_ERR_NULL_POINTER;
    if (labels && !loss) return SFB_ERR_NULL_POINTER;
    if (dtype != SFB_F32 && dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (dtype == SFB_BF16 && !w->tok_embed_bf16) return SFB_ERR_NULL_POINTER;
    const uint32_t ctx = ctx_blks * block_size;
    const size_t m = (size_t)batch_dim * ctx, n = (size_t)head_dim * state_dim;
    if (!m || !n || !ffn || !vocab || (n & 3u) || (ffn & 3u)) return SFB_ERR_SHAPE;
    if (workspace_bytes < sfb_model_workspace_bytes(batch_dim, ctx, head_dim, state_dim, ffn, vocab, dtype) ||
        ((uintptr_t)workspace & 255u))
        return SFB_ERR_WORKSPACE;
    const size_t layer_bytes = align256(sfb_encoder_layer_workspace_bytes(batch_dim, ctx, head_dim, state_dim, ffn, dtype));
    uint8_t* p = (uint8_t*)workspace;
    void* layer_ws = p;              p += layer_bytes;
    float* xa = (float*)p;           p += align256(m * n * sizeof(float));
    float* xb = (float*)p;           p += align256(m * n * sizeof(float));
    float* lg = (float*)p;           p += align256(m * (size_t)vocab * sizeof(float));
    float* row_loss = (float*)p;     p += align256(m * sizeof(float));
    void* x16 = dtype == SFB_BF16 ? (void*)p : nullptr;
    if (logits) lg = logits;
    int rc;
#define SFB_TRY(call) do { rc = (call); if (rc != SFB_OK) return rc; } while (0)
    SFB_TRY(sfb_embedding_lookup(stream, xa, w->tok_embed, ids, w->pos_embed, m, (uint32_t)n, ctx, vocab));
    for (uint32_t i = 0; i < w->n_layers; ++i) {
        if (pre_ln)
            SFB_TRY(sfb_encoder_layer_forward_pre_ln(stream, xb, xa, w->layers + i, dtype, nn_lut, mask, valid_len, items,
                                                     n_items, n_heavy, n_slots, n_parts, attn_workspace,
                                                     attn_workspace_bytes, block_size, blocks, batch_dim, ctx_blks,
                                                     head_dim, state_dim, ffn, layer_ws, layer_bytes));
        else
            SFB_TRY(sfb_encoder_layer_forward(stream, xb, xa, w->layers + i, dtype, nn_lut, mask, valid_len, items,
                                              n_items, n_heavy, n_slots, n_parts, attn_workspace, attn_workspace_bytes,
                                              block_size, blocks, batch_dim, ctx_blks, head_dim, state_dim, ffn,
                                              layer_ws, layer_bytes));
        float* swap = xa; xa = xb; xb = swap;
    }
    if (hidden && hipMemcpyAsync(hidden, xa, m * n * sizeof(float), hipMemcpyDeviceToDevice, (hipStream_t)stream) !=
                      hipSuccess)
        return SFB_ERR_LAUNCH;
    // logits = hidden . tok_embed^T (transformer_inference_part.cpp:236)
    const void* hin = xa;
    const void* table = w->tok_embed;
    if (dtype == SFB_BF16) {
        SFB_TRY(sfb_cast_f32_bf16(stream, x16, xa, m * n));
        hin = x16;
        table = w->tok_embed_bf16;
    }
    SFB_TRY(sfb_gemm_nt(stream, lg, hin, table, dtype, (uint32_t)m, vocab, (uint32_t)n));
    if (labels) SFB_TRY(sfb_softmax_cross_entropy(stream, loss, row_loss, nullptr, lg, labels, m, vocab));
#undef SFB_TRY
    return SFB_OK;
}
