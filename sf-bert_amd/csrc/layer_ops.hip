// Encoder-layer ops around the attention path: LayerNorm, bias (+ sigmoid-GELU) (+ residual),
// residual / position adds, embedding gather, fp32 -> bf16 casts.  All are one pass over HBM.
// Arithmetic follows the reference CPU functions (layernorm.h:13-38, ewops.h:10-17, 32-43, 276-301,
// embedding.h:5-12); their GPU twins are cuda_kernels.h:334-372, 459-489, 561-581, 449-457, 526-535,
// 210-221.
#include "common.hip.h"

namespace sfb {

// x * 1/(1 + exp(-1.702 x))  (ewops.h:32-43)
__device__ __forceinline__ float sigmoid_gelu(float x) {
    return x * (1.0f / (1.0f + exp2_fast(-1.702f * kLog2e * x)));
}

__device__ __forceinline__ void store_out(float* p, f32x4 v) { *(f32x4*)p = v; }
__device__ __forceinline__ void store_out(__bf16* p, f32x4 v) {
    const u32x2 r = {pack_bf16(v.x, v.y), pack_bf16(v.z, v.w)};
    *(u32x2*)p = r;
}

// out[r][c] = act(in[r][c] + bias[c]) + residual[r][c]; cols % 4 == 0.
template <typename TOut, int ACT>
__global__ __launch_bounds__(256) void bias_act_kernel(TOut* out, const float* in, const float* bias,
                                                       const float* residual, uint64_t vecs,
                                                       uint32_t cols4) {
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < vecs;
         i += (uint64_t)gridDim.x * blockDim.x) {
        f32x4 v = ((const f32x4*)in)[i];
        if (bias) v += ((const f32x4*)bias)[i % cols4];
        if (ACT == 1) {
            v.x = sigmoid_gelu(v.x); v.y = sigmoid_gelu(v.y); v.z = sigmoid_gelu(v.z); v.w = sigmoid_gelu(v.w);
        }
        if (residual) v += ((const f32x4*)residual)[i];
        store_out(out + i * 4, v);
    }
}

// One wave per row: mean and E[x^2] over the row, rstd = 1/sqrt(E[x^2] - mean^2 + 1e-5)
// (layernorm.h:16-30), y = ((x - mean) * rstd) * g + b (layernorm.h:34).  state % 4 == 0.
template <typename TOut>
__global__ __launch_bounds__(256) void layernorm_kernel(TOut* out, float* mean_out, float* rstd_out,
                                                        const float* in, const float* gain,
                                                        const float* bias, uint32_t rows, uint32_t state) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x * 4 + wave;
    if (row >= rows) return;
    const f32x4* x = (const f32x4*)(in + (size_t)row * state);
    const uint32_t vecs = state / 4;
    float sum = 0.f, sq = 0.f;
    for (uint32_t i = lane; i < vecs; i += 64) {
        const f32x4 v = x[i];
        sum += (v.x + v.y) + (v.z + v.w);
        sq += (v.x * v.x + v.y * v.y) + (v.z * v.z + v.w * v.w);
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        sum += __shfl_xor(sum, d);
        sq += __shfl_xor(sq, d);
    }
    const float mean = sum / (float)state;
    const float var = sq / (float)state - mean * mean;
    const float rstd = 1.0f / sqrtf(var + 1e-5f);
    if (lane == 0) {
        if (mean_out) mean_out[row] = mean;
        if (rstd_out) rstd_out[row] = rstd;
    }
    TOut* y = out + (size_t)row * state;
    for (uint32_t i = lane; i < vecs; i += 64) {
        const f32x4 v = x[i], g = ((const f32x4*)gain)[i], b = ((const f32x4*)bias)[i];
        const f32x4 r = {((v.x - mean) * rstd) * g.x + b.x, ((v.y - mean) * rstd) * g.y + b.y,
                         ((v.z - mean) * rstd) * g.z + b.z, ((v.w - mean) * rstd) * g.w + b.w};
        store_out(y + i * 4, r);
    }
}

// y = LayerNorm((in + bias) + residual) in one pass over memory: the row stays in registers between
// the sums and the normalisation (one wave per row, VECS float4 per lane).  Same arithmetic, in the same
// order, as bias_act_kernel followed by layernorm_kernel.  Optionally also writes y rounded to bf16.
template <int VECS>
__global__ __launch_bounds__(256) void bias_residual_layernorm_kernel(float* out, __bf16* out_bf16, const float* in,
                                                                      const float* bias, const float* residual,
                                                                      const float* gain, const float* beta,
                                                                      uint32_t rows, uint32_t state) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x * 4 + wave;
    if (row >= rows) return;
    const uint32_t vecs = state / 4;
    const f32x4* x = (const f32x4*)(in + (size_t)row * state);
    const f32x4* r = residual ? (const f32x4*)(residual + (size_t)row * state) : nullptr;
    f32x4 v[VECS];
    float sum = 0.f, sq = 0.f;
#pragma unroll
    for (int k = 0; k < VECS; ++k) {
        const uint32_t i = lane + 64 * k;
        if (i < vecs) {
            f32x4 t = x[i];
            if (bias) t += ((const f32x4*)bias)[i];
            if (r) t += r[i];
            v[k] = t;
            sum += (t.x + t.y) + (t.z + t.w);
            sq += (t.x * t.x + t.y * t.y) + (t.z * t.z + t.w * t.w);
        }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        sum += __shfl_xor(sum, d);
        sq += __shfl_xor(sq, d);
    }
    const float mean = sum / (float)state;
    const float var = sq / (float)state - mean * mean;
    const float rstd = 1.0f / sqrtf(var + 1e-5f);
#pragma unroll
    for (int k = 0; k < VECS; ++k) {
        const uint32_t i = lane + 64 * k;
        if (i < vecs) {
            const f32x4 t = v[k], g = ((const f32x4*)gain)[i], b = ((const f32x4*)beta)[i];
            const f32x4 y = {((t.x - mean) * rstd) * g.x + b.x, ((t.y - mean) * rstd) * g.y + b.y,
                             ((t.z - mean) * rstd) * g.z + b.z, ((t.w - mean) * rstd) * g.w + b.w};
            store_out(out + (size_t)row * state + i * 4, y);
            if (out_bf16) store_out(out_bf16 + (size_t)row * state + i * 4, y);
        }
    }
}

// out[b][i] = a[b][i] + m[i]  (ewops.h:276-282: position embedding broadcast over the batch)
__global__ __launch_bounds__(256) void add_matrix_kernel(float* out, const float* a, const float* m,
                                                         uint64_t vecs, uint64_t inner4) {
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < vecs;
         i += (uint64_t)gridDim.x * blockDim.x)
        ((f32x4*)out)[i] = ((const f32x4*)a)[i] + ((const f32x4*)m)[i % inner4];
}

// dst[a][c][b][:] = src[a][b][c][:]  (ewops.h:314-331: [B, L, H, d] <-> [B, H, L, d]); rows of d3 floats stay whole
__global__ __launch_bounds__(256) void transpose_0213_kernel(float* dst, const float* src, uint64_t vecs, uint32_t d1,
                                                             uint32_t d2, uint32_t d3_4) {
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < vecs;
         i += (uint64_t)gridDim.x * blockDim.x) {
        const uint32_t x = (uint32_t)(i % d3_4);
        const uint64_t row = i / d3_4;               // output row (a, c, b)
        const uint32_t b = (uint32_t)(row % d1);
        const uint64_t ac = row / d1;
        const uint32_t c = (uint32_t)(ac % d2);
        const uint64_t a = ac / d2;
        ((f32x4*)dst)[i] = ((const f32x4*)src)[((a * d1 + b) * d2 + c) * d3_4 + x];
    }
}

// out[t][:] = table[ids[t]][:] (+ pos[t % seq_len][:])  (embedding.h:5-12, ewops.h:276-282)
__global__ __launch_bounds__(256) void embedding_kernel(float* out, const float* table, const int32_t* ids,
                                                        const float* pos, uint64_t tokens, uint32_t state4,
                                                        uint32_t seq_len, uint32_t vocab) {
    const uint64_t total = tokens * state4;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t tok = i / state4;
        const uint32_t c = (uint32_t)(i % state4);
        uint32_t id = (uint32_t)ids[tok];
        if (id >= vocab) id = vocab - 1;   // out-of-range ids read the last row instead of faulting
        f32x4 v = ((const f32x4*)table)[(size_t)id * state4 + c];
        if (pos) v += ((const f32x4*)pos)[(size_t)(tok % seq_len) * state4 + c];
        ((f32x4*)out)[i] = v;
    }
}

// Softmax cross-entropy of one row per work-group (ewops.h:233-261 with the one-hot matrix of ewops.h:352-361
// given by its label): loss = log(sum_j exp(x_j)) - x_label, computed relative to the row maximum;
// d (optional) = softmax(x) - onehot.  A label outside [0, vocab) selects no column: loss 0, no -1 in d.
__global__ __launch_bounds__(256) void cross_entropy_kernel(float* row_loss, float* d, const float* logits,
                                                            const int32_t* labels, uint32_t vocab) {
    __shared__ float red[4];
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const size_t row = blockIdx.x;
    const float* x = logits + row * vocab;
    const int32_t label = labels[row];
    const bool hot = label >= 0 && (uint32_t)label < vocab;
    const float x_label = hot ? x[label] : 0.f;   // read before d may overwrite the row in place
    // one pass over the row: running maximum and the sum of exponentials relative to it, four columns per step
    float m = -3.0e38f, sum = 0.f;
    for (uint32_t j0 = t; j0 < vocab; j0 += 1024) {
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = (j0 + 256 * u < vocab) ? x[j0 + 256 * u] : -3.0e38f;
        const float m_new = fmaxf(fmaxf(fmaxf(m, v[0]), fmaxf(v[1], v[2])), v[3]);
        sum *= exp2_fast((m - m_new) * kLog2e);
#pragma unroll
        for (int u = 0; u < 4; ++u) sum += exp2_fast((v[u] - m_new) * kLog2e);
        m = m_new;
    }
    // merge the (maximum, sum) pairs of the 256 threads
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) {
        const float m_o = __shfl_xor(m, s), sum_o = __shfl_xor(sum, s);
        const float m_new = fmaxf(m, m_o);
        sum = sum * exp2_fast((m - m_new) * kLog2e) + sum_o * exp2_fast((m_o - m_new) * kLog2e);
        m = m_new;
    }
    __shared__ float red_sum[4];
    if (lane == 0) { red[wave] = m; red_sum[wave] = sum; }
    __syncthreads();
    m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    sum = 0.f;
#pragma unroll
    for (int w4 = 0; w4 < 4; ++w4) sum += red_sum[w4] * exp2_fast((red[w4] - m) * kLog2e);
    if (t == 0) row_loss[row] = hot ? (m + logf(sum)) - x_label : 0.f;
    if (d) {
        const float inv = 1.0f / sum;
        float* out = d + row * vocab;
        for (uint32_t j = t; j < vocab; j += 256) {
            const float pj = exp2_fast((x[j] - m) * kLog2e) * inv;
            out[j] = (hot && j == (uint32_t)label) ? pj - 1.0f : pj;
        }
    }
}

// out[0] = (sum of in[0..n)) / n by one work-group, in a fixed order: every launch gives the same bits
__global__ __launch_bounds__(1024) void mean_kernel(float* out, const float* in, uint64_t n) {
    __shared__ float red[1024];
    float sum = 0.f;
    for (uint64_t i = threadIdx.x; i < n; i += 1024) sum += in[i];
    red[threadIdx.x] = sum;
    __syncthreads();
    for (uint32_t s = 512; s >= 1; s >>= 1) {
        if (threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = red[0] / (float)n;
}

static inline uint32_t grid_for(uint64_t work_items) {
    const uint64_t blocks = (work_items + 255) / 256;
    return (uint32_t)(blocks < 1 ? 1 : (blocks > 16384 ? 16384 : blocks));
}

static inline int launched() { return launch_status(); }

}  // namespace sfb

using namespace sfb;

extern "C" int sfb_bias_act(sfb_stream_t stream, void* out, int out_dtype, const float* in, const float* bias,
                            const float* residual, int act, uint64_t rows, uint32_t cols) {
    if (!out || !in) return SFB_ERR_NULL_POINTER;
    if (out_dtype != SFB_F32 && out_dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (act != 0 && act != 1) return SFB_ERR_ARGUMENT;
    if (rows == 0 || cols == 0 || (cols & 3u)) return SFB_ERR_SHAPE;
    if (((uintptr_t)out | (uintptr_t)in | (uintptr_t)bias | (uintptr_t)residual) & 15u) return SFB_ERR_ALIGNMENT;
    const uint64_t vecs = rows * (cols / 4);
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
    const dim3 grid(grid_for(vecs));
#define SFB_BA(T, A) bias_act_kernel<T, A><<<grid, 256, 0, s>>>((T*)out, in, bias, residual, vecs, cols / 4)
    if (out_dtype == SFB_F32) { if (act) SFB_BA(float, 1); else SFB_BA(float, 0); }
    else { if (act) SFB_BA(__bf16, 1); else SFB_BA(__bf16, 0); }
#undef SFB_BA
    return launched();
}

extern "C" int sfb_layernorm(sfb_stream_t stream, void* out, int out_dtype, float* mean, float* rstd,
                             const float* in, const float* gain, const float* bias, uint32_t rows,
                             uint32_t state) {
    if (!out || !in || !gain || !bias) return SFB_ERR_NULL_POINTER;
    if (out_dtype != SFB_F32 && out_dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (rows == 0 || state == 0 || (state & 3u)) return SFB_ERR_SHAPE;
    if (((uintptr_t)out | (uintptr_t)in | (uintptr_t)gain | (uintptr_t)bias) & 15u) return SFB_ERR_ALIGNMENT;
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
    const dim3 grid((rows + 3) / 4);
    if (out_dtype == SFB_F32)
        layernorm_kernel<float><<<grid, 256, 0, s>>>((float*)out, mean, rstd, in, gain, bias, rows, state);
    else
        layernorm_kernel<__bf16><<<grid, 256, 0, s>>>((__bf16*)out, mean, rstd, in, gain, bias, rows, state);
    return launched();
}

extern "C" int sfb_bias_residual_layernorm(sfb_stream_t stream, float* out, void* out_bf16, const float* in,
                                          const float* bias, const float* residual, const float* gain,
                                          const float* beta, uint32_t rows, uint32_t state) {
    if (!out || !in || !gain || !beta) return SFB_ERR_NULL_POINTER;
    if (rows == 0 || state == 0 || (state & 3u) || state > 64u * 4u * 8u) return SFB_ERR_SHAPE;
    if (((uintptr_t)out | (uintptr_t)in | (uintptr_t)bias | (uintptr_t)residual | (uintptr_t)gain | (uintptr_t)beta) & 15u)
        return SFB_ERR_ALIGNMENT;
    if ((uintptr_t)out_bf16 & 7u) return SFB_ERR_ALIGNMENT;
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
    const dim3 grid((rows + 3) / 4);
    const uint32_t vecs_per_lane = (state / 4 + 63) / 64;
#define SFB_BRL(V) bias_residual_layernorm_kernel<V><<<grid, 256, 0, s>>>(out, (__bf16*)out_bf16, in, bias, residual, gain, beta, rows, state)
    if (vecs_per_lane <= 1) SFB_BRL(1);
    else if (vecs_per_lane <= 2) SFB_BRL(2);
    else if (vecs_per_lane <= 4) SFB_BRL(4);
    else SFB_BRL(8);
#undef SFB_BRL
    return launched();
}

extern "C" int sfb_add_matrix(sfb_stream_t stream, float* out, const float* a, const float* m, uint32_t dim0,
                              uint64_t inner) {
    if (!out || !a || !m) return SFB_ERR_NULL_POINTER;
    if (dim0 == 0 || inner == 0 || (inner & 3u)) return SFB_ERR_SHAPE;
    if (((uintptr_t)out | (uintptr_t)a | (uintptr_t)m) & 15u) return SFB_ERR_ALIGNMENT;
    const uint64_t vecs = dim0 * (inner / 4);
    clear_stale_error();
    add_matrix_kernel<<<dim3(grid_for(vecs)), 256, 0, (hipStream_t)stream>>>(out, a, m, vecs, inner / 4);
    return launched();
}

extern "C" int sfb_transpose_0213(sfb_stream_t stream, float* dst, const float* src, uint32_t d0, uint32_t d1,
                                  uint32_t d2, uint32_t d3) {
    if (!dst || !src) return SFB_ERR_NULL_POINTER;
    if (d0 == 0 || d1 == 0 || d2 == 0 || d3 == 0 || (d3 & 3u)) return SFB_ERR_SHAPE;
    if (dst == src) return SFB_ERR_ARGUMENT;
    if (((uintptr_t)dst | (uintptr_t)src) & 15u) return SFB_ERR_ALIGNMENT;
    const uint64_t vecs = (uint64_t)d0 * d1 * d2 * (d3 / 4);
    clear_stale_error();
    transpose_0213_kernel<<<dim3(grid_for(vecs)), 256, 0, (hipStream_t)stream>>>(dst, src, vecs, d1, d2, d3 / 4);
    return launched();
}

extern "C" int sfb_embedding_lookup(sfb_stream_t stream, float* out, const float* table, const int32_t* ids,
                                    const float* pos, uint64_t tokens, uint32_t state, uint32_t seq_len,
                                    uint32_t vocab) {
    if (!out || !table || !ids) return SFB_ERR_NULL_POINTER;
    if (tokens == 0 || state == 0 || (state & 3u) || vocab == 0 || (pos && seq_len == 0)) return SFB_ERR_SHAPE;
    if (((uintptr_t)out | (uintptr_t)table | (uintptr_t)pos) & 15u) return SFB_ERR_ALIGNMENT;
    clear_stale_error();
    embedding_kernel<<<dim3(grid_for(tokens * (state / 4))), 256, 0, (hipStream_t)stream>>>(
        out, table, ids, pos, tokens, state / 4, seq_len ? seq_len : 1, vocab);
    return launched();
}

extern "C" int sfb_cast_f32_bf16(sfb_stream_t stream, void* out, const float* in, uint64_t n) {
    if (!out || !in) return SFB_ERR_NULL_POINTER;
    if (n == 0 || (n & 3u)) return SFB_ERR_SHAPE;
    if (((uintptr_t)out & 7u) || ((uintptr_t)in & 15u)) return SFB_ERR_ALIGNMENT;
    clear_stale_error();
    bias_act_kernel<__bf16, 0><<<dim3(grid_for(n / 4)), 256, 0, (hipStream_t)stream>>>(
        (__bf16*)out, in, nullptr, nullptr, n / 4, 1);
    return launched();
}

extern "C" int sfb_softmax_cross_entropy(sfb_stream_t stream, float* loss, float* row_loss, float* d_logits,
                                         const float* logits, const int32_t* labels, uint64_t rows,
                                         uint32_t vocab) {
    if (!loss || !row_loss || !logits || !labels) return SFB_ERR_NULL_POINTER;
    if (rows == 0 || rows > 0x7fffffffull || vocab == 0) return SFB_ERR_SHAPE;
    clear_stale_error();
    cross_entropy_kernel<<<dim3((uint32_t)rows), 256, 0, (hipStream_t)stream>>>(row_loss, d_logits, logits, labels,
                                                                                vocab);
    mean_kernel<<<dim3(1), 1024, 0, (hipStream_t)stream>>>(loss, row_loss, rows);
    return launched();
}
