// The encoder-layer ops with the names and argument order of the reference's CPU functions
// (layernorm.h:13, ewops.h:10, 32, 276, 296, embedding.h:5), operating on DEVICE pointers; the GPU
// twins of the reference are launched by hand in transformer_attention_optimize.cu:672-783.  Each takes
// a trailing stream argument (default: the null stream) and returns true on success.
#ifndef SFB_HOST_DEVICE_OPS_H
#define SFB_HOST_DEVICE_OPS_H

#include "gpu_types.h"

inline bool layernorm(float* out, float* mean, float* rstd, const float* input, const float* gain,
                      const float* bias_, int batch_size, int seq_len, int state, CUstream stream = nullptr) {
    return sfb_host::ok(sfb_layernorm(stream, out, SFB_F32, mean, rstd, input, gain, bias_,
                                      (uint32_t)(batch_size * seq_len), (uint32_t)state));
}
inline bool bias(float* output, const float* input, const float* bias_, int n, int m, CUstream stream = nullptr) {
    return sfb_host::ok(sfb_bias_act(stream, output, SFB_F32, input, bias_, nullptr, 0, (uint64_t)m, (uint32_t)n));
}
inline bool gelu(float* C, const float* A, int batch_size, int seq_len, int state, CUstream stream = nullptr) {
    return sfb_host::ok(sfb_bias_act(stream, C, SFB_F32, A, nullptr, nullptr, 1, (uint64_t)batch_size * seq_len,
                                     (uint32_t)state));
}
inline bool tensor_add_tensor(float* C, const float* A, const float* B, int dim_0, int dim_1, int dim_2,
                              CUstream stream = nullptr) {
    return sfb_host::ok(sfb_bias_act(stream, C, SFB_F32, A, nullptr, B, 0, (uint64_t)dim_0 * dim_1, (uint32_t)dim_2));
}
inline bool tensor_add_matrix(float* C, const float* A, const float* B, int dim_0, int dim_1, int dim_2,
                              CUstream stream = nullptr) {
    return sfb_host::ok(sfb_add_matrix(stream, C, A, B, (uint32_t)dim_0, (uint64_t)dim_1 * dim_2));
}
// ewops.h:314-331; the attention launchers take [B, L, H, d] directly, this is for callers that keep [B, H, L, d].
inline bool transpose_0123to0213(const float* src, float* dst, int dim_0, int dim_1, int dim_2, int dim_3,
                                 CUstream stream = nullptr) {
    return sfb_host::ok(sfb_transpose_0213(stream, dst, src, (uint32_t)dim_0, (uint32_t)dim_1, (uint32_t)dim_2,
                                           (uint32_t)dim_3));
}
// vocab bounds the ids (the reference does not check them).
inline bool embedding_lookup(float* C, const float* A, const int* B, int batch_size, int seq_len, int head_num,
                             int size_per_head, int vocab, CUstream stream = nullptr) {
    return sfb_host::ok(sfb_embedding_lookup(stream, C, A, B, nullptr, (uint64_t)batch_size * seq_len,
                                             (uint32_t)(head_num * size_per_head), (uint32_t)seq_len, (uint32_t)vocab));
}

// The loss of ewops.h:233-261 over integer labels (the reference expands them with to_one_hot, ewops.h:352-361,
// and returns the mean on the host).  loss: 1 float, row_loss: batch*seq floats, D: softmax - onehot or NULL; all
// device pointers.
inline bool softmax_cross_entropy_with_logits(float* loss, float* row_loss, float* D, const float* A, const int* labels,
                                              int batch_size, int seq_len, int vocab_size, CUstream stream = nullptr) {
    return sfb_host::ok(sfb_softmax_cross_entropy(stream, loss, row_loss, D, A, labels,
                                                  (uint64_t)batch_size * seq_len, (uint32_t)vocab_size));
}

#endif
