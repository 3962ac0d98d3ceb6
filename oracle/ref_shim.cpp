// Build recipe input for oracle/_ref/libsfbert_ref.so -- TEST INFRASTRUCTURE ONLY.
//
// This translation unit contains no reference code.  It includes the reference's CPU headers where
// they lie (the Makefile passes -I$(REFERENCE)) and exports C symbols around the functions the
// oracle restates, so tests can bit-compare the restatement with the reference's own arithmetic.
// It is compiled only where the reference checkout exists; the resulting library is git-ignored.
#include "matmul.h"      // multiheadmatmulNT / multiheadmatmulNN / multiheadmatmulTN
#include "ewops.h"       // softmax, softmax_grad, bias, gelu, tensor_add_*, transpose_0123to0213
#include "layernorm.h"   // layernorm
#include "embedding.h"   // embedding_lookup

extern "C" {

void ref_multiheadmatmulNT(float* C, float* A, float* B, int batch, int heads, int mA, int nA, int mB) {
    multiheadmatmulNT<float, float, float>(C, A, B, batch, heads, mA, nA, mB);
}
void ref_multiheadmatmulNN(float* C, float* A, float* B, int batch, int heads, int mA, int nA, int nB) {
    multiheadmatmulNN<float, float, float>(C, A, B, batch, heads, mA, nA, nB);
}
void ref_softmax(float* C, float* A, float scaler, int seq_len, int batch, int heads) {
    softmax<float, float>(C, A, scaler, seq_len, batch, heads);
}
void ref_softmax_grad(float* out, float* dy, float* y, float scaler, int batch, int heads, int seq_len) {
    softmax_grad<float, float, float>(out, dy, y, scaler, batch, heads, seq_len);
}
void ref_multiheadmatmulTN(float* C, float* A, float* B, int batch, int heads, int mA, int nA, int nB) {
    multiheadmatmulTN<float, float, float>(C, A, B, batch, heads, mA, nA, nB);
}
void ref_transpose_0123to0213(float* src, float* dst, int d0, int d1, int d2, int d3) {
    transpose_0123to0213(src, dst, d0, d1, d2, d3);
}
void ref_layernorm(float* out, float* mean, float* rstd, const float* in, const float* gain,
                   const float* bias_, int batch, int seq_len, int state) {
    layernorm(out, mean, rstd, in, gain, bias_, batch, seq_len, state);
}
void ref_gelu(float* C, float* A, int batch, int seq_len, int state) { gelu(C, A, batch, seq_len, state); }
void ref_bias(float* out, const float* in, const float* b, int n, int m) { bias(out, in, b, n, m); }
void ref_tensor_add_tensor(float* C, float* A, float* B, int d0, int d1, int d2) {
    tensor_add_tensor(C, A, B, d0, d1, d2);
}
void ref_tensor_add_matrix(float* C, float* A, float* B, int d0, int d1, int d2) {
    tensor_add_matrix(C, A, B, d0, d1, d2);
}
void ref_embedding_lookup(float* C, float* A, int* B, int batch, int seq_len, int heads, int size_per_head) {
    embedding_lookup(C, A, B, batch, seq_len, heads, size_per_head);
}

// labels -> one-hot (to_one_hot), then the loss; logits are overwritten by their logarithms as in the reference
float ref_softmax_cross_entropy(float* D, float* logits, int* labels, int* one_hot_scratch, int batch, int seq_len,
                                int vocab) {
    to_one_hot(one_hot_scratch, labels, batch, seq_len, vocab);
    return softmax_cross_entropy_with_logits(D, logits, one_hot_scratch, batch, seq_len, vocab);
}

}  // extern "C"
