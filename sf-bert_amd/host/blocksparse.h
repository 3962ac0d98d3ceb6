// The unfused trio and its backward stages with the reference's signatures (blocksparse.h:202, 425, 649-658,
// 965-972, 1164-1173).
#ifndef SFB_HOST_BLOCKSPARSE_H
#define SFB_HOST_BLOCKSPARSE_H

#include "openai_blocksparse.h"

// fp32-output variant of the sdd (blocksparse.h:202 bst_sgemm_nt_float; never called by the reference).
inline bool bst_sgemm_nt_float(CUstream stream, const uint2* lut, const float* a, const float* b, float* c,
                               uint block_size, uint blocks, uint batch_dim, uint ctx_blks_a, uint ctx_blks_b,
                               uint head_dim, uint state_dim, uint lut_heads, uint lut_dim) {
    return sfb_host::ok(sfb_sdd_nt(stream, sfb_host::lut_cast(lut), a, b, c, SFB_F32, SFB_F32, block_size, blocks,
                                   batch_dim, ctx_blks_a, ctx_blks_b, head_dim, state_dim, lut_heads, lut_dim));
}

// T = bhalf or float output; V (the reference's vector type parameter) is accepted and unused.
// lut: NN LUT; mask: ROW-major words (uint32 for block 32, uint64 for block 64) or NULL; x: bf16 scores.
template <typename T, typename V>
bool BlocksparseMaskedSoftmax(CUstream stream, const uint2* lut, const uint* mask, const bhalf* x, T* y,
                              uint block_size, uint blocks, uint batch_dim, uint head_dim, uint ctx_blks,
                              uint lut_heads, uint lut_dim, uint max_lut, uint mask_heads, float scale) {
    return sfb_host::ok(sfb_masked_softmax(stream, sfb_host::lut_cast(lut), mask, x, y, SFB_BF16,
                                           sfb_host::dtype_of<T>::value, nullptr, block_size, blocks, batch_dim,
                                           head_dim, ctx_blks, lut_heads, lut_dim, max_lut, mask_heads, scale));
}

// dx = (dy - sum_k dy*y) * y * scale over each sparse row (blocksparse.h:1164-1173); T = bhalf or float for dy,
// y and dx alike; V is accepted and unused.  lut: NN LUT.
template <typename T, typename V>
bool BlocksparseMaskedSoftmaxGrad(CUstream stream, const uint2* lut, const T* dy, const T* y, T* dx,
                                  uint block_size, uint blocks, uint batch_dim, uint head_dim, uint ctx_blks,
                                  uint lut_heads, uint lut_dim, uint max_lut, float scale) {
    return sfb_host::ok(sfb_masked_softmax_grad(stream, sfb_host::lut_cast(lut), dy, y, dx,
                                                sfb_host::dtype_of<T>::value, block_size, blocks, batch_dim,
                                                head_dim, ctx_blks, lut_heads, lut_dim, max_lut, scale));
}

// a: bf16 sparse operand, b: fp32 dense operand, c: fp32 result.  op = NN_OP with the NN LUT (O = P V, dQ = dS K)
// or TN_OP with the TN LUT (dV = P^T dO, dK = dS^T Q).
inline bool bst_sgemm_xn(CUstream stream, const uint2* lut, const bhalf* a, const float* b, float* c,
                         uint block_size, uint blocks, uint batch_dim, uint ctx_blks_b, uint ctx_blks_c,
                         uint head_dim, uint state_dim, uint lut_heads, uint lut_dim, uint op, uint magic,
                         uint shift, uint max_lut) {
    return sfb_host::ok(sfb_dsd_xn(stream, sfb_host::lut_cast(lut), a, b, c, SFB_BF16, SFB_F32, block_size, blocks,
                                   batch_dim, ctx_blks_b, ctx_blks_c, head_dim, state_dim, lut_heads, lut_dim, op,
                                   magic, shift, max_lut));
}

#endif
