// The fused entry points with the reference's signatures (fusion_blocksparse.h:400-416, 1212-1227,
// 1636, 2030, 2456, 2990-3007), forwarding to the C ABI.
//
// fusion_attention1 / 2 / _full / _local / 2_64: sdd + masked softmax -> Y (probabilities, sparse
// layout).  The reference's variants differ only in how work-groups exchange row maxima and sums
// through global scratch; here one work-group owns a block-row, so rblk_flag, rblk_flag1, rblk_lut,
// Max, Sum and the dummy c are accepted and ignored (they may be NULL and need no zeroing).
// fusion_attention: the full fusion, e = V in, f = O out; Y is not written.
// Mask is BLOCK-major (fusion_blocksparse.h:690).  a, b (and e) are fp32 [batch, ctx, heads, state].
#ifndef SFB_HOST_FUSION_BLOCKSPARSE_H
#define SFB_HOST_FUSION_BLOCKSPARSE_H

#include "gpu_types.h"

namespace sfb_host {
template <typename T>
inline bool fused_sdd_softmax(CUstream stream, const uint2* nn_lut, const float* a, const float* b, const void* Mask,
                              T* Y, uint block_size, uint blocks, uint batch_dim, uint ctx_blks_a, uint head_dim,
                              uint state_dim, uint lut_heads, uint lut_dim, uint mask_heads, float scale) {
    // the reference passes the NT LUT length as lut_dim and derives the NN stride itself (:434)
    return ok(sfb_fused_sdd_softmax(stream, lut_cast(nn_lut), a, b, Y, SFB_F32, dtype_of<T>::value, Mask, nullptr,
                                    /*row_order*/ nullptr, block_size, blocks, batch_dim, ctx_blks_a, head_dim, state_dim, lut_heads,
                                    lut_dim + ctx_blks_a, mask_heads, scale));
}
}  // namespace sfb_host

template <typename T, typename V>
bool fusion_attention1(CUstream stream, const uint2* nt_lut, const float* a, const float* b, bhalf* c,
                       const uint2* nn_lut, int* rblk_flag, int* rblk_flag1, uint2* rblk_lut, const uint* Mask,
                       float* Max, float* Sum, T* Y, uint block_size, uint blocks, uint batch_dim, uint ctx_blks_a,
                       uint ctx_blks_b, uint head_dim, uint state_dim, uint lut_heads, uint lut_dim,
                       uint mask_heads, float scale) {
    (void)nt_lut; (void)c; (void)rblk_flag; (void)rblk_flag1; (void)rblk_lut; (void)Max; (void)Sum; (void)ctx_blks_b;
    return sfb_host::fused_sdd_softmax<T>(stream, nn_lut, a, b, Mask, Y, block_size, blocks, batch_dim, ctx_blks_a,
                                          head_dim, state_dim, lut_heads, lut_dim, mask_heads, scale);
}

// MASK: the reference's mask word of the variant (one word per query row and block: uint up to 32 x 32 blocks,
// uint64 for fusion_attention2_64, fusion_blocksparse.h:2465)
#define SFB_FUSION_VARIANT(NAME, MASK)                                                                            \
    template <typename T, typename V>                                                                             \
    bool NAME(CUstream stream, const uint2* nt_lut, const float* a, const float* b, bhalf* c, const uint2* nn_lut, \
              int* rblk_flag, int* rblk_flag1, const MASK* Mask, float* Max, float* Sum, T* Y, uint block_size,    \
              uint blocks, uint batch_dim, uint ctx_blks_a, uint ctx_blks_b, uint head_dim, uint state_dim,        \
              uint lut_heads, uint lut_dim, uint mask_heads, float scale) {                                        \
        (void)nt_lut; (void)c; (void)rblk_flag; (void)rblk_flag1; (void)Max; (void)Sum; (void)ctx_blks_b;          \
        return sfb_host::fused_sdd_softmax<T>(stream, nn_lut, a, b, Mask, Y, block_size, blocks, batch_dim,        \
                                              ctx_blks_a, head_dim, state_dim, lut_heads, lut_dim, mask_heads,     \
                                              scale);                                                              \
    }
SFB_FUSION_VARIANT(fusion_attention2, uint)
SFB_FUSION_VARIANT(fusion_attention_full, uint)
SFB_FUSION_VARIANT(fusion_attention_local, uint)
SFB_FUSION_VARIANT(fusion_attention2_64, uint64)
#undef SFB_FUSION_VARIANT

// Full fusion (fusion_blocksparse.h:2990-3007): O (f) = softmax(scale * a b^T, masked) e.
template <typename T, typename V>
bool fusion_attention(CUstream stream, const uint2* nt_lut, const float* a, const float* b, bhalf* c,
                      const uint2* nn_lut, int* rblk_flag, int* rblk_flag1, const uint* Mask, float* Max, float* Sum,
                      T* Y, float* e, float* f, uint block_size, uint blocks, uint batch_dim, uint ctx_blks_a,
                      uint ctx_blks_b, uint ctx_blks_c, uint head_dim, uint state_dim, uint lut_heads, uint lut_dim,
                      uint mask_heads, float scale, uint max_lut) {
    (void)nt_lut; (void)c; (void)rblk_flag; (void)rblk_flag1; (void)Max; (void)Sum; (void)Y; (void)ctx_blks_b;
    (void)ctx_blks_c; (void)max_lut;
    return sfb_host::ok(sfb_fused_attention(stream, a, b, e, f, SFB_F32, sfb_host::lut_cast(nn_lut), Mask, nullptr,
                                            nullptr, block_size, blocks, batch_dim, ctx_blks_a, head_dim, state_dim,
                                            lut_heads, lut_dim + ctx_blks_a, mask_heads, scale));
}

#endif
