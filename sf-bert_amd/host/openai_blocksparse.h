// bst_sgemm_nt with the reference's signature (openai_blocksparse.h:202-209), forwarding to the C ABI.
// a, b: fp32 [batch, ctx, heads, state]; c: bf16 sparse [batch][heads][blocks][bs][bs].
// Differences from the reference: block sizes 32 AND 64 are implemented, and an unsupported block
// size returns false (status in sfb_host::last_status()) instead of silently doing nothing
// (openai_blocksparse.h:225-232).
#ifndef SFB_HOST_OPENAI_BLOCKSPARSE_H
#define SFB_HOST_OPENAI_BLOCKSPARSE_H

#include "gpu_types.h"

inline bool bst_sgemm_nt(CUstream stream, const uint2* lut, const float* a, const float* b, bhalf* c,
                         uint block_size, uint blocks, uint batch_dim, uint ctx_blks_a, uint ctx_blks_b,
                         uint head_dim, uint state_dim, uint lut_heads, uint lut_dim) {
    return sfb_host::ok(sfb_sdd_nt(stream, sfb_host::lut_cast(lut), a, b, c, SFB_F32, SFB_BF16, block_size,
                                   blocks, batch_dim, ctx_blks_a, ctx_blks_b, head_dim, state_dim, lut_heads,
                                   lut_dim));
}

#endif
