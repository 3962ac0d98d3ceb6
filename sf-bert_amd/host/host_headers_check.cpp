// Syntax check: the host headers are plain C++ and compile without the HIP headers (g++ -fsyntax-only).
#include "blocksparse.h"
#include "device_ops.h"
#include "fusion_blocksparse.h"

bool sfb_host_headers_instantiate(CUstream s, const uint2* lut, const float* a, float* y, bhalf* h, const uint* m,
                                  const uint64* m64) {
    bool ok = bst_sgemm_nt(s, lut, a, a, h, 32, 1, 1, 1, 1, 1, 64, 1, 1);
    ok = ok && BlocksparseMaskedSoftmax<float, float>(s, lut, m, h, y, 32, 1, 1, 1, 1, 1, 2, 1, 1, 0.125f);
    ok = ok && fusion_attention1<float, float>(s, lut, a, a, h, lut, nullptr, nullptr, nullptr, m, nullptr, nullptr, y, 32,
                                               1, 1, 1, 1, 1, 64, 1, 1, 1, 0.125f);
    ok = ok && fusion_attention_local<bhalf, bhalf2>(s, lut, a, a, h, lut, nullptr, nullptr, m, nullptr, nullptr, h, 32, 1,
                                                     1, 1, 1, 1, 64, 1, 1, 1, 0.125f);
    // blocks of 64 keys: one 64-bit mask word per query row and block, as the reference declares it
    ok = ok && fusion_attention2_64<float, float>(s, lut, a, a, h, lut, nullptr, nullptr, m64, nullptr, nullptr, y, 64, 1, 1,
                                                  1, 1, 1, 64, 1, 1, 1, 0.125f);
    ok = ok && layernorm(y, nullptr, nullptr, a, a, a, 1, 1, 64) && gelu(y, a, 1, 1, 64);
    return ok;
}
