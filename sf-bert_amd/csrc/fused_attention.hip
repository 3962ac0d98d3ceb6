// Fully fused block-sparse attention for gfx950 (MI355X).
//
// One work-group owns one (batch, head, block-row) of BS queries and walks the key blocks that the
// NN look-up table lists for that row.  Each wave owns 32 queries.  Per key block it
//   1. computes the transposed score tile  S^T = K_blk . Q^T  on MFMA (A = K from LDS, B = Q kept in
//      registers for the whole row), so that every lane ends up with keys of ONE query: the row
//      maximum / sum need only lane-local work plus one exchange between lane l and lane l+32;
//   2. does the scaled, masked online softmax on the accumulators (exp2 with log2(e) folded in);
//   3. feeds the probabilities, still in registers, as the B operand of  O^T += V_blk^T . P^T.
//      The accumulator layout of step 1 is exactly the B-operand layout of step 3 once V^T is laid
//      out in LDS with its keys permuted the same way, so P never moves between lanes.
// O is normalised and written once at the end; S and P never exist in memory; no flags, no
// inter-work-group communication.
//
// Arithmetic follows the reference CPU path: scores are raw dot products, the maximum is taken over
// kept keys with seed -1000000 (ewops.h:70), p = exp((s-max)*scale) (ewops.h:86), the row is divided
// by sum + 1e-6 (ewops.h:93), and O = P.V (matmul.h:6-20).
#include "common.hip.h"

namespace sfb {

struct FusedParams {
    const void* q;
    const void* k;
    const void* v;
    float* o;
    const sfb_uint2* nn_lut;
    const void* mask;           // block-major keep words, or nullptr
    const int32_t* valid_len;   // per batch, or nullptr
    const uint32_t* row_order;  // rank -> block-row, or nullptr
    uint32_t batch, heads, nb, blocks;
    uint32_t lut_stride;   // entries between heads' LUTs (0 = shared)
    uint32_t mask_stride;  // words between heads' masks (0 = shared)
    uint32_t groups;       // ceil(batch*heads / 8)
    float scale_log2e;
    float slack;           // raw-score distance a block maximum may exceed the reference maximum
};

// Keep-bits of one lane's query row for one key block, with key padding folded in.
template <int BS>
__device__ __forceinline__ uint64_t load_keep_word(const void* mask, size_t word_index, int limit) {
    uint64_t w = ~0ull;
    if (mask) {
        if (BS == 64) w = ((const uint64_t*)mask)[word_index];
        else w = ((const uint32_t*)mask)[word_index];
    }
    if (limit < BS) w &= (limit <= 0) ? 0ull : ((1ull << limit) - 1ull);
    return w;
}

// Online-softmax step on one key block.  s[kt][i] holds, for this lane's query, the raw score of key
//   kt*32 + (i/4)*8 + half*4 + i%4      (half = lane / 32)
// and is overwritten by the unnormalised probability (PACK: pk[kt*8 + i/2] receives the pair
// (i, i+1) rounded to bf16, and the row sum is taken over those rounded values, i.e. over exactly
// what the P.V product uses).
//
// The probabilities are taken relative to a reference maximum m_used that is only moved when a
// block's maximum exceeds it by more than `slack` (raw-score units; 2^8 in probability), so the
// rescaling of the output accumulators is rare.  m_true tracks the exact running maximum; the final
// normalisation uses both, which keeps the result identical to softmax relative to the true maximum
// including the +1e-6 term of the denominator.
struct RowState {
    float m_used;   // reference maximum the stored probabilities are relative to (raw units)
    float m_true;   // exact running maximum over kept keys, seeded like the CPU path
    float l;        // this lane's partial sum of probabilities relative to m_used
};

template <int KT, int NO, bool PACK>
__device__ __forceinline__ void softmax_block(f32x16 (&s)[KT], uint32_t (&pk)[KT * 8], f32x16 (&o)[NO],
                                              RowState& st, float c, float slack, bool masked,
                                              uint64_t keep, uint32_t half) {
    if (masked) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            uint32_t w = (uint32_t)(keep >> (kt * 32)) >> (half * 4);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t bit = (i / 4) * 8 + (i % 4);
                s[kt][i] = ((w >> bit) & 1u) ? s[kt][i] : kMaskedScore;
            }
        }
    }
    float mx0 = s[0][0], mx1 = s[0][1];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int i = 0; i < 16; i += 4) {
            mx0 = fmaxf(fmaxf(mx0, s[kt][i]), s[kt][i + 1]);
            mx1 = fmaxf(fmaxf(mx1, s[kt][i + 2]), s[kt][i + 3]);
        }
    }
    float mloc = fmaxf(mx0, mx1);
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32));
    st.m_true = fmaxf(st.m_true, mloc);
    if (__builtin_amdgcn_ballot_w64(mloc > st.m_used + slack) != 0) {
        const float m_new = fmaxf(st.m_used, mloc);
        const float alpha = exp2_fast((st.m_used - m_new) * c);
        st.m_used = m_new;
        st.l *= alpha;
#pragma unroll
        for (int n = 0; n < NO; ++n) o[n] *= alpha;
    }
    const float mc = st.m_used * c;
    float sum0 = 0.f, sum1 = 0.f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int i = 0; i < 16; i += 4) {
            const float p0 = exp2_fast(__builtin_fmaf(s[kt][i + 0], c, -mc));
            const float p1 = exp2_fast(__builtin_fmaf(s[kt][i + 1], c, -mc));
            const float p2 = exp2_fast(__builtin_fmaf(s[kt][i + 2], c, -mc));
            const float p3 = exp2_fast(__builtin_fmaf(s[kt][i + 3], c, -mc));
            if (PACK) {
                const uint32_t a = pack_bf16(p0, p1), b = pack_bf16(p2, p3);
                pk[kt * 8 + i / 2] = a;
                pk[kt * 8 + i / 2 + 1] = b;
                sum0 = dot2_bf16_ones(a, sum0);
                sum1 = dot2_bf16_ones(b, sum1);
            } else {
                s[kt][i + 0] = p0; s[kt][i + 1] = p1; s[kt][i + 2] = p2; s[kt][i + 3] = p3;
                sum0 += p0 + p1;
                sum1 += p2 + p3;
            }
        }
    }
    st.l += sum0 + sum1;
}

// Normalise and store this lane's part of O: o[mt][i] is output column mt*32 + (i/4)*8 + half*4 + i%4.
template <int NO>
__device__ __forceinline__ void store_output(float* o_row, f32x16 (&o)[NO], const RowState& st, float c,
                                             uint32_t half) {
    // sum relative to the true maximum = total / f with f = 2^((m_true - m_used) c); hence
    // O = acc / (total + 1e-6 f)  (ewops.h:93 divides by sum + 1e-6).
    const float total = st.l + __shfl_xor(st.l, 32);
    const float f = exp2_fast((st.m_true - st.m_used) * c);
    const float inv = 1.0f / (total + 1e-6f * f);
#pragma unroll
    for (int mt = 0; mt < NO; ++mt) {
#pragma unroll
        for (int ig = 0; ig < 4; ++ig) {
            f32x4 out = {o[mt][ig * 4 + 0] * inv, o[mt][ig * 4 + 1] * inv, o[mt][ig * 4 + 2] * inv,
                         o[mt][ig * 4 + 3] * inv};
            *(f32x4*)(o_row + mt * 32 + ig * 8 + half * 4) = out;
        }
    }
}

// ------------------------------------------------------------------------------------------------
// bf16 inputs, fp32 accumulation: v_mfma_f32_32x32x16_bf16
// ------------------------------------------------------------------------------------------------
//
// LDS per buffer: K tile [BS keys][D + 8] bf16 (row-major, 16 B pad -> conflict-free 128-bit reads),
//                 V^T tile [D][BS + 8] bf16 with the 4-key groups of a row stored in the order the
//                 P^T operand needs: group g = 4u + 2a + hf sits at byte (2u + hf)*16 + a*8.
// Two buffers, one barrier per key block: block j+1 is fetched into registers while block j is
// multiplied, written to the other buffer afterwards.
template <int BS, int D>
__global__ __launch_bounds__(BS * 2, 2) void fused_attention_bf16_kernel(FusedParams p) {
    constexpr int NT = BS * 2;
    constexpr int KT = BS / 32;      // 32-key tiles per block
    constexpr int NO = D / 32;       // 32-column tiles of O
    constexpr int KS = D / 16;       // MFMA k-steps over the head dimension
    constexpr int PU = BS / 16;      // MFMA k-steps over the keys of a block
    constexpr int K_STRIDE = (D + 8) * 2;   // bytes
    constexpr int V_STRIDE = (BS + 8) * 2;  // bytes
    constexpr int K_BYTES = BS * K_STRIDE;
    constexpr int V_BYTES = D * V_STRIDE;
    constexpr int K_CHUNKS = D / 16;  // 16-byte chunks of K per thread per block
    constexpr int V_ITEMS = (D + 63) / 64;  // (4 keys x 8 columns) items of V per thread per block
    static_assert(D % 64 == 0, "head state must be a multiple of 64");

    __shared__ __attribute__((aligned(16))) uint8_t smem[2 * (K_BYTES + V_BYTES)];

    const WorkId work = decode_work(blockIdx.x, p.batch * p.heads, p.groups);
    if (!work.valid) return;
    const uint32_t b = work.bh / p.heads, h = work.bh % p.heads;
    const uint32_t r = p.row_order ? p.row_order[work.rank] : (p.nb - 1 - work.rank);
    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint32_t qn = lane & 31, half = lane >> 5;

    const sfb_uint2* lut = p.nn_lut + (size_t)h * p.lut_stride;
    const uint32_t lut_off = lut[r].x, count = lut[r].y;
    const uint32_t q_token = r * BS + wave * 32 + qn;
    float* o_row = p.o + token_offset(b, q_token, h, L, p.heads, D);

    if (count == 0) {
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int x = 0; x < D / 8; ++x) *(f32x4*)(o_row + half * (D / 2) + x * 4) = zero;
        return;
    }

    const __bf16* Q = (const __bf16*)p.q;
    const __bf16* K = (const __bf16*)p.k;
    const __bf16* V = (const __bf16*)p.v;
    const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
    const int valid = p.valid_len ? p.valid_len[b] : (int)L;

    // Q^T operand: k-slot (ks, half, j) is head-dimension index (2ks + half)*8 + j.
    bf16x8 qf[KS];
    {
        const __bf16* q_row = Q + token_offset(b, q_token, h, L, p.heads, D);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[ks] = *(const bf16x8*)(q_row + (2 * ks + half) * 8);
    }

    u32x4 gk[K_CHUNKS];
    u32x4 gv[V_ITEMS][4];

    auto fetch = [&](uint32_t col) {
        const size_t base = token_offset(b, col * BS, h, L, p.heads, D);
        const size_t row_stride = (size_t)p.heads * D;
#pragma unroll
        for (int i = 0; i < K_CHUNKS; ++i) {
            const uint32_t cid = i * NT + t, row = cid / (D / 8), c = cid % (D / 8);
            gk[i] = *(const u32x4*)(K + base + row * row_stride + c * 8);
        }
#pragma unroll
        for (int ii = 0; ii < V_ITEMS; ++ii) {
            const uint32_t id = ii * NT + t, g = id % (BS / 4), c = id / (BS / 4);
            if (c < D / 8) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    gv[ii][e] = *(const u32x4*)(V + base + (4 * g + e) * row_stride + c * 8);
            }
        }
    };

    auto stage = [&](uint32_t buf) {
        uint8_t* k_lds = smem + buf * (K_BYTES + V_BYTES);
        uint8_t* v_lds = k_lds + K_BYTES;
#pragma unroll
        for (int i = 0; i < K_CHUNKS; ++i) {
            const uint32_t cid = i * NT + t, row = cid / (D / 8), c = cid % (D / 8);
            *(u32x4*)(k_lds + row * K_STRIDE + c * 16) = gk[i];
        }
#pragma unroll
        for (int ii = 0; ii < V_ITEMS; ++ii) {
            const uint32_t id = ii * NT + t, g = id % (BS / 4), c = id / (BS / 4);
            if (c < D / 8) {
                const uint32_t pos = (2 * (g / 4) + (g & 1)) * 16 + ((g & 3) >> 1) * 8;
#pragma unroll
                for (int dd = 0; dd < 8; ++dd) {
                    const uint32_t x0 = gv[ii][0][dd / 2], x1 = gv[ii][1][dd / 2];
                    const uint32_t x2 = gv[ii][2][dd / 2], x3 = gv[ii][3][dd / 2];
                    u32x2 out;
                    if (dd & 1) {
                        out.x = (x0 >> 16) | (x1 & 0xffff0000u);
                        out.y = (x2 >> 16) | (x3 & 0xffff0000u);
                    } else {
                        out.x = (x0 & 0xffffu) | (x1 << 16);
                        out.y = (x2 & 0xffffu) | (x3 << 16);
                    }
                    *(u32x2*)(v_lds + (c * 8 + dd) * V_STRIDE + pos) = out;
                }
            }
        }
    };

    f32x16 o_acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[n][i] = 0.f;
    RowState st = {kMaxSeed, kMaxSeed, 0.f};
    const float c = p.scale_log2e, slack = p.slack;

    sfb_uint2 entry = lut[lut_off];
    fetch(entry.y);
    stage(0);
    __syncthreads();

    for (uint32_t j = 0; j < count; ++j) {
        const uint32_t cur = j & 1;
        const sfb_uint2 here = entry;
        const bool more = (j + 1 < count);
        if (more) {
            entry = lut[lut_off + j + 1];
            fetch(entry.y);
        }
        const uint8_t* k_lds = smem + cur * (K_BYTES + V_BYTES);
        const uint8_t* v_lds = k_lds + K_BYTES;

        // S^T = K . Q^T
        f32x16 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s[kt][i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8 a = *(const bf16x8*)(k_lds + (kt * 32 + qn) * K_STRIDE + (2 * ks + half) * 16);
                s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s[kt], 0, 0, 0);
            }
        }

        const int limit = valid - (int)(here.y * BS);
        const bool masked = (mask != nullptr) || (limit < BS);
        uint64_t keep = ~0ull;
        if (masked) keep = load_keep_word<BS>(mask, (size_t)here.x * BS + wave * 32 + qn, limit);
        uint32_t pk[KT * 8];
        softmax_block<KT, NO, true>(s, pk, o_acc, st, c, slack, masked, keep, half);

        // O^T += V^T . P^T
#pragma unroll
        for (int u = 0; u < PU; ++u) {
            const u32x4 pb = {pk[u * 4 + 0], pk[u * 4 + 1], pk[u * 4 + 2], pk[u * 4 + 3]};
            const bf16x8 bfrag = __builtin_bit_cast(bf16x8, pb);
#pragma unroll
            for (int mt = 0; mt < NO; ++mt) {
                const bf16x8 a = *(const bf16x8*)(v_lds + (mt * 32 + qn) * V_STRIDE + (2 * u + half) * 16);
                o_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, bfrag, o_acc[mt], 0, 0, 0);
            }
        }

        if (more) stage(cur ^ 1);
        __syncthreads();
    }

    store_output<NO>(o_row, o_acc, st, c, half);
}

// ------------------------------------------------------------------------------------------------
// fp32 inputs: v_mfma_f32_32x32x2_f32 (true fp32 products and accumulation)
// ------------------------------------------------------------------------------------------------
//
// LDS: K tile [BS][D + 4] fp32, V tile [BS][D + 8] fp32, one buffer; the next block waits in
// registers.  k-slot (step, half) of the score MFMA is head-dimension index 8*(step/4) + 4*half +
// step%4, so one 128-bit LDS read feeds four MFMA steps.  The P.V product needs no transposition in
// fp32: MFMA step (kt, i) consumes key kt*32 + (i/4)*8 + half*4 + i%4, whose V row is read as 32
// consecutive floats.
template <int BS, int D>
__global__ __launch_bounds__(BS * 2, 2) void fused_attention_f32_kernel(FusedParams p) {
    constexpr int NT = BS * 2;
    constexpr int KT = BS / 32;
    constexpr int NO = D / 32;
    constexpr int QG = D / 8;               // float4 groups of Q per lane
    constexpr int K_STRIDE = D + 4;         // floats
    constexpr int V_STRIDE = D + 8;         // floats
    constexpr int CHUNKS = D / 8;           // float4 chunks per thread per tile
    static_assert(D % 32 == 0, "head state must be a multiple of 32");

    __shared__ __attribute__((aligned(16))) float k_lds[BS * K_STRIDE];
    __shared__ __attribute__((aligned(16))) float v_lds[BS * V_STRIDE];

    const WorkId work = decode_work(blockIdx.x, p.batch * p.heads, p.groups);
    if (!work.valid) return;
    const uint32_t b = work.bh / p.heads, h = work.bh % p.heads;
    const uint32_t r = p.row_order ? p.row_order[work.rank] : (p.nb - 1 - work.rank);
    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint32_t qn = lane & 31, half = lane >> 5;

    const sfb_uint2* lut = p.nn_lut + (size_t)h * p.lut_stride;
    const uint32_t lut_off = lut[r].x, count = lut[r].y;
    const uint32_t q_token = r * BS + wave * 32 + qn;
    float* o_row = p.o + token_offset(b, q_token, h, L, p.heads, D);

    if (count == 0) {
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int x = 0; x < D / 8; ++x) *(f32x4*)(o_row + half * (D / 2) + x * 4) = zero;
        return;
    }

    const float* Q = (const float*)p.q;
    const float* K = (const float*)p.k;
    const float* V = (const float*)p.v;
    const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
    const int valid = p.valid_len ? p.valid_len[b] : (int)L;

    f32x4 qf[QG];
    {
        const float* q_row = Q + token_offset(b, q_token, h, L, p.heads, D);
#pragma unroll
        for (int g = 0; g < QG; ++g) qf[g] = *(const f32x4*)(q_row + 8 * g + 4 * half);
    }

    f32x4 gk[CHUNKS], gv[CHUNKS];
    auto fetch = [&](uint32_t col) {
        const size_t base = token_offset(b, col * BS, h, L, p.heads, D);
        const size_t row_stride = (size_t)p.heads * D;
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
            const uint32_t cid = i * NT + t, row = cid / (D / 4), cc = cid % (D / 4);
            gk[i] = *(const f32x4*)(K + base + row * row_stride + cc * 4);
            gv[i] = *(const f32x4*)(V + base + row * row_stride + cc * 4);
        }
    };
    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
            const uint32_t cid = i * NT + t, row = cid / (D / 4), cc = cid % (D / 4);
            *(f32x4*)(k_lds + row * K_STRIDE + cc * 4) = gk[i];
            *(f32x4*)(v_lds + row * V_STRIDE + cc * 4) = gv[i];
        }
    };

    f32x16 o_acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[n][i] = 0.f;
    RowState st = {kMaxSeed, kMaxSeed, 0.f};
    const float c = p.scale_log2e, slack = p.slack;

    sfb_uint2 entry = lut[lut_off];
    fetch(entry.y);

    for (uint32_t j = 0; j < count; ++j) {
        const sfb_uint2 here = entry;
        stage();
        __syncthreads();
        if (j + 1 < count) {
            entry = lut[lut_off + j + 1];
            fetch(entry.y);
        }

        f32x16 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s[kt][i] = 0.f;
#pragma unroll
            for (int g = 0; g < QG; ++g) {
                const f32x4 a = *(const f32x4*)(k_lds + (kt * 32 + qn) * K_STRIDE + 8 * g + 4 * half);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    s[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], qf[g][e], s[kt], 0, 0, 0);
            }
        }

        const int limit = valid - (int)(here.y * BS);
        const bool masked = (mask != nullptr) || (limit < BS);
        uint64_t keep = ~0ull;
        if (masked) keep = load_keep_word<BS>(mask, (size_t)here.x * BS + wave * 32 + qn, limit);
        uint32_t pk_unused[KT * 8];
        softmax_block<KT, NO, false>(s, pk_unused, o_acc, st, c, slack, masked, keep, half);

#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t key = kt * 32 + (i / 4) * 8 + half * 4 + (i % 4);
#pragma unroll
                for (int mt = 0; mt < NO; ++mt) {
                    const float a = v_lds[key * V_STRIDE + mt * 32 + qn];
                    o_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[kt][i], o_acc[mt], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }

    store_output<NO>(o_row, o_acc, st, c, half);
}

template <int BS, int D>
static int launch_fused(hipStream_t stream, const FusedParams& p, int in_dtype) {
    const uint32_t grid = p.groups * 8u * p.nb;
    if (in_dtype == SFB_BF16)
        fused_attention_bf16_kernel<BS, D><<<dim3(grid), dim3(BS * 2), 0, stream>>>(p);
    else
        fused_attention_f32_kernel<BS, D><<<dim3(grid), dim3(BS * 2), 0, stream>>>(p);
    return hipGetLastError() == hipSuccess ? SFB_OK : SFB_ERR_LAUNCH;
}

}  // namespace sfb

extern "C" int sfb_fused_attention(sfb_stream_t stream, const void* q, const void* k, const void* v,
                                   float* o, int in_dtype, const sfb_uint2* nn_lut, const void* mask,
                                   const int32_t* valid_len, const uint32_t* row_order,
                                   uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                   uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                   uint32_t lut_heads, uint32_t lut_dim, uint32_t mask_heads,
                                   float scale) {
    using namespace sfb;
    if (!q || !k || !v || !o || !nn_lut) return SFB_ERR_NULL_POINTER;
    if (in_dtype != SFB_F32 && in_dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (state_dim != 64) return SFB_ERR_HEAD_STATE;
    if (!(scale > 0.f) || !(scale < 3.0e38f)) return SFB_ERR_ARGUMENT;
    if (batch_dim == 0 || ctx_blks == 0 || head_dim == 0 || lut_heads == 0 || mask_heads == 0)
        return SFB_ERR_SHAPE;
    if (lut_heads > 1 && (lut_heads != head_dim || lut_dim != ctx_blks + blocks)) return SFB_ERR_SHAPE;
    if (mask_heads > 1 && mask_heads != head_dim) return SFB_ERR_SHAPE;
    if ((uint64_t)batch_dim * head_dim * ctx_blks > 0x7fffffffull / 8) return SFB_ERR_SHAPE;
    const uintptr_t align = (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o;
    if (align & 15u) return SFB_ERR_ALIGNMENT;

    FusedParams p;
    p.q = q; p.k = k; p.v = v; p.o = o;
    p.nn_lut = nn_lut; p.mask = mask; p.valid_len = valid_len; p.row_order = row_order;
    p.batch = batch_dim; p.heads = head_dim; p.nb = ctx_blks; p.blocks = blocks;
    p.lut_stride = lut_heads > 1 ? lut_dim : 0;
    p.mask_stride = mask_heads > 1 ? blocks * block_size : 0;
    p.groups = bh_groups(batch_dim * head_dim);
    p.scale_log2e = scale * kLog2e;
    p.slack = kLazyRescaleLog2 / p.scale_log2e;
    hipStream_t s = (hipStream_t)stream;
    if (block_size == 64) return launch_fused<64, 64>(s, p, in_dtype);
    return launch_fused<32, 64>(s, p, in_dtype);
}
