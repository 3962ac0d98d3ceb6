// Fused backward of the block-sparse attention: dQ, dK, dV from Q, K, V, dO, the forward output O and the
// forward's row statistics, without P, dP or dS ever reaching memory.  The reference's backward is the unfused
// sequence TN, NT, softmax gradient, TN, NN over sparse tensors in memory
// (transformer_attention_optimize.cu:924-965); the arithmetic here is the same (ewops.h:101-124, matmul.h:81-99):
//     P  = exp2(S c - lse)                  S = Q K^T, lse from the forward (sfb_fused_attention_scheduled_lse)
//     dV = P^T dO      dP = dO V^T      dS = P (dP - delta) scale      dK = dS^T Q      dQ = dS K
// with delta_q = sum_d dO_qd O_qd in place of the gradient's sum over the sparse row (equal, since O = P V).
//
// Two kernels, both with the tile machinery of the forward kernel (LDS-direct loads into swizzled tiles, see
// Bf16DirectTiles; k_frag reads a tile row-wise, v_frag reads it transposed):
//   * dq kernel, one work-group per (batch, head, block-row), a lane owns one query: per key block
//         S^T = K Q^T, dP^T = V dO^T (row-wise reads of the K and V tiles), dS^T lane-local,
//         dQ^T += K^T dS^T (transposed read of the K tile);
//   * dkdv kernel, one work-group per (batch, head, key-block column), a lane owns one key: per query block
//         S = Q K^T, dP = dO V^T (row-wise reads of the Q and dO tiles; lse and delta per accumulator element),
//         dV^T += dO^T P, dK^T += Q^T dS (transposed reads of the dO and Q tiles).
// bf16 or fp32 tensors (the latter with true fp32 products, further down), head sizes 32 / 64 / 96 / 128 and, through
// the RAGGED forms of the same kernels, every multiple of 8 (bf16) or 4 (fp32) between them, block
// size 32 or 64; fp32 accumulation and fp32 gradients.
#include "tiles.hip.h"

namespace sfb {

struct BackwardParams {
    const void* q;
    const void* k;
    const void* v;
    const void* d_out;
    const float* lse;           // [batch][heads][ctx]
    const float* delta;         // [batch][heads][ctx]
    float* dq;
    float* dk;
    float* dv;
    const sfb_uint2* nn_lut;
    const sfb_uint2* tn_lut;
    const void* mask;           // block-major keep words, or nullptr
    const int32_t* valid_len;
    const sfb_work_item* items; // rank -> chunk of a block-row (dq) / block-column (dkdv), or nullptr: whole rows
    float* partials;            // partial results of split rows / columns, or nullptr
    uint32_t ranks, heavy, n_parts;
    uint32_t batch, heads, nb, blocks, mask_stride;
    uint32_t state;             // head size of the tensors (the kernels' D is the next multiple of 32)
    uint32_t lut_stride;        // entries between the tables of consecutive heads, 0: one table for all
    float scale, scale_log2e;
};

// What a work-group does: key (query) blocks [first, first + count) of the LUT segment of block-row (column)
// `line`; the result goes to the output rows, or, for a chunk of a split line, to partial record `slot`.
struct LineWork {
    uint32_t bh, line, first, count;
    int32_t slot;   // -1: write the output directly
    bool valid;
};
__device__ __forceinline__ LineWork decode_line_work(const BackwardParams& p, const sfb_uint2* lut, uint32_t wg) {
    const WorkId id = decode_work(wg, p.batch * p.heads, p.ranks, p.heavy);
    LineWork w;
    w.valid = id.valid;
    w.bh = id.bh;
    w.slot = -1;
    if (p.items) {
        const sfb_work_item it = p.items[id.rank];
        w.line = it.row;
        w.first = it.lut_first;
        w.count = it.count;
        if (it.nchunks > 1) w.slot = (int32_t)(it.part + it.chunk);
    } else {
        const sfb_uint2* mine = lut + (size_t)(id.valid ? id.bh % p.heads : 0u) * p.lut_stride;
        w.line = id.rank;
        w.first = mine[id.valid ? id.rank : 0u].x;
        w.count = id.valid ? mine[id.rank].y : 0u;
    }
    return w;
}

// acc element i of tile kt <-> index kt*32 + (i/4)*8 + half*4 + i%4 along the block; chunk u (16 indices) of the
// packed bf16 operand takes elements i0 .. i0+7 of tile u/2 with i0 = (u%2)*8
template <int KT>
__device__ __forceinline__ void pack_chunks(uint32_t (&pk)[KT * 8], const f32x16 (&x)[KT]) {
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; i += 2) pk[kt * 8 + i / 2] = pack_bf16(x[kt][i], x[kt][i + 1]);
}

template <int NO>
__device__ __forceinline__ void store_rows_f32(float* row, const f32x16 (&acc)[NO], uint32_t half) {
#pragma unroll
    for (int mt = 0; mt < NO; ++mt)
#pragma unroll
        for (int ig = 0; ig < 4; ++ig) {
            const f32x4 out = {acc[mt][ig * 4 + 0], acc[mt][ig * 4 + 1], acc[mt][ig * 4 + 2], acc[mt][ig * 4 + 3]};
            *(f32x4*)(row + mt * 32 + ig * 8 + half * 4) = out;
        }
}

// rows of hd < NO * 32 floats (hd a multiple of 4): the columns beyond hd are dropped
template <int NO>
__device__ __forceinline__ void store_rows_f32_ragged(float* row, const f32x16 (&acc)[NO], uint32_t half, uint32_t hd) {
#pragma unroll
    for (int mt = 0; mt < NO; ++mt)
#pragma unroll
        for (int ig = 0; ig < 4; ++ig) {
            const f32x4 out = {acc[mt][ig * 4 + 0], acc[mt][ig * 4 + 1], acc[mt][ig * 4 + 2], acc[mt][ig * 4 + 3]};
            if (mt * 32 + ig * 8 + half * 4 < hd) *(f32x4*)(row + mt * 32 + ig * 8 + half * 4) = out;
        }
}

// The same rows to an output tensor through a wave-private LDS slab (32 rows of D floats + 16 bytes each), so that
// memory sees whole 256-byte rows as streaming stores instead of 32-byte pieces of 32 rows per instruction: the
// gradients are written once and read by nobody in this launch.  my_row: this lane's row; row_floats: distance
// between the rows of consecutive tokens.
template <int NO>
__device__ __forceinline__ void store_rows_slab(float* my_row, uint32_t row_floats, const f32x16 (&acc)[NO],
                                                uint32_t lane, uint8_t* slab) {
    constexpr int D = NO * 32, PITCH = D * 4 + 16, CHUNKS = D / 4;
    const uint32_t qn = lane & 31, half = lane >> 5;
    store_rows_f32<NO>((float*)(slab + qn * PITCH), acc, half);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    float* const wave_rows = my_row - (size_t)qn * row_floats;
#pragma unroll
    for (int pass = 0; pass < CHUNKS / 2; ++pass) {
        const uint32_t idx = pass * 64 + lane, row = idx / CHUNKS, ch = idx % CHUNKS;
        __builtin_nontemporal_store(*(const f32x4*)(slab + row * PITCH + ch * 16),
                                    (f32x4*)(wave_rows + (size_t)row * row_floats + ch * 4));
    }
    // the slab is reused by the next tensor of the same wave
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// ------------------------------------------------------------------------------------------------
// dQ: row owner
// ------------------------------------------------------------------------------------------------
// wg: index of the work-group among those of this part of the launch; smem: 4 tiles (K0 K1 V0 V1)
// RAGGED: tensors with rows of hd = p.state < D elements.  The query-side operands are loaded with zeros in place of
// the missing features, so whatever the tiles hold there (other features of the same rows) drops out of the
// score-like products; in the transposed products it only reaches output columns that are not stored.
template <int BS, int D, bool MASKED, bool RAGGED = false>
__device__ __forceinline__ void attention_dq(const BackwardParams& p, uint32_t wg, uint8_t* smem) {
    using T = Bf16DirectTiles<BS, D>;
    constexpr int KT = BS / 32, NO = D / 32, KS = D / 16, PU = BS / 16, TILE = T::TILE_BYTES;

    const LineWork work = decode_line_work(p, p.nn_lut, wg);
    if (!work.valid) return;
    const uint32_t b = work.bh / p.heads, h = work.bh % p.heads;
    const uint32_t r = work.line;
    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t qn = lane & 31, half = lane >> 5;
    const uint32_t q_in_block = wave * 32 + qn;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const uint32_t row_bytes = p.heads * hd * 2;
    const uint32_t off = __builtin_amdgcn_readfirstlane(work.first), count = __builtin_amdgcn_readfirstlane(work.count);
    const size_t my_row = token_offset(b, r * BS + q_in_block, h, L, p.heads, hd);

    f32x16 dq_acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) dq_acc[n][i] = 0.f;

    if (count > 0) {
        const size_t bh_bytes = token_offset(b, 0, h, L, p.heads, hd) * 2;
        const uint8_t* const k_base = (const uint8_t*)p.k + bh_bytes;
        const uint8_t* const v_base = (const uint8_t*)p.v + bh_bytes;
        const typename T::Sources src = RAGGED ? T::sources_ragged(lane, row_bytes, hd) : T::sources(lane, row_bytes);
        const uint32_t lds0 = T::lds_address(smem);
        const uint32_t k_lane = T::k_lane_base(qn, half), v_lane = T::v_lane_base(lane);
        const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
        const int valid = p.valid_len ? p.valid_len[b] : (int)L;
        const float c = p.scale_log2e;

        bf16x8 qf[KS], dof[KS];
        if constexpr (RAGGED) {
            T::load_q_ragged(qf, (const __bf16*)p.q + my_row, half, hd);
            T::load_q_ragged(dof, (const __bf16*)p.d_out + my_row, half, hd);
        } else {
            T::load_q(qf, (const __bf16*)p.q + my_row, half);
            T::load_q(dof, (const __bf16*)p.d_out + my_row, half);
        }
        const size_t stat = ((size_t)work.bh * p.nb + r) * BS + q_in_block;
        const float lse = p.lse[stat], delta = p.delta[stat];

        auto uniform = [](const sfb_uint2 e) -> sfb_uint2 {
            const sfb_uint2 u = {(uint32_t)__builtin_amdgcn_readfirstlane(e.x), (uint32_t)__builtin_amdgcn_readfirstlane(e.y)};
            return u;
        };
        auto fetch = [&](const sfb_uint2 e, uint32_t buf) {
            T::template load_tile_all<RAGGED>(lds0 + buf * TILE, k_base + (size_t)e.y * BS * row_bytes, wave, src, row_bytes);
            T::template load_tile_all<RAGGED>(lds0 + (2 + buf) * TILE, v_base + (size_t)e.y * BS * row_bytes, wave, src, row_bytes);
        };
        const sfb_uint2* const nn_lut = p.nn_lut + (size_t)h * p.lut_stride;
        sfb_uint2 e = uniform(nn_lut[off]);
        fetch(e, 0);
        for (uint32_t j = 0; j < count; ++j) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();   // tiles of block j have landed for every wave; every wave is done with block j-1
            const sfb_uint2 e_next = uniform(nn_lut[off + (j + 1 < count ? j + 1 : j)]);
            fetch(e_next, (j + 1) & 1);
            const uint8_t* k_tile = smem + (j & 1) * TILE;
            const uint8_t* v_tile = smem + (2 + (j & 1)) * TILE;

            f32x16 s[KT], dp[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
                for (int i = 0; i < 16; ++i) { s[kt][i] = 0.f; dp[kt][i] = 0.f; }
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::k_frag(k_tile, k_lane, kt, ks), qf[ks], s[kt], 0, 0, 0);
                    dp[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::k_frag(v_tile, k_lane, kt, ks), dof[ks], dp[kt], 0, 0, 0);
                }
            }
            if (MASKED) {
                const int limit = valid - (int)(e.y * BS);
                if ((mask != nullptr) || (limit < BS))
                    apply_keep<KT>(s, load_keep_word<BS>(mask, (size_t)e.x * BS + q_in_block, limit), half);
            }
            // dS^T for this lane's query: P (dP - delta) scale; a masked score is -3e38, its probability an exact 0
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float prob = exp2_fast(__builtin_fmaf(s[kt][i], c, -lse));
                    s[kt][i] = prob * (dp[kt][i] - delta) * p.scale;
                }
            uint32_t pk[KT * 8];
            pack_chunks<KT>(pk, s);
#pragma unroll
            for (int u = 0; u < PU; ++u) {
                const u32x4 pb = {pk[u * 4 + 0], pk[u * 4 + 1], pk[u * 4 + 2], pk[u * 4 + 3]};
                const bf16x8 bfrag = __builtin_bit_cast(bf16x8, pb);
#pragma unroll
                for (int mt = 0; mt < NO; ++mt)
                    dq_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::v_frag(k_tile, v_lane, mt, u), bfrag, dq_acc[mt], 0, 0, 0);
            }
            e = e_next;
        }
    }
    if (work.slot < 0) {
        // the last iteration's look-ahead tile loads have landed and every wave is done with the tiles: their
        // memory carries the output slabs now
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if constexpr (RAGGED) store_rows_f32_ragged<NO>(p.dq + my_row, dq_acc, half, hd);
        else store_rows_slab<NO>(p.dq + my_row, p.heads * D, dq_acc, lane, smem + wave * (32 * (D * 4 + 16)));
    } else store_rows_f32<NO>(p.partials + (((size_t)work.bh * p.n_parts + work.slot) * BS + q_in_block) * D, dq_acc, half);
}

// ------------------------------------------------------------------------------------------------
// dK, dV: column owner
// ------------------------------------------------------------------------------------------------
// wg: index of the work-group among those of this part of the launch; smem: 4 tiles (Q0 Q1 dO0 dO1)
template <int BS, int D, bool MASKED, bool RAGGED = false>
__device__ __forceinline__ void attention_dkdv(const BackwardParams& p, uint32_t wg, uint8_t* smem) {
    using T = Bf16DirectTiles<BS, D>;
    constexpr int KT = BS / 32, NO = D / 32, KS = D / 16, PU = BS / 16, TILE = T::TILE_BYTES;

    const LineWork work = decode_line_work(p, p.tn_lut, wg);
    if (!work.valid) return;
    const uint32_t b = work.bh / p.heads, h = work.bh % p.heads;
    const uint32_t col = work.line;
    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t kn = lane & 31, half = lane >> 5;
    const uint32_t key_in_block = wave * 32 + kn;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const uint32_t row_bytes = p.heads * hd * 2;
    const uint32_t off = __builtin_amdgcn_readfirstlane(work.first), count = __builtin_amdgcn_readfirstlane(work.count);
    const size_t my_row = token_offset(b, col * BS + key_in_block, h, L, p.heads, hd);

    f32x16 dk_acc[NO], dv_acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) { dk_acc[n][i] = 0.f; dv_acc[n][i] = 0.f; }

    if (count > 0) {
        const size_t bh_bytes = token_offset(b, 0, h, L, p.heads, hd) * 2;
        const uint8_t* const q_base = (const uint8_t*)p.q + bh_bytes;
        const uint8_t* const do_base = (const uint8_t*)p.d_out + bh_bytes;
        const typename T::Sources src = RAGGED ? T::sources_ragged(lane, row_bytes, hd) : T::sources(lane, row_bytes);
        const uint32_t lds0 = T::lds_address(smem);
        const uint32_t k_lane = T::k_lane_base(kn, half), v_lane = T::v_lane_base(lane);
        const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
        const int valid = p.valid_len ? p.valid_len[b] : (int)L;
        const bool key_valid = (int)(col * BS + key_in_block) < valid;
        const float c = p.scale_log2e;
        const float* lse_bh = p.lse + (size_t)work.bh * L;
        const float* delta_bh = p.delta + (size_t)work.bh * L;

        bf16x8 kf[KS], vf[KS];   // this lane's key as the B operand of both score-like products
        if constexpr (RAGGED) {
            T::load_q_ragged(kf, (const __bf16*)p.k + my_row, half, hd);
            T::load_q_ragged(vf, (const __bf16*)p.v + my_row, half, hd);
        } else {
            T::load_q(kf, (const __bf16*)p.k + my_row, half);
            T::load_q(vf, (const __bf16*)p.v + my_row, half);
        }

        auto uniform = [](const sfb_uint2 e) -> sfb_uint2 {
            const sfb_uint2 u = {(uint32_t)__builtin_amdgcn_readfirstlane(e.x), (uint32_t)__builtin_amdgcn_readfirstlane(e.y)};
            return u;
        };
        auto fetch = [&](const sfb_uint2 e, uint32_t buf) {   // e = {block id, row block}
            T::template load_tile_all<RAGGED>(lds0 + buf * TILE, q_base + (size_t)e.y * BS * row_bytes, wave, src, row_bytes);
            T::template load_tile_all<RAGGED>(lds0 + (2 + buf) * TILE, do_base + (size_t)e.y * BS * row_bytes, wave, src, row_bytes);
        };
        const sfb_uint2* const tn_lut = p.tn_lut + (size_t)h * p.lut_stride;
        sfb_uint2 e = uniform(tn_lut[off]);
        fetch(e, 0);
        for (uint32_t j = 0; j < count; ++j) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            const sfb_uint2 e_next = uniform(tn_lut[off + (j + 1 < count ? j + 1 : j)]);
            fetch(e_next, (j + 1) & 1);
            const uint8_t* q_tile = smem + (j & 1) * TILE;
            const uint8_t* do_tile = smem + (2 + (j & 1)) * TILE;

            // S[query][key], dP[query][key]: element i of tile kt is query kt*32 + (i/4)*8 + half*4 + i%4, key = lane's
            f32x16 s[KT], dp[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
                for (int i = 0; i < 16; ++i) { s[kt][i] = 0.f; dp[kt][i] = 0.f; }
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::k_frag(q_tile, k_lane, kt, ks), kf[ks], s[kt], 0, 0, 0);
                    dp[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::k_frag(do_tile, k_lane, kt, ks), vf[ks], dp[kt], 0, 0, 0);
                }
            }
            const float* lse_blk = lse_bh + (size_t)e.y * BS;
            const float* delta_blk = delta_bh + (size_t)e.y * BS;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int ig = 0; ig < 4; ++ig) {
                    const uint32_t q0 = kt * 32 + ig * 8 + half * 4;
                    const f32x4 lse4 = *(const f32x4*)(lse_blk + q0), delta4 = *(const f32x4*)(delta_blk + q0);
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        const int i = ig * 4 + x;
                        float prob = exp2_fast(__builtin_fmaf(s[kt][i], c, -lse4[x]));
                        if (MASKED) {
                            bool keep = key_valid;
                            if (mask != nullptr) {
                                const size_t word = (size_t)e.x * BS + q0 + x;
                                const uint64_t bits = (BS == 64) ? ((const uint64_t*)mask)[word] : ((const uint32_t*)mask)[word];
                                keep = keep && ((bits >> key_in_block) & 1u);
                            }
                            prob = keep ? prob : 0.f;
                        }
                        s[kt][i] = prob;
                        dp[kt][i] = prob * (dp[kt][i] - delta4[x]) * p.scale;
                    }
                }
            uint32_t pk_p[KT * 8], pk_ds[KT * 8];
            pack_chunks<KT>(pk_p, s);
            pack_chunks<KT>(pk_ds, dp);
#pragma unroll
            for (int u = 0; u < PU; ++u) {
                const u32x4 pb = {pk_p[u * 4 + 0], pk_p[u * 4 + 1], pk_p[u * 4 + 2], pk_p[u * 4 + 3]};
                const u32x4 db = {pk_ds[u * 4 + 0], pk_ds[u * 4 + 1], pk_ds[u * 4 + 2], pk_ds[u * 4 + 3]};
                const bf16x8 pfrag = __builtin_bit_cast(bf16x8, pb), dsfrag = __builtin_bit_cast(bf16x8, db);
#pragma unroll
                for (int mt = 0; mt < NO; ++mt) {
                    dv_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::v_frag(do_tile, v_lane, mt, u), pfrag, dv_acc[mt], 0, 0, 0);
                    dk_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::v_frag(q_tile, v_lane, mt, u), dsfrag, dk_acc[mt], 0, 0, 0);
                }
            }
            e = e_next;
        }
    }
    if (work.slot < 0) {
        // the last iteration's look-ahead tile loads have landed and every wave is done with the tiles: their
        // memory carries the output slabs now
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        uint8_t* const slab = smem + wave * (32 * (D * 4 + 16));
        if constexpr (RAGGED) {
            store_rows_f32_ragged<NO>(p.dk + my_row, dk_acc, half, hd);
            store_rows_f32_ragged<NO>(p.dv + my_row, dv_acc, half, hd);
        } else {
            store_rows_slab<NO>(p.dk + my_row, p.heads * D, dk_acc, lane, slab);
            store_rows_slab<NO>(p.dv + my_row, p.heads * D, dv_acc, lane, slab);
        }
    } else {   // partial record of a split column: dK rows, then dV rows
        float* part = p.partials + (((size_t)work.bh * p.n_parts + work.slot) * 2 * BS + key_in_block) * D;
        store_rows_f32<NO>(part, dk_acc, half);
        store_rows_f32<NO>(part + (size_t)BS * D, dv_acc, half);
    }
}

// Sum of the partial records of split block-rows (TENSORS = 1: dQ) or block-columns (TENSORS = 2: dK, dV), in chunk
// order, by the work-group of the line's first chunk; all other work-groups leave at once.  A separate launch: the
// partials are complete when it starts, nobody has to wait for anybody.
// One launch for both halves of the backward pass: the first col_wgs work-groups own key columns (dK, dV: the longer
// items, so they go first), the others own query rows (dQ).  As two launches, the second waits until the last
// work-group of the first is done; as one, its work-groups fill the slots as the first's drain.  col_wgs is a
// multiple of 8, so both halves see the same work-group -> XCD assignment as a launch of their own.
template <int BS, int D, bool MASKED, bool RAGGED = false>
__global__ __launch_bounds__(BS * 2, D > 64 ? 1 : 2) void attention_backward_kernel(BackwardParams cols, BackwardParams rows,
                                                                       uint32_t col_wgs) {
    __shared__ __attribute__((aligned(1024))) uint8_t smem[4 * Bf16DirectTiles<BS, D>::TILE_BYTES];
    if (blockIdx.x < col_wgs) attention_dkdv<BS, D, MASKED, RAGGED>(cols, blockIdx.x, smem);
    else attention_dq<BS, D, MASKED, RAGGED>(rows, blockIdx.x - col_wgs, smem);
}

// ------------------------------------------------------------------------------------------------
// fp32 tensors: the same two halves on v_mfma_f32_32x32x2_f32 (true fp32 products), tiles staged through registers
// into one LDS buffer each as in the fp32 forward kernel (F32Tiles; rows of D + 4 floats, read row-wise as 128-bit
// fragments for the score-like products and element-wise down a column for the transposed ones)
// ------------------------------------------------------------------------------------------------
// element (row 32 kt + (i/4) 8 + 4 half + i%4, column 32 mt + qn) of a tile in the K layout of F32Tiles: the A operand
// of a transposed product step, as F32Tiles::v_elem is for the V layout
template <int BS, int D>
__device__ __forceinline__ float tile_column_elem(const float* lds, int kt, int i, int mt, uint32_t qn, uint32_t half) {
    const uint32_t row = kt * 32 + (i / 4) * 8 + half * 4 + (i % 4);
    return lds[row * F32Tiles<BS, D>::K_STRIDE + mt * 32 + qn];
}

template <int BS, int D, bool MASKED, bool RAGGED = false>
__device__ __forceinline__ void attention_dq_f32(const BackwardParams& p, uint32_t wg, float* k_lds, float* v_lds) {
    using T = F32Tiles<BS, D>;
    constexpr int KT = BS / 32, NO = D / 32, QG = D / 8;

    const LineWork work = decode_line_work(p, p.nn_lut, wg);
    if (!work.valid) return;
    const uint32_t b = work.bh / p.heads, h = work.bh % p.heads;
    const uint32_t r = work.line;
    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint32_t qn = lane & 31, half = lane >> 5;
    const uint32_t q_in_block = wave * 32 + qn;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const uint32_t row_stride = p.heads * hd;
    const uint32_t off = work.first, count = work.count;
    const size_t my_row = token_offset(b, r * BS + q_in_block, h, L, p.heads, hd);
    auto fetch = [&](typename T::Regs& regs, const float* X, size_t base) {   // missing features of short rows: zeros
        if constexpr (RAGGED) T::fetch_ragged(regs, X, base, row_stride, t, hd);
        else T::fetch(regs, X, base, row_stride, t);
    };

    f32x16 dq_acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) dq_acc[n][i] = 0.f;

    if (count > 0) {
        const float* K = (const float*)p.k;
        const float* V = (const float*)p.v;
        const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
        const int valid = p.valid_len ? p.valid_len[b] : (int)L;
        const float c = p.scale_log2e;

        f32x4 qf[QG], dof[QG];
        if constexpr (RAGGED) {
            T::load_q_ragged(qf, (const float*)p.q + my_row, half, hd);
            T::load_q_ragged(dof, (const float*)p.d_out + my_row, half, hd);
        } else {
            T::load_q(qf, (const float*)p.q + my_row, half);
            T::load_q(dof, (const float*)p.d_out + my_row, half);
        }
        const size_t stat = ((size_t)work.bh * p.nb + r) * BS + q_in_block;
        const float lse = p.lse[stat], delta = p.delta[stat];

        const sfb_uint2* const nn_lut = p.nn_lut + (size_t)h * p.lut_stride;
        typename T::Regs gk, gv;
        sfb_uint2 entry = nn_lut[off];
        {
            const size_t base = token_offset(b, entry.y * BS, h, L, p.heads, hd);
            fetch(gk, K, base);
            fetch(gv, V, base);
        }
        for (uint32_t j = 0; j < count; ++j) {
            const sfb_uint2 e = entry;
            T::template stage<T::K_STRIDE>(k_lds, gk, t);
            T::template stage<T::K_STRIDE>(v_lds, gv, t);
            __syncthreads();
            if (j + 1 < count) {
                entry = nn_lut[off + j + 1];
                const size_t base = token_offset(b, entry.y * BS, h, L, p.heads, hd);
                fetch(gk, K, base);
                fetch(gv, V, base);
            }
            f32x16 s[KT], dp[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int i = 0; i < 16; ++i) { s[kt][i] = 0.f; dp[kt][i] = 0.f; }
#pragma unroll
            for (int g = 0; g < QG; ++g)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
                    const f32x4 ka = T::k_frag(k_lds, kt, g, qn, half), va = T::k_frag(v_lds, kt, g, qn, half);
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        s[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[x], qf[g][x], s[kt], 0, 0, 0);
                        dp[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[x], dof[g][x], dp[kt], 0, 0, 0);
                    }
                }
            if (MASKED) {
                const int limit = valid - (int)(e.y * BS);
                if ((mask != nullptr) || (limit < BS))
                    apply_keep<KT>(s, load_keep_word<BS>(mask, (size_t)e.x * BS + q_in_block, limit), half);
            }
            // dS^T for this lane's query: P (dP - delta) scale; a masked score is -3e38, its probability an exact 0
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float prob = exp2_fast(__builtin_fmaf(s[kt][i], c, -lse));
                    s[kt][i] = prob * (dp[kt][i] - delta) * p.scale;
                }
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int i = 0; i < 16; ++i)
#pragma unroll
                    for (int mt = 0; mt < NO; ++mt)
                        dq_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(tile_column_elem<BS, D>(k_lds, kt, i, mt, qn, half),
                                                                          s[kt][i], dq_acc[mt], 0, 0, 0);
            __syncthreads();   // every wave is done with the tiles before the next block is staged
        }
    }
    if (work.slot < 0) {
        if constexpr (RAGGED) store_rows_f32_ragged<NO>(p.dq + my_row, dq_acc, half, hd);
        else store_rows_f32<NO>(p.dq + my_row, dq_acc, half);
    } else store_rows_f32<NO>(p.partials + (((size_t)work.bh * p.n_parts + work.slot) * BS + q_in_block) * D, dq_acc, half);
}

template <int BS, int D, bool MASKED, bool RAGGED = false>
__device__ __forceinline__ void attention_dkdv_f32(const BackwardParams& p, uint32_t wg, float* q_lds, float* do_lds) {
    using T = F32Tiles<BS, D>;
    constexpr int KT = BS / 32, NO = D / 32, QG = D / 8;

    const LineWork work = decode_line_work(p, p.tn_lut, wg);
    if (!work.valid) return;
    const uint32_t b = work.bh / p.heads, h = work.bh % p.heads;
    const uint32_t col = work.line;
    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint32_t kn = lane & 31, half = lane >> 5;
    const uint32_t key_in_block = wave * 32 + kn;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const uint32_t row_stride = p.heads * hd;
    const uint32_t off = work.first, count = work.count;
    const size_t my_row = token_offset(b, col * BS + key_in_block, h, L, p.heads, hd);
    auto fetch = [&](typename T::Regs& regs, const float* X, size_t base) {
        if constexpr (RAGGED) T::fetch_ragged(regs, X, base, row_stride, t, hd);
        else T::fetch(regs, X, base, row_stride, t);
    };

    f32x16 dk_acc[NO], dv_acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) { dk_acc[n][i] = 0.f; dv_acc[n][i] = 0.f; }

    if (count > 0) {
        const float* Q = (const float*)p.q;
        const float* DO = (const float*)p.d_out;
        const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
        const int valid = p.valid_len ? p.valid_len[b] : (int)L;
        const bool key_valid = (int)(col * BS + key_in_block) < valid;
        const float c = p.scale_log2e;
        const float* lse_bh = p.lse + (size_t)work.bh * L;
        const float* delta_bh = p.delta + (size_t)work.bh * L;

        f32x4 kf[QG], vf[QG];   // this lane's key as the B operand of both score-like products
        if constexpr (RAGGED) {
            T::load_q_ragged(kf, (const float*)p.k + my_row, half, hd);
            T::load_q_ragged(vf, (const float*)p.v + my_row, half, hd);
        } else {
            T::load_q(kf, (const float*)p.k + my_row, half);
            T::load_q(vf, (const float*)p.v + my_row, half);
        }

        const sfb_uint2* const tn_lut = p.tn_lut + (size_t)h * p.lut_stride;
        typename T::Regs gq, gd;
        sfb_uint2 entry = tn_lut[off];   // {block id, row block}
        {
            const size_t base = token_offset(b, entry.y * BS, h, L, p.heads, hd);
            fetch(gq, Q, base);
            fetch(gd, DO, base);
        }
        for (uint32_t j = 0; j < count; ++j) {
            const sfb_uint2 e = entry;
            T::template stage<T::K_STRIDE>(q_lds, gq, t);
            T::template stage<T::K_STRIDE>(do_lds, gd, t);
            __syncthreads();
            if (j + 1 < count) {
                entry = tn_lut[off + j + 1];
                const size_t base = token_offset(b, entry.y * BS, h, L, p.heads, hd);
                fetch(gq, Q, base);
                fetch(gd, DO, base);
            }
            // S[query][key], dP[query][key]: element i of tile kt is query kt*32 + (i/4)*8 + half*4 + i%4, key = lane's
            f32x16 s[KT], dp[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int i = 0; i < 16; ++i) { s[kt][i] = 0.f; dp[kt][i] = 0.f; }
#pragma unroll
            for (int g = 0; g < QG; ++g)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
                    const f32x4 qa = T::k_frag(q_lds, kt, g, kn, half), da = T::k_frag(do_lds, kt, g, kn, half);
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        s[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[x], kf[g][x], s[kt], 0, 0, 0);
                        dp[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(da[x], vf[g][x], dp[kt], 0, 0, 0);
                    }
                }
            const float* lse_blk = lse_bh + (size_t)e.y * BS;
            const float* delta_blk = delta_bh + (size_t)e.y * BS;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int ig = 0; ig < 4; ++ig) {
                    const uint32_t q0 = kt * 32 + ig * 8 + half * 4;
                    const f32x4 lse4 = *(const f32x4*)(lse_blk + q0), delta4 = *(const f32x4*)(delta_blk + q0);
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        const int i = ig * 4 + x;
                        float prob = exp2_fast(__builtin_fmaf(s[kt][i], c, -lse4[x]));
                        if (MASKED) {
                            bool keep = key_valid;
                            if (mask != nullptr) {
                                const size_t word = (size_t)e.x * BS + q0 + x;
                                const uint64_t bits = (BS == 64) ? ((const uint64_t*)mask)[word] : ((const uint32_t*)mask)[word];
                                keep = keep && ((bits >> key_in_block) & 1u);
                            }
                            prob = keep ? prob : 0.f;
                        }
                        s[kt][i] = prob;
                        dp[kt][i] = prob * (dp[kt][i] - delta4[x]) * p.scale;
                    }
                }
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int i = 0; i < 16; ++i)
#pragma unroll
                    for (int mt = 0; mt < NO; ++mt) {
                        dv_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(tile_column_elem<BS, D>(do_lds, kt, i, mt, kn, half),
                                                                          s[kt][i], dv_acc[mt], 0, 0, 0);
                        dk_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(tile_column_elem<BS, D>(q_lds, kt, i, mt, kn, half),
                                                                          dp[kt][i], dk_acc[mt], 0, 0, 0);
                    }
            __syncthreads();
        }
    }
    if (work.slot < 0) {
        if constexpr (RAGGED) {
            store_rows_f32_ragged<NO>(p.dk + my_row, dk_acc, half, hd);
            store_rows_f32_ragged<NO>(p.dv + my_row, dv_acc, half, hd);
        } else {
            store_rows_f32<NO>(p.dk + my_row, dk_acc, half);
            store_rows_f32<NO>(p.dv + my_row, dv_acc, half);
        }
    } else {   // partial record of a split column: dK rows, then dV rows
        float* part = p.partials + (((size_t)work.bh * p.n_parts + work.slot) * 2 * BS + key_in_block) * D;
        store_rows_f32<NO>(part, dk_acc, half);
        store_rows_f32<NO>(part + (size_t)BS * D, dv_acc, half);
    }
}

template <int BS, int D, bool MASKED, bool RAGGED = false>
__global__ __launch_bounds__(BS * 2, 1) void attention_backward_f32_kernel(BackwardParams cols, BackwardParams rows,
                                                                           uint32_t col_wgs) {
    using T = F32Tiles<BS, D>;
    __shared__ __attribute__((aligned(16))) float a_lds[T::K_FLOATS];
    __shared__ __attribute__((aligned(16))) float b_lds[T::K_FLOATS];
    if (blockIdx.x < col_wgs) attention_dkdv_f32<BS, D, MASKED, RAGGED>(cols, blockIdx.x, a_lds, b_lds);
    else attention_dq_f32<BS, D, MASKED, RAGGED>(rows, blockIdx.x - col_wgs, a_lds, b_lds);
}

// Sum of the partial records of one split line, in chunk order (so the result does not depend on which chunk
// finished when), written to the line's rows of the output tensors.
template <int BS, int D, int TENSORS>
__device__ __forceinline__ void reduce_line(float* out0, float* out1, const float* partials, const sfb_work_item& it,
                                            uint32_t n_parts, uint32_t bh, uint32_t heads, uint32_t ctx, uint32_t hd) {
    const uint32_t b = bh / heads, h = bh % heads;
    constexpr int VECS = BS * D / 4;
    for (int tensor = 0; tensor < TENSORS; ++tensor) {
        float* out = tensor == 0 ? out0 : out1;
        for (uint32_t vec = threadIdx.x; vec < VECS; vec += 256) {
            const uint32_t row = vec / (D / 4), c4 = vec % (D / 4);
            f32x4 sum = {0.f, 0.f, 0.f, 0.f};
            for (uint32_t ch = 0; ch < it.nchunks; ++ch)
                sum += *(const f32x4*)(partials + ((((size_t)bh * n_parts + it.part + ch) * TENSORS + tensor) * BS + row) * D + c4 * 4);
            if (c4 * 4 < hd) *(f32x4*)(out + token_offset(b, it.row * BS + row, h, ctx, heads, hd) + c4 * 4) = sum;
        }
    }
}

// grid (n_col_items + n_row_items, batch*heads): the work-groups of the first chunk of a split column (dK, dV) or
// row (dQ) do the sums, all others leave at once
template <int BS, int D>
__global__ __launch_bounds__(256) void reduce_partials_kernel(float* dk, float* dv, float* dq, const float* col_partials,
                                                              const float* row_partials, const sfb_work_item* col_items,
                                                              const sfb_work_item* row_items, uint32_t n_col_items,
                                                              uint32_t n_col_parts, uint32_t n_row_parts, uint32_t heads,
                                                              uint32_t ctx, uint32_t hd) {
    const bool column = blockIdx.x < n_col_items;
    const sfb_work_item it = column ? col_items[blockIdx.x] : row_items[blockIdx.x - n_col_items];
    if (it.nchunks <= 1 || it.chunk != 0) return;
    if (column) reduce_line<BS, D, 2>(dk, dv, col_partials, it, n_col_parts, blockIdx.y, heads, ctx, hd);
    else reduce_line<BS, D, 1>(dq, nullptr, row_partials, it, n_row_parts, blockIdx.y, heads, ctx, hd);
}

template <int BS, int D>
static int launch_backward(hipStream_t stream, int dtype, const BackwardParams& p, const sfb_work_item* row_items,
                           uint32_t n_row_items, uint32_t n_row_heavy, uint32_t n_row_parts,
                           const sfb_work_item* col_items, uint32_t n_col_items, uint32_t n_col_heavy,
                           uint32_t n_col_parts, float* row_partials, float* col_partials) {
    const bool masked = p.mask != nullptr || p.valid_len != nullptr;
    const uint32_t groups = bh_groups(p.batch * p.heads);
    BackwardParams rows = p, cols = p;
    rows.items = row_items; rows.ranks = row_items ? n_row_items : p.nb; rows.heavy = row_items ? n_row_heavy : 0;
    rows.n_parts = n_row_parts; rows.partials = row_partials;
    cols.items = col_items; cols.ranks = col_items ? n_col_items : p.nb; cols.heavy = col_items ? n_col_heavy : 0;
    cols.n_parts = n_col_parts; cols.partials = col_partials;
    clear_stale_error();
    const uint32_t col_wgs = groups * 8u * cols.ranks, row_wgs = groups * 8u * rows.ranks;
    const dim3 grid(col_wgs + row_wgs), block(BS * 2);
    if (p.state != (uint32_t)D) {   // head sizes between the multiples of 32: the masked form serves both
        if (dtype == SFB_F32) attention_backward_f32_kernel<BS, D, true, true><<<grid, block, 0, stream>>>(cols, rows, col_wgs);
        else attention_backward_kernel<BS, D, true, true><<<grid, block, 0, stream>>>(cols, rows, col_wgs);
    } else if (dtype == SFB_F32) {
        if (masked) attention_backward_f32_kernel<BS, D, true><<<grid, block, 0, stream>>>(cols, rows, col_wgs);
        else attention_backward_f32_kernel<BS, D, false><<<grid, block, 0, stream>>>(cols, rows, col_wgs);
    } else if (masked) {
        attention_backward_kernel<BS, D, true><<<grid, block, 0, stream>>>(cols, rows, col_wgs);
    } else {
        attention_backward_kernel<BS, D, false><<<grid, block, 0, stream>>>(cols, rows, col_wgs);
    }
    const uint32_t reduce_cols = (col_items && n_col_parts) ? n_col_items : 0u;
    const uint32_t reduce_rows = (row_items && n_row_parts) ? n_row_items : 0u;
    if (reduce_cols + reduce_rows)
        reduce_partials_kernel<BS, D><<<dim3(reduce_cols + reduce_rows, p.batch * p.heads), dim3(256), 0, stream>>>(
            p.dk, p.dv, p.dq, col_partials, row_partials, col_items, row_items, reduce_cols, n_col_parts, n_row_parts,
            p.heads, p.nb * BS, p.state);
    return launch_status();
}

}  // namespace sfb

extern "C" size_t sfb_backward_workspace_bytes(uint32_t n_row_parts, uint32_t n_col_parts, uint32_t batch_dim,
                                               uint32_t head_dim, uint32_t block_size, uint32_t state_dim) {
    const size_t record = (size_t)block_size * ((state_dim + 31u) / 32u * 32u) * sizeof(float);   // rows of the kernels' D floats
    return (size_t)batch_dim * head_dim * ((size_t)n_row_parts + 2 * (size_t)n_col_parts) * record;
}

extern "C" int sfb_fused_attention_backward(sfb_stream_t stream, const void* q, const void* k, const void* v,
                                            const float* o, const void* d_out, const float* lse, float* delta,
                                            float* dq, float* dk, float* dv, int dtype, const sfb_uint2* nn_lut,
                                            const sfb_uint2* tn_lut, const void* mask, const int32_t* valid_len,
                                            const sfb_work_item* row_items, uint32_t n_row_items,
                                            uint32_t n_row_heavy, uint32_t n_row_parts,
                                            const sfb_work_item* col_items, uint32_t n_col_items,
                                            uint32_t n_col_heavy, uint32_t n_col_parts, void* workspace,
                                            size_t workspace_bytes, uint32_t block_size, uint32_t blocks,
                                            uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                                            uint32_t state_dim, uint32_t lut_heads, uint32_t lut_dim,
                                            uint32_t mask_heads, float scale) {
    using namespace sfb;
    if (!q || !k || !v || !o || !d_out || !lse || !delta || !dq || !dk || !dv || !nn_lut || !tn_lut)
        return SFB_ERR_NULL_POINTER;
    if (dtype != SFB_BF16 && dtype != SFB_F32) return SFB_ERR_DTYPE;
    if (block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    // every multiple of the 16-byte vector up to 128 (32, 64, 96, 128: what the tiles divide; the others run the kernel
    // of the next multiple of 32 with its short-row loads and stores)
    if (state_dim == 0 || state_dim > 128 || state_dim % (dtype == SFB_BF16 ? 8u : 4u) != 0) return SFB_ERR_HEAD_STATE;
    if (!(scale > 0.f) || !(scale < 3.0e38f)) return SFB_ERR_ARGUMENT;
    if (!batch_dim || !ctx_blks || !head_dim || !mask_heads || !lut_heads) return SFB_ERR_SHAPE;
    if (mask_heads > 1 && mask_heads != head_dim) return SFB_ERR_SHAPE;
    if (lut_heads > 1 && (lut_heads != head_dim || lut_dim != ctx_blks + blocks)) return SFB_ERR_SHAPE;
    // work items describe one layout: with a table per head every line is done whole by one work-group
    if (lut_heads > 1 && (row_items || col_items)) return SFB_ERR_SHAPE;
    if ((row_items && (!n_row_items || n_row_heavy >= n_row_items)) ||
        (col_items && (!n_col_items || n_col_heavy >= n_col_items)))
        return SFB_ERR_SHAPE;
    const uint64_t most = (row_items ? n_row_items : ctx_blks) > (col_items ? n_col_items : ctx_blks)
                              ? (row_items ? n_row_items : ctx_blks) : (col_items ? n_col_items : ctx_blks);
    if ((uint64_t)batch_dim * head_dim * most > 0x7fffffffull / 64) return SFB_ERR_SHAPE;
    if (!row_items) n_row_parts = 0;
    if (!col_items) n_col_parts = 0;
    const size_t need = sfb_backward_workspace_bytes(n_row_parts, n_col_parts, batch_dim, head_dim, block_size, state_dim);
    if (need && (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255u))) return SFB_ERR_WORKSPACE;
    const uintptr_t align = (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o | (uintptr_t)d_out |
                            (uintptr_t)lse | (uintptr_t)delta | (uintptr_t)dq | (uintptr_t)dk | (uintptr_t)dv;
    if (align & 15u) return SFB_ERR_ALIGNMENT;
    const int rc = sfb_row_dot(stream, delta, d_out, o, dtype, batch_dim, ctx_blks * block_size, head_dim, state_dim);
    if (rc != SFB_OK) return rc;
    BackwardParams p = {};
    p.q = q; p.k = k; p.v = v; p.d_out = d_out; p.lse = lse; p.delta = delta; p.dq = dq; p.dk = dk; p.dv = dv;
    p.nn_lut = nn_lut; p.tn_lut = tn_lut; p.mask = mask; p.valid_len = valid_len;
    p.batch = batch_dim; p.heads = head_dim; p.nb = ctx_blks; p.blocks = blocks; p.state = state_dim;
    p.mask_stride = mask_heads > 1 ? blocks * block_size : 0;
    p.lut_stride = lut_heads > 1 ? lut_dim : 0;
    p.scale = scale; p.scale_log2e = scale * kLog2e;
    float* row_partials = (float*)workspace;
    const uint32_t padded = (state_dim + 31u) / 32u * 32u;
    float* col_partials = row_partials + (size_t)batch_dim * head_dim * n_row_parts * block_size * padded;
    hipStream_t s = (hipStream_t)stream;
#define SFB_CALL(BSV, DV)                                                                                        \
    return launch_backward<BSV, DV>(s, dtype, p, row_items, n_row_items, n_row_heavy, n_row_parts, col_items, n_col_items, \
                                    n_col_heavy, n_col_parts, row_partials, col_partials)
    if (block_size == 64) {
        if (padded == 64) SFB_CALL(64, 64);
        if (padded == 32) SFB_CALL(64, 32);
        if (padded == 96) SFB_CALL(64, 96);
        SFB_CALL(64, 128);
    }
    if (padded == 64) SFB_CALL(32, 64);
    if (padded == 32) SFB_CALL(32, 32);
    if (padded == 96) SFB_CALL(32, 96);
    SFB_CALL(32, 128);
#undef SFB_CALL
}
