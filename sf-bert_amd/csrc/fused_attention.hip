// Fully fused block-sparse attention for gfx950 (MI355X).
//
// One work-group owns one (batch, head, block-row) of BS queries -- or, for block-rows that the
// schedule splits, one contiguous chunk of that row's key blocks -- and walks the key blocks the NN
// look-up table lists.  Each wave owns 32 queries.  Per key block it
//   1. computes the transposed score tile  S^T = K_blk . Q^T  on MFMA (A = K from LDS, B = Q kept in
//      registers for the whole row), so that every lane ends up with keys of ONE query: the row
//      maximum / sum need only lane-local work plus one exchange between lane l and lane l+32;
//   2. does the scaled, masked online softmax on the accumulators (exp2 with log2(e) folded in);
//   3. feeds the probabilities, still in registers, as the B operand of  O^T += V_blk^T . P^T.
// O is normalised and written once at the end; S and P never exist in memory and no work-group ever
// waits for another.  Chunks of a split row leave (O, max, sum) partials in a workspace and bump a
// counter; whichever chunk arrives last merges them and writes O (nobody spins).
//
// Arithmetic follows the reference CPU path: scores are raw dot products, the maximum is taken over
// kept keys with seed -1000000 (ewops.h:70), p = exp((s-max)*scale) (ewops.h:86), the row is divided
// by sum + 1e-6 (ewops.h:93), and O = P.V (matmul.h:6-20).
#include "tiles.hip.h"

#include <mutex>

#ifndef SFB_TILE_LOAD_ONCE
#define SFB_TILE_LOAD_ONCE 0   // 1: the fused bf16 kernel for head size 64 issues a tile's loads as one group (load_tile_once)
#endif
#ifndef SFB_TILE_LOAD_STAGED
#define SFB_TILE_LOAD_STAGED 0   // 1: ... brings the tiles of its loop in through registers (staged_fetch / staged_commit)
#endif
#include <type_traits>

namespace sfb {

struct FusedParams {
    const void* q;
    const void* k;
    const void* v;
    float* o;                       // fp32, or bf16 (o_bf16 != 0) behind the same pointer
    float* lse;                     // [batch][heads][ctx] base-2 log of each row's softmax denominator, or nullptr
    const sfb_uint2* nn_lut;
    const void* mask;               // block-major keep words, or nullptr
    const int32_t* valid_len;       // per batch, or nullptr
    const uint32_t* row_order;      // rank -> block-row (unscheduled launches), or nullptr
    const sfb_work_item* items;     // rank -> work item (scheduled launches), or nullptr
    const void* st_slots;           // streamed launches: sfb_stream_slot per resident work-group,
    const void* st_blocks;          //   sfb_stream_block, sfb_stream_item and sfb_stream_merge arrays
    const void* st_items;
    const void* st_merges;
    uint32_t* st_flags;             // one flag per partial record of a streamed launch
    uint32_t* st_status;            // set to 1 when a merge task's wait ran out
    uint32_t* counters;             // [batch*heads][n_slots] arrival counters of split rows
    float* partials;                // [batch*heads][n_parts][BS*D + 4*BS]
    uint32_t n_slots, n_parts;
    uint32_t o_bf16;                // output element type: 0 fp32, 1 bf16 (rounded once from the fp32 result)
    uint32_t batch, heads, nb, blocks;
    uint32_t state;                 // the tensors' head size; smaller than the kernel's (padded) one in ragged launches
    uint32_t in_stride;             // elements between the rows of consecutive tokens in Q, K and V (heads * d when dense)
    uint32_t lut_stride;            // entries between heads' LUTs (0 = shared)
    uint32_t item_stride;           // work items between heads' lists (0 = shared)
    uint32_t mask_stride;           // words between heads' masks (0 = shared)
    uint32_t groups;                // ceil(batch*heads / 8)
    uint32_t ranks;                 // work items per (batch, head)
    uint32_t heavy;                 // leading items issued for all heads first
    float scale_log2e;
    float scale_pow2;               // scale_log2e = scale_pow2 * scale_rest, scale_pow2 a power of two (exact on bf16 queries),
    float scale_rest;               //   scale_rest in [1/sqrt 2, sqrt 2)
    float slack;                    // raw-score distance a block maximum may exceed the reference maximum
};

// Element offset of (b, token, h, 0) in Q, K or V, whose token rows are p.in_stride elements apart.
__device__ __forceinline__ size_t input_offset(const FusedParams& p, uint32_t b, uint32_t token, uint32_t h, uint32_t L,
                                               uint32_t d) {
    return ((size_t)b * L + token) * p.in_stride + (size_t)h * d;
}

// What this work-group has to do.
struct RowWork {
    uint32_t bh, b, h, row;
    uint32_t first, count;          // key blocks [first, first+count) of the row's LUT segment
    uint32_t nchunks, slot, part;   // split rows: number of chunks, counter index, first partial index
    uint32_t chunk;
    uint32_t lut_first;             // index of the item's first entry in the head's NN LUT
    uint32_t valid;
};

__device__ __forceinline__ RowWork decode_row_work(const FusedParams& p) {
    RowWork w;
    const WorkId id = decode_work(blockIdx.x, p.batch * p.heads, p.ranks, p.heavy);
    w.valid = id.valid;
    w.bh = __builtin_amdgcn_readfirstlane(id.bh);
    w.b = __builtin_amdgcn_readfirstlane(id.bh / p.heads);
    w.h = __builtin_amdgcn_readfirstlane(id.bh % p.heads);
    if (p.items) {
        const sfb_work_item it = p.items[(size_t)(id.valid ? w.h : 0u) * p.item_stride + id.rank];
        if (it.row == SFB_WORK_ITEM_SKIP) w.valid = 0;   // filler of a head whose list is shorter than the longest
        w.row = it.row; w.first = it.first; w.count = it.count;
        w.nchunks = it.nchunks; w.slot = it.slot; w.part = it.part; w.chunk = it.chunk;
        w.lut_first = it.lut_first;
    } else {
        w.row = p.row_order ? p.row_order[id.rank] : (p.nb - 1 - id.rank);
        w.first = 0;
        const sfb_uint2 header = p.nn_lut[(size_t)w.h * p.lut_stride + (id.valid ? w.row : 0u)];
        w.count = id.valid ? header.y : 0;
        w.lut_first = header.x;
        w.nchunks = 1; w.slot = 0; w.part = 0; w.chunk = 0;
    }
    return w;
}

// LUT entries of key blocks [first, first + 64) of an item, one per lane (clamped to the item's last one).
__device__ __forceinline__ sfb_uint2 lut_window(const FusedParams& p, const RowWork& w, uint32_t first, uint32_t lane) {
    sfb_uint2 none = {0u, 0u};
    if (w.count == 0) return none;
    const uint32_t idx = first + lane;
    return p.nn_lut[(size_t)w.h * p.lut_stride + w.lut_first + (idx < w.count ? idx : w.count - 1)];
}

// The probabilities of a row are kept relative to a reference maximum m_used that is only moved
// when a block's maximum exceeds it by more than `slack` (2^8 in probability), so rescaling the
// output accumulators is rare.  m_true tracks the exact running maximum; the final normalisation
// uses both, which keeps the result identical to a softmax relative to the true maximum, including
// the +1e-6 term of the denominator.
struct RowState {
    float m_used;   // reference maximum the stored probabilities are relative to (raw units)
    float m_true;   // exact running maximum over kept keys, seeded like the CPU path
    float l;        // this lane's partial sum of probabilities relative to m_used
};

// Online-softmax step on one key block.  s[kt][i] holds, for this lane's query, the raw score of key
// kt*32 + (i/4)*8 + half*4 + i%4 and is overwritten by the unnormalised probability (PACK:
// pk[kt*8 + i/2] receives the pair (i, i+1) rounded to bf16 and the row sum is taken over those
// rounded values, i.e. over exactly what the P.V product uses).
template <int KT, int NO, bool PACK>
__device__ __forceinline__ void softmax_block(f32x16 (&s)[KT], uint32_t (&pk)[KT * 8], f32x16 (&o)[NO],
                                              RowState& st, float c, float slack, bool masked,
                                              uint64_t keep, uint32_t half) {
    if (masked) apply_keep<KT>(s, keep, half);
    const float mloc = block_row_max<KT>(s);
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

// o[mt][i] is output column mt*32 + (i/4)*8 + half*4 + i%4 of this lane's query row.
template <int NO, typename F>
__device__ __forceinline__ void for_each_out_vec(F&& f) {
#pragma unroll
    for (int mt = 0; mt < NO; ++mt)
#pragma unroll
        for (int ig = 0; ig < 4; ++ig) f(mt, ig);
}

// Normalise and store: the sum relative to the true maximum is total / f with
// f = 2^((m_true - m_used) c), hence O = acc / (total + 1e-6 f)  (ewops.h:93 divides by sum + 1e-6).
// Address of the output row of one query: o_row points at element 0 of the row in either element type.
__device__ __forceinline__ float* output_row(const FusedParams& p, size_t element_offset) {
    return (float*)((uint8_t*)p.o + element_offset * (p.o_bf16 ? 2u : 4u));
}

// lse_row (may be null): receives m_used c + log2(total + 1e-6 f), so that the normalised probability of a key
// with raw score s is exp2(s c - lse) -- what a backward pass needs to rebuild P without the row's other keys.
//
// The rows go to memory through a wave-private LDS slab (32 padded rows): straight from the accumulator layout a
// store instruction would touch all 32 rows of the wave with 32 bytes each; from the slab every instruction writes
// whole rows (1 KiB of 256-byte or 128-byte rows), as streaming (non-temporal) stores: O is written once and never
// read by this launch, so it should not displace the K and V blocks that later work-groups of the head find in the
// L2.  (Streaming stores of the 32-byte pieces were slower than cached ones; of whole rows they are faster.)
// o_row is this lane's own row, o_row_bytes the distance between the rows of consecutive queries; slab must hold
// 32 * (row size + 16) bytes and be free of other users.
// RAGGED (head sizes that are not a multiple of 32, computed by the kernel of the next multiple): only the first
// `hd` columns exist in memory; they are stored straight from the accumulators, four at a time.
template <int NO, bool RAGGED = false>
__device__ __forceinline__ void store_output(float* o_row, uint32_t o_row_bytes, uint32_t as_bf16, float* lse_row,
                                             f32x16 (&o)[NO], float m_used, float m_true, float total, float c,
                                             uint32_t lane, uint8_t* slab, uint32_t hd = NO * 32) {
    constexpr int D = NO * 32;
    const uint32_t qn = lane & 31, half = lane >> 5;
    const float f = exp2_fast((m_true - m_used) * c);
    const float inv = 1.0f / (total + 1e-6f * f);
    if (lse_row != nullptr && half == 0) *lse_row = __builtin_fmaf(m_used, c, __builtin_log2f(total + 1e-6f * f));
    if constexpr (RAGGED) {
        for_each_out_vec<NO>([&](int mt, int ig) {
            const uint32_t col = mt * 32 + ig * 8 + half * 4;
            if (col >= hd) return;
            const f32x4 out = {o[mt][ig * 4 + 0] * inv, o[mt][ig * 4 + 1] * inv, o[mt][ig * 4 + 2] * inv,
                               o[mt][ig * 4 + 3] * inv};
            if (as_bf16) {
                const u32x2 packed = {pack_bf16(out.x, out.y), pack_bf16(out.z, out.w)};
                *(u32x2*)((uint8_t*)o_row + col * 2) = packed;
            } else {
                *(f32x4*)(o_row + col) = out;
            }
        });
        return;
    }
    uint8_t* const wave_rows = (uint8_t*)o_row - (size_t)qn * o_row_bytes;   // row of the wave's first query
    const uint32_t pitch = as_bf16 ? D * 2 + 16 : D * 4 + 16;
    uint8_t* const mine = slab + qn * pitch;
    for_each_out_vec<NO>([&](int mt, int ig) {
        const f32x4 out = {o[mt][ig * 4 + 0] * inv, o[mt][ig * 4 + 1] * inv, o[mt][ig * 4 + 2] * inv,
                           o[mt][ig * 4 + 3] * inv};
        const uint32_t col = mt * 32 + ig * 8 + half * 4;
        if (as_bf16) {
            const u32x2 packed = {pack_bf16(out.x, out.y), pack_bf16(out.z, out.w)};
            *(u32x2*)(mine + col * 2) = packed;
        } else {
            *(f32x4*)(mine + col * 4) = out;
        }
    });
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (as_bf16) {
        constexpr int CHUNKS = D / 8;   // 16-byte chunks per row
#pragma unroll
        for (int pass = 0; pass < CHUNKS / 2; ++pass) {
            const uint32_t idx = pass * 64 + lane, row = idx / CHUNKS, ch = idx % CHUNKS;
            __builtin_nontemporal_store(*(const u32x4*)(slab + row * pitch + ch * 16), (u32x4*)(wave_rows + (size_t)row * o_row_bytes + ch * 16));
        }
    } else {
        constexpr int CHUNKS = D / 4;
#pragma unroll
        for (int pass = 0; pass < CHUNKS / 2; ++pass) {
            const uint32_t idx = pass * 64 + lane, row = idx / CHUNKS, ch = idx % CHUNKS;
            __builtin_nontemporal_store(*(const u32x4*)(slab + row * pitch + ch * 16), (u32x4*)(wave_rows + (size_t)row * o_row_bytes + ch * 16));
        }
    }
}

// Partial records are exchanged between work-groups of one launch.  They are written with
// device-scope write-through stores and read with relaxed device-scope atomic loads, both of which
// act at the level of the memory system that is coherent for the whole device, so no cache
// write-back or invalidation is needed; the writer only has to wait until its stores have completed
// before it bumps the row's counter.
__device__ __forceinline__ void coherent_store4(float* p, f32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ float coherent_load(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// two consecutive floats (8-byte aligned) in one access
__device__ __forceinline__ f32x2 coherent_load2(const float* p) {
    const uint64_t bits = __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __builtin_bit_cast(f32x2, bits);
}
// Partial-record offset (floats) of output vector (mt, ig) of a lane: vectors of one (mt, ig, half)
// are contiguous over the block's queries, so every store instruction writes whole lines.
template <int BS>
__device__ __forceinline__ uint32_t partial_offset(int mt, int ig, uint32_t half, uint32_t q_in_block) {
    return (((mt * 4 + ig) * 2 + half) * BS + q_in_block) * 4;
}

template <int BS, int D, bool RAGGED = false>
__device__ __forceinline__ void merge_partials(const float* base, uint32_t nchunks, float* o_row, uint32_t o_row_bytes,
                                               uint32_t as_bf16, float* lse_row, float c, uint32_t q_in_block,
                                               uint32_t lane, uint8_t* slab, uint32_t hd = D);

// End of a work item.  Unsplit rows are normalised and stored.  A chunk of a split row writes its
// partial (unnormalised O, reference maximum, true maximum, sum) and bumps the row's counter; the
// chunk that finds every other chunk already arrived merges all partials, stores O and resets the
// counter for the next launch.  Nobody waits.  lds: shared memory of the work-group that nobody uses any more, at
// least 32 * (row size + 16) bytes per wave (the output rows pass through it).
template <int BS, int D, bool RAGGED = false>
__device__ __forceinline__ void finish_row(const FusedParams& p, const RowWork& w, float* o_row,
                                           f32x16 (&o)[D / 32], const RowState& st, float c,
                                           uint32_t q_in_block, uint32_t half, uint32_t t, uint8_t* lds) {
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const uint32_t lane = t & 63, o_row_bytes = p.heads * hd * (p.o_bf16 ? 2u : 4u);
    uint8_t* const slab = lds + (t >> 6) * (32u * (D * 4 + 16));
    float* const lse_row = p.lse ? p.lse + ((size_t)w.bh * p.nb + w.row) * BS + q_in_block : nullptr;
    constexpr int NO = D / 32;
    constexpr int PART = BS * D + 4 * BS;   // floats per partial
    const float total = st.l + __shfl_xor(st.l, 32);
    if (w.nchunks <= 1) {
        store_output<NO, RAGGED>(o_row, o_row_bytes, p.o_bf16, lse_row, o, st.m_used, st.m_true, total, c, lane, slab, hd);
        return;
    }
    float* base = p.partials + ((size_t)w.bh * p.n_parts + w.part) * PART;
    {
        float* mine = base + (size_t)w.chunk * PART;
        for_each_out_vec<NO>([&](int mt, int ig) {
            const f32x4 out = {o[mt][ig * 4 + 0], o[mt][ig * 4 + 1], o[mt][ig * 4 + 2], o[mt][ig * 4 + 3]};
            coherent_store4(mine + partial_offset<BS>(mt, ig, half, q_in_block), out);
        });
        if (half == 0) {
            const f32x4 sv = {st.m_used, st.m_true, total, 0.f};
            coherent_store4(mine + BS * D + q_in_block * 4, sv);
        }
    }
    __shared__ uint32_t last_flag;
    // every wave waits for its own stores to complete, then the barrier collects the waves
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
    __syncthreads();
    uint32_t* counter = p.counters + (size_t)w.bh * p.n_slots + w.slot;
    if (t == 0) {
        const uint32_t seen = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = (seen == w.nchunks - 1) ? 1u : 0u;
    }
    __syncthreads();
    if (!last_flag) return;
    merge_partials<BS, D, RAGGED>(base, w.nchunks, o_row, o_row_bytes, p.o_bf16, lse_row, c, q_in_block, lane, slab, hd);
    if (t == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Merge of the partial records of a split row (run by the chunk that arrived last).
template <int BS, int D, bool RAGGED>
__device__ __forceinline__ void merge_partials(const float* base, uint32_t nchunks, float* o_row, uint32_t o_row_bytes,
                                               uint32_t as_bf16, float* lse_row, float c, uint32_t q_in_block,
                                               uint32_t lane, uint8_t* slab, uint32_t hd) {
    const uint32_t half = lane >> 5;
    constexpr int NO = D / 32;
    constexpr int PART = BS * D + 4 * BS;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    float m_used = kMaxSeed, m_true = kMaxSeed;
    for (uint32_t ch = 0; ch < nchunks; ++ch) {
        const float* stats = base + (size_t)ch * PART + BS * D + q_in_block * 4;
        m_used = fmaxf(m_used, coherent_load(stats + 0));
        m_true = fmaxf(m_true, coherent_load(stats + 1));
    }
    f32x16 acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[n][i] = 0.f;
    float sum = 0.f;
    for (uint32_t ch = 0; ch < nchunks; ++ch) {
        const float* part = base + (size_t)ch * PART;
        const float* stats = part + BS * D + q_in_block * 4;
        const float wgt = exp2_fast((coherent_load(stats + 0) - m_used) * c);
        sum += coherent_load(stats + 2) * wgt;
        for_each_out_vec<NO>([&](int mt, int ig) {
            const float* src = part + partial_offset<BS>(mt, ig, half, q_in_block);
            const f32x2 lo = coherent_load2(src), hi = coherent_load2(src + 2);
            acc[mt][ig * 4 + 0] += lo.x * wgt;
            acc[mt][ig * 4 + 1] += lo.y * wgt;
            acc[mt][ig * 4 + 2] += hi.x * wgt;
            acc[mt][ig * 4 + 3] += hi.y * wgt;
        });
    }
    store_output<NO, RAGGED>(o_row, o_row_bytes, as_bf16, lse_row, acc, m_used, m_true, sum, c, lane, slab, hd);
}

// the same for a row of hd elements (hd a multiple of 4): the two lanes of a query take alternate groups of 4
__device__ __forceinline__ void store_zero_row_ragged(float* o_row, uint32_t as_bf16, uint32_t half, uint32_t hd) {
    for (uint32_t col = half * 4; col < hd; col += 8) {
        if (as_bf16) {
            const u32x2 zero = {0u, 0u};
            *(u32x2*)((uint8_t*)o_row + col * 2) = zero;
        } else {
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            *(f32x4*)(o_row + col) = zero;
        }
    }
}

template <int D>
__device__ __forceinline__ void store_zero_row(float* o_row, uint32_t as_bf16, uint32_t half) {
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    // this lane's half of the row: D/2 elements = D/8 (fp32) or D/16 (bf16) 16-byte stores
    uint8_t* dst = (uint8_t*)o_row + half * (D / 2) * (as_bf16 ? 2 : 4);
    const int n = as_bf16 ? D / 16 : D / 8;
    for (int x = 0; x < n; ++x) *(f32x4*)(dst + x * 16) = zero;
}

// ------------------------------------------------------------------------------------------------
// bf16 inputs, fp32 accumulation: v_mfma_f32_32x32x16_bf16
// ------------------------------------------------------------------------------------------------
// Exponentials of chunk u (16 keys) of a score block: pk[4u .. 4u+3] receive the probabilities rounded to
// bf16, in the order the P^T operand of product step u wants them; the row sum is taken over the rounded
// values, i.e. over exactly what the P.V product uses.
template <int KT, int NO>
__device__ __forceinline__ void exp_chunk(const f32x16 (&s)[KT], uint32_t (&pk)[KT * 8], int u, float c,
                                          float mc, float& sum0, float& sum1) {
    const int kt = u / 2, i0 = (u % 2) * 8;
    const float p0 = exp2_fast(__builtin_fmaf(s[kt][i0 + 0], c, -mc));
    const float p1 = exp2_fast(__builtin_fmaf(s[kt][i0 + 1], c, -mc));
    const float p2 = exp2_fast(__builtin_fmaf(s[kt][i0 + 2], c, -mc));
    const float p3 = exp2_fast(__builtin_fmaf(s[kt][i0 + 3], c, -mc));
    const float p4 = exp2_fast(__builtin_fmaf(s[kt][i0 + 4], c, -mc));
    const float p5 = exp2_fast(__builtin_fmaf(s[kt][i0 + 5], c, -mc));
    const float p6 = exp2_fast(__builtin_fmaf(s[kt][i0 + 6], c, -mc));
    const float p7 = exp2_fast(__builtin_fmaf(s[kt][i0 + 7], c, -mc));
    const uint32_t a = pack_bf16(p0, p1), b = pack_bf16(p2, p3), d = pack_bf16(p4, p5), e = pack_bf16(p6, p7);
    pk[u * 4 + 0] = a; pk[u * 4 + 1] = b; pk[u * 4 + 2] = d; pk[u * 4 + 3] = e;
    sum0 = dot2_bf16_ones(a, sum0);
    sum1 = dot2_bf16_ones(b, sum1);
    sum0 = dot2_bf16_ones(d, sum0);
    sum1 = dot2_bf16_ones(e, sum1);
}

// The same for scores that carry the power-of-two part of the scale and the row's offset already (folded into the
// score product): one multiplication by the rest of the scale and one exponential per element; the row sum is
// taken over the fp32 values with plain additions, which -- unlike v_dot2c -- run while the matrix pipe is busy.
template <int KT>
__device__ __forceinline__ void exp_chunk_slim(const f32x16 (&s)[KT], uint32_t (&pk)[KT * 8], int u, float r, float& sum0,
                                               float& sum1) {
    const int kt = u / 2, i0 = (u % 2) * 8;
    const float p0 = exp2_fast(s[kt][i0 + 0] * r), p1 = exp2_fast(s[kt][i0 + 1] * r);
    const float p2 = exp2_fast(s[kt][i0 + 2] * r), p3 = exp2_fast(s[kt][i0 + 3] * r);
    const float p4 = exp2_fast(s[kt][i0 + 4] * r), p5 = exp2_fast(s[kt][i0 + 5] * r);
    const float p6 = exp2_fast(s[kt][i0 + 6] * r), p7 = exp2_fast(s[kt][i0 + 7] * r);
    pk[u * 4 + 0] = pack_bf16(p0, p1); pk[u * 4 + 1] = pack_bf16(p2, p3);
    pk[u * 4 + 2] = pack_bf16(p4, p5); pk[u * 4 + 3] = pack_bf16(p6, p7);
    sum0 += (p0 + p2) + (p4 + p6);
    sum1 += (p1 + p3) + (p5 + p7);
}

// q * c as bf16 (round to nearest even).  The kernels call it with a power of two, for which the product is exact
// (short of the exponent range's ends): the scores it leads to are then as exact as those of unscaled queries.
__device__ __forceinline__ bf16x8 scale_bf16x8(bf16x8 q, float c) {
    const u32x4 bits = __builtin_bit_cast(u32x4, q);
    u32x4 out;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        out[i] = pack_bf16(bf16_bits_to_f32(bits[i] & 0xffffu) * c, __builtin_bit_cast(float, bits[i] & 0xffff0000u) * c);
    return __builtin_bit_cast(bf16x8, out);
}

// The order in which the instructions of the chunks of one key block are to be issued (slim loop): the LDS reads of
// chunk u + 1 ahead of the matrix instructions of chunk u, and behind every matrix instruction an equal share of the
// vector work -- first the packing and adding of exponentials that were issued a slot earlier (their results are
// ready by then) and the multiplications that feed the next exponentials, then those exponentials.
template <int BS, int D>
__device__ __forceinline__ void schedule_chunks() {
    constexpr int KT = BS / 32, NO = D / 32, KS = D / 16, PU = BS / 16, KPC = KS / PU;
    constexpr int MF = KPC * KT + NO;                    // matrix instructions per chunk
    constexpr int DS = KPC * KT + 2 * NO;                // LDS reads per chunk
    constexpr int EXP = BS / 2 / PU / MF;                // exponentials per slot (BS/2 elements per lane and key block)
    constexpr int REST = (BS / 4 + BS / 2 + BS / 2) / PU / MF;   // pack + add + multiply per slot
#pragma unroll
    for (int u = 0; u < PU; ++u) {
        if (u + 1 < PU) __builtin_amdgcn_sched_group_barrier(0x100, DS, 0);
#pragma unroll
        for (int m = 0; m < MF; ++m) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (u > 0 || m > 0) {
                if (u + 1 < PU || m == 0) __builtin_amdgcn_sched_group_barrier(0x002, REST, 0);
            }
            if (u + 1 < PU) __builtin_amdgcn_sched_group_barrier(0x400, EXP, 0);
        }
    }
}

// K and V tiles of a key block are fetched with LDS-direct loads into swizzled row-major buffers (see
// Bf16DirectTiles; no staging registers, no LDS writes by the waves), V^T fragments come from transposing
// LDS reads.  Software pipeline over the key blocks of the item; in iteration j a wave
//   * issues the loads of K(j+2) and V(j+1) into the buffers that iteration j-1 finished reading;
//   * finds the row maximum of S(j), then, chunk by chunk, exponentiates S(j), feeds V(j)^T . P^T and
//     computes a slice of S(j+1) = K(j+1) . Q^T;
//   * waits for its own loads and meets the other waves at the one barrier of the iteration.
// SLIM (launches without element mask and key padding): the probabilities of the whole item are taken relative to
// one fixed offset, the row maximum of the item's first key block, so the loop needs no per-block maximum and never
// rescales its accumulators.  The offset is a real score of the row, hence the row sum is at least about 1 and cannot
// vanish; a later block whose scores exceed the offset by more than 2^100 in probability makes the sum overflow,
// which the end of the item detects, and the item is then redone by the general loop (returns false).  The 1e-6 of
// the reference's denominator is applied relative to the offset instead of the true row maximum, a relative
// difference of at most 1e-6.
//
// finish(o_acc, st) ends the item: it gets the unnormalised output accumulators and the row state (maxima in raw-score
// units, this lane's part of the sum).
// RAGGED: the tensors' head size p.state is smaller than D (a multiple of 8 above D - 32): queries are padded with
// zeros, the tiles' last slice holds filler beyond the row's features, only p.state output columns are stored.
template <int BS, int D, bool MASKED, bool SLIM, bool RAGGED = false, typename Finish>
__device__ __forceinline__ bool attend_item_bf16(const FusedParams& p, const RowWork& w, uint8_t* smem, uint32_t* retry_flag,
                                                 sfb_uint2 first_window, Finish&& finish) {
    using T = Bf16DirectTiles<BS, D>;
    constexpr int KT = BS / 32, NO = D / 32, KS = D / 16, PU = BS / 16;
    constexpr int TILE = T::TILE_BYTES;
    constexpr int SC = PU >= 2 ? PU / 2 : 1;   // chunks that carry a slice of the next block's scores
    static_assert(!(MASKED && SLIM), "masked launches take the general loop");
    static_assert(!(RAGGED && SLIM), "ragged head sizes take the general loop");

    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t qn = lane & 31, half = lane >> 5;
    const uint32_t q_in_block = wave * 32 + qn;
    const uint32_t row_bytes = p.in_stride * 2;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;

    const uint32_t count = __builtin_amdgcn_readfirstlane(w.count);
    float* o_row = output_row(p, token_offset(w.b, w.row * BS + q_in_block, w.h, L, p.heads, hd));

    const __bf16* Q = (const __bf16*)p.q;
    const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)w.h * p.mask_stride * (BS / 8) : nullptr;
    const int valid = p.valid_len ? p.valid_len[w.b] : (int)L;

    // byte address of (b, token 0, h, 0) in K and V; key block column col starts col*BS rows further
    const size_t bh_bytes = input_offset(p, w.b, 0, w.h, L, hd) * 2;
    const uint8_t* const k_base = (const uint8_t*)p.k + bh_bytes;
    const uint8_t* const v_base = (const uint8_t*)p.v + bh_bytes;
    const typename T::Sources src = RAGGED ? T::sources_ragged(lane, row_bytes, hd) : T::sources(lane, row_bytes);
#if SFB_TILE_LOAD_ONCE
    // experimental form of the tile loads (one M0 write and one scalar address per tile), head size 64 only
    constexpr bool kOnce = D == 64 && !RAGGED;
    typename T::OnceSources once;
    if constexpr (kOnce) once = T::once_sources(lane, wave, row_bytes);
#else
    constexpr bool kOnce = false;
#endif
#if SFB_TILE_LOAD_STAGED
    // experimental: the loop's tiles go through registers; the prologue keeps the LDS-direct loads
    constexpr bool kStaged = D == 64 && !RAGGED;
    const uint32_t staged_src = T::I::staged_source(lane, row_bytes);
    const uint32_t staged_even = T::I::staged_lds_offset(lane, 0), staged_odd = T::I::staged_lds_offset(lane, 1);
#else
    constexpr bool kStaged = false;
#endif
    const uint32_t lds0 = T::lds_address(smem);
    // LUT entries of key blocks [win, win + 64) of this item, one per lane (clamped to the last one)
    uint32_t win = 0;
    sfb_uint2 entries = first_window;
    auto refill = [&](uint32_t first) {
        win = first;
        entries = lut_window(p, w, first, lane);
    };
    auto column_of = [&](uint32_t j) -> uint32_t {
        const uint32_t jj = j < count ? j : count - 1;
        return __builtin_amdgcn_readlane(entries.y, jj - win);
    };
    auto load_tile = [&](uint32_t dst, const uint8_t* g_tile) {
#if SFB_TILE_LOAD_ONCE
        if constexpr (kOnce) {
            T::load_tile_once(dst, g_tile, wave, once, row_bytes);
            return;
        }
#endif
        T::template load_tile_all<RAGGED>(dst, g_tile, wave, src, row_bytes);
    };
    auto load_k = [&](uint32_t j, uint32_t buf) {
        load_tile(lds0 + buf * TILE, k_base + (size_t)column_of(j) * BS * row_bytes);
    };
    auto load_v = [&](uint32_t j, uint32_t buf) {
        load_tile(lds0 + (2 + buf) * TILE, v_base + (size_t)column_of(j) * BS * row_bytes);
    };
    auto loads_landed = [&]() {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    };

    load_k(0, 0);
    load_v(0, 0);
    load_k(1, 1);
    if (SLIM && t == 0) *retry_flag = 0;
    const float c = p.scale_log2e, slack = p.slack;

    bf16x8 qf[KS];
    if constexpr (RAGGED) T::load_q_ragged(qf, Q + input_offset(p, w.b, w.row * BS + q_in_block, w.h, L, hd), half, hd);
    else T::load_q(qf, Q + input_offset(p, w.b, w.row * BS + q_in_block, w.h, L, D), half);
    const float c2 = p.scale_pow2, rest = p.scale_rest;
    if constexpr (SLIM) {
        // The score product then delivers base-2 exponents up to the factor `rest`.  Only the power-of-two part of
        // the scale goes into the queries: that product is exact, whereas rounding q * scale * log2(e) to bf16 a
        // second time moves every exponent by up to 2^-9 of the products it is made of -- an error that grows with
        // the scores and passes the tolerance for peaked rows (|score * scale| of a few tens).
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[ks] = scale_bf16x8(qf[ks], c2);
    }
    const uint32_t k_lane = T::k_lane_base(qn, half), v_lane = T::v_lane_base(lane);

    f32x16 o_acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[n][i] = 0.f;
    RowState st = {kMaxSeed, kMaxSeed, 0.f};

    f32x16 s_even[KT], s_odd[KT];
    loads_landed();
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s_even[kt][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            s_even[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::k_frag(smem, k_lane, kt, ks), qf[ks], s_even[kt], 0, 0, 0);
    }
    // SLIM: -offset in every element, the accumulator input of each later block's first product step
    f32x16 off_vec;
    if constexpr (SLIM) {
        const float m_scaled = block_row_max<KT>(s_even);
        st.m_used = st.m_true = m_scaled / c2;
#pragma unroll
        for (int i = 0; i < 16; ++i) off_vec[i] = -m_scaled;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) s_even[kt] += off_vec;
    }
    __syncthreads();   // every wave has read K(0) before iteration 0 overwrites its buffer

    auto iteration = [&](uint32_t j, f32x16 (&s)[KT], f32x16 (&s_next)[KT]) {
        const uint32_t par = j & 1;
        const uint8_t* const k_read = smem + (par ^ 1) * TILE;       // K(j+1)
        const uint8_t* const v_read = smem + (2 + par) * TILE;       // V(j)
        if (j + 2 >= win + 64) refill(j);
        // K(j+2) replaces K(j), V(j+1) replaces V(j-1); the loads are issued right after the first exponentials
        // (behind the row maximum, which the next instructions depend on) so that they have the whole
        // iteration to land: issued later, spread over the chunks, the last of them were still in flight at
        // the end of the iteration and every wave waited for them there
        const uint8_t* const k_src = k_base + (size_t)column_of(j + 2) * BS * row_bytes;
        const uint8_t* const v_src = v_base + (size_t)column_of(j + 1) * BS * row_bytes;
        const uint32_t k_dst = lds0 + par * TILE, v_dst = lds0 + (2 + (par ^ 1)) * TILE;

        if (MASKED) {
            const sfb_uint2 here = {(uint32_t)__builtin_amdgcn_readlane(entries.x, j - win),
                                    (uint32_t)__builtin_amdgcn_readlane(entries.y, j - win)};
            const int limit = valid - (int)(here.y * BS);
            if ((mask != nullptr) || (limit < BS)) {
                // most blocks of a causal or padded layout keep every key: the per-element selection is only done
                // when some lane of the wave has a key to drop
                const uint64_t keep = load_keep_word<BS>(mask, (size_t)here.x * BS + q_in_block, limit);
                constexpr uint64_t kAll = BS == 64 ? ~0ull : 0xffffffffull;
                if (__builtin_amdgcn_ballot_w64((keep & kAll) != kAll) != 0) apply_keep<KT>(s, keep, half);
            }
        }
        if constexpr (!SLIM) {
            const float mloc = block_row_max<KT>(s);
            st.m_true = fmaxf(st.m_true, mloc);
            if (__builtin_amdgcn_ballot_w64(mloc > st.m_used + slack) != 0) {
                const float m_new = fmaxf(st.m_used, mloc);
                const float alpha = exp2_fast((st.m_used - m_new) * c);
                st.m_used = m_new;
                st.l *= alpha;
#pragma unroll
                for (int n = 0; n < NO; ++n) o_acc[n] *= alpha;
            }
        }
        const float mc = st.m_used * c;
        float sum0 = 0.f, sum1 = 0.f;
        uint32_t pk[KT * 8];
        auto exps = [&](int u) {
            if constexpr (SLIM) exp_chunk_slim<KT>(s, pk, u, rest, sum0, sum1);
            else exp_chunk<KT, NO>(s, pk, u, c, mc, sum0, sum1);
        };
        // Every chunk carries the same work: the exponentials of the next chunk, one slice (KS / PU product steps) of
        // the next block's scores and one step of the output product.  The fragments of a chunk are requested from
        // LDS one chunk ahead of the matrix instructions that consume them.
        // (chunk u takes steps u*KS/PU .. (u+1)*KS/PU - 1: one each for 64 features and 64 keys, up to two
        // otherwise)
        constexpr int KPC = (KS + PU - 1) / PU;   // most score product steps of a chunk
        bf16x8 kfr[PU][KPC][KT], vfr[PU][NO];
        auto fragments = [&](int u) {
#pragma unroll
            for (int kk = 0; kk < KPC; ++kk)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
                    if (u * KS / PU + kk < (u + 1) * KS / PU) kfr[u][kk][kt] = T::k_frag(k_read, k_lane, kt, u * KS / PU + kk);
#pragma unroll
            for (int mt = 0; mt < NO; ++mt) vfr[u][mt] = T::v_frag(v_read, v_lane, mt, u);
        };
        fragments(0);
        exps(0);
#if SFB_TILE_LOAD_STAGED
        typename T::Staged k_staged, v_staged;
        if constexpr (kStaged) {
            T::staged_fetch(k_staged, k_src, wave, staged_src, row_bytes);
            T::staged_fetch(v_staged, v_src, wave, staged_src, row_bytes);
        } else
#endif
        if constexpr (kOnce) {
            load_tile(k_dst, k_src);
            load_tile(v_dst, v_src);
        } else {
#pragma unroll
            for (int i = 0; i < T::LOADS; ++i) {
                T::template load_rows_all<RAGGED>(k_dst, k_src, i, wave, src, row_bytes);
                T::template load_rows_all<RAGGED>(v_dst, v_src, i, wave, src, row_bytes);
            }
        }
        if constexpr (SLIM) __builtin_amdgcn_sched_barrier(0);   // the tile loads are issued here, not later
#pragma unroll
        for (int u = 0; u < PU; ++u) {
            if (u + 1 < PU) {
                fragments(u + 1);
                exps(u + 1);
            }
#pragma unroll
            for (int kk = 0; kk < KPC; ++kk)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
                    const int ks = u * KS / PU + kk;
                    if (ks >= (u + 1) * KS / PU) continue;
                    if (ks == 0) {
                        const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                        s_next[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[u][kk][kt], qf[ks], SLIM ? off_vec : zero, 0, 0, 0);
                    } else {
                        s_next[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[u][kk][kt], qf[ks], s_next[kt], 0, 0, 0);
                    }
                }
            const u32x4 pb = {pk[u * 4 + 0], pk[u * 4 + 1], pk[u * 4 + 2], pk[u * 4 + 3]};
            const bf16x8 bfrag = __builtin_bit_cast(bf16x8, pb);
#pragma unroll
            for (int mt = 0; mt < NO; ++mt)
                o_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr[u][mt], bfrag, o_acc[mt], 0, 0, 0);
        }
        if constexpr (SLIM && D == 64) {
            schedule_chunks<BS, D>();   // issue order worked out for this head size
        }
        st.l += sum0 + sum1;
        if constexpr (SLIM) __builtin_amdgcn_sched_barrier(0);   // the wait for the tiles comes last
#if SFB_TILE_LOAD_STAGED
        if constexpr (kStaged) {
            // K(j) and V(j-1), whose buffers these tiles take, were last read in iteration j-1, before its barrier
            T::staged_commit(k_staged, smem + par * TILE, wave, staged_even, staged_odd);
            T::staged_commit(v_staged, smem + (2 + (par ^ 1)) * TILE, wave, staged_even, staged_odd);
        }
#endif
        loads_landed();
    };

    for (uint32_t j = 0; j < count; j += 2) {
        iteration(j, s_even, s_odd);
        if (j + 1 < count) iteration(j + 1, s_odd, s_even);
    }

    if constexpr (SLIM) {
        const float total = st.l + __shfl_xor(st.l, 32);
        if (__builtin_amdgcn_ballot_w64(!(total < 0x1p100f)) != 0 && lane == 0) *retry_flag = 1;   // overflow, or NaN
        __syncthreads();
        if (*retry_flag != 0) return false;
    }
    finish(o_acc, st);
    return true;
}

template <int BS, int D, bool MASKED, bool RAGGED = false>
__global__ __launch_bounds__(BS * 2, D > 64 ? 1 : 2) void fused_attention_bf16_kernel(FusedParams p) {
    using T = Bf16DirectTiles<BS, D>;
    constexpr int TILE = T::TILE_BYTES;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[4 * TILE];   // K0 K1 V0 V1
    __shared__ uint32_t retry_flag;
    static_assert(4 * TILE >= BS * (D * 4 + 16), "the tiles' memory doubles as the output slabs");

    const uint32_t lane = threadIdx.x & 63;
    const RowWork w = decode_row_work(p);
    if (!w.valid) return;
    const uint32_t L = p.nb * BS, q_in_block = (threadIdx.x >> 6) * 32 + (lane & 31);
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    float* o_row = output_row(p, token_offset(w.b, w.row * BS + q_in_block, w.h, L, p.heads, hd));
    if (w.count == 0) {
        if constexpr (RAGGED) store_zero_row_ragged(o_row, p.o_bf16, lane >> 5, hd);
        else store_zero_row<D>(o_row, p.o_bf16, lane >> 5);
        if (p.lse && (lane >> 5) == 0) p.lse[((size_t)w.bh * p.nb + w.row) * BS + q_in_block] = 0.f;
        return;
    }
    const sfb_uint2 window = lut_window(p, w, 0, lane);
    auto finish = [&](f32x16 (&o_acc)[D / 32], const RowState& st) {
        finish_row<BS, D, RAGGED>(p, w, o_row, o_acc, st, p.scale_log2e, q_in_block, lane >> 5, threadIdx.x, smem);
    };
    if constexpr (!MASKED && !RAGGED) {
        if (attend_item_bf16<BS, D, false, true>(p, w, smem, &retry_flag, window, finish)) return;
    }
    attend_item_bf16<BS, D, MASKED, false, RAGGED>(p, w, smem, &retry_flag, window, finish);
}

// ------------------------------------------------------------------------------------------------
// fp32 inputs: v_mfma_f32_32x32x2_f32 (true fp32 products and accumulation)
// ------------------------------------------------------------------------------------------------
// One LDS buffer (K tile and V tile); the next block waits in registers.
template <int BS, int D, bool RAGGED = false, typename Finish>
__device__ __forceinline__ void attend_item_f32(const FusedParams& p, const RowWork& w, float* k_lds, float* v_lds,
                                                Finish&& finish) {
    using T = F32Tiles<BS, D>;
    constexpr int KT = BS / 32;
    constexpr int NO = D / 32;
    constexpr int QG = D / 8;        // float4 groups of Q per lane
    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint32_t qn = lane & 31, half = lane >> 5;
    const uint32_t q_in_block = wave * 32 + qn;
    const uint32_t row_stride = p.in_stride;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;

    const sfb_uint2* lut = p.nn_lut + (size_t)w.h * p.lut_stride;
    const uint32_t lut_off = w.lut_first, count = w.count;
    float* o_row = output_row(p, token_offset(w.b, w.row * BS + q_in_block, w.h, L, p.heads, hd));

    if (count == 0) {
        if constexpr (RAGGED) store_zero_row_ragged(o_row, p.o_bf16, half, hd);
        else store_zero_row<D>(o_row, p.o_bf16, half);
        if (p.lse && half == 0) p.lse[((size_t)w.bh * p.nb + w.row) * BS + q_in_block] = 0.f;
        return;
    }

    const float* Q = (const float*)p.q;
    const float* K = (const float*)p.k;
    const float* V = (const float*)p.v;
    const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)w.h * p.mask_stride * (BS / 8) : nullptr;
    const int valid = p.valid_len ? p.valid_len[w.b] : (int)L;

    f32x4 qf[QG];
    if constexpr (RAGGED) T::load_q_ragged(qf, Q + input_offset(p, w.b, w.row * BS + q_in_block, w.h, L, hd), half, hd);
    else T::load_q(qf, Q + input_offset(p, w.b, w.row * BS + q_in_block, w.h, L, D), half);

    typename T::Regs gk, gv;

    f32x16 o_acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[n][i] = 0.f;
    RowState st = {kMaxSeed, kMaxSeed, 0.f};
    const float c = p.scale_log2e, slack = p.slack;

    sfb_uint2 entry = lut[lut_off];
    {
        const size_t base = input_offset(p, w.b, entry.y * BS, w.h, L, hd);
        if constexpr (RAGGED) {
            T::fetch_ragged(gk, K, base, row_stride, t, hd);
            T::fetch_ragged(gv, V, base, row_stride, t, hd);
        } else {
            T::fetch(gk, K, base, row_stride, t);
            T::fetch(gv, V, base, row_stride, t);
        }
    }

    for (uint32_t j = 0; j < count; ++j) {
        const sfb_uint2 here = entry;
        T::template stage<T::K_STRIDE>(k_lds, gk, t);
        T::template stage<T::V_STRIDE>(v_lds, gv, t);
        __syncthreads();
        if (j + 1 < count) {
            entry = lut[lut_off + j + 1];
            const size_t base = input_offset(p, w.b, entry.y * BS, w.h, L, hd);
            if constexpr (RAGGED) {
                T::fetch_ragged(gk, K, base, row_stride, t, hd);
                T::fetch_ragged(gv, V, base, row_stride, t, hd);
            } else {
                T::fetch(gk, K, base, row_stride, t);
                T::fetch(gv, V, base, row_stride, t);
            }
        }

        f32x16 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 16; ++i) s[kt][i] = 0.f;
#pragma unroll
        for (int g = 0; g < QG; ++g) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const f32x4 a = T::k_frag(k_lds, kt, g, qn, half);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    s[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], qf[g][e], s[kt], 0, 0, 0);
            }
        }

        const int limit = valid - (int)(here.y * BS);
        const bool masked = (mask != nullptr) || (limit < BS);
        uint64_t keep = ~0ull;
        if (masked) keep = load_keep_word<BS>(mask, (size_t)here.x * BS + q_in_block, limit);
        uint32_t pk_unused[KT * 8];
        softmax_block<KT, NO, false>(s, pk_unused, o_acc, st, c, slack, masked, keep, half);

#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 16; ++i)
#pragma unroll
                for (int mt = 0; mt < NO; ++mt)
                    o_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(T::v_elem(v_lds, kt, i, mt, qn, half),
                                                                     s[kt][i], o_acc[mt], 0, 0, 0);
        __syncthreads();
    }

    finish(o_acc, st);
}

template <int BS, int D, bool RAGGED = false>
__global__ __launch_bounds__(BS * 2, D > 64 ? 1 : 2) void fused_attention_f32_kernel(FusedParams p) {
    using T = F32Tiles<BS, D>;
    __shared__ __attribute__((aligned(16))) float k_lds[T::K_FLOATS];
    __shared__ __attribute__((aligned(16))) float v_lds[T::V_FLOATS];
    static_assert(T::K_FLOATS * 4 >= BS * (D * 4 + 16), "the K tile's memory doubles as the output slabs");
    const RowWork w = decode_row_work(p);
    if (!w.valid) return;
    const uint32_t t = threadIdx.x, lane = t & 63, q_in_block = (t >> 6) * 32 + (lane & 31);
    float* o_row = output_row(p, token_offset(w.b, w.row * BS + q_in_block, w.h, p.nb * BS, p.heads, RAGGED ? p.state : (uint32_t)D));
    attend_item_f32<BS, D, RAGGED>(p, w, k_lds, v_lds, [&](f32x16 (&o_acc)[D / 32], const RowState& st) {
        finish_row<BS, D, RAGGED>(p, w, o_row, o_acc, st, p.scale_log2e, q_in_block, lane >> 5, t, (uint8_t*)k_lds);
    });
}

// ------------------------------------------------------------------------------------------------
// Streamed launches: resident work-groups, each walking one stream of key blocks
// ------------------------------------------------------------------------------------------------
// The arrays of a stream are read through the constant address space: nothing writes them during a launch, and
// the loads then go through the scalar unit, so entries wait in scalar registers while the blocks before them are
// computed.
typedef const uint32_t __attribute__((address_space(4)))* const_words;

struct StreamBlock {
    uint32_t kv_off, info, col;
    uint32_t q_off;     // first block of an item: the item's first query row
};
// What the pipeline carries of an item: where its queries and its output are, and what becomes of the result.
struct StreamItem {
    uint32_t q_off;     // first query row
    uint32_t tag;       // 0: whole row, written to O; otherwise index + 1 of the partial record the chunk leaves
    uint32_t lse_off;   // index of the row's first query in the lse output
    uint32_t batch, head;
};
// Entry i of a run of n block entries; past the end: the last entry without its flags (its tiles are loaded once
// more and never used).
// (Every value here is the same for all lanes; readfirstlane says so where the compiler cannot see it, which keeps
// the entries and everything computed from them in scalar registers.)
__device__ __forceinline__ uint32_t uni(uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); }
__device__ __forceinline__ StreamBlock stream_block(const_words base, uint32_t i, uint32_t n) {
    i = uni(i);
    const const_words w = base + (size_t)(i < n ? i : n - 1) * (sizeof(sfb_stream_block) / 4);
    StreamBlock e = {uni(w[0]), i < n ? uni(w[1]) : 0u, uni(w[2]), uni(w[3])};
    return e;
}
template <bool MASKED = true>
__device__ __forceinline__ StreamItem stream_item(const_words base, uint32_t i, uint32_t n) {
    i = uni(i);
    const const_words w = base + (size_t)(i < n ? i : n - 1) * (sizeof(sfb_stream_item) / 4);
    // words: q_off, batch, head, row | kind, part, lse_off, lut_first | count, first, nchunks, chunk
    return StreamItem{uni(w[0]), w[4] != 0 ? uni(w[5]) + 1u : 0u, uni(w[6]), MASKED ? uni(w[1]) : 0u, MASKED ? uni(w[2]) : 0u};
}
__device__ __forceinline__ StreamBlock uni(const StreamBlock& e) { return StreamBlock{uni(e.kv_off), uni(e.info), uni(e.col), uni(e.q_off)}; }
__device__ __forceinline__ StreamItem uni(const StreamItem& it) {
    return StreamItem{uni(it.q_off), uni(it.tag), uni(it.lse_off), uni(it.batch), uni(it.head)};
}
// The whole record, as the work of a launch that does item after item.
__device__ __forceinline__ RowWork stream_row_work(const FusedParams& p, const_words base, uint32_t i) {
    const const_words w = base + (size_t)uni(i) * (sizeof(sfb_stream_item) / 4);
    RowWork r;
    r.valid = 1;
    r.b = w[1]; r.h = w[2]; r.bh = w[1] * p.heads + w[2];
    r.row = w[3]; r.first = w[9]; r.count = w[8];
    r.nchunks = w[10]; r.chunk = w[11]; r.slot = 0; r.part = w[5];
    r.lut_first = w[7];
    return r;
}

// End of a streamed item.  A whole row is normalised and stored straight from the accumulators; a chunk of a cut
// row leaves its partial record and returns the record's index + 1: its flag is to be set once these stores have
// completed (the caller does that after its next wait for memory).  Returns 0 otherwise.
template <int BS, int D, bool RAGGED = false>
__device__ __forceinline__ uint32_t stream_end_item(const FusedParams& p, const StreamItem& it, f32x16 (&o)[D / 32],
                                                    float m_used, float m_true, float l, float c, uint32_t t) {
    constexpr int NO = D / 32, PART = BS * D + 4 * BS;
    const uint32_t lane = t & 63, qn = lane & 31, half = lane >> 5, q_in_block = (t >> 6) * 32 + qn;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const float total = l + __shfl_xor(l, 32);
    if (it.tag == 0) {
        float* o_row = output_row(p, ((size_t)it.q_off + (size_t)q_in_block * p.heads) * hd);
        const float f = exp2_fast((m_true - m_used) * c);
        const float inv = 1.0f / (total + 1e-6f * f);
        if (p.lse != nullptr && half == 0)
            p.lse[(size_t)it.lse_off + q_in_block] = __builtin_fmaf(m_used, c, __builtin_log2f(total + 1e-6f * f));
        for_each_out_vec<NO>([&](int mt, int ig) {
            const f32x4 out = {o[mt][ig * 4 + 0] * inv, o[mt][ig * 4 + 1] * inv, o[mt][ig * 4 + 2] * inv,
                               o[mt][ig * 4 + 3] * inv};
            const uint32_t col = mt * 32 + ig * 8 + half * 4;
            if (RAGGED && col >= hd) return;
            if (p.o_bf16) {
                const u32x2 packed = {pack_bf16(out.x, out.y), pack_bf16(out.z, out.w)};
                *(u32x2*)((uint8_t*)o_row + col * 2) = packed;
            } else {
                *(f32x4*)(o_row + col) = out;
            }
        });
        return 0;
    }
    float* mine = p.partials + (size_t)(it.tag - 1) * PART;
    for_each_out_vec<NO>([&](int mt, int ig) {
        const f32x4 out = {o[mt][ig * 4 + 0], o[mt][ig * 4 + 1], o[mt][ig * 4 + 2], o[mt][ig * 4 + 3]};
        coherent_store4(mine + partial_offset<BS>(mt, ig, half, q_in_block), out);
    });
    if (half == 0) {
        const f32x4 sv = {m_used, m_true, total, 0.f};
        coherent_store4(mine + BS * D + q_in_block * 4, sv);
    }
    return it.tag;
}

__device__ __forceinline__ void stream_set_flag(const FusedParams& p, uint32_t part_plus_1) {
    __hip_atomic_store(p.st_flags + (part_plus_1 - 1), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Merge tasks of a work-group, done after its stream: wait (bounded) for the flags of the row's partial records, add
// the records, write the row, clear the flags for the next launch.  lds: at least BS * (D * 4 + 16) bytes that nobody
// uses any more.
template <int BS, int D, bool RAGGED = false>
__device__ __forceinline__ void stream_merges(const FusedParams& p, const_words merges, uint32_t n_merges, uint8_t* lds) {
    constexpr int PART = BS * D + 4 * BS;
    constexpr uint32_t kMaxPolls = 1u << 20;   // of about a microsecond each
    const uint32_t t = threadIdx.x, lane = t & 63, q_in_block = (t >> 6) * 32 + (lane & 31);
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const uint32_t o_row_bytes = p.heads * hd * (p.o_bf16 ? 2u : 4u);
    uint8_t* const slab = lds + (t >> 6) * (32u * (D * 4 + 16));
    for (uint32_t i = 0; i < n_merges; ++i) {
        const const_words w = merges + (size_t)i * (sizeof(sfb_stream_merge) / 4);
        const uint32_t q_off = w[0], batch = w[1], head = w[2], row = w[3], part = w[4], nparts = w[5];
        float* o_row = output_row(p, ((size_t)q_off + (size_t)q_in_block * p.heads) * hd);
        float* lse_row = p.lse ? p.lse + ((size_t)(batch * p.heads + head) * p.nb + row) * BS + q_in_block : nullptr;
        if (nparts == 0) {
            if constexpr (RAGGED) store_zero_row_ragged(o_row, p.o_bf16, lane >> 5, hd);
            else store_zero_row<D>(o_row, p.o_bf16, lane >> 5);
            if (lse_row && (lane >> 5) == 0) *lse_row = 0.f;
            continue;
        }
        int ready = 1;
        for (uint32_t f = t; f < nparts; f += BS * 2) {
            uint32_t polls = 0;
            while (__hip_atomic_load(p.st_flags + part + f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u) {
                if (++polls > kMaxPolls) { ready = 0; break; }
                __builtin_amdgcn_s_sleep(32);
            }
        }
        ready = __syncthreads_and(ready);
        if (!ready) {
            if (t == 0) __hip_atomic_store(p.st_status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            continue;
        }
        merge_partials<BS, D, RAGGED>(p.partials + (size_t)part * PART, nparts, o_row, o_row_bytes, p.o_bf16, lse_row,
                                      p.scale_log2e, q_in_block, lane, slab, hd);
        for (uint32_t f = t; f < nparts; f += BS * 2)
            __hip_atomic_store(p.st_flags + part + f, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();   // the slabs are used again by the next merge
    }
}

// bf16 tensors: the items of a stream are chained.  The loop over an item's key blocks is the one of attend_item_bf16
// (one barrier per block, K(j+2) and V(j+1) in flight while block j is worked on), but the blocks it fetches ahead are
// taken from the stream, so that the last two iterations of an item fetch the first tiles of the next one instead of
// nothing; the next item's queries and record are requested before the loop and arrive under it.  Between two items
// stand only the end of one (normalisation and stores straight from the accumulators) and the first score block of
// the other, whose tiles are already in LDS.  Block g of the stream uses tile buffers g % 2.
template <int BS, int D, bool MASKED>
__device__ __forceinline__ void stream_items_bf16(const FusedParams& p, uint8_t* smem, uint32_t* retry_flag,
                                                  const_words blocks, uint32_t n, const_words items, uint32_t n_items) {
    constexpr bool SLIM = !MASKED;
    using T = Bf16DirectTiles<BS, D>;
    constexpr int KT = BS / 32, NO = D / 32, KS = D / 16, PU = BS / 16;
    constexpr int TILE = T::TILE_BYTES;
    constexpr int KPC = KS / PU;   // score product steps per chunk
    static_assert(KS % PU == 0, "the score product is spread evenly over the chunks");

    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t qn = lane & 31, half = lane >> 5;
    const uint32_t q_in_block = wave * 32 + qn;
    const uint32_t row_bytes = p.heads * D * 2;
    const __bf16* const Q = (const __bf16*)p.q;
    const uint8_t* const k_base = (const uint8_t*)p.k;
    const uint8_t* const v_base = (const uint8_t*)p.v;
    const uint32_t src_even = T::lane_source(lane, 0, row_bytes), src_odd = T::lane_source(lane, 1, row_bytes);
    const uint32_t lds0 = T::lds_address(smem);
    const uint32_t k_lane = T::k_lane_base(qn, half), v_lane = T::v_lane_base(lane);
    const float c = p.scale_log2e, slack = p.slack, c2 = p.scale_pow2, rest = p.scale_rest;
    const sfb_stream_block* const entries = (const sfb_stream_block*)(uintptr_t)blocks;
    auto q_row_of = [&](uint32_t q_off) { return Q + ((size_t)q_off + (size_t)q_in_block * p.heads) * D; };
    auto loads_landed = [&]() {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    };

    // the stream's entries [win, win + 64), one per lane (clamped to the last one)
    uint32_t win = 0, w_kv = 0, w_info = 0, w_col = 0;
    auto refill = [&](uint32_t first) {
        win = first;
        const uint32_t idx = first + lane < n ? first + lane : n - 1;
        w_kv = entries[idx].kv_off;
        if constexpr (MASKED) {
            w_info = entries[idx].info;
            w_col = entries[idx].col;
        }
    };
    auto kv_of = [&](uint32_t g) -> size_t {
        const uint32_t gg = g < n ? g : n - 1;
        return (size_t)(uint32_t)__builtin_amdgcn_readlane(w_kv, gg - win) * (D * 2);
    };
    auto load_k = [&](uint32_t g) {   // K(g) into buffer g % 2
        T::load_tile(lds0 + (g & 1) * TILE, k_base + kv_of(g), wave, src_even, src_odd, row_bytes);
    };
    auto load_v = [&](uint32_t g) {
        T::load_tile(lds0 + (2 + (g & 1)) * TILE, v_base + kv_of(g), wave, src_even, src_odd, row_bytes);
    };

    if (SLIM && t == 0) *retry_flag = 0;
    uint32_t pending = 0;   // partial record (index + 1) whose flag waits for the record's stores to complete
    uint32_t pos = 0;       // stream position of the current item's first block
    uint32_t index = 0;     // the current item
    bool primed = false;    // the tiles of blocks pos and pos + 1 are in LDS or on their way

    bf16x8 qf[KS], qf_next[KS];
    f32x16 o_acc[NO];
#pragma unroll
    for (int nn = 0; nn < NO; ++nn)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[nn][i] = 0.f;
    refill(0);
    StreamItem rec = stream_item<MASKED>(items, 0, n_items);
    uint32_t count = uni(((const_words)items)[8]);
    T::load_q(qf_next, q_row_of(rec.q_off), half);

    for (;;) {
        if (!primed) {
            if (pos + 2 >= win + 64 || pos < win) refill(pos);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            load_k(pos);
            load_v(pos);
            load_k(pos + 1);
            primed = true;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[ks] = SLIM ? scale_bf16x8(qf_next[ks], c2) : qf_next[ks];
        // the record and the queries of the next item
        const bool more = index + 1 < n_items;
        const StreamItem rec_next = stream_item<MASKED>(items, index + 1, n_items);
        const uint32_t count_next = uni(((const_words)items)[(size_t)(more ? index + 1 : index) * (sizeof(sfb_stream_item) / 4) + 8]);
        asm volatile("" : : "s"(rec_next.q_off), "s"(rec_next.tag), "s"(rec_next.lse_off), "s"(count_next));   // arrived: nothing scalar is in flight under the loop
        const uint8_t* mask = nullptr;
        int valid = (int)L;
        if constexpr (MASKED) {
            mask = p.mask ? (const uint8_t*)p.mask + (size_t)rec.head * p.mask_stride * (BS / 8) : nullptr;
            valid = p.valid_len ? p.valid_len[rec.batch] : (int)L;
        }
        RowState st = {kMaxSeed, kMaxSeed, 0.f};

        f32x16 s_even[KT], s_odd[KT];
        loads_landed();
        if (more) T::load_q(qf_next, q_row_of(rec_next.q_off), half);
        {
            const uint8_t* const k0 = smem + (pos & 1) * TILE;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
                for (int i = 0; i < 16; ++i) s_even[kt][i] = 0.f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
                    s_even[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(T::k_frag(k0, k_lane, kt, ks), qf[ks], s_even[kt], 0, 0, 0);
            }
        }
        f32x16 off_vec;
        float m_item = 0.f;
        if constexpr (SLIM) {
            m_item = block_row_max<KT>(s_even);
#pragma unroll
            for (int i = 0; i < 16; ++i) off_vec[i] = -m_item;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) s_even[kt] += off_vec;
        }
        __syncthreads();   // every wave has read K(pos) before the first iteration overwrites its buffer

        auto iteration = [&](uint32_t j, f32x16 (&s)[KT], f32x16 (&s_next)[KT]) {
            const uint32_t g = pos + j, par = g & 1;
            const uint8_t* const k_read = smem + (par ^ 1) * TILE;       // K(g+1)
            const uint8_t* const v_read = smem + (2 + par) * TILE;       // V(g)
            if (g + 2 >= win + 64) refill(g);
            const uint8_t* const k_src = k_base + kv_of(g + 2);
            const uint8_t* const v_src = v_base + kv_of(g + 1);
            const uint32_t k_dst = lds0 + par * TILE, v_dst = lds0 + (2 + (par ^ 1)) * TILE;

            if constexpr (MASKED) {
                const uint32_t blk = (uint32_t)__builtin_amdgcn_readlane(w_info, g - win) & SFB_STREAM_BLOCK_INDEX;
                const uint32_t col = (uint32_t)__builtin_amdgcn_readlane(w_col, g - win);
                const int limit = valid - (int)(col * BS);
                if ((mask != nullptr) || (limit < BS)) {
                    const uint64_t keep = load_keep_word<BS>(mask, (size_t)blk * BS + q_in_block, limit);
                    constexpr uint64_t kAll = BS == 64 ? ~0ull : 0xffffffffull;
                    if (__builtin_amdgcn_ballot_w64((keep & kAll) != kAll) != 0) apply_keep<KT>(s, keep, half);
                }
                const float mloc = block_row_max<KT>(s);
                st.m_true = fmaxf(st.m_true, mloc);
                if (__builtin_amdgcn_ballot_w64(mloc > st.m_used + slack) != 0) {
                    const float m_new = fmaxf(st.m_used, mloc);
                    const float alpha = exp2_fast((st.m_used - m_new) * c);
                    st.m_used = m_new;
                    st.l *= alpha;
#pragma unroll
                    for (int nn = 0; nn < NO; ++nn) o_acc[nn] *= alpha;
                }
            }
            const float mc = st.m_used * c;
            float sum0 = 0.f, sum1 = 0.f;
            uint32_t pk[KT * 8];
            auto exps = [&](int u) {
                if constexpr (SLIM) exp_chunk_slim<KT>(s, pk, u, rest, sum0, sum1);
                else exp_chunk<KT, NO>(s, pk, u, c, mc, sum0, sum1);
            };
            bf16x8 kfr[PU][KPC][KT], vfr[PU][NO];
            auto fragments = [&](int u) {
#pragma unroll
                for (int kk = 0; kk < KPC; ++kk)
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) kfr[u][kk][kt] = T::k_frag(k_read, k_lane, kt, u * KPC + kk);
#pragma unroll
                for (int mt = 0; mt < NO; ++mt) vfr[u][mt] = T::v_frag(v_read, v_lane, mt, u);
            };
            fragments(0);
            exps(0);
#pragma unroll
            for (int i = 0; i < T::LOADS; ++i) {
                T::load_rows(k_dst, k_src, i, wave, src_even, src_odd, row_bytes);
                T::load_rows(v_dst, v_src, i, wave, src_even, src_odd, row_bytes);
            }
            if constexpr (SLIM) __builtin_amdgcn_sched_barrier(0);   // the tile loads are issued here, not later
#pragma unroll
            for (int u = 0; u < PU; ++u) {
                if (u + 1 < PU) {
                    fragments(u + 1);
                    exps(u + 1);
                }
#pragma unroll
                for (int kk = 0; kk < KPC; ++kk)
#pragma unroll
                    for (int kt = 0; kt < KT; ++kt) {
                        const int ks = u * KPC + kk;
                        if (ks == 0) {
                            const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                            s_next[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[u][kk][kt], qf[ks], SLIM ? off_vec : zero, 0, 0, 0);
                        } else {
                            s_next[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[u][kk][kt], qf[ks], s_next[kt], 0, 0, 0);
                        }
                    }
                const u32x4 pb = {pk[u * 4 + 0], pk[u * 4 + 1], pk[u * 4 + 2], pk[u * 4 + 3]};
                const bf16x8 bfrag = __builtin_bit_cast(bf16x8, pb);
#pragma unroll
                for (int mt = 0; mt < NO; ++mt)
                    o_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfr[u][mt], bfrag, o_acc[mt], 0, 0, 0);
            }
            if constexpr (SLIM) {
                schedule_chunks<BS, D>();
            }
            st.l += sum0 + sum1;
            if constexpr (SLIM) __builtin_amdgcn_sched_barrier(0);   // the wait for the tiles comes last
            loads_landed();
        };

        for (uint32_t j = 0; j < count; j += 2) {
            iteration(j, s_even, s_odd);
            if (j + 1 < count) iteration(j + 1, s_odd, s_even);
        }

        // the record left by the item before this one is complete by now (every iteration waited for memory)
        if (pending != 0) {
            if (t == 0) stream_set_flag(p, pending);
            pending = 0;
        }
        bool redo = false;
        if constexpr (SLIM) {
            const float total = st.l + __shfl_xor(st.l, 32);
            if (__builtin_amdgcn_ballot_w64(!(total < 0x1p100f)) != 0 && lane == 0) *retry_flag = 1;   // overflow, or NaN
            __syncthreads();
            redo = __builtin_amdgcn_readfirstlane(*retry_flag) != 0;
            st.m_used = st.m_true = m_item / c2;
        }
        if (!redo) {
            pending = uni(stream_end_item<BS, D>(p, rec, o_acc, st.m_used, st.m_true, st.l, c, t));
        } else {
            // The sum overflowed with the offset of the item's first block: the item is done again by the loop that
            // follows the running maximum, and the tiles of the next item are fetched anew behind it.
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (t == 0) *retry_flag = 0;
            const RowWork w = stream_row_work(p, items, index);
            uint32_t made = 0;
            attend_item_bf16<BS, D, MASKED, false>(p, w, smem, retry_flag, lut_window(p, w, 0, lane),
                                                   [&](f32x16 (&o)[NO], const RowState& rs) {
                                                       made = stream_end_item<BS, D>(p, rec, o, rs.m_used, rs.m_true, rs.l, c, t);
                                                   });
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (made != 0 && t == 0) stream_set_flag(p, made);
            primed = false;
        }
#pragma unroll
        for (int nn = 0; nn < NO; ++nn)
#pragma unroll
            for (int i = 0; i < 16; ++i) o_acc[nn][i] = 0.f;
        if (!more) break;
        pos = uni(pos + count);
        index = uni(index + 1);
        rec = uni(rec_next);
        count = count_next;
    }
    if (pending != 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (t == 0) stream_set_flag(p, pending);
    }
}

template <int BS, int D, bool MASKED>
__global__ __launch_bounds__(BS * 2, 2) void fused_attention_stream_bf16_kernel(FusedParams p) {
    using T = Bf16DirectTiles<BS, D>;
    constexpr int TILE = T::TILE_BYTES;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[4 * TILE];   // K0 K1 V0 V1
    __shared__ uint32_t retry_flag;
    static_assert(4 * TILE >= BS * (D * 4 + 16), "the tiles' memory doubles as the output slabs");
    const const_words slot = (const_words)(uintptr_t)p.st_slots + (size_t)blockIdx.x * (sizeof(sfb_stream_slot) / 4);
    const uint32_t block_begin = slot[0], n_blocks = slot[1], item_begin = slot[2], n_items = slot[3];
    const uint32_t merge_begin = slot[4], n_merges = slot[5];
    if (n_blocks != 0)
        stream_items_bf16<BS, D, MASKED>(p, smem, &retry_flag,
                                         (const_words)(uintptr_t)p.st_blocks + (size_t)block_begin * (sizeof(sfb_stream_block) / 4), n_blocks,
                                         (const_words)(uintptr_t)p.st_items + (size_t)item_begin * (sizeof(sfb_stream_item) / 4), n_items);
    if (n_merges != 0) {
        __syncthreads();   // the tiles' memory becomes the output slabs
        stream_merges<BS, D>(p, (const_words)(uintptr_t)p.st_merges + (size_t)merge_begin * (sizeof(sfb_stream_merge) / 4), n_merges, smem);
    }
}

// Other element types and head sizes: the work-group does the items of its stream one after the other.
// bf16 tensors with a head size other than 64: the stream's items one after the other (the chained form above is
// built around one score product step per chunk, which is what 64 features give).
template <int BS, int D, bool MASKED, bool RAGGED = false>
__global__ __launch_bounds__(BS * 2, D > 64 ? 1 : 2) void fused_attention_stream_items_bf16_kernel(FusedParams p) {
    using T = Bf16DirectTiles<BS, D>;
    constexpr int TILE = T::TILE_BYTES;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[4 * TILE];   // K0 K1 V0 V1
    __shared__ uint32_t retry_flag;
    static_assert(4 * TILE >= BS * (D * 4 + 16), "the tiles' memory doubles as the output slabs");
    const const_words slot = (const_words)(uintptr_t)p.st_slots + (size_t)blockIdx.x * (sizeof(sfb_stream_slot) / 4);
    const uint32_t item_begin = slot[2], n_items = slot[3], merge_begin = slot[4], n_merges = slot[5];
    const const_words items = (const_words)(uintptr_t)p.st_items + (size_t)item_begin * (sizeof(sfb_stream_item) / 4);
    const uint32_t t = threadIdx.x, lane = t & 63;
    for (uint32_t i = 0; i < n_items; ++i) {
        const StreamItem it = stream_item(items, i, n_items);
        const RowWork w = stream_row_work(p, items, i);
        const sfb_uint2 window = lut_window(p, w, 0, lane);
        uint32_t made = 0;
        auto finish = [&](f32x16 (&o)[D / 32], const RowState& rs) {
            made = stream_end_item<BS, D, RAGGED>(p, it, o, rs.m_used, rs.m_true, rs.l, p.scale_log2e, t);
        };
        bool done = false;
        if constexpr (!MASKED && !RAGGED) done = attend_item_bf16<BS, D, false, true>(p, w, smem, &retry_flag, window, finish);
        if (!done) attend_item_bf16<BS, D, MASKED, false, RAGGED>(p, w, smem, &retry_flag, window, finish);
        if (made != 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();   // the record is complete, and the tiles' memory is free for the next item
        if (made != 0 && t == 0) stream_set_flag(p, made);
    }
    if (n_merges != 0)
        stream_merges<BS, D, RAGGED>(p, (const_words)(uintptr_t)p.st_merges + (size_t)merge_begin * (sizeof(sfb_stream_merge) / 4),
                                     n_merges, smem);
}

template <int BS, int D, bool RAGGED = false>
__global__ __launch_bounds__(BS * 2, D > 64 ? 1 : 2) void fused_attention_stream_f32_kernel(FusedParams p) {
    using T = F32Tiles<BS, D>;
    __shared__ __attribute__((aligned(16))) float k_lds[T::K_FLOATS];
    __shared__ __attribute__((aligned(16))) float v_lds[T::V_FLOATS];
    static_assert(T::K_FLOATS * 4 >= BS * (D * 4 + 16), "the K tile's memory doubles as the output slabs");
    const const_words slot = (const_words)(uintptr_t)p.st_slots + (size_t)blockIdx.x * (sizeof(sfb_stream_slot) / 4);
    const uint32_t item_begin = slot[2], n_items = slot[3], merge_begin = slot[4], n_merges = slot[5];
    const const_words items = (const_words)(uintptr_t)p.st_items + (size_t)item_begin * (sizeof(sfb_stream_item) / 4);
    const uint32_t t = threadIdx.x;
    for (uint32_t i = 0; i < n_items; ++i) {
        const StreamItem it = stream_item(items, i, n_items);
        uint32_t made = 0;
        attend_item_f32<BS, D, RAGGED>(p, stream_row_work(p, items, i), k_lds, v_lds, [&](f32x16 (&o)[D / 32], const RowState& rs) {
            made = stream_end_item<BS, D, RAGGED>(p, it, o, rs.m_used, rs.m_true, rs.l, p.scale_log2e, t);
        });
        if (made != 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (made != 0 && t == 0) stream_set_flag(p, made);
    }
    if (n_merges != 0)
        stream_merges<BS, D, RAGGED>(p, (const_words)(uintptr_t)p.st_merges + (size_t)merge_begin * (sizeof(sfb_stream_merge) / 4),
                                     n_merges, (uint8_t*)k_lds);
}

// Fill kernel (a captured graph must not hold a memset node): words[0 .. n) = 0.
__global__ void clear_words_kernel(uint32_t* words, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) words[i] = 0u;
}

// Head sizes the fused forward takes: rows of whole 16-byte vectors, at most 128 features.
static bool head_size_supported(int in_dtype, uint32_t state_dim) {
    const uint32_t granule = in_dtype == SFB_BF16 ? 8u : 4u;
    return state_dim >= granule && state_dim <= 128 && state_dim % granule == 0;
}

template <int BS, int D>
static int launch_fused(hipStream_t stream, FusedParams& p, int in_dtype, uint32_t ranks) {
    p.ranks = ranks;
    const bool streamed = p.st_slots != nullptr;
    const uint32_t grid = streamed ? ranks : p.groups * 8u * ranks;   // streamed launches: ranks = resident work-groups
    clear_stale_error();
    // the loop that folds scale and offset into the score product rounds the scaled queries to bf16 once more: fine
    // for the output, but a log-sum-exp that a backward pass pairs with its own scores is made by the exact loop
    const bool masked = p.mask || p.valid_len || p.lse;
    const dim3 g(grid), b(BS * 2);
    if (in_dtype == SFB_BF16) {
        if constexpr (D == 64) {
            if (masked && streamed) fused_attention_stream_bf16_kernel<BS, D, true><<<g, b, 0, stream>>>(p);
            else if (masked) fused_attention_bf16_kernel<BS, D, true><<<g, b, 0, stream>>>(p);
            else if (streamed) fused_attention_stream_bf16_kernel<BS, D, false><<<g, b, 0, stream>>>(p);
            else fused_attention_bf16_kernel<BS, D, false><<<g, b, 0, stream>>>(p);
        } else {
            if (masked && streamed) fused_attention_stream_items_bf16_kernel<BS, D, true><<<g, b, 0, stream>>>(p);
            else if (masked) fused_attention_bf16_kernel<BS, D, true><<<g, b, 0, stream>>>(p);
            else if (streamed) fused_attention_stream_items_bf16_kernel<BS, D, false><<<g, b, 0, stream>>>(p);
            else fused_attention_bf16_kernel<BS, D, false><<<g, b, 0, stream>>>(p);
        }
    } else if (streamed)
        fused_attention_stream_f32_kernel<BS, D><<<g, b, 0, stream>>>(p);
    else
        fused_attention_f32_kernel<BS, D><<<g, b, 0, stream>>>(p);
    return launch_status();
}

// Work-groups per compute unit the device keeps resident of the kernel a streamed launch of this kind runs (the
// same choice as launch_fused makes); 0 if the runtime cannot say.
template <int BS, int D>
static int stream_kernel_occupancy(int in_dtype, bool masked, bool ragged = false) {
    const void* kernel;
    if (ragged) {
        kernel = in_dtype == SFB_BF16 ? (const void*)fused_attention_stream_items_bf16_kernel<BS, D, true, true>
                                      : (const void*)fused_attention_stream_f32_kernel<BS, D, true>;
    } else if (in_dtype == SFB_BF16) {
        if constexpr (D == 64) {
            kernel = masked ? (const void*)fused_attention_stream_bf16_kernel<BS, D, true>
                            : (const void*)fused_attention_stream_bf16_kernel<BS, D, false>;
        } else {
            kernel = masked ? (const void*)fused_attention_stream_items_bf16_kernel<BS, D, true>
                            : (const void*)fused_attention_stream_items_bf16_kernel<BS, D, false>;
        }
    } else {
        kernel = (const void*)fused_attention_stream_f32_kernel<BS, D>;
    }
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, BS * 2, 0) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return per_cu;
}
template <int BS>
static int stream_kernel_occupancy_any(int in_dtype, bool masked, uint32_t state_dim) {
    switch (state_dim) {
        case 64: return stream_kernel_occupancy<BS, 64>(in_dtype, masked);
        case 32: return stream_kernel_occupancy<BS, 32>(in_dtype, masked);
        case 96: return stream_kernel_occupancy<BS, 96>(in_dtype, masked);
        case 128: return stream_kernel_occupancy<BS, 128>(in_dtype, masked);
        default: break;
    }
    switch ((state_dim + 31) / 32) {   // head sizes between: the kernel of the next multiple of 32
        case 1: return stream_kernel_occupancy<BS, 32>(in_dtype, true, true);
        case 2: return stream_kernel_occupancy<BS, 64>(in_dtype, true, true);
        case 3: return stream_kernel_occupancy<BS, 96>(in_dtype, true, true);
        case 4: return stream_kernel_occupancy<BS, 128>(in_dtype, true, true);
        default: return 0;
    }
}

// Head sizes that are not a multiple of 32 (the reference's kernels take any multiple of 4,
// openai_blocksparse.h:221-222): the kernel of the next multiple of 32 with zero-padded queries, the general loop
// only.  Streamed launches walk their items one after the other (the masked form serves both kinds of launch).
template <int BS, int D>
static int launch_fused_ragged(hipStream_t stream, FusedParams& p, int in_dtype, uint32_t ranks) {
    p.ranks = ranks;
    clear_stale_error();
    if (p.st_slots != nullptr) {   // ranks = resident work-groups
        if (in_dtype == SFB_BF16) fused_attention_stream_items_bf16_kernel<BS, D, true, true><<<dim3(ranks), dim3(BS * 2), 0, stream>>>(p);
        else fused_attention_stream_f32_kernel<BS, D, true><<<dim3(ranks), dim3(BS * 2), 0, stream>>>(p);
        return launch_status();
    }
    const dim3 g(p.groups * 8u * ranks), b(BS * 2);
    if (in_dtype == SFB_BF16) fused_attention_bf16_kernel<BS, D, true, true><<<g, b, 0, stream>>>(p);
    else fused_attention_f32_kernel<BS, D, true><<<g, b, 0, stream>>>(p);
    return launch_status();
}

// head sizes 32, 64, 96 and 128 for both input types; other multiples of 8 (bf16) or 4 (fp32) up to 128 through
// the padded kernels
template <int BS>
static int launch_fused_any(hipStream_t stream, FusedParams& p, int in_dtype, uint32_t ranks, uint32_t state_dim) {
    if (p.in_stride == 0) p.in_stride = p.heads * state_dim;
    p.state = state_dim;
    switch (state_dim) {
        case 64: return launch_fused<BS, 64>(stream, p, in_dtype, ranks);
        case 32: return launch_fused<BS, 32>(stream, p, in_dtype, ranks);
        case 96: return launch_fused<BS, 96>(stream, p, in_dtype, ranks);
        case 128: return launch_fused<BS, 128>(stream, p, in_dtype, ranks);
        default: break;
    }
    if (!head_size_supported(in_dtype, state_dim)) return SFB_ERR_HEAD_STATE;
    switch ((state_dim + 31) / 32) {
        case 1: return launch_fused_ragged<BS, 32>(stream, p, in_dtype, ranks);
        case 2: return launch_fused_ragged<BS, 64>(stream, p, in_dtype, ranks);
        case 3: return launch_fused_ragged<BS, 96>(stream, p, in_dtype, ranks);
        default: return launch_fused_ragged<BS, 128>(stream, p, in_dtype, ranks);
    }
}

static int check_common(const void* q, const void* k, const void* v, const void* o, int in_dtype,
                        const sfb_uint2* nn_lut, uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                        uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim, uint32_t lut_heads,
                        uint32_t lut_dim, uint32_t mask_heads, float scale) {
    if (!q || !k || !v || !o || !nn_lut) return SFB_ERR_NULL_POINTER;
    if (in_dtype != SFB_F32 && in_dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (!head_size_supported(in_dtype, state_dim)) return SFB_ERR_HEAD_STATE;
    if (!(scale > 0.f) || !(scale < 3.0e38f)) return SFB_ERR_ARGUMENT;
    if (batch_dim == 0 || ctx_blks == 0 || head_dim == 0 || lut_heads == 0 || mask_heads == 0)
        return SFB_ERR_SHAPE;
    if (lut_heads > 1 && (lut_heads != head_dim || lut_dim != ctx_blks + blocks)) return SFB_ERR_SHAPE;
    if (mask_heads > 1 && mask_heads != head_dim) return SFB_ERR_SHAPE;
    if ((uint64_t)batch_dim * head_dim * ctx_blks > 0x7fffffffull / 64) return SFB_ERR_SHAPE;
    const uintptr_t align = (uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)o;
    if (align & 15u) return SFB_ERR_ALIGNMENT;
    return SFB_OK;
}

}  // namespace sfb

extern "C" void sfb_scale_parts(float scale, float* pow2, float* rest) {
    int e = 0;
    const float mant = frexpf(scale * sfb::kLog2e, &e);      // scale * log2(e) = mant * 2^e, mant in [0.5, 1)
    const bool up = mant >= 0.70710678f;                      // the nearest power of two in the logarithm
    *pow2 = ldexpf(1.0f, up ? e : e - 1);
    *rest = up ? mant : mant * 2.0f;
}

namespace sfb {

static void fill_common(FusedParams& p, const void* q, const void* k, const void* v, void* o, int out_dtype,
                        const sfb_uint2* nn_lut, const void* mask, const int32_t* valid_len,
                        uint32_t block_size, uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks,
                        uint32_t head_dim, uint32_t lut_heads, uint32_t lut_dim, uint32_t mask_heads,
                        float scale) {
    p.q = q; p.k = k; p.v = v; p.o = (float*)o; p.o_bf16 = out_dtype == SFB_BF16 ? 1u : 0u;
    p.lse = nullptr;
    p.nn_lut = nn_lut; p.mask = mask; p.valid_len = valid_len;
    p.row_order = nullptr; p.items = nullptr; p.counters = nullptr; p.partials = nullptr;
    p.st_slots = nullptr; p.st_blocks = nullptr; p.st_items = nullptr; p.st_merges = nullptr;
    p.st_flags = nullptr; p.st_status = nullptr;
    p.n_slots = 0; p.n_parts = 0; p.heavy = 0;
    p.batch = batch_dim; p.heads = head_dim; p.nb = ctx_blks; p.blocks = blocks;
    p.in_stride = 0;   // set by the launcher: heads * d unless the caller gives a token stride
    p.lut_stride = lut_heads > 1 ? lut_dim : 0;
    p.item_stride = 0;
    p.mask_stride = mask_heads > 1 ? blocks * block_size : 0;
    p.groups = bh_groups(batch_dim * head_dim);
    p.scale_log2e = scale * kLog2e;
    sfb_scale_parts(scale, &p.scale_pow2, &p.scale_rest);
    p.slack = kLazyRescaleLog2 / p.scale_log2e;
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
    const int rc = check_common(q, k, v, o, in_dtype, nn_lut, block_size, blocks, batch_dim, ctx_blks,
                                head_dim, state_dim, lut_heads, lut_dim, mask_heads, scale);
    if (rc != SFB_OK) return rc;
    FusedParams p;
    fill_common(p, q, k, v, o, SFB_F32, nn_lut, mask, valid_len, block_size, blocks, batch_dim, ctx_blks, head_dim,
                lut_heads, lut_dim, mask_heads, scale);
    p.row_order = row_order;
    hipStream_t s = (hipStream_t)stream;
    if (block_size == 64) return launch_fused_any<64>(s, p, in_dtype, ctx_blks, state_dim);
    return launch_fused_any<32>(s, p, in_dtype, ctx_blks, state_dim);
}

extern "C" size_t sfb_schedule_workspace_bytes(uint32_t n_slots, uint32_t n_parts, uint32_t batch_dim,
                                               uint32_t head_dim, uint32_t block_size,
                                               uint32_t state_dim) {
    const size_t bh = (size_t)batch_dim * head_dim;
    const size_t counters = (bh * n_slots * sizeof(uint32_t) + 255) / 256 * 256;
    const size_t padded = ((size_t)state_dim + 31) / 32 * 32;   // records have the layout of the kernel that writes them
    const size_t part = ((size_t)block_size * padded + 4 * (size_t)block_size) * sizeof(float);
    return counters + bh * n_parts * part;
}

static int fused_attention_scheduled(sfb_stream_t stream, const void* q, const void* k,
                                             const void* v, void* o, float* lse, int in_dtype, int out_dtype,
                                             const sfb_uint2* nn_lut, const void* mask,
                                             const int32_t* valid_len, const sfb_work_item* items,
                                             uint32_t n_items, uint32_t n_heavy, uint32_t n_slots,
                                             uint32_t n_parts, void* workspace, size_t workspace_bytes,
                                             uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                             uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                             uint32_t mask_heads, float scale, uint32_t token_stride = 0,
                                             uint32_t lut_heads = 1, uint32_t lut_dim = 0) {
    using namespace sfb;
    if (lut_heads <= 1) lut_dim = ctx_blks + blocks;
    const int rc = check_common(q, k, v, o, in_dtype, nn_lut, block_size, blocks, batch_dim, ctx_blks,
                                head_dim, state_dim, lut_heads, lut_dim, mask_heads, scale);
    if (rc != SFB_OK) return rc;
    if (out_dtype != SFB_F32 && out_dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (!items) return SFB_ERR_NULL_POINTER;
    // rows of 16-byte vectors: the stride keeps every row aligned
    if (token_stride != 0 && (token_stride < head_dim * state_dim || token_stride % (in_dtype == SFB_BF16 ? 8u : 4u) != 0))
        return SFB_ERR_SHAPE;
    if (n_items == 0 || n_heavy >= n_items) return SFB_ERR_SHAPE;
    if ((uint64_t)batch_dim * head_dim * n_items > 0x7fffffffull / 64) return SFB_ERR_SHAPE;
    const size_t need = sfb_schedule_workspace_bytes(n_slots, n_parts, batch_dim, head_dim, block_size, state_dim);
    if (n_parts > 0 && (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255u)))
        return SFB_ERR_WORKSPACE;
    FusedParams p;
    fill_common(p, q, k, v, o, out_dtype, nn_lut, mask, valid_len, block_size, blocks, batch_dim, ctx_blks, head_dim,
                lut_heads, lut_dim, mask_heads, scale);
    p.items = items;
    p.item_stride = lut_heads > 1 ? n_items : 0;
    p.lse = lse;
    p.in_stride = token_stride;
    p.n_slots = n_slots; p.n_parts = n_parts; p.heavy = n_heavy;
    const size_t bh = (size_t)batch_dim * head_dim;
    const size_t counters = (bh * n_slots * sizeof(uint32_t) + 255) / 256 * 256;
    p.counters = (uint32_t*)workspace;
    p.partials = (float*)((uint8_t*)workspace + counters);
    hipStream_t s = (hipStream_t)stream;
    if (block_size == 64) return launch_fused_any<64>(s, p, in_dtype, n_items, state_dim);
    return launch_fused_any<32>(s, p, in_dtype, n_items, state_dim);
}

extern "C" int sfb_fused_attention_scheduled(sfb_stream_t stream, const void* q, const void* k,
                                             const void* v, float* o, int in_dtype,
                                             const sfb_uint2* nn_lut, const void* mask,
                                             const int32_t* valid_len, const sfb_work_item* items,
                                             uint32_t n_items, uint32_t n_heavy, uint32_t n_slots,
                                             uint32_t n_parts, void* workspace, size_t workspace_bytes,
                                             uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                             uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                             uint32_t mask_heads, float scale) {
    return fused_attention_scheduled(stream, q, k, v, o, nullptr, in_dtype, SFB_F32, nn_lut, mask, valid_len, items, n_items,
                                     n_heavy, n_slots, n_parts, workspace, workspace_bytes, block_size, blocks,
                                     batch_dim, ctx_blks, head_dim, state_dim, mask_heads, scale);
}

extern "C" int sfb_fused_attention_scheduled_to(sfb_stream_t stream, const void* q, const void* k,
                                                const void* v, void* o, int in_dtype, int out_dtype,
                                                const sfb_uint2* nn_lut, const void* mask,
                                                const int32_t* valid_len, const sfb_work_item* items,
                                                uint32_t n_items, uint32_t n_heavy, uint32_t n_slots,
                                                uint32_t n_parts, void* workspace, size_t workspace_bytes,
                                                uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                                uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                                uint32_t mask_heads, float scale) {
    return fused_attention_scheduled(stream, q, k, v, o, nullptr, in_dtype, out_dtype, nn_lut, mask, valid_len, items, n_items,
                                     n_heavy, n_slots, n_parts, workspace, workspace_bytes, block_size, blocks,
                                     batch_dim, ctx_blks, head_dim, state_dim, mask_heads, scale);
}

extern "C" int sfb_fused_attention_scheduled_strided(sfb_stream_t stream, const void* q, const void* k,
                                                     const void* v, void* o, int in_dtype, int out_dtype,
                                                     const sfb_uint2* nn_lut, const void* mask,
                                                     const int32_t* valid_len, const sfb_work_item* items,
                                                     uint32_t n_items, uint32_t n_heavy, uint32_t n_slots,
                                                     uint32_t n_parts, void* workspace, size_t workspace_bytes,
                                                     uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                                     uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                                     uint32_t token_stride, uint32_t mask_heads, float scale) {
    if (token_stride == 0) return SFB_ERR_SHAPE;
    return fused_attention_scheduled(stream, q, k, v, o, nullptr, in_dtype, out_dtype, nn_lut, mask, valid_len, items,
                                     n_items, n_heavy, n_slots, n_parts, workspace, workspace_bytes, block_size, blocks,
                                     batch_dim, ctx_blks, head_dim, state_dim, mask_heads, scale, token_stride);
}

extern "C" int sfb_fused_attention_scheduled_lse(sfb_stream_t stream, const void* q, const void* k,
                                                 const void* v, void* o, float* lse, int in_dtype, int out_dtype,
                                                 const sfb_uint2* nn_lut, const void* mask,
                                                 const int32_t* valid_len, const sfb_work_item* items,
                                                 uint32_t n_items, uint32_t n_heavy, uint32_t n_slots,
                                                 uint32_t n_parts, void* workspace, size_t workspace_bytes,
                                                 uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                                 uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                                 uint32_t mask_heads, float scale) {
    if (!lse) return SFB_ERR_NULL_POINTER;
    return fused_attention_scheduled(stream, q, k, v, o, lse, in_dtype, out_dtype, nn_lut, mask, valid_len, items,
                                     n_items, n_heavy, n_slots, n_parts, workspace, workspace_bytes, block_size, blocks,
                                     batch_dim, ctx_blks, head_dim, state_dim, mask_heads, scale);
}

extern "C" int sfb_fused_attention_scheduled_heads(sfb_stream_t stream, const void* q, const void* k, const void* v,
                                                   void* o, float* lse, int in_dtype, int out_dtype,
                                                   const sfb_uint2* nn_lut, const void* mask, const int32_t* valid_len,
                                                   const sfb_work_item* items, uint32_t n_items, uint32_t n_heavy,
                                                   uint32_t n_slots, uint32_t n_parts, void* workspace,
                                                   size_t workspace_bytes, uint32_t block_size, uint32_t blocks,
                                                   uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                                                   uint32_t state_dim, uint32_t lut_heads, uint32_t lut_dim,
                                                   uint32_t mask_heads, float scale) {
    if (lut_heads == 0) return SFB_ERR_SHAPE;
    return fused_attention_scheduled(stream, q, k, v, o, lse, in_dtype, out_dtype, nn_lut, mask, valid_len, items,
                                     n_items, n_heavy, n_slots, n_parts, workspace, workspace_bytes, block_size, blocks,
                                     batch_dim, ctx_blks, head_dim, state_dim, mask_heads, scale, 0, lut_heads, lut_dim);
}

extern "C" size_t sfb_stream_workspace_bytes(const sfb_stream_plan* plan, uint32_t state_dim) {
    if (!plan) return 0;
    const size_t flags = ((size_t)plan->n_parts * sizeof(uint32_t) + 255) / 256 * 256;
    const size_t padded = (state_dim + 31u) / 32u * 32u;   // records hold rows of the kernels' D floats
    const size_t part = ((size_t)plan->block_size * padded + 4 * (size_t)plan->block_size) * sizeof(float);
    return flags + (size_t)plan->n_parts * part + 256;   // the last 256 bytes hold the status word (at their end)
}

extern "C" uint32_t sfb_resident_work_groups_for(int in_dtype, uint32_t block_size, uint32_t state_dim, int masked) {
    using namespace sfb;
    if ((in_dtype != SFB_F32 && in_dtype != SFB_BF16) || (block_size != 32 && block_size != 64)) return 0;
    int device = 0, cus = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) {
        (void)hipGetLastError();
        return 0;
    }
    const int per_cu = block_size == 64 ? stream_kernel_occupancy_any<64>(in_dtype, masked != 0, state_dim)
                                        : stream_kernel_occupancy_any<32>(in_dtype, masked != 0, state_dim);
    // (a runtime that cannot answer: what the kernels' registers and LDS allow by design)
    return (uint32_t)(per_cu > 0 ? per_cu : (state_dim > 64 || state_dim % 32 != 0 ? 2 : 4)) * (uint32_t)cus;
}

// bf16 tensors, blocks of 64, head size 64, no mask: the benched case
extern "C" uint32_t sfb_resident_work_groups(void) { return sfb_resident_work_groups_for(SFB_BF16, 64, 64, 0); }

extern "C" int sfb_stream_reset(sfb_stream_t stream, const sfb_stream_plan* plan, uint32_t state_dim, void* workspace) {
    using namespace sfb;
    if (!plan || !workspace) return SFB_ERR_NULL_POINTER;
    if ((uintptr_t)workspace & 255u) return SFB_ERR_WORKSPACE;
    const size_t need = sfb_stream_workspace_bytes(plan, state_dim);
    const size_t flag_words = ((size_t)plan->n_parts * sizeof(uint32_t) + 255) / 256 * 64;
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
    if (flag_words > 0)
        clear_words_kernel<<<dim3((unsigned)((flag_words + 255) / 256)), dim3(256), 0, s>>>((uint32_t*)workspace,
                                                                                          (uint32_t)flag_words);
    clear_words_kernel<<<dim3(1), dim3(64), 0, s>>>((uint32_t*)((uint8_t*)workspace + need - 256), 64u);
    return launch_status();
}

extern "C" int sfb_stream_status(const sfb_stream_plan* plan, uint32_t state_dim, const void* workspace) {
    if (!plan || !workspace) return -1;
    uint32_t word = 0;
    if (hipMemcpy(&word, (const uint8_t*)workspace + sfb_stream_workspace_bytes(plan, state_dim) - 4, 4, hipMemcpyDeviceToHost) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    return word != 0 ? 1 : 0;
}

extern "C" int sfb_fused_attention_streamed(sfb_stream_t stream, const void* q, const void* k, const void* v, void* o,
                                            float* lse, int in_dtype, int out_dtype, const sfb_uint2* nn_lut,
                                            const void* mask, const int32_t* valid_len, const sfb_stream_plan* plan,
                                            const void* blob, void* workspace, size_t workspace_bytes,
                                            uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                            uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                            uint32_t lut_heads, uint32_t lut_dim, uint32_t mask_heads, float scale) {
    using namespace sfb;
    const int rc = check_common(q, k, v, o, in_dtype, nn_lut, block_size, blocks, batch_dim, ctx_blks, head_dim,
                                state_dim, lut_heads, lut_dim, mask_heads, scale);
    if (rc != SFB_OK) return rc;
    if (out_dtype != SFB_F32 && out_dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (!plan || !blob) return SFB_ERR_NULL_POINTER;
    if (plan->wg_slots == 0 || plan->block_size != block_size || plan->batch_dim != batch_dim ||
        plan->head_dim != head_dim || plan->ctx_blks != ctx_blks)
        return SFB_ERR_SHAPE;
    if ((uintptr_t)blob & 15u) return SFB_ERR_ALIGNMENT;
    const size_t need = sfb_stream_workspace_bytes(plan, state_dim);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255u)) return SFB_ERR_WORKSPACE;
    FusedParams p;
    fill_common(p, q, k, v, o, out_dtype, nn_lut, mask, valid_len, block_size, blocks, batch_dim, ctx_blks, head_dim,
                lut_heads, lut_dim, mask_heads, scale);
    p.lse = lse;
    p.st_slots = (const uint8_t*)blob + plan->slots_offset;
    p.st_blocks = (const uint8_t*)blob + plan->blocks_offset;
    p.st_items = (const uint8_t*)blob + plan->items_offset;
    p.st_merges = (const uint8_t*)blob + plan->merges_offset;
    const size_t flags = ((size_t)plan->n_parts * sizeof(uint32_t) + 255) / 256 * 256;
    p.st_flags = (uint32_t*)workspace;
    p.partials = (float*)((uint8_t*)workspace + flags);
    p.st_status = (uint32_t*)((uint8_t*)workspace + need - 4);
    hipStream_t s = (hipStream_t)stream;
    if (block_size == 64) return launch_fused_any<64>(s, p, in_dtype, plan->wg_slots, state_dim);
    return launch_fused_any<32>(s, p, in_dtype, plan->wg_slots, state_dim);
}

// ------------------------------------------------------------------------------------------------
// Scheduled launch that allocates nothing: the arrival counters and partial records of split rows live in a
// static device array instead of a caller's workspace.
// ------------------------------------------------------------------------------------------------
namespace sfb {

constexpr size_t kStaticScratchBytes = SFB_STATIC_SCRATCH_BYTES;
// Every device the library runs on holds its own copy of this array until the process ends.  In host code the
// name is only a handle for hipGetSymbolAddress; kernels and fills get the device address kept in scratch_ptr.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void* scratch_ptr[kMaxDevices];   // device address of `scratch` on each device, looked up on first use
static std::mutex scratch_mutex;

// Device address of the current device's copy of `scratch`.
static int static_scratch(void** out) {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
        (void)hipGetLastError();
        return SFB_ERR_LAUNCH;
    }
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_ptr[device] == nullptr) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
            (void)hipGetLastError();
            return SFB_ERR_LAUNCH;
        }
        scratch_ptr[device] = ptr;
    }
    *out = scratch_ptr[device];
    return SFB_OK;
}

}  // namespace sfb

extern "C" size_t sfb_static_scratch_bytes(void) { return sfb::kStaticScratchBytes; }

extern "C" int sfb_fused_attention_scheduled_noalloc(sfb_stream_t stream, const void* q, const void* k, const void* v,
                                                     void* o, int in_dtype, int out_dtype, const sfb_uint2* nn_lut,
                                                     const void* mask, const int32_t* valid_len,
                                                     const sfb_work_item* items, uint32_t n_items, uint32_t n_heavy,
                                                     uint32_t n_slots, uint32_t n_parts, uint32_t block_size,
                                                     uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks,
                                                     uint32_t head_dim, uint32_t state_dim, uint32_t mask_heads,
                                                     float scale) {
    using namespace sfb;
    // the largest launch this entry point takes: its counters and partial records must fit the static array
    const size_t need = sfb_schedule_workspace_bytes(n_slots, n_parts, batch_dim, head_dim, block_size, state_dim);
    if (need > kStaticScratchBytes) return SFB_ERR_SCRATCH_LIMIT;
    void* ptr = nullptr;
    const int rc = static_scratch(&ptr);
    if (rc != SFB_OK) return rc;
    hipStream_t s = (hipStream_t)stream;
    // The array keeps what the previous call on this device left in it.  Partial records are written before they
    // are read; the arrival counters must start at zero, so they are cleared here (a launch that ran to its end
    // leaves them at zero, one that was cut short need not).
    const size_t counter_words = (size_t)batch_dim * head_dim * n_slots;
    if (n_parts > 0 && counter_words > 0) {
        clear_stale_error();
        clear_words_kernel<<<dim3((unsigned)((counter_words + 255) / 256)), dim3(256), 0, s>>>((uint32_t*)ptr,
                                                                                             (uint32_t)counter_words);
        if (launch_status() != SFB_OK) return SFB_ERR_LAUNCH;
    }
    return fused_attention_scheduled(stream, q, k, v, o, nullptr, in_dtype, out_dtype, nn_lut, mask, valid_len, items,
                                     n_items, n_heavy, n_slots, n_parts, ptr, kStaticScratchBytes, block_size, blocks,
                                     batch_dim, ctx_blks, head_dim, state_dim, mask_heads, scale);
}
