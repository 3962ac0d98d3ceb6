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
    const sfb_plan_entry* plan;     // planned launches: one list of work items per resident work-group
    uint32_t plan_stride;           // entries between the lists of consecutive work-groups
    uint32_t* counters;             // [batch*heads][n_slots] arrival counters of split rows
    float* partials;                // [batch*heads][n_parts][BS*D + 4*BS]
    uint32_t n_slots, n_parts;
    uint32_t o_bf16;                // output element type: 0 fp32, 1 bf16 (rounded once from the fp32 result)
    uint32_t batch, heads, nb, blocks;
    uint32_t lut_stride;            // entries between heads' LUTs (0 = shared)
    uint32_t mask_stride;           // words between heads' masks (0 = shared)
    uint32_t groups;                // ceil(batch*heads / 8)
    uint32_t ranks;                 // work items per (batch, head)
    uint32_t heavy;                 // leading items issued for all heads first
    float scale_log2e;
    float slack;                    // raw-score distance a block maximum may exceed the reference maximum
};

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
        const sfb_work_item it = p.items[id.rank];
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

// Work of one entry of a planned launch.
__device__ __forceinline__ RowWork plan_row_work(const FusedParams& p, const sfb_plan_entry& e) {
    RowWork w;
    w.valid = 1;
    w.b = e.batch;
    w.h = e.head;
    w.bh = e.batch * p.heads + e.head;
    w.row = e.row; w.first = e.first; w.count = e.count;
    w.nchunks = e.nchunks; w.slot = e.slot; w.part = e.part; w.chunk = e.chunk;
    w.lut_first = e.lut_first;
    return w;
}
constexpr uint32_t kPlanEnd = 0xffffffffu;
// Plan entries are read through the constant address space: nothing writes them during a launch, and the
// loads then go through the scalar unit, so an entry waits in scalar registers while an item is computed.
typedef const uint32_t __attribute__((address_space(4)))* plan_words;
struct PlanList {
    plan_words words;
    __device__ __forceinline__ sfb_plan_entry operator[](uint32_t i) const {
        const plan_words w = words + (size_t)i * (sizeof(sfb_plan_entry) / 4);
        sfb_plan_entry e;
        e.batch = w[0]; e.head = w[1]; e.row = w[2]; e.first = w[3]; e.count = w[4]; e.nchunks = w[5];
        e.chunk = w[6]; e.slot = w[7]; e.part = w[8]; e.lut_first = w[9];
        e.reserved[0] = 0; e.reserved[1] = 0;
        return e;
    }
};
__device__ __forceinline__ PlanList plan_list_of(const FusedParams& p) {
    return PlanList{(plan_words)(uintptr_t)(p.plan + (size_t)blockIdx.x * p.plan_stride)};
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
template <int NO>
__device__ __forceinline__ void store_output(float* o_row, uint32_t o_row_bytes, uint32_t as_bf16, float* lse_row,
                                             f32x16 (&o)[NO], float m_used, float m_true, float total, float c,
                                             uint32_t lane, uint8_t* slab) {
    constexpr int D = NO * 32;
    const uint32_t qn = lane & 31, half = lane >> 5;
    const float f = exp2_fast((m_true - m_used) * c);
    const float inv = 1.0f / (total + 1e-6f * f);
    if (lse_row != nullptr && half == 0) *lse_row = __builtin_fmaf(m_used, c, __builtin_log2f(total + 1e-6f * f));
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

template <int BS, int D>
__device__ __forceinline__ void merge_partials(const float* base, uint32_t nchunks, float* o_row, uint32_t o_row_bytes,
                                               uint32_t as_bf16, float* lse_row, float c, uint32_t q_in_block,
                                               uint32_t lane, uint8_t* slab);

// End of a work item.  Unsplit rows are normalised and stored.  A chunk of a split row writes its
// partial (unnormalised O, reference maximum, true maximum, sum) and bumps the row's counter; the
// chunk that finds every other chunk already arrived merges all partials, stores O and resets the
// counter for the next launch.  Nobody waits.  lds: shared memory of the work-group that nobody uses any more, at
// least 32 * (row size + 16) bytes per wave (the output rows pass through it).
template <int BS, int D>
__device__ __forceinline__ void finish_row(const FusedParams& p, const RowWork& w, float* o_row,
                                           f32x16 (&o)[D / 32], const RowState& st, float c,
                                           uint32_t q_in_block, uint32_t half, uint32_t t, uint8_t* lds) {
    const uint32_t lane = t & 63, o_row_bytes = p.heads * D * (p.o_bf16 ? 2u : 4u);
    uint8_t* const slab = lds + (t >> 6) * (32u * (D * 4 + 16));
    float* const lse_row = p.lse ? p.lse + ((size_t)w.bh * p.nb + w.row) * BS + q_in_block : nullptr;
    constexpr int NO = D / 32;
    constexpr int PART = BS * D + 4 * BS;   // floats per partial
    const float total = st.l + __shfl_xor(st.l, 32);
    if (w.nchunks <= 1) {
        store_output<NO>(o_row, o_row_bytes, p.o_bf16, lse_row, o, st.m_used, st.m_true, total, c, lane, slab);
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
    merge_partials<BS, D>(base, w.nchunks, o_row, o_row_bytes, p.o_bf16, lse_row, c, q_in_block, lane, slab);
    if (t == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Merge of the partial records of a split row (run by the chunk that arrived last).
template <int BS, int D>
__device__ __forceinline__ void merge_partials(const float* base, uint32_t nchunks, float* o_row, uint32_t o_row_bytes,
                                               uint32_t as_bf16, float* lse_row, float c, uint32_t q_in_block,
                                               uint32_t lane, uint8_t* slab) {
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
    store_output<NO>(o_row, o_row_bytes, as_bf16, lse_row, acc, m_used, m_true, sum, c, lane, slab);
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

// The same for scores that already are base-2 exponents (scale and offset folded into the score product): one
// exponential per element and nothing else; the row sum is taken over the fp32 values with plain additions, which --
// unlike v_dot2c -- run while the matrix pipe is busy.
template <int KT>
__device__ __forceinline__ void exp_chunk_slim(const f32x16 (&s)[KT], uint32_t (&pk)[KT * 8], int u, float& sum0,
                                               float& sum1) {
    const int kt = u / 2, i0 = (u % 2) * 8;
    const float p0 = exp2_fast(s[kt][i0 + 0]), p1 = exp2_fast(s[kt][i0 + 1]);
    const float p2 = exp2_fast(s[kt][i0 + 2]), p3 = exp2_fast(s[kt][i0 + 3]);
    const float p4 = exp2_fast(s[kt][i0 + 4]), p5 = exp2_fast(s[kt][i0 + 5]);
    const float p6 = exp2_fast(s[kt][i0 + 6]), p7 = exp2_fast(s[kt][i0 + 7]);
    pk[u * 4 + 0] = pack_bf16(p0, p1); pk[u * 4 + 1] = pack_bf16(p2, p3);
    pk[u * 4 + 2] = pack_bf16(p4, p5); pk[u * 4 + 3] = pack_bf16(p6, p7);
    sum0 += (p0 + p2) + (p4 + p6);
    sum1 += (p1 + p3) + (p5 + p7);
}

// q * c, rounded to bf16 again (round to nearest even).
__device__ __forceinline__ bf16x8 scale_bf16x8(bf16x8 q, float c) {
    const u32x4 bits = __builtin_bit_cast(u32x4, q);
    u32x4 out;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        out[i] = pack_bf16(bf16_bits_to_f32(bits[i] & 0xffffu) * c, __builtin_bit_cast(float, bits[i] & 0xffff0000u) * c);
    return __builtin_bit_cast(bf16x8, out);
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
template <int BS, int D, bool MASKED, bool SLIM>
__device__ __forceinline__ bool attend_item_bf16(const FusedParams& p, const RowWork& w, uint8_t* smem, uint32_t* retry_flag,
                                                 sfb_uint2 first_window) {
    using T = Bf16DirectTiles<BS, D>;
    constexpr int KT = BS / 32, NO = D / 32, KS = D / 16, PU = BS / 16;
    constexpr int TILE = T::TILE_BYTES;
    constexpr int SC = PU >= 2 ? PU / 2 : 1;   // chunks that carry a slice of the next block's scores
    static_assert(!(MASKED && SLIM), "masked launches take the general loop");

    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t qn = lane & 31, half = lane >> 5;
    const uint32_t q_in_block = wave * 32 + qn;
    const uint32_t row_bytes = p.heads * D * 2;

    const uint32_t count = __builtin_amdgcn_readfirstlane(w.count);
    float* o_row = output_row(p, token_offset(w.b, w.row * BS + q_in_block, w.h, L, p.heads, D));

    const __bf16* Q = (const __bf16*)p.q;
    const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)w.h * p.mask_stride * (BS / 8) : nullptr;
    const int valid = p.valid_len ? p.valid_len[w.b] : (int)L;

    // byte address of (b, token 0, h, 0) in K and V; key block column col starts col*BS rows further
    const size_t bh_bytes = token_offset(w.b, 0, w.h, L, p.heads, D) * 2;
    const uint8_t* const k_base = (const uint8_t*)p.k + bh_bytes;
    const uint8_t* const v_base = (const uint8_t*)p.v + bh_bytes;
    const uint32_t src_even = T::lane_source(lane, 0, row_bytes), src_odd = T::lane_source(lane, 1, row_bytes);
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
    auto load_k = [&](uint32_t j, uint32_t buf) {
        T::load_tile(lds0 + buf * TILE, k_base + (size_t)column_of(j) * BS * row_bytes, wave, src_even, src_odd, row_bytes);
    };
    auto load_v = [&](uint32_t j, uint32_t buf) {
        T::load_tile(lds0 + (2 + buf) * TILE, v_base + (size_t)column_of(j) * BS * row_bytes, wave, src_even, src_odd, row_bytes);
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
    T::load_q(qf, Q + token_offset(w.b, w.row * BS + q_in_block, w.h, L, p.heads, D), half);
    if constexpr (SLIM) {
        // the score product then delivers base-2 exponents; the second rounding of Q moves them by less than the
        // rounding of the probabilities does
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[ks] = scale_bf16x8(qf[ks], c);
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
        st.m_used = st.m_true = m_scaled / c;
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
            if constexpr (SLIM) exp_chunk_slim<KT>(s, pk, u, sum0, sum1);
            else exp_chunk<KT, NO>(s, pk, u, c, mc, sum0, sum1);
        };
        // Every chunk carries the same work: the exponentials of the next chunk, one slice (KS / PU product steps) of
        // the next block's scores and one step of the output product.  The fragments of a chunk are requested from
        // LDS one chunk ahead of the matrix instructions that consume them.
        constexpr int KPC = KS / PU;   // score product steps per chunk
        static_assert(KS % PU == 0, "the score product is spread evenly over the chunks");
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
            // the order the instructions are to be issued in: the LDS reads of chunk u + 1 before the matrix
            // instructions of chunk u, and between two matrix instructions an equal share of the vector work
            constexpr int MF = KPC * KT + NO;                    // matrix instructions per chunk
            constexpr int DS = KPC * KT + 2 * NO;                // LDS reads per chunk
            constexpr int VA = (BS / 2 + BS / 4 + BS / 2) / PU;  // exp + pack + add per chunk (BS/2 elements per lane)
#pragma unroll
            for (int u = 0; u < PU; ++u) {
                if (u + 1 < PU) __builtin_amdgcn_sched_group_barrier(0x100, DS, 0);
#pragma unroll
                for (int m = 0; m < MF; ++m) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (u + 1 < PU) {
                        __builtin_amdgcn_sched_group_barrier(0x400, BS / 2 / PU / MF, 0);        // exponentials
                        __builtin_amdgcn_sched_group_barrier(0x002, (BS / 4 + BS / 2) / PU / MF, 0);   // pack, add
                    }
                }
            }
        }
        st.l += sum0 + sum1;
        if constexpr (SLIM) __builtin_amdgcn_sched_barrier(0);   // the wait for the tiles comes last
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
    finish_row<BS, D>(p, w, o_row, o_acc, st, c, q_in_block, half, t, smem);
    return true;
}

template <int BS, int D, bool MASKED, bool PLANNED>
__global__ __launch_bounds__(BS * 2, 2) void fused_attention_bf16_kernel(FusedParams p) {
    using T = Bf16DirectTiles<BS, D>;
    constexpr int TILE = T::TILE_BYTES;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[4 * TILE];   // K0 K1 V0 V1
    __shared__ uint32_t retry_flag;
    static_assert(4 * TILE >= BS * (D * 4 + 16), "the tiles' memory doubles as the output slabs");

    const uint32_t lane = threadIdx.x & 63;
    auto run = [&](const RowWork& w, sfb_uint2 window) {
        if (w.count == 0) {
            const uint32_t L = p.nb * BS, q_in_block = (threadIdx.x >> 6) * 32 + (lane & 31);
            float* o_row = output_row(p, token_offset(w.b, w.row * BS + q_in_block, w.h, L, p.heads, D));
            store_zero_row<D>(o_row, p.o_bf16, lane >> 5);
            if (p.lse && (lane >> 5) == 0) p.lse[((size_t)w.bh * p.nb + w.row) * BS + q_in_block] = 0.f;
            return;
        }
        if constexpr (!MASKED) {
            if (attend_item_bf16<BS, D, false, true>(p, w, smem, &retry_flag, window)) return;
        }
        attend_item_bf16<BS, D, MASKED, false>(p, w, smem, &retry_flag, window);
    };
    if constexpr (!PLANNED) {
        const RowWork w = decode_row_work(p);
        if (!w.valid) return;
        run(w, lut_window(p, w, 0, lane));
        return;
    }
    // Planned launch: this work-group stays resident and walks its own list of work items.  The list entry two
    // items ahead and the first LUT window of the next item are requested before the current item starts and
    // arrive while it is computed, so an item's first tile loads wait for nothing but themselves.  (Every list
    // ends with two end marks.)
    const PlanList mine = plan_list_of(p);
    sfb_plan_entry e = mine[0];
    if (e.count == kPlanEnd) return;
    sfb_plan_entry e_next = mine[1];
    RowWork w = plan_row_work(p, e);
    sfb_uint2 window = lut_window(p, w, 0, lane);
    for (uint32_t i = 2;; ++i) {
        const bool more = e_next.count != kPlanEnd;
        const RowWork w_next = plan_row_work(p, e_next);     // an end mark decodes to an item without key blocks
        const sfb_uint2 window_next = more ? lut_window(p, w_next, 0, lane) : window;
        e_next = mine[i];
        run(w, window);
        if (!more) break;
        // the output rows left through the tiles' memory, which the next item's loads overwrite: every wave must
        // have read its slab (LDS reads complete) before any wave goes on; the stores to memory may still be in flight
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        w = w_next;
        window = window_next;
    }
}

// ------------------------------------------------------------------------------------------------
// fp32 inputs: v_mfma_f32_32x32x2_f32 (true fp32 products and accumulation)
// ------------------------------------------------------------------------------------------------
// One LDS buffer (K tile and V tile); the next block waits in registers.
template <int BS, int D>
__device__ __forceinline__ void attend_item_f32(const FusedParams& p, const RowWork& w, float* k_lds, float* v_lds) {
    using T = F32Tiles<BS, D>;
    constexpr int KT = BS / 32;
    constexpr int NO = D / 32;
    constexpr int QG = D / 8;        // float4 groups of Q per lane
    const uint32_t L = p.nb * BS;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const uint32_t qn = lane & 31, half = lane >> 5;
    const uint32_t q_in_block = wave * 32 + qn;
    const uint32_t row_stride = p.heads * D;

    const sfb_uint2* lut = p.nn_lut + (size_t)w.h * p.lut_stride;
    const uint32_t lut_off = w.lut_first, count = w.count;
    float* o_row = output_row(p, token_offset(w.b, w.row * BS + q_in_block, w.h, L, p.heads, D));

    if (count == 0) {
        store_zero_row<D>(o_row, p.o_bf16, half);
        if (p.lse && half == 0) p.lse[((size_t)w.bh * p.nb + w.row) * BS + q_in_block] = 0.f;
        return;
    }

    const float* Q = (const float*)p.q;
    const float* K = (const float*)p.k;
    const float* V = (const float*)p.v;
    const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)w.h * p.mask_stride * (BS / 8) : nullptr;
    const int valid = p.valid_len ? p.valid_len[w.b] : (int)L;

    f32x4 qf[QG];
    T::load_q(qf, Q + token_offset(w.b, w.row * BS + q_in_block, w.h, L, p.heads, D), half);

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
        const size_t base = token_offset(w.b, entry.y * BS, w.h, L, p.heads, D);
        T::fetch(gk, K, base, row_stride, t);
        T::fetch(gv, V, base, row_stride, t);
    }

    for (uint32_t j = 0; j < count; ++j) {
        const sfb_uint2 here = entry;
        T::template stage<T::K_STRIDE>(k_lds, gk, t);
        T::template stage<T::V_STRIDE>(v_lds, gv, t);
        __syncthreads();
        if (j + 1 < count) {
            entry = lut[lut_off + j + 1];
            const size_t base = token_offset(w.b, entry.y * BS, w.h, L, p.heads, D);
            T::fetch(gk, K, base, row_stride, t);
            T::fetch(gv, V, base, row_stride, t);
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

    finish_row<BS, D>(p, w, o_row, o_acc, st, c, q_in_block, half, t, (uint8_t*)k_lds);
}

template <int BS, int D, bool PLANNED>
__global__ __launch_bounds__(BS * 2, D > 64 ? 1 : 2) void fused_attention_f32_kernel(FusedParams p) {
    using T = F32Tiles<BS, D>;
    __shared__ __attribute__((aligned(16))) float k_lds[T::K_FLOATS];
    __shared__ __attribute__((aligned(16))) float v_lds[T::V_FLOATS];
    static_assert(T::K_FLOATS * 4 >= BS * (D * 4 + 16), "the K tile's memory doubles as the output slabs");
    if constexpr (!PLANNED) {
        const RowWork w = decode_row_work(p);
        if (w.valid) attend_item_f32<BS, D>(p, w, k_lds, v_lds);
        return;
    }
    // planned launch: a resident work-group walks its list of work items
    const PlanList mine = plan_list_of(p);
    sfb_plan_entry e = mine[0];
    for (uint32_t i = 1; e.count != kPlanEnd; ++i) {
        const sfb_plan_entry e_next = mine[i];
        attend_item_f32<BS, D>(p, plan_row_work(p, e), k_lds, v_lds);
        __syncthreads();   // the output rows left through the K tile's memory
        e = e_next;
    }
}

template <int BS, int D>
static int launch_fused(hipStream_t stream, FusedParams& p, int in_dtype, uint32_t ranks) {
    p.ranks = ranks;
    const uint32_t grid = p.plan ? ranks : p.groups * 8u * ranks;   // planned launches: ranks = resident work-groups
    clear_stale_error();
    const bool masked = p.mask || p.valid_len, planned = p.plan != nullptr;
    const dim3 g(grid), b(BS * 2);
    if (in_dtype == SFB_BF16) {
        if constexpr (D == 64) {
            if (masked && planned) fused_attention_bf16_kernel<BS, D, true, true><<<g, b, 0, stream>>>(p);
            else if (masked) fused_attention_bf16_kernel<BS, D, true, false><<<g, b, 0, stream>>>(p);
            else if (planned) fused_attention_bf16_kernel<BS, D, false, true><<<g, b, 0, stream>>>(p);
            else fused_attention_bf16_kernel<BS, D, false, false><<<g, b, 0, stream>>>(p);
        } else {
            return SFB_ERR_HEAD_STATE;   // the bf16 kernel is built for head size 64 only
        }
    } else if (planned)
        fused_attention_f32_kernel<BS, D, true><<<g, b, 0, stream>>>(p);
    else
        fused_attention_f32_kernel<BS, D, false><<<g, b, 0, stream>>>(p);
    return launch_status();
}

// head sizes: 64 for both input types; 32, 96 and 128 for fp32 inputs
template <int BS>
static int launch_fused_any(hipStream_t stream, FusedParams& p, int in_dtype, uint32_t ranks, uint32_t state_dim) {
    switch (state_dim) {
        case 64: return launch_fused<BS, 64>(stream, p, in_dtype, ranks);
        case 32: return launch_fused<BS, 32>(stream, p, in_dtype, ranks);
        case 96: return launch_fused<BS, 96>(stream, p, in_dtype, ranks);
        case 128: return launch_fused<BS, 128>(stream, p, in_dtype, ranks);
        default: return SFB_ERR_HEAD_STATE;
    }
}

static int check_common(const void* q, const void* k, const void* v, const void* o, int in_dtype,
                        const sfb_uint2* nn_lut, uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                        uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim, uint32_t lut_heads,
                        uint32_t lut_dim, uint32_t mask_heads, float scale) {
    if (!q || !k || !v || !o || !nn_lut) return SFB_ERR_NULL_POINTER;
    if (in_dtype != SFB_F32 && in_dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (state_dim != 64 && (in_dtype != SFB_F32 || (state_dim != 32 && state_dim != 96 && state_dim != 128)))
        return SFB_ERR_HEAD_STATE;
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

static void fill_common(FusedParams& p, const void* q, const void* k, const void* v, void* o, int out_dtype,
                        const sfb_uint2* nn_lut, const void* mask, const int32_t* valid_len,
                        uint32_t block_size, uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks,
                        uint32_t head_dim, uint32_t lut_heads, uint32_t lut_dim, uint32_t mask_heads,
                        float scale) {
    p.q = q; p.k = k; p.v = v; p.o = (float*)o; p.o_bf16 = out_dtype == SFB_BF16 ? 1u : 0u;
    p.lse = nullptr;
    p.nn_lut = nn_lut; p.mask = mask; p.valid_len = valid_len;
    p.row_order = nullptr; p.items = nullptr; p.counters = nullptr; p.partials = nullptr;
    p.plan = nullptr; p.plan_stride = 0;
    p.n_slots = 0; p.n_parts = 0; p.heavy = 0;
    p.batch = batch_dim; p.heads = head_dim; p.nb = ctx_blks; p.blocks = blocks;
    p.lut_stride = lut_heads > 1 ? lut_dim : 0;
    p.mask_stride = mask_heads > 1 ? blocks * block_size : 0;
    p.groups = bh_groups(batch_dim * head_dim);
    p.scale_log2e = scale * kLog2e;
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
    const size_t part = ((size_t)block_size * state_dim + 4 * (size_t)block_size) * sizeof(float);
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
                                             uint32_t mask_heads, float scale) {
    using namespace sfb;
    const int rc = check_common(q, k, v, o, in_dtype, nn_lut, block_size, blocks, batch_dim, ctx_blks,
                                head_dim, state_dim, 1, ctx_blks + blocks, mask_heads, scale);
    if (rc != SFB_OK) return rc;
    if (out_dtype != SFB_F32 && out_dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (!items) return SFB_ERR_NULL_POINTER;
    if (n_items == 0 || n_heavy >= n_items) return SFB_ERR_SHAPE;
    if ((uint64_t)batch_dim * head_dim * n_items > 0x7fffffffull / 64) return SFB_ERR_SHAPE;
    const size_t need = sfb_schedule_workspace_bytes(n_slots, n_parts, batch_dim, head_dim, block_size, state_dim);
    if (n_parts > 0 && (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255u)))
        return SFB_ERR_WORKSPACE;
    FusedParams p;
    fill_common(p, q, k, v, o, out_dtype, nn_lut, mask, valid_len, block_size, blocks, batch_dim, ctx_blks, head_dim,
                1, ctx_blks + blocks, mask_heads, scale);
    p.items = items;
    p.lse = lse;
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

extern "C" int sfb_fused_attention_planned(sfb_stream_t stream, const void* q, const void* k, const void* v, void* o,
                                           float* lse, int in_dtype, int out_dtype, const sfb_uint2* nn_lut,
                                           const void* mask, const int32_t* valid_len, const sfb_plan_entry* plan,
                                           uint32_t wg_slots, uint32_t plan_stride, uint32_t n_slots,
                                           uint32_t n_parts, void* workspace, size_t workspace_bytes,
                                           uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                           uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                           uint32_t lut_heads, uint32_t lut_dim, uint32_t mask_heads, float scale) {
    using namespace sfb;
    const int rc = check_common(q, k, v, o, in_dtype, nn_lut, block_size, blocks, batch_dim, ctx_blks, head_dim,
                                state_dim, lut_heads, lut_dim, mask_heads, scale);
    if (rc != SFB_OK) return rc;
    if (out_dtype != SFB_F32 && out_dtype != SFB_BF16) return SFB_ERR_DTYPE;
    if (!plan) return SFB_ERR_NULL_POINTER;
    if (wg_slots == 0 || plan_stride < 3) return SFB_ERR_SHAPE;
    if ((uintptr_t)plan & 15u) return SFB_ERR_ALIGNMENT;
    const size_t need = sfb_schedule_workspace_bytes(n_slots, n_parts, batch_dim, head_dim, block_size, state_dim);
    if (n_parts > 0 && (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255u)))
        return SFB_ERR_WORKSPACE;
    FusedParams p;
    fill_common(p, q, k, v, o, out_dtype, nn_lut, mask, valid_len, block_size, blocks, batch_dim, ctx_blks, head_dim,
                lut_heads, lut_dim, mask_heads, scale);
    p.plan = plan;
    p.plan_stride = plan_stride;
    p.lse = lse;
    p.n_slots = n_slots; p.n_parts = n_parts;
    const size_t bh = (size_t)batch_dim * head_dim;
    const size_t counters = (bh * n_slots * sizeof(uint32_t) + 255) / 256 * 256;
    p.counters = (uint32_t*)workspace;
    p.partials = (float*)((uint8_t*)workspace + counters);
    hipStream_t s = (hipStream_t)stream;
    if (block_size == 64) return launch_fused_any<64>(s, p, in_dtype, wg_slots, state_dim);
    return launch_fused_any<32>(s, p, in_dtype, wg_slots, state_dim);
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

// Fill kernel (a captured graph must not hold a memset node): words[0 .. n) = 0.
__global__ void clear_words_kernel(uint32_t* words, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) words[i] = 0u;
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
