// The unfused block-sparse attention trio, kept as the comparison path for the fused kernel:
//   sdd  : S_blk = Q_rowblk . K_colblk^T for every block of the NT look-up table   (sfb_sdd_nt)
//   softmax over the sparse row (scaled, masked)                                    (sfb_masked_softmax)
//   dsd  : O_rowblk = sum_blk P_blk . V_colblk                                      (sfb_dsd_xn)
// S and P live in memory as [batch][heads][blocks][bs][bs] (openai_blocksparse.h:148), fp32 or bf16.
// Also here: the two-stage fusion  sdd + softmax -> P  of the reference's fusion_attention1/2
// (sfb_fused_sdd_softmax), done by one work-group per block-row without any inter-group exchange.
//
// Arithmetic follows the CPU path of the reference (matmul.h:53-78, ewops.h:64-98, matmul.h:6-20).
#include <type_traits>

#include "tiles.hip.h"

namespace sfb {

// relaxed device-scope load: reads what another work-group of the same launch published
__device__ __forceinline__ float coherent_load_f32(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static __device__ __forceinline__ float load(const float* p) { return *p; }
    static __device__ __forceinline__ f32x4 load4(const float* p) { return *(const f32x4*)p; }
    static __device__ __forceinline__ void store4(float* p, f32x4 v) { *(f32x4*)p = v; }
    static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <> struct Elem<__bf16> {
    static __device__ __forceinline__ float load(const __bf16* p) {
        return bf16_bits_to_f32(*(const uint16_t*)p);
    }
    static __device__ __forceinline__ f32x4 load4(const __bf16* p) {
        const u32x2 r = *(const u32x2*)p;
        const f32x4 v = {bf16_bits_to_f32(r.x & 0xffffu), bf16_bits_to_f32(r.x >> 16),
                         bf16_bits_to_f32(r.y & 0xffffu), bf16_bits_to_f32(r.y >> 16)};
        return v;
    }
    static __device__ __forceinline__ void store4(__bf16* p, f32x4 v) {
        const u32x2 r = {pack_bf16(v.x, v.y), pack_bf16(v.z, v.w)};
        *(u32x2*)p = r;
    }
    static __device__ __forceinline__ void store(__bf16* p, float v) {
        *(uint16_t*)p = (uint16_t)(pack_bf16(v, 0.f) & 0xffffu);
    }
};

// Transposed score tile of one wave (32 queries x BS keys), operands read straight from memory.
// Accumulator element i of key tile kt is key kt*32 + (i/4)*8 + half*4 + i%4 of query qn.
// RAGGED: rows of hd < D elements (hd a multiple of the 16-byte vector); the missing features count as zeros on
// both sides and nothing beyond a row is read.
template <bool RAGGED, typename Vec, typename T>
__device__ __forceinline__ Vec operand_vector(const T* row, uint32_t first, uint32_t hd) {
    if constexpr (RAGGED) {
        const u32x4 zero = {0u, 0u, 0u, 0u};
        return first < hd ? *(const Vec*)(row + first) : __builtin_bit_cast(Vec, zero);
    } else {
        return *(const Vec*)(row + first);
    }
}

template <int BS, int D, typename TIn, bool RAGGED = false>
__device__ __forceinline__ void score_tile_direct(f32x16 (&s)[BS / 32], const TIn* q_row, const TIn* k_blk,
                                                  uint32_t row_stride, uint32_t qn, uint32_t half, uint32_t hd = D) {
    constexpr int KT = BS / 32;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kt][i] = 0.f;
    if constexpr (sizeof(TIn) == 2) {
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
            const bf16x8 b = operand_vector<RAGGED, bf16x8>(q_row, (2 * ks + half) * 8, hd);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const bf16x8 a = operand_vector<RAGGED, bf16x8>(k_blk + (size_t)(kt * 32 + qn) * row_stride, (2 * ks + half) * 8, hd);
                s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, s[kt], 0, 0, 0);
            }
        }
    } else {
#pragma unroll
        for (int g = 0; g < D / 8; ++g) {
            const f32x4 b = operand_vector<RAGGED, f32x4>(q_row, 8 * g + 4 * half, hd);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const f32x4 a = operand_vector<RAGGED, f32x4>(k_blk + (size_t)(kt * 32 + qn) * row_stride, 8 * g + 4 * half, hd);
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    s[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], s[kt], 0, 0, 0);
            }
        }
    }
}

// The same product with the operands fetched ahead of their use: a lane's share of one K tile (KTile) and of its
// query row (QRow) in MFMA operand layout, so that the next tile can be in flight while this one is multiplied.
template <int BS, int D, typename TIn>
struct KTile {
    static constexpr int KT = BS / 32, STEPS = sizeof(TIn) == 2 ? D / 16 : D / 8;
    typedef typename std::conditional<sizeof(TIn) == 2, bf16x8, f32x4>::type Vec;
    Vec v[KT][STEPS];
    template <bool RAGGED = false>
    __device__ __forceinline__ void load(const TIn* k_blk, uint32_t row_stride, uint32_t qn, uint32_t half, uint32_t hd = D) {
        constexpr int W = sizeof(TIn) == 2 ? 8 : 4;   // elements per vector
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int st = 0; st < STEPS; ++st)
                v[kt][st] = operand_vector<RAGGED, Vec>(k_blk + (size_t)(kt * 32 + qn) * row_stride, (2 * st + half) * W, hd);
    }
};
template <int D, typename TIn>
struct QRow {
    static constexpr int STEPS = sizeof(TIn) == 2 ? D / 16 : D / 8;
    typedef typename std::conditional<sizeof(TIn) == 2, bf16x8, f32x4>::type Vec;
    Vec v[STEPS];
    template <bool RAGGED = false>
    __device__ __forceinline__ void load(const TIn* q_row, uint32_t half, uint32_t hd = D) {
        constexpr int W = sizeof(TIn) == 2 ? 8 : 4;
#pragma unroll
        for (int st = 0; st < STEPS; ++st) v[st] = operand_vector<RAGGED, Vec>(q_row, (2 * st + half) * W, hd);
    }
};
template <int BS, int D, typename TIn>
__device__ __forceinline__ void score_tile(f32x16 (&s)[BS / 32], const KTile<BS, D, TIn>& k, const QRow<D, TIn>& q) {
    constexpr int KT = BS / 32;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kt][i] = 0.f;
#pragma unroll
    for (int st = 0; st < QRow<D, TIn>::STEPS; ++st)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
            if constexpr (sizeof(TIn) == 2) {
                s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k.v[kt][st], q.v[st], s[kt], 0, 0, 0);
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    s[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(k.v[kt][st][e], q.v[st][e], s[kt], 0, 0, 0);
            }
        }
}

// A wave's 32 x BS part of a sparse block between registers (MFMA layout: a lane holds one query row in groups of
// 4 keys) and memory, through a wave-private LDS slab so that memory sees whole rows: the 32 rows are contiguous
// in memory (32 * BS elements); straight from the MFMA layout a store instruction would touch all 32 rows with 8
// or 16 bytes each, here every instruction moves 1 KiB of consecutive bytes.
template <int BS, typename T>
struct RowSlab {
    using I = RowSlabIndex<BS, (int)sizeof(T)>;
    static constexpr int ROW_BYTES = I::ROW_BYTES;
    static constexpr int PITCH = I::PITCH;                // padded LDS row
    static constexpr int BYTES = I::BYTES;                // per wave
    static constexpr int CHUNKS = I::CHUNKS;              // 16-byte chunks per row
    static constexpr int ROWS_PER_PASS = I::ROWS_PER_PASS, PASSES = I::PASSES;

    // registers (this lane's query row, groups of 4 keys) -> memory; rows: the wave's first row in memory
    static __device__ __forceinline__ void store(T* rows, const f32x16 (&s)[BS / 32], uint8_t* slab, uint32_t lane) {
        const uint32_t qn = lane & 31, half = lane >> 5;
        T* mine = (T*)(slab + qn * PITCH);
#pragma unroll
        for (int kt = 0; kt < BS / 32; ++kt)
#pragma unroll
            for (int ig = 0; ig < 4; ++ig) {
                const f32x4 v = {s[kt][ig * 4 + 0], s[kt][ig * 4 + 1], s[kt][ig * 4 + 2], s[kt][ig * 4 + 3]};
                Elem<T>::store4(mine + kt * 32 + ig * 8 + half * 4, v);
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            const uint32_t row = pass * ROWS_PER_PASS + lane / CHUNKS, c = lane % CHUNKS;
            const u32x4 v = *(const u32x4*)(slab + row * PITCH + c * 16);
            __builtin_nontemporal_store(v, (u32x4*)((uint8_t*)rows + row * ROW_BYTES + c * 16));
        }
    }
    // memory -> registers in the same layout
    static __device__ __forceinline__ void load(f32x16 (&s)[BS / 32], const T* rows, uint8_t* slab, uint32_t lane) {
        const uint32_t qn = lane & 31, half = lane >> 5;
#pragma unroll
        for (int pass = 0; pass < PASSES; ++pass) {
            const uint32_t row = pass * ROWS_PER_PASS + lane / CHUNKS, c = lane % CHUNKS;
            *(u32x4*)(slab + row * PITCH + c * 16) = *(const u32x4*)((const uint8_t*)rows + row * ROW_BYTES + c * 16);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const T* mine = (const T*)(slab + qn * PITCH);
#pragma unroll
        for (int kt = 0; kt < BS / 32; ++kt)
#pragma unroll
            for (int ig = 0; ig < 4; ++ig) {
                const f32x4 v = Elem<T>::load4(mine + kt * 32 + ig * 8 + half * 4);
                s[kt][ig * 4 + 0] = v.x; s[kt][ig * 4 + 1] = v.y; s[kt][ig * 4 + 2] = v.z; s[kt][ig * 4 + 3] = v.w;
            }
    }
};

// ---------------------------------------------------------------------------------------------
// sdd: grid (blocks, batch, heads), one BS x BS block per work-group (openai_blocksparse.h:224)
// ---------------------------------------------------------------------------------------------
struct SddParams {
    const sfb_uint2* lut;
    const void* a;
    const void* b;
    void* c;
    uint32_t blocks, heads, ctx_a, ctx_b, lut_stride, batch, by_xcd;
    uint32_t state;   // head size of the tensors (the kernels' D is the next multiple of 32)
};

// Blocks per work-group: a launch of one work-group per block is bound by the rate at which work-groups start,
// not by memory; a group of consecutive blocks also keeps the next block's operands in flight under the
// current block's product and write-out.
constexpr uint32_t kSddGroup = 2;

template <int BS, int D, typename TIn, typename TOut, bool RAGGED = false>
__global__ __launch_bounds__(BS * 2) void sdd_nt_kernel(SddParams p) {
    const uint32_t b = blockIdx.y, h = blockIdx.z;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6, qn = lane & 31, half = lane >> 5;
    const uint32_t blk0 = blockIdx.x * kSddGroup;
    const uint32_t n = p.blocks - blk0 < kSddGroup ? p.blocks - blk0 : kSddGroup;
    const sfb_uint2* lut = p.lut + (size_t)h * p.lut_stride + blk0;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const uint32_t row_stride = p.heads * hd;
    __shared__ __attribute__((aligned(16))) uint8_t slabs[BS / 32][RowSlab<BS, TOut>::BYTES];
    TOut* out = (TOut*)p.c + ((((size_t)b * p.heads + h) * p.blocks + blk0) * BS + wave * 32) * BS;
    KTile<BS, D, TIn> k_tile[2];
    QRow<D, TIn> q_row[2];
    auto fetch = [&](uint32_t g, int buf) {
        const sfb_uint2 e = lut[g];
        q_row[buf].template load<RAGGED>((const TIn*)p.a + token_offset(b, e.x * BS + wave * 32 + qn, h, p.ctx_a, p.heads, hd),
                                         half, hd);
        k_tile[buf].template load<RAGGED>((const TIn*)p.b + token_offset(b, e.y * BS, h, p.ctx_b, p.heads, hd), row_stride, qn,
                                          half, hd);
    };
    fetch(0, 0);
#pragma unroll
    for (uint32_t g = 0; g < kSddGroup; ++g) {
        if (g < n) {
            if (g + 1 < n) fetch(g + 1, (g + 1) & 1);
            f32x16 s[BS / 32];
            score_tile<BS, D, TIn>(s, k_tile[g & 1], q_row[g & 1]);
            RowSlab<BS, TOut>::store(out + (size_t)g * BS * BS, s, slabs[wave], lane);
        }
    }
}

// The same product for bf16 operands, 64 x 64 blocks and 64 features: a work-group of two waves walks
// kSddStreamGroup consecutive blocks of the look-up table.  K tiles go straight into LDS (whole 128-byte lines,
// fetched once per block; read as fragments out of memory every line is fetched by both waves in 32-byte pieces),
// two blocks ahead in a ring of three; the query fragments stay in registers while the block-row does not change.
// Every wait is counted in the loads and stores actually issued, which complete in issue order: K(g) is followed
// by the stores of blocks g-2 and g-1 and the loads of K(g+1).
constexpr uint32_t kSddStreamGroup = 8;

template <typename TOut>
__global__ __launch_bounds__(128) void sdd_nt_stream_kernel(SddParams p) {
    constexpr int BS = 64, D = 64, KT = BS / 32;
    using TD = Bf16DirectTiles<BS, D>;
    using Slab = RowSlab<BS, TOut>;
    constexpr int TILE = TD::TILE_BYTES;
    typedef const uint32_t __attribute__((address_space(4)))* const_words;
    __shared__ __attribute__((aligned(1024))) uint8_t tiles[3 * TILE];
    __shared__ __attribute__((aligned(16))) uint8_t slabs[BS / 32][Slab::BYTES];
    // all groups of one (batch, head) run on one XCD (consecutive work-group ids go round the 8 XCDs), one
    // (batch, head) after the other: its K is then fetched into one L2 only and stays there while it is used
    // (the launcher asks for that when there are enough of them to keep all XCDs busy: p.by_xcd)
    const uint32_t groups = (p.blocks + kSddStreamGroup - 1) / kSddStreamGroup;
    const uint32_t bh = p.by_xcd ? (blockIdx.x / 8 / groups) * 8 + blockIdx.x % 8 : blockIdx.x / groups;
    if (bh >= p.batch * p.heads) return;
    const uint32_t b = bh / p.heads, h = bh % p.heads;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t qn = lane & 31, half = lane >> 5;
    const uint32_t blk0 = (p.by_xcd ? blockIdx.x / 8 % groups : blockIdx.x % groups) * kSddStreamGroup;
    const uint32_t n = p.blocks - blk0 < kSddStreamGroup ? p.blocks - blk0 : kSddStreamGroup, last = n - 1;
    const const_words lut_words = (const_words)(uintptr_t)(p.lut + (size_t)h * p.lut_stride + blk0);
    const uint32_t row_bytes = p.heads * D * 2;
    const uint8_t* const k_base = (const uint8_t*)p.b + token_offset(b, 0, h, p.ctx_b, p.heads, D) * 2;
    const uint8_t* const q_base = (const uint8_t*)p.a + token_offset(b, 0, h, p.ctx_a, p.heads, D) * 2;
    const uint32_t src_even = TD::lane_source(lane, 0, row_bytes), src_odd = TD::lane_source(lane, 1, row_bytes);
    const uint32_t lds0 = TD::lds_address(tiles), k_lane = TD::k_lane_base(qn, half);
    const uint32_t q_lane = (wave * 32 + qn) * row_bytes + half * 16;   // k-step ks: 32 bytes further each
    TOut* out = (TOut*)p.c + ((((size_t)b * p.heads + h) * p.blocks + blk0) * BS + wave * 32) * BS;
    auto fetch_k = [&](uint32_t g, uint32_t buf) {
        const uint32_t col = lut_words[2 * g + 1];
        TD::load_tile(lds0 + buf * TILE, k_base + (size_t)col * BS * row_bytes, wave, src_even, src_odd, row_bytes);
    };
    // a fetch past the group's end repeats the last block: the counts stay the same in every step
    fetch_k(0, 0);
    fetch_k(1 < n ? 1 : last, 1);
    u32x4 qf[D / 16];
    uint32_t cur_row = 0xffffffffu;
    for (uint32_t g = 0; g < n; ++g) {
        const uint32_t row = lut_words[2 * g];
        if (row != cur_row) {
            // a new block-row (in the first step, and wherever the group of entries crosses into the next
            // block-row): its query fragments, waited for at once -- which also drains the tiles in flight
            static_assert(D / 16 == 4, "four k-steps");
            const uint8_t* q_rows = q_base + (size_t)row * BS * row_bytes;
            asm volatile("global_load_dwordx4 %0, %4, %5\n\t"
                         "global_load_dwordx4 %1, %4, %5 offset:32\n\t"
                         "global_load_dwordx4 %2, %4, %5 offset:64\n\t"
                         "global_load_dwordx4 %3, %4, %5 offset:96\n\t"
                         "s_waitcnt vmcnt(0)"
                         : "=&v"(qf[0]), "=&v"(qf[1]), "=&v"(qf[2]), "=&v"(qf[3])
                         : "v"(q_lane), "s"(q_rows)
                         : "memory");
            cur_row = row;
        }
        // K(g+1)'s loads and the stores of two blocks: 4 + 2 x 4 (bf16 S) or 4 + 2 x 8 (fp32 S)
        static_assert(Slab::PASSES == SddStreamWait<sizeof(TOut)>::PASSES && TD::LOADS == SddStreamWait<sizeof(TOut)>::LOADS,
                      "the wait counts what this loop issues");
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SddStreamWait<sizeof(TOut)>::COUNT) : "memory");
        __syncthreads();   // K(g) is in LDS for every wave, and every wave is done with K(g-1)
        fetch_k(g + 2 < n ? g + 2 : last, (g + 2) % 3u);
        const uint8_t* k_read = tiles + (g % 3u) * TILE;
        f32x16 s[KT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int i = 0; i < 16; ++i) s[kt][i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks)
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
                s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(TD::k_frag(k_read, k_lane, kt, ks),
                                                                __builtin_bit_cast(bf16x8, qf[ks]), s[kt], 0, 0, 0);
        Slab::store(out + (size_t)g * BS * BS, s, slabs[wave], lane);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing in flight towards LDS when the group ends
}

// ---------------------------------------------------------------------------------------------
// dS = (dO V^T - delta) * P * scale per block: the NT product of the backward pass and the softmax gradient in
// one kernel.  The row term of the gradient, sum_k dP_k P_k (ewops.h:108-113), equals delta_q = sum_d dO_qd O_qd
// because O = P V, so no reduction over the sparse row is needed and dP never goes to memory.
// Grid (blocks, batch, heads) as the sdd.
// ---------------------------------------------------------------------------------------------
struct SddGradParams {
    const sfb_uint2* lut;    // NT LUT
    const void* d_out;       // dO [batch, ctx, heads, D]
    const void* v;           // V  [batch, ctx, heads, D]
    const void* p;           // P  sparse
    const float* delta;      // [batch][heads][ctx]
    void* ds;                // dS sparse
    uint32_t blocks, heads, ctx, lut_stride;
    float scale;
    uint32_t state;          // head size of the tensors
};

template <int BS, int D, typename TIn, typename TS, bool RAGGED = false>
__global__ __launch_bounds__(BS * 2) void sdd_softmax_grad_kernel(SddGradParams p) {
    const uint32_t blk = blockIdx.x, b = blockIdx.y, h = blockIdx.z;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6, qn = lane & 31, half = lane >> 5;
    const sfb_uint2 e = p.lut[(size_t)h * p.lut_stride + blk];
    const uint32_t q = e.x * BS + wave * 32 + qn;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const TIn* do_row = (const TIn*)p.d_out + token_offset(b, q, h, p.ctx, p.heads, hd);
    const TIn* v_blk = (const TIn*)p.v + token_offset(b, e.y * BS, h, p.ctx, p.heads, hd);
    f32x16 s[BS / 32];
    score_tile_direct<BS, D, TIn, RAGGED>(s, do_row, v_blk, p.heads * hd, qn, half, hd);   // dP^T: this lane's query, 16 keys per tile
    const float delta = p.delta[((size_t)b * p.heads + h) * p.ctx + q];
    __shared__ __attribute__((aligned(16))) uint8_t slabs[BS / 32][RowSlab<BS, TS>::BYTES];
    const size_t rows = ((((size_t)b * p.heads + h) * p.blocks + blk) * BS + wave * 32) * BS;   // the wave's 32 rows
    f32x16 pv[BS / 32];
    RowSlab<BS, TS>::load(pv, (const TS*)p.p + rows, slabs[wave], lane);
#pragma unroll
    for (int kt = 0; kt < BS / 32; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kt][i] = (s[kt][i] - delta) * pv[kt][i] * p.scale;
    // the slab is reused: every lane has taken its values out before any lane overwrites them
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    RowSlab<BS, TS>::store((TS*)p.ds + rows, s, slabs[wave], lane);
}

// delta[b][h][q] = sum_d dO[b][q][h][d] * O[b][q][h][d]; 16 lanes per (token, head) row of D elements
template <int D, typename TIn>
__global__ __launch_bounds__(256) void row_dot_kernel(float* delta, const TIn* d_out, const float* o, uint32_t batch,
                                                      uint32_t ctx, uint32_t heads) {
    constexpr int PER = D / 16;   // elements per lane
    const uint64_t row = ((uint64_t)blockIdx.x * 256 + threadIdx.x) / 16;   // over batch * ctx * heads
    const uint32_t part = threadIdx.x & 15;
    if (row >= (uint64_t)batch * ctx * heads) return;
    const TIn* a = d_out + row * D + part * PER;
    const float* c = o + row * D + part * PER;
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) sum += Elem<TIn>::load(a + i) * c[i];
#pragma unroll
    for (int d = 8; d >= 1; d >>= 1) sum += __shfl_xor(sum, d);
    if (part == 0) {
        const uint32_t hh = (uint32_t)(row % heads);
        const uint64_t tok = row / heads;
        const uint32_t bb = (uint32_t)(tok / ctx), qq = (uint32_t)(tok % ctx);
        delta[((size_t)bb * heads + hh) * ctx + qq] = sum;
    }
}

// ---------------------------------------------------------------------------------------------
// masked softmax and its gradient.  One wave owns 4 consecutive query rows of one block-row; a lane owns 8
// consecutive keys, so a wave step covers 8 (BS 64) or 16 (BS 32) key blocks of a row.  The wave has 8
// register slots of one step each: rows of up to 2 steps are processed 4 at a time, rows of up to 4 steps 2
// at a time, rows of up to 8 steps one by one -- one read and one write of memory each; longer rows take
// three passes.  The rows of a block-row share their look-up table entries, which are read once per wave.
// (blocksparse.h:459-722 keeps one CTA per query row; the row-major mask order is the same)
// ---------------------------------------------------------------------------------------------
struct SoftmaxParams {
    const sfb_uint2* lut;     // NN LUT
    const void* mask;         // row-major words[row*blocks + blk], or nullptr
    const int32_t* valid_len;
    const void* x;
    void* y;
    uint32_t blocks, batch, heads, nb, lut_stride, mask_stride;
    float scale_log2e;
};

constexpr int kSoftmaxSlots = 8;      // register slots (steps) of a wave
constexpr int kSoftmaxWaveRows = 4;   // query rows per wave

// The wave's position: rows q0 .. q0+3 of block-row r of (batch, head) bh.
struct SoftmaxWave {
    uint32_t q0, r, bh;
    bool valid;
};
template <int BS>
__device__ __forceinline__ SoftmaxWave softmax_wave(uint32_t batch, uint32_t heads, uint32_t nb) {
    constexpr uint32_t UNITS = BS / kSoftmaxWaveRows;   // waves per block-row
    const uint64_t unit = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    SoftmaxWave w;
    w.valid = unit < (uint64_t)batch * heads * nb * UNITS;
    w.q0 = (uint32_t)(unit % UNITS) * kSoftmaxWaveRows;
    w.r = (uint32_t)((unit / UNITS) % nb);
    w.bh = (uint32_t)(unit / ((uint64_t)UNITS * nb));
    return w;
}
inline uint64_t softmax_grid(uint32_t batch, uint32_t heads, uint32_t nb, uint32_t bs) {
    const uint64_t waves = (uint64_t)batch * heads * nb * (bs / kSoftmaxWaveRows);
    return (waves + 3) / 4;
}

__device__ __forceinline__ float wave_max(float m) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d));
    return m;
}
__device__ __forceinline__ float wave_sum(float l) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) l += __shfl_xor(l, d);
    return l;
}

// 8 consecutive elements of a lane: one 16-byte access for bf16, two for fp32.  S and P are streamed -- read once,
// written once, far larger than the L2 -- so the bf16 accesses carry the non-temporal hint.
template <typename T>
__device__ __forceinline__ void load8(const T* src, float (&v)[8]) {
    if constexpr (sizeof(T) == 2) {
        const u32x4 r = __builtin_nontemporal_load((const u32x4*)src);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = bf16_bits_to_f32(r[i] & 0xffffu);
            v[2 * i + 1] = __builtin_bit_cast(float, r[i] & 0xffff0000u);
        }
    } else {
        const f32x4 lo = *(const f32x4*)src, hi = *(const f32x4*)(src + 4);
        v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
    }
}
template <typename T>
__device__ __forceinline__ void store8(T* dst, const float (&v)[8]) {
    if constexpr (sizeof(T) == 2) {
        const u32x4 r = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
        __builtin_nontemporal_store(r, (u32x4*)dst);
    } else {
        const f32x4 lo = {v[0], v[1], v[2], v[3]}, hi = {v[4], v[5], v[6], v[7]};
        *(f32x4*)dst = lo;
        *(f32x4*)(dst + 4) = hi;
    }
}

// The same 8 elements kept in their storage type (4 registers for bf16, 8 for fp32) until they are used
template <typename T> struct Packed8;
template <> struct Packed8<float> {
    f32x4 lo, hi;
    __device__ __forceinline__ void load(const float* src) { lo = *(const f32x4*)src; hi = *(const f32x4*)(src + 4); }
    __device__ __forceinline__ float get(int i) const { return i < 4 ? lo[i] : hi[i - 4]; }
    __device__ __forceinline__ void unpack_after(float&) {}
};
template <> struct Packed8<__bf16> {
    u32x4 r;
    __device__ __forceinline__ void load(const __bf16* src) { r = __builtin_nontemporal_load((const u32x4*)src); }
    __device__ __forceinline__ float get(int i) const {
        return (i & 1) ? __builtin_bit_cast(float, r[i >> 1] & 0xffff0000u) : bf16_bits_to_f32(r[i >> 1] & 0xffffu);
    }
    // Keeps the compiler from unpacking all elements long before `dep` is known (which would cost the registers
    // that the packed form saves): later get() calls depend on this point.
    __device__ __forceinline__ void unpack_after(float& dep) {
        uint32_t a = r[0], b = r[1], c = r[2], d = r[3];
        asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d), "+v"(dep));
        r[0] = a; r[1] = b; r[2] = c; r[3] = d;
    }
};

template <int BS, typename TX, typename TY>
struct SoftmaxRows {
    static constexpr int LPB = BS / 8;     // lanes per key block: every lane owns 8 consecutive keys
    static constexpr int PER = 64 / LPB;   // key blocks covered by one wave step
    const sfb_uint2* lut;    // this head's table
    const uint8_t* mask;     // this head's row-major words, or nullptr
    const TX* x;             // this (batch, head)'s blocks
    TY* y;
    uint32_t off, count, blocks, sub, key0;
    int valid;
    float c;

    // keep bits of this lane's 8 keys of query row qi in key block e
    __device__ __forceinline__ uint32_t keep_bits(const sfb_uint2 e, uint32_t qi) const {
        const int left = valid - (int)(e.y * BS + key0);
        uint32_t k = left >= 8 ? 0xffu : (left <= 0 ? 0u : ((1u << left) - 1u));
        if (mask) {
            const size_t w = (size_t)qi * blocks + e.x;
            uint64_t word;
            if (BS == 64) word = ((const uint64_t*)mask)[w];
            else if (BS == 32) word = ((const uint32_t*)mask)[w];
            else if (BS == 16) word = ((const uint16_t*)mask)[w];
            else word = mask[w];
            k &= (uint32_t)(word >> key0);
        }
        return k;
    }
    __device__ __forceinline__ size_t at(const sfb_uint2 e, uint32_t qi) const {
        return ((size_t)e.x * BS + qi) * BS + key0;
    }

    // R rows of up to S steps each, all in registers: one read, one write.  Maximum over kept keys (seed as
    // ewops.h:70), sum relative to it, normalised probabilities with zeros at masked keys (ewops.h:82).
    // MASKED = false skips the keep bits (no element mask, no key padding).  Masked scores are replaced by
    // kMaskedScore, whose exponential is an exact zero.
    template <int R, int S, bool MASKED>
    __device__ __forceinline__ void in_registers(uint32_t q0) const {
        static_assert(R * S == kSoftmaxSlots, "slots");
        float v[R][S][8];
        sfb_uint2 ent[S];
#pragma unroll
        for (int st = 0; st < S; ++st) {
            const uint32_t j = st * PER + sub;
            ent[st].x = 0xffffffffu;
            if (j < count) ent[st] = lut[off + j];
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int st = 0; st < S; ++st) {
                if (ent[st].x != 0xffffffffu) {
                    load8<TX>(x + at(ent[st], q0 + rr), v[rr][st]);
                    if (MASKED) {
                        const uint32_t keep = keep_bits(ent[st], q0 + rr);
#pragma unroll
                        for (int i = 0; i < 8; ++i) v[rr][st][i] = ((keep >> i) & 1u) ? v[rr][st][i] : kMaskedScore;
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[rr][st][i] = kMaskedScore;
                }
            }
        float m[R];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            float m0 = kMaxSeed, m1 = kMaxSeed;
#pragma unroll
            for (int st = 0; st < S; ++st)
#pragma unroll
                for (int i = 0; i < 8; i += 4) {
                    m0 = fmaxf(fmaxf(m0, v[rr][st][i]), v[rr][st][i + 1]);
                    m1 = fmaxf(fmaxf(m1, v[rr][st][i + 2]), v[rr][st][i + 3]);
                }
            m[rr] = fmaxf(m0, m1);
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) m[rr] = wave_max(m[rr]);
        float l[R];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const float mc = m[rr] * c;
            float l0 = 0.f, l1 = 0.f;
#pragma unroll
            for (int st = 0; st < S; ++st)
#pragma unroll
                for (int i = 0; i < 8; i += 2) {
                    v[rr][st][i] = exp2_fast(__builtin_fmaf(v[rr][st][i], c, -mc));
                    v[rr][st][i + 1] = exp2_fast(__builtin_fmaf(v[rr][st][i + 1], c, -mc));
                    l0 += v[rr][st][i];
                    l1 += v[rr][st][i + 1];
                }
            l[rr] = l0 + l1;
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) l[rr] = wave_sum(l[rr]);
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const float inv = 1.0f / (l[rr] + 1e-6f);
#pragma unroll
            for (int st = 0; st < S; ++st)
                if (ent[st].x != 0xffffffffu) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) v[rr][st][i] *= inv;
                    store8<TY>(y + at(ent[st], q0 + rr), v[rr][st]);
                }
        }
    }
    // The same for bf16 scores, which stay packed in registers (half the registers, twice the waves per SIMD);
    // the exponentials are computed once for the sum and once more for the result.
    template <int R, int S, bool MASKED>
    __device__ __forceinline__ void in_registers_packed(uint32_t q0) const {
        static_assert(R * S == kSoftmaxSlots && sizeof(TX) == 2, "slots");
        constexpr uint32_t kMaskedPair = 0xff7fff7fu;   // two bf16 of -3.39e38
        Packed8<TX> v[R][S];
        sfb_uint2 ent[S];
#pragma unroll
        for (int st = 0; st < S; ++st) {
            const uint32_t j = st * PER + sub;
            ent[st].x = 0xffffffffu;
            if (j < count) ent[st] = lut[off + j];
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int st = 0; st < S; ++st) {
#pragma unroll
                for (int i = 0; i < 4; ++i) v[rr][st].r[i] = kMaskedPair;
                if (ent[st].x != 0xffffffffu) {
                    v[rr][st].load(x + at(ent[st], q0 + rr));
                    if (MASKED) {
                        const uint32_t keep = keep_bits(ent[st], q0 + rr);
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const uint32_t lo = 0u - ((keep >> (2 * i)) & 1u), hi = 0u - ((keep >> (2 * i + 1)) & 1u);
                            const uint32_t sel = (lo & 0xffffu) | (hi & 0xffff0000u);
                            v[rr][st].r[i] = (v[rr][st].r[i] & sel) | (kMaskedPair & ~sel);
                        }
                    }
                }
            }
        float m[R];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            float m0 = kMaxSeed, m1 = kMaxSeed;
#pragma unroll
            for (int st = 0; st < S; ++st)
#pragma unroll
                for (int i = 0; i < 8; i += 4) {
                    m0 = fmaxf(fmaxf(m0, v[rr][st].get(i)), v[rr][st].get(i + 1));
                    m1 = fmaxf(fmaxf(m1, v[rr][st].get(i + 2)), v[rr][st].get(i + 3));
                }
            m[rr] = fmaxf(m0, m1);
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) m[rr] = wave_max(m[rr]);
        float l[R];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            float mc = m[rr] * c;
            float l0 = 0.f, l1 = 0.f;
#pragma unroll
            for (int st = 0; st < S; ++st) {
                v[rr][st].unpack_after(mc);
#pragma unroll
                for (int i = 0; i < 8; i += 2) {
                    l0 += exp2_fast(__builtin_fmaf(v[rr][st].get(i), c, -mc));
                    l1 += exp2_fast(__builtin_fmaf(v[rr][st].get(i + 1), c, -mc));
                }
            }
            l[rr] = l0 + l1;
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) l[rr] = wave_sum(l[rr]);
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const float mc = m[rr] * c;
            float inv = 1.0f / (l[rr] + 1e-6f);
#pragma unroll
            for (int st = 0; st < S; ++st)
                if (ent[st].x != 0xffffffffu) {
                    v[rr][st].unpack_after(inv);
                    float out[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) out[i] = exp2_fast(__builtin_fmaf(v[rr][st].get(i), c, -mc)) * inv;
                    store8<TY>(y + at(ent[st], q0 + rr), out);
                }
        }
    }
    template <int R, int S>
    __device__ __forceinline__ void in_registers(uint32_t q0, bool masked) const {
        if constexpr (sizeof(TX) == 2) {
            if (masked) in_registers_packed<R, S, true>(q0);
            else in_registers_packed<R, S, false>(q0);
        } else {
            if (masked) in_registers<R, S, true>(q0);
            else in_registers<R, S, false>(q0);
        }
    }

    // a row of any length: three passes over memory
    __device__ __forceinline__ void in_passes(uint32_t qi) const {
        float m = kMaxSeed;
        for (uint32_t j = sub; j < count; j += PER) {
            const sfb_uint2 e = lut[off + j];
            float v[8];
            load8<TX>(x + at(e, qi), v);
            const uint32_t k = keep_bits(e, qi);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if ((k >> i) & 1u) m = fmaxf(m, v[i]);
        }
        m = wave_max(m);
        float l = 0.f;
        for (uint32_t j = sub; j < count; j += PER) {
            const sfb_uint2 e = lut[off + j];
            float v[8];
            load8<TX>(x + at(e, qi), v);
            const uint32_t k = keep_bits(e, qi);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if ((k >> i) & 1u) l += exp2_fast((v[i] - m) * c);
        }
        l = wave_sum(l);
        const float inv = 1.0f / (l + 1e-6f);
        for (uint32_t j = sub; j < count; j += PER) {
            const sfb_uint2 e = lut[off + j];
            float v[8];
            load8<TX>(x + at(e, qi), v);
            const uint32_t k = keep_bits(e, qi);
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = ((k >> i) & 1u) ? exp2_fast((v[i] - m) * c) * inv : 0.f;
            store8<TY>(y + at(e, qi), v);
        }
    }
};

template <int BS, typename TX, typename TY>
__global__ __launch_bounds__(256) void masked_softmax_kernel(SoftmaxParams p) {
    using Rows = SoftmaxRows<BS, TX, TY>;
    const SoftmaxWave w = softmax_wave<BS>(p.batch, p.heads, p.nb);
    if (!w.valid) return;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t b = w.bh / p.heads, h = w.bh % p.heads;
    Rows rows;
    rows.lut = p.lut + (size_t)h * p.lut_stride;
    rows.mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
    rows.x = (const TX*)p.x + (size_t)w.bh * p.blocks * BS * BS;
    rows.y = (TY*)p.y + (size_t)w.bh * p.blocks * BS * BS;
    rows.off = rows.lut[w.r].x;
    rows.count = rows.lut[w.r].y;
    rows.blocks = p.blocks;
    rows.sub = lane / Rows::LPB;
    rows.key0 = (lane % Rows::LPB) * 8;
    rows.valid = p.valid_len ? p.valid_len[b] : (int)(p.nb * BS);
    rows.c = p.scale_log2e;
    const uint32_t steps = (rows.count + Rows::PER - 1) / Rows::PER;
    const bool masked = rows.mask != nullptr || rows.valid < (int)(p.nb * BS);
    if (steps <= 2) {
        rows.template in_registers<4, 2>(w.q0, masked);
    } else if (steps <= 4) {
        rows.template in_registers<2, 4>(w.q0, masked);
        rows.template in_registers<2, 4>(w.q0 + 2, masked);
    } else if (steps <= 8) {
        for (uint32_t i = 0; i < kSoftmaxWaveRows; ++i) rows.template in_registers<1, 8>(w.q0 + i, masked);
    } else {
        for (uint32_t i = 0; i < kSoftmaxWaveRows; ++i) rows.in_passes(w.q0 + i);
    }
}

// ---------------------------------------------------------------------------------------------
// The same softmax for bf16 scores in 64 x 64 blocks, by units of 8 query rows: 8 lanes hold one row of a key
// block (16 bytes each), so a wave instruction moves 8 whole rows = 1 KiB of consecutive bytes, the row
// reductions stay inside groups of 8 lanes (three DPP steps), and a wave needs one register slot per block of the
// row -- no slot is spent on blocks the row does not have.  A work-group of four waves owns 32 rows of a
// block-row: rows of up to 16 blocks one unit per wave, rows of up to 64 blocks one unit after the other with a
// quarter of the blocks per wave (maximum and sum combined through LDS), longer rows in three passes over memory.
// ---------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
// all-reduce over aligned groups of 8 lanes: lane ^ 1, lane ^ 2 (quad permutes), then the mirrored half row
__device__ __forceinline__ float max_of_8(float x) {
    x = fmaxf(x, dpp_move<0xB1>(x));
    x = fmaxf(x, dpp_move<0x4E>(x));
    return fmaxf(x, dpp_move<0x141>(x));
}
__device__ __forceinline__ float sum_of_8(float x) {
    x += dpp_move<0xB1>(x);
    x += dpp_move<0x4E>(x);
    return x + dpp_move<0x141>(x);
}

template <typename TY>
struct SoftmaxUnit {
    static constexpr int BS = 64, SLOTS = 16;
    static constexpr uint32_t kMaskedPair = 0xff7fff7fu;   // two bf16 of -3.39e38
    typedef const uint32_t __attribute__((address_space(4)))* const_words;
    const_words lut;          // entries of this block-row part: {block, column} pairs
    const uint8_t* mask;      // this head's row-major words, or nullptr
    const uint8_t* x;         // this (batch, head)'s blocks
    uint8_t* y;
    uint32_t blocks, lane;
    int valid;
    float c;

    __device__ __forceinline__ uint32_t keep_bits(uint32_t blk, uint32_t col, uint32_t qi) const {
        const uint32_t key0 = (lane & 7u) * 8u;
        const int left = valid - (int)(col * BS + key0);
        uint32_t k = left >= 8 ? 0xffu : (left <= 0 ? 0u : ((1u << left) - 1u));
        if (mask) k &= (uint32_t)(((const uint64_t*)mask)[(size_t)qi * blocks + blk] >> key0);
        return k;
    }
    static __device__ __forceinline__ float elem(const u32x4& r, int i) {
        return (i & 1) ? __builtin_bit_cast(float, r[i >> 1] & 0xffff0000u) : bf16_bits_to_f32(r[i >> 1] & 0xffffu);
    }
    // Keeps the compiler from unpacking a slot long before `dep` is known and holding the floats from one pass
    // to the next (which would cost the registers that the packed form saves).
    static __device__ __forceinline__ void unpack_after(u32x4& r, float& dep) {
        uint32_t a = r[0], b = r[1], c2 = r[2], d = r[3];
        asm volatile("" : "+v"(a), "+v"(b), "+v"(c2), "+v"(d), "+v"(dep));
        r[0] = a; r[1] = b; r[2] = c2; r[3] = d;
    }
    __device__ __forceinline__ void store(uint32_t blk, uint32_t q0, const float (&out)[8]) const {
        if constexpr (sizeof(TY) == 2) {
            const u32x4 r = {pack_bf16(out[0], out[1]), pack_bf16(out[2], out[3]), pack_bf16(out[4], out[5]),
                             pack_bf16(out[6], out[7])};
            __builtin_nontemporal_store(r, (u32x4*)(y + ((size_t)blk * (BS * BS * 2) + q0 * (BS * 2)) + lane * 16u));
        } else {
            float* dst = (float*)(y + ((size_t)blk * (BS * BS * 4) + q0 * (BS * 4)) + lane * 32u);
            const f32x4 lo = {out[0], out[1], out[2], out[3]}, hi = {out[4], out[5], out[6], out[7]};
            __builtin_nontemporal_store(lo, (f32x4*)dst);
            __builtin_nontemporal_store(hi, (f32x4*)(dst + 4));
        }
    }

    // Rows q0 .. q0+7 over `count` <= NS blocks starting at entry `first`, all in registers.  NS is count rounded
    // up to 4: only the last three slots need a look at count.  SHARED: the row's other blocks are with the other
    // three waves; red: [2][4][8] floats.
    template <int NS, bool MASKED, bool SHARED>
    __device__ __forceinline__ void in_registers(uint32_t q0, uint32_t first, uint32_t count, float* red,
                                                 uint32_t wave) const {
        u32x4 v[NS];
        uint32_t blk[NS];
        const uint32_t qi = q0 + (lane >> 3), lane16 = lane * 16;
#define SFB_LIVE(s) ((s) <= NS - 4 || (uint32_t)(s) < count)
#pragma unroll
        for (int s = 0; s < NS; ++s)
            if (SFB_LIVE(s)) {
                blk[s] = lut[2 * (first + s)];
                // uniform base + 32-bit lane offset
                v[s] = __builtin_nontemporal_load((const u32x4*)(x + ((size_t)blk[s] * (BS * BS * 2) + q0 * (BS * 2)) + lane16));
                if (MASKED) {
                    const uint32_t keep = keep_bits(blk[s], lut[2 * (first + s) + 1], qi);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const uint32_t lo = 0u - ((keep >> (2 * i)) & 1u), hi = 0u - ((keep >> (2 * i + 1)) & 1u);
                        const uint32_t sel = (lo & 0xffffu) | (hi & 0xffff0000u);
                        v[s][i] = (v[s][i] & sel) | (kMaskedPair & ~sel);
                    }
                }
            }
        float m0 = kMaxSeed, m1 = kMaxSeed;
#pragma unroll
        for (int s = 0; s < NS; ++s)
            if (SFB_LIVE(s)) {
#pragma unroll
                for (int i = 0; i < 8; i += 4) {
                    m0 = fmaxf(fmaxf(m0, elem(v[s], i)), elem(v[s], i + 1));
                    m1 = fmaxf(fmaxf(m1, elem(v[s], i + 2)), elem(v[s], i + 3));
                }
            }
        float m = max_of_8(fmaxf(m0, m1));
        if (SHARED) {
            if ((lane & 7u) == 0) red[wave * 8 + (lane >> 3)] = m;
            __syncthreads();
            const uint32_t g = lane >> 3;
            m = fmaxf(fmaxf(red[g], red[8 + g]), fmaxf(red[16 + g], red[24 + g]));
        }
        float mc = m * c;
        float l0 = 0.f, l1 = 0.f;
#pragma unroll
        for (int s = 0; s < NS; ++s)
            if (SFB_LIVE(s)) {
                unpack_after(v[s], mc);
#pragma unroll
                for (int i = 0; i < 8; i += 2) {
                    l0 += exp2_fast(__builtin_fmaf(elem(v[s], i), c, -mc));
                    l1 += exp2_fast(__builtin_fmaf(elem(v[s], i + 1), c, -mc));
                }
            }
        float l = sum_of_8(l0 + l1);
        if (SHARED) {
            if ((lane & 7u) == 0) red[32 + wave * 8 + (lane >> 3)] = l;
            __syncthreads();
            const uint32_t g = lane >> 3;
            l = (red[32 + g] + red[40 + g]) + (red[48 + g] + red[56 + g]);
        }
        float inv = 1.0f / (l + 1e-6f);
#pragma unroll
        for (int s = 0; s < NS; ++s)
            if (SFB_LIVE(s)) {
                unpack_after(v[s], inv);
                float out[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) out[i] = exp2_fast(__builtin_fmaf(elem(v[s], i), c, -mc)) * inv;
                store(blk[s], q0, out);
            }
#undef SFB_LIVE
    }
    template <bool SHARED>
    __device__ __forceinline__ void in_registers(uint32_t q0, uint32_t first, uint32_t count, bool masked, float* red,
                                                 uint32_t wave) const {
#define SFB_ROWS(NS)                                                                      \
    do {                                                                                  \
        if (masked) in_registers<NS, true, SHARED>(q0, first, count, red, wave);          \
        else in_registers<NS, false, SHARED>(q0, first, count, red, wave);                \
    } while (0)
        if (count <= 4) SFB_ROWS(4);
        else if (count <= 8) SFB_ROWS(8);
        else if (count <= 12) SFB_ROWS(12);
        else SFB_ROWS(16);
#undef SFB_ROWS
    }

    // rows q0 .. q0+7 of any length: three passes over memory
    __device__ __forceinline__ void in_passes(uint32_t q0, uint32_t count) const {
        const uint32_t qi = q0 + (lane >> 3);
        auto fetch = [&](uint32_t j, u32x4& r, uint32_t& keep) -> uint32_t {
            const uint32_t blk = lut[2 * j];
            r = *(const u32x4*)(x + (size_t)blk * (BS * BS * 2) + q0 * (BS * 2) + lane * 16);
            keep = keep_bits(blk, lut[2 * j + 1], qi);
            return blk;
        };
        float m = kMaxSeed;
        for (uint32_t j = 0; j < count; ++j) {
            u32x4 r;
            uint32_t keep;
            fetch(j, r, keep);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if ((keep >> i) & 1u) m = fmaxf(m, elem(r, i));
        }
        m = max_of_8(m);
        float l = 0.f;
        for (uint32_t j = 0; j < count; ++j) {
            u32x4 r;
            uint32_t keep;
            fetch(j, r, keep);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if ((keep >> i) & 1u) l += exp2_fast((elem(r, i) - m) * c);
        }
        l = sum_of_8(l);
        const float inv = 1.0f / (l + 1e-6f);
        for (uint32_t j = 0; j < count; ++j) {
            u32x4 r;
            uint32_t keep;
            const uint32_t blk = fetch(j, r, keep);
            float out[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) out[i] = ((keep >> i) & 1u) ? exp2_fast((elem(r, i) - m) * c) * inv : 0.f;
            store(blk, q0, out);
        }
    }
};

template <typename TY>
__global__ __launch_bounds__(256) void masked_softmax_rows8_kernel(SoftmaxParams p) {
    constexpr int BS = 64;
    using Unit = SoftmaxUnit<TY>;
    __shared__ float red[64];
    // 32 rows of a block-row per work-group.  Block-rows are taken from both ends of the context inwards, the last
    // and the first one of every (batch, head) before anything else: the long rows of causal layouts are the
    // last ones, those of layouts with global tokens the first and the last, and a long row that starts late is
    // the tail of the launch.
    const uint32_t part = blockIdx.x & 1u, item = blockIdx.x >> 1, num_bh = p.batch * p.heads;
    const uint32_t ends = p.nb >= 2 ? 2u : 0u;
    uint32_t rank, bh;
    if (item < ends * num_bh) {
        rank = item / num_bh;
        bh = item % num_bh;
    } else {
        rank = ends + (item - ends * num_bh) % (p.nb - ends);
        bh = (item - ends * num_bh) / (p.nb - ends);
    }
    const uint32_t r = (rank & 1u) ? rank / 2 : p.nb - 1 - rank / 2;
    const uint32_t b = bh / p.heads, h = bh % p.heads;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const sfb_uint2* lut = p.lut + (size_t)h * p.lut_stride;
    const typename Unit::const_words head = (typename Unit::const_words)(uintptr_t)lut;
    const uint32_t off = head[2 * r], count = head[2 * r + 1];
    Unit u;
    u.lut = head + 2 * (size_t)off;
    u.mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
    u.x = (const uint8_t*)p.x + (size_t)bh * p.blocks * (BS * BS * 2);
    u.y = (uint8_t*)p.y + (size_t)bh * p.blocks * (BS * BS * sizeof(TY));
    u.blocks = p.blocks;
    u.lane = threadIdx.x & 63;
    u.valid = p.valid_len ? p.valid_len[b] : (int)(p.nb * BS);
    u.c = p.scale_log2e;
    const bool masked = u.mask != nullptr || u.valid < (int)(p.nb * BS);
    const uint32_t q0 = part * 32;
    if (count <= Unit::SLOTS) {
        if (count > 0) u.template in_registers<false>(q0 + wave * 8, 0, count, masked, red, wave);
    } else if (count <= 4 * Unit::SLOTS) {
        const uint32_t per = (count + 3) / 4, first = wave * per;
        const uint32_t mine = first >= count ? 0u : (count - first < per ? count - first : per);
        for (uint32_t unit = 0; unit < 4; ++unit)
            u.template in_registers<true>(q0 + unit * 8, first < count ? first : 0u, mine, masked, red, wave);
    } else {
        u.in_passes(q0 + wave * 8, count);
    }
}

// dx = (dy - sum_k dy*y) * y * scale per query row (ewops.h:101-124); same decomposition, with register
// slots for dy and for y that hold the storage type
struct SoftmaxGradParams {
    const sfb_uint2* lut;     // NN LUT
    const void* dy;
    const void* y;
    void* dx;
    uint32_t blocks, batch, heads, nb, lut_stride;
    float scale;
};

template <int BS, typename T>
struct SoftmaxGradRows {
    static constexpr int LPB = BS / 8, PER = 64 / LPB;
    const sfb_uint2* lut;
    const T* dy;
    const T* y;
    T* dx;
    uint32_t off, count, sub, key0;
    float scale;

    __device__ __forceinline__ size_t at(uint32_t blk, uint32_t qi) const {
        return ((size_t)blk * BS + qi) * BS + key0;
    }
    // register slots for dy and for y: 8 steps each (32 registers for bf16, 64 for fp32)
    static constexpr int SLOTS = kSoftmaxSlots;
    template <int R, int S>
    __device__ __forceinline__ void in_registers(uint32_t q0) const {
        static_assert(R * S == SLOTS, "slots");
        Packed8<T> g[R][S], v[R][S];
        uint32_t blk[S];
#pragma unroll
        for (int st = 0; st < S; ++st) {
            const uint32_t j = st * PER + sub;
            blk[st] = 0xffffffffu;
            if (j < count) blk[st] = lut[off + j].x;
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int st = 0; st < S; ++st)
                if (blk[st] != 0xffffffffu) {
                    g[rr][st].load(dy + at(blk[st], q0 + rr));
                    v[rr][st].load(y + at(blk[st], q0 + rr));
                }
        float sum[R];
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int st = 0; st < S; ++st)
                if (blk[st] != 0xffffffffu) {
#pragma unroll
                    for (int i = 0; i < 8; i += 2) {
                        s0 = __builtin_fmaf(g[rr][st].get(i), v[rr][st].get(i), s0);
                        s1 = __builtin_fmaf(g[rr][st].get(i + 1), v[rr][st].get(i + 1), s1);
                    }
                }
            sum[rr] = s0 + s1;
        }
#pragma unroll
        for (int rr = 0; rr < R; ++rr) sum[rr] = wave_sum(sum[rr]);
#pragma unroll
        for (int rr = 0; rr < R; ++rr)
#pragma unroll
            for (int st = 0; st < S; ++st)
                if (blk[st] != 0xffffffffu) {
                    g[rr][st].unpack_after(sum[rr]);
                    v[rr][st].unpack_after(sum[rr]);
                    float out[8];
#pragma unroll
                    for (int i = 0; i < 8; ++i) out[i] = (g[rr][st].get(i) - sum[rr]) * v[rr][st].get(i) * scale;
                    store8<T>(dx + at(blk[st], q0 + rr), out);
                }
    }
    __device__ __forceinline__ void in_passes(uint32_t qi) const {
        float sum = 0.f;
        for (uint32_t j = sub; j < count; j += PER) {
            const uint32_t b = lut[off + j].x;
            float g[8], v[8];
            load8<T>(dy + at(b, qi), g);
            load8<T>(y + at(b, qi), v);
#pragma unroll
            for (int i = 0; i < 8; ++i) sum += g[i] * v[i];
        }
        sum = wave_sum(sum);
        for (uint32_t j = sub; j < count; j += PER) {
            const uint32_t b = lut[off + j].x;
            float g[8], v[8];
            load8<T>(dy + at(b, qi), g);
            load8<T>(y + at(b, qi), v);
#pragma unroll
            for (int i = 0; i < 8; ++i) g[i] = (g[i] - sum) * v[i] * scale;
            store8<T>(dx + at(b, qi), g);
        }
    }
};

template <int BS, typename T>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(sizeof(T) == 2 ? 4 : 2))) void masked_softmax_grad_kernel(
    SoftmaxGradParams p) {
    using Rows = SoftmaxGradRows<BS, T>;
    const SoftmaxWave w = softmax_wave<BS>(p.batch, p.heads, p.nb);
    if (!w.valid) return;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t h = w.bh % p.heads;
    const size_t head_base = (size_t)w.bh * p.blocks * BS * BS;
    Rows rows;
    rows.lut = p.lut + (size_t)h * p.lut_stride;
    rows.dy = (const T*)p.dy + head_base;
    rows.y = (const T*)p.y + head_base;
    rows.dx = (T*)p.dx + head_base;
    rows.off = rows.lut[w.r].x;
    rows.count = rows.lut[w.r].y;
    rows.sub = lane / Rows::LPB;
    rows.key0 = (lane % Rows::LPB) * 8;
    rows.scale = p.scale;
    constexpr int SLOTS = Rows::SLOTS;
    const uint32_t steps = (rows.count + Rows::PER - 1) / Rows::PER;
    if (steps <= SLOTS / 4) {
        rows.template in_registers<4, SLOTS / 4>(w.q0);
    } else if (steps <= SLOTS / 2) {
        rows.template in_registers<2, SLOTS / 2>(w.q0);
        rows.template in_registers<2, SLOTS / 2>(w.q0 + 2);
    } else if (steps <= SLOTS) {
        for (uint32_t i = 0; i < kSoftmaxWaveRows; ++i) rows.template in_registers<1, SLOTS>(w.q0 + i);
    } else {
        for (uint32_t i = 0; i < kSoftmaxWaveRows; ++i) rows.in_passes(w.q0 + i);
    }
}

// the same for rows of any length (head sizes that are not multiples of 32): lane `part` takes elements part, part + 16, ..
template <typename TIn>
__global__ __launch_bounds__(256) void row_dot_any_kernel(float* delta, const TIn* d_out, const float* o, uint32_t batch,
                                                          uint32_t ctx, uint32_t heads, uint32_t hd) {
    const uint64_t row = ((uint64_t)blockIdx.x * 256 + threadIdx.x) / 16;
    const uint32_t part = threadIdx.x & 15;
    const bool live = row < (uint64_t)batch * ctx * heads;   // whole groups of 16 lanes: the shuffles below stay among live lanes
    float sum = 0.f;
    if (live)
        for (uint32_t i = part; i < hd; i += 16) sum += Elem<TIn>::load(d_out + row * hd + i) * o[row * hd + i];
#pragma unroll
    for (int d = 8; d >= 1; d >>= 1) sum += __shfl_xor(sum, d);
    if (live && part == 0) {
        const uint32_t hh = (uint32_t)(row % heads);
        const uint64_t tok = row / heads;
        const uint32_t bb = (uint32_t)(tok / ctx), qq = (uint32_t)(tok % ctx);
        delta[((size_t)bb * heads + hh) * ctx + qq] = sum;
    }
}

// ---------------------------------------------------------------------------------------------
// dsd, transposed sparse operand (TN): C[col block] = sum over the column's blocks of A_blk^T . B_rowblk
// (matmul.h:81-99; dV = P^T dO and dK = dS^T Q of the backward pass).  One work-group per (batch, head,
// key-block column); wave w owns keys 32w .. 32w+31 of the column block and all D output columns:
//   C^T[col][key] += sum_q B[q][col] * A[q][key]      (MFMA: A-operand = B^T tile, B-operand = A tile)
// Both tiles are stored row-major with the contraction index q as the row, so both operands are read
// k-major: bf16 tiles through the transposing LDS read, fp32 one element per lane.
// ---------------------------------------------------------------------------------------------
struct DsdParams {
    const sfb_uint2* lut;   // NN LUT (header per block-row) or TN LUT (header per block-column)
    const void* a;          // sparse operand: P, or dS
    const void* b;          // dense operand: V, or dO / Q
    float* c;               // dense result
    uint32_t blocks, batch, heads, nb_b, nb_c, lut_stride, groups;
    uint32_t state;         // head size of the dense tensors (the kernels' D is the next multiple of 32)
    // Scheduled launches (items != nullptr): one work-group per work item of sfb_build_schedule over `lut` instead of
    // one per line.  A chunk of a split line leaves its sum in a record of `partials`
    // ([batch * heads][n_parts][BS][D] floats); dsd_reduce_kernel adds the records of a line afterwards.
    const sfb_work_item* items;
    uint32_t item_stride, ranks, heavy, n_parts;
    float* partials;
};

// The line (block-row of an NN launch, block-column of a TN launch) of a work-group, or the part of it that a work
// item of a scheduled launch covers.
struct DsdLine {
    uint32_t bh, line;
    uint32_t off, count;    // the look-up entries lut[off .. off + count) of the head's table
    uint32_t record;        // chunk of a split line: index + 1 of its record among the (batch, head)'s; else 0
    bool valid;
};

template <bool ITEMS>
__device__ __forceinline__ DsdLine decode_dsd_line(const DsdParams& p) {
    DsdLine w;
    if constexpr (ITEMS) {
        const WorkId id = decode_work(blockIdx.x, p.batch * p.heads, p.ranks, p.heavy);
        w.valid = id.valid;
        w.bh = id.bh;
        const sfb_work_item it = p.items[(size_t)(id.valid ? id.bh % p.heads : 0u) * p.item_stride + id.rank];
        if (it.row == SFB_WORK_ITEM_SKIP) w.valid = false;   // filler of a head whose list is shorter than the longest
        w.line = __builtin_amdgcn_readfirstlane(it.row);
        w.off = __builtin_amdgcn_readfirstlane(it.lut_first);
        w.count = __builtin_amdgcn_readfirstlane(it.count);
        w.record = __builtin_amdgcn_readfirstlane(it.nchunks > 1 ? it.part + it.chunk + 1 : 0u);
        return w;
    }
    // Lines are taken from both ends of the context inwards, the last and the first one of every head before
    // anything else: the long rows of causal layouts are the last ones (blocksparse.h:746-748), those of layouts
    // with global tokens the first and the last; started late, a long line is the tail of the launch.
    const WorkId id = decode_work(blockIdx.x, p.batch * p.heads, p.nb_c, p.nb_c >= 2 ? 2 : 0);
    w.valid = id.valid;
    w.bh = id.bh;
    w.line = (id.rank & 1u) ? id.rank / 2 : p.nb_c - 1 - id.rank / 2;
    w.record = 0;
    if (id.valid) {
        const sfb_uint2 header = p.lut[(size_t)(id.bh % p.heads) * p.lut_stride + w.line];
        w.off = __builtin_amdgcn_readfirstlane(header.x);
        w.count = __builtin_amdgcn_readfirstlane(header.y);
    } else {
        w.off = w.count = 0;
    }
    return w;
}

// Where a lane's output row goes: the dense result, or the record of a split line's chunk (rows of D floats).
template <int BS, int D, bool ITEMS>
__device__ __forceinline__ float* dsd_output_row(const DsdParams& p, const DsdLine& w, uint32_t b, uint32_t h,
                                                 uint32_t row_in_block, uint32_t hd) {
    if (ITEMS && w.record) return p.partials + ((((size_t)w.bh * p.n_parts + (w.record - 1)) * BS) + row_in_block) * D;
    return p.c + token_offset(b, w.line * BS + row_in_block, h, p.nb_c * BS, p.heads, hd);
}

template <int BS, int D, typename TA, typename TB, bool RAGGED = false, bool ITEMS = false>
__global__ __launch_bounds__(BS * 2, (D > 64 && BS == 64 && sizeof(TA) == 2 && sizeof(TB) == 2) ? 1 : 2) void dsd_tn_kernel(DsdParams p) {
    constexpr int NO = D / 32;
    constexpr bool kFast = sizeof(TA) == 2 && sizeof(TB) == 2 && BS == 64;
    using TD = Bf16DirectTiles<BS, D>;
    constexpr int TILE = TD::TILE_BYTES;
    constexpr int X_STRIDE = D + 8;   // floats, generic path
    constexpr int LDS_BYTES = kFast ? 4 * TILE : BS * X_STRIDE * 4;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[LDS_BYTES];

    // block-columns (the columns of global tokens are the long ones), or work items
    const DsdLine work = decode_dsd_line<ITEMS>(p);
    if (!work.valid) return;
    const uint32_t b = work.bh / p.heads, h = work.bh % p.heads;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t kn = lane & 31, half = lane >> 5;
    const uint32_t key_in_block = wave * 32 + kn;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const uint32_t row_stride = p.heads * hd;
    const sfb_uint2* lut = p.lut + (size_t)h * p.lut_stride;
    const uint32_t off = work.off, count = work.count;
    float* c_row = dsd_output_row<BS, D, ITEMS>(p, work, b, h, key_in_block, hd);
    const TA* A = (const TA*)p.a + (size_t)work.bh * p.blocks * BS * BS;
    const TB* X = (const TB*)p.b;

    f32x16 acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[n][i] = 0.f;

    if constexpr (kFast) {
        // tiles 0, 1: X row blocks [q][D]; tiles 2, 3: sparse blocks [q][key]; LDS-direct loads, double-buffered
        const uint32_t row_bytes = row_stride * 2;
        // (a short last slice holds other features of its rows in place of the missing ones: they only reach output
        // columns that are not stored)
        const typename TD::Sources x_src = RAGGED ? TD::sources_ragged(lane, row_bytes, hd) : TD::sources(lane, row_bytes);
        const uint32_t a_even = TD::lane_source(lane, 0, BS * 2), a_odd = TD::lane_source(lane, 1, BS * 2);
        const uint32_t lds0 = TD::lds_address(smem);
        const uint32_t x_lane = TD::v_lane_base(lane);
        const uint8_t* const x_base = (const uint8_t*)X + token_offset(b, 0, h, p.nb_b * BS, p.heads, hd) * 2;
        auto fetch = [&](const sfb_uint2 e, uint32_t buf) {
            TD::template load_tile_all<RAGGED>(lds0 + buf * TILE, x_base + (size_t)e.y * BS * row_bytes, wave, x_src, row_bytes);
            TD::load_tile(lds0 + (2 + buf) * TILE, (const uint8_t*)A + (size_t)e.x * BS * BS * 2, wave, a_even, a_odd,
                          BS * 2);
        };
        auto uniform = [](const sfb_uint2 e) -> sfb_uint2 {
            const sfb_uint2 u = {(uint32_t)__builtin_amdgcn_readfirstlane(e.x), (uint32_t)__builtin_amdgcn_readfirstlane(e.y)};
            return u;
        };
        if (count > 0) fetch(uniform(lut[off]), 0);
        for (uint32_t j = 0; j < count; ++j) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            fetch(uniform(lut[off + (j + 1 < count ? j + 1 : j)]), (j + 1) & 1);
            const uint8_t* x_read = smem + (j & 1) * TILE;
            const uint8_t* a_read = smem + (2 + (j & 1)) * TILE;
#pragma unroll
            for (int u = 0; u < BS / 16; ++u) {
                // B-operand: the sparse block [q][key]; this wave's 32 keys are its "column tile" number `wave`
                const bf16x8 bfrag = TD::v_frag(a_read, x_lane, (int)wave, u);
#pragma unroll
                for (int mt = 0; mt < NO; ++mt)
                    acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(TD::v_frag(x_read, x_lane, mt, u), bfrag, acc[mt], 0, 0, 0);
            }
        }
    } else {
        // generic path: fp32 MFMA (k = 2 per step, one element per lane and operand); the X row block is staged
        // in LDS as fp32, the sparse block is read from memory, 32 consecutive keys per half-wave
        // The next block's X tile and this lane's column of the next sparse block wait in registers while the
        // current block is multiplied.
        float* x_lds = (float*)smem;
        constexpr int XV = D / 8;   // float4 of the X tile per thread: BS * D / 4 over BS * 2 threads
        f32x4 xr[XV];
        float a_cur[BS / 2], a_next[BS / 2];
        auto fetch_block = [&](uint32_t j, float (&adst)[BS / 2]) {
            const sfb_uint2 e = lut[off + j];
            const TB* x_blk = X + token_offset(b, e.y * BS, h, p.nb_b * BS, p.heads, hd);
            const TA* a_blk = A + (size_t)e.x * BS * BS;
#pragma unroll
            for (int i = 0; i < XV; ++i) {
                const uint32_t cid = i * BS * 2 + t, row = cid / (D / 4), cc = cid % (D / 4);
                const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
                xr[i] = (!RAGGED || cc * 4 < hd) ? Elem<TB>::load4(x_blk + (size_t)row * row_stride + cc * 4) : zero;
            }
#pragma unroll
            for (int s2 = 0; s2 < BS / 2; ++s2) adst[s2] = Elem<TA>::load(a_blk + (size_t)(2 * s2 + half) * BS + key_in_block);
        };
        if (count > 0) fetch_block(0, a_cur);
        for (uint32_t j = 0; j < count; ++j) {
#pragma unroll
            for (int i = 0; i < XV; ++i) {
                const uint32_t cid = i * BS * 2 + t, row = cid / (D / 4), cc = cid % (D / 4);
                *(f32x4*)(x_lds + row * X_STRIDE + cc * 4) = xr[i];
            }
            __syncthreads();
            if (j + 1 < count) fetch_block(j + 1, a_next);
#pragma unroll
            for (int s2 = 0; s2 < BS / 2; ++s2) {
                const uint32_t q = 2 * s2 + half;
#pragma unroll
                for (int mt = 0; mt < NO; ++mt)
                    acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(x_lds[q * X_STRIDE + mt * 32 + kn], a_cur[s2], acc[mt], 0, 0, 0);
            }
            __syncthreads();
#pragma unroll
            for (int s2 = 0; s2 < BS / 2; ++s2) a_cur[s2] = a_next[s2];
        }
    }
    // accumulator element i of column tile mt is column mt*32 + (i/4)*8 + half*4 + i%4 of this lane's key row;
    // columns without blocks write zeros
#pragma unroll
    for (int mt = 0; mt < NO; ++mt)
#pragma unroll
        for (int ig = 0; ig < 4; ++ig) {
            const f32x4 out = {acc[mt][ig * 4 + 0], acc[mt][ig * 4 + 1], acc[mt][ig * 4 + 2], acc[mt][ig * 4 + 3]};
            // (the rows of a record are D wide; the reduction reads their first hd columns only)
            if (!RAGGED || (ITEMS && work.record) || mt * 32 + ig * 8 + half * 4 < hd) *(f32x4*)(c_row + mt * 32 + ig * 8 + half * 4) = out;
        }
}

// ---------------------------------------------------------------------------------------------
// dsd: one work-group per (batch, head, block-row), V staged through LDS, P read in operand layout
// ---------------------------------------------------------------------------------------------
template <int BS, int D, typename TP, typename TV, bool RAGGED = false, bool ITEMS = false>
__global__ __launch_bounds__(BS * 2, 2) void dsd_nn_kernel(DsdParams p) {
    constexpr int KT = BS / 32, NO = D / 32;
    constexpr bool kBf16 = sizeof(TV) == 2;
    using TD = Bf16DirectTiles<BS, D>;
    using TF = F32Tiles<BS, D>;
    constexpr bool kRing = kBf16 && sizeof(TP) == 2 && BS == 64 && D == 64 && !RAGGED;   // the streaming form below
    constexpr int LDS_BYTES = kBf16 ? (kRing ? 4 : 2) * TD::TILE_BYTES : TF::V_FLOATS * 4;
    __shared__ __attribute__((aligned(1024))) uint8_t smem[LDS_BYTES];

    // block-rows, or work items
    const DsdLine work = decode_dsd_line<ITEMS>(p);
    if (!work.valid) return;
    const uint32_t b = work.bh / p.heads, h = work.bh % p.heads;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t qn = lane & 31, half = lane >> 5;
    const uint32_t q_in_block = wave * 32 + qn;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const uint32_t row_stride = p.heads * hd;
    const sfb_uint2* lut = p.lut + (size_t)h * p.lut_stride;
    const uint32_t off = work.off, count = work.count;
    float* o_row = dsd_output_row<BS, D, ITEMS>(p, work, b, h, q_in_block, hd);
    const TP* P = (const TP*)p.a + (size_t)work.bh * p.blocks * BS * BS;
    const TV* V = (const TV*)p.b;

    f32x16 o_acc[NO];
#pragma unroll
    for (int n = 0; n < NO; ++n)
#pragma unroll
        for (int i = 0; i < 16; ++i) o_acc[n][i] = 0.f;

    if constexpr (kRing) {
        // bf16 P and V.  P is the stream from memory: it is read once, straight into registers in operand layout,
        // kDepth key blocks ahead, so that a work-group keeps several tiles in flight without spending LDS on
        // them (LDS would bound the work-groups per CU, and with them the bytes in flight).  For that a lane's 8
        // k-slots of a product step must be 8 consecutive keys (one 16-byte load): the V tile is laid into LDS
        // with its key rows in the matching order (lane_source_by_halves).  V tiles (L2 hits mostly) go through a
        // ring of four LDS buffers, two blocks per barrier.  Loads complete in issue order, which the counted
        // waits below rely on.
        constexpr int PU = BS / 16, TILE = TD::TILE_BYTES, kDepth = DsdStreamWait::DEPTH;
        static_assert(PU == DsdStreamWait::P_LOADS && TD::LOADS == DsdStreamWait::V_LOADS, "the wait counts what this loop issues");
        const uint32_t row_bytes = row_stride * 2;
        const uint32_t v_even = TD::lane_source_by_halves(lane, 0, row_bytes);
        const uint32_t v_odd = TD::lane_source_by_halves(lane, 1, row_bytes);
        const uint32_t lds0 = TD::lds_address(smem), v_lane = TD::v_lane_base(lane);
        const uint8_t* const v_base = (const uint8_t*)V + token_offset(b, 0, h, p.nb_b * BS, p.heads, D) * 2;
        // step u of this lane: keys 32*half + 8u .. + 7 of query row q_in_block
        const uint32_t p_lane = q_in_block * (BS * 2u) + half * 64u;
        u32x4 pr[kDepth][PU];
        // look-up entries through scalar loads (constant address space): a vector load here would be waited for
        // with vmcnt(0), which drains every tile in flight
        typedef const uint32_t __attribute__((address_space(4)))* const_words;
        const const_words lut_words = (const_words)(uintptr_t)(lut + off);
        // The P loads are written out (scalar base + lane offset) so that every wait in the loop can be stated in
        // loads actually issued: the compiler does not count the LDS-direct loads of the V tiles, and its own
        // waits for P registers would fall short of the depth.  The registers are tied to the wait below.
        auto fetch_p = [&](u32x4 (&dst)[PU], uint32_t j, bool real) {
            static_assert(PU == 4, "four 16-byte loads per lane and block");
            const uint32_t blk = lut_words[2 * j];
            const uint32_t lane_offset = real ? p_lane : 0u;   // a fetch past the row's end: one cache line
            const uint8_t* base = (const uint8_t*)P + (size_t)blk * (BS * BS * 2u);
            // no non-temporal hint: the four loads of a lane share their cache lines with the neighbouring lane's,
            // and with the hint every one of them goes to L2 by itself (measured: 1.5 x the time)
            asm volatile("global_load_dwordx4 %0, %4, %5\n\t"
                         "global_load_dwordx4 %1, %4, %5 offset:16\n\t"
                         "global_load_dwordx4 %2, %4, %5 offset:32\n\t"
                         "global_load_dwordx4 %3, %4, %5 offset:48"
                         : "=&v"(dst[0]), "=&v"(dst[1]), "=&v"(dst[2]), "=&v"(dst[3])
                         : "v"(lane_offset), "s"(base)
                         : "memory");
        };
        auto fetch_v = [&](uint32_t j, uint32_t buf) {
            const uint32_t col = lut_words[2 * j + 1];
            TD::load_tile_by_halves(lds0 + buf * TILE, v_base + (size_t)col * BS * row_bytes, wave, v_even, v_odd,
                                    row_bytes);
        };
        // Issue order: V(0) V(1) P(0) .. P(kDepth-1), then per pair of blocks j, j+1: V(j+2) V(j+3), [products],
        // P(j+kDepth) P(j+kDepth+1).  Every fetch is issued whether or not its block exists (past the row's end
        // the last block is fetched again, a cache hit, into a buffer or registers that nobody reads, and the
        // step multiplies by zeros): the number of loads between a tile and its use is then the same in every
        // step, which is what a counted wait needs -- an exit or a branch inside the unrolled group would leave
        // the compiler with paths on which the counts, or the registers, differ.  V(j+1) is followed by two P
        // tiles (more in the first step), 4 loads per wave each; P(j), P(j+1) were issued before V(j).
        if (count > 0) {
            const uint32_t last = count - 1;
            fetch_v(0, 0);
            fetch_v(1 < count ? 1 : last, 1);
#pragma unroll
            for (int d = 0; d < kDepth; ++d) fetch_p(pr[d], (uint32_t)d < count ? d : last, (uint32_t)d < count);
            for (uint32_t j0 = 0; j0 < count; j0 += kDepth) {
#pragma unroll
                for (int d = 0; d < kDepth; d += 2) {
                    const uint32_t j = j0 + d;
                    asm volatile("s_waitcnt vmcnt(%8)"
                                 : "+v"(pr[d][0]), "+v"(pr[d][1]), "+v"(pr[d][2]), "+v"(pr[d][3]), "+v"(pr[d + 1][0]),
                                   "+v"(pr[d + 1][1]), "+v"(pr[d + 1][2]), "+v"(pr[d + 1][3])
                                 : "n"(DsdStreamWait::COUNT)
                                 : "memory");
                    __syncthreads();   // V(j), V(j+1) are in LDS for every wave; every wave is done with V(j-2), V(j-1)
                    fetch_v(j + 2 < count ? j + 2 : last, (j + 2) % 4u);
                    fetch_v(j + 3 < count ? j + 3 : last, (j + 3) % 4u);
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const uint8_t* v_read = smem + ((j + e) % 4u) * TILE;
                        const uint32_t live = j + e < count ? 0xffffffffu : 0u;
#pragma unroll
                        for (int u = 0; u < PU; ++u) {
                            const u32x4 pv = {pr[d + e][u].x & live, pr[d + e][u].y & live, pr[d + e][u].z & live,
                                              pr[d + e][u].w & live};
                            const bf16x8 bfrag = __builtin_bit_cast(bf16x8, pv);
#pragma unroll
                            for (int mt = 0; mt < NO; ++mt)
                                o_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(TD::v_frag(v_read, v_lane, mt, u),
                                                                                    bfrag, o_acc[mt], 0, 0, 0);
                        }
                    }
                    // the registers of P(j), P(j+1) take the next tiles: not before the products have read them
                    __builtin_amdgcn_sched_barrier(0);
                    fetch_p(pr[d], j + kDepth < count ? j + kDepth : last, j + kDepth < count);
                    fetch_p(pr[d + 1], j + kDepth + 1 < count ? j + kDepth + 1 : last, j + kDepth + 1 < count);
                }
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    } else if constexpr (kBf16) {
        // V tiles double-buffered in LDS by LDS-direct loads, V^T fragments by transposing reads (see
        // Bf16DirectTiles); the P values of the next block are fetched into registers while this one is
        // multiplied.  One barrier per key block.
        constexpr int PU = BS / 16;
        const uint32_t row_bytes = row_stride * 2;
        const typename TD::Sources src = RAGGED ? TD::sources_ragged(lane, row_bytes, hd) : TD::sources(lane, row_bytes);
        const uint32_t lds0 = TD::lds_address(smem), v_lane = TD::v_lane_base(lane);
        const uint8_t* const v_base = (const uint8_t*)V + token_offset(b, 0, h, p.nb_b * BS, p.heads, hd) * 2;
        // slots j of product step u: keys 16u + 8(j/4) + 4*half + j%4
        f32x4 pc[2 * PU], pn[2 * PU];
        auto fetch_p = [&](f32x4 (&dst)[2 * PU], uint32_t blk) {
            const TP* p_row = P + ((size_t)blk * BS + q_in_block) * BS;
#pragma unroll
            for (int u = 0; u < PU; ++u) {
                dst[2 * u] = Elem<TP>::load4(p_row + 16 * u + 4 * half);
                dst[2 * u + 1] = Elem<TP>::load4(p_row + 16 * u + 8 + 4 * half);
            }
        };
        auto fetch_v = [&](uint32_t col, uint32_t buf) {
            TD::template load_tile_all<RAGGED>(lds0 + buf * TD::TILE_BYTES, v_base + (size_t)col * BS * row_bytes, wave, src,
                                               row_bytes);
        };
        if (count > 0) {
            const sfb_uint2 e0 = lut[off];
            fetch_v(__builtin_amdgcn_readfirstlane(e0.y), 0);
            fetch_p(pc, __builtin_amdgcn_readfirstlane(e0.x));
        }
        for (uint32_t j = 0; j < count; ++j) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();   // V(j) is in LDS for every wave, and every wave is done with V(j-1)
            const sfb_uint2 en = lut[off + (j + 1 < count ? j + 1 : j)];
            fetch_v(__builtin_amdgcn_readfirstlane(en.y), (j + 1) & 1);
            fetch_p(pn, __builtin_amdgcn_readfirstlane(en.x));
            const uint8_t* v_read = smem + (j & 1) * TD::TILE_BYTES;
#pragma unroll
            for (int u = 0; u < PU; ++u) {
                const f32x4 lo = pc[2 * u], hi = pc[2 * u + 1];
                const u32x4 pb = {pack_bf16(lo.x, lo.y), pack_bf16(lo.z, lo.w), pack_bf16(hi.x, hi.y),
                                  pack_bf16(hi.z, hi.w)};
                const bf16x8 bfrag = __builtin_bit_cast(bf16x8, pb);
#pragma unroll
                for (int mt = 0; mt < NO; ++mt)
                    o_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(TD::v_frag(v_read, v_lane, mt, u), bfrag,
                                                                        o_acc[mt], 0, 0, 0);
            }
#pragma unroll
            for (int x = 0; x < 2 * PU; ++x) pc[x] = pn[x];
        }
    } else {
        // fp32 V: the tile goes through registers into LDS; the next block's V tile and P values are fetched while
        // this block is multiplied
        float* v_lds = (float*)smem;
        typename TF::Regs gv;
        f32x4 pc[KT][4], pn[KT][4];
        auto fetch_block = [&](uint32_t j, f32x4 (&pdst)[KT][4]) {
            const sfb_uint2 e = lut[off + j];
            if constexpr (RAGGED) TF::fetch_ragged(gv, (const float*)V, token_offset(b, e.y * BS, h, p.nb_b * BS, p.heads, hd), row_stride, t, hd);
            else TF::fetch(gv, (const float*)V, token_offset(b, e.y * BS, h, p.nb_b * BS, p.heads, D), row_stride, t);
            const TP* p_row = P + ((size_t)e.x * BS + q_in_block) * BS;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int ig = 0; ig < 4; ++ig) pdst[kt][ig] = Elem<TP>::load4(p_row + kt * 32 + ig * 8 + half * 4);
        };
        if (count > 0) fetch_block(0, pc);
        for (uint32_t j = 0; j < count; ++j) {
            TF::template stage<TF::V_STRIDE>(v_lds, gv, t);
            __syncthreads();
            if (j + 1 < count) fetch_block(j + 1, pn);
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int ig = 0; ig < 4; ++ig)
#pragma unroll
                    for (int e4 = 0; e4 < 4; ++e4)
#pragma unroll
                        for (int mt = 0; mt < NO; ++mt)
                            o_acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                                TF::v_elem(v_lds, kt, ig * 4 + e4, mt, qn, half), pc[kt][ig][e4], o_acc[mt], 0, 0, 0);
            __syncthreads();
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int ig = 0; ig < 4; ++ig) pc[kt][ig] = pn[kt][ig];
        }
    }
    // block-rows without blocks write zeros (blocksparse.h:949-962)
#pragma unroll
    for (int mt = 0; mt < NO; ++mt)
#pragma unroll
        for (int ig = 0; ig < 4; ++ig) {
            const f32x4 out = {o_acc[mt][ig * 4 + 0], o_acc[mt][ig * 4 + 1], o_acc[mt][ig * 4 + 2],
                               o_acc[mt][ig * 4 + 3]};
            if (!RAGGED || (ITEMS && work.record) || mt * 32 + ig * 8 + half * 4 < hd) *(f32x4*)(o_row + mt * 32 + ig * 8 + half * 4) = out;
        }
}

// Sum of the records of the split lines of a scheduled dsd launch, in chunk order (so the result does not depend on
// which chunk finished when), written to the lines' rows of the result.  grid (n_items, batch * heads): the
// work-groups of the first chunk of a split line do the sums, all others leave at once.  The records are complete when
// this kernel starts: nobody waits for anybody.
__global__ __launch_bounds__(256) void dsd_reduce_kernel(DsdParams p, uint32_t bs, uint32_t dpad) {
    const uint32_t bh = blockIdx.y, b = bh / p.heads, h = bh % p.heads;
    const sfb_work_item it = p.items[(size_t)h * p.item_stride + blockIdx.x];
    if (it.row == SFB_WORK_ITEM_SKIP || it.nchunks <= 1 || it.chunk != 0) return;
    const uint32_t vecs_per_row = dpad / 4, vecs = bs * vecs_per_row;
    for (uint32_t vec = threadIdx.x; vec < vecs; vec += 256) {
        const uint32_t row = vec / vecs_per_row, c4 = vec % vecs_per_row;
        if (c4 * 4 >= p.state) continue;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
        for (uint32_t ch = 0; ch < it.nchunks; ++ch)
            sum += *(const f32x4*)(p.partials + (((size_t)bh * p.n_parts + it.part + ch) * bs + row) * dpad + c4 * 4);
        *(f32x4*)(p.c + token_offset(b, it.row * bs + row, h, p.nb_c * bs, p.heads, p.state) + c4 * 4) = sum;
    }
}

// ---------------------------------------------------------------------------------------------
// sdd + softmax -> P in one kernel, one work-group per block-row, two passes over the row's key
// blocks (statistics, then normalised probabilities).  Replaces fusion_attention1/2, whose
// per-block work-groups exchange row maxima and sums through global flags and spin on them
// (fusion_blocksparse.h:224-366); a work-group that owns the whole block-row needs neither.
// ---------------------------------------------------------------------------------------------
struct SddSoftmaxParams {
    const sfb_uint2* nn_lut;
    const void* a;
    const void* b;
    void* y;
    const void* mask;        // block-major words
    const int32_t* valid_len;
    const uint32_t* row_order;   // rank -> block-row, or nullptr
    uint32_t blocks, batch, heads, nb, lut_stride, mask_stride, groups;
    float scale_log2e;
    uint32_t state;              // head size of the tensors
};

// bf16 operands, 64 x 64 blocks, 64 features: the work-group of a block-row (two waves, 32 queries each, the
// query fragments in registers) walks the row's key blocks twice -- statistics, then probabilities; the scores are
// recomputed rather than kept -- with the K tiles coming through a ring of three LDS buffers two blocks ahead
// (LDS-direct loads of whole lines; K is read from L2 the second time) and P leaving through the waves' LDS slabs
// as whole rows.  Every wait is counted in the loads and stores actually issued (they complete in issue order): in
// the second pass K(j) is followed by the stores of blocks j-2 and j-1 and the loads of K(j+1).
template <typename TOut>
__global__ __launch_bounds__(128) void sdd_softmax_stream_kernel(SddSoftmaxParams p) {
    constexpr int BS = 64, D = 64, KT = BS / 32, KS = D / 16;
    using TD = Bf16DirectTiles<BS, D>;
    using Slab = RowSlab<BS, TOut>;
    constexpr int TILE = TD::TILE_BYTES;
    typedef const uint32_t __attribute__((address_space(4)))* const_words;
    __shared__ __attribute__((aligned(1024))) uint8_t tiles[3 * TILE];
    __shared__ __attribute__((aligned(16))) uint8_t slabs[BS / 32][Slab::BYTES];
    // the two longest block-rows of every (batch, head) before anything else (with row_order: its first two; else
    // the last and the first row, where causal layouts and layouts with global tokens have them)
    const WorkId work = decode_work(blockIdx.x, p.batch * p.heads, p.nb, p.nb >= 2 ? 2 : 0);
    if (!work.valid) return;
    const uint32_t b = work.bh / p.heads, h = work.bh % p.heads;
    const uint32_t r = p.row_order ? p.row_order[work.rank]
                                   : ((work.rank & 1u) ? work.rank / 2 : p.nb - 1 - work.rank / 2);
    const uint32_t t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t qn = lane & 31, half = lane >> 5, q_in_block = wave * 32 + qn;
    const uint32_t L = p.nb * BS, row_bytes = p.heads * D * 2;
    const const_words head = (const_words)(uintptr_t)(p.nn_lut + (size_t)h * p.lut_stride);
    const uint32_t off = head[2 * r], count = head[2 * r + 1];
    if (count == 0) return;
    const uint32_t last = count - 1;
    const const_words lut_words = head + 2 * (size_t)off;
    const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
    const int valid = p.valid_len ? p.valid_len[b] : (int)L;
    const float c = p.scale_log2e;
    TOut* Y = (TOut*)p.y + (size_t)work.bh * p.blocks * BS * BS;
    const uint8_t* const k_base = (const uint8_t*)p.b + token_offset(b, 0, h, L, p.heads, D) * 2;
    const uint32_t src_even = TD::lane_source(lane, 0, row_bytes), src_odd = TD::lane_source(lane, 1, row_bytes);
    const uint32_t lds0 = TD::lds_address(tiles), k_lane = TD::k_lane_base(qn, half);
    auto fetch_k = [&](uint32_t j, uint32_t buf) {
        const uint32_t col = lut_words[2 * j + 1];
        TD::load_tile(lds0 + buf * TILE, k_base + (size_t)col * BS * row_bytes, wave, src_even, src_odd, row_bytes);
    };
    bf16x8 qf[KS];
    TD::load_q(qf, (const __bf16*)p.a + token_offset(b, r * BS + q_in_block, h, L, p.heads, D), half);
    // a use here, so that the fragments are waited for before the loop: inside it the compiler would wait for them
    // at their first use in every step, with a count that ignores the LDS-direct loads, and drain the tiles in flight
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(qf[ks]));
    float m = kMaxSeed, l = 0.f;   // exact running maximum and the sum relative to it (this lane's keys)
    float inv = 0.f;
    for (int pass = 0; pass < 2; ++pass) {
        if (pass == 1) {
            inv = 1.0f / (l + __shfl_xor(l, 32) + 1e-6f);
            __syncthreads();   // every wave is done with the tiles of the first pass
        }
        // a fetch past the row's end repeats the last block: the counts stay the same in every step
        fetch_k(0, 0);
        fetch_k(1 < count ? 1 : last, 1);
        for (uint32_t j = 0; j < count; ++j) {
            // K(j) has landed once only what was issued after it is outstanding: K(j+1), and in the second pass
            // the stores of blocks j-2 and j-1 (4 or 8 per wave each) -- for j < 2 fewer, so the stricter count
            static_assert(Slab::PASSES == SddStreamWait<sizeof(TOut)>::PASSES && TD::LOADS == SddStreamWait<sizeof(TOut)>::LOADS,
                          "the wait counts what this loop issues");
            if (pass == 0 || j < 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SddStreamWait<sizeof(TOut)>::LOADS) : "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(SddStreamWait<sizeof(TOut)>::COUNT) : "memory");
            __syncthreads();   // K(j) is in LDS for every wave, and every wave is done with K(j-1)
            fetch_k(j + 2 < count ? j + 2 : last, (j + 2) % 3u);
            const uint8_t* k_read = tiles + (j % 3u) * TILE;
            const uint32_t blk = lut_words[2 * j], col = lut_words[2 * j + 1];
            f32x16 s[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int i = 0; i < 16; ++i) s[kt][i] = 0.f;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
                    s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(TD::k_frag(k_read, k_lane, kt, ks), qf[ks], s[kt], 0, 0, 0);
            const int limit = valid - (int)(col * BS);
            if ((mask != nullptr) || (limit < BS))
                apply_keep<KT>(s, load_keep_word<BS>(mask, (size_t)blk * BS + q_in_block, limit), half);
            if (pass == 0) {
                const float m_new = fmaxf(m, block_row_max<KT>(s));
                l *= exp2_fast((m - m_new) * c);
                m = m_new;
                const float mc = m * c;
                float l0 = 0.f, l1 = 0.f;
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int i = 0; i < 16; i += 2) {
                        l0 += exp2_fast(__builtin_fmaf(s[kt][i], c, -mc));
                        l1 += exp2_fast(__builtin_fmaf(s[kt][i + 1], c, -mc));
                    }
                l += l0 + l1;
            } else {
                const float mc = m * c;
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) s[kt][i] = exp2_fast(__builtin_fmaf(s[kt][i], c, -mc)) * inv;
                Slab::store(Y + ((size_t)blk * BS + wave * 32) * BS, s, slabs[wave], lane);
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing in flight towards LDS when the group ends
}

// Waves of a work-group: BS/32 query halves x kSddSoftmaxKeyGroups key groups.  Key group g takes the row's blocks
// g, g + 2, ...; the groups meet once, through LDS, to agree on the row maximum and sum.  A long block-row thus
// has two independent streams of tile loads in flight per query half instead of one (four measured the same on
// rows of 64 blocks and slower on rows of 11, where the larger work-group leaves fewer of them per CU).
constexpr int kSddSoftmaxKeyGroups = 2;

template <int BS, int D, typename TIn, typename TOut, bool RAGGED = false>
__global__ __launch_bounds__(BS * 2 * kSddSoftmaxKeyGroups) void sdd_softmax_kernel(SddSoftmaxParams p) {
    constexpr int KT = BS / 32, QW = BS / 32, KG = kSddSoftmaxKeyGroups;
    __shared__ float stats[KG][BS][2];
    __shared__ __attribute__((aligned(16))) uint8_t slabs[QW * KG][RowSlab<BS, TOut>::BYTES];
    const WorkId work = decode_work(blockIdx.x, p.batch * p.heads, p.nb);
    if (!work.valid) return;
    const uint32_t b = work.bh / p.heads, h = work.bh % p.heads;
    const uint32_t r = p.row_order ? p.row_order[work.rank] : p.nb - 1 - work.rank;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6, qn = lane & 31, half = lane >> 5;
    const uint32_t group = wave / QW;
    const uint32_t q_in_block = (wave % QW) * 32 + qn;
    const uint32_t hd = RAGGED ? p.state : (uint32_t)D;
    const uint32_t L = p.nb * BS, row_stride = p.heads * hd;
    const sfb_uint2* lut = p.nn_lut + (size_t)h * p.lut_stride;
    const uint32_t off = lut[r].x, count = lut[r].y;
    const TIn* q_row = (const TIn*)p.a + token_offset(b, r * BS + q_in_block, h, L, p.heads, hd);
    const TIn* K = (const TIn*)p.b;
    const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
    const int valid = p.valid_len ? p.valid_len[b] : (int)L;
    const float c = p.scale_log2e;
    TOut* Y = (TOut*)p.y + (size_t)work.bh * p.blocks * BS * BS;

    QRow<D, TIn> q_ops;
    q_ops.template load<RAGGED>(q_row, half, hd);
    float m = kMaxSeed, l = 0.f;   // exact running maximum and the sum relative to it (this lane's keys)
    for (int pass = 0; pass < 2; ++pass) {
        float inv = 0.f;
        if (pass == 1) {
            // this group's statistics (both lanes of a query hold the same maximum; their sums add up), then
            // the row's: maximum over the groups, sums rescaled to it
            const float mine = l + __shfl_xor(l, 32);
            if (half == 0) {
                stats[group][q_in_block][0] = m;
                stats[group][q_in_block][1] = mine;
            }
            __syncthreads();
            float m_row = kMaxSeed;
#pragma unroll
            for (int g = 0; g < KG; ++g) m_row = fmaxf(m_row, stats[g][q_in_block][0]);
            float total = 0.f;
#pragma unroll
            for (int g = 0; g < KG; ++g)
                total += stats[g][q_in_block][1] * exp2_fast((stats[g][q_in_block][0] - m_row) * c);
            m = m_row;
            inv = 1.0f / (total + 1e-6f);
        }
        // the K tile of this group's next block is fetched while the current one is multiplied
        KTile<BS, D, TIn> k_cur, k_next;
        sfb_uint2 e = group < count ? lut[off + group] : sfb_uint2{0u, 0u};
        if (group < count) k_cur.template load<RAGGED>(K + token_offset(b, e.y * BS, h, L, p.heads, hd), row_stride, qn, half, hd);
        for (uint32_t j = group; j < count; j += KG) {
            const sfb_uint2 e_next = lut[off + (j + KG < count ? j + KG : j)];
            k_next.template load<RAGGED>(K + token_offset(b, e_next.y * BS, h, L, p.heads, hd), row_stride, qn, half, hd);
            f32x16 s[KT];
            score_tile<BS, D, TIn>(s, k_cur, q_ops);
            const int limit = valid - (int)(e.y * BS);
            const bool masked = (mask != nullptr) || (limit < BS);
            if (masked) apply_keep<KT>(s, load_keep_word<BS>(mask, (size_t)e.x * BS + q_in_block, limit), half);
            const uint32_t blk = e.x;
            e = e_next;
            k_cur = k_next;
            if (pass == 0) {
                const float m_new = fmaxf(m, block_row_max<KT>(s));
                l *= exp2_fast((m - m_new) * c);
                m = m_new;
                const float mc = m * c;
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) l += exp2_fast(__builtin_fmaf(s[kt][i], c, -mc));
            } else {
                const float mc = m * c;
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int i = 0; i < 16; ++i) s[kt][i] = exp2_fast(__builtin_fmaf(s[kt][i], c, -mc)) * inv;
                RowSlab<BS, TOut>::store(Y + ((size_t)blk * BS + (wave % QW) * 32) * BS, s, slabs[wave], lane);
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// sdd + softmax -> P with ONE WORK-GROUP PER BLOCK, the decomposition of the reference's fusion_nt_softmax2
// (fusion_blocksparse.h:458-833): every work-group computes its block's scores, publishes the row maxima of
// the block, counts itself in on the block-row's flag and spins until all blocks of the row have done so;
// takes the row maximum over the published values, publishes its partial row sums, spins on a second flag, and
// normalises.  Kept as the comparison for sdd_softmax_kernel above, which needs none of this because one
// work-group owns the whole block-row.  The spins are bounded: a work-group that runs out of its budget sets
// *status and leaves without writing its block (the scheme only makes progress while every work-group of a
// block-row is resident or can become resident, which a launch cannot guarantee).
// ---------------------------------------------------------------------------------------------
struct SplitSoftmaxParams {
    const sfb_uint2* nt_lut;
    const sfb_uint2* nn_lut;
    const void* a;
    const void* b;
    void* y;
    const void* mask;         // block-major words
    const int32_t* valid_len;
    float* row_max;           // [batch][heads][blocks][BS]
    float* row_sum;           // [batch][heads][blocks][BS]
    uint32_t* flags;          // [batch][heads][nb][2], zero at launch
    uint32_t* status;         // set to 1 by a work-group whose spin budget ran out
    uint32_t blocks, heads, nb, nt_stride, nn_stride, mask_stride, spin_limit;
    float scale_log2e;
};

// Thread 0 waits until *flag reaches `want`; every thread learns whether it did.
__device__ __forceinline__ bool wait_for_row(uint32_t* flag, uint32_t want, uint32_t spin_limit, uint32_t t) {
    __shared__ uint32_t arrived;
    if (t == 0) {
        uint32_t seen = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (uint32_t spin = 0; seen < want && spin < spin_limit; ++spin) {
            __builtin_amdgcn_s_sleep(4);
            seen = __hip_atomic_load(flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        arrived = seen >= want ? 1u : 0u;
    }
    __syncthreads();
    const bool ok = arrived != 0;
    __syncthreads();   // `arrived` is reused by the second wait
    return ok;
}

template <int BS, int D, typename TIn, typename TOut>
__global__ __launch_bounds__(BS * 2) void sdd_softmax_split_kernel(SplitSoftmaxParams p) {
    constexpr int KT = BS / 32;
    const uint32_t blk = blockIdx.x, b = blockIdx.y, h = blockIdx.z;
    const uint32_t t = threadIdx.x, lane = t & 63, wave = t >> 6, qn = lane & 31, half = lane >> 5;
    const uint32_t q_in_block = wave * 32 + qn;
    const uint32_t bh = b * p.heads + h;
    const sfb_uint2 e = p.nt_lut[(size_t)h * p.nt_stride + blk];   // {row block, col block}
    const sfb_uint2* nn = p.nn_lut + (size_t)h * p.nn_stride;
    const uint32_t off = nn[e.x].x, count = nn[e.x].y;
    const uint32_t L = p.nb * BS, row_stride = p.heads * D;
    const float c = p.scale_log2e;

    f32x16 s[KT];
    const TIn* q_row = (const TIn*)p.a + token_offset(b, e.x * BS + q_in_block, h, L, p.heads, D);
    score_tile_direct<BS, D, TIn>(s, q_row, (const TIn*)p.b + token_offset(b, e.y * BS, h, L, p.heads, D), row_stride,
                                  qn, half);
    const uint8_t* mask = p.mask ? (const uint8_t*)p.mask + (size_t)h * p.mask_stride * (BS / 8) : nullptr;
    const int valid = p.valid_len ? p.valid_len[b] : (int)L;
    const int limit = valid - (int)(e.y * BS);
    if (mask != nullptr || limit < BS)
        apply_keep<KT>(s, load_keep_word<BS>(mask, (size_t)blk * BS + q_in_block, limit), half);

    // phase 1: the block's row maxima (seeded as ewops.h:70), then the block-row's first flag
    const size_t head_rows = (size_t)bh * p.blocks * BS;
    const float m_blk = fmaxf(kMaxSeed, block_row_max<KT>(s));
    if (half == 0) __hip_atomic_store(p.row_max + head_rows + (size_t)blk * BS + q_in_block, m_blk, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
    __syncthreads();
    uint32_t* flags = p.flags + ((size_t)bh * p.nb + e.x) * 2;
    if (t == 0) __hip_atomic_fetch_add(flags, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (!wait_for_row(flags, count, p.spin_limit, t)) {
        if (t == 0) __hip_atomic_store(p.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    float m = kMaxSeed;
    for (uint32_t j = 0; j < count; ++j)
        m = fmaxf(m, coherent_load_f32(p.row_max + head_rows + (size_t)nn[off + j].x * BS + q_in_block));

    // phase 2: partial row sums relative to the row maximum, second flag
    const float mc = m * c;
    float l = 0.f;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            s[kt][i] = exp2_fast(__builtin_fmaf(s[kt][i], c, -mc));
            l += s[kt][i];
        }
    l += __shfl_xor(l, 32);
    if (half == 0) __hip_atomic_store(p.row_sum + head_rows + (size_t)blk * BS + q_in_block, l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
    __syncthreads();
    if (t == 0) __hip_atomic_fetch_add(flags + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (!wait_for_row(flags + 1, count, p.spin_limit, t)) {
        if (t == 0) __hip_atomic_store(p.status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }
    float total = 0.f;
    for (uint32_t j = 0; j < count; ++j)
        total += coherent_load_f32(p.row_sum + head_rows + (size_t)nn[off + j].x * BS + q_in_block);
    const float inv = 1.0f / (total + 1e-6f);
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[kt][i] *= inv;
    __shared__ __attribute__((aligned(16))) uint8_t slabs[BS / 32][RowSlab<BS, TOut>::BYTES];
    TOut* Y = (TOut*)p.y + (size_t)bh * p.blocks * BS * BS;
    RowSlab<BS, TOut>::store(Y + ((size_t)blk * BS + wave * 32) * BS, s, slabs[wave], lane);
}

__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t* words, uint32_t n) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) words[i] = 0u;
}

static int check_dtype(int d) { return (d == SFB_F32 || d == SFB_BF16) ? SFB_OK : SFB_ERR_DTYPE; }

}  // namespace sfb

using namespace sfb;

// Head sizes: every multiple of the 16-byte vector (4 floats, 8 bf16) up to 128, with every type combination (the
// reference's K64 = false paths take d % 4 == 0, openai_blocksparse.h:221-222).  32, 64, 96 and 128 are what the
// MFMA tiles divide; the sizes between run the kernel of the next multiple of 32 with its RAGGED form of loads and
// stores.
static int check_head_state(uint32_t state_dim, int dense_dtype) {
    const uint32_t vec = dense_dtype == SFB_BF16 ? 8u : 4u;
    return state_dim >= vec && state_dim <= 128 && state_dim % vec == 0 ? SFB_OK : SFB_ERR_HEAD_STATE;
}
static uint32_t padded_head_state(uint32_t state_dim) { return (state_dim + 31u) / 32u * 32u; }
// CALL(D, TD, TS) for a head size other than 64: TD = the dense tensors' type, TS = the sparse tensor's
#define SFB_DISPATCH_D(DV, TDN, TS, CALL)                                            \
    do {                                                                             \
        if ((TDN) == SFB_F32) {                                                      \
            if ((TS) == SFB_F32) { CALL(DV, float, float); } else { CALL(DV, float, __bf16); }   \
        } else {                                                                     \
            if ((TS) == SFB_F32) { CALL(DV, __bf16, float); } else { CALL(DV, __bf16, __bf16); } \
        }                                                                            \
    } while (0)
#define SFB_DISPATCH_OTHER_D(STATE, TDN, TS, CALL)                         \
    do {                                                                  \
        if ((STATE) == 32) SFB_DISPATCH_D(32, TDN, TS, CALL);              \
        else if ((STATE) == 96) SFB_DISPATCH_D(96, TDN, TS, CALL);         \
        else SFB_DISPATCH_D(128, TDN, TS, CALL);                           \
    } while (0)

#define SFB_DISPATCH_PADDED_D(PAD, TDN, TS, CALL)                          \
    do {                                                                  \
        if ((PAD) == 64) SFB_DISPATCH_D(64, TDN, TS, CALL);                \
        else SFB_DISPATCH_OTHER_D(PAD, TDN, TS, CALL);                     \
    } while (0)

#define SFB_DISPATCH_2(BSV, T0, T1, CALL)                                                  \
    do {                                                                                   \
        if ((T0) == SFB_F32 && (T1) == SFB_F32) { CALL(BSV, float, float); }               \
        else if ((T0) == SFB_F32 && (T1) == SFB_BF16) { CALL(BSV, float, __bf16); }        \
        else if ((T0) == SFB_BF16 && (T1) == SFB_F32) { CALL(BSV, __bf16, float); }        \
        else { CALL(BSV, __bf16, __bf16); }                                                \
    } while (0)

extern "C" int sfb_sdd_nt(sfb_stream_t stream, const sfb_uint2* lut, const void* a, const void* b, void* c,
                          int in_dtype, int out_dtype, uint32_t block_size, uint32_t blocks,
                          uint32_t batch_dim, uint32_t ctx_blks_a, uint32_t ctx_blks_b, uint32_t head_dim,
                          uint32_t state_dim, uint32_t lut_heads, uint32_t lut_dim) {
    if (!lut || !a || !b || !c) return SFB_ERR_NULL_POINTER;
    if (check_dtype(in_dtype) || check_dtype(out_dtype)) return SFB_ERR_DTYPE;
    if (block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (check_head_state(state_dim, in_dtype)) return SFB_ERR_HEAD_STATE;
    if (!blocks || !batch_dim || !head_dim || !ctx_blks_a || !ctx_blks_b || !lut_heads) return SFB_ERR_SHAPE;
    if (lut_heads > 1 && lut_heads != head_dim) return SFB_ERR_SHAPE;
    if (batch_dim > 65535 || head_dim > 65535) return SFB_ERR_SHAPE;
    if (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15u) return SFB_ERR_ALIGNMENT;
    SddParams p = {lut, a, b, c, blocks, head_dim, ctx_blks_a * block_size, ctx_blks_b * block_size,
                   lut_heads > 1 ? lut_dim : 0, batch_dim, 0, state_dim};
    const dim3 grid((blocks + kSddGroup - 1) / kSddGroup, batch_dim, head_dim);
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
    if (state_dim % 32 != 0) {
#define SFB_CALL64(DV, TI, TO) sdd_nt_kernel<64, DV, TI, TO, true><<<grid, dim3(128), 0, s>>>(p)
#define SFB_CALL32(DV, TI, TO) sdd_nt_kernel<32, DV, TI, TO, true><<<grid, dim3(64), 0, s>>>(p)
        if (block_size == 64) SFB_DISPATCH_PADDED_D(padded_head_state(state_dim), in_dtype, out_dtype, SFB_CALL64);
        else SFB_DISPATCH_PADDED_D(padded_head_state(state_dim), in_dtype, out_dtype, SFB_CALL32);
#undef SFB_CALL64
#undef SFB_CALL32
        return launch_status();
    }
    if (state_dim != 64) {
#define SFB_CALL64(DV, TI, TO) sdd_nt_kernel<64, DV, TI, TO><<<grid, dim3(128), 0, s>>>(p)
#define SFB_CALL32(DV, TI, TO) sdd_nt_kernel<32, DV, TI, TO><<<grid, dim3(64), 0, s>>>(p)
        if (block_size == 64) SFB_DISPATCH_OTHER_D(state_dim, in_dtype, out_dtype, SFB_CALL64);
        else SFB_DISPATCH_OTHER_D(state_dim, in_dtype, out_dtype, SFB_CALL32);
#undef SFB_CALL64
#undef SFB_CALL32
        return launch_status();
    }
    if (block_size == 64 && in_dtype == SFB_BF16) {
        const uint32_t num_bh = batch_dim * head_dim;
        p.by_xcd = num_bh % 8 == 0 || num_bh >= 32;
        const uint64_t wgs = (uint64_t)((blocks + kSddStreamGroup - 1) / kSddStreamGroup) *
                             (p.by_xcd ? bh_groups(num_bh) * 8 : num_bh);
        if (wgs > 0x7fffffffull) return SFB_ERR_SHAPE;
        const dim3 stream_grid((uint32_t)wgs);
        if (out_dtype == SFB_BF16) sdd_nt_stream_kernel<__bf16><<<stream_grid, dim3(128), 0, s>>>(p);
        else sdd_nt_stream_kernel<float><<<stream_grid, dim3(128), 0, s>>>(p);
        return launch_status();
    }
#define SFB_CALL(BSV, TI, TO) sdd_nt_kernel<BSV, 64, TI, TO><<<grid, dim3(BSV * 2), 0, s>>>(p)
    if (block_size == 64) SFB_DISPATCH_2(64, in_dtype, out_dtype, SFB_CALL);
    else SFB_DISPATCH_2(32, in_dtype, out_dtype, SFB_CALL);
#undef SFB_CALL
    return launch_status();
}

extern "C" int sfb_masked_softmax(sfb_stream_t stream, const sfb_uint2* lut, const void* mask, const void* x,
                                  void* y, int x_dtype, int y_dtype, const int32_t* valid_len,
                                  uint32_t block_size, uint32_t blocks, uint32_t batch_dim, uint32_t head_dim,
                                  uint32_t ctx_blks, uint32_t lut_heads, uint32_t lut_dim, uint32_t max_lut,
                                  uint32_t mask_heads, float scale) {
    (void)max_lut;  // sizes the reference's shared memory (blocksparse.h:671-686); not needed here
    if (!lut || !x || !y) return SFB_ERR_NULL_POINTER;
    if (check_dtype(x_dtype) || check_dtype(y_dtype)) return SFB_ERR_DTYPE;
    if (block_size != 8 && block_size != 16 && block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (!blocks || !batch_dim || !head_dim || !ctx_blks || !lut_heads || !mask_heads) return SFB_ERR_SHAPE;
    if (lut_heads > 1 && (lut_heads != head_dim || lut_dim != ctx_blks + blocks)) return SFB_ERR_SHAPE;
    if (mask_heads > 1 && mask_heads != head_dim) return SFB_ERR_SHAPE;
    if (!(scale > 0.f) || !(scale < 3.0e38f)) return SFB_ERR_ARGUMENT;
    if (((uintptr_t)x | (uintptr_t)y) & 15u) return SFB_ERR_ALIGNMENT;
    SoftmaxParams p = {lut, mask, valid_len, x, y, blocks, batch_dim, head_dim, ctx_blks,
                       lut_heads > 1 ? lut_dim : 0, mask_heads > 1 ? blocks * block_size : 0, scale * kLog2e};
    const uint64_t groups = softmax_grid(batch_dim, head_dim, ctx_blks, block_size);
    if (groups > 0x7fffffffull) return SFB_ERR_SHAPE;
    const dim3 grid((uint32_t)groups);
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
    if (block_size == 64 && x_dtype == SFB_BF16) {
        const uint64_t units = (uint64_t)batch_dim * head_dim * ctx_blks * 2;   // 32 rows each
        if (units > 0x7fffffffull) return SFB_ERR_SHAPE;
        if (y_dtype == SFB_BF16) masked_softmax_rows8_kernel<__bf16><<<dim3((uint32_t)units), dim3(256), 0, s>>>(p);
        else masked_softmax_rows8_kernel<float><<<dim3((uint32_t)units), dim3(256), 0, s>>>(p);
        return launch_status();
    }
#define SFB_CALL(BSV, TX, TY) masked_softmax_kernel<BSV, TX, TY><<<grid, dim3(256), 0, s>>>(p)
    if (block_size == 64) SFB_DISPATCH_2(64, x_dtype, y_dtype, SFB_CALL);
    else if (block_size == 32) SFB_DISPATCH_2(32, x_dtype, y_dtype, SFB_CALL);
    else if (block_size == 16) SFB_DISPATCH_2(16, x_dtype, y_dtype, SFB_CALL);
    else SFB_DISPATCH_2(8, x_dtype, y_dtype, SFB_CALL);
#undef SFB_CALL
    return launch_status();
}

extern "C" size_t sfb_dsd_workspace_bytes(uint32_t n_parts, uint32_t batch_dim, uint32_t head_dim, uint32_t block_size,
                                          uint32_t state_dim) {
    // records of the kernels' D floats a row
    return (size_t)batch_dim * head_dim * n_parts * block_size * padded_head_state(state_dim) * sizeof(float);
}

// One launch of a dsd kernel: a work-group per line (items null) or per work item.
static int dsd_launch(hipStream_t s, const DsdParams& p, int a_dtype, int b_dtype, uint32_t block_size, uint32_t state_dim,
                      uint32_t op);

static int dsd_xn(sfb_stream_t stream, const sfb_uint2* lut, const void* a, const void* b, float* c, int a_dtype,
                  int b_dtype, const sfb_work_item* items, uint32_t n_items, uint32_t n_heavy, uint32_t n_parts,
                  void* workspace, size_t workspace_bytes, uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                  uint32_t ctx_blks_b, uint32_t ctx_blks_c, uint32_t head_dim, uint32_t state_dim, uint32_t lut_heads,
                  uint32_t lut_dim, uint32_t op) {
    if (!lut || !a || !b || !c) return SFB_ERR_NULL_POINTER;
    if (check_dtype(a_dtype) || check_dtype(b_dtype)) return SFB_ERR_DTYPE;
    if (op != SFB_NN_OP && op != SFB_TN_OP) return SFB_ERR_ARGUMENT;
    if (block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (check_head_state(state_dim, b_dtype)) return SFB_ERR_HEAD_STATE;
    if (!blocks || !batch_dim || !head_dim || !ctx_blks_b || !ctx_blks_c || !lut_heads) return SFB_ERR_SHAPE;
    if (lut_heads > 1 && (lut_heads != head_dim || lut_dim != ctx_blks_c + blocks)) return SFB_ERR_SHAPE;
    if (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15u) return SFB_ERR_ALIGNMENT;
    DsdParams p = {lut, a, b, c, blocks, batch_dim, head_dim, ctx_blks_b, ctx_blks_c,
                   lut_heads > 1 ? lut_dim : 0, bh_groups(batch_dim * head_dim), state_dim};
    if (items) {
        if (a_dtype != b_dtype) return SFB_ERR_DTYPE;
        if (n_items == 0 || n_heavy >= n_items) return SFB_ERR_SHAPE;
        if ((uint64_t)p.groups * 8u * n_items > 0x7fffffffull || (uint64_t)batch_dim * head_dim > 65535u) return SFB_ERR_SHAPE;
        const size_t need = sfb_dsd_workspace_bytes(n_parts, batch_dim, head_dim, block_size, state_dim);
        if (need && (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255u))) return SFB_ERR_WORKSPACE;
        p.items = items;
        p.item_stride = lut_heads > 1 ? n_items : 0;
        p.ranks = n_items; p.heavy = n_heavy; p.n_parts = n_parts;
        p.partials = (float*)workspace;
    }
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
    const int rc = dsd_launch(s, p, a_dtype, b_dtype, block_size, state_dim, op);
    if (rc != SFB_OK || !items || !n_parts) return rc;
    dsd_reduce_kernel<<<dim3(n_items, batch_dim * head_dim), dim3(256), 0, s>>>(p, block_size, padded_head_state(state_dim));
    return launch_status();
}

extern "C" int sfb_dsd_xn(sfb_stream_t stream, const sfb_uint2* lut, const void* a, const void* b, float* c,
                          int a_dtype, int b_dtype, uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                          uint32_t ctx_blks_b, uint32_t ctx_blks_c, uint32_t head_dim, uint32_t state_dim,
                          uint32_t lut_heads, uint32_t lut_dim, uint32_t op, uint32_t magic, uint32_t shift,
                          uint32_t max_lut) {
    (void)magic; (void)shift; (void)max_lut;  // grid decomposition / smem sizing of the reference kernel
    return dsd_xn(stream, lut, a, b, c, a_dtype, b_dtype, nullptr, 0, 0, 0, nullptr, 0, block_size, blocks, batch_dim,
                  ctx_blks_b, ctx_blks_c, head_dim, state_dim, lut_heads, lut_dim, op);
}

extern "C" int sfb_dsd_xn_scheduled(sfb_stream_t stream, const sfb_uint2* lut, const void* a, const void* b, float* c,
                                    int a_dtype, int b_dtype, const sfb_work_item* items, uint32_t n_items,
                                    uint32_t n_heavy, uint32_t n_parts, void* workspace, size_t workspace_bytes,
                                    uint32_t block_size, uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks_b,
                                    uint32_t ctx_blks_c, uint32_t head_dim, uint32_t state_dim, uint32_t lut_heads,
                                    uint32_t lut_dim, uint32_t op) {
    if (!items) return SFB_ERR_NULL_POINTER;
    return dsd_xn(stream, lut, a, b, c, a_dtype, b_dtype, items, n_items, n_heavy, n_parts, workspace, workspace_bytes,
                  block_size, blocks, batch_dim, ctx_blks_b, ctx_blks_c, head_dim, state_dim, lut_heads, lut_dim, op);
}

static int dsd_launch(hipStream_t s, const DsdParams& p, int a_dtype, int b_dtype, uint32_t block_size, uint32_t state_dim,
                      uint32_t op) {
    const dim3 grid(p.groups * 8u * (p.items ? p.ranks : p.nb_c));
    if (p.items) {
        // work items: both operands of one type; the streaming kernels of bf16 operands with 64 x 64 blocks and 64
        // features, otherwise the forms that take any head size
        if (block_size == 64 && state_dim == 64 && b_dtype == SFB_BF16) {
            if (op == SFB_TN_OP) dsd_tn_kernel<64, 64, __bf16, __bf16, false, true><<<grid, dim3(128), 0, s>>>(p);
            else dsd_nn_kernel<64, 64, __bf16, __bf16, false, true><<<grid, dim3(128), 0, s>>>(p);
            return launch_status();
        }
        const uint32_t pad = padded_head_state(state_dim);
#define SFB_ITEMS(BSV, DV)                                                                                            \
    do {                                                                                                              \
        if (op == SFB_TN_OP) {                                                                                        \
            if (b_dtype == SFB_BF16) dsd_tn_kernel<BSV, DV, __bf16, __bf16, true, true><<<grid, dim3(BSV * 2), 0, s>>>(p); \
            else dsd_tn_kernel<BSV, DV, float, float, true, true><<<grid, dim3(BSV * 2), 0, s>>>(p);                  \
        } else {                                                                                                      \
            if (b_dtype == SFB_BF16) dsd_nn_kernel<BSV, DV, __bf16, __bf16, true, true><<<grid, dim3(BSV * 2), 0, s>>>(p); \
            else dsd_nn_kernel<BSV, DV, float, float, true, true><<<grid, dim3(BSV * 2), 0, s>>>(p);                  \
        }                                                                                                             \
    } while (0)
        if (block_size == 64) {
            if (pad == 32) SFB_ITEMS(64, 32); else if (pad == 64) SFB_ITEMS(64, 64); else if (pad == 96) SFB_ITEMS(64, 96); else SFB_ITEMS(64, 128);
        } else {
            if (pad == 32) SFB_ITEMS(32, 32); else if (pad == 64) SFB_ITEMS(32, 64); else if (pad == 96) SFB_ITEMS(32, 96); else SFB_ITEMS(32, 128);
        }
#undef SFB_ITEMS
        return launch_status();
    }
    if (state_dim % 32 != 0) {
        const uint32_t pad = padded_head_state(state_dim);
#define SFB_TN64(DV, TB, TA) dsd_tn_kernel<64, DV, TA, TB, true><<<grid, dim3(128), 0, s>>>(p)
#define SFB_TN32(DV, TB, TA) dsd_tn_kernel<32, DV, TA, TB, true><<<grid, dim3(64), 0, s>>>(p)
#define SFB_NN64(DV, TB, TA) dsd_nn_kernel<64, DV, TA, TB, true><<<grid, dim3(128), 0, s>>>(p)
#define SFB_NN32(DV, TB, TA) dsd_nn_kernel<32, DV, TA, TB, true><<<grid, dim3(64), 0, s>>>(p)
        if (op == SFB_TN_OP) {
            if (block_size == 64) SFB_DISPATCH_PADDED_D(pad, b_dtype, a_dtype, SFB_TN64);
            else SFB_DISPATCH_PADDED_D(pad, b_dtype, a_dtype, SFB_TN32);
        } else {
            if (block_size == 64) SFB_DISPATCH_PADDED_D(pad, b_dtype, a_dtype, SFB_NN64);
            else SFB_DISPATCH_PADDED_D(pad, b_dtype, a_dtype, SFB_NN32);
        }
#undef SFB_TN64
#undef SFB_TN32
#undef SFB_NN64
#undef SFB_NN32
        return launch_status();
    }
    if (state_dim != 64) {
#define SFB_TN64(DV, TB, TA) dsd_tn_kernel<64, DV, TA, TB><<<grid, dim3(128), 0, s>>>(p)
#define SFB_TN32(DV, TB, TA) dsd_tn_kernel<32, DV, TA, TB><<<grid, dim3(64), 0, s>>>(p)
#define SFB_NN64(DV, TB, TA) dsd_nn_kernel<64, DV, TA, TB><<<grid, dim3(128), 0, s>>>(p)
#define SFB_NN32(DV, TB, TA) dsd_nn_kernel<32, DV, TA, TB><<<grid, dim3(64), 0, s>>>(p)
        if (op == SFB_TN_OP) {
            if (block_size == 64) SFB_DISPATCH_OTHER_D(state_dim, b_dtype, a_dtype, SFB_TN64);
            else SFB_DISPATCH_OTHER_D(state_dim, b_dtype, a_dtype, SFB_TN32);
        } else {
            if (block_size == 64) SFB_DISPATCH_OTHER_D(state_dim, b_dtype, a_dtype, SFB_NN64);
            else SFB_DISPATCH_OTHER_D(state_dim, b_dtype, a_dtype, SFB_NN32);
        }
#undef SFB_TN64
#undef SFB_TN32
#undef SFB_NN64
#undef SFB_NN32
        return launch_status();
    }
    if (op == SFB_TN_OP) {
#define SFB_CALL(BSV, TA, TB) dsd_tn_kernel<BSV, 64, TA, TB><<<grid, dim3(BSV * 2), 0, s>>>(p)
        if (block_size == 64) SFB_DISPATCH_2(64, a_dtype, b_dtype, SFB_CALL);
        else SFB_DISPATCH_2(32, a_dtype, b_dtype, SFB_CALL);
#undef SFB_CALL
        return launch_status();
    }
#define SFB_CALL(BSV, TP, TV) dsd_nn_kernel<BSV, 64, TP, TV><<<grid, dim3(BSV * 2), 0, s>>>(p)
    if (block_size == 64) SFB_DISPATCH_2(64, a_dtype, b_dtype, SFB_CALL);
    else SFB_DISPATCH_2(32, a_dtype, b_dtype, SFB_CALL);
#undef SFB_CALL
    return launch_status();
}

extern "C" int sfb_masked_softmax_grad(sfb_stream_t stream, const sfb_uint2* lut, const void* dy, const void* y,
                                       void* dx, int dtype, uint32_t block_size, uint32_t blocks,
                                       uint32_t batch_dim, uint32_t head_dim, uint32_t ctx_blks,
                                       uint32_t lut_heads, uint32_t lut_dim, uint32_t max_lut, float scale) {
    (void)max_lut;  // sizes the reference's shared memory (blocksparse.h:671-686); not needed here
    if (!lut || !dy || !y || !dx) return SFB_ERR_NULL_POINTER;
    if (check_dtype(dtype)) return SFB_ERR_DTYPE;
    if (block_size != 8 && block_size != 16 && block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (!blocks || !batch_dim || !head_dim || !ctx_blks || !lut_heads) return SFB_ERR_SHAPE;
    if (lut_heads > 1 && (lut_heads != head_dim || lut_dim != ctx_blks + blocks)) return SFB_ERR_SHAPE;
    if (!(scale > 0.f) || !(scale < 3.0e38f)) return SFB_ERR_ARGUMENT;
    if (((uintptr_t)dy | (uintptr_t)y | (uintptr_t)dx) & 15u) return SFB_ERR_ALIGNMENT;
    SoftmaxGradParams p = {lut, dy, y, dx, blocks, batch_dim, head_dim, ctx_blks, lut_heads > 1 ? lut_dim : 0, scale};
    const uint64_t groups = softmax_grid(batch_dim, head_dim, ctx_blks, block_size);
    if (groups > 0x7fffffffull) return SFB_ERR_SHAPE;
    const dim3 grid((uint32_t)groups);
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
#define SFB_CALL(BSV)                                                                            \
    do {                                                                                         \
        if (dtype == SFB_F32) masked_softmax_grad_kernel<BSV, float><<<grid, dim3(256), 0, s>>>(p); \
        else masked_softmax_grad_kernel<BSV, __bf16><<<grid, dim3(256), 0, s>>>(p);               \
    } while (0)
    if (block_size == 64) SFB_CALL(64);
    else if (block_size == 32) SFB_CALL(32);
    else if (block_size == 16) SFB_CALL(16);
    else SFB_CALL(8);
#undef SFB_CALL
    return launch_status();
}

extern "C" int sfb_fused_sdd_softmax(sfb_stream_t stream, const sfb_uint2* nn_lut, const void* a,
                                     const void* b, void* y, int in_dtype, int y_dtype, const void* mask,
                                     const int32_t* valid_len, const uint32_t* row_order, uint32_t block_size,
                                     uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                                     uint32_t state_dim, uint32_t lut_heads, uint32_t lut_dim,
                                     uint32_t mask_heads, float scale) {
    if (!nn_lut || !a || !b || !y) return SFB_ERR_NULL_POINTER;
    if (check_dtype(in_dtype) || check_dtype(y_dtype)) return SFB_ERR_DTYPE;
    if (block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (check_head_state(state_dim, in_dtype)) return SFB_ERR_HEAD_STATE;
    if (!blocks || !batch_dim || !head_dim || !ctx_blks || !lut_heads || !mask_heads) return SFB_ERR_SHAPE;
    if (lut_heads > 1 && (lut_heads != head_dim || lut_dim != ctx_blks + blocks)) return SFB_ERR_SHAPE;
    if (mask_heads > 1 && mask_heads != head_dim) return SFB_ERR_SHAPE;
    if (!(scale > 0.f) || !(scale < 3.0e38f)) return SFB_ERR_ARGUMENT;
    if (((uintptr_t)a | (uintptr_t)b | (uintptr_t)y) & 15u) return SFB_ERR_ALIGNMENT;
    SddSoftmaxParams p = {nn_lut, a, b, y, mask, valid_len, row_order, blocks, batch_dim, head_dim, ctx_blks,
                          lut_heads > 1 ? lut_dim : 0, mask_heads > 1 ? blocks * block_size : 0,
                          bh_groups(batch_dim * head_dim), scale * kLog2e, state_dim};
    const dim3 grid(p.groups * 8u * ctx_blks);
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
    if (state_dim % 32 != 0) {
#define SFB_CALL64(DV, TI, TO) sdd_softmax_kernel<64, DV, TI, TO, true><<<grid, dim3(128 * kSddSoftmaxKeyGroups), 0, s>>>(p)
#define SFB_CALL32(DV, TI, TO) sdd_softmax_kernel<32, DV, TI, TO, true><<<grid, dim3(64 * kSddSoftmaxKeyGroups), 0, s>>>(p)
        if (block_size == 64) SFB_DISPATCH_PADDED_D(padded_head_state(state_dim), in_dtype, y_dtype, SFB_CALL64);
        else SFB_DISPATCH_PADDED_D(padded_head_state(state_dim), in_dtype, y_dtype, SFB_CALL32);
#undef SFB_CALL64
#undef SFB_CALL32
        return launch_status();
    }
    if (state_dim != 64) {
#define SFB_CALL64(DV, TI, TO) sdd_softmax_kernel<64, DV, TI, TO><<<grid, dim3(128 * kSddSoftmaxKeyGroups), 0, s>>>(p)
#define SFB_CALL32(DV, TI, TO) sdd_softmax_kernel<32, DV, TI, TO><<<grid, dim3(64 * kSddSoftmaxKeyGroups), 0, s>>>(p)
        if (block_size == 64) SFB_DISPATCH_OTHER_D(state_dim, in_dtype, y_dtype, SFB_CALL64);
        else SFB_DISPATCH_OTHER_D(state_dim, in_dtype, y_dtype, SFB_CALL32);
#undef SFB_CALL64
#undef SFB_CALL32
        return launch_status();
    }
    if (block_size == 64 && in_dtype == SFB_BF16) {
        if (y_dtype == SFB_BF16) sdd_softmax_stream_kernel<__bf16><<<grid, dim3(128), 0, s>>>(p);
        else sdd_softmax_stream_kernel<float><<<grid, dim3(128), 0, s>>>(p);
        return launch_status();
    }
#define SFB_CALL(BSV, TI, TO) sdd_softmax_kernel<BSV, 64, TI, TO><<<grid, dim3(BSV * 2 * kSddSoftmaxKeyGroups), 0, s>>>(p)
    if (block_size == 64) SFB_DISPATCH_2(64, in_dtype, y_dtype, SFB_CALL);
    else SFB_DISPATCH_2(32, in_dtype, y_dtype, SFB_CALL);
#undef SFB_CALL
    return launch_status();
}

extern "C" size_t sfb_split_softmax_scratch_bytes(uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                                  uint32_t head_dim, uint32_t ctx_blks) {
    const size_t bh = (size_t)batch_dim * head_dim;
    const size_t stats = (bh * blocks * block_size * sizeof(float) + 255) / 256 * 256;
    const size_t flags = (bh * ctx_blks * 2 * sizeof(uint32_t) + 255) / 256 * 256;
    return 2 * stats + flags + 256;
}

extern "C" int sfb_fused_sdd_softmax_split(sfb_stream_t stream, const sfb_uint2* nt_lut, const sfb_uint2* nn_lut,
                                           const void* a, const void* b, void* y, int in_dtype, int y_dtype,
                                           const void* mask, const int32_t* valid_len, void* scratch,
                                           size_t scratch_bytes, uint32_t spin_limit, uint32_t block_size,
                                           uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                                           uint32_t state_dim, uint32_t lut_heads, uint32_t mask_heads, float scale) {
    if (!nt_lut || !nn_lut || !a || !b || !y || !scratch) return SFB_ERR_NULL_POINTER;
    if (check_dtype(in_dtype) || check_dtype(y_dtype)) return SFB_ERR_DTYPE;
    if (block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (state_dim != 64) return SFB_ERR_HEAD_STATE;
    if (!blocks || !batch_dim || !head_dim || !ctx_blks || !lut_heads || !mask_heads) return SFB_ERR_SHAPE;
    if (lut_heads > 1 && lut_heads != head_dim) return SFB_ERR_SHAPE;
    if (mask_heads > 1 && mask_heads != head_dim) return SFB_ERR_SHAPE;
    if (batch_dim > 65535 || head_dim > 65535) return SFB_ERR_SHAPE;
    if (!(scale > 0.f) || !(scale < 3.0e38f)) return SFB_ERR_ARGUMENT;
    if (((uintptr_t)a | (uintptr_t)b | (uintptr_t)y) & 15u) return SFB_ERR_ALIGNMENT;
    if (scratch_bytes < sfb_split_softmax_scratch_bytes(block_size, blocks, batch_dim, head_dim, ctx_blks) ||
        ((uintptr_t)scratch & 255u))
        return SFB_ERR_WORKSPACE;
    const size_t bh = (size_t)batch_dim * head_dim;
    const size_t stats = (bh * blocks * block_size * sizeof(float) + 255) / 256 * 256;
    const size_t flags = (bh * ctx_blks * 2 * sizeof(uint32_t) + 255) / 256 * 256;
    uint8_t* base = (uint8_t*)scratch;
    SplitSoftmaxParams p = {nt_lut, nn_lut, a, b, y, mask, valid_len, (float*)base, (float*)(base + stats),
                            (uint32_t*)(base + 2 * stats), (uint32_t*)(base + 2 * stats + flags), blocks, head_dim,
                            ctx_blks, lut_heads > 1 ? blocks : 0, lut_heads > 1 ? ctx_blks + blocks : 0,
                            mask_heads > 1 ? blocks * block_size : 0, spin_limit, scale * kLog2e};
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
    // the flags and the status word start at zero on every launch (the reference's callers clear rblk_flag,
    // rblk_flag1 with cudaMemset before each launch, fixed_fusion_test.cu:348-351)
    zero_words_kernel<<<dim3((uint32_t)((flags + 256) / 4 / 256 + 1)), dim3(256), 0, s>>>(p.flags, (uint32_t)((flags + 256) / 4));
    const dim3 grid(blocks, batch_dim, head_dim);
#define SFB_CALL(BSV, TI, TO) sdd_softmax_split_kernel<BSV, 64, TI, TO><<<grid, dim3(BSV * 2), 0, s>>>(p)
    if (block_size == 64) SFB_DISPATCH_2(64, in_dtype, y_dtype, SFB_CALL);
    else SFB_DISPATCH_2(32, in_dtype, y_dtype, SFB_CALL);
#undef SFB_CALL
    return launch_status();
}

extern "C" int sfb_row_dot(sfb_stream_t stream, float* delta, const void* d_out, const float* o, int dtype,
                           uint32_t batch_dim, uint32_t ctx, uint32_t head_dim, uint32_t state_dim) {
    if (!delta || !d_out || !o) return SFB_ERR_NULL_POINTER;
    if (check_dtype(dtype)) return SFB_ERR_DTYPE;
    if (check_head_state(state_dim, dtype)) return SFB_ERR_HEAD_STATE;
    if (!batch_dim || !ctx || !head_dim) return SFB_ERR_SHAPE;
    const uint64_t rows = (uint64_t)batch_dim * ctx * head_dim;
    if ((rows * 16 + 255) / 256 > 0x7fffffffull) return SFB_ERR_SHAPE;
    const dim3 grid((uint32_t)((rows * 16 + 255) / 256));
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
#define SFB_CALL(DV)                                                                                          \
    do {                                                                                                      \
        if (dtype == SFB_F32) row_dot_kernel<DV, float><<<grid, dim3(256), 0, s>>>(delta, (const float*)d_out, o, batch_dim, ctx, head_dim); \
        else row_dot_kernel<DV, __bf16><<<grid, dim3(256), 0, s>>>(delta, (const __bf16*)d_out, o, batch_dim, ctx, head_dim);                 \
    } while (0)
    if (state_dim == 64) SFB_CALL(64);
    else if (state_dim == 32) SFB_CALL(32);
    else if (state_dim == 96) SFB_CALL(96);
    else if (state_dim == 128) SFB_CALL(128);
    else if (dtype == SFB_F32) row_dot_any_kernel<float><<<grid, dim3(256), 0, s>>>(delta, (const float*)d_out, o, batch_dim, ctx, head_dim, state_dim);
    else row_dot_any_kernel<__bf16><<<grid, dim3(256), 0, s>>>(delta, (const __bf16*)d_out, o, batch_dim, ctx, head_dim, state_dim);
#undef SFB_CALL
    return launch_status();
}

extern "C" int sfb_sdd_softmax_grad(sfb_stream_t stream, const sfb_uint2* nt_lut, const void* d_out, const void* v,
                                    const void* p, const float* delta, void* ds, int in_dtype, int sparse_dtype,
                                    uint32_t block_size, uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks,
                                    uint32_t head_dim, uint32_t state_dim, uint32_t lut_heads, float scale) {
    if (!nt_lut || !d_out || !v || !p || !delta || !ds) return SFB_ERR_NULL_POINTER;
    if (check_dtype(in_dtype) || check_dtype(sparse_dtype)) return SFB_ERR_DTYPE;
    if (block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (check_head_state(state_dim, in_dtype)) return SFB_ERR_HEAD_STATE;
    if (!blocks || !batch_dim || !head_dim || !ctx_blks || !lut_heads) return SFB_ERR_SHAPE;
    if (lut_heads > 1 && lut_heads != head_dim) return SFB_ERR_SHAPE;
    if (batch_dim > 65535 || head_dim > 65535) return SFB_ERR_SHAPE;
    if (!(scale > 0.f) || !(scale < 3.0e38f)) return SFB_ERR_ARGUMENT;
    if (((uintptr_t)d_out | (uintptr_t)v | (uintptr_t)p | (uintptr_t)ds) & 15u) return SFB_ERR_ALIGNMENT;
    SddGradParams g = {nt_lut, d_out, v, p, delta, ds, blocks, head_dim, ctx_blks * block_size,
                       lut_heads > 1 ? blocks : 0, scale, state_dim};
    const dim3 grid(blocks, batch_dim, head_dim);
    hipStream_t s = (hipStream_t)stream;
    clear_stale_error();
    if (state_dim % 32 != 0) {
#define SFB_CALL64(DV, TI, TS) sdd_softmax_grad_kernel<64, DV, TI, TS, true><<<grid, dim3(128), 0, s>>>(g)
#define SFB_CALL32(DV, TI, TS) sdd_softmax_grad_kernel<32, DV, TI, TS, true><<<grid, dim3(64), 0, s>>>(g)
        if (block_size == 64) SFB_DISPATCH_PADDED_D(padded_head_state(state_dim), in_dtype, sparse_dtype, SFB_CALL64);
        else SFB_DISPATCH_PADDED_D(padded_head_state(state_dim), in_dtype, sparse_dtype, SFB_CALL32);
#undef SFB_CALL64
#undef SFB_CALL32
        return launch_status();
    }
    if (state_dim != 64) {
#define SFB_CALL64(DV, TI, TS) sdd_softmax_grad_kernel<64, DV, TI, TS><<<grid, dim3(128), 0, s>>>(g)
#define SFB_CALL32(DV, TI, TS) sdd_softmax_grad_kernel<32, DV, TI, TS><<<grid, dim3(64), 0, s>>>(g)
        if (block_size == 64) SFB_DISPATCH_OTHER_D(state_dim, in_dtype, sparse_dtype, SFB_CALL64);
        else SFB_DISPATCH_OTHER_D(state_dim, in_dtype, sparse_dtype, SFB_CALL32);
#undef SFB_CALL64
#undef SFB_CALL32
        return launch_status();
    }
#define SFB_CALL(BSV, TI, TS) sdd_softmax_grad_kernel<BSV, 64, TI, TS><<<grid, dim3(BSV * 2), 0, s>>>(g)
    if (block_size == 64) SFB_DISPATCH_2(64, in_dtype, sparse_dtype, SFB_CALL);
    else SFB_DISPATCH_2(32, in_dtype, sparse_dtype, SFB_CALL);
#undef SFB_CALL
    return launch_status();
}
