// LDS tiles and MFMA fragment access shared by the attention kernels.
//
// A work-group of NT = 2*BS threads (BS/32 waves, each owning 32 query rows) walks key blocks of BS
// keys.  Lane l of a wave is query column qn = l % 32 and half = l / 32 of the 32x32 MFMA shapes.
//
// Score tile, transposed:  S^T[key][query] = sum_k K[key][k] Q[query][k]      (A = K, B = Q^T)
//   accumulator element i of key tile kt is key  kt*32 + (i/4)*8 + half*4 + i%4  of query qn.
// Output tile, transposed: O^T[col][query] += sum_key V[key][col] P[query][key] (A = V^T, B = P^T)
//   accumulator element i of column tile mt is column  mt*32 + (i/4)*8 + half*4 + i%4.
// Because both accumulators keep one query per lane, the softmax is lane-local and P feeds the
// second product without leaving its registers.
#pragma once

#include "common.hip.h"
#include "tile_index.h"

namespace sfb {

// ------------------------------------------------------------------------------------------------
// bf16 operands, v_mfma_f32_32x32x16_bf16 (8 bf16 per lane per step: k-slots half*8 .. half*8+7);
// tiles copied from memory straight into LDS (global_load_lds_dwordx4)
// ------------------------------------------------------------------------------------------------
// K and V tiles are both kept row-major, [BS keys][D] bf16 = 128-byte rows of eight 16-byte chunks, with
// no padding: an LDS-direct load writes the 64 lanes' 16 bytes back to back (1 KiB = 8 rows per
// instruction), so the layout inside a row is chosen through the *global* address each lane fetches.
// Chunk c of row r is stored at position c ^ swz(r), swz(r) = rotate-right of the 3-bit value (r/2)%8:
//   * score fragments (ds_read_b128; 16 lanes = 16 consecutive rows, one chunk) hit 16 different
//     16-byte slots of the 256-byte bank window, because rows 2a and 2a+1 sit in different halves of
//     the window and swz() is distinct over a = 0..7;
//   * V^T fragments are read with ds_read_b64_tr_b16, which transposes inside groups of 16 lanes: source
//     lane s = 4j + q supplies 4 consecutive columns of key row j (j = 0..3) starting at column 4q, and
//     result lane i receives the 4 consecutive keys of column i.  The lowest bit of r/2 becomes the
//     highest bit of swz(), which moves key rows j = 2, 3 into the other 64-byte half of the row, so
//     the 4 rows x 64 bytes that 32 lanes touch are disjoint in the bank window.
// No registers are spent on staging and no ds_write / v_perm instructions are needed.
template <int BS, int D>
struct Bf16DirectTiles {
    // Head sizes other than 64 are cut into slices of 64 features, each slice a tile of 128-byte rows in the layout
    // above (slice f of a K or V tile starts 128*f bytes into the tensor's rows and BS*128*f bytes into the LDS
    // tile).  A last slice of 32 features (head sizes 32 and 96) fills only the first four chunks of its rows: its
    // lanes fetch chunk (c ^ swz) & 3 instead of c ^ swz, so that nothing beyond the row is read, and the fragment
    // readers, which only ever ask for chunks 0..3 of such a slice, find them where they expect them.
    // Every offset comes from TileIndex (tile_index.h), which a host program can compile and check.
    using I = TileIndex<BS, D>;
    static constexpr int NW = I::NW;                   // waves per work-group
    static constexpr int SLICES = I::SLICES;
    static constexpr bool PARTIAL = I::PARTIAL;        // the last slice has 32 features
    static constexpr int SLICE_BYTES = I::SLICE_BYTES;
    static constexpr int TILE_BYTES = I::TILE_BYTES;
    static constexpr int GROUPS = I::GROUPS;           // 8-row groups (one load instruction each)

    typedef uint32_t __attribute__((address_space(3)))* lds_u32_ptr;
    // LDS byte address of a pointer into a __shared__ array
    static __device__ __forceinline__ uint32_t lds_address(const void* p) {
        return (uint32_t)(uintptr_t)(lds_u32_ptr)p;
    }
    static __device__ __forceinline__ uint32_t swz(uint32_t row) { return I::swz(row); }
    // Byte offset, relative to row 0 of an 8-row group, of the 16 bytes this lane fetches; `odd` says
    // whether the group index is odd (rows 8..15 of a 16-row period).
    static __device__ __forceinline__ uint32_t lane_source(uint32_t lane, uint32_t odd, uint32_t row_bytes) {
        return I::lane_source(lane, odd, row_bytes);
    }
    // The same for a last slice of 32 features.
    static __device__ __forceinline__ uint32_t lane_source_part(uint32_t lane, uint32_t odd, uint32_t row_bytes) {
        return I::lane_source_part(lane, odd, row_bytes);
    }
    // The four lane offsets a work-group needs to fetch whole tiles.
    struct Sources {
        uint32_t even, odd, even_part, odd_part;
    };
    static __device__ __forceinline__ Sources sources(uint32_t lane, uint32_t row_bytes) {
        Sources s;
        s.even = lane_source(lane, 0, row_bytes);
        s.odd = lane_source(lane, 1, row_bytes);
        s.even_part = PARTIAL ? lane_source_part(lane, 0, row_bytes) : s.even;
        s.odd_part = PARTIAL ? lane_source_part(lane, 1, row_bytes) : s.odd;
        return s;
    }
    // Sources for tensors whose head size hd (a multiple of 8, more than D - 32) is smaller than D: the last slice's
    // lanes stay inside the hd features of their rows (TileIndex::lane_source_ragged).  Used with
    // load_rows_all<true> / load_tile_all<true>, which treat the last slice as the partial one whatever D is.
    static __device__ __forceinline__ Sources sources_ragged(uint32_t lane, uint32_t row_bytes, uint32_t hd) {
        Sources s;
        s.even = lane_source(lane, 0, row_bytes);
        s.odd = lane_source(lane, 1, row_bytes);
        s.even_part = I::lane_source_ragged(lane, 0, row_bytes, I::last_slice_chunks(hd));
        s.odd_part = I::lane_source_ragged(lane, 1, row_bytes, I::last_slice_chunks(hd));
        return s;
    }
    // The same for a tile whose LDS rows hold the source rows in the order that makes the 8 k-slots of a lane
    // in the second product 8 consecutive source rows.  Used with load_rows<4>: the group's base advances by 4
    // source rows.
    static __device__ __forceinline__ uint32_t lane_source_by_halves(uint32_t lane, uint32_t odd, uint32_t row_bytes) {
        return I::lane_source_by_halves(lane, odd, row_bytes);
    }
    // Load number i (0 .. LOADS-1) of this wave's share of one tile: 8 rows = 1 KiB.  g_tile: address of
    // the tile's first row (uniform); lds_tile: LDS byte address of the tile (uniform); src_even /
    // src_odd from lane_source().
    static constexpr int LOADS = I::LOADS;
    template <int GROUP_ROWS = 8>
    static __device__ __forceinline__ void load_rows(uint32_t lds_tile, const uint8_t* g_tile, int i, uint32_t wave,
                                                     uint32_t src_even, uint32_t src_odd, uint32_t row_bytes) {
        const uint32_t n = I::load_group(i, wave);      // 8-row group
        const uint32_t src = I::load_group_odd(i, wave) ? src_odd : src_even;
        // scalar 64-bit base + 32-bit lane offset: no vector address arithmetic.  The instruction takes its
        // LDS destination from M0, which is written in the same statement.  M0 cannot be named as a clobber (the
        // compiler reserves it and rejects it there); it never keeps a value in M0 across statements -- it writes
        // M0 directly before each instruction of its own that reads it -- and these kernels use none of the
        // operations for which it would (LDS-direct builtins, messages, relative register moves): in the compiled
        // kernels every write of M0 is one of these, each followed by its load, which a test of the assembly checks.
        const uint64_t ga = (uint64_t)(g_tile + (size_t)n * (uint32_t)GROUP_ROWS * row_bytes);
        const uint32_t ga_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(ga >> 32));
        const uint32_t ga_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)ga);   // unsigned: no sign extension
        const uint64_t base = ((uint64_t)ga_hi << 32) | (uint64_t)ga_lo;
        const uint32_t dst = (uint32_t)__builtin_amdgcn_readfirstlane(lds_tile + n * 1024u);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :
                     : "s"(dst), "v"(src), "s"(base)
                     : "memory");
    }
    static __device__ __forceinline__ void load_tile(uint32_t lds_tile, const uint8_t* g_tile, uint32_t wave,
                                                     uint32_t src_even, uint32_t src_odd, uint32_t row_bytes) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) load_rows(lds_tile, g_tile, i, wave, src_even, src_odd, row_bytes);
    }
    // A wave's whole share of a one-slice tile as one group of loads: M0 is written once, the step from one 8-row
    // group to the next rides in the instruction offsets (which go into the global and the LDS address alike) and
    // the lanes' global offsets make up the difference (TileIndex::once_*).  Against load_tile that is one M0 write
    // and one 64-bit scalar address per tile instead of four of each.  off[i] = once_lane_offset(lane, i, wave, ..).
    struct OnceSources {
        uint32_t off[I::LOADS];
    };
    static __device__ __forceinline__ OnceSources once_sources(uint32_t lane, uint32_t wave, uint32_t row_bytes) {
        OnceSources s;
#pragma unroll
        for (int i = 0; i < I::LOADS; ++i) s.off[i] = I::once_lane_offset(lane, i, wave, row_bytes);
        return s;
    }
    static __device__ __forceinline__ void load_tile_once(uint32_t lds_tile, const uint8_t* g_tile, uint32_t wave,
                                                          const OnceSources& src, uint32_t row_bytes) {
        static_assert(SLICES == 1 && !PARTIAL && I::LOADS == 4, "whole one-slice tiles");
        const uint64_t ga = (uint64_t)(g_tile + I::once_base(wave, row_bytes));
        const uint32_t ga_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(ga >> 32));
        const uint32_t ga_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)ga);
        const uint64_t base = ((uint64_t)ga_hi << 32) | (uint64_t)ga_lo;
        const uint32_t m0 = (uint32_t)__builtin_amdgcn_readfirstlane(lds_tile + I::once_m0(wave));
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                     "global_load_lds_dwordx4 %1, %5 offset:%6\n\t"
                     "global_load_lds_dwordx4 %2, %5 offset:%7\n\t"
                     "global_load_lds_dwordx4 %3, %5 offset:%8\n\t"
                     "global_load_lds_dwordx4 %4, %5 offset:%9"
                     :
                     : "s"(m0), "v"(src.off[0]), "v"(src.off[1]), "v"(src.off[2]), "v"(src.off[3]), "s"(base),
                       "n"(I::once_inst_offset(0)), "n"(I::once_inst_offset(1)), "n"(I::once_inst_offset(2)),
                       "n"(I::once_inst_offset(3))
                     : "memory");
    }
    // A wave's share of a one-slice tile on its way through registers: fetch() issues ordinary 16-byte loads of whole
    // rows (the wave is free again as soon as they are issued), commit() writes them to LDS with the swizzle applied
    // on that side (TileIndex::staged_*).  Against the LDS-direct form this costs 16 registers per tile in flight
    // and four ds_write_b128 per wave and tile.
    struct Staged {
        u32x4 r[I::LOADS];
    };
    static __device__ __forceinline__ void staged_fetch(Staged& st, const uint8_t* g_tile, uint32_t wave, uint32_t lane_src,
                                                        uint32_t row_bytes) {
        static_assert(SLICES == 1 && !PARTIAL, "whole one-slice tiles");
#pragma unroll
        for (int i = 0; i < I::LOADS; ++i)
            st.r[i] = *(const u32x4*)(g_tile + (size_t)I::load_group(i, wave) * 8u * row_bytes + lane_src);
    }
    static __device__ __forceinline__ void staged_commit(const Staged& st, uint8_t* lds_tile, uint32_t wave,
                                                         uint32_t dst_even, uint32_t dst_odd) {
#pragma unroll
        for (int i = 0; i < I::LOADS; ++i)
            *(u32x4*)(lds_tile + I::load_group(i, wave) * 1024u + (I::load_group_odd(i, wave) ? dst_odd : dst_even)) = st.r[i];
    }
    // Load number i of this wave's share of every slice of a tile.
    template <bool RAGGED = false>
    static __device__ __forceinline__ void load_rows_all(uint32_t lds_tile, const uint8_t* g_tile, int i, uint32_t wave,
                                                         const Sources& src, uint32_t row_bytes) {
#pragma unroll
        for (int f = 0; f < SLICES; ++f) {
            const bool part = (PARTIAL || RAGGED) && f == SLICES - 1;
            load_rows(lds_tile + f * SLICE_BYTES, g_tile + f * 128, i, wave, part ? src.even_part : src.even,
                      part ? src.odd_part : src.odd, row_bytes);
        }
    }
    template <bool RAGGED = false>
    static __device__ __forceinline__ void load_tile_all(uint32_t lds_tile, const uint8_t* g_tile, uint32_t wave,
                                                         const Sources& src, uint32_t row_bytes) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) load_rows_all<RAGGED>(lds_tile, g_tile, i, wave, src, row_bytes);
    }
    // with src_even / src_odd from lane_source_by_halves()
    static __device__ __forceinline__ void load_tile_by_halves(uint32_t lds_tile, const uint8_t* g_tile, uint32_t wave,
                                                               uint32_t src_even, uint32_t src_odd,
                                                               uint32_t row_bytes) {
#pragma unroll
        for (int i = 0; i < LOADS; ++i) load_rows<4>(lds_tile, g_tile, i, wave, src_even, src_odd, row_bytes);
    }
    // Per-lane byte offset of the score fragment of k-step 0 in key tile 0; k-step ks is at (base ^ ks*32),
    // key tile kt 4096 bytes further.
    static __device__ __forceinline__ uint32_t k_lane_base(uint32_t qn, uint32_t half) {
        return I::k_lane_base(qn, half);
    }
    static __device__ __forceinline__ bf16x8 k_frag(const uint8_t* k_lds, uint32_t lane_base, int kt, int ks) {
        return *(const bf16x8*)(k_lds + I::k_frag_const(kt, ks) + I::k_frag_lane(lane_base, ks));
    }
    // Per-lane byte offset of the transposing read for (column tile 0, first 4-key group of product step
    // 0); column tile mt and second group x are at (base ^ (mt*64 + x*32)) + x*1024, step u 2048 bytes on.
    static __device__ __forceinline__ uint32_t v_lane_base(uint32_t lane) {
        return I::v_lane_base(lane);
    }
    static __device__ __forceinline__ bf16x8 v_frag(const uint8_t* v_lds, uint32_t lane_base, int mt, int u) {
        typedef short s16x4 __attribute__((ext_vector_type(4)));
        typedef s16x4 __attribute__((address_space(3)))* lds_ptr;
        const uint8_t* a0 = v_lds + I::v_frag_const(mt, u, 0) + I::v_frag_lane(lane_base, mt, 0);
        const uint8_t* a1 = v_lds + I::v_frag_const(mt, u, 1) + I::v_frag_lane(lane_base, mt, 1);
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)a0);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)a1);
        const u32x4 r = {__builtin_bit_cast(u32x2, lo).x, __builtin_bit_cast(u32x2, lo).y,
                         __builtin_bit_cast(u32x2, hi).x, __builtin_bit_cast(u32x2, hi).y};
        return __builtin_bit_cast(bf16x8, r);
    }
    static __device__ __forceinline__ void load_q(bf16x8 (&qf)[D / 16], const __bf16* q_row, uint32_t half) {
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) qf[ks] = *(const bf16x8*)(q_row + (2 * ks + half) * 8);
    }
    // a row of hd < D features: the missing ones are zeros, so whatever the K tile holds in their place drops out
    static __device__ __forceinline__ void load_q_ragged(bf16x8 (&qf)[D / 16], const __bf16* q_row, uint32_t half,
                                                         uint32_t hd) {
#pragma unroll
        for (int ks = 0; ks < D / 16; ++ks) {
            const uint32_t first = (2 * ks + half) * 8;
            const u32x4 zero = {0u, 0u, 0u, 0u};
            qf[ks] = first < hd ? *(const bf16x8*)(q_row + first) : __builtin_bit_cast(bf16x8, zero);
        }
    }
};

// ------------------------------------------------------------------------------------------------
// fp32 operands, v_mfma_f32_32x32x2_f32 (one float per lane per step: k-slot = half)
// ------------------------------------------------------------------------------------------------
// K tile in LDS: [BS][D + 4] floats; score k-slot (step, half) is head-dimension index
//   8*(step/4) + 4*half + step%4, so one 128-bit read feeds four steps.
// V tile in LDS: [BS][D + 8] floats, row-major (no transposition needed: product step (kt, i)
//   consumes key kt*32 + (i/4)*8 + half*4 + i%4 and reads 32 consecutive floats of that row).
template <int BS, int D>
struct F32Tiles {
    static constexpr int NT = BS * 2;
    static constexpr int K_STRIDE = D + 4;  // floats
    static constexpr int V_STRIDE = D + 8;  // floats
    static constexpr int K_FLOATS = BS * K_STRIDE;
    static constexpr int V_FLOATS = BS * V_STRIDE;
    static constexpr int CHUNKS = D / 8;    // float4 chunks per thread per tile
    static_assert(D % 32 == 0, "head state must be a multiple of 32");

    struct Regs { f32x4 g[CHUNKS]; };

    static __device__ __forceinline__ void fetch(Regs& r, const float* X, size_t base,
                                                 uint32_t row_stride, uint32_t t) {
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
            const uint32_t cid = i * NT + t, row = cid / (D / 4), cc = cid % (D / 4);
            r.g[i] = *(const f32x4*)(X + base + (size_t)(row * row_stride + cc * 4));
        }
    }
    // rows of hd < D floats (hd a multiple of 4): the missing chunks are zeros and nothing beyond the row is read
    static __device__ __forceinline__ void fetch_ragged(Regs& r, const float* X, size_t base, uint32_t row_stride,
                                                        uint32_t t, uint32_t hd) {
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
            const uint32_t cid = i * NT + t, row = cid / (D / 4), cc = cid % (D / 4);
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            r.g[i] = cc * 4 < hd ? *(const f32x4*)(X + base + (size_t)(row * row_stride + cc * 4)) : zero;
        }
    }
    template <int STRIDE>
    static __device__ __forceinline__ void stage(float* lds, const Regs& r, uint32_t t) {
#pragma unroll
        for (int i = 0; i < CHUNKS; ++i) {
            const uint32_t cid = i * NT + t, row = cid / (D / 4), cc = cid % (D / 4);
            *(f32x4*)(lds + row * STRIDE + cc * 4) = r.g[i];
        }
    }
    static __device__ __forceinline__ f32x4 k_frag(const float* k_lds, int kt, int g, uint32_t qn,
                                                   uint32_t half) {
        return *(const f32x4*)(k_lds + (kt * 32 + qn) * K_STRIDE + 8 * g + 4 * half);
    }
    static __device__ __forceinline__ float v_elem(const float* v_lds, int kt, int i, int mt,
                                                   uint32_t qn, uint32_t half) {
        const uint32_t key = kt * 32 + (i / 4) * 8 + half * 4 + (i % 4);
        return v_lds[key * V_STRIDE + mt * 32 + qn];
    }
    static __device__ __forceinline__ void load_q(f32x4 (&qf)[D / 8], const float* q_row, uint32_t half) {
#pragma unroll
        for (int g = 0; g < D / 8; ++g) qf[g] = *(const f32x4*)(q_row + 8 * g + 4 * half);
    }
    static __device__ __forceinline__ void load_q_ragged(f32x4 (&qf)[D / 8], const float* q_row, uint32_t half,
                                                         uint32_t hd) {
#pragma unroll
        for (int g = 0; g < D / 8; ++g) {
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            qf[g] = 8 * g + 4 * half < hd ? *(const f32x4*)(q_row + 8 * g + 4 * half) : zero;
        }
    }
};

// Keep-bits of one lane's query row for one key block (block-major mask words), key padding folded in.
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

// Replace the scores of masked keys by kMaskedScore.  keep bit k = key k of the block is kept.
template <int KT>
__device__ __forceinline__ void apply_keep(f32x16 (&s)[KT], uint64_t keep, uint32_t half) {
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        const uint32_t w = (uint32_t)(keep >> (kt * 32)) >> (half * 4);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t bit = (i / 4) * 8 + (i % 4);
            s[kt][i] = ((w >> bit) & 1u) ? s[kt][i] : kMaskedScore;
        }
    }
}

// Maximum over this lane's scores of one block and over the partner lane (the other 16 keys of each
// 32-key tile of the same query).
template <int KT>
__device__ __forceinline__ float block_row_max(const f32x16 (&s)[KT]) {
    float mx0 = s[0][0], mx1 = s[0][1];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
        for (int i = 0; i < 16; i += 4) {
            mx0 = fmaxf(fmaxf(mx0, s[kt][i]), s[kt][i + 1]);
            mx1 = fmaxf(fmaxf(mx1, s[kt][i + 2]), s[kt][i + 3]);
        }
    }
    const float m = fmaxf(mx0, mx1);
    return fmaxf(m, __shfl_xor(m, 32));
}

}  // namespace sfb
