// Index arithmetic of the bf16 LDS tiles and of the counted waits, free of device code: the kernels take every
// offset from here (through Bf16DirectTiles in tiles.hip.h), and so does a host program, which can therefore check
// on the CPU that the lanes that fill a tile and the lanes that read its fragments agree, that no lane reads past
// its row and that no LDS offset leaves the tile.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define SFB_INDEX_FN __host__ __device__ __forceinline__
#else
#define SFB_INDEX_FN inline
#endif

namespace sfb {

// A tile is BS rows (keys, or queries for the transposed products of the backward pass) of D bf16 features, cut into
// slices of 64 features = 128-byte rows of eight 16-byte chunks.  An LDS-direct load instruction moves 1 KiB: lane l
// of the wave delivers bytes [16 l, 16 l + 16) of the destination, i.e. chunk position l % 8 of row l / 8 of an
// 8-row group, and fetches them from wherever its own address says.  Chunk c of row r is kept at position
// c ^ swz(r), so the lane at position pos of row r fetches chunk pos ^ swz(r).
template <int BS, int D>
struct TileIndex {
    static constexpr int NW = BS / 32;                 // waves per work-group
    static constexpr int SLICES = (D + 63) / 64;
    static constexpr bool PARTIAL = D % 64 != 0;       // the last slice has 32 features
    static constexpr int SLICE_BYTES = BS * 128;
    static constexpr int TILE_BYTES = SLICES * SLICE_BYTES;
    static constexpr int GROUPS = BS / 8;              // 8-row groups (one load instruction each)
    static constexpr int LOADS = GROUPS / NW;          // load instructions per wave and slice
    static_assert(D % 32 == 0 && D >= 32 && D <= 128, "head sizes 32, 64, 96, 128");

    static SFB_INDEX_FN uint32_t swz(uint32_t row) {
        const uint32_t x = (row >> 1) & 7u;
        return ((x & 1u) << 2) | (x >> 1);
    }
    // Byte offset, relative to row 0 of an 8-row group, of the 16 bytes this lane fetches; `odd` says whether the
    // group index is odd (rows 8..15 of a 16-row period: swz has period 16).
    static SFB_INDEX_FN uint32_t lane_source(uint32_t lane, uint32_t odd, uint32_t row_bytes) {
        const uint32_t rr = lane >> 3, pos = lane & 7u;
        return rr * row_bytes + ((pos ^ swz(8u * odd + rr)) << 4);
    }
    // The same for a last slice of 32 features: only chunks 0..3 exist, and the fragment readers only ever ask for
    // those, so the lanes fetch chunk (pos ^ swz) & 3 and nothing beyond the row is read.
    static SFB_INDEX_FN uint32_t lane_source_part(uint32_t lane, uint32_t odd, uint32_t row_bytes) {
        const uint32_t rr = lane >> 3, pos = lane & 7u;
        return rr * row_bytes + (((pos ^ swz(8u * odd + rr)) & 3u) << 4);
    }
    // The same for a last slice of which only the first nch chunks (1..8) exist in memory -- head sizes that are not
    // a multiple of 32, run through the kernel of the next multiple: positions whose chunk would lie beyond the row
    // fetch chunk (pos ^ swz) % nch instead (finite filler the readers multiply by zero queries or never store).
    static SFB_INDEX_FN uint32_t lane_source_ragged(uint32_t lane, uint32_t odd, uint32_t row_bytes, uint32_t nch) {
        const uint32_t rr = lane >> 3, pos = lane & 7u, x = pos ^ swz(8u * odd + rr);
        return rr * row_bytes + ((x < nch ? x : x % nch) << 4);
    }
    // Chunks of the last slice that a head size of hd features (a multiple of 8, SLICES slices) has in memory.
    static SFB_INDEX_FN uint32_t last_slice_chunks(uint32_t hd) { return (hd - 64u * (uint32_t)(SLICES - 1)) / 8u; }
    // The same for a tile whose LDS rows hold the source rows in the order that makes the 8 k-slots of a lane in
    // the second product, rows 16u + 8(j/4) + 4*half + j%4 of the tile, the 8 consecutive source rows
    // 32*half + 8u + j: LDS row 16u + 8a + 4h + c holds source row 32h + 8u + 4a + c, which is 4n + 32(rr/4) + rr%4
    // for row rr of 8-row group n.  The group's base then advances by 4 source rows per group.
    static SFB_INDEX_FN uint32_t lane_source_by_halves(uint32_t lane, uint32_t odd, uint32_t row_bytes) {
        const uint32_t rr = lane >> 3, pos = lane & 7u;
        return (32u * (rr >> 2) + (rr & 3u)) * row_bytes + ((pos ^ swz(8u * odd + rr)) << 4);
    }
    // Load number i (0 .. LOADS-1) of a wave's share of one slice: which 8-row group it fills and whether that
    // group's index is odd.  The group lands 1024 * group bytes into the slice and starts group_rows * group source
    // rows into the tile (group_rows = 8, or 4 with lane_source_by_halves).
    static SFB_INDEX_FN uint32_t load_group(int i, uint32_t wave) { return (uint32_t)(NW * i) + wave; }
    static SFB_INDEX_FN uint32_t load_group_odd(int i, uint32_t wave) {
        return NW % 2 == 0 ? (wave & 1u) : ((uint32_t)i & 1u);   // an even number of waves: the parity is the wave's
    }
    // A wave's LOADS loads of one slice issued as one group with a single LDS base: an LDS-direct load adds its
    // instruction offset to the global address *and* to the LDS address (M0 + offset + 16 lane), so the step from
    // one 8-row group to the wave's next (NW KiB in LDS) can ride in the instruction, with the lane's global offset
    // making up the difference.  Load i then fetches from  base + once_lane_offset(i) + once_inst_offset(i)  into
    // M0 + once_inst_offset(i) + 16 lane, where, relative to the slice's first source row and its LDS address,
    //   base = wave * 8 * row_bytes + ONCE_CENTER,   M0 = wave * 1024 + ONCE_CENTER;
    // ONCE_CENTER keeps the four instruction offsets inside the signed 13-bit field.  Only for whole slices in
    // source-row order (8 * row_bytes >= 1024, so the lane offsets never go negative).
    static constexpr int ONCE_CENTER = NW == 2 ? 4096 : 0;
    static SFB_INDEX_FN int once_inst_offset(int i) { return i * NW * 1024 - ONCE_CENTER; }
    static SFB_INDEX_FN uint32_t once_lane_offset(uint32_t lane, int i, uint32_t wave, uint32_t row_bytes) {
        return lane_source(lane, load_group_odd(i, wave), row_bytes) + (uint32_t)(i * NW) * (8u * row_bytes - 1024u);
    }
    static SFB_INDEX_FN uint32_t once_base(uint32_t wave, uint32_t row_bytes) {
        return wave * 8u * row_bytes + (uint32_t)ONCE_CENTER;
    }
    static SFB_INDEX_FN uint32_t once_m0(uint32_t wave) { return wave * 1024u + (uint32_t)ONCE_CENTER; }
    static_assert(LOADS == 4 && (LOADS - 1) * NW * 1024 - ONCE_CENTER <= 4095 && -ONCE_CENTER >= -4096,
                  "four loads per wave and slice, offsets of 13 signed bits");

    // The same tile filled through registers (ordinary 16-byte loads, then ds_write_b128): the lanes read whole rows
    // in order -- lane l the chunk l % 8 of row l / 8 of an 8-row group -- and apply the swizzle on the LDS side.
    // Both offsets are relative to the group's first source row / its 1 KiB of LDS.
    static SFB_INDEX_FN uint32_t staged_source(uint32_t lane, uint32_t row_bytes) {
        return (lane >> 3) * row_bytes + ((lane & 7u) << 4);
    }
    static SFB_INDEX_FN uint32_t staged_lds_offset(uint32_t lane, uint32_t odd) {
        const uint32_t rr = lane >> 3, c = lane & 7u;
        return rr * 128u + ((c ^ swz(8u * odd + rr)) << 4);
    }

    // Per-lane byte offset of the score fragment (16 bytes: 8 features of one row) of k-step 0 in row tile 0;
    // k-step ks (features 16 ks + 8 half ..) is at (base ^ (ks % 4) * 32) in slice ks / 4, row tile kt 4096 bytes on.
    static SFB_INDEX_FN uint32_t k_lane_base(uint32_t qn, uint32_t half) {
        return qn * 128u + ((half ^ swz(qn)) << 4);
    }
    // (in two parts, so that the kernels can add the constant part to the tile's address first: it then ends up in
    // the LDS instruction's offset field)
    static SFB_INDEX_FN uint32_t k_frag_const(int kt, int ks) { return (uint32_t)((ks / 4) * SLICE_BYTES + kt * 4096); }
    static SFB_INDEX_FN uint32_t k_frag_lane(uint32_t lane_base, int ks) { return lane_base ^ (uint32_t)((ks % 4) * 32); }
    static SFB_INDEX_FN uint32_t k_frag_offset(uint32_t lane_base, int kt, int ks) {
        return k_frag_const(kt, ks) + k_frag_lane(lane_base, ks);
    }
    // Per-lane byte offset of the transposing read (8 bytes) for (column tile 0, first 4-row group of product
    // step 0); column tile mt and second group x are at (base ^ ((mt % 2) * 64 + x * 32)) + x * 1024 in slice
    // mt / 2, step u 2048 bytes on.
    static SFB_INDEX_FN uint32_t v_lane_base(uint32_t lane) {
        const uint32_t G = lane >> 4, s = lane & 15u, j = s >> 2, q = s & 3u, h = G >> 1, g2 = G & 1u;
        const uint32_t lp = (2u * g2 + (q >> 1)) ^ (((j >> 1) << 2) | h);
        return (h * 4u + j) * 128u + (lp << 4) + (q & 1u) * 8u;
    }
    static SFB_INDEX_FN uint32_t v_frag_const(int mt, int u, int x) {
        return (uint32_t)((mt / 2) * SLICE_BYTES + u * 2048 + x * 1024);
    }
    static SFB_INDEX_FN uint32_t v_frag_lane(uint32_t lane_base, int mt, int x) {
        return lane_base ^ (uint32_t)((mt % 2) * 64 + x * 32);
    }
    static SFB_INDEX_FN uint32_t v_frag_offset(uint32_t lane_base, int mt, int u, int x) {
        return v_frag_const(mt, u, x) + v_frag_lane(lane_base, mt, x);
    }
};

// A wave's 32 x BS part of a sparse block on its way between registers and memory: whole rows through an LDS slab,
// 64 lanes x 16 bytes per instruction.
template <int BS, int ELEM_BYTES>
struct RowSlabIndex {
    static constexpr int ROW_BYTES = BS * ELEM_BYTES;
    static constexpr int PITCH = ROW_BYTES + 16;          // padded LDS row
    static constexpr int BYTES = 32 * PITCH;              // per wave
    static constexpr int CHUNKS = ROW_BYTES / 16;         // 16-byte chunks per row
    static constexpr int ROWS_PER_PASS = 64 / CHUNKS, PASSES = 32 / ROWS_PER_PASS;   // memory instructions per wave
};

// Counted waits.  Vector memory operations of a wave complete in the order they were issued, so
// `s_waitcnt vmcnt(N)` returns once all but the last N issued have completed.  Each kernel below states, per step
// of its loop, what a wave issues after the operations whose results the step reads; N is that number.
//
// sdd and the two-stage fusion's second pass (bf16, block 64, 64 features), step g: waits for K(g); since K(g)'s
// loads the wave has issued the stores of blocks g-2 and g-1 and the loads of K(g+1).  The count is exact, so it
// holds only while a step issues exactly LOADS tile loads and PASSES stores and nothing else -- no spill, no split
// store -- which a test of the compiled loop checks.
template <int SPARSE_ELEM_BYTES>
struct SddStreamWait {
    static constexpr int LOADS = TileIndex<64, 64>::LOADS;
    static constexpr int PASSES = RowSlabIndex<64, SPARSE_ELEM_BYTES>::PASSES;
    static constexpr int COUNT = LOADS + 2 * PASSES;
    static_assert(COUNT < 64, "vmcnt has 6 bits");
};
// dsd (bf16 P and V, block 64), pair of key blocks (j, j+1): waits for V(j), V(j+1) and P(j), P(j+1); behind them
// stand the loads of two later P blocks (DEPTH = 4 blocks ahead, 4 loads per lane and block).
struct DsdStreamWait {
    static constexpr int DEPTH = 4;
    static constexpr int P_LOADS = 4;                     // 16-byte loads per lane and block
    static constexpr int V_LOADS = TileIndex<64, 64>::LOADS;
    static constexpr int COUNT = (DEPTH - 2) * P_LOADS;
};

}  // namespace sfb
