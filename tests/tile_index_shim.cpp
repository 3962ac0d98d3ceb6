// Host build of the kernels' index arithmetic (sf-bert_amd/csrc/tile_index.h) for the CPU tests: plain C entry
// points that dispatch on (block size, head size).  Compiled by tests/tile_index_lib.py with g++; test
// infrastructure, never part of the product library.
#include "../sf-bert_amd/csrc/tile_index.h"

using namespace sfb;

#define DISPATCH(bs, d, EXPR)                                                   \
    do {                                                                        \
        if (bs == 32 && d == 32) { using I = TileIndex<32, 32>; return EXPR; }  \
        if (bs == 32 && d == 64) { using I = TileIndex<32, 64>; return EXPR; }  \
        if (bs == 32 && d == 96) { using I = TileIndex<32, 96>; return EXPR; }  \
        if (bs == 32 && d == 128) { using I = TileIndex<32, 128>; return EXPR; } \
        if (bs == 64 && d == 32) { using I = TileIndex<64, 32>; return EXPR; }  \
        if (bs == 64 && d == 64) { using I = TileIndex<64, 64>; return EXPR; }  \
        if (bs == 64 && d == 96) { using I = TileIndex<64, 96>; return EXPR; }  \
        if (bs == 64 && d == 128) { using I = TileIndex<64, 128>; return EXPR; } \
        return 0xffffffffu;                                                     \
    } while (0)

extern "C" {

uint32_t ti_const(int bs, int d, int which) {
    DISPATCH(bs, d, (uint32_t)(which == 0 ? I::NW : which == 1 ? I::SLICES : which == 2 ? (int)I::PARTIAL
                             : which == 3 ? I::SLICE_BYTES : which == 4 ? I::TILE_BYTES : which == 5 ? I::GROUPS
                             : I::LOADS));
}
uint32_t ti_swz(int bs, int d, uint32_t row) { DISPATCH(bs, d, I::swz(row)); }
uint32_t ti_lane_source(int bs, int d, uint32_t lane, uint32_t odd, uint32_t row_bytes) {
    DISPATCH(bs, d, I::lane_source(lane, odd, row_bytes));
}
uint32_t ti_lane_source_part(int bs, int d, uint32_t lane, uint32_t odd, uint32_t row_bytes) {
    DISPATCH(bs, d, I::lane_source_part(lane, odd, row_bytes));
}
uint32_t ti_lane_source_by_halves(int bs, int d, uint32_t lane, uint32_t odd, uint32_t row_bytes) {
    DISPATCH(bs, d, I::lane_source_by_halves(lane, odd, row_bytes));
}
uint32_t ti_lane_source_ragged(int bs, int d, uint32_t lane, uint32_t odd, uint32_t row_bytes, uint32_t nch) {
    DISPATCH(bs, d, I::lane_source_ragged(lane, odd, row_bytes, nch));
}
uint32_t ti_last_slice_chunks(int bs, int d, uint32_t hd) { DISPATCH(bs, d, I::last_slice_chunks(hd)); }
uint32_t ti_load_group(int bs, int d, int i, uint32_t wave) { DISPATCH(bs, d, I::load_group(i, wave)); }
uint32_t ti_load_group_odd(int bs, int d, int i, uint32_t wave) { DISPATCH(bs, d, I::load_group_odd(i, wave)); }
int ti_once_inst_offset(int bs, int d, int i) { DISPATCH(bs, d, I::once_inst_offset(i)); }
uint32_t ti_once_lane_offset(int bs, int d, uint32_t lane, int i, uint32_t wave, uint32_t row_bytes) {
    DISPATCH(bs, d, I::once_lane_offset(lane, i, wave, row_bytes));
}
uint32_t ti_once_base(int bs, int d, uint32_t wave, uint32_t row_bytes) { DISPATCH(bs, d, I::once_base(wave, row_bytes)); }
uint32_t ti_once_m0(int bs, int d, uint32_t wave) { DISPATCH(bs, d, I::once_m0(wave)); }
uint32_t ti_staged_source(int bs, int d, uint32_t lane, uint32_t row_bytes) { DISPATCH(bs, d, I::staged_source(lane, row_bytes)); }
uint32_t ti_staged_lds_offset(int bs, int d, uint32_t lane, uint32_t odd) { DISPATCH(bs, d, I::staged_lds_offset(lane, odd)); }
uint32_t ti_k_lane_base(int bs, int d, uint32_t qn, uint32_t half) { DISPATCH(bs, d, I::k_lane_base(qn, half)); }
uint32_t ti_k_frag_offset(int bs, int d, uint32_t lane_base, int kt, int ks) {
    DISPATCH(bs, d, I::k_frag_offset(lane_base, kt, ks));
}
uint32_t ti_v_lane_base(int bs, int d, uint32_t lane) { DISPATCH(bs, d, I::v_lane_base(lane)); }
uint32_t ti_v_frag_offset(int bs, int d, uint32_t lane_base, int mt, int u, int x) {
    DISPATCH(bs, d, I::v_frag_offset(lane_base, mt, u, x));
}

// sparse-block slabs and counted waits; elem_bytes = 2 (bf16) or 4 (fp32)
int ti_slab_passes(int elem_bytes) { return elem_bytes == 2 ? RowSlabIndex<64, 2>::PASSES : RowSlabIndex<64, 4>::PASSES; }
int ti_sdd_wait_count(int elem_bytes) { return elem_bytes == 2 ? SddStreamWait<2>::COUNT : SddStreamWait<4>::COUNT; }
int ti_sdd_wait_loads(int elem_bytes) { return elem_bytes == 2 ? SddStreamWait<2>::LOADS : SddStreamWait<4>::LOADS; }
int ti_dsd_wait_count() { return DsdStreamWait::COUNT; }
int ti_dsd_depth() { return DsdStreamWait::DEPTH; }
int ti_dsd_p_loads() { return DsdStreamWait::P_LOADS; }
int ti_dsd_v_loads() { return DsdStreamWait::V_LOADS; }

}  // extern "C"
