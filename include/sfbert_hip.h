/*
 * libsfbert_hip -- C ABI of the MI355X (gfx950) block-sparse attention path.
 *
 * Plain pointers and sizes only.  Device pointers are marked [dev], host pointers [host].  Every
 * device entry point enqueues work on the given HIP stream and returns without synchronising.  The
 * attention and layer-op entry points allocate nothing and keep no state.  The GEMM entry points
 * (sfb_gemm*, sfb_encoder_layer_forward*, sfb_model_forward) go through rocBLAS / hipBLASLt: the
 * library keeps one handle of each per process and one plan per GEMM problem, made on first use
 * behind one mutex and kept until sfb_gemm_release(); making a plan times the library's candidate
 * kernels on the caller's operands, which synchronises with the stream once (skipped when the
 * stream is being captured into a graph).  Tensors Q/K/V/O are [batch, ctx, heads, head_state]
 * contiguous (element offset b*ctx*H*d + token*H*d + h*d + k), sparse S/P tensors are
 * [batch][heads][blocks][bs][bs], exactly as the reference lays them out
 * (openai_blocksparse.h:40-41,148).  Each declaration cites the reference interface it replaces.
 *
 * All functions return an sfb_status (0 = ok) unless stated otherwise.
 */
#ifndef SFBERT_HIP_H
#define SFBERT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The reference's CUDA uint2 LUT entry (openai_blocksparse.h:203) as a plain POD. */
typedef struct { uint32_t x, y; } sfb_uint2;

/* hipStream_t, passed as an opaque pointer (the reference passes CUstream, openai_blocksparse.h:202). */
typedef void* sfb_stream_t;

typedef enum {
    SFB_OK = 0,
    SFB_ERR_NULL_POINTER = 1,   /* a required pointer is NULL */
    SFB_ERR_BLOCK_SIZE = 2,     /* block size not supported by this entry point */
    SFB_ERR_HEAD_STATE = 3,     /* head_state (d) not supported */
    SFB_ERR_SHAPE = 4,          /* zero / inconsistent dimensions */
    SFB_ERR_DTYPE = 5,          /* unknown or unsupported element type */
    SFB_ERR_ALIGNMENT = 6,      /* a tensor pointer is not 16-byte aligned */
    SFB_ERR_LAUNCH = 7,         /* hipGetLastError() reported a failure after the launch */
    SFB_ERR_ARGUMENT = 8,       /* other invalid argument (op code, pattern parameter ...) */
    SFB_ERR_WORKSPACE = 9,      /* workspace missing or too small */
    SFB_ERR_SCRATCH_LIMIT = 10  /* the launch needs more scratch than the library's static device array holds */
} sfb_status;

typedef enum { SFB_F32 = 0, SFB_BF16 = 1 } sfb_dtype;

/* NT_OP / NN_OP / TN_OP of gpu_types.h:135-137 */
enum { SFB_NT_OP = 0, SFB_NN_OP = 1, SFB_TN_OP = 2 };

const char* sfb_status_string(int status);
/* 1 when the library was built for gfx950 and a HIP device is usable, else 0. */
int sfb_device_available(void);

/* ================================================================================================
 * Host-side descriptors (integer work on [host] arrays; bit-exact with the reference's formats)
 * ============================================================================================== */

/* layout[heads][nb][nb], 1 = (query block row, key block column) attended. */
/* no_fusion_test.cu:47-62 (causal != 0: i >= j; causal == 0: dense). */
int sfb_layout_full(uint32_t* layout, int nb, int causal);
/* local_fusion_test.cu:46-63 (bidirectional == 0: the reference's causal band; != 0: |i-j| <= extra_diag). */
int sfb_layout_local(uint32_t* layout, int nb, int extra_diag, int bidirectional);
/* fixed_fusion_test.cu:52-106: per-head summary column phase stride-(h+1), own chunk, optional causal cut. */
int sfb_layout_fixed(uint32_t* layout, int heads, int nb, int stride, int causal);
/* stride_fusion_test.cu:48-71: j <= i && j + (i % block_chunks) >= i. */
int sfb_layout_strided_chunks(uint32_t* layout, int nb, int block_chunks);
/* Block form of the element rule ewops.h:462-503: band of `band` blocks plus (i-j) % stride == 0. */
int sfb_layout_strided(uint32_t* layout, int nb, int band, int stride, int causal);
/* big_bird_fusion_test.cu:50-99: window, `nglobal` dense rows+columns (first ones, or split between both
 * ends), plus rand_cols[nb][nrand] random key blocks per row (-1 = none; NULL = no random blocks). */
int sfb_layout_bigbird(uint32_t* layout, int nb, int window, int nglobal, int global_both_ends,
                       const int32_t* rand_cols, int nrand);
/* Seeded replacement of the reference's unseeded rand()%10 draw (big_bird_fusion_test.cu:81-99):
 * nrand distinct still-empty columns per block-row, splitmix64 + partial Fisher-Yates. */
int sfb_bigbird_draw(int32_t* rand_cols, int nb, int window, int nglobal, int global_both_ends,
                     int nrand, uint64_t seed);

/* local_fusion_test.cu:78-85: number of nonzero blocks of one head's layout. */
uint32_t sfb_count_blocks(const uint32_t* layout, int nb);
/* local_fusion_test.cu:89-99: nt_lut[blocks] = {row block, col block}, row-major scan. */
int sfb_build_nt_lut(sfb_uint2* nt_lut, const uint32_t* layout, int nb);
/* local_fusion_test.cu:106-133: nn_lut[nb + blocks]; *nn_max is read as the initial value and updated. */
int sfb_build_nn_lut(sfb_uint2* nn_lut, const sfb_uint2* nt_lut, uint32_t blocks, int nb,
                     uint32_t* nn_max);
/* local_fusion_test.cu:229-237: rblk_lut[blocks] = {block id, row block}. */
int sfb_build_rblk_lut(sfb_uint2* rblk_lut, const sfb_uint2* nn_lut, int nb);
/* TN look-up table of the backward products dV = P^T dO and dK = dS^T Q
 * (transformer_attention_optimize.cu:924, 948 pass it as tn_ptr; the reference's builder survives only as the
 * commented causal case generate_tn_lut, ewops.h:675-701): tn_lut[nb + blocks], per key-block column a
 * header {offset, count} with offsets starting at nb, then that column's blocks in ascending row order as
 * {block id in NT order, row block}.  *tn_max (may be NULL) receives the largest count. */
int sfb_build_tn_lut(sfb_uint2* tn_lut, const sfb_uint2* nt_lut, uint32_t blocks, int nb, uint32_t* tn_max);
/* blocksparse.h:1016-1043 */
void sfb_magicu64(uint32_t d, uint32_t* magic, uint32_t* shift);

/* Element masks, keep[blocks][bs][bs] bytes. kind: 0 all ones; 1 diagonal blocks lower-triangular
 * (no_fusion_test.cu:124-143); 2 local rule (local_fusion_test.cu:146-175); 3 every block
 * lower-triangular (stride_fusion_test.cu:141-160). */
int sfb_element_mask(uint8_t* keep, const sfb_uint2* nt_lut, uint32_t blocks, int bs, int kind,
                     int local_attn_ctx);
/* no_fusion_test.cu:145-157: block-major words[blk*bs + row], bit j = keep key column j.
 * Word type follows blocksparse.h:684-720: uint8 / uint16 / uint32 / uint64 for bs 8 / 16 / 32 / 64. */
int sfb_pack_mask(void* words, const uint8_t* keep, uint32_t blocks, int bs);
/* no_fusion_test.cu:159-163: row-major words[row*blocks + blk] for the unfused softmax. */
int sfb_transpose_mask(void* row_major, const void* block_major, uint32_t blocks, int bs);

/* MI355X addition (no reference counterpart): launch order of block-rows, longest first, ties by
 * ascending row; row_order[nb].  Passing it to the fused entry points is optional. */
int sfb_build_row_order(uint32_t* row_order, const sfb_uint2* nn_lut, int nb);

/* MI355X addition (no reference counterpart): work items of a scheduled fused launch.  Block-rows
 * with more than max_blocks key blocks (BigBird's global rows) are cut into ceil(count/max_blocks)
 * chunks of near-equal length so that no work-group walks a long row alone; the chunks' partial
 * results are merged by whichever chunk finishes last.  Items are sorted longest first. */
typedef struct {
    uint32_t row;      /* query block row */
    uint32_t first;    /* first key block of this item, relative to the row's NN-LUT segment */
    uint32_t count;    /* number of key blocks of this item */
    uint32_t nchunks;  /* chunks the row was cut into (1 = whole row) */
    uint32_t chunk;    /* index of this chunk within the row */
    uint32_t slot;     /* index of the row among split rows (arrival counter), 0 if not split */
    uint32_t part;     /* index of the row's first partial-result record, 0 if not split */
    uint32_t lut_first; /* index of the item's first entry in the NN LUT: nn_lut[row].x + first */
} sfb_work_item;
/* items may be NULL to query the counts; otherwise it must hold *n_items entries as returned by a
 * query call.  n_slots = number of split rows, n_parts = total chunks of split rows, n_heavy = number
 * of leading items with at least twice the median number of key blocks (launched for all heads
 * before the rest; always < n_items). */
int sfb_build_schedule(sfb_work_item* items, uint32_t* n_items, uint32_t* n_heavy, uint32_t* n_slots,
                       uint32_t* n_parts, const sfb_uint2* nn_lut, int nb, uint32_t max_blocks);
/* The same for one layout per head (lut_heads tables of lut_dim entries, the reference's `fixed` pattern,
 * fixed_fusion_test.cu:38-39): items [lut_heads][*n_items], every head's list longest first and filled up to the
 * longest list's length with items whose row is SFB_WORK_ITEM_SKIP (no work).  A query call (items NULL) returns
 * that length in *n_items; the filling call takes the stride of the array in *n_items and leaves it unchanged.
 * n_slots and n_parts are the largest any head needs (the workspace is laid out per (batch, head)), n_heavy the
 * number of leading ranks that are heavy in every head.  For sfb_fused_attention_scheduled_heads. */
#define SFB_WORK_ITEM_SKIP 0xffffffffu
int sfb_build_schedule_heads(sfb_work_item* items, uint32_t* n_items, uint32_t* n_heavy, uint32_t* n_slots,
                             uint32_t* n_parts, const sfb_uint2* nn_lut, int nb, uint32_t lut_heads, uint32_t lut_dim,
                             uint32_t max_blocks);
/* MI355X addition: a max_blocks for sfb_build_schedule that suits a launch over batch_heads = batch x heads
 * (batch, head) pairs: 1.25 x the key blocks one of the device's 1024 resident work-group slots gets to process in
 * the whole launch, at least 16.  (BigBird L = 4096, 12 heads: 16 for one sequence, 19 for two, 37 -- global rows cut in
 * two -- for four, no cut from eight on.) */
uint32_t sfb_suggest_max_blocks(const sfb_uint2* nn_lut, int nb, uint32_t batch_heads);
/* Bytes of the [dev] workspace a scheduled launch needs: arrival counters + partial records.  The
 * workspace must be zero-filled once before its first use; launches leave the counters at zero. */
size_t sfb_schedule_workspace_bytes(uint32_t n_slots, uint32_t n_parts, uint32_t batch_dim,
                                    uint32_t head_dim, uint32_t block_size, uint32_t state_dim);

/* MI355X addition (no reference counterpart): streams of a launch whose work-groups stay resident.  Instead of
 * one work-group per work item, wg_slots work-groups (sfb_resident_work_groups(): as many as the device runs at once)
 * each walk one stream of key blocks that strings its work items together, so that the tiles, the queries and the
 * descriptors of an item are fetched while its predecessor is still being computed and no work-group is dispatched
 * in the middle of the launch.  The streams are made to cost the same (key blocks plus charges per item, partial
 * record and merge): block-rows are placed whole, longest first, on the least loaded stream; rows too long for that
 * (BigBird's global rows) are cut and poured into the streams up to the common level.  The chunks of a cut row
 * stand first in their streams and leave partial records (unnormalised output, maxima, sum) in a workspace, each
 * followed by a flag; one stream ends with the row's merge task, which finds the flags set, adds the records and
 * writes the row.  Streams of one die (slot index mod 8) only hold (batch, head) pairs of the same residue mod 8,
 * so that a head's K and V stay in one L2.  All of it is one blob, built on the host and copied to the device. */
typedef struct {
    uint32_t kv_off;   /* ((batch * ctx + key column * block_size) * heads + head): first key row of the block, in rows of head_state elements */
    uint32_t info;     /* SFB_STREAM_BLOCK_INDEX: index of the block in the layout (mask words); SFB_STREAM_FIRST / _LAST: first / last block of its item */
    uint32_t col;      /* key block column */
    uint32_t q_off;    /* first block of an item: the item's q_off (its queries are requested two blocks ahead); else 0 */
} sfb_stream_block;
#define SFB_STREAM_BLOCK_INDEX 0x0fffffffu
#define SFB_STREAM_FIRST 0x40000000u
#define SFB_STREAM_LAST 0x80000000u
typedef struct {
    uint32_t q_off;      /* ((batch * ctx + row * block_size) * heads + head): first query row, same unit as kv_off */
    uint32_t batch, head, row;
    uint32_t kind;       /* 0: the whole block-row, written to O; 1: chunk of a cut row, leaves partial record `part` */
    uint32_t part;
    uint32_t lse_off;    /* (batch * heads + head) * ctx + row * block_size: the row's first query in the lse output */
    uint32_t lut_first;  /* index of the item's first entry in the head's NN LUT */
    uint32_t count;      /* key blocks */
    uint32_t first;      /* first key block, relative to the row's LUT segment */
    uint32_t nchunks, chunk;
    uint32_t reserved[4];   /* items are 64 bytes */
} sfb_stream_item;
typedef struct {
    uint32_t q_off, batch, head, row;
    uint32_t part;       /* first partial record of the row */
    uint32_t nparts;     /* number of records to add; 0: the row has no key blocks and is written as zeros */
    uint32_t reserved[2];
} sfb_stream_merge;
typedef struct {
    uint32_t block_begin, n_blocks;   /* this work-group's run of sfb_stream_block entries */
    uint32_t item_begin, n_items;     /* ... of sfb_stream_item entries, in the order their blocks appear */
    uint32_t merge_begin, n_merges;   /* ... of sfb_stream_merge entries, done after the stream */
    uint32_t reserved[2];
} sfb_stream_slot;
typedef struct {
    uint32_t wg_slots, n_blocks, n_items, n_merges;
    uint32_t n_parts;                 /* partial records (and flags) the launch uses */
    uint32_t block_size, batch_dim, head_dim, ctx_blks;   /* what the streams were built for */
    float balance;                    /* mean stream cost / largest stream cost, over the resident streams */
    uint32_t resident;                /* the first `resident` streams are the long ones (one per resident work-group) */
    uint64_t slots_offset, blocks_offset, items_offset, merges_offset;   /* byte offsets of the four arrays in the blob */
    uint64_t total_bytes;             /* size of the blob */
} sfb_stream_plan;
/*   nn_lut [host] lut_heads tables of lut_dim entries (lut_heads = 1: one layout for all heads; = head_dim:
 *   per-head layouts as fixed_fusion_test.cu:38-39 builds them).  blob [host] NULL: only *plan (sizes) is filled;
 *   otherwise blob_bytes >= plan->total_bytes as returned by such a call.
 *   wg_slots: work-groups of the launch; at most sfb_resident_work_groups_for() if every merge is to find its records'
 *   producers running (more slots than that still give correct results as long as no bounded wait runs out, which
 *   sfb_stream_status() reports).  level != 0: cut rows are poured into the streams up to a common level (pieces of
 *   any length from 2 blocks up); 0: cut into equal pieces of at least 2 blocks, placed like whole rows.
 *   tail_percent (0..90, used with level = 0): that share of every stream's cost is held back and handed, as
 *   additional short streams of one row or one merge beyond the first plan->resident ones, to whichever work-group
 *   slots free up first; 0: none. */
int sfb_build_stream(sfb_stream_plan* plan, void* blob, size_t blob_bytes, const sfb_uint2* nn_lut, int nb,
                     uint32_t lut_heads, uint32_t lut_dim, uint32_t batch_dim, uint32_t head_dim, uint32_t block_size,
                     uint32_t wg_slots, int level, uint32_t tail_percent);
/* Bytes of the [dev] workspace a streamed launch needs: one flag per partial record, the records, a status word.
 * The workspace must be zero-filled once before its first use; a launch whose merges all found their records
 * (sfb_stream_status() == 0) leaves the flags at zero.  After a launch that reports status 1 the flags of the rows
 * it gave up on are still set (their producers set them after the merge had left) and the status word stays 1:
 * the workspace must be cleared with sfb_stream_reset() before the next launch uses it, or that launch would add
 * records its producers have not written yet. */
size_t sfb_stream_workspace_bytes(const sfb_stream_plan* plan, uint32_t state_dim);
/* How the bf16 kernels apply `scale` in launches without mask, key padding and log-sum-exp output (host helper, no
 * device needed): scale * log2(e) = *pow2 * *rest with *pow2 a power of two and *rest in [1/sqrt(2), sqrt(2)).  The
 * queries are multiplied by *pow2, which is exact in bf16, so the score product delivers base-2 exponents up to the
 * factor *rest, applied in fp32 per score: p = exp2((s - offset) * rest) follows ewops.h:86's exp((s - max) * scale)
 * without a second rounding of the queries. */
void sfb_scale_parts(float scale, float* pow2, float* rest);
/* Clears the flags and the status word of a streamed launch's workspace (fill kernels on `stream`; the partial
 * records need no clearing).  Also usable instead of the initial zero-fill. */
int sfb_stream_reset(sfb_stream_t stream, const sfb_stream_plan* plan, uint32_t state_dim, void* workspace);
/* Work-groups the current device keeps resident of the kernel that a streamed launch with these tensors runs
 * (asked of the runtime for that kernel: 4 per compute unit for head sizes up to 64, 2 for 96 and 128, whose tiles
 * take twice the LDS); masked != 0: the launch has an element mask, key padding or a log-sum-exp output.  This is
 * the wg_slots for which every merge finds its records' producers running.  0 without a device. */
uint32_t sfb_resident_work_groups_for(int in_dtype, uint32_t block_size, uint32_t state_dim, int masked);
/* The same for bf16 tensors, blocks of 64 and head size 64 without mask. */
uint32_t sfb_resident_work_groups(void);

/* ================================================================================================
 * Device entry points
 * ============================================================================================== */

/* state_dim (the head size d).  Every attention entry point takes every multiple of 4 (fp32 tensors) or 8 (bf16
 * tensors: rows are whole 16-byte vectors) up to 128 -- the reference's `d % 4 == 0` of its K64 = false paths,
 * openai_blocksparse.h:221-222: the fused forward (plain, scheduled and streamed launches), the products of the unfused path
 * (sfb_sdd_nt, sfb_dsd_xn, sfb_fused_sdd_softmax, sfb_sdd_softmax_grad, sfb_row_dot) and the fused backward.  32, 64,
 * 96 and 128 are what the kernels' tiles divide; a size between them runs the kernel of the next multiple of 32 with
 * the missing features read as zeros and only d output columns stored.  sfb_fused_sdd_softmax_split (the per-block
 * comparison kernel) takes 64 only.  Anything else returns SFB_ERR_HEAD_STATE. */

/* Fully fused attention: O = softmax_rows(scale * Q K^T restricted to layout & mask & key<valid_len) V,
 * one work-group per (batch, head, block-row), no S/P in memory.  Replaces the sequence
 * bst_sgemm_nt -> BlocksparseMaskedSoftmax -> bst_sgemm_xn (transformer_attention_optimize.cu:728-748)
 * and the unfinished fusion_attention / fusion_kernel (fusion_blocksparse.h:2518-3050); arithmetic
 * follows the CPU path (matmul.h:53-78, ewops.h:64-98, matmul.h:6-20).
 *   q,k,v [dev]  in_dtype (SFB_F32 or SFB_BF16);  o [dev] fp32
 *   nn_lut [dev] lut_heads * lut_dim entries, lut_dim = ctx_blks + blocks
 *   mask [dev]   block-major words (uint32 for bs 32, uint64 for bs 64), NULL = all ones
 *   valid_len [dev] int32[batch] keys >= valid_len[b] are masked, NULL = none (MI355X addition)
 *   row_order [dev] uint32[ctx_blks] from sfb_build_row_order, NULL = descending row index */
int sfb_fused_attention(sfb_stream_t stream, const void* q, const void* k, const void* v, float* o,
                        int in_dtype, const sfb_uint2* nn_lut, const void* mask,
                        const int32_t* valid_len, const uint32_t* row_order, uint32_t block_size,
                        uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                        uint32_t state_dim, uint32_t lut_heads, uint32_t lut_dim, uint32_t mask_heads,
                        float scale);

/* The same operation launched over sfb_build_schedule's work items (one layout shared by all heads).
 *   items [dev] n_items entries;  workspace [dev] 256-byte aligned, sfb_schedule_workspace_bytes()
 *   bytes, zero-filled before first use (may be NULL when n_parts == 0).  Launches that share a
 *   workspace must be ordered on one stream. */
int sfb_fused_attention_scheduled(sfb_stream_t stream, const void* q, const void* k, const void* v,
                                  float* o, int in_dtype, const sfb_uint2* nn_lut, const void* mask,
                                  const int32_t* valid_len, const sfb_work_item* items,
                                  uint32_t n_items, uint32_t n_heavy, uint32_t n_slots, uint32_t n_parts,
                                  void* workspace, size_t workspace_bytes, uint32_t block_size,
                                  uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks,
                                  uint32_t head_dim, uint32_t state_dim, uint32_t mask_heads,
                                  float scale);
/* The same launch with the output element type chosen by the caller: o [dev] [batch, ctx, heads, state] of
 * out_dtype (SFB_F32 or SFB_BF16).  bf16 output is the fp32 result rounded once to nearest even; it feeds a bf16
 * GEMM (the layer's output projection) without a separate conversion pass. */
int sfb_fused_attention_scheduled_to(sfb_stream_t stream, const void* q, const void* k, const void* v,
                                  void* o, int in_dtype, int out_dtype, const sfb_uint2* nn_lut, const void* mask,
                                  const int32_t* valid_len, const sfb_work_item* items,
                                  uint32_t n_items, uint32_t n_heavy, uint32_t n_slots, uint32_t n_parts,
                                  void* workspace, size_t workspace_bytes, uint32_t block_size,
                                  uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks,
                                  uint32_t head_dim, uint32_t state_dim, uint32_t mask_heads,
                                  float scale);
/* sfb_fused_attention_scheduled_to with one look-up table (and work-item list) per head: nn_lut [dev] lut_heads
 * tables of lut_dim = ctx_blks + blocks entries, items [dev] [lut_heads][n_items] from sfb_build_schedule_heads;
 * lut_heads = head_dim (or 1, which is the plain scheduled launch); lse may be NULL. */
int sfb_fused_attention_scheduled_heads(sfb_stream_t stream, const void* q, const void* k, const void* v, void* o,
                                        float* lse, int in_dtype, int out_dtype, const sfb_uint2* nn_lut,
                                        const void* mask, const int32_t* valid_len, const sfb_work_item* items,
                                        uint32_t n_items, uint32_t n_heavy, uint32_t n_slots, uint32_t n_parts,
                                        void* workspace, size_t workspace_bytes, uint32_t block_size, uint32_t blocks,
                                        uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                        uint32_t lut_heads, uint32_t lut_dim, uint32_t mask_heads, float scale);
/* sfb_fused_attention_scheduled_to for Q, K and V whose token rows are token_stride elements apart instead of
 * head_dim * state_dim (o stays dense): q, k, v may then be column slices of one [batch * ctx, token_stride] matrix,
 * e.g. of the result of one merged Q/K/V projection (transformer.cpp:516-522 does three products).  token_stride >=
 * head_dim * state_dim and a multiple of 8 (bf16) or 4 (fp32) elements; q, k, v 16-byte aligned. */
int sfb_fused_attention_scheduled_strided(sfb_stream_t stream, const void* q, const void* k, const void* v, void* o,
                                          int in_dtype, int out_dtype, const sfb_uint2* nn_lut, const void* mask,
                                          const int32_t* valid_len, const sfb_work_item* items, uint32_t n_items,
                                          uint32_t n_heavy, uint32_t n_slots, uint32_t n_parts, void* workspace,
                                          size_t workspace_bytes, uint32_t block_size, uint32_t blocks,
                                          uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                          uint32_t token_stride, uint32_t mask_heads, float scale);
/* No counterpart in the reference.  For callers that cannot allocate device memory or pass a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The same launch as
 * sfb_fused_attention_scheduled_to, with the arrival counters and partial records of split rows kept in a static
 * device array of SFB_STATIC_SCRATCH_BYTES inside the library (each device the library runs on holds one until the
 * process ends) instead of a caller's workspace; the call allocates nothing.  A launch whose
 * sfb_schedule_workspace_bytes() exceeds SFB_STATIC_SCRATCH_BYTES returns SFB_ERR_SCRATCH_LIMIT (BigBird L = 4096,
 * 12 heads, head size 64 needs 0.8 MiB per sequence while its global rows are cut, nothing from 8 sequences on).
 * All calls on one device share the array: calls that overlap in time on one device (two streams, two threads)
 * race and must be ordered by the caller. */
#define SFB_STATIC_SCRATCH_BYTES (8u << 20)
size_t sfb_static_scratch_bytes(void);
int sfb_fused_attention_scheduled_noalloc(sfb_stream_t stream, const void* q, const void* k, const void* v, void* o,
                                          int in_dtype, int out_dtype, const sfb_uint2* nn_lut, const void* mask,
                                          const int32_t* valid_len, const sfb_work_item* items, uint32_t n_items,
                                          uint32_t n_heavy, uint32_t n_slots, uint32_t n_parts, uint32_t block_size,
                                          uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                                          uint32_t state_dim, uint32_t mask_heads, float scale);

/* The same launch for a training step: additionally writes lse [dev] fp32 [batch][heads][ctx], the base-2
 * logarithm of each query row's softmax denominator in units where the normalised probability of a key with raw
 * score s is exp2(s * scale * log2(e) - lse).  sfb_fused_attention_backward rebuilds P from it. */
int sfb_fused_attention_scheduled_lse(sfb_stream_t stream, const void* q, const void* k, const void* v, void* o,
                                      float* lse, int in_dtype, int out_dtype, const sfb_uint2* nn_lut,
                                      const void* mask, const int32_t* valid_len, const sfb_work_item* items,
                                      uint32_t n_items, uint32_t n_heavy, uint32_t n_slots, uint32_t n_parts,
                                      void* workspace, size_t workspace_bytes, uint32_t block_size, uint32_t blocks,
                                      uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                      uint32_t mask_heads, float scale);

/* The same operation launched over sfb_build_stream's streams: plan->wg_slots resident work-groups, each walking
 * its stream (bf16 tensors with head size 64: tiles, queries and descriptors of the next item in flight while an
 * item is computed; other cases: item after item).  Takes per-head look-up tables and masks (lut_heads, mask_heads
 * = head_dim) as well as shared ones.  plan [host] as sfb_build_stream filled it, blob [dev] a copy of the blob;
 * lse may be NULL; out_dtype SFB_F32 or SFB_BF16; workspace [dev] sfb_stream_workspace_bytes() bytes, 256-byte
 * aligned.  A merge task waits for the flags of its records with a bounded number of polls (their producers stand
 * first in their streams, so they are set long before); if the launch has more work-groups than the device keeps
 * resident and a wait runs out, the row is left unwritten and the workspace's status word is set to 1: sfb_stream_status() reads it after the stream has been synchronised. */
int sfb_fused_attention_streamed(sfb_stream_t stream, const void* q, const void* k, const void* v, void* o, float* lse,
                                 int in_dtype, int out_dtype, const sfb_uint2* nn_lut, const void* mask,
                                 const int32_t* valid_len, const sfb_stream_plan* plan, const void* blob,
                                 void* workspace, size_t workspace_bytes, uint32_t block_size, uint32_t blocks,
                                 uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                                 uint32_t lut_heads, uint32_t lut_dim, uint32_t mask_heads, float scale);
/* Status word of a streamed launch's workspace (synchronous copy from the device): 0 = every merge found its
 * records, 1 = a wait ran out, negative = the copy failed. */
int sfb_stream_status(const sfb_stream_plan* plan, uint32_t state_dim, const void* workspace);

/* MI355X addition: the whole backward of the attention in one pass over the blocks, with P, dP and dS kept on chip.  Same
 * arithmetic as the reference's sequence TN, NT, softmax gradient, TN, NN (transformer_attention_optimize.cu:
 * 924-965; ewops.h:101-124; matmul.h:81-99): P = exp2(S scale log2e - lse), dV = P^T dO, dS = P (dO V^T - delta)
 * scale, dK = dS^T Q, dQ = dS K, where delta = rowsum(dO * O) (computed here into the caller's buffer) stands for
 * the gradient's sum over the sparse row.  q, k, v, d_out [dev] bf16 or fp32 (dtype; fp32 tensors get true fp32
 * products) [batch, ctx, heads, state_dim], state_dim a multiple of 8 (bf16) or 4 (fp32) up to 128; o [dev] fp32, the
 * forward output; lse [dev] from sfb_fused_attention_scheduled_lse; delta [dev] fp32 [batch][heads][ctx]
 * (scratch, overwritten); dq, dk, dv [dev] fp32; nn_lut, tn_lut [dev]: one layout for all heads (lut_heads 1), or
 * one table per head, lut_dim = ctx_blks + blocks entries apart, every head with the same number of blocks
 * (lut_heads = head_dim; then without work items: every line is done whole); mask block-major, one for all
 * heads or one per head (mask_heads).  row_items / col_items [dev] (may be NULL: one work-group per block-row / block-column in index
 * order): work items of sfb_build_schedule over nn_lut / over tn_lut, longest first, with lines of more than
 * max_blocks blocks cut into chunks; the chunks of a split line write partial records into workspace ([dev],
 * 256-byte aligned, sfb_backward_workspace_bytes() bytes; n_*_parts as returned by sfb_build_schedule) and a
 * follow-up kernel adds them in chunk order, so results do not depend on timing. */
size_t sfb_backward_workspace_bytes(uint32_t n_row_parts, uint32_t n_col_parts, uint32_t batch_dim,
                                    uint32_t head_dim, uint32_t block_size, uint32_t state_dim);
int sfb_fused_attention_backward(sfb_stream_t stream, const void* q, const void* k, const void* v, const float* o,
                                 const void* d_out, const float* lse, float* delta, float* dq, float* dk, float* dv,
                                 int dtype, const sfb_uint2* nn_lut, const sfb_uint2* tn_lut, const void* mask,
                                 const int32_t* valid_len, const sfb_work_item* row_items, uint32_t n_row_items,
                                 uint32_t n_row_heavy, uint32_t n_row_parts, const sfb_work_item* col_items,
                                 uint32_t n_col_items, uint32_t n_col_heavy, uint32_t n_col_parts, void* workspace,
                                 size_t workspace_bytes, uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                                 uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim, uint32_t lut_heads,
                                 uint32_t lut_dim, uint32_t mask_heads, float scale);


/* ---- the unfused trio (kept as the no_fusion comparison) ------------------------------------ */

/* bst_sgemm_nt (openai_blocksparse.h:202-233; blocksparse.h:425): S_blk = A_rowblk . B_colblk^T for
 * every entry of the NT LUT.  a, b [dev] [batch, ctx, heads, state] of in_dtype; c [dev] sparse
 * [batch][heads][blocks][bs][bs] of out_dtype (the reference stores bf16; fp32 is offered so the fp32
 * configurations keep fp32 scores).  lut_dim = blocks.  Unsupported block sizes are an error, not the
 * reference's silent no-op (openai_blocksparse.h:225-232). */
int sfb_sdd_nt(sfb_stream_t stream, const sfb_uint2* lut, const void* a, const void* b, void* c,
               int in_dtype, int out_dtype, uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
               uint32_t ctx_blks_a, uint32_t ctx_blks_b, uint32_t head_dim, uint32_t state_dim,
               uint32_t lut_heads, uint32_t lut_dim);

/* BlocksparseMaskedSoftmax<T,V> (blocksparse.h:649-722): y = softmax over each sparse row of x.
 * block_size 8, 16, 32 or 64 (blocksparse.h:684-720; the matrix products take 32 and 64 only).
 * lut = NN LUT, lut_dim = ctx_blks + blocks; mask [dev] ROW-major words[row*blocks + blk] (uint8 / uint16 /
 * uint32 / uint64 for bs 8 / 16 / 32 / 64) or NULL; valid_len [dev] int32[batch] or NULL (MI355X addition); scale is
 * the raw 1/sqrt(d) -- log2(e) is folded inside, as blocksparse.h:669 does.  max_lut is accepted for
 * signature compatibility.  Numerics follow the CPU softmax (ewops.h:64-98), not the reference GPU
 * kernel's approximations. */
int sfb_masked_softmax(sfb_stream_t stream, const sfb_uint2* lut, const void* mask, const void* x,
                       void* y, int x_dtype, int y_dtype, const int32_t* valid_len, uint32_t block_size,
                       uint32_t blocks, uint32_t batch_dim, uint32_t head_dim, uint32_t ctx_blks,
                       uint32_t lut_heads, uint32_t lut_dim, uint32_t max_lut, uint32_t mask_heads,
                       float scale);

/* BlocksparseMaskedSoftmaxGrad<T,V> (blocksparse.h:1164-1228): dx = (dy - sum_k dy*y) * y * scale over each
 * sparse row (ewops.h:101-124; masked keys hold y = 0).  dy, y, dx [dev] in the sparse layout, all of
 * `dtype`; block_size 8, 16, 32 or 64; lut = NN LUT; max_lut is accepted for signature compatibility. */
int sfb_masked_softmax_grad(sfb_stream_t stream, const sfb_uint2* lut, const void* dy, const void* y, void* dx,
                            int dtype, uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
                            uint32_t head_dim, uint32_t ctx_blks, uint32_t lut_heads, uint32_t lut_dim,
                            uint32_t max_lut, float scale);

/* MI355X additions: the NT product dP = dO V^T and the softmax gradient of the backward pass
 * (transformer_attention_optimize.cu:936, 945) in one kernel, dS = (dO V^T - delta) * P * scale per block, where
 * delta[b][h][q] = sum_d dO[b][q][h][d] * O[b][q][h][d] (sfb_row_dot) replaces the gradient's sum over the sparse
 * row (ewops.h:108-113): the two are equal because O = P V.  dP is never written.  d_out, v [dev] [batch, ctx,
 * heads, state] of in_dtype; o [dev] fp32 (the forward output); p, ds [dev] sparse, of sparse_dtype; delta [dev]
 * fp32 [batch][heads][ctx]; nt_lut [dev]. */
int sfb_row_dot(sfb_stream_t stream, float* delta, const void* d_out, const float* o, int dtype, uint32_t batch_dim,
                uint32_t ctx, uint32_t head_dim, uint32_t state_dim);
int sfb_sdd_softmax_grad(sfb_stream_t stream, const sfb_uint2* nt_lut, const void* d_out, const void* v,
                         const void* p, const float* delta, void* ds, int in_dtype, int sparse_dtype,
                         uint32_t block_size, uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks,
                         uint32_t head_dim, uint32_t state_dim, uint32_t lut_heads, float scale);

/* bst_sgemm_xn (blocksparse.h:965-1014).  op = SFB_NN_OP: C_rowblk = sum over the row's blocks of
 * A_blk . B_colblk, lut = NN LUT.  op = SFB_TN_OP (the backward products dV = P^T dO, dK = dS^T Q;
 * matmul.h:81-99): C_colblk = sum over the column's blocks of A_blk^T . B_rowblk, lut = TN LUT.
 * a [dev] sparse operand of a_dtype; b [dev] [batch, ctx_b, heads, state] of b_dtype; c [dev] fp32
 * [batch, ctx_c, heads, state]; block-rows (columns) without blocks are zero-filled
 * (blocksparse.h:949-962).  The product runs on bf16 MFMA when the operands are bf16, on fp32 MFMA
 * otherwise.  magic/shift/max_lut are accepted for signature compatibility. */
int sfb_dsd_xn(sfb_stream_t stream, const sfb_uint2* lut, const void* a, const void* b, float* c,
               int a_dtype, int b_dtype, uint32_t block_size, uint32_t blocks, uint32_t batch_dim,
               uint32_t ctx_blks_b, uint32_t ctx_blks_c, uint32_t head_dim, uint32_t state_dim,
               uint32_t lut_heads, uint32_t lut_dim, uint32_t op, uint32_t magic, uint32_t shift,
               uint32_t max_lut);

/* MI355X addition (no reference counterpart): sfb_dsd_xn launched over work items instead of lines, so that no
 * work-group walks a long block-row (NN) or block-column (TN) alone -- BigBird's global rows and columns have 64 blocks
 * at L = 4096 against 8 elsewhere, and the work-group that owns one is the tail of the plain launch.  items [dev]:
 * sfb_build_schedule() over the same look-up table (the NN LUT for SFB_NN_OP, the TN LUT for SFB_TN_OP), or
 * [lut_heads][n_items] from sfb_build_schedule_heads() with one table per head; n_items, n_heavy, n_parts as returned
 * there.  The chunks of a cut line leave their sums in workspace ([dev], 256-byte aligned,
 * sfb_dsd_workspace_bytes() bytes, no initial contents needed; may be NULL when n_parts is 0) and a second small
 * kernel adds them in chunk order, so results do not depend on timing.  Both operands must have one type
 * (SFB_ERR_DTYPE otherwise); head sizes as for sfb_dsd_xn. */
size_t sfb_dsd_workspace_bytes(uint32_t n_parts, uint32_t batch_dim, uint32_t head_dim, uint32_t block_size,
                               uint32_t state_dim);
int sfb_dsd_xn_scheduled(sfb_stream_t stream, const sfb_uint2* lut, const void* a, const void* b, float* c,
                         int a_dtype, int b_dtype, const sfb_work_item* items, uint32_t n_items, uint32_t n_heavy,
                         uint32_t n_parts, void* workspace, size_t workspace_bytes, uint32_t block_size,
                         uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks_b, uint32_t ctx_blks_c,
                         uint32_t head_dim, uint32_t state_dim, uint32_t lut_heads, uint32_t lut_dim, uint32_t op);

/* fusion_attention1 / fusion_attention2 (fusion_blocksparse.h:400-455, 1212-1268): sdd + masked
 * softmax in one kernel, y = P in the sparse layout (fp32 or bf16).  One work-group owns a whole
 * block-row, so the reference's rblk_flag / rblk_flag1 / Max / Sum scratch and its spin-waits are not
 * needed.  mask is BLOCK-major here (fusion_blocksparse.h:690).  row_order [dev] uint32[ctx_blks] (from
 * sfb_build_row_order: block-rows by falling block count) or NULL: the order in which block-rows are handed to
 * work-groups; with it the longest rows start first instead of forming the tail of the launch. */
int sfb_fused_sdd_softmax(sfb_stream_t stream, const sfb_uint2* nn_lut, const void* a, const void* b,
                          void* y, int in_dtype, int y_dtype, const void* mask,
                          const int32_t* valid_len, const uint32_t* row_order, uint32_t block_size,
                          uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                          uint32_t state_dim, uint32_t lut_heads, uint32_t lut_dim, uint32_t mask_heads,
                          float scale);

/* Comparison variant of sfb_fused_sdd_softmax with the reference's own decomposition (fusion_nt_softmax2 /
 * fusion_attention2, fusion_blocksparse.h:458-833, 1212-1268): one work-group per block; the blocks of a
 * block-row exchange row maxima and row sums through global scratch and wait for each other on two flags per
 * block-row.  Same results as sfb_fused_sdd_softmax.  nt_lut, nn_lut [dev]; mask BLOCK-major; scratch [dev]
 * 256-byte aligned, sfb_split_softmax_scratch_bytes() bytes (Max, Sum, the flags, one status word; cleared by
 * the call).  The waits are bounded by spin_limit polls: a work-group whose wait runs out leaves its block
 * unwritten and sets the status word (the last 256 bytes of scratch, uint32: 0 = every block written), because
 * the scheme cannot finish unless all work-groups of a block-row get to run at the same time. */
size_t sfb_split_softmax_scratch_bytes(uint32_t block_size, uint32_t blocks, uint32_t batch_dim, uint32_t head_dim,
                                       uint32_t ctx_blks);
int sfb_fused_sdd_softmax_split(sfb_stream_t stream, const sfb_uint2* nt_lut, const sfb_uint2* nn_lut,
                                const void* a, const void* b, void* y, int in_dtype, int y_dtype, const void* mask,
                                const int32_t* valid_len, void* scratch, size_t scratch_bytes, uint32_t spin_limit,
                                uint32_t block_size, uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks,
                                uint32_t head_dim, uint32_t state_dim, uint32_t lut_heads, uint32_t mask_heads,
                                float scale);

/* ---- encoder-layer ops (one pass over HBM each) ------------------------------------------------ */

/* bias (ewops.h:10-17; cuda_kernels.h:459-489), gelu (ewops.h:32-43; cuda_kernels.h:561-581: the
 * sigmoid form x/(1+exp(-1.702x))) and tensor_add_tensor (ewops.h:296-301; cuda_kernels.h:449-457)
 * as one kernel: out = act(in + bias[col]) + residual.  bias, residual may be NULL; act 0 = none,
 * 1 = GELU; out of out_dtype (fp32, or bf16 to feed a bf16 GEMM / attention); cols % 4 == 0;
 * out may alias in. */
int sfb_bias_act(sfb_stream_t stream, void* out, int out_dtype, const float* in, const float* bias,
                 const float* residual, int act, uint64_t rows, uint32_t cols);
/* layernorm (layernorm.h:13-38; cuda_kernels.h:334-372): mean and E[x^2] per row, eps 1e-5 inside the
 * root, affine; mean / rstd [dev] rows floats or NULL; state % 4 == 0. */
int sfb_layernorm(sfb_stream_t stream, void* out, int out_dtype, float* mean, float* rstd, const float* in,
                  const float* gain, const float* bias, uint32_t rows, uint32_t state);
/* tensor_add_matrix (ewops.h:276-282; cuda_kernels.h:526-535): out[b][i] = a[b][i] + m[i]. */
int sfb_add_matrix(sfb_stream_t stream, float* out, const float* a, const float* m, uint32_t dim0,
                   uint64_t inner);
/* transpose_0123to0213 (ewops.h:314-331): dst[a][c][b][:] = src[a][b][c][:], the [B, L, H, d] <-> [B, H, L, d]
 * exchange the reference's CPU attention makes around its products (transformer.cpp:533-545).  The attention
 * entry points of this library take [B, L, H, d] directly and need no such copy; it is provided for callers that
 * keep tensors in the other order.  fp32, d3 % 4 == 0, dst != src. */
int sfb_transpose_0213(sfb_stream_t stream, float* dst, const float* src, uint32_t d0, uint32_t d1, uint32_t d2,
                       uint32_t d3);
/* MI355X addition: bias + tensor_add_tensor + layernorm (ewops.h:10-17, 296-301, layernorm.h:13-38) in one
 * pass over memory: out = LayerNorm((in + bias[col]) + residual), same arithmetic and order as
 * sfb_bias_act followed by sfb_layernorm.  bias, residual may be NULL; out_bf16 [dev] optional second copy
 * of the result rounded to bf16 (NULL = none); state % 4 == 0, state <= 2048; out may alias in. */
int sfb_bias_residual_layernorm(sfb_stream_t stream, float* out, void* out_bf16, const float* in,
                                const float* bias, const float* residual, const float* gain, const float* beta,
                                uint32_t rows, uint32_t state);
/* embedding_lookup (embedding.h:5-12; cuda_kernels.h:210-221), optionally fused with the position add:
 * out[t] = table[ids[t]] (+ pos[t % seq_len]); pos may be NULL. */
int sfb_embedding_lookup(sfb_stream_t stream, float* out, const float* table, const int32_t* ids,
                         const float* pos, uint64_t tokens, uint32_t state, uint32_t seq_len, uint32_t vocab);
/* fp32 -> bf16, round to nearest even (the reference's to_bhalf, ew_op_gpu.h:241-254, rounds half
 * away from zero; inputs of the bf16 configurations are defined as RNE-rounded); n % 4 == 0. */
int sfb_cast_f32_bf16(sfb_stream_t stream, void* out, const float* in, uint64_t n);

/* Destroys the GEMM plans and the rocBLAS / hipBLASLt handles the GEMM entry points made (they are made again on
 * the next use).  Call it when no GEMM of this library is in flight. */
void sfb_gemm_release(void);
/* How a GEMM plan picks its kernel when it is made (first call of a shape): level 0 (default) times the library's
 * short list of candidates for the problem, level 1 times every kernel of the library that supports the problem
 * (a second or two per shape, once).  Plans already made keep their kernel until sfb_gemm_release().  Returns
 * SFB_ERR_ARGUMENT for other levels. */
int sfb_gemm_tuning(int level);

/* cblas_sgemm(RowMajor, NoTrans, NoTrans, m, n, k, 1, A, k, W, n, 0, C, n) (transformer.cpp:516-522, 547,
 * 562, 571; cublasSgemm twins transformer_attention_optimize.cu:693-716): C[m][n] = A[m][k] W[k][n],
 * a and w of dtype (fp32, or bf16 with fp32 accumulation), c fp32.  Runs on rocBLAS. */
int sfb_gemm(sfb_stream_t stream, float* c, const void* a, const void* w, int dtype, uint32_t m, uint32_t n,
             uint32_t k);

/* The same product followed by bias (ewops.h:10-17), as the reference issues them back to back
 * (transformer.cpp:516-527), in one kernel: C[m][n] = A[m][k] W[k][n] + bias[n], c of out_dtype (fp32 or bf16,
 * rounded once from the fp32 sum).  Runs on hipBLASLt with the bias in the GEMM epilogue; returns SFB_ERR_LAUNCH
 * if that library has no kernel for the shape and out_dtype is bf16 (fp32 output falls back to sfb_gemm +
 * sfb_bias_act in place).  n % 4 == 0. */
int sfb_gemm_bias(sfb_stream_t stream, void* c, int out_dtype, const void* a, const void* w, const float* bias,
                  int dtype, uint32_t m, uint32_t n, uint32_t k);

/* The product followed by bias and GELU (transformer.cpp:562-569: cblas_sgemm, bias, gelu) in one kernel:
 * C[m][n] = gelu(A[m][k] W[k][n] + bias[n]) with the reference's sigmoid form gelu(x) = x / (1 + exp(-1.702 x))
 * (ewops.h:32-43), evaluated on the fp32 sums; c of out_dtype, c != a.  Runs on hipBLASLt (Swish epilogue with
 * slope 1.702).  Where the hipBLASLt in the process has no such kernel or no slope argument (older builds, e.g. the
 * one PyTorch loads), fp32 output falls back to sfb_gemm + sfb_bias_act in place and bf16 output returns
 * SFB_ERR_LAUNCH.  n % 4 == 0. */
int sfb_gemm_bias_gelu(sfb_stream_t stream, void* c, int out_dtype, const void* a, const void* w, const float* bias,
                       int dtype, uint32_t m, uint32_t n, uint32_t k);

/* MI355X addition: the same in a form every hipBLASLt with a Swish epilogue can run.  C = *scale x gelu(A W + bias);
 * *scale [host, out] is 1 where the library takes the slope, otherwise 1.702: x / (1 + exp(-s x)) = Swish_1(s x) / s,
 * so the product and a copy of the bias (bias_scratch [dev] n floats) are scaled by s going in and the result is left
 * s times too large -- a caller that multiplies C by a matrix next passes 1 / *scale as that product's factor (as
 * the encoder layer does).  Returns SFB_ERR_LAUNCH if the library has no kernel for the shape.  n % 4 == 0. */
int sfb_gemm_bias_gelu_scaled(sfb_stream_t stream, void* c, int out_dtype, float* scale, float* bias_scratch,
                              const void* a, const void* w, const float* bias, int dtype, uint32_t m, uint32_t n,
                              uint32_t k);

/* Weights of one encoder layer, [in][out] row-major (transformer.cpp:98-136): matrices in the compute
 * dtype (fp32 or bf16), biases and LayerNorm parameters fp32.  All [dev]. */
typedef struct {
    const void *wq, *wk, *wv, *wo, *w1, *w2;
    const float *bq, *bk, *bv, *bo, *b1, *b2;
    const float *ln1_g, *ln1_b, *ln2_g, *ln2_b;
    /* optional (NULL: three products, as transformer.cpp:516-522 makes them): [Wq | Wk | Wv] as one [n][3n] matrix
     * and [bq | bk | bv], filled by sfb_pack_qkv; layers whose attention is a scheduled launch then make Q, K and V
     * with one product and hand the attention column slices of its result */
    const void* wqkv;
    const float* bqkv;
} sfb_layer_weights;
/* wqkv [dev] n x 3n of dtype, bqkv [dev] 3n floats from the layer's wq, wk, wv (n x n) and bq, bk, bv (copies on the
 * stream; the caller then stores the two pointers in the layer's sfb_layer_weights). */
int sfb_pack_qkv(sfb_stream_t stream, void* wqkv, float* bqkv, const sfb_layer_weights* wt, int dtype, uint32_t n);
size_t sfb_encoder_layer_workspace_bytes(uint32_t batch_dim, uint32_t ctx, uint32_t head_dim,
                                         uint32_t state_dim, uint32_t ffn, int dtype);
/* One post-LN encoder layer forward (op arithmetic and order of transformer.cpp:513-580, no dropout):
 * x1 = LN1(x + Attn(xWq+bq, xWk+bk, xWv+bv) Wo + bo); y = LN2(x1 + gelu(x1 W1 + b1) W2 + b2).
 * x, y [dev] fp32 [batch*ctx, heads*state]; dtype selects fp32 or bf16 operands for the GEMMs and the
 * attention (accumulation, LayerNorm, residuals and y stay fp32).  items may be NULL (one work-group
 * per block-row); otherwise items / n_* / attn_workspace are those of sfb_fused_attention_scheduled.
 * workspace [dev] 256-byte aligned, sfb_encoder_layer_workspace_bytes() bytes. */
int sfb_encoder_layer_forward(sfb_stream_t stream, float* y, const float* x, const sfb_layer_weights* wt,
                              int dtype, const sfb_uint2* nn_lut, const void* mask, const int32_t* valid_len,
                              const sfb_work_item* items, uint32_t n_items, uint32_t n_heavy, uint32_t n_slots,
                              uint32_t n_parts, void* attn_workspace, size_t attn_workspace_bytes, uint32_t block_size,
                              uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                              uint32_t state_dim, uint32_t ffn, void* workspace, size_t workspace_bytes);

/* The same layer in the reference's own wiring (transformer.cpp:513-580,
 * transformer_inference_part.cpp:209-232; pre-LN, dropout omitted):
 * a = LN1(x); x1 = x + Attn(aWq+bq, aWk+bk, aWv+bv) Wo + bo; y = x1 + gelu(LN2(x1) W1 + b1) W2 + b2.
 * Arguments and workspace as sfb_encoder_layer_forward. */
int sfb_encoder_layer_forward_pre_ln(sfb_stream_t stream, float* y, const float* x, const sfb_layer_weights* wt,
                                     int dtype, const sfb_uint2* nn_lut, const void* mask, const int32_t* valid_len,
                                     const sfb_work_item* items, uint32_t n_items, uint32_t n_heavy, uint32_t n_slots,
                                     uint32_t n_parts, void* attn_workspace, size_t attn_workspace_bytes,
                                     uint32_t block_size, uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks,
                                     uint32_t head_dim, uint32_t state_dim, uint32_t ffn, void* workspace,
                                     size_t workspace_bytes);

/* Either layer (pre_ln = 0: sfb_encoder_layer_forward's wiring, 1: sfb_encoder_layer_forward_pre_ln's) with its
 * attention launched over sfb_build_stream's streams: per-head look-up tables and masks (lut_heads, mask_heads =
 * head_dim; the reference's `fixed` pattern, fixed_fusion_test.cu:38-39) as well as shared ones.  plan / blob /
 * attn_workspace as for sfb_fused_attention_streamed; the other arguments as for sfb_encoder_layer_forward. */
int sfb_encoder_layer_forward_streamed(sfb_stream_t stream, float* y, const float* x, const sfb_layer_weights* wt,
                                       int dtype, int pre_ln, const sfb_uint2* nn_lut, const void* mask,
                                       const int32_t* valid_len, const sfb_stream_plan* plan, const void* blob,
                                       void* attn_workspace, size_t attn_workspace_bytes, uint32_t block_size,
                                       uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim,
                                       uint32_t state_dim, uint32_t lut_heads, uint32_t lut_dim, uint32_t mask_heads,
                                       uint32_t ffn, void* workspace, size_t workspace_bytes);

/* cblas_sgemm(RowMajor, NoTrans, Trans, m, n, k, 1, A, k, W, k, 0, C, n) (transformer_inference_part.cpp:236, the
 * tied-embedding logits): C[m][n] = A[m][k] W[n][k]^T, a and w of dtype, c fp32.  Runs on rocBLAS. */
int sfb_gemm_nt(sfb_stream_t stream, float* c, const void* a, const void* w, int dtype, uint32_t m, uint32_t n,
                uint32_t k);

/* softmax_cross_entropy_with_logits over to_one_hot labels (ewops.h:233-261, 352-361): row_loss[r] =
 * log(sum_j exp(logits[r][j])) - logits[r][labels[r]] (computed relative to the row maximum), loss[0] = their
 * mean, summed in a fixed order.  d_logits (may be NULL, may alias logits) = softmax - onehot, the reference's D.
 * A label outside [0, vocab) selects no column (row loss 0).  loss [dev] 1 float, row_loss [dev] rows floats,
 * logits [dev] rows x vocab fp32, labels [dev] rows int32. */
int sfb_softmax_cross_entropy(sfb_stream_t stream, float* loss, float* row_loss, float* d_logits,
                              const float* logits, const int32_t* labels, uint64_t rows, uint32_t vocab);

/* Weights of the whole model (transformer_inference_part.cpp:60-148): token embedding [vocab][state] (also the
 * logits matrix), position embedding [ctx][state], both fp32 [dev]; tok_embed_bf16 [dev] the token embedding
 * rounded to bf16 (needed when dtype is bf16, else may be NULL); layers: HOST array of n_layers structs of device
 * pointers. */
typedef struct {
    const float* tok_embed;
    const float* pos_embed;
    const void* tok_embed_bf16;
    const sfb_layer_weights* layers;
    uint32_t n_layers;
} sfb_model_weights;
size_t sfb_model_workspace_bytes(uint32_t batch_dim, uint32_t ctx, uint32_t head_dim, uint32_t state_dim,
                                 uint32_t ffn, uint32_t vocab, int dtype);
/* Forward pass of the whole model in the shape of transformer_inference_part.cpp:190-256 (dropout omitted):
 * x = tok_embed[ids] + pos_embed; n_layers encoder layers (pre_ln != 0: the reference's wiring, 0: post-LN);
 * logits = x tok_embed^T; loss[0] = mean cross-entropy against labels.  ids, labels [dev] batch*ctx int32
 * (labels may be NULL: no loss); logits [dev] batch*ctx x vocab fp32 or NULL (kept in the workspace); hidden
 * [dev] batch*ctx x heads*state fp32 or NULL (copy of the last layer's output); the attention arguments are
 * those of sfb_encoder_layer_forward; workspace [dev] 256-byte aligned, sfb_model_workspace_bytes() bytes. */
int sfb_model_forward(sfb_stream_t stream, float* loss, float* logits, float* hidden, const int32_t* ids,
                      const int32_t* labels, const sfb_model_weights* w, int dtype, int pre_ln,
                      const sfb_uint2* nn_lut, const void* mask, const int32_t* valid_len,
                      const sfb_work_item* items, uint32_t n_items, uint32_t n_heavy, uint32_t n_slots,
                      uint32_t n_parts, void* attn_workspace, size_t attn_workspace_bytes, uint32_t block_size,
                      uint32_t blocks, uint32_t batch_dim, uint32_t ctx_blks, uint32_t head_dim, uint32_t state_dim,
                      uint32_t ffn, uint32_t vocab, void* workspace, size_t workspace_bytes);

#ifdef __cplusplus
}
#endif
#endif /* SFBERT_HIP_H */
