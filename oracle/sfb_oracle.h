/*
 * CPU oracle for SF-BERT block-sparse attention and the encoder-layer ops around it.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's CPU fp32 path and of
 * its host-side descriptor construction.  It exists so that the HIP kernels can be checked against
 * it; nothing the library ships may include, link or call it.  Only the tests, the smoke check and
 * the CPU-baseline leg of the benchmark use it.
 *
 * Every function names the reference file:line it follows.  Pinning status (what independent
 * evidence fixes each function) is listed at the top of sfb_oracle.c.
 */
#ifndef SFB_ORACLE_H
#define SFB_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct { uint32_t x, y; } orc_uint2;

/* ---- block layouts: uint32 layout[heads][nb][nb], 1 = (query block, key block) attended ---- */
void orc_layout_full(uint32_t* layout, int nb, int causal);
void orc_layout_local(uint32_t* layout, int nb, int extra_diag, int bidirectional);
void orc_layout_fixed(uint32_t* layout, int heads, int nb, int stride, int causal);
void orc_layout_strided_chunks(uint32_t* layout, int nb, int block_chunks);
void orc_layout_strided(uint32_t* layout, int nb, int band, int stride, int causal);
void orc_layout_bigbird(uint32_t* layout, int nb, int window, int nglobal, int global_both_ends,
                        const int32_t* rand_cols, int nrand);
/* seeded draw of `nrand` distinct still-empty columns per block-row (rows already full get -1) */
void orc_bigbird_draw(int32_t* rand_cols, int nb, int window, int nglobal, int global_both_ends,
                      int nrand, uint64_t seed);

/* ---- look-up tables ---- */
uint32_t orc_count_blocks(const uint32_t* layout, int nb);
void     orc_build_nt_lut(orc_uint2* nt_lut, const uint32_t* layout, int nb);
uint32_t orc_build_nn_lut(orc_uint2* nn_lut, const orc_uint2* nt_lut, uint32_t blocks, int nb,
                          uint32_t nn_max_init);
void     orc_build_rblk_lut(orc_uint2* rblk_lut, const orc_uint2* nn_lut, int nb);
uint32_t orc_build_tn_lut(orc_uint2* tn_lut, const orc_uint2* nt_lut, uint32_t blocks, int nb);
void     orc_magicu64(uint32_t d, uint32_t* magic, uint32_t* shift);
uint32_t orc_div64(uint32_t value, uint32_t magic, uint32_t shift);

/* ---- element masks: keep[blocks][bs][bs] bytes, then packed words ---- */
enum { ORC_MASK_ALL = 0, ORC_MASK_CAUSAL_DIAG = 1, ORC_MASK_LOCAL = 2, ORC_MASK_TRIANGULAR_ALL = 3 };
void orc_element_mask(uint8_t* keep, const orc_uint2* nt_lut, uint32_t blocks, int bs, int kind,
                      int local_attn_ctx);
/* block-major words[blk*bs + row]; word_bytes = 4 (bs 32) or 8 (bs 64) */
void orc_pack_mask(void* words, const uint8_t* keep, uint32_t blocks, int bs, int word_bytes);
/* row-major words[row*blocks + blk] from block-major */
void orc_transpose_mask(void* row_major, const void* block_major, uint32_t blocks, int bs,
                        int word_bytes);

/* ---- attention, fp32, tensors [B, L, H, d] ---- */
/* mask_block_major may be NULL (all ones); valid_len may be NULL (no key padding).
 * nthreads <= 1 runs single-threaded, as the reference is built. */
void orc_blocksparse_attention(float* O, const float* Q, const float* K, const float* V,
                               const orc_uint2* nn_lut, const void* mask_block_major,
                               int mask_word_bytes, const int32_t* valid_len, int B, int L, int H,
                               int d, int bs, float scale, int lut_heads, uint32_t lut_dim_nn,
                               int mask_heads, uint32_t blocks, int nthreads);
/* the three stages separately; S and P are sparse [B][H][blocks][bs][bs] fp32 */
void orc_sdd_nt(float* S, const float* Q, const float* K, const orc_uint2* nt_lut, int B, int L,
                int H, int d, int bs, uint32_t blocks, int lut_heads);
void orc_masked_softmax(float* P, const float* S, const orc_uint2* nn_lut,
                        const void* mask_block_major, int mask_word_bytes,
                        const int32_t* valid_len, int B, int H, int nb, int bs, uint32_t blocks,
                        float scale, int lut_heads, int mask_heads);
void orc_dsd_nn(float* O, const float* P, const float* V, const orc_uint2* nn_lut, int B, int L,
                int H, int d, int bs, uint32_t blocks, int lut_heads);
/* backward stages of the unfused path (transformer_attention_optimize.cu:924-964) */
void orc_masked_softmax_grad(float* dS, const float* dP, const float* P, const orc_uint2* nn_lut, int B,
                             int H, int nb, int bs, uint32_t blocks, float scale, int lut_heads);
void orc_dsd_tn(float* C, const float* A, const float* X, const orc_uint2* tn_lut, int B, int L, int H,
                int d, int bs, uint32_t blocks, int lut_heads);

/* ---- bf16 storage helpers ---- */
uint16_t orc_f32_to_bf16_rne(float x);
float    orc_bf16_to_f32(uint16_t x);
uint16_t orc_f32_to_bf16_half_away(float x);
void     orc_round_to_bf16_rne(float* x, long n);

/* ---- encoder-layer ops ---- */
void orc_layernorm(float* out, float* mean, float* rstd, const float* in, const float* gain,
                   const float* bias, int rows, int state);
void orc_gelu(float* out, const float* in, long n);
void orc_bias(float* out, const float* in, const float* bias, int n, int m);
void orc_add(float* out, const float* a, const float* b, long n);
void orc_add_matrix(float* out, const float* a, const float* b, int dim0, long inner);
void orc_embedding_lookup(float* out, const float* table, const int32_t* ids, long tokens,
                          int state);
void orc_transpose_0213(const float* src, float* dst, int d0, int d1, int d2, int d3);
void orc_sgemm(float* C, const float* A, const float* W, int m, int n, int k, int nthreads);

typedef struct {
    const float *wq, *wk, *wv, *wo, *w1, *w2;  /* [in][out] row-major */
    const float *bq, *bk, *bv, *bo, *b1, *b2;
    const float *ln1_g, *ln1_b, *ln2_g, *ln2_b;
} orc_layer_weights;
/* post-LN BERT encoder layer with block-sparse attention inside; operands_bf16 != 0 rounds every
 * GEMM / attention operand to bf16 (RNE) before use, accumulating in fp32. */
void orc_encoder_layer(float* y, const float* x, const orc_layer_weights* w,
                       const orc_uint2* nn_lut, const void* mask_block_major, int mask_word_bytes,
                       const int32_t* valid_len, int B, int L, int H, int d, int ffn, int bs,
                       uint32_t blocks, int operands_bf16, int nthreads);

/* the reference's own pre-LN wiring of the same ops (transformer.cpp:513-580) */
void orc_encoder_layer_pre_ln(float* y, const float* x, const orc_layer_weights* w,
                       const orc_uint2* nn_lut, const void* mask_block_major, int mask_word_bytes,
                       const int32_t* valid_len, int B, int L, int H, int d, int ffn, int bs,
                       uint32_t blocks, int operands_bf16, int nthreads);

/* C[m][n] = A[m][k] W[n][k]^T (transformer_inference_part.cpp:236) */
void orc_sgemm_nt(float* C, const float* A, const float* W, int m, int n, int k, int nthreads);

/* ewops.h:233-261 with one-hot labels (ewops.h:352-361); returns the mean loss */
float orc_softmax_cross_entropy(float* d_out, float* row_loss, const float* logits, const int32_t* labels,
                                long rows, int vocab);

/* transformer_inference_part.cpp:190-256 without dropout; returns the loss */
float orc_model_forward(float* logits, float* hidden, const int32_t* ids, const int32_t* labels,
                        const float* tok, const float* pos, const orc_layer_weights* layers, int n_layers,
                        int pre_ln, const orc_uint2* nn_lut, const void* mask_block_major, int mask_word_bytes,
                        const int32_t* valid_len, int B, int L, int H, int d, int ffn, int bs, uint32_t blocks,
                        int vocab, int operands_bf16, int nthreads);

/* ---- seeded generator shared by tests and bench (splitmix64 + Box-Muller) ---- */
void orc_fill_normal(float* x, long n, uint64_t seed, float std);
void orc_fill_uniform_int(int32_t* x, long n, uint64_t seed, int32_t lo, int32_t hi);

#ifdef __cplusplus
}
#endif
#endif
