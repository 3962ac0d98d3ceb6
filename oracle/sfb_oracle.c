/*
 * CPU oracle -- TEST INFRASTRUCTURE ONLY (see sfb_oracle.h).  Never linked into the shipped library.
 *
 * Reference = /root/reference (HeyHaoh/SF-Bert).  Each function cites the lines it restates.
 *
 * Pinning status (what, other than this file, fixes each function's results):
 *   orc_layout_*, orc_build_*_lut, orc_pack/transpose_mask : the reference builds these inline in
 *       CUDA test mains that cannot be compiled here; pinned by the reference's hard-coded sizes
 *       (10-block causal: 55 blocks, nn_lut_dim 65, nn_max 10 -- test.cu:24,39-40,45; fixed stride 4
 *       head 0: nn_max 5 -- test.cu:574), by the worked nb=4 'local' example, by brute-force dense
 *       scans and by structural invariants (tests/test_oracle_descriptors.py).
 *   orc_magicu64 / orc_div64 : exhaustive n/d check.
 *   orc_blocksparse_attention, orc_sdd_nt, orc_masked_softmax, orc_dsd_nn : bit-compared with the
 *       reference's own multiheadmatmulNT / softmax / multiheadmatmulNN compiled from
 *       /root/reference into oracle/_ref (dense-causal special case) and with the fixtures under
 *       tests/golden written by that build; float64 numpy brute force for every other pattern,
 *       closed forms (all-ones inputs), torch SDPA for the full layout.
 *   orc_masked_softmax_grad, orc_dsd_tn (backward stages) : bit-compared with the reference's own
 *       softmax_grad / multiheadmatmulTN in oracle/_ref on the dense-causal case (the whole chain dV, dP,
 *       dS, dK, dQ) and with tests/golden/attention_backward_dense_causal.npz written by that build; torch
 *       autograd of a float64 dense attention for every pattern, masks and padding included.
 *   orc_build_tn_lut : the reference only has the commented causal builder (ewops.h:675-701); pinned by a
 *       brute-force column scan for every pattern and by that builder's count pattern nb, nb-1, ..., 1.
 *   orc_layernorm, orc_gelu, orc_bias, orc_add*, orc_embedding_lookup, orc_transpose_0213 :
 *       bit-compared with the reference functions in oracle/_ref + golden fixtures; float64 numpy.
 *   orc_sgemm : the reference calls OpenBLAS cblas_sgemm (not vendored, no version pinned) --
 *       PARITY UNPINNED against the reference; checked as a textbook GEMM against float64 numpy.
 *   orc_encoder_layer : composition of the above in the order of transformer.cpp:513-580 with the
 *       post-LN structure the workload definition asks for; checked against a float64 numpy layer.
 *   orc_f32_to_bf16_* : exhaustive check over all bf16 neighbours.
 *   orc_softmax_cross_entropy : bit-compared with the reference's softmax_cross_entropy_with_logits + to_one_hot
 *       in oracle/_ref + golden fixture; float64 log-sum-exp.
 *   orc_sgemm_nt : like orc_sgemm, the reference calls OpenBLAS -- PARITY UNPINNED; float64 numpy.
 *   orc_encoder_layer_pre_ln, orc_model_forward : compositions of the above in the order of
 *       transformer_inference_part.cpp:190-256 (dropout omitted); checked against a float64 numpy model.
 */
#include "sfb_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------ */
/* layouts                                                                                     */
/* ------------------------------------------------------------------------------------------ */

/* no_fusion_test.cu:47-62 (causal: layout[i][j] = i>=j); causal==0 gives the dense layout. */
void orc_layout_full(uint32_t* layout, int nb, int causal) {
    for (int i = 0; i < nb; i++)
        for (int j = 0; j < nb; j++) layout[i * nb + j] = (!causal || i >= j) ? 1u : 0u;
}

/* local_fusion_test.cu:46-63: start from all ones, clear (extra_diag!=0 && j+extra_diag<i) || j>i.
 * bidirectional != 0 keeps |i-j| <= extra_diag instead (the band on both sides). */
void orc_layout_local(uint32_t* layout, int nb, int extra_diag, int bidirectional) {
    for (int i = 0; i < nb * nb; i++) layout[i] = 1;
    for (int i = 0; i < nb; i++) {
        for (int j = 0; j < nb; j++) {
            if (bidirectional) {
                int dist = i > j ? i - j : j - i;
                if (dist > extra_diag) layout[i * nb + j] = 0;
            } else {
                if (((extra_diag != 0) && ((j + extra_diag) < i)) || (j > i)) layout[i * nb + j] = 0;
            }
        }
    }
}

/* fixed_fusion_test.cu:52-106: per head h the summary columns are k = stride-(h+1), +stride, ...;
 * every block-row also attends its own chunk [row/stride*stride, +stride); causal clears j<k. */
void orc_layout_fixed(uint32_t* layout, int heads, int nb, int stride, int causal) {
    for (int i = 0; i < heads * nb * nb; i++) layout[i] = 0;
    for (int h = 0; h < heads; h++) {
        int first = stride - (h + 1);
        if (first < 0) first = ((first % stride) + stride) % stride;
        for (int j = 0; j < nb; j++)
            for (int k = first; k < nb; k += stride) layout[h * nb * nb + j * nb + k] = 1;
    }
    for (int h = 0; h < heads; h++) {
        for (int j = 0; j < nb; j++) {
            int row = j / stride;
            int right = ((row + 1) * stride) > nb ? nb : ((row + 1) * stride);
            for (int k = row * stride; k < right; k++) layout[h * nb * nb + j * nb + k] = 1;
        }
    }
    if (causal) {
        for (int h = 0; h < heads; h++)
            for (int j = 0; j < nb; j++)
                for (int k = 0; k < nb; k++)
                    if (j < k) layout[h * nb * nb + j * nb + k] = 0;
    }
}

/* stride_fusion_test.cu:48-71: keep j<=i && j + (i % block_chunks) >= i. */
void orc_layout_strided_chunks(uint32_t* layout, int nb, int block_chunks) {
    for (int i = 0; i < nb * nb; i++) layout[i] = 0;
    for (int i = 0; i < nb; i++) {
        for (int j = 0; j < nb; j++) {
            uint32_t offset = (uint32_t)i % (uint32_t)block_chunks;
            if (((uint32_t)j + offset >= (uint32_t)i) && (j <= i)) layout[i * nb + j] = 1;
        }
    }
}

/* Block-level form of the element rule in ewops.h:462-503 / dense_tf_transfomer.py:98-108:
 * a local band of `band` blocks (itself and band-1 previous) united with every column whose
 * distance from the row is a multiple of `stride`; causal restricts the strided term to j<=i. */
void orc_layout_strided(uint32_t* layout, int nb, int band, int stride, int causal) {
    for (int i = 0; i < nb; i++) {
        for (int j = 0; j < nb; j++) {
            int diff = i - j;
            int local = (diff >= 0) && (diff < band);
            int adiff = diff < 0 ? -diff : diff;
            int strided = ((adiff % stride) == 0) && (!causal || diff >= 0);
            layout[i * nb + j] = (local || strided) ? 1u : 0u;
        }
    }
}

static void bigbird_global_set(int* is_global, int nb, int nglobal, int both_ends) {
    for (int i = 0; i < nb; i++) is_global[i] = 0;
    if (!both_ends) {
        for (int i = 0; i < nglobal && i < nb; i++) is_global[i] = 1;
    } else {
        int head = (nglobal + 1) / 2, tail = nglobal / 2;
        for (int i = 0; i < head && i < nb; i++) is_global[i] = 1;
        for (int i = 0; i < tail && i < nb; i++) is_global[nb - 1 - i] = 1;
    }
}

/* big_bird_fusion_test.cu:50-99: window |i-j|<=window written column by column, then `nglobal`
 * dense block-rows and block-columns, then the random columns of each row.  The reference takes the
 * first `global` rows/cols; global_both_ends splits them between the first and last positions. */
void orc_layout_bigbird(uint32_t* layout, int nb, int window, int nglobal, int global_both_ends,
                        const int32_t* rand_cols, int nrand) {
    for (int i = 0; i < nb * nb; i++) layout[i] = 0;
    for (int i = 0; i < nb; i++) {
        for (int j = 0; j <= window; j++) {
            if ((i + j) < nb) layout[(i + j) * nb + i] = 1;
            if ((i - j) >= 0) layout[(i - j) * nb + i] = 1;
        }
    }
    int* is_global = (int*)malloc(sizeof(int) * (size_t)nb);
    bigbird_global_set(is_global, nb, nglobal, global_both_ends);
    for (int i = 0; i < nb; i++) {
        if (!is_global[i]) continue;
        for (int j = 0; j < nb; j++) {
            layout[i * nb + j] = 1;
            layout[j * nb + i] = 1;
        }
    }
    free(is_global);
    if (rand_cols) {
        for (int i = 0; i < nb; i++)
            for (int t = 0; t < nrand; t++) {
                int32_t c = rand_cols[i * nrand + t];
                if (c >= 0 && c < nb) layout[i * nb + c] = 1;
            }
    }
}

static uint64_t splitmix64(uint64_t* state) {
    uint64_t z = (*state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

/* Seeded replacement for the reference's unseeded rand()%10 draw (big_bird_fusion_test.cu:81-99):
 * per block-row, in row order, a partial Fisher-Yates shuffle of the ascending list of columns that
 * window+global left empty; one splitmix64 stream for the whole layout. */
void orc_bigbird_draw(int32_t* rand_cols, int nb, int window, int nglobal, int global_both_ends,
                      int nrand, uint64_t seed) {
    uint32_t* base = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)nb * (size_t)nb);
    int32_t* empty = (int32_t*)malloc(sizeof(int32_t) * (size_t)nb);
    orc_layout_bigbird(base, nb, window, nglobal, global_both_ends, NULL, 0);
    uint64_t state = seed;
    for (int i = 0; i < nb; i++) {
        int n_empty = 0;
        for (int j = 0; j < nb; j++)
            if (!base[i * nb + j]) empty[n_empty++] = j;
        for (int t = 0; t < nrand; t++) {
            if (t >= n_empty) {
                rand_cols[i * nrand + t] = -1;
                continue;
            }
            uint64_t r = splitmix64(&state);
            int pick = t + (int)(r % (uint64_t)(n_empty - t));
            int32_t tmp = empty[t];
            empty[t] = empty[pick];
            empty[pick] = tmp;
            rand_cols[i * nrand + t] = empty[t];
        }
    }
    free(base);
    free(empty);
}

/* ------------------------------------------------------------------------------------------ */
/* look-up tables                                                                              */
/* ------------------------------------------------------------------------------------------ */

/* local_fusion_test.cu:78-85 */
uint32_t orc_count_blocks(const uint32_t* layout, int nb) {
    uint32_t n = 0;
    for (int i = 0; i < nb * nb; i++)
        if (layout[i] == 1) n++;
    return n;
}

/* local_fusion_test.cu:89-99: row-major scan, {x = row block, y = col block}. */
void orc_build_nt_lut(orc_uint2* nt_lut, const uint32_t* layout, int nb) {
    int count = 0;
    for (int i = 0; i < nb * nb; i++) {
        if (layout[i] == 1) {
            nt_lut[count].x = (uint32_t)(i / nb);
            nt_lut[count].y = (uint32_t)(i % nb);
            count++;
        }
    }
}

/* local_fusion_test.cu:106-133: header {offset,count} per block-row, offsets start at nb; body
 * {block id, key block}.  Returns nn_max = max(nn_max_init, max count). */
uint32_t orc_build_nn_lut(orc_uint2* nn_lut, const orc_uint2* nt_lut, uint32_t blocks, int nb,
                          uint32_t nn_max_init) {
    uint32_t dim = blocks + (uint32_t)nb;
    for (uint32_t i = 0; i < dim; i++) {
        nn_lut[i].x = 0;
        nn_lut[i].y = 0;
    }
    for (uint32_t i = 0; i < blocks; i++) {
        nn_lut[nt_lut[i].x].y++;
        nn_lut[(uint32_t)nb + i].x = i;
        nn_lut[(uint32_t)nb + i].y = nt_lut[i].y;
    }
    nn_lut[0].x = (uint32_t)nb;
    for (int i = 1; i < nb; i++) nn_lut[i].x = nn_lut[i - 1].x + nn_lut[i - 1].y;
    uint32_t nn_max = nn_max_init;
    for (int i = 0; i < nb; i++) nn_max = nn_max > nn_lut[i].y ? nn_max : nn_lut[i].y;
    return nn_max;
}

/* local_fusion_test.cu:229-237: {x = block id, y = row block}. */
void orc_build_rblk_lut(orc_uint2* rblk_lut, const orc_uint2* nn_lut, int nb) {
    uint32_t count = 0;
    for (int i = 0; i < nb; i++) {
        for (uint32_t j = 0; j < nn_lut[i].y; j++) {
            rblk_lut[count].x = count;
            rblk_lut[count].y = (uint32_t)i;
            count++;
        }
    }
}

/* TN look-up table of the transposed products (dV = P^T dO, dK = dS^T Q;
 * transformer_attention_optimize.cu:924-957 passes it as tn_ptr): per key-block column c a header
 * {offset, count}, offsets starting at nb, then the blocks of that column in ascending row order as
 * {block id in NT order, row block} -- the column-wise twin of the NN table; the reference's own builder
 * exists only as the commented causal special case generate_tn_lut (ewops.h:675-701).  Returns the
 * largest count. */
uint32_t orc_build_tn_lut(orc_uint2* tn_lut, const orc_uint2* nt_lut, uint32_t blocks, int nb) {
    uint32_t offset = (uint32_t)nb, tn_max = 0, at = (uint32_t)nb;
    for (int c = 0; c < nb; c++) {
        uint32_t count = 0;
        for (uint32_t blk = 0; blk < blocks; blk++)
            if ((int)nt_lut[blk].y == c) {   /* NT order is row-major, so rows come out ascending */
                tn_lut[at].x = blk;
                tn_lut[at].y = nt_lut[blk].x;
                at++;
                count++;
            }
        tn_lut[c].x = offset;
        tn_lut[c].y = count;
        offset += count;
        if (count > tn_max) tn_max = count;
    }
    return tn_max;
}

/* blocksparse.h:1016-1043 */
void orc_magicu64(uint32_t d, uint32_t* magic, uint32_t* shift) {
    if (d == 1) { *magic = 1; *shift = 0; }
    else if (d == 2) { *magic = 1; *shift = 1; }
    else if (d == 4) { *magic = 1; *shift = 2; }
    else if (d == 8) { *magic = 1; *shift = 3; }
    else {
        uint32_t nbits = d == 3 ? (2 * 32) + 1 : (2 * 31) + 1;
        uint64_t nmax = d == 3 ? 0xffffffffull : 0x7fffffffull;
        uint64_t d64 = d;
        uint64_t nc = ((nmax + 1ull) / d64) * d64 - 1ull;
        for (uint32_t p = 0; p < nbits; p++) {
            if ((1ull << p) > nc * (d64 - 1ull - ((1ull << p) - 1ull) % d64)) {
                *magic = (uint32_t)(((1ull << p) + d64 - 1ull - ((1ull << p) - 1ull) % d64) / d64);
                *shift = *magic == 1 ? p : p - 32;
                return;
            }
        }
    }
}

/* gpu_hmma.h:4-20: magic==1 is a plain shift, otherwise high word of the product, then shift. */
uint32_t orc_div64(uint32_t value, uint32_t magic, uint32_t shift) {
    uint64_t res64 = (uint64_t)value * (uint64_t)magic;
    uint32_t hi = (magic != 1) ? (uint32_t)(res64 >> 32) : value;
    return hi >> shift;
}

/* ------------------------------------------------------------------------------------------ */
/* element masks                                                                               */
/* ------------------------------------------------------------------------------------------ */

/* ORC_MASK_CAUSAL_DIAG   : no_fusion_test.cu:124-143 (diagonal blocks lower-triangular, rest ones)
 * ORC_MASK_LOCAL         : local_fusion_test.cu:146-175 (col<=row && col+local_attn_ctx>row)
 * ORC_MASK_TRIANGULAR_ALL: stride_fusion_test.cu:141-160 (every block lower-triangular) */
void orc_element_mask(uint8_t* keep, const orc_uint2* nt_lut, uint32_t blocks, int bs, int kind,
                      int local_attn_ctx) {
    for (size_t i = 0; i < (size_t)blocks * bs * bs; i++) keep[i] = 1;
    if (kind == ORC_MASK_ALL) return;
    for (uint32_t l = 0; l < blocks; l++) {
        uint32_t i_idx = nt_lut[l].x, j_idx = nt_lut[l].y;
        for (int i = 0; i < bs; i++) {
            for (int j = 0; j < bs; j++) {
                size_t at = (size_t)l * bs * bs + (size_t)i * bs + j;
                if (kind == ORC_MASK_CAUSAL_DIAG) {
                    if (i_idx == j_idx && !(i >= j)) keep[at] = 0;
                } else if (kind == ORC_MASK_LOCAL) {
                    if (i_idx == j_idx && j > i) keep[at] = 0;
                    uint32_t row_idx = i_idx * (uint32_t)bs + (uint32_t)i;
                    uint32_t col_idx = j_idx * (uint32_t)bs + (uint32_t)j;
                    if ((col_idx > row_idx) || ((col_idx + (uint32_t)local_attn_ctx) <= row_idx))
                        keep[at] = 0;
                } else if (kind == ORC_MASK_TRIANGULAR_ALL) {
                    if (i < j) keep[at] = 0;
                }
            }
        }
    }
}

/* no_fusion_test.cu:145-157: bit j of word[blk*bs+row] = keep[blk][row][j]. */
void orc_pack_mask(void* words, const uint8_t* keep, uint32_t blocks, int bs, int word_bytes) {
    for (size_t i = 0; i < (size_t)blocks * bs; i++) {
        uint64_t w = 0;
        for (int j = 0; j < bs; j++) {
            uint64_t k = keep[i * bs + j] ? 1ull : 0ull;
            w |= k << j;
        }
        if (word_bytes == 8) ((uint64_t*)words)[i] = w;
        else if (word_bytes == 4) ((uint32_t*)words)[i] = (uint32_t)w;
        else if (word_bytes == 2) ((uint16_t*)words)[i] = (uint16_t)w;   /* block 16: blocksparse.h:705 */
        else ((uint8_t*)words)[i] = (uint8_t)w;                          /* block 8: blocksparse.h:714 */
    }
}

/* no_fusion_test.cu:159-163: mask[row*blocks + blk] = mask_np[blk*bs + row]. */
void orc_transpose_mask(void* row_major, const void* block_major, uint32_t blocks, int bs,
                        int word_bytes) {
    for (uint32_t i = 0; i < blocks; i++) {
        for (int j = 0; j < bs; j++) {
            size_t src = (size_t)i * bs + j, dst = (size_t)j * blocks + i;
            memcpy((char*)row_major + dst * (size_t)word_bytes, (const char*)block_major + src * (size_t)word_bytes,
                   (size_t)word_bytes);
        }
    }
}

static inline int mask_bit(const void* words, int word_bytes, size_t word_index, int bit) {
    if (!words) return 1;
    if (word_bytes == 8) return (int)((((const uint64_t*)words)[word_index] >> bit) & 1ull);
    if (word_bytes == 4) return (int)((((const uint32_t*)words)[word_index] >> bit) & 1u);
    if (word_bytes == 2) return (int)((((const uint16_t*)words)[word_index] >> bit) & 1u);
    return (int)((((const uint8_t*)words)[word_index] >> bit) & 1u);
}

/* ------------------------------------------------------------------------------------------ */
/* attention                                                                                   */
/* ------------------------------------------------------------------------------------------ */

/* Token-major offset of element (b, token, h, k) in a [B, L, H, d] tensor
 * (openai_blocksparse.h:40-41; equal to the [B,H,L,d] view the CPU path reaches through
 * transpose_0123to0213, ewops.h:314-331). */
static inline size_t tok(int b, int t, int h, int L, int H, int d) {
    return (((size_t)b * L + t) * H + h) * (size_t)d;
}

/* One block-row of queries: matmul.h:53-78 (float dot, ascending n) -> ewops.h:64-98 (max seeded
 * with -1000000.0, exp((s-max)*scale) through double exp, float running sum over kept keys in
 * ascending key order, divide by sum+1e-6f) -> matmul.h:6-20 (float accumulation, ascending key).
 * The reference's hard-wired k>=m test is replaced by layout bit & mask bit & key<valid_len[b]. */
static void attention_block_row(float* O, const float* Q, const float* K, const float* V,
                                const orc_uint2* lut, const void* mask, int mask_word_bytes,
                                int valid, int b, int h, int r, int L, int H, int d, int bs,
                                float scale, float* srow, float* acc) {
    uint32_t offset = lut[r].x, count = lut[r].y;
    for (int qi = 0; qi < bs; qi++) {
        int qtok = r * bs + qi;
        const float* q = Q + tok(b, qtok, h, L, H, d);
        float max = -1000000.0f;
        for (uint32_t jj = 0; jj < count; jj++) {
            uint32_t blk = lut[offset + jj].x, col = lut[offset + jj].y;
            for (int kk = 0; kk < bs; kk++) {
                int ktok = (int)col * bs + kk;
                const float* kv = K + tok(b, ktok, h, L, H, d);
                float sum = 0;
                for (int n = 0; n < d; n++) sum += q[n] * kv[n];
                srow[jj * bs + kk] = sum;
                int keep = mask_bit(mask, mask_word_bytes, (size_t)blk * bs + qi, kk) && ktok < valid;
                if (keep && sum > max) max = sum;
            }
        }
        float sum_of_c = 0.0f;
        for (uint32_t jj = 0; jj < count; jj++) {
            uint32_t blk = lut[offset + jj].x, col = lut[offset + jj].y;
            for (int kk = 0; kk < bs; kk++) {
                int ktok = (int)col * bs + kk;
                int keep = mask_bit(mask, mask_word_bytes, (size_t)blk * bs + qi, kk) && ktok < valid;
                float p = 0.0f;
                if (keep) {
                    p = (float)exp((srow[jj * bs + kk] - max) * scale);
                    sum_of_c += p;
                }
                srow[jj * bs + kk] = p;
            }
        }
        float denom = sum_of_c + 1e-6f;
        for (uint32_t jj = 0; jj < count; jj++)
            for (int kk = 0; kk < bs; kk++) srow[jj * bs + kk] /= denom;
        for (int m = 0; m < d; m++) acc[m] = 0.0f;
        /* matmul.h:12-15 sums over every key; keys outside the layout carry P == 0 and leave the
         * float sum unchanged, so only the attended blocks are visited (ascending key order). */
        for (int m = 0; m < d; m++) {
            float sum = 0;
            for (uint32_t jj = 0; jj < count; jj++) {
                uint32_t col = lut[offset + jj].y;
                for (int kk = 0; kk < bs; kk++) {
                    int ktok = (int)col * bs + kk;
                    sum += srow[jj * bs + kk] * V[tok(b, ktok, h, L, H, d) + m];
                }
            }
            acc[m] = sum;
        }
        float* o = O + tok(b, qtok, h, L, H, d);
        for (int m = 0; m < d; m++) o[m] = acc[m];
    }
}

void orc_blocksparse_attention(float* O, const float* Q, const float* K, const float* V,
                               const orc_uint2* nn_lut, const void* mask_block_major,
                               int mask_word_bytes, const int32_t* valid_len, int B, int L, int H,
                               int d, int bs, float scale, int lut_heads, uint32_t lut_dim_nn,
                               int mask_heads, uint32_t blocks, int nthreads) {
    int nb = L / bs;
    long total = (long)B * H * nb;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel num_threads(nthreads)
    {
        float* srow = (float*)malloc(sizeof(float) * (size_t)L);
        float* acc = (float*)malloc(sizeof(float) * (size_t)d);
#pragma omp for schedule(dynamic, 1)
        for (long w = 0; w < total; w++) {
            int r = (int)(w % nb);
            int h = (int)((w / nb) % H);
            int b = (int)(w / ((long)nb * H));
            const orc_uint2* lut = nn_lut + (lut_heads > 1 ? (size_t)h * lut_dim_nn : 0);
            const void* mask = NULL;
            if (mask_block_major) {
                size_t head_words = mask_heads > 1 ? (size_t)h * blocks * bs : 0;
                mask = (const char*)mask_block_major + head_words * (size_t)mask_word_bytes;
            }
            int valid = valid_len ? valid_len[b] : L;
            attention_block_row(O, Q, K, V, lut, mask, mask_word_bytes, valid, b, h, r, L, H, d, bs,
                                scale, srow, acc);
        }
        free(srow);
        free(acc);
    }
}

/* matmul.h:53-78 restricted to the blocks of the NT LUT; S is [B][H][blocks][bs][bs]
 * (openai_blocksparse.h:148), no mask applied at this stage. */
void orc_sdd_nt(float* S, const float* Q, const float* K, const orc_uint2* nt_lut, int B, int L,
                int H, int d, int bs, uint32_t blocks, int lut_heads) {
    for (int b = 0; b < B; b++)
        for (int h = 0; h < H; h++) {
            const orc_uint2* lut = nt_lut + (lut_heads > 1 ? (size_t)h * blocks : 0);
            for (uint32_t blk = 0; blk < blocks; blk++) {
                float* s = S + (((size_t)b * H + h) * blocks + blk) * bs * bs;
                for (int i = 0; i < bs; i++)
                    for (int j = 0; j < bs; j++) {
                        const float* q = Q + tok(b, (int)lut[blk].x * bs + i, h, L, H, d);
                        const float* k = K + tok(b, (int)lut[blk].y * bs + j, h, L, H, d);
                        float sum = 0;
                        for (int n = 0; n < d; n++) sum += q[n] * k[n];
                        s[i * bs + j] = sum;
                    }
            }
        }
}

/* ewops.h:64-98 over the sparse storage, rows gathered through the NN LUT. */
void orc_masked_softmax(float* P, const float* S, const orc_uint2* nn_lut,
                        const void* mask_block_major, int mask_word_bytes,
                        const int32_t* valid_len, int B, int H, int nb, int bs, uint32_t blocks,
                        float scale, int lut_heads, int mask_heads) {
    for (int b = 0; b < B; b++)
        for (int h = 0; h < H; h++) {
            const orc_uint2* lut = nn_lut + (lut_heads > 1 ? (size_t)h * (blocks + nb) : 0);
            const void* mask = NULL;
            if (mask_block_major) {
                size_t head_words = mask_heads > 1 ? (size_t)h * blocks * bs : 0;
                mask = (const char*)mask_block_major + head_words * (size_t)mask_word_bytes;
            }
            int valid = valid_len ? valid_len[b] : nb * bs;
            const float* s = S + ((size_t)b * H + h) * blocks * bs * bs;
            float* p = P + ((size_t)b * H + h) * blocks * bs * bs;
            for (int r = 0; r < nb; r++) {
                uint32_t offset = lut[r].x, count = lut[r].y;
                for (int qi = 0; qi < bs; qi++) {
                    float max = -1000000.0f;
                    for (uint32_t jj = 0; jj < count; jj++) {
                        uint32_t blk = lut[offset + jj].x, col = lut[offset + jj].y;
                        for (int kk = 0; kk < bs; kk++) {
                            int keep = mask_bit(mask, mask_word_bytes, (size_t)blk * bs + qi, kk) &&
                                       (int)col * bs + kk < valid;
                            float v = s[((size_t)blk * bs + qi) * bs + kk];
                            if (keep && v > max) max = v;
                        }
                    }
                    float sum_of_c = 0.0f;
                    for (uint32_t jj = 0; jj < count; jj++) {
                        uint32_t blk = lut[offset + jj].x, col = lut[offset + jj].y;
                        for (int kk = 0; kk < bs; kk++) {
                            int keep = mask_bit(mask, mask_word_bytes, (size_t)blk * bs + qi, kk) &&
                                       (int)col * bs + kk < valid;
                            size_t at = ((size_t)blk * bs + qi) * bs + kk;
                            p[at] = 0.0f;
                            if (keep) {
                                p[at] = (float)exp((s[at] - max) * scale);
                                sum_of_c += p[at];
                            }
                        }
                    }
                    for (uint32_t jj = 0; jj < count; jj++) {
                        uint32_t blk = lut[offset + jj].x;
                        for (int kk = 0; kk < bs; kk++)
                            p[((size_t)blk * bs + qi) * bs + kk] /= (sum_of_c + 1e-6f);
                    }
                }
            }
        }
}

/* matmul.h:6-20 over the sparse P; block-rows with no blocks produce zeros. */
void orc_dsd_nn(float* O, const float* P, const float* V, const orc_uint2* nn_lut, int B, int L,
                int H, int d, int bs, uint32_t blocks, int lut_heads) {
    int nb = L / bs;
    for (int b = 0; b < B; b++)
        for (int h = 0; h < H; h++) {
            const orc_uint2* lut = nn_lut + (lut_heads > 1 ? (size_t)h * (blocks + nb) : 0);
            const float* p = P + ((size_t)b * H + h) * blocks * bs * bs;
            for (int r = 0; r < nb; r++) {
                uint32_t offset = lut[r].x, count = lut[r].y;
                for (int qi = 0; qi < bs; qi++) {
                    float* o = O + tok(b, r * bs + qi, h, L, H, d);
                    for (int m = 0; m < d; m++) {
                        float sum = 0;
                        for (uint32_t jj = 0; jj < count; jj++) {
                            uint32_t blk = lut[offset + jj].x, col = lut[offset + jj].y;
                            for (int kk = 0; kk < bs; kk++)
                                sum += p[((size_t)blk * bs + qi) * bs + kk] *
                                       V[tok(b, (int)col * bs + kk, h, L, H, d) + m];
                        }
                        o[m] = sum;
                    }
                }
            }
        }
}

/* ewops.h:101-124 over the sparse storage: per query row sum = sum_k dy*y (float, ascending key; masked
 * keys hold y = 0 and add nothing), out = (dy - sum) * y * scaler. */
void orc_masked_softmax_grad(float* dS, const float* dP, const float* P, const orc_uint2* nn_lut, int B,
                             int H, int nb, int bs, uint32_t blocks, float scale, int lut_heads) {
    for (int b = 0; b < B; b++)
        for (int h = 0; h < H; h++) {
            const orc_uint2* lut = nn_lut + (lut_heads > 1 ? (size_t)h * (blocks + nb) : 0);
            const size_t base = ((size_t)b * H + h) * blocks * bs * bs;
            for (int r = 0; r < nb; r++) {
                uint32_t offset = lut[r].x, count = lut[r].y;
                for (int qi = 0; qi < bs; qi++) {
                    float sum = 0;
                    for (uint32_t jj = 0; jj < count; jj++) {
                        const size_t at = base + ((size_t)lut[offset + jj].x * bs + qi) * bs;
                        for (int kk = 0; kk < bs; kk++) sum += dP[at + kk] * P[at + kk];
                    }
                    for (uint32_t jj = 0; jj < count; jj++) {
                        const size_t at = base + ((size_t)lut[offset + jj].x * bs + qi) * bs;
                        for (int kk = 0; kk < bs; kk++) dS[at + kk] = (dP[at + kk] - sum) * P[at + kk] * scale;
                    }
                }
            }
        }
}

/* matmul.h:81-99 restricted to the blocks of the TN LUT: C[b, c*bs + kk, h, m] = sum over the column's
 * blocks (ascending row block) and their query rows qi (ascending) of A_blk[qi][kk] * X[b, row*bs + qi, h, m],
 * float accumulation in that order. */
void orc_dsd_tn(float* Cout, const float* A, const float* X, const orc_uint2* tn_lut, int B, int L, int H,
                int d, int bs, uint32_t blocks, int lut_heads) {
    int nb = L / bs;
    for (int b = 0; b < B; b++)
        for (int h = 0; h < H; h++) {
            const orc_uint2* lut = tn_lut + (lut_heads > 1 ? (size_t)h * (blocks + nb) : 0);
            const float* a = A + ((size_t)b * H + h) * blocks * bs * bs;
            for (int c = 0; c < nb; c++) {
                uint32_t offset = lut[c].x, count = lut[c].y;
                for (int kk = 0; kk < bs; kk++) {
                    float* out = Cout + tok(b, c * bs + kk, h, L, H, d);
                    for (int m = 0; m < d; m++) {
                        float sum = 0;
                        for (uint32_t jj = 0; jj < count; jj++) {
                            uint32_t blk = lut[offset + jj].x, row = lut[offset + jj].y;
                            for (int qi = 0; qi < bs; qi++)
                                sum += a[((size_t)blk * bs + qi) * bs + kk] *
                                       X[tok(b, (int)row * bs + qi, h, L, H, d) + m];
                        }
                        out[m] = sum;
                    }
                }
            }
        }
}

/* ------------------------------------------------------------------------------------------ */
/* bf16                                                                                        */
/* ------------------------------------------------------------------------------------------ */

uint16_t orc_f32_to_bf16_rne(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7f800000u) == 0x7f800000u && (u & 0x007fffffu)) return (uint16_t)((u >> 16) | 0x40);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

/* ew_op_gpu.h:193-203: the 16 stored bits are the high half of the float. */
float orc_bf16_to_f32(uint16_t x) {
    uint32_t u = (uint32_t)x << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* ew_op_gpu.h:241-254: fma.rz(x, 2^-8-scaled unit, x) then truncate = round half away from zero. */
uint16_t orc_f32_to_bf16_half_away(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7f800000u) == 0x7f800000u) return (uint16_t)(u >> 16);
    u += 0x8000u;
    return (uint16_t)(u >> 16);
}

void orc_round_to_bf16_rne(float* x, long n) {
    for (long i = 0; i < n; i++) x[i] = orc_bf16_to_f32(orc_f32_to_bf16_rne(x[i]));
}

/* ------------------------------------------------------------------------------------------ */
/* encoder-layer ops                                                                           */
/* ------------------------------------------------------------------------------------------ */

/* layernorm.h:13-38: double sums of x and of the float product x*x, float mean, double variance
 * from the float mean squared in float, + 1e-5, double sqrt, float rstd, float affine. */
void orc_layernorm(float* out, float* mean, float* rstd, const float* in, const float* gain,
                   const float* bias, int rows, int state) {
    for (int i = 0; i < rows; i++) {
        double sum_of_row = 0.0, sum_of_row_sqr = 0.0, mean_of_row_sqr = 0.0;
        for (int j = 0; j < state; j++) {
            sum_of_row += in[(size_t)i * state + j];
            sum_of_row_sqr += (in[(size_t)i * state + j] * in[(size_t)i * state + j]);
        }
        float mu = (float)(sum_of_row / state);
        mean_of_row_sqr = sum_of_row_sqr / state;
        float rs = (float)(1.0f / (double)sqrt(mean_of_row_sqr - (mu * mu) + 1e-5));
        if (mean) mean[i] = mu;
        if (rstd) rstd[i] = rs;
        for (int j = 0; j < state; j++)
            out[(size_t)i * state + j] = ((in[(size_t)i * state + j] - mu) * rs) * gain[j] + bias[j];
    }
}

/* ewops.h:32-43: x * 1/(exp(-1.702 x)+1), exp and reciprocal in double, stored to float. */
void orc_gelu(float* out, const float* in, long n) {
    for (long i = 0; i < n; i++) {
        float ex = (float)exp(-(1.702 * in[i]));
        float rcp = (float)(1.0 / (ex + 1.0));
        out[i] = in[i] * rcp;
    }
}

/* ewops.h:10-17: output[i*n+j] = input[i*n+j] + bias[j], m rows of n. */
void orc_bias(float* out, const float* in, const float* bias, int n, int m) {
    for (int i = 0; i < m; i++)
        for (int j = 0; j < n; j++) out[(size_t)i * n + j] = in[(size_t)i * n + j] + bias[j];
}

/* ewops.h:296-301 */
void orc_add(float* out, const float* a, const float* b, long n) {
    for (long i = 0; i < n; i++) out[i] = a[i] + b[i];
}

/* ewops.h:276-282: B broadcast over dim0. */
void orc_add_matrix(float* out, const float* a, const float* b, int dim0, long inner) {
    for (int i = 0; i < dim0; i++)
        for (long j = 0; j < inner; j++) out[i * inner + j] = a[i * inner + j] + b[j];
}

/* embedding.h:5-12 */
void orc_embedding_lookup(float* out, const float* table, const int32_t* ids, long tokens,
                          int state) {
    for (long i = 0; i < tokens; i++)
        for (int j = 0; j < state; j++) out[i * state + j] = table[(size_t)ids[i] * state + j];
}

/* ewops.h:314-331 */
void orc_transpose_0213(const float* src, float* dst, int d0, int d1, int d2, int d3) {
    for (int i = 0; i < d0; i++)
        for (int j = 0; j < d1; j++)
            for (int k = 0; k < d2; k++)
                for (int m = 0; m < d3; m++)
                    dst[(size_t)i * d1 * d2 * d3 + (size_t)k * d1 * d3 + (size_t)j * d3 + m] =
                        src[(size_t)i * d1 * d2 * d3 + (size_t)j * d2 * d3 + (size_t)k * d3 + m];
}

/* Call sites cblas_sgemm(RowMajor,N,N,m,n,k,1,A,k,W,n,0,C,n) at transformer.cpp:516-522,547,562,571.
 * OpenBLAS itself is outside the reference: textbook C = A.W, float accumulation, ascending k. */
void orc_sgemm(float* C, const float* A, const float* W, int m, int n, int k, int nthreads) {
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int i = 0; i < m; i++) {
        float* c = C + (size_t)i * n;
        for (int j = 0; j < n; j++) c[j] = 0.0f;
        for (int p = 0; p < k; p++) {
            float a = A[(size_t)i * k + p];
            const float* w = W + (size_t)p * n;
            for (int j = 0; j < n; j++) c[j] += a * w[j];
        }
    }
}

static float* rounded_copy(const float* src, long n, int to_bf16) {
    float* p = (float*)malloc(sizeof(float) * (size_t)n);
    memcpy(p, src, sizeof(float) * (size_t)n);
    if (to_bf16) orc_round_to_bf16_rne(p, n);
    return p;
}

/* Op order of transformer.cpp:513-580 (sgemm, bias, attention, out-proj, bias, residual, layernorm,
 * FFN sgemm, bias, gelu, sgemm, bias, residual) rearranged to post-LN, dropout omitted:
 *   x1 = LN1(x + (Attn(xWq+bq, xWk+bk, xWv+bv) Wo + bo));  y = LN2(x1 + (gelu(x1 W1 + b1) W2 + b2)). */
void orc_encoder_layer(float* y, const float* x, const orc_layer_weights* w,
                       const orc_uint2* nn_lut, const void* mask_block_major, int mask_word_bytes,
                       const int32_t* valid_len, int B, int L, int H, int d, int ffn, int bs,
                       uint32_t blocks, int operands_bf16, int nthreads) {
    int m = B * L, n = H * d;
    long mn = (long)m * n, mf = (long)m * ffn;
    int r = operands_bf16;
    float* xr = rounded_copy(x, mn, r);
    float* wq = rounded_copy(w->wq, (long)n * n, r);
    float* wk = rounded_copy(w->wk, (long)n * n, r);
    float* wv = rounded_copy(w->wv, (long)n * n, r);
    float* wo = rounded_copy(w->wo, (long)n * n, r);
    float* w1 = rounded_copy(w->w1, (long)n * ffn, r);
    float* w2 = rounded_copy(w->w2, (long)n * ffn, r);
    float* q = (float*)malloc(sizeof(float) * (size_t)mn);
    float* k = (float*)malloc(sizeof(float) * (size_t)mn);
    float* v = (float*)malloc(sizeof(float) * (size_t)mn);
    float* a = (float*)malloc(sizeof(float) * (size_t)mn);
    float* t = (float*)malloc(sizeof(float) * (size_t)mn);
    float* x1 = (float*)malloc(sizeof(float) * (size_t)mn);
    float* f = (float*)malloc(sizeof(float) * (size_t)mf);

    orc_sgemm(q, xr, wq, m, n, n, nthreads); orc_bias(q, q, w->bq, n, m);
    orc_sgemm(k, xr, wk, m, n, n, nthreads); orc_bias(k, k, w->bk, n, m);
    orc_sgemm(v, xr, wv, m, n, n, nthreads); orc_bias(v, v, w->bv, n, m);
    if (r) { orc_round_to_bf16_rne(q, mn); orc_round_to_bf16_rne(k, mn); orc_round_to_bf16_rne(v, mn); }
    orc_blocksparse_attention(a, q, k, v, nn_lut, mask_block_major, mask_word_bytes, valid_len, B, L,
                              H, d, bs, 1.0f / sqrtf((float)d), 1, blocks + (uint32_t)(L / bs), 1,
                              blocks, nthreads);
    if (r) orc_round_to_bf16_rne(a, mn);
    orc_sgemm(t, a, wo, m, n, n, nthreads); orc_bias(t, t, w->bo, n, m);
    orc_add(t, x, t, mn);
    orc_layernorm(x1, NULL, NULL, t, w->ln1_g, w->ln1_b, m, n);

    float* x1r = rounded_copy(x1, mn, r);
    orc_sgemm(f, x1r, w1, m, ffn, n, nthreads); orc_bias(f, f, w->b1, ffn, m);
    orc_gelu(f, f, mf);
    if (r) orc_round_to_bf16_rne(f, mf);
    orc_sgemm(t, f, w2, m, n, ffn, nthreads); orc_bias(t, t, w->b2, n, m);
    orc_add(t, x1, t, mn);
    orc_layernorm(y, NULL, NULL, t, w->ln2_g, w->ln2_b, m, n);

    free(xr); free(wq); free(wk); free(wv); free(wo); free(w1); free(w2);
    free(q); free(k); free(v); free(a); free(t); free(x1); free(f); free(x1r);
}

/* The reference's own wiring (transformer.cpp:513-580, transformer_inference_part.cpp:209-232), pre-LN,
 * dropout omitted:  a = LN1(x); x1 = x + (Attn(aWq+bq, aWk+bk, aWv+bv) Wo + bo);
 *                   y = x1 + (gelu(LN2(x1) W1 + b1) W2 + b2). */
void orc_encoder_layer_pre_ln(float* y, const float* x, const orc_layer_weights* w,
                              const orc_uint2* nn_lut, const void* mask_block_major, int mask_word_bytes,
                              const int32_t* valid_len, int B, int L, int H, int d, int ffn, int bs,
                              uint32_t blocks, int operands_bf16, int nthreads) {
    int m = B * L, n = H * d;
    long mn = (long)m * n, mf = (long)m * ffn;
    int r = operands_bf16;
    float* wq = rounded_copy(w->wq, (long)n * n, r);
    float* wk = rounded_copy(w->wk, (long)n * n, r);
    float* wv = rounded_copy(w->wv, (long)n * n, r);
    float* wo = rounded_copy(w->wo, (long)n * n, r);
    float* w1 = rounded_copy(w->w1, (long)n * ffn, r);
    float* w2 = rounded_copy(w->w2, (long)n * ffn, r);
    float* a = (float*)malloc(sizeof(float) * (size_t)mn);
    float* q = (float*)malloc(sizeof(float) * (size_t)mn);
    float* k = (float*)malloc(sizeof(float) * (size_t)mn);
    float* v = (float*)malloc(sizeof(float) * (size_t)mn);
    float* t = (float*)malloc(sizeof(float) * (size_t)mn);
    float* x1 = (float*)malloc(sizeof(float) * (size_t)mn);
    float* f = (float*)malloc(sizeof(float) * (size_t)mf);

    orc_layernorm(a, NULL, NULL, x, w->ln1_g, w->ln1_b, m, n);
    if (r) orc_round_to_bf16_rne(a, mn);
    orc_sgemm(q, a, wq, m, n, n, nthreads); orc_bias(q, q, w->bq, n, m);
    orc_sgemm(k, a, wk, m, n, n, nthreads); orc_bias(k, k, w->bk, n, m);
    orc_sgemm(v, a, wv, m, n, n, nthreads); orc_bias(v, v, w->bv, n, m);
    if (r) { orc_round_to_bf16_rne(q, mn); orc_round_to_bf16_rne(k, mn); orc_round_to_bf16_rne(v, mn); }
    orc_blocksparse_attention(a, q, k, v, nn_lut, mask_block_major, mask_word_bytes, valid_len, B, L,
                              H, d, bs, 1.0f / sqrtf((float)d), 1, blocks + (uint32_t)(L / bs), 1,
                              blocks, nthreads);
    if (r) orc_round_to_bf16_rne(a, mn);
    orc_sgemm(t, a, wo, m, n, n, nthreads); orc_bias(t, t, w->bo, n, m);
    orc_add(x1, x, t, mn);

    orc_layernorm(a, NULL, NULL, x1, w->ln2_g, w->ln2_b, m, n);
    if (r) orc_round_to_bf16_rne(a, mn);
    orc_sgemm(f, a, w1, m, ffn, n, nthreads); orc_bias(f, f, w->b1, ffn, m);
    orc_gelu(f, f, mf);
    if (r) orc_round_to_bf16_rne(f, mf);
    orc_sgemm(t, f, w2, m, n, ffn, nthreads); orc_bias(t, t, w->b2, n, m);
    orc_add(y, x1, t, mn);

    free(wq); free(wk); free(wv); free(wo); free(w1); free(w2);
    free(a); free(q); free(k); free(v); free(t); free(x1); free(f);
}

/* cblas_sgemm(RowMajor, NoTrans, Trans, m, n, k, 1, A, k, W, k, 0, C, n)
 * (transformer_inference_part.cpp:236, the tied-embedding logits): C[m][n] = A[m][k] W[n][k]^T, float
 * accumulation in ascending k. */
void orc_sgemm_nt(float* C, const float* A, const float* W, int m, int n, int k, int nthreads) {
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int i = 0; i < m; i++)
        for (int j = 0; j < n; j++) {
            float sum = 0.0f;
            for (int p = 0; p < k; p++) sum += A[(size_t)i * k + p] * W[(size_t)j * k + p];
            C[(size_t)i * n + j] = sum;
        }
}

/* softmax_cross_entropy_with_logits (ewops.h:233-261) with the one-hot matrix of to_one_hot (ewops.h:352-361)
 * given by its label column: per row, exp of every logit (double exp of the float, stored as float), their
 * float sum in ascending column order, D = exp/sum, loss_row = sum_j -(log(D_j) * onehot_j) accumulated in
 * float in column order, D_label -= 1; the result is the float sum of the row losses in row order divided
 * by the row count.  d_out (rows x vocab, may be NULL) receives softmax - onehot; row_loss may be NULL. */
float orc_softmax_cross_entropy(float* d_out, float* row_loss, const float* logits, const int32_t* labels,
                                long rows, int vocab) {
    float* e = (float*)malloc(sizeof(float) * (size_t)vocab);
    float sum_of_loss = 0;
    for (long i = 0; i < rows; i++) {
        const float* a = logits + (size_t)i * vocab;
        float sum_of_row = 0.0f;
        float loss = 0;
        for (int j = 0; j < vocab; j++) {
            e[j] = (float)exp((double)a[j]);
            sum_of_row += e[j];
        }
        for (int j = 0; j < vocab; j++) {
            float dj = e[j] / sum_of_row;
            float lg = (float)log((double)dj);
            int hot = (j == labels[i]) ? 1 : 0;
            if (d_out) d_out[(size_t)i * vocab + j] = dj - (float)hot;
            loss += -(lg * (float)hot);
        }
        if (row_loss) row_loss[i] = loss;
        sum_of_loss += loss;
    }
    free(e);
    return sum_of_loss / (float)rows;
}

/* Forward pass of the whole model in the shape of transformer_inference_part.cpp:190-256 (dropout omitted):
 * x = tok[ids] + pos; n_layers encoder layers (pre_ln != 0: the reference's wiring; 0: post-LN);
 * logits = x tok^T (tied embedding); loss = softmax cross-entropy against labels.  logits (tokens x vocab,
 * may be NULL) and hidden (tokens x state, may be NULL) receive the intermediate results. */
float orc_model_forward(float* logits, float* hidden, const int32_t* ids, const int32_t* labels,
                        const float* tok, const float* pos, const orc_layer_weights* layers, int n_layers,
                        int pre_ln, const orc_uint2* nn_lut, const void* mask_block_major, int mask_word_bytes,
                        const int32_t* valid_len, int B, int L, int H, int d, int ffn, int bs, uint32_t blocks,
                        int vocab, int operands_bf16, int nthreads) {
    long tokens = (long)B * L;
    int n = H * d;
    float* x = (float*)malloc(sizeof(float) * (size_t)tokens * n);
    float* y = (float*)malloc(sizeof(float) * (size_t)tokens * n);
    orc_embedding_lookup(x, tok, ids, tokens, n);
    orc_add_matrix(x, x, pos, B, (long)L * n);
    for (int i = 0; i < n_layers; i++) {
        if (pre_ln)
            orc_encoder_layer_pre_ln(y, x, layers + i, nn_lut, mask_block_major, mask_word_bytes, valid_len, B, L, H,
                                     d, ffn, bs, blocks, operands_bf16, nthreads);
        else
            orc_encoder_layer(y, x, layers + i, nn_lut, mask_block_major, mask_word_bytes, valid_len, B, L, H, d,
                              ffn, bs, blocks, operands_bf16, nthreads);
        float* swap = x; x = y; y = swap;
    }
    if (hidden) memcpy(hidden, x, sizeof(float) * (size_t)tokens * n);
    float* lg = logits ? logits : (float*)malloc(sizeof(float) * (size_t)tokens * vocab);
    float* xr = rounded_copy(x, tokens * n, operands_bf16);
    float* tr = rounded_copy(tok, (long)vocab * n, operands_bf16);
    orc_sgemm_nt(lg, xr, tr, (int)tokens, vocab, n, nthreads);
    float loss = orc_softmax_cross_entropy(NULL, NULL, lg, labels, tokens, vocab);
    if (!logits) free(lg);
    free(xr); free(tr); free(x); free(y);
    return loss;
}

/* ------------------------------------------------------------------------------------------ */
/* seeded data                                                                                 */
/* ------------------------------------------------------------------------------------------ */

void orc_fill_normal(float* x, long n, uint64_t seed, float std) {
    uint64_t state = seed;
    for (long i = 0; i < n; i += 2) {
        double u1 = (double)((splitmix64(&state) >> 11) + 1ull) * (1.0 / 9007199254740992.0);
        double u2 = (double)(splitmix64(&state) >> 11) * (1.0 / 9007199254740992.0);
        double rad = sqrt(-2.0 * log(u1)), ang = 6.283185307179586476925 * u2;
        x[i] = (float)(rad * cos(ang)) * std;
        if (i + 1 < n) x[i + 1] = (float)(rad * sin(ang)) * std;
    }
}

void orc_fill_uniform_int(int32_t* x, long n, uint64_t seed, int32_t lo, int32_t hi) {
    uint64_t state = seed;
    uint64_t span = (uint64_t)(hi - lo) + 1ull;
    for (long i = 0; i < n; i++) x[i] = lo + (int32_t)(splitmix64(&state) % span);
}
