// Host-side sparsity descriptors of libsfbert_hip: block layouts for the full / local / fixed /
// strided / BigBird patterns, the NT and NN look-up tables, the row-block LUT, packed element masks
// in both memory orders, magic-number division constants and the launch order of block-rows.
// Formats are those of the reference's test mains (file:line cited in include/sfbert_hip.h); the
// results must be bit-identical to what those mains build.
#include <algorithm>
#include <cstring>
#include <numeric>
#include <vector>

#include "../../include/sfbert_hip.h"

namespace {

template <typename Pred>
void fill_layout(uint32_t* layout, int nb, Pred keep) {
    for (int row = 0; row < nb; ++row)
        for (int col = 0; col < nb; ++col) layout[(size_t)row * nb + col] = keep(row, col) ? 1u : 0u;
}

std::vector<char> global_blocks(int nb, int nglobal, bool both_ends) {
    std::vector<char> g((size_t)nb, 0);
    if (!both_ends) {
        for (int i = 0; i < std::min(nglobal, nb); ++i) g[i] = 1;
    } else {
        const int head = (nglobal + 1) / 2, tail = nglobal / 2;
        for (int i = 0; i < std::min(head, nb); ++i) g[i] = 1;
        for (int i = 0; i < std::min(tail, nb); ++i) g[nb - 1 - i] = 1;
    }
    return g;
}

struct SplitMix64 {
    uint64_t state;
    uint64_t next() {
        uint64_t z = (state += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
};

// one mask word per (block, row): uchar / ushort / uint / uint64 for block 8 / 16 / 32 / 64 (blocksparse.h:684-720)
inline int word_bytes_for(int bs) { return bs == 64 ? 8 : bs == 32 ? 4 : bs == 16 ? 2 : bs == 8 ? 1 : 0; }

}  // namespace

extern "C" {

const char* sfb_status_string(int status) {
    switch (status) {
        case SFB_OK: return "ok";
        case SFB_ERR_NULL_POINTER: return "a required pointer is NULL";
        case SFB_ERR_BLOCK_SIZE: return "unsupported block size";
        case SFB_ERR_HEAD_STATE: return "unsupported head state size";
        case SFB_ERR_SHAPE: return "zero or inconsistent dimensions";
        case SFB_ERR_DTYPE: return "unsupported element type";
        case SFB_ERR_ALIGNMENT: return "tensor pointer not 16-byte aligned";
        case SFB_ERR_LAUNCH: return "kernel launch failed";
        case SFB_ERR_ARGUMENT: return "invalid argument";
        case SFB_ERR_WORKSPACE: return "workspace missing or too small";
        case SFB_ERR_SCRATCH_LIMIT: return "the launch needs more scratch than the library's static device array holds";
        default: return "unknown status";
    }
}

int sfb_layout_full(uint32_t* layout, int nb, int causal) {
    if (!layout) return SFB_ERR_NULL_POINTER;
    if (nb <= 0) return SFB_ERR_SHAPE;
    fill_layout(layout, nb, [&](int r, int c) { return !causal || c <= r; });
    return SFB_OK;
}

int sfb_layout_local(uint32_t* layout, int nb, int extra_diag, int bidirectional) {
    if (!layout) return SFB_ERR_NULL_POINTER;
    if (nb <= 0 || extra_diag < 0) return SFB_ERR_SHAPE;
    if (bidirectional) {
        fill_layout(layout, nb, [&](int r, int c) { return std::abs(r - c) <= extra_diag; });
    } else {
        // extra_diag == 0 disables the lower cut in the reference, leaving the full causal triangle
        fill_layout(layout, nb, [&](int r, int c) {
            return c <= r && (extra_diag == 0 || c + extra_diag >= r);
        });
    }
    return SFB_OK;
}

int sfb_layout_fixed(uint32_t* layout, int heads, int nb, int stride, int causal) {
    if (!layout) return SFB_ERR_NULL_POINTER;
    if (nb <= 0 || heads <= 0 || stride <= 0) return SFB_ERR_SHAPE;
    for (int h = 0; h < heads; ++h) {
        int phase = stride - (h + 1);
        phase = ((phase % stride) + stride) % stride;
        fill_layout(layout + (size_t)h * nb * nb, nb, [&](int r, int c) {
            const bool summary = (c % stride) == phase;
            const bool own_chunk = (c / stride) == (r / stride);
            return (summary || own_chunk) && (!causal || c <= r);
        });
    }
    return SFB_OK;
}

int sfb_layout_strided_chunks(uint32_t* layout, int nb, int block_chunks) {
    if (!layout) return SFB_ERR_NULL_POINTER;
    if (nb <= 0 || block_chunks <= 0) return SFB_ERR_SHAPE;
    fill_layout(layout, nb, [&](int r, int c) { return c <= r && c + (r % block_chunks) >= r; });
    return SFB_OK;
}

int sfb_layout_strided(uint32_t* layout, int nb, int band, int stride, int causal) {
    if (!layout) return SFB_ERR_NULL_POINTER;
    if (nb <= 0 || band <= 0 || stride <= 0) return SFB_ERR_SHAPE;
    fill_layout(layout, nb, [&](int r, int c) {
        const int diff = r - c;
        if (diff >= 0 && diff < band) return true;
        if (causal && diff < 0) return false;
        return (std::abs(diff) % stride) == 0;
    });
    return SFB_OK;
}

int sfb_layout_bigbird(uint32_t* layout, int nb, int window, int nglobal, int global_both_ends,
                       const int32_t* rand_cols, int nrand) {
    if (!layout) return SFB_ERR_NULL_POINTER;
    if (nb <= 0 || window < 0 || nglobal < 0 || nrand < 0) return SFB_ERR_SHAPE;
    const std::vector<char> g = global_blocks(nb, nglobal, global_both_ends != 0);
    fill_layout(layout, nb, [&](int r, int c) { return std::abs(r - c) <= window || g[r] || g[c]; });
    if (rand_cols) {
        for (int r = 0; r < nb; ++r)
            for (int t = 0; t < nrand; ++t) {
                const int32_t c = rand_cols[(size_t)r * nrand + t];
                if (c >= 0 && c < nb) layout[(size_t)r * nb + c] = 1u;
            }
    }
    return SFB_OK;
}

int sfb_bigbird_draw(int32_t* rand_cols, int nb, int window, int nglobal, int global_both_ends,
                     int nrand, uint64_t seed) {
    if (!rand_cols) return SFB_ERR_NULL_POINTER;
    if (nb <= 0 || window < 0 || nglobal < 0 || nrand < 0) return SFB_ERR_SHAPE;
    const std::vector<char> g = global_blocks(nb, nglobal, global_both_ends != 0);
    SplitMix64 rng{seed};
    std::vector<int32_t> candidates;
    for (int r = 0; r < nb; ++r) {
        candidates.clear();
        if (!g[r])
            for (int c = 0; c < nb; ++c)
                if (std::abs(r - c) > window && !g[c]) candidates.push_back(c);
        const int avail = (int)candidates.size();
        for (int t = 0; t < nrand; ++t) {
            if (t >= avail) {
                rand_cols[(size_t)r * nrand + t] = -1;
                continue;
            }
            const int pick = t + (int)(rng.next() % (uint64_t)(avail - t));
            std::swap(candidates[t], candidates[pick]);
            rand_cols[(size_t)r * nrand + t] = candidates[t];
        }
    }
    return SFB_OK;
}

uint32_t sfb_count_blocks(const uint32_t* layout, int nb) {
    if (!layout || nb <= 0) return 0;
    return (uint32_t)std::count(layout, layout + (size_t)nb * nb, 1u);
}

int sfb_build_nt_lut(sfb_uint2* nt_lut, const uint32_t* layout, int nb) {
    if (!nt_lut || !layout) return SFB_ERR_NULL_POINTER;
    if (nb <= 0) return SFB_ERR_SHAPE;
    sfb_uint2* out = nt_lut;
    for (int r = 0; r < nb; ++r)
        for (int c = 0; c < nb; ++c)
            if (layout[(size_t)r * nb + c] == 1u) *out++ = sfb_uint2{(uint32_t)r, (uint32_t)c};
    return SFB_OK;
}

int sfb_build_nn_lut(sfb_uint2* nn_lut, const sfb_uint2* nt_lut, uint32_t blocks, int nb,
                     uint32_t* nn_max) {
    if (!nn_lut || (!nt_lut && blocks)) return SFB_ERR_NULL_POINTER;
    if (nb <= 0) return SFB_ERR_SHAPE;
    std::vector<uint32_t> count((size_t)nb, 0u);
    for (uint32_t id = 0; id < blocks; ++id) {
        if (nt_lut[id].x >= (uint32_t)nb) return SFB_ERR_ARGUMENT;
        ++count[nt_lut[id].x];
        nn_lut[(size_t)nb + id] = sfb_uint2{id, nt_lut[id].y};
    }
    uint32_t offset = (uint32_t)nb, longest = nn_max ? *nn_max : 0u;
    for (int r = 0; r < nb; ++r) {
        nn_lut[r] = sfb_uint2{offset, count[r]};
        offset += count[r];
        longest = std::max(longest, count[r]);
    }
    if (nn_max) *nn_max = longest;
    return SFB_OK;
}

int sfb_build_rblk_lut(sfb_uint2* rblk_lut, const sfb_uint2* nn_lut, int nb) {
    if (!rblk_lut || !nn_lut) return SFB_ERR_NULL_POINTER;
    if (nb <= 0) return SFB_ERR_SHAPE;
    uint32_t id = 0;
    for (int r = 0; r < nb; ++r)
        for (uint32_t j = 0; j < nn_lut[r].y; ++j, ++id) rblk_lut[id] = sfb_uint2{id, (uint32_t)r};
    return SFB_OK;
}

int sfb_build_tn_lut(sfb_uint2* tn_lut, const sfb_uint2* nt_lut, uint32_t blocks, int nb, uint32_t* tn_max) {
    if (!tn_lut || !nt_lut) return SFB_ERR_NULL_POINTER;
    if (nb <= 0) return SFB_ERR_SHAPE;
    // bucket the blocks by column; the NT table is a row-major scan, so rows come out ascending
    std::vector<uint32_t> count((size_t)nb, 0u);
    for (uint32_t blk = 0; blk < blocks; ++blk) {
        if (nt_lut[blk].y >= (uint32_t)nb || nt_lut[blk].x >= (uint32_t)nb) return SFB_ERR_ARGUMENT;
        ++count[nt_lut[blk].y];
    }
    uint32_t offset = (uint32_t)nb, longest = 0;
    std::vector<uint32_t> next((size_t)nb);
    for (int c = 0; c < nb; ++c) {
        tn_lut[c] = sfb_uint2{offset, count[c]};
        next[c] = offset;
        offset += count[c];
        if (count[c] > longest) longest = count[c];
    }
    for (uint32_t blk = 0; blk < blocks; ++blk) tn_lut[next[nt_lut[blk].y]++] = sfb_uint2{blk, nt_lut[blk].x};
    if (tn_max) *tn_max = longest;
    return SFB_OK;
}

void sfb_magicu64(uint32_t d, uint32_t* magic, uint32_t* shift) {
    if (!magic || !shift || d == 0) return;
    if (d <= 8 && (d & (d - 1)) == 0) {  // 1, 2, 4, 8: plain shifts
        *magic = 1;
        *shift = d == 1 ? 0 : d == 2 ? 1 : d == 4 ? 2 : 3;
        return;
    }
    // smallest p with 2^p > nc * (d - 1 - (2^p - 1) mod d); 3 needs the full 32-bit range
    const uint32_t nbits = d == 3 ? 65 : 63;
    const uint64_t nmax = d == 3 ? 0xffffffffull : 0x7fffffffull;
    const uint64_t dd = d;
    const uint64_t nc = ((nmax + 1) / dd) * dd - 1;
    for (uint32_t p = 0; p < nbits; ++p) {
        const uint64_t two_p = 1ull << p;
        const uint64_t rem = dd - 1 - (two_p - 1) % dd;
        if (two_p > nc * rem) {
            *magic = (uint32_t)((two_p + rem) / dd);
            *shift = *magic == 1 ? p : p - 32;
            return;
        }
    }
}

int sfb_element_mask(uint8_t* keep, const sfb_uint2* nt_lut, uint32_t blocks, int bs, int kind,
                     int local_attn_ctx) {
    if (!keep || (!nt_lut && blocks)) return SFB_ERR_NULL_POINTER;
    if (bs <= 0) return SFB_ERR_BLOCK_SIZE;
    if (kind < 0 || kind > 3) return SFB_ERR_ARGUMENT;
    for (uint32_t id = 0; id < blocks; ++id) {
        const uint32_t rb = nt_lut[id].x, cb = nt_lut[id].y;
        uint8_t* blk = keep + (size_t)id * bs * bs;
        for (int i = 0; i < bs; ++i)
            for (int j = 0; j < bs; ++j) {
                bool k = true;
                if (kind == 1) k = (rb != cb) || j <= i;
                else if (kind == 3) k = j <= i;
                else if (kind == 2) {
                    const uint32_t row = rb * (uint32_t)bs + (uint32_t)i, col = cb * (uint32_t)bs + (uint32_t)j;
                    k = col <= row && col + (uint32_t)local_attn_ctx > row;
                }
                blk[i * bs + j] = k ? 1 : 0;
            }
    }
    return SFB_OK;
}

int sfb_pack_mask(void* words, const uint8_t* keep, uint32_t blocks, int bs) {
    if (!words || !keep) return SFB_ERR_NULL_POINTER;
    const int wb = word_bytes_for(bs);
    if (!wb) return SFB_ERR_BLOCK_SIZE;
    const size_t rows = (size_t)blocks * bs;
    for (size_t row = 0; row < rows; ++row) {
        uint64_t w = 0;
        const uint8_t* src = keep + row * bs;
        for (int j = 0; j < bs; ++j) w |= (uint64_t)(src[j] != 0) << j;
        if (wb == 8) static_cast<uint64_t*>(words)[row] = w;
        else if (wb == 4) static_cast<uint32_t*>(words)[row] = (uint32_t)w;
        else if (wb == 2) static_cast<uint16_t*>(words)[row] = (uint16_t)w;
        else static_cast<uint8_t*>(words)[row] = (uint8_t)w;
    }
    return SFB_OK;
}

int sfb_transpose_mask(void* row_major, const void* block_major, uint32_t blocks, int bs) {
    if (!row_major || !block_major) return SFB_ERR_NULL_POINTER;
    const int wb = word_bytes_for(bs);
    if (!wb) return SFB_ERR_BLOCK_SIZE;
    const char* src = static_cast<const char*>(block_major);
    char* dst = static_cast<char*>(row_major);
    for (uint32_t id = 0; id < blocks; ++id)
        for (int row = 0; row < bs; ++row)
            std::memcpy(dst + ((size_t)row * blocks + id) * wb, src + ((size_t)id * bs + row) * wb, wb);
    return SFB_OK;
}

int sfb_build_row_order(uint32_t* row_order, const sfb_uint2* nn_lut, int nb) {
    if (!row_order || !nn_lut) return SFB_ERR_NULL_POINTER;
    if (nb <= 0) return SFB_ERR_SHAPE;
    std::iota(row_order, row_order + nb, 0u);
    std::stable_sort(row_order, row_order + nb,
                     [&](uint32_t a, uint32_t b) { return nn_lut[a].y > nn_lut[b].y; });
    return SFB_OK;
}

uint32_t sfb_suggest_max_blocks(const sfb_uint2* nn_lut, int nb, uint32_t batch_heads) {
    if (!nn_lut || nb <= 0 || batch_heads == 0) return 16;
    // The device keeps 256 x 4 work-groups of the fused kernel resident.  A work item should not be longer than
    // what one of those slots gets to do in the whole launch (else it alone decides when the launch ends), and
    // every cut costs a partial record, a device-wide counter update and a share of a merge, so rows are cut into
    // as few chunks as that allows; with few (batch, head) pairs the chunks stay at 16 key blocks so that the
    // long rows spread over the idle slots.
    constexpr uint64_t kResidentWorkGroups = 1024;
    uint64_t total = 0;
    for (int r = 0; r < nb; ++r) total += nn_lut[r].y;
    const uint64_t per_slot = (5 * total * batch_heads + 4 * kResidentWorkGroups - 1) / (4 * kResidentWorkGroups);
    return (uint32_t)(per_slot > 16 ? (per_slot < 0xffffffffull ? per_slot : 0xffffffffull) : 16);
}

}  // extern "C"

// Work items of one head's NN look-up table, longest first; *slots / *parts count the split rows and their chunks.
static std::vector<sfb_work_item> work_items_of(const sfb_uint2* nn_lut, int nb, uint32_t max_blocks,
                                                uint32_t* slots_out, uint32_t* parts_out) {
    std::vector<sfb_work_item> all;
    uint32_t slots = 0, parts = 0;
    for (int r = 0; r < nb; ++r) {
        const uint32_t count = nn_lut[r].y;
        const uint32_t chunks = count > max_blocks ? (count + max_blocks - 1) / max_blocks : 1;
        if (chunks == 1) {
            all.push_back(sfb_work_item{(uint32_t)r, 0u, count, 1u, 0u, 0u, 0u, nn_lut[r].x});
            continue;
        }
        const uint32_t base = count / chunks, extra = count % chunks;
        uint32_t first = 0;
        for (uint32_t c = 0; c < chunks; ++c) {
            const uint32_t len = base + (c < extra ? 1u : 0u);
            all.push_back(sfb_work_item{(uint32_t)r, first, len, chunks, c, slots, parts, nn_lut[r].x + first});
            first += len;
        }
        ++slots;
        parts += chunks;
    }
    std::stable_sort(all.begin(), all.end(),
                     [](const sfb_work_item& a, const sfb_work_item& b) { return a.count > b.count; });
    *slots_out = slots;
    *parts_out = parts;
    return all;
}

extern "C" {

int sfb_build_plan(sfb_plan_entry* plan, uint32_t* plan_stride, uint32_t* n_slots, uint32_t* n_parts,
                   const sfb_uint2* nn_lut, int nb, uint32_t lut_heads, uint32_t lut_dim, uint32_t batch_dim,
                   uint32_t head_dim, uint32_t wg_slots, uint32_t max_blocks) {
    if (!plan_stride || !n_slots || !n_parts || !nn_lut) return SFB_ERR_NULL_POINTER;
    if (nb <= 0 || batch_dim == 0 || head_dim == 0 || wg_slots == 0 || lut_heads == 0) return SFB_ERR_SHAPE;
    if (lut_heads > 1 && lut_heads != head_dim) return SFB_ERR_SHAPE;
    if (max_blocks == 0) return SFB_ERR_ARGUMENT;
    const uint64_t num_bh64 = (uint64_t)batch_dim * head_dim;
    if (num_bh64 > 0x7fffffffull) return SFB_ERR_SHAPE;
    const uint32_t num_bh = (uint32_t)num_bh64;

    // item tables: one per look-up table (shared by all heads, or one per head)
    std::vector<std::vector<sfb_work_item>> tables(lut_heads);
    uint32_t slots = 0, parts = 0;
    for (uint32_t h = 0; h < lut_heads; ++h) {
        uint32_t s = 0, q = 0;
        tables[h] = work_items_of(nn_lut + (size_t)h * lut_dim, nb, max_blocks, &s, &q);
        slots = std::max(slots, s);
        parts = std::max(parts, q);
    }

    // A work item costs its key blocks plus a fixed charge (start-up, write-out) of about two key blocks' time.
    constexpr uint64_t kItemCharge = 2;
    // Slots are dealt to the 8 dies like consecutive work-group ids; a (batch, head) whose index has residue x
    // mod 8 is worked on by the slots of die x only, so its K and V stay in one L2.  The last batch*heads % 8
    // pairs have no die of their own and go wherever the load is smallest.
    const uint32_t dies = (wg_slots % 8 == 0 && num_bh >= 8) ? 8 : 1;
    const uint32_t bound_bh = dies == 8 ? num_bh - num_bh % 8 : num_bh;
    std::vector<std::vector<sfb_plan_entry>> lists(wg_slots);
    std::vector<uint64_t> load(wg_slots, 0);
    auto place = [&](uint32_t bh, const sfb_work_item& it) {
        uint32_t best = 0xffffffffu;
        const bool bound = dies == 8 && bh < bound_bh;
        for (uint32_t s = bound ? bh % 8 : 0; s < wg_slots; s += bound ? 8 : 1)
            if (best == 0xffffffffu || load[s] < load[best]) best = s;
        lists[best].push_back(sfb_plan_entry{bh / head_dim, bh % head_dim, it.row, it.first, it.count, it.nchunks,
                                             it.chunk, it.slot, it.part, it.lut_first, {0u, 0u}});
        load[best] += it.count + kItemCharge;
    };
    auto table_of = [&](uint32_t bh) { return lut_heads > 1 ? bh % head_dim : 0u; };
    // long items (at least twice the median) of every (batch, head) first, longest first; then the rest, one
    // (batch, head) after the other, so that the slots of a die work on the same few heads at any time
    std::vector<uint32_t> heavy(lut_heads, 0);
    uint32_t longest = 0;
    for (uint32_t h = 0; h < lut_heads; ++h) {
        const auto& tb = tables[h];
        if (tb.empty()) continue;
        const uint32_t median = tb[tb.size() / 2].count;
        while (heavy[h] < tb.size() && tb[heavy[h]].count >= 2 * median && tb[heavy[h]].count > median) ++heavy[h];
        longest = std::max(longest, tb[0].count);
    }
    for (uint32_t len = longest; len > 0; --len)
        for (uint32_t bh = 0; bh < num_bh; ++bh) {
            const uint32_t h = table_of(bh);
            for (uint32_t i = 0; i < heavy[h]; ++i)
                if (tables[h][i].count == len) place(bh, tables[h][i]);
        }
    for (uint32_t bh = 0; bh < num_bh; ++bh) {
        const uint32_t h = table_of(bh);
        for (uint32_t i = heavy[h]; i < tables[h].size(); ++i) place(bh, tables[h][i]);
    }
    uint32_t stride = 0;
    for (const auto& l : lists) stride = std::max(stride, (uint32_t)l.size());
    stride += 2;   // two end marks: a work-group reads two entries ahead

    if (plan) {
        if (*plan_stride < stride) return SFB_ERR_ARGUMENT;
        const sfb_plan_entry end = {0u, 0u, 0u, 0u, 0xffffffffu, 0u, 0u, 0u, 0u, 0u, {0u, 0u}};
        for (uint32_t s = 0; s < wg_slots; ++s)
            for (uint32_t i = 0; i < stride; ++i)
                plan[(size_t)s * stride + i] = i < lists[s].size() ? lists[s][i] : end;
    }
    *plan_stride = stride;
    *n_slots = slots;
    *n_parts = parts;
    return SFB_OK;
}

int sfb_build_schedule(sfb_work_item* items, uint32_t* n_items, uint32_t* n_heavy, uint32_t* n_slots,
                       uint32_t* n_parts, const sfb_uint2* nn_lut, int nb, uint32_t max_blocks) {
    if (!n_items || !n_heavy || !n_slots || !n_parts || !nn_lut) return SFB_ERR_NULL_POINTER;
    if (nb <= 0) return SFB_ERR_SHAPE;
    if (max_blocks == 0) return SFB_ERR_ARGUMENT;
    std::vector<sfb_work_item> all;
    uint32_t slots = 0, parts = 0;
    for (int r = 0; r < nb; ++r) {
        const uint32_t count = nn_lut[r].y;
        const uint32_t chunks = count > max_blocks ? (count + max_blocks - 1) / max_blocks : 1;
        if (chunks == 1) {
            all.push_back(sfb_work_item{(uint32_t)r, 0u, count, 1u, 0u, 0u, 0u, nn_lut[r].x});
            continue;
        }
        const uint32_t base = count / chunks, extra = count % chunks;
        uint32_t first = 0;
        for (uint32_t c = 0; c < chunks; ++c) {
            const uint32_t len = base + (c < extra ? 1u : 0u);
            all.push_back(sfb_work_item{(uint32_t)r, first, len, chunks, c, slots, parts, nn_lut[r].x + first});
            first += len;
        }
        ++slots;
        parts += chunks;
    }
    std::stable_sort(all.begin(), all.end(),
                     [](const sfb_work_item& a, const sfb_work_item& b) { return a.count > b.count; });
    if (items) {
        if (*n_items < all.size()) return SFB_ERR_ARGUMENT;
        std::copy(all.begin(), all.end(), items);
    }
    // items at least twice as long as the median item are "heavy"
    const uint32_t median = all[all.size() / 2].count;
    uint32_t heavy = 0;
    while (heavy + 1 < all.size() && all[heavy].count >= 2 * median && all[heavy].count > median) ++heavy;
    *n_heavy = heavy;
    *n_items = (uint32_t)all.size();
    *n_slots = slots;
    *n_parts = parts;
    return SFB_OK;
}

}  // extern "C"
