// Host-side sparsity descriptors of libsfbert_hip: block layouts for the full / local / fixed /
// strided / BigBird patterns, the NT and NN look-up tables, the row-block LUT, packed element masks
// in both memory orders, magic-number division constants and the launch order of block-rows.
// Formats are those of the reference's test mains (file:line cited in include/sfbert_hip.h); the
// results must be bit-identical to what those mains build.
#include <algorithm>
#include <cmath>
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

extern "C" {

// ------------------------------------------------------------------------------------------------
// Streams of a launch whose work-groups stay resident
// ------------------------------------------------------------------------------------------------
}  // extern "C"

namespace {

struct StreamRow {
    uint32_t bh, row, count, lut_first;
};
struct StreamPiece {      // an item as it is being placed
    uint32_t bh, row, first, count, lut_first;
    uint32_t nchunks, chunk, part;
};
struct StreamMerge {
    uint32_t bh, row, part, nparts;
};

constexpr double kItemCharge = 1.0;     // start and end of an item, in key blocks' time
constexpr double kPartialCharge = 0.5;  // writing a partial record
constexpr double kMergeBase = 2.0, kMergePerPart = 1.0;
constexpr uint32_t kMinChunk = 2;       // no chunk shorter than this unless the row is

uint32_t least_loaded(const std::vector<uint32_t>& slots, const std::vector<double>& load) {
    uint32_t best = slots[0];
    for (uint32_t s : slots)
        if (load[s] < load[best]) best = s;
    return best;
}

// Places rows (any order) on the given slots.  Rows that fit are placed whole, longest first, each on the least
// loaded slot.  Rows too long for that are cut: `level` = true pours them into the slots up to a common level (one
// chunk per slot, as long as the slot's room allows, so the streams end together at the price of many partial
// records); false cuts each into the fewest near-equal chunks that fit a slot's share and places the chunks like
// rows (few records, streams differ by up to a short row).  Cut rows get partial-record indices from *parts on and
// one merge task each.
void place_rows(std::vector<StreamRow> rows, const std::vector<uint32_t>& slots, std::vector<double>& load,
                std::vector<std::vector<StreamPiece>>& whole, std::vector<std::vector<StreamPiece>>& chunks,
                std::vector<std::vector<StreamMerge>>& merges, uint32_t* parts, bool level, double tail,
                std::vector<StreamRow>* late_rows, std::vector<StreamMerge>* late_merges) {
    if (rows.empty()) return;
    std::stable_sort(rows.begin(), rows.end(), [](const StreamRow& a, const StreamRow& b) { return a.count > b.count; });
    double total = 0;
    for (uint32_t s : slots) total += load[s];
    for (const StreamRow& r : rows) total += r.count + kItemCharge;
    const double share = total / (double)slots.size();
    // a row is "long" when it alone would take more than 0.6 of a slot's share
    size_t n_long = 0;
    while (n_long < rows.size() && rows[n_long].count + kItemCharge > 0.6 * share && rows[n_long].count >= 2 * kMinChunk)
        ++n_long;
    // tail > 0 (chunks of long rows and whole rows alike): the streams are only filled up to (1 - tail) of their
    // share; the rows that do not fit any more -- the shortest ones -- and the merges are handed back
    const double cap = (!level && tail > 0) ? share * (1.0 - tail) : 1e300;
    auto place_whole = [&](const StreamRow& r) {
        const uint32_t s = least_loaded(slots, load);
        if (load[s] + r.count + kItemCharge > cap) { late_rows->push_back(r); return; }
        whole[s].push_back(StreamPiece{r.bh, r.row, 0u, r.count, r.lut_first, 1u, 0u, 0u});
        load[s] += r.count + kItemCharge;
    };
    auto place_cut = [&](const StreamRow& r, const std::vector<std::pair<uint32_t, StreamPiece>>& placed, uint32_t merger) {
        for (size_t c = 0; c < placed.size(); ++c) {
            StreamPiece pc = placed[c].second;
            pc.nchunks = (uint32_t)placed.size();
            pc.chunk = (uint32_t)c;
            pc.part = *parts + (uint32_t)c;
            chunks[placed[c].first].push_back(pc);
        }
        if (merger == 0xffffffffu) late_merges->push_back(StreamMerge{r.bh, r.row, *parts, (uint32_t)placed.size()});
        else merges[merger].push_back(StreamMerge{r.bh, r.row, *parts, (uint32_t)placed.size()});
        *parts += (uint32_t)placed.size();
    };
    if (!level) {
        // chunks of long rows and whole rows alike, longest first, each on the least loaded slot
        size_t next_short = n_long;
        for (size_t i = 0; i < n_long; ++i) {
            const StreamRow& r = rows[i];
            const uint32_t pieces = std::min<uint32_t>(r.count / kMinChunk, std::max<uint32_t>(2u, (uint32_t)std::ceil((r.count + kItemCharge) / share)));
            const uint32_t base = r.count / pieces, extra = r.count % pieces;
            while (next_short < rows.size() && rows[next_short].count > base + 1) place_whole(rows[next_short++]);
            std::vector<std::pair<uint32_t, StreamPiece>> placed;
            uint32_t first = 0;
            for (uint32_t c = 0; c < pieces; ++c) {
                const uint32_t len = base + (c < extra ? 1u : 0u);
                const uint32_t s = least_loaded(slots, load);
                placed.push_back({s, StreamPiece{r.bh, r.row, first, len, r.lut_first + first, 0u, 0u, 0u}});
                load[s] += len + kItemCharge + kPartialCharge;
                first += len;
            }
            uint32_t m = 0xffffffffu;
            if (cap > 1e299) {
                m = least_loaded(slots, load);
                load[m] += kMergeBase + kMergePerPart * pieces;
            }
            place_cut(r, placed, m);
        }
        for (size_t i = next_short; i < rows.size(); ++i) place_whole(rows[i]);
        return;
    }
    for (size_t i = n_long; i < rows.size(); ++i) place_whole(rows[i]);
    if (n_long == 0) return;
    // mergers first (the least loaded slots), charged with a guess at their work
    double volume = 0;
    for (size_t i = 0; i < n_long; ++i) volume += rows[i].count;
    const double room_guess = std::max((double)kMinChunk, volume / (double)slots.size());
    std::vector<uint32_t> merger(n_long);
    for (size_t i = 0; i < n_long; ++i) {
        merger[i] = least_loaded(slots, load);
        load[merger[i]] += kMergeBase + kMergePerPart * std::max(2.0, std::ceil(rows[i].count / room_guess));
    }
    // the level up to which the slots are filled: sum over slots of the room (where it is at least a chunk) = volume
    const double fixed = kItemCharge + kPartialCharge;
    double lo = 0, hi = 0;
    for (uint32_t s : slots) hi = std::max(hi, load[s]);
    hi += volume + fixed + kMinChunk;
    for (int it = 0; it < 60; ++it) {
        const double mid = 0.5 * (lo + hi);
        double got = 0;
        for (uint32_t s : slots) {
            const double room = std::floor(mid - load[s] - fixed);
            if (room >= kMinChunk) got += room;
        }
        (got >= volume ? hi : lo) = mid;
    }
    const double water = hi;
    // slots in the order of their room, most first; the long rows one after the other
    std::vector<uint32_t> order(slots);
    std::stable_sort(order.begin(), order.end(), [&](uint32_t a, uint32_t b) { return load[a] < load[b]; });
    size_t next_slot = 0;
    for (size_t i = 0; i < n_long; ++i) {
        const StreamRow& r = rows[i];
        std::vector<std::pair<uint32_t, StreamPiece>> placed;
        uint32_t first = 0;
        while (first < r.count) {
            uint32_t s;
            uint32_t take;
            const uint32_t remaining = r.count - first;
            if (next_slot < order.size()) {
                s = order[next_slot];
                const double room = std::floor(water - load[s] - fixed);
                if (room < kMinChunk) { ++next_slot; continue; }   // used up by the row before
                take = (uint32_t)room;
                if (take >= remaining) take = remaining;          // the slot keeps room for the next row
                else ++next_slot;
                if (remaining - take > 0 && remaining - take < kMinChunk) take = remaining;
            } else {
                s = least_loaded(slots, load);                    // rounding left a few blocks over
                take = remaining;
            }
            placed.push_back({s, StreamPiece{r.bh, r.row, first, take, r.lut_first + first, 0u, 0u, 0u}});
            load[s] += take + fixed;
            first += take;
        }
        if (placed.size() == 1) {
            StreamPiece pc = placed[0].second;
            pc.nchunks = 1;
            load[placed[0].first] -= kPartialCharge;
            whole[placed[0].first].push_back(pc);
            continue;
        }
        place_cut(r, placed, merger[i]);
    }
}

size_t align256(size_t n) { return (n + 255) / 256 * 256; }

}  // namespace

extern "C" {

int sfb_build_stream(sfb_stream_plan* plan, void* blob, size_t blob_bytes, const sfb_uint2* nn_lut, int nb,
                     uint32_t lut_heads, uint32_t lut_dim, uint32_t batch_dim, uint32_t head_dim, uint32_t block_size,
                     uint32_t wg_slots, int level, uint32_t tail_percent) {
    if (!plan || !nn_lut) return SFB_ERR_NULL_POINTER;
    if (nb <= 0 || batch_dim == 0 || head_dim == 0 || wg_slots == 0 || lut_heads == 0) return SFB_ERR_SHAPE;
    if (lut_heads > 1 && lut_heads != head_dim) return SFB_ERR_SHAPE;
    if (block_size != 32 && block_size != 64) return SFB_ERR_BLOCK_SIZE;
    if (tail_percent > 90) return SFB_ERR_ARGUMENT;
    const uint64_t num_bh64 = (uint64_t)batch_dim * head_dim;
    if (num_bh64 * (uint64_t)nb > 0x7fffffffull / 64) return SFB_ERR_SHAPE;
    const uint32_t num_bh = (uint32_t)num_bh64;
    const uint32_t L = (uint32_t)nb * block_size;

    // Slots are dealt to the 8 dies like consecutive work-group ids; a (batch, head) whose index has residue x
    // mod 8 is worked on by the slots of die x only, so its K and V stay in one L2.  The last batch*heads % 8
    // pairs have no die of their own and go wherever the load is smallest.
    const uint32_t dies = (wg_slots % 8 == 0 && num_bh >= 8) ? 8 : 1;
    const uint32_t bound_bh = dies == 8 ? num_bh - num_bh % 8 : num_bh;
    std::vector<std::vector<StreamPiece>> whole(wg_slots), chunks(wg_slots);
    std::vector<std::vector<StreamMerge>> merges(wg_slots);
    std::vector<double> load(wg_slots, 0.0);
    uint32_t parts = 0;
    auto rows_of = [&](uint32_t bh, std::vector<StreamRow>& rows, std::vector<StreamMerge>& empty) {
        const sfb_uint2* table = nn_lut + (size_t)(lut_heads > 1 ? bh % head_dim : 0u) * lut_dim;
        for (int r = 0; r < nb; ++r) {
            if (table[r].y == 0) empty.push_back(StreamMerge{bh, (uint32_t)r, 0u, 0u});   // the row is written as zeros
            else rows.push_back(StreamRow{bh, (uint32_t)r, table[r].y, table[r].x});
        }
    };
    std::vector<StreamMerge> empty_rows;
    const double tail = level ? 0.0 : tail_percent / 100.0;
    std::vector<std::vector<StreamRow>> late_rows(dies + 1);        // per die, and [dies]: heads without a die
    std::vector<std::vector<StreamMerge>> late_merges(dies + 1);
    for (uint32_t die = 0; die < dies; ++die) {
        std::vector<uint32_t> slots;
        for (uint32_t s = die; s < wg_slots; s += dies) slots.push_back(s);
        std::vector<StreamRow> rows;
        for (uint32_t bh = die; bh < bound_bh; bh += dies) rows_of(bh, rows, empty_rows);
        place_rows(rows, slots, load, whole, chunks, merges, &parts, level != 0, tail, &late_rows[die], &late_merges[die]);
    }
    {
        std::vector<uint32_t> slots(wg_slots);
        for (uint32_t s = 0; s < wg_slots; ++s) slots[s] = s;
        std::vector<StreamRow> rows;
        for (uint32_t bh = bound_bh; bh < num_bh; ++bh) rows_of(bh, rows, empty_rows);
        place_rows(rows, slots, load, whole, chunks, merges, &parts, level != 0, tail, &late_rows[dies], &late_merges[dies]);
        for (const StreamMerge& z : empty_rows) {
            const uint32_t m = least_loaded(slots, load);
            merges[m].push_back(z);
            load[m] += 0.25;
        }
    }
    // Streams behind the resident ones, one row or one merge each, dispatched as the resident ones end: they level
    // what the unequal pace of the work-groups leaves.  Stream wg_slots + dies * k + x belongs to die x; the heads
    // without a die take what is left over.  A merge stands behind all chunks of its row.
    const uint32_t resident = wg_slots;
    {
        std::vector<std::vector<StreamPiece>> tail_items(dies);
        std::vector<std::vector<StreamMerge>> tail_merges(dies);
        for (uint32_t die = 0; die < dies; ++die) {
            for (const StreamRow& r : late_rows[die])
                tail_items[die].push_back(StreamPiece{r.bh, r.row, 0u, r.count, r.lut_first, 1u, 0u, 0u});
            tail_merges[die] = late_merges[die];
        }
        for (size_t i = 0; i < late_rows[dies].size(); ++i) {
            const StreamRow& r = late_rows[dies][i];
            uint32_t best = 0;
            for (uint32_t die = 1; die < dies; ++die)
                if (tail_items[die].size() < tail_items[best].size()) best = die;
            tail_items[best].push_back(StreamPiece{r.bh, r.row, 0u, r.count, r.lut_first, 1u, 0u, 0u});
        }
        for (const StreamMerge& m : late_merges[dies]) tail_merges[0].push_back(m);
        size_t longest = 0;
        for (uint32_t die = 0; die < dies; ++die) longest = std::max(longest, tail_items[die].size() + tail_merges[die].size());
        const uint64_t total_streams = (uint64_t)wg_slots + (uint64_t)dies * longest;
        if (total_streams > 0x7fffffffull) return SFB_ERR_SHAPE;
        wg_slots = (uint32_t)total_streams;
        whole.resize(wg_slots); chunks.resize(wg_slots); merges.resize(wg_slots); load.resize(wg_slots, 0.0);
        for (uint32_t die = 0; die < dies; ++die) {
            uint32_t k = 0;
            for (const StreamPiece& pc : tail_items[die]) whole[resident + dies * (k++) + die].push_back(pc);
            for (const StreamMerge& m : tail_merges[die]) merges[resident + dies * (k++) + die].push_back(m);
        }
    }

    // sizes and offsets
    uint64_t n_blocks = 0, n_items = 0, n_merges = 0;
    for (uint32_t s = 0; s < wg_slots; ++s) {
        for (const auto& pc : chunks[s]) n_blocks += pc.count;
        for (const auto& pc : whole[s]) n_blocks += pc.count;
        n_items += chunks[s].size() + whole[s].size();
        n_merges += merges[s].size();
    }
    if (n_blocks > 0x7fffffffull) return SFB_ERR_SHAPE;
    sfb_stream_plan out;
    memset(&out, 0, sizeof(out));
    out.wg_slots = wg_slots;
    out.n_blocks = (uint32_t)n_blocks;
    out.n_items = (uint32_t)n_items;
    out.n_merges = (uint32_t)n_merges;
    out.n_parts = parts;
    out.block_size = block_size;
    out.batch_dim = batch_dim;
    out.head_dim = head_dim;
    out.ctx_blks = (uint32_t)nb;
    out.slots_offset = 0;
    out.blocks_offset = align256((size_t)wg_slots * sizeof(sfb_stream_slot));
    out.items_offset = out.blocks_offset + align256((size_t)(n_blocks + 1) * sizeof(sfb_stream_block));
    out.merges_offset = out.items_offset + align256((size_t)(n_items + 1) * sizeof(sfb_stream_item));
    out.total_bytes = out.merges_offset + align256((size_t)(n_merges + 1) * sizeof(sfb_stream_merge));
    double worst = 0, sum = 0;
    for (uint32_t s = 0; s < resident; ++s) { worst = std::max(worst, load[s]); sum += load[s]; }
    out.balance = worst > 0 ? (float)(sum / resident / worst) : 1.0f;
    out.resident = resident;
    if (!blob) { *plan = out; return SFB_OK; }
    if (blob_bytes < out.total_bytes) return SFB_ERR_ARGUMENT;

    memset(blob, 0, out.total_bytes);
    sfb_stream_slot* slot_out = (sfb_stream_slot*)((uint8_t*)blob + out.slots_offset);
    sfb_stream_block* block_out = (sfb_stream_block*)((uint8_t*)blob + out.blocks_offset);
    sfb_stream_item* item_out = (sfb_stream_item*)((uint8_t*)blob + out.items_offset);
    sfb_stream_merge* merge_out = (sfb_stream_merge*)((uint8_t*)blob + out.merges_offset);
    uint32_t nblk = 0, nitem = 0, nmerge = 0;
    for (uint32_t s = 0; s < wg_slots; ++s) {
        // producers of partial records first (their mergers find them ready), then whole rows, one (batch, head)
        // after the other so that the slots of a die walk through the heads in step
        std::vector<StreamPiece> list = chunks[s];
        std::vector<StreamPiece> rest = whole[s];
        std::stable_sort(rest.begin(), rest.end(), [](const StreamPiece& a, const StreamPiece& b) {
            return a.bh != b.bh ? a.bh < b.bh : a.row < b.row;
        });
        list.insert(list.end(), rest.begin(), rest.end());
        sfb_stream_slot& so = slot_out[s];
        so.block_begin = nblk;
        so.item_begin = nitem;
        so.merge_begin = nmerge;
        for (const StreamPiece& pc : list) {
            const uint32_t b = pc.bh / head_dim, h = pc.bh % head_dim;
            const sfb_uint2* table = nn_lut + (size_t)(lut_heads > 1 ? h : 0u) * lut_dim;
            sfb_stream_item& it = item_out[nitem++];
            it.q_off = (b * L + pc.row * block_size) * head_dim + h;
            it.batch = b; it.head = h; it.row = pc.row;
            it.kind = pc.nchunks > 1 ? 1u : 0u;
            it.part = pc.part;
            it.lut_first = pc.lut_first;
            it.count = pc.count;
            it.first = pc.first;
            it.nchunks = pc.nchunks;
            it.chunk = pc.chunk;
            it.lse_off = (b * head_dim + h) * L + pc.row * block_size;
            for (uint32_t i = 0; i < pc.count; ++i) {
                const sfb_uint2 e = table[pc.lut_first + i];
                sfb_stream_block& bo = block_out[nblk++];
                bo.kv_off = (b * L + e.y * block_size) * head_dim + h;
                bo.info = (e.x & SFB_STREAM_BLOCK_INDEX) | (i == 0 ? SFB_STREAM_FIRST : 0u) |
                          (i + 1 == pc.count ? SFB_STREAM_LAST : 0u);
                bo.col = e.y;
                bo.q_off = i == 0 ? it.q_off : 0u;
            }
        }
        so.n_blocks = nblk - so.block_begin;
        so.n_items = nitem - so.item_begin;
        for (const StreamMerge& m : merges[s]) {
            const uint32_t b = m.bh / head_dim, h = m.bh % head_dim;
            sfb_stream_merge& mo = merge_out[nmerge++];
            mo.q_off = (b * L + m.row * block_size) * head_dim + h;
            mo.batch = b; mo.head = h; mo.row = m.row;
            mo.part = m.part;
            mo.nparts = m.nparts;
        }
        so.n_merges = nmerge - so.merge_begin;
    }
    *plan = out;
    return SFB_OK;
}

// Work items of one layout, longest first; returns the number of leading "heavy" items.
static uint32_t schedule_layout(std::vector<sfb_work_item>& all, uint32_t& slots, uint32_t& parts, const sfb_uint2* nn_lut,
                                int nb, uint32_t max_blocks) {
    all.clear();
    slots = parts = 0;
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
    // items at least twice as long as the median item are "heavy"
    const uint32_t median = all[all.size() / 2].count;
    uint32_t heavy = 0;
    while (heavy + 1 < all.size() && all[heavy].count >= 2 * median && all[heavy].count > median) ++heavy;
    return heavy;
}

int sfb_build_schedule(sfb_work_item* items, uint32_t* n_items, uint32_t* n_heavy, uint32_t* n_slots,
                       uint32_t* n_parts, const sfb_uint2* nn_lut, int nb, uint32_t max_blocks) {
    if (!n_items || !n_heavy || !n_slots || !n_parts || !nn_lut) return SFB_ERR_NULL_POINTER;
    if (nb <= 0) return SFB_ERR_SHAPE;
    if (max_blocks == 0) return SFB_ERR_ARGUMENT;
    std::vector<sfb_work_item> all;
    uint32_t slots = 0, parts = 0;
    const uint32_t heavy = schedule_layout(all, slots, parts, nn_lut, nb, max_blocks);
    if (items) {
        if (*n_items < all.size()) return SFB_ERR_ARGUMENT;
        std::copy(all.begin(), all.end(), items);
    }
    *n_heavy = heavy;
    *n_items = (uint32_t)all.size();
    *n_slots = slots;
    *n_parts = parts;
    return SFB_OK;
}

int sfb_build_schedule_heads(sfb_work_item* items, uint32_t* n_items, uint32_t* n_heavy, uint32_t* n_slots,
                             uint32_t* n_parts, const sfb_uint2* nn_lut, int nb, uint32_t lut_heads, uint32_t lut_dim,
                             uint32_t max_blocks) {
    if (!n_items || !n_heavy || !n_slots || !n_parts || !nn_lut) return SFB_ERR_NULL_POINTER;
    if (nb <= 0 || lut_heads == 0 || lut_dim < (uint32_t)nb) return SFB_ERR_SHAPE;
    if (max_blocks == 0) return SFB_ERR_ARGUMENT;
    std::vector<std::vector<sfb_work_item>> lists(lut_heads);
    uint32_t longest = 0, heavy = 0xffffffffu, slots = 0, parts = 0;
    for (uint32_t h = 0; h < lut_heads; ++h) {
        uint32_t s = 0, p = 0;
        const uint32_t hv = schedule_layout(lists[h], s, p, nn_lut + (size_t)h * lut_dim, nb, max_blocks);
        longest = std::max<uint32_t>(longest, (uint32_t)lists[h].size());
        heavy = std::min(heavy, hv);   // ranks that are long in every head
        slots = std::max(slots, s);
        parts = std::max(parts, p);
    }
    if (items) {
        if (*n_items < longest) return SFB_ERR_ARGUMENT;
        const sfb_work_item skip = {SFB_WORK_ITEM_SKIP, 0u, 0u, 1u, 0u, 0u, 0u, 0u};
        for (uint32_t h = 0; h < lut_heads; ++h) {
            sfb_work_item* out = items + (size_t)h * *n_items;
            std::copy(lists[h].begin(), lists[h].end(), out);
            std::fill(out + lists[h].size(), out + *n_items, skip);
        }
    } else {
        *n_items = longest;
    }
    *n_heavy = heavy;
    *n_slots = slots;
    *n_parts = parts;
    return SFB_OK;
}

}  // extern "C"
