"""CPU tests of the index arithmetic the bf16 kernels stand on (sf-bert_amd/csrc/tile_index.h, compiled for the host):
the lanes that fill an LDS tile with LDS-direct loads and the lanes that read MFMA fragments from it must agree, no
lane may read beyond its tensor row, no LDS offset may leave the tile -- for block sizes 32 / 64 and head sizes
32 / 64 / 96 / 128.  The instructions are modelled lane by lane in tile_index_lib.py; the checks fail for a wrong
swizzle, a wrong lane base or a wrong slice rule (see the tests at the end)."""
import numpy as np
import pytest

from tile_index_lib import Lds, TileIndex, accumulator_row, mfma_32x32x16

SHAPES = [(bs, d) for bs in (32, 64) for d in (32, 64, 96, 128)]
POISON = 0xFFFF


def element_id(row, feature):
    return (row << 8) | feature


class Tensor:
    """A [tokens][heads][d] bf16 tensor of element ids with one tile (bs rows of one head) marked as readable."""

    def __init__(self, bs, d, heads=3, head=1, blocks=3, block=1):
        self.bs, self.d = bs, d
        self.row_elems = heads * d
        self.row_bytes = self.row_elems * 2
        ids = np.full((blocks * bs, self.row_elems), POISON, np.uint16)
        allowed = np.zeros((blocks * bs, self.row_elems), bool)
        r0, c0 = block * bs, head * d
        for r in range(bs):
            ids[r0 + r, c0:c0 + d] = [element_id(r, f) for f in range(d)]
        allowed[r0:r0 + bs, c0:c0 + d] = True
        self.bytes = ids.reshape(-1).view(np.uint8)
        self.allowed = np.repeat(allowed.reshape(-1), 2)
        self.tile_base = (r0 * self.row_elems + c0) * 2


def fill_tile(ti, tensor, lds, lds_tile=0, by_halves=False, ragged_hd=None):
    """What load_tile_all (or load_tile_by_halves) does, for all waves of the work-group.  ragged_hd: the tensor's
    head size when it is smaller than the kernel's (load_tile_all<true> with sources_ragged)."""
    group_rows = 4 if by_halves else 8
    for wave in range(ti.NW):
        for i in range(ti.LOADS):
            for f in range(ti.SLICES):
                part = (bool(ti.PARTIAL) or ragged_hd is not None) and f == ti.SLICES - 1
                n, odd = ti.load_group(i, wave), ti.load_group_odd(i, wave)
                assert odd == n % 2
                if by_halves:
                    source = ti.lane_source_by_halves
                elif part and ragged_hd is not None:
                    nch = ti.last_slice_chunks(ragged_hd)
                    source = lambda lane, odd, row_bytes: ti.lane_source_ragged(lane, odd, row_bytes, nch)
                else:
                    source = ti.lane_source_part if part else ti.lane_source
                offsets = [source(lane, odd, tensor.row_bytes) for lane in range(64)]
                lds.global_load_lds_dwordx4(lds_tile + f * ti.SLICE_BYTES + n * 1024, tensor.bytes,
                                            tensor.tile_base + f * 128 + n * group_rows * tensor.row_bytes,
                                            offsets, tensor.allowed)


def fill_tile_once(ti, tensor, lds, lds_tile=0):
    """What load_tile_once does: the four loads of a wave with one LDS base and the steps in the instruction offsets."""
    assert ti.SLICES == 1 and not ti.PARTIAL
    for wave in range(ti.NW):
        for i in range(ti.LOADS):
            offsets = [ti.once_lane_offset(lane, i, wave, tensor.row_bytes) for lane in range(64)]
            lds.global_load_lds_dwordx4(lds_tile + ti.once_m0(wave), tensor.bytes,
                                        tensor.tile_base + ti.once_base(wave, tensor.row_bytes), offsets,
                                        tensor.allowed, inst_offset=ti.once_inst_offset(i))


def fill_tile_staged(ti, tensor, lds, lds_tile=0):
    """What the register-staged form does: 16-byte loads of whole rows, then ds_write_b128 to the swizzled places."""
    assert ti.SLICES == 1 and not ti.PARTIAL
    for wave in range(ti.NW):
        for i in range(ti.LOADS):
            n, odd = ti.load_group(i, wave), ti.load_group_odd(i, wave)
            base = tensor.tile_base + n * 8 * tensor.row_bytes
            data, addresses = [], []
            for lane in range(64):
                src = base + ti.staged_source(lane, tensor.row_bytes)
                assert tensor.allowed[src:src + 16].all(), "lane %d reads bytes outside its row" % lane
                data.append(tensor.bytes[src:src + 16])
                addresses.append(lds_tile + n * 1024 + ti.staged_lds_offset(lane, odd))
            lds.ds_write_b128(addresses, data)


def check_fill(ti, lds, lds_tile=0):
    written = lds.writes[lds_tile:lds_tile + ti.TILE_BYTES]
    assert (written == 1).all(), "every byte of the tile is written exactly once"
    assert lds.writes.sum() == ti.TILE_BYTES, "nothing outside the tile is written"


def check_score_fragments(ti, lds, lds_tile=0):
    """k_frag(kt, ks) of lane (qn, half) = features 16 ks + 8 half .. + 7 of row 32 kt + qn."""
    for kt in range(ti.bs // 32):
        for ks in range(ti.d // 16):
            addresses = [lds_tile + ti.k_frag_offset(ti.k_lane_base(lane % 32, lane // 32), kt, ks) for lane in range(64)]
            got = lds.ds_read_b128(addresses)
            for lane in range(64):
                qn, half = lane % 32, lane // 32
                want = [element_id(32 * kt + qn, 16 * ks + 8 * half + e) for e in range(8)]
                assert got[lane].tolist() == want, (kt, ks, lane)


def read_transposed(ti, lds, mt, u, lds_tile=0):
    lo = lds.ds_read_b64_tr_b16([lds_tile + ti.v_frag_offset(ti.v_lane_base(lane), mt, u, 0) for lane in range(64)])
    hi = lds.ds_read_b64_tr_b16([lds_tile + ti.v_frag_offset(ti.v_lane_base(lane), mt, u, 1) for lane in range(64)])
    return np.concatenate([lo, hi], axis=1)   # [64][8]: the A operand of product step u


def check_transposed_fragments(ti, lds, source_row, lds_tile=0):
    """v_frag(mt, u) of lane (m, half): k-slot 8 half + 4 a + c  <->  LDS row 16 u + 8 a + 4 half + c, feature
    32 mt + m; source_row(lds_row) says which tensor row that LDS row holds."""
    for mt in range(ti.d // 32):
        for u in range(ti.bs // 16):
            got = read_transposed(ti, lds, mt, u, lds_tile)
            for lane in range(64):
                m, half = lane % 32, lane // 32
                want = [element_id(source_row(16 * u + 8 * a + 4 * half + c), 32 * mt + m)
                        for a in range(2) for c in range(4)]
                assert got[lane].tolist() == want, (mt, u, lane)


def rows_by_halves(lds_row):
    u, a, h, c = lds_row // 16, (lds_row // 8) % 2, (lds_row // 4) % 2, lds_row % 4
    return 32 * h + 8 * u + 4 * a + c


@pytest.mark.parametrize("bs,d", SHAPES)
def test_tile_constants(bs, d):
    ti = TileIndex(bs, d)
    assert ti.NW == bs // 32 and ti.SLICES == (d + 63) // 64 and ti.PARTIAL == (d % 64 != 0)
    assert ti.TILE_BYTES == ti.SLICES * bs * 128 and ti.LOADS * ti.NW * 8 == bs
    # swz is a bijection on chunk positions for every row and has period 16 in the row
    for row in range(64):
        assert sorted(c ^ ti.swz(row) for c in range(8)) == list(range(8))
        assert ti.swz(row) == ti.swz(row % 16)


@pytest.mark.parametrize("bs,d", SHAPES)
def test_loaders_and_score_fragment_readers_agree(bs, d):
    ti = TileIndex(bs, d)
    tensor = Tensor(bs, d)
    lds = Lds(4 * ti.TILE_BYTES)
    fill_tile(ti, tensor, lds, lds_tile=ti.TILE_BYTES)           # not at LDS address 0: offsets must be relative
    check_fill(ti, lds, lds_tile=ti.TILE_BYTES)
    check_score_fragments(ti, lds, lds_tile=ti.TILE_BYTES)


@pytest.mark.parametrize("bs,d", SHAPES)
def test_loaders_and_transposed_fragment_readers_agree(bs, d):
    ti = TileIndex(bs, d)
    tensor = Tensor(bs, d)
    lds = Lds(ti.TILE_BYTES)
    fill_tile(ti, tensor, lds)
    check_transposed_fragments(ti, lds, source_row=lambda r: r)


@pytest.mark.parametrize("bs", [32, 64])
@pytest.mark.parametrize("heads", [1, 3, 12])
def test_one_lds_base_per_tile_fills_the_same_tile(bs, heads):
    """The grouped form of the tile load (one M0 per tile, steps in the instruction offsets) leaves LDS exactly as
    the one-M0-per-load form does, for the narrowest rows too."""
    ti = TileIndex(bs, 64)
    tensor = Tensor(bs, 64, heads=heads, head=heads // 2)
    a, b = Lds(3 * ti.TILE_BYTES), Lds(3 * ti.TILE_BYTES)
    fill_tile(ti, tensor, a, lds_tile=2 * ti.TILE_BYTES)
    fill_tile_once(ti, tensor, b, lds_tile=2 * ti.TILE_BYTES)
    assert np.array_equal(a.mem, b.mem) and np.array_equal(a.writes, b.writes)
    check_score_fragments(ti, b, lds_tile=2 * ti.TILE_BYTES)
    # and so does the form that goes through registers and applies the swizzle on the LDS write
    c = Lds(3 * ti.TILE_BYTES)
    fill_tile_staged(ti, tensor, c, lds_tile=2 * ti.TILE_BYTES)
    assert np.array_equal(a.mem, c.mem) and np.array_equal(a.writes, c.writes)


@pytest.mark.parametrize("bs", [32, 64])
@pytest.mark.parametrize("hd", [8, 16, 24, 40, 48, 56, 72, 80, 88, 104, 112, 120])
def test_head_sizes_between_the_kernels(bs, hd):
    """A head size that is not a multiple of 32 runs through the kernel of the next multiple: the loaders must stay
    inside the hd features of their rows (the neighbouring head's features, or the end of the allocation, lie right
    behind them), every LDS byte the readers touch must have been written, the features that exist must be where
    the readers expect them, and with zero-padded queries the score product must come out exact."""
    D = (hd + 31) // 32 * 32
    ti = TileIndex(bs, D)
    tensor = Tensor(bs, hd, heads=3, head=2, blocks=2, block=1)      # the last head of the last block: the
    lds = Lds(ti.TILE_BYTES)                                         # allocation ends with the tile's last row
    assert ti.last_slice_chunks(hd) == (hd - 64 * (ti.SLICES - 1)) // 8 >= 1
    fill_tile(ti, tensor, lds, ragged_hd=hd)
    check_fill(ti, lds)
    rng = np.random.default_rng(hd)
    K = rng.integers(-3, 4, (bs, hd)).astype(np.float64)
    Q = rng.integers(-3, 4, (bs, hd)).astype(np.float64)
    S = K @ Q.T
    for wave in range(bs // 32):
        acc = [np.zeros((64, 16)) for _ in range(bs // 32)]
        for ks in range(D // 16):
            q_regs = np.zeros((64, 8))
            for lane in range(64):
                first = 16 * ks + 8 * (lane // 32)
                if first < hd:                                       # load_q_ragged: zeros beyond the row
                    q_regs[lane] = Q[32 * wave + lane % 32, first:first + 8]
            for kt in range(bs // 32):
                addresses = [ti.k_frag_offset(ti.k_lane_base(lane % 32, lane // 32), kt, ks) for lane in range(64)]
                ids = lds.ds_read_b128(addresses)
                assert (ids != POISON).all(), "filler must come from the tile's own rows"
                k_regs = np.zeros((64, 8))
                for lane in range(64):
                    first = 16 * ks + 8 * (lane // 32)
                    if first < hd:
                        want = [element_id(32 * kt + lane % 32, first + e) for e in range(8)]
                        assert ids[lane].tolist() == want, (kt, ks, lane)
                        k_regs[lane] = K[ids[lane] >> 8, ids[lane] & 0xFF]
                    else:
                        k_regs[lane] = 99.0                          # whatever the filler is, it meets zeros
                acc[kt] = mfma_32x32x16(k_regs, q_regs, acc[kt])
        for kt in range(bs // 32):
            for lane in range(64):
                for i in range(16):
                    assert acc[kt][lane, i] == S[32 * kt + accumulator_row(i, lane // 32), 32 * wave + lane % 32]
    # the second product reads columns: those below hd are the tile's own
    for mt in range(D // 32):
        for u in range(bs // 16):
            got = read_transposed(ti, lds, mt, u)
            assert (got != POISON).all()
            for lane in range(64):
                m, half = lane % 32, lane // 32
                if 32 * mt + m < hd:
                    want = [element_id(16 * u + 8 * a + 4 * half + c, 32 * mt + m) for a in range(2) for c in range(4)]
                    assert got[lane].tolist() == want, (mt, u, lane)


def test_row_order_of_the_dsd_tile():
    """lane_source_by_halves: LDS row 16u + 8a + 4h + c holds key 32h + 8u + 4a + c, so the 8 k-slots of a lane in
    product step u are the 8 consecutive keys 32 half + 8u .. + 7 (one 16-byte load of a P row)."""
    ti = TileIndex(64, 64)
    tensor = Tensor(64, 64)
    lds = Lds(ti.TILE_BYTES)
    fill_tile(ti, tensor, lds, by_halves=True)
    check_fill(ti, lds)
    check_transposed_fragments(ti, lds, source_row=rows_by_halves)
    for u in range(4):
        for half in range(2):
            keys = [rows_by_halves(16 * u + 8 * a + 4 * half + c) for a in range(2) for c in range(4)]
            assert keys == list(range(32 * half + 8 * u, 32 * half + 8 * u + 8))


@pytest.mark.parametrize("bs,d", SHAPES)
def test_lane_offsets_stay_inside_the_rows(bs, d):
    """Every lane offset is (row of the 8-row group) * row_bytes + a chunk inside the slice: < 128 bytes for a whole
    slice, < 64 bytes for a last slice of 32 features."""
    ti = TileIndex(bs, d)
    for row_bytes in (d * 2, 3 * d * 2, 12 * d * 2 * 3):
        for odd in (0, 1):
            for lane in range(64):
                for source, limit in ((ti.lane_source, 128), (ti.lane_source_part, 64)):
                    off = source(lane, odd, row_bytes)
                    assert off // row_bytes == lane // 8 or row_bytes < limit
                    assert off - (lane // 8) * row_bytes in range(0, limit, 16)


@pytest.mark.parametrize("bs,d", [(32, 64), (64, 64), (64, 96), (64, 128), (32, 32)])
def test_both_products_through_the_tiles(bs, d):
    """S^T = K Q^T from score fragments and O^T = V^T P^T from transposed fragments, P taken from the score
    accumulators without leaving its registers: the whole chain against numpy."""
    rng = np.random.default_rng(bs * 1000 + d)
    ti = TileIndex(bs, d)
    K = rng.integers(-3, 4, (bs, d)).astype(np.float64)
    V = rng.integers(-3, 4, (bs, d)).astype(np.float64)
    Q = rng.integers(-3, 4, (bs, d)).astype(np.float64)
    tensor = Tensor(bs, d)
    lds = Lds(2 * ti.TILE_BYTES)
    fill_tile(ti, tensor, lds, lds_tile=0)               # K tile and V tile hold the same ids: values by look-up
    fill_tile(ti, tensor, lds, lds_tile=ti.TILE_BYTES)

    def values(ids, table):
        return table[ids >> 8, ids & 0xFF]

    S = K @ Q.T          # [key][query]
    P = np.mod(S, 5.0)   # any function of the scores will do
    O = P.T @ V          # [query][feature]
    for wave in range(bs // 32):
        acc = [np.zeros((64, 16)) for _ in range(bs // 32)]
        for ks in range(d // 16):
            q_regs = np.array([Q[32 * wave + lane % 32, 16 * ks + 8 * (lane // 32):16 * ks + 8 * (lane // 32) + 8]
                               for lane in range(64)])
            for kt in range(bs // 32):
                addresses = [ti.k_frag_offset(ti.k_lane_base(lane % 32, lane // 32), kt, ks) for lane in range(64)]
                acc[kt] = mfma_32x32x16(values(lds.ds_read_b128(addresses), K), q_regs, acc[kt])
        for kt in range(bs // 32):
            for lane in range(64):
                for i in range(16):
                    assert acc[kt][lane, i] == S[32 * kt + accumulator_row(i, lane // 32), 32 * wave + lane % 32]
        p_regs = [np.mod(a, 5.0) for a in acc]
        out = [np.zeros((64, 16)) for _ in range(d // 32)]
        for u in range(bs // 16):
            kt, i0 = u // 2, (u % 2) * 8
            b_regs = p_regs[kt][:, i0:i0 + 8]
            for mt in range(d // 32):
                a_regs = values(read_transposed(ti, lds, mt, u, lds_tile=ti.TILE_BYTES), V)
                out[mt] = mfma_32x32x16(a_regs, b_regs, out[mt])
        for mt in range(d // 32):
            for lane in range(64):
                for i in range(16):
                    assert out[mt][lane, i] == O[32 * wave + lane % 32, 32 * mt + accumulator_row(i, lane // 32)]


# ---------------------------------------------------------------------------------------------------------------
# the checks above do fail for plausible mistakes
# ---------------------------------------------------------------------------------------------------------------
class Broken(TileIndex):
    def __init__(self, bs, d, **replace):
        super().__init__(bs, d)
        for name, fn in replace.items():
            setattr(self, name, fn.__get__(self))


def test_a_wrong_swizzle_is_caught():
    def unswizzled(self, lane, odd, row_bytes):
        return (lane // 8) * row_bytes + (lane % 8) * 16
    ti = Broken(64, 64, lane_source=unswizzled)
    lds = Lds(ti.TILE_BYTES)
    fill_tile(ti, Tensor(64, 64), lds)
    check_fill(ti, lds)
    with pytest.raises(AssertionError):
        check_score_fragments(ti, lds)
    with pytest.raises(AssertionError):
        check_transposed_fragments(ti, lds, source_row=lambda r: r)


def test_a_wrong_group_parity_is_caught():
    ti = Broken(64, 64, load_group_odd=lambda self, i, wave: 0)
    lds = Lds(ti.TILE_BYTES)
    with pytest.raises(AssertionError):
        fill_tile(ti, Tensor(64, 64), lds)


def test_reading_past_a_short_slice_is_caught():
    """A last slice of 32 features filled with the rule for whole slices reads the next head's features."""
    ti = TileIndex(64, 96)
    ti.lane_source_part = ti.lane_source
    with pytest.raises(AssertionError, match="outside its row"):
        fill_tile(ti, Tensor(64, 96), Lds(ti.TILE_BYTES))


def test_a_wrong_transposed_lane_base_is_caught():
    good = TileIndex(64, 64)
    ti = Broken(64, 64, v_lane_base=lambda self, lane: good.v_lane_base(lane ^ 4))
    lds = Lds(ti.TILE_BYTES)
    fill_tile(ti, Tensor(64, 64), lds)
    with pytest.raises(AssertionError):
        check_transposed_fragments(ti, lds, source_row=lambda r: r)
