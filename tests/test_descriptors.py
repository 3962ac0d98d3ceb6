"""Host descriptor builders of the library (through the C ABI) against the CPU oracle: bit-exact."""
import ctypes as C
import re
import os

import numpy as np
import pytest

import oracle_lib as orc
from sfb import sfb, ROOT


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "sfbert_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = sorted(set(re.findall(r"\b(sfb_[a-z0-9_]+)\s*\(", header)))
    assert declared, "no declarations found"
    for name in declared:
        assert hasattr(sfb.lib, name), "missing export " + name
    assert sorted(sfb.capi.EXPORTED) == declared


def test_status_strings():
    assert sfb.lib.sfb_status_string(0) == b"ok"
    assert len({sfb.lib.sfb_status_string(i) for i in range(10)}) == 10


LAYOUT_CASES = [
    ("full", (10, True)), ("full", (7, False)),
    ("local", (16, 1, True)), ("local", (16, 1, False)), ("local", (9, 0, False)), ("local", (12, 3, False)),
    ("strided_chunks", (32, 1)), ("strided_chunks", (16, 4)),
    ("strided", (32, 4, 4, False)), ("strided", (32, 4, 4, True)), ("strided", (17, 2, 5, False)),
]


@pytest.mark.parametrize("name,args", LAYOUT_CASES)
def test_layouts_bit_exact(name, args):
    got = getattr(sfb, "layout_" + name)(*args)
    want = getattr(orc, "layout_" + name)(*args)
    assert got.dtype == np.uint32 and np.array_equal(got, want)


@pytest.mark.parametrize("heads,nb,stride,causal", [(4, 10, 4, True), (1, 32, 4, False), (4, 33, 4, True),
                                                     (3, 8, 2, False)])
def test_fixed_layout_bit_exact(heads, nb, stride, causal):
    assert np.array_equal(sfb.layout_fixed(heads, nb, stride, causal), orc.layout_fixed(heads, nb, stride, causal))


@pytest.mark.parametrize("nb,window,nglobal,both,nrand,seed", [(64, 1, 2, True, 3, 1234), (10, 1, 2, False, 1, 0),
                                                               (20, 2, 3, True, 4, 99), (6, 1, 2, True, 3, 5),
                                                               (5, 0, 0, False, 7, 1)])
def test_bigbird_bit_exact(nb, window, nglobal, both, nrand, seed):
    rc = sfb.bigbird_draw(nb, window, nglobal, both, nrand, seed)
    assert np.array_equal(rc, orc.bigbird_draw(nb, window, nglobal, both, nrand, seed))
    assert np.array_equal(sfb.layout_bigbird(nb, window, nglobal, both, rc),
                          orc.layout_bigbird(nb, window, nglobal, both, rc))
    assert np.array_equal(sfb.layout_bigbird(nb, window, nglobal, both), orc.layout_bigbird(nb, window, nglobal, both))


def _random_layouts():
    rng = np.random.default_rng(0)
    for nb in (1, 2, 7, 16, 64):
        lay = (rng.random((nb, nb)) < 0.3).astype(np.uint32)
        if nb > 3:
            lay[3] = 0
        yield lay
    yield orc.layout_full(10)
    yield orc.layout_bigbird(64, 1, 2, True, orc.bigbird_draw(64, 1, 2, True, 3, 1234))
    yield np.zeros((4, 4), np.uint32)


@pytest.mark.parametrize("layout", list(_random_layouts()))
def test_luts_bit_exact(layout):
    for init in (0, 2):
        got, want = sfb.build_luts(layout, init), orc.build_luts(layout, init)
        for key in ("nt_lut", "nn_lut", "rblk_lut"):
            assert np.array_equal(got[key], want[key]), key
        assert got["nn_max"] == want["nn_max"] and got["blocks"] == want["blocks"]
        tn, tn_max = orc.build_tn_lut(want["nt_lut"], layout.shape[0])
        assert np.array_equal(got["tn_lut"], tn) and got["tn_max"] == tn_max
    counts = layout.sum(axis=1)
    order = got["row_order"]
    assert sorted(order.tolist()) == list(range(layout.shape[0]))
    assert all((counts[a] > counts[b]) or (counts[a] == counts[b] and a < b)
               for a, b in zip(order[:-1], order[1:]))


@pytest.mark.parametrize("bs", [8, 16, 32, 64])
@pytest.mark.parametrize("kind", [0, 1, 2, 3])
def test_masks_bit_exact(bs, kind):
    luts = orc.build_luts(orc.layout_local(6, 2))
    keep = sfb.element_mask(luts["nt_lut"], bs, kind, local_attn_ctx=bs + 5)
    assert np.array_equal(keep, orc.element_mask(luts["nt_lut"], bs, kind, local_attn_ctx=bs + 5))
    words = sfb.pack_mask(keep)
    assert words.dtype.itemsize == bs // 8
    assert np.array_equal(words, orc.pack_mask(keep))
    blocks = keep.shape[0]
    assert np.array_equal(sfb.transpose_mask(words, blocks, bs), orc.transpose_mask(words, blocks, bs))
    rnd = (np.random.default_rng(bs + kind).random(keep.shape) < 0.5).astype(np.uint8)
    assert np.array_equal(sfb.pack_mask(rnd), orc.pack_mask(rnd))


def test_magicu64_bit_exact():
    for d in list(range(1, 300)) + [1000, 4096, 65537, 2 ** 20 + 3]:
        assert sfb.magicu64(d) == orc.magicu64(d), d


def test_error_codes():
    lay = np.zeros((4, 4), np.uint32)
    assert sfb.lib.sfb_layout_full(None, 4, 1) == 1
    assert sfb.lib.sfb_layout_full(lay.ctypes.data_as(C.c_void_p), 0, 1) == 4
    assert sfb.lib.sfb_pack_mask(lay.ctypes.data_as(C.c_void_p), lay.ctypes.data_as(C.c_void_p), 1, 24) == 2
    with pytest.raises(sfb.capi.SfbError):
        sfb.layout_local(4, -1)
    # device entry points check their arguments before they touch the device
    assert sfb.lib.sfb_pack_qkv(None, None, None, None, sfb.BF16, C.c_uint32(64)) == 1
    u32 = C.c_uint32
    strided = sfb.lib.sfb_fused_attention_scheduled_strided
    args_tail = (u32(64), u32(1), u32(1), u32(1), u32(1), u32(64))
    assert strided(None, None, None, None, None, sfb.BF16, sfb.F32, None, None, None, None, u32(1), u32(0), u32(0),
                   u32(0), None, C.c_size_t(0), *args_tail, u32(0), u32(1), C.c_float(0.125)) == 4   # no stride given
    assert strided(None, None, None, None, None, sfb.BF16, sfb.F32, None, None, None, None, u32(1), u32(0), u32(0),
                   u32(0), None, C.c_size_t(0), *args_tail, u32(64), u32(1), C.c_float(0.125)) == 1   # NULL tensors


def test_argument_checks_of_the_newer_entry_points():
    """Checked before anything touches the device, so they can be exercised without one."""
    u32, ptr = C.c_uint32, C.c_void_p
    buf = np.zeros(4096, np.uint8)
    p = ptr(buf.ctypes.data)          # 16-byte aligned host memory standing in for tensors: never dereferenced here
    heads = sfb.lib.sfb_fused_attention_scheduled_heads

    def call(q=p, dtype=sfb.BF16, d=64, lut_heads=4, lut_dim=10, head_dim=4, items=p, n_items=3, n_heavy=0):
        return heads(None, q, p, p, p, None, dtype, sfb.F32, p, None, None, items, u32(n_items), u32(n_heavy), u32(0),
                     u32(0), None, C.c_size_t(0), u32(64), u32(6), u32(1), u32(4), u32(head_dim), u32(d), u32(lut_heads),
                     u32(lut_dim), u32(1), C.c_float(0.125))
    assert call(q=None) == 1
    assert call(items=None) == 1
    assert call(lut_heads=3) == 4           # one table per head or one for all
    assert call(lut_dim=11) == 4            # lut_dim = ctx_blks + blocks
    assert call(lut_heads=0) == 4
    assert call(n_heavy=3) == 4
    assert call(d=44) == 3 and call(d=136) == 3 and call(d=0) == 3      # bf16 rows: multiples of 8 up to 128
    assert call(d=44, dtype=sfb.F32, q=None) == 1                       # fp32: multiples of 4 (passes the size check)
    assert call(d=42, dtype=sfb.F32) == 3
    assert sfb.lib.sfb_stream_reset(None, None, u32(64), p) == 1
    assert sfb.lib.sfb_resident_work_groups_for(7, u32(64), u32(64), 0) == 0
    assert sfb.lib.sfb_resident_work_groups_for(sfb.BF16, u32(48), u32(64), 0) == 0
    n = u32(0)
    assert sfb.lib.sfb_build_schedule_heads(None, C.byref(n), C.byref(n), C.byref(n), C.byref(n), None, 4, u32(1), u32(8),
                                            u32(4)) == 1
    assert sfb.lib.sfb_build_schedule_heads(None, C.byref(n), C.byref(n), C.byref(n), C.byref(n), p, 4, u32(2), u32(3),
                                            u32(4)) == 4    # a table shorter than its header
    assert sfb.lib.sfb_build_schedule_heads(None, C.byref(n), C.byref(n), C.byref(n), C.byref(n), p, 4, u32(1), u32(8),
                                            u32(0)) == 8    # max_blocks
    # the fused backward takes every multiple of 8 (bf16) / 4 (fp32) up to 128
    bwd = sfb.lib.sfb_fused_attention_backward

    def backward(d, dtype=sfb.BF16):
        return bwd(None, p, p, p, p, p, p, p, p, p, p, dtype, p, p, None, None, None, u32(0), u32(0), u32(0), None, u32(0),
                   u32(0), u32(0), None, C.c_size_t(0), u32(64), u32(6), u32(1), u32(4), u32(4), u32(d), u32(1), u32(10),
                   u32(1), C.c_float(-1.0))
    assert backward(44) == 3 and backward(42, sfb.F32) == 3 and backward(136) == 3 and backward(64, 7) == 5
    assert backward(48) == 8 and backward(44, sfb.F32) == 8   # head sizes taken: the call gets as far as the scale check
    assert backward(96) == 8 and backward(32) == 8 and backward(128) == 8   # size accepted; the scale is what is wrong


def test_suggested_chunk_length():
    """1.25 x (key blocks of one head x batch x heads / 1024 resident work-groups), rounded up, at least 16."""
    lay = orc.layout_bigbird(64, 1, 2, True, orc.bigbird_draw(64, 1, 2, True, 3, 1234))
    luts = sfb.build_luts(lay)
    total = int(lay.sum())
    assert total == 622
    got = [sfb.suggest_max_blocks(luts["nn_lut"], 64, bh) for bh in (1, 12, 24, 48, 96, 192)]
    want = [max(16, -(-5 * total * bh // 4096)) for bh in (1, 12, 24, 48, 96, 192)]
    assert got == want == [16, 16, 19, 37, 73, 146]
    # what it means for the two global rows of 64 key blocks: four chunks, four, two, none
    for mb, chunks in ((16, 4), (19, 4), (37, 2), (73, 1)):
        sched = sfb.build_schedule(luts["nn_lut"], 64, mb)
        assert int((sched["items"]["row"] == 0).sum()) == chunks
    assert sfb.suggest_max_blocks(luts["nn_lut"], 64, 0) == 16


@pytest.mark.parametrize("max_blocks", [1, 3, 8, 100])
def test_schedule_covers_every_block_once(max_blocks):
    lay = orc.layout_bigbird(64, 1, 2, True, orc.bigbird_draw(64, 1, 2, True, 3, 1234))
    lay[5] = 0
    luts = sfb.build_luts(lay)
    sched = sfb.build_schedule(luts["nn_lut"], 64, max_blocks)
    items = sched["items"]
    counts = lay.sum(axis=1)
    assert sched["n_items"] == len(items)
    median = items["count"][len(items) // 2]
    heavy = (items["count"] >= 2 * median) & (items["count"] > median)
    assert sched["n_heavy"] == min(int(heavy.sum()), len(items) - 1)
    assert (items["count"] <= max(max_blocks, 1)).all()
    assert (np.diff(items["count"].astype(np.int64)) <= 0).all()  # longest first
    split_rows = [r for r in range(64) if counts[r] > max_blocks]
    assert sched["n_slots"] == len(split_rows)
    assert sched["n_parts"] == sum(-(-int(counts[r]) // max_blocks) for r in split_rows)
    slots, parts = set(), []
    for r in range(64):
        mine = np.sort(items[items["row"] == r], order="first")
        assert len(mine) >= 1 and (mine["nchunks"] == len(mine)).all()
        assert mine["first"][0] == 0 and mine["count"].sum() == counts[r]
        assert (mine["first"][1:] == np.cumsum(mine["count"])[:-1]).all()
        assert sorted(mine["chunk"].tolist()) == list(range(len(mine)))
        if len(mine) > 1:
            assert mine["count"].max() - mine["count"].min() <= 1
            assert len(set(mine["slot"].tolist())) == 1 and len(set(mine["part"].tolist())) == 1
            slots.add(int(mine["slot"][0]))
            parts.append((int(mine["part"][0]), len(mine)))
    assert slots == set(range(sched["n_slots"]))
    parts.sort()
    assert all(parts[i][0] + parts[i][1] == parts[i + 1][0] for i in range(len(parts) - 1))
    assert not parts or (parts[0][0] == 0 and parts[-1][0] + parts[-1][1] == sched["n_parts"])
    nbytes = sfb.schedule_workspace_bytes(sched, 4, 12, 64, 64)
    assert nbytes == (4 * 12 * sched["n_slots"] * 4 + 255) // 256 * 256 + 4 * 12 * sched["n_parts"] * (64 * 64 + 256) * 4


@pytest.mark.parametrize("max_blocks", [2, 5, 100])
def test_schedule_per_head_is_each_heads_own_schedule(max_blocks):
    """sfb_build_schedule_heads on the reference's per-head `fixed` pattern plus one head with emptied rows: every
    head's list is what sfb_build_schedule makes of its table, filled up with skip items; counts are the maxima."""
    H, nb = 4, 16
    lay = sfb.layout_fixed(H, nb, 4, causal=True)
    lay[2][3] = 0
    lay[2][3][:9] = 1                      # one long row in one head only
    per_head = [sfb.build_luts(lay[h]) for h in range(H)]
    width = max(len(p["nn_lut"]) for p in per_head)
    nn = np.zeros((H, width, 2), np.uint32)
    for h, p in enumerate(per_head):
        nn[h, :len(p["nn_lut"])] = p["nn_lut"]
    sched = sfb.build_schedule_heads(nn, nb, H, max_blocks)
    singles = [sfb.build_schedule(nn[h], nb, max_blocks) for h in range(H)]
    assert sched["lut_dim"] == width and sched["items"].shape == (H, sched["n_items"])
    assert sched["n_items"] == max(s["n_items"] for s in singles)
    assert sched["n_slots"] == max(s["n_slots"] for s in singles)
    assert sched["n_parts"] == max(s["n_parts"] for s in singles)
    assert sched["n_heavy"] == min(s["n_heavy"] for s in singles) < sched["n_items"]
    for h, single in enumerate(singles):
        mine = sched["items"][h]
        assert np.array_equal(mine[:single["n_items"]], single["items"])
        rest = mine[single["n_items"]:]
        assert (rest["row"] == sfb.WORK_ITEM_SKIP).all() and (rest["count"] == 0).all()
        assert (mine[:single["n_items"]]["row"] < nb).all()
    if max_blocks == 5:
        assert any(s["n_items"] < sched["n_items"] for s in singles), "the case has lists of different lengths"
    # one table: the plain schedule
    one = sfb.build_schedule_heads(nn[1], nb, 1, max_blocks)
    assert np.array_equal(one["items"][0], singles[1]["items"])


def check_stream(stream, luts_per_head, nb, B, H, bs):
    """Every key block of every (batch, head, row) appears exactly once, in LUT order inside its item; the flags,
    the item records, the partial records and the merge tasks are consistent."""
    plan, slots, blocks, items, merges = (stream[k] for k in ("plan", "slots", "blocks", "items", "merges"))
    L = nb * bs
    assert slots["n_blocks"].sum() == plan.n_blocks == len(blocks)
    assert slots["n_items"].sum() == plan.n_items == len(items)
    assert slots["n_merges"].sum() == plan.n_merges == len(merges)
    seen = {}       # (b, h, row) -> list of (first, count, kind, part, chunk, nchunks)
    for s in range(plan.wg_slots):
        so = slots[s]
        blk = blocks[so["block_begin"]:so["block_begin"] + so["n_blocks"]]
        its = items[so["item_begin"]:so["item_begin"] + so["n_items"]]
        # the FIRST flags of the run are the item boundaries, in the order of the item records
        starts = np.flatnonzero(blk["info"] & sfb.STREAM_FIRST)
        ends = np.flatnonzero(blk["info"] & sfb.STREAM_LAST)
        assert len(starts) == len(ends) == len(its)
        assert np.array_equal(ends - starts + 1, its["count"]) and (len(starts) == 0 or starts[0] == 0)
        assert np.array_equal(starts[1:], ends[:-1] + 1)
        kinds = its["kind"]
        assert (np.diff(kinds.astype(int)) <= 0).all(), "chunks of cut rows lead the stream"
        for it, a in zip(its, starts):
            b, h, row = int(it["batch"]), int(it["head"]), int(it["row"])
            lut = luts_per_head[h if len(luts_per_head) > 1 else 0]["nn_lut"]
            assert it["q_off"] == (b * L + row * bs) * H + h and it["lse_off"] == (b * H + h) * L + row * bs
            assert it["lut_first"] == lut[row, 0] + it["first"] and it["first"] + it["count"] <= lut[row, 1]
            ent = lut[it["lut_first"]:it["lut_first"] + it["count"]]
            mine = blk[a:a + it["count"]]
            assert np.array_equal(mine["info"] & sfb.STREAM_BLOCK_INDEX, ent[:, 0])
            assert np.array_equal(mine["col"], ent[:, 1])
            assert mine["q_off"][0] == it["q_off"] and (mine["q_off"][1:] == 0).all()
            assert np.array_equal(mine["kv_off"], (b * L + ent[:, 1] * bs) * H + h)
            assert (it["kind"] == 1) == (it["nchunks"] > 1)
            seen.setdefault((b, h, row), []).append(tuple(int(it[f]) for f in ("first", "count", "kind", "part", "chunk", "nchunks")))
    merge_of = {(int(m["batch"]), int(m["head"]), int(m["row"])): m for m in merges}
    parts_used = []
    for b in range(B):
        for h in range(H):
            lut = luts_per_head[h if len(luts_per_head) > 1 else 0]["nn_lut"]
            for row in range(nb):
                count = int(lut[row, 1])
                pieces = sorted(seen.get((b, h, row), []))
                if count == 0:
                    assert not pieces and merge_of[(b, h, row)]["nparts"] == 0
                    continue
                assert sum(pc[1] for pc in pieces) == count
                assert [pc[0] for pc in pieces] == list(np.cumsum([0] + [pc[1] for pc in pieces[:-1]]))
                if len(pieces) == 1:
                    assert pieces[0][2] == 0 and (b, h, row) not in merge_of
                else:
                    m = merge_of[(b, h, row)]
                    assert m["nparts"] == len(pieces) and m["q_off"] == (b * L + row * bs) * H + h
                    assert [pc[3] for pc in pieces] == list(range(int(m["part"]), int(m["part"]) + len(pieces)))
                    assert [pc[4] for pc in pieces] == list(range(len(pieces))) and all(pc[5] == len(pieces) for pc in pieces)
                    parts_used += [pc[3] for pc in pieces]
    assert sorted(parts_used) == list(range(plan.n_parts))


def test_stream_covers_every_block_once():
    nb, B, H, bs = 64, 4, 12, 64
    luts = sfb.build_luts(sfb.layout_bigbird(nb, 1, 2, True, sfb.bigbird_draw(nb, 1, 2, True, 3, 1234)))
    stream = sfb.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=1024)
    check_stream(stream, [luts], nb, B, H, bs)
    plan, slots, items = stream["plan"], stream["slots"], stream["items"]
    assert plan.n_blocks == 622 * B * H
    # a (batch, head) only appears in the streams of slots of the same residue mod 8
    for s in range(plan.wg_slots):
        its = items[slots[s]["item_begin"]:slots[s]["item_begin"] + slots[s]["n_items"]]
        assert ((its["batch"] * H + its["head"]) % 8 == s % 8).all()
    # the streams are level: only the two 64-block rows of a head are cut, every stream costs about the same
    assert plan.balance > 0.93
    assert (items["count"][items["kind"] == 0] <= 8).all()
    assert plan.n_merges == 2 * B * H
    assert slots["n_blocks"].max() <= 33
    # few, long chunks instead: streams differ by up to a short row
    coarse = sfb.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=1024, level=False)
    check_stream(coarse, [luts], nb, B, H, bs)
    assert coarse["plan"].n_parts == 3 * 2 * B * H and coarse["plan"].balance > 0.9
    assert coarse["plan"].resident == coarse["plan"].wg_slots == 1024
    # resident streams filled to 70 % of their share, the shortest rows and the merges in streams of their own behind
    tailed = sfb.build_stream(luts["nn_lut"], nb, B, H, bs, wg_slots=1024, level=False, tail_percent=30)
    check_stream(tailed, [luts], nb, B, H, bs)
    tp, ts, ti = tailed["plan"], tailed["slots"], tailed["items"]
    assert tp.resident == 1024 and tp.wg_slots > 1024 and (tp.wg_slots - 1024) % 8 == 0
    late = ts[1024:]
    assert ((late["n_items"] + late["n_merges"]) <= 1).all()
    assert ts[:1024]["n_merges"].sum() == 0 and late["n_merges"].sum() == 2 * B * H
    assert 0.6 < ts[:1024]["n_blocks"].sum() / tp.n_blocks < 0.8
    for s in np.flatnonzero(late["n_items"]):
        it = ti[late[s]["item_begin"]]
        assert (it["batch"] * H + it["head"]) % 8 == (1024 + s) % 8 and it["kind"] == 0
    # a merge stands in a stream behind those of all chunks of its row
    owner = np.repeat(np.arange(tp.wg_slots), ts["n_items"])
    for m, s in zip(tailed["merges"], np.repeat(np.arange(tp.wg_slots), ts["n_merges"])):
        if m["nparts"]:
            mine = (ti["kind"] == 1) & (ti["part"] >= m["part"]) & (ti["part"] < m["part"] + m["nparts"])
            assert mine.sum() == m["nparts"] and owner[mine].max() < s
    nbytes = sfb.stream_workspace_bytes(stream, 64)
    assert nbytes == (plan.n_parts * 4 + 255) // 256 * 256 + plan.n_parts * (64 * 64 + 256) * 4 + 256


def test_stream_per_head_tables_odd_sizes_and_empty_rows():
    nb, B, H, bs = 16, 3, 4, 32
    lay = sfb.layout_fixed(H, nb, 4, causal=True)
    per_head = [sfb.build_luts(lay[h]) for h in range(H)]
    nn = np.concatenate([p["nn_lut"] for p in per_head])
    for wg_slots in (1, 7, 40, 256):
        for level in (True, False):
            stream = sfb.build_stream(nn, nb, B, H, bs, lut_heads=H, wg_slots=wg_slots, level=level)
            check_stream(stream, per_head, nb, B, H, bs)
    holed = sfb.layout_bigbird(nb, 1, 2, True, sfb.bigbird_draw(nb, 1, 2, True, 3, 5)).copy()
    holed[5, :] = 0        # a block-row without key blocks
    holed = sfb.build_luts(holed)
    for wg_slots in (3, 64, 1024):   # 1024: far more streams than rows
        for level in (True, False):
            stream = sfb.build_stream(holed["nn_lut"], nb, B, H, bs, wg_slots=wg_slots, level=level)
            check_stream(stream, [holed], nb, B, H, bs)
            assert (stream["merges"]["nparts"] == 0).sum() == B * H
            assert (stream["items"]["count"] > 0).all()
    dense = sfb.build_luts(sfb.layout_full(8, causal=False))
    for wg_slots, B2 in ((16, 1), (1024, 2)):
        stream = sfb.build_stream(dense["nn_lut"], 8, B2, 3, 64, wg_slots=wg_slots)
        check_stream(stream, [dense], 8, B2, 3, 64)
