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


def test_plan_lists_cover_every_item_once():
    nb, B, H = 64, 4, 12
    luts = sfb.build_luts(sfb.layout_bigbird(nb, 1, 2, True, sfb.bigbird_draw(nb, 1, 2, True, 3, 1234)))
    plan = sfb.build_plan(luts["nn_lut"], nb, B, H, max_blocks=37, wg_slots=1024)
    sched = sfb.build_schedule(luts["nn_lut"], nb, 37)
    entries = plan["plan"]
    assert entries.shape == (1024, plan["plan_stride"])
    live = entries["count"] != sfb.PLAN_END
    assert live.sum() == B * H * sched["n_items"]
    assert (plan["n_slots"], plan["n_parts"]) == (sched["n_slots"], sched["n_parts"])
    # every (batch, head) gets every work item of the schedule exactly once
    fields = ("row", "first", "count", "nchunks", "chunk", "slot", "part", "lut_first")
    want = sorted(tuple(int(it[f]) for f in fields) for it in sched["items"])
    for b in range(B):
        for h in range(H):
            sel = live & (entries["batch"] == b) & (entries["head"] == h)
            assert sorted(tuple(int(e[f]) for f in fields) for e in entries[sel]) == want
    # live entries lead every list, followed by at least two end marks
    assert (np.diff(live.astype(int), axis=1) <= 0).all() and not live[:, -2:].any()
    # a (batch, head) only appears in the lists of slots of the same residue mod 8
    slot = np.broadcast_to(np.arange(1024)[:, None], live.shape)
    bh = entries["batch"] * H + entries["head"]
    assert np.array_equal(slot[live] % 8, bh[live] % 8)
    # the lists are balanced (key blocks + 2 per item) and the cut global rows lead their lists
    loads = np.where(live, entries["count"].astype(np.int64) + 2, 0).sum(axis=1)
    assert loads.max() <= loads.mean() + 10, (loads.max(), loads.mean())
    assert (entries["count"][:, 1:][live[:, 1:]] <= 8).all()


def test_plan_per_head_tables_and_odd_sizes():
    nb, B, H = 16, 3, 4
    lay = sfb.layout_fixed(H, nb, 4, causal=True)
    per_head = [sfb.build_luts(lay[h]) for h in range(H)]
    nn = np.concatenate([p["nn_lut"] for p in per_head])
    for wg_slots in (1, 7, 40):
        plan = sfb.build_plan(nn, nb, B, H, max_blocks=2, lut_heads=H, wg_slots=wg_slots)
        entries = plan["plan"]
        live = entries["count"] != sfb.PLAN_END
        for h in range(H):
            sched = sfb.build_schedule(per_head[h]["nn_lut"], nb, 2)
            sel = live & (entries["head"] == h)
            assert sel.sum() == B * sched["n_items"]
            assert sorted(entries["lut_first"][sel & (entries["batch"] == 0)]) == sorted(sched["items"]["lut_first"])
        assert not live[:, -2:].any()
