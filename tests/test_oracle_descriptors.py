"""Pins the oracle's descriptor construction (layouts, LUTs, masks, magic division) against the
constants the reference hard-codes, its worked small cases, brute-force scans and invariants."""
import numpy as np
import pytest

import oracle_lib as orc


def test_causal_10_blocks_matches_reference_constants():
    # test.cu:24,39-40,45 / use_blocksparse.cu:21,40: 10 causal blocks -> 55 blocks, nn_lut_dim 65, nn_max 10
    lay = orc.layout_full(10, causal=True)
    luts = orc.build_luts(lay)
    assert luts["blocks"] == 55
    assert luts["nn_lut"].shape[0] == 65
    assert luts["nn_max"] == 10


def test_fixed_stride4_head0_nn_max_5():
    # test.cu:574 fixed_nn_max = 5 for nb=10, stride 4 (local_attn_ctx 128 / block 32), causal, head 0
    lay = orc.layout_fixed(4, 10, 4, causal=True)
    luts = orc.build_luts(lay[0])
    assert luts["nn_max"] == 5


def test_local_worked_example_nb4():
    # local_fusion_test.cu:48-63 with extra_diag = 1, nb = 4 (causal band)
    lay = orc.layout_local(4, 1)
    assert lay.tolist() == [[1, 0, 0, 0], [1, 1, 0, 0], [0, 1, 1, 0], [0, 0, 1, 1]]
    luts = orc.build_luts(lay, nn_max_init=2)
    assert luts["nt_lut"].tolist() == [[0, 0], [1, 0], [1, 1], [2, 1], [2, 2], [3, 2], [3, 3]]
    assert luts["nn_lut"].tolist() == [[4, 1], [5, 2], [7, 2], [9, 2],
                                       [0, 0], [1, 0], [2, 1], [3, 1], [4, 2], [5, 2], [6, 3]]
    assert luts["nn_max"] == 2
    assert luts["rblk_lut"].tolist() == [[0, 0], [1, 1], [2, 1], [3, 2], [4, 2], [5, 3], [6, 3]]
    keep = orc.element_mask(luts["nt_lut"], 32, orc.MASK_LOCAL, local_attn_ctx=32)
    words = orc.pack_mask(keep)
    for blk, (r, c) in enumerate(luts["nt_lut"].tolist()):
        for row in range(32):
            tri = (1 << (row + 1)) - 1
            want = tri if r == c else (~tri) & 0xFFFFFFFF
            assert int(words[blk * 32 + row]) == want, (blk, row)
    rm = orc.transpose_mask(words, 7, 32)
    assert all(int(rm[row * 7 + blk]) == int(words[blk * 32 + row]) for blk in range(7) for row in range(32))


def test_local_extra_diag_zero_is_full_causal():
    assert (orc.layout_local(6, 0) == orc.layout_full(6, causal=True)).all()


def test_causal_diag_mask_words():
    # no_fusion_test.cu:126-157: diagonal block row r keeps bits 0..r
    luts = orc.build_luts(orc.layout_full(3))
    for bs, full in ((32, 0xFFFFFFFF), (64, 0xFFFFFFFFFFFFFFFF)):
        words = orc.pack_mask(orc.element_mask(luts["nt_lut"], bs, orc.MASK_CAUSAL_DIAG))
        for blk, (r, c) in enumerate(luts["nt_lut"].tolist()):
            for row in range(bs):
                want = (1 << (row + 1)) - 1 if r == c else full
                assert int(words[blk * bs + row]) == want


def test_strided_chunks_reference_constants_is_diagonal():
    # stride_fusion_test.cu:55-71 with seq 1024, stride_attn_ctx 32, block 32 -> block_chunks 1
    lay = orc.layout_strided_chunks(32, 1)
    assert (lay == np.eye(32, dtype=np.uint32)).all()
    lay = orc.layout_strided_chunks(8, 4)
    want = np.array([[int(j <= i and j + (i % 4) >= i) for j in range(8)] for i in range(8)])
    assert (lay == want).all()


@pytest.mark.parametrize("nb", [1, 2, 5, 16, 33])
def test_luts_structural_invariants_random_layouts(nb):
    rng = np.random.default_rng(nb)
    lay = (rng.random((nb, nb)) < 0.4).astype(np.uint32)
    if nb > 2:
        lay[2, :] = 0  # an empty block-row
    luts = orc.build_luts(lay)
    nt, nn, blocks = luts["nt_lut"], luts["nn_lut"], luts["blocks"]
    rows, cols = np.nonzero(lay)  # row-major order
    assert blocks == len(rows)
    assert (nt[:, 0] == rows).all() and (nt[:, 1] == cols).all()
    counts = lay.sum(axis=1)
    assert (nn[:nb, 1] == counts).all()
    assert nn[0, 0] == nb
    assert (nn[:nb, 0] == nb + np.concatenate([[0], np.cumsum(counts)[:-1]])).all()
    assert (nn[nb:, 0] == np.arange(blocks)).all()
    assert (nn[nb:, 1] == nt[:, 1]).all()
    assert luts["nn_max"] == (counts.max() if blocks else 0)
    assert (luts["rblk_lut"][:, 0] == np.arange(blocks)).all()
    assert (luts["rblk_lut"][:, 1] == nt[:, 0]).all()
    for r in range(nb):  # every header slice addresses exactly the row's blocks
        off, cnt = nn[r]
        assert (nt[nn[off:off + cnt, 0], 0] == r).all()


def test_config_layout_counts():
    # workload constants: C1 local nb16 -> 46; C2 fixed nb32 -> 352 (11/row); C3 strided nb32 -> 346;
    # C4 BigBird nb64 -> 622, rows 64/7/8
    assert orc.layout_local(16, 1, bidirectional=True).sum() == 46
    c2 = orc.layout_fixed(1, 32, 4, causal=False)[0]
    assert c2.sum() == 352 and (c2.sum(axis=1) == 11).all()
    want = np.array([[int(i // 4 == j // 4 or j % 4 == 3) for j in range(32)] for i in range(32)])
    assert (c2 == want).all()
    c3 = orc.layout_strided(32, 4, 4, causal=False)
    want = np.array([[int(0 <= i - j <= 3 or (i - j) % 4 == 0) for j in range(32)] for i in range(32)])
    assert (c3 == want).all() and c3.sum() == 346
    assert orc.layout_strided(32, 4, 4, causal=True).sum() == 234
    rc = orc.bigbird_draw(64, 1, 2, True, 3, seed=1234)
    c4 = orc.layout_bigbird(64, 1, 2, True, rc)
    assert c4.sum() == 622
    per_row = c4.sum(axis=1)
    assert per_row[0] == 64 and per_row[63] == 64 and per_row[1] == 7 and per_row[62] == 7
    assert (per_row[2:62] == 8).all()


def test_bigbird_reference_shape_and_draw_properties():
    # big_bird_fusion_test.cu:50-79: window 1, global = first 2 rows and columns
    lay = orc.layout_bigbird(10, 1, 2, False)
    want = np.array([[int(abs(i - j) <= 1 or i < 2 or j < 2) for j in range(10)] for i in range(10)])
    assert (lay == want).all()
    base = orc.layout_bigbird(20, 1, 2, True)
    rc = orc.bigbird_draw(20, 1, 2, True, 3, seed=7)
    rc2 = orc.bigbird_draw(20, 1, 2, True, 3, seed=7)
    assert (rc == rc2).all()
    assert (orc.bigbird_draw(20, 1, 2, True, 3, seed=8) != rc).any()
    for i in range(20):
        if base[i].all():
            assert (rc[i] == -1).all()
        else:
            assert len(set(rc[i].tolist())) == 3 and all(base[i, c] == 0 for c in rc[i])


def test_magicu64_div64_exhaustive_small():
    rng = np.random.default_rng(0)
    for d in list(range(1, 130)) + [255, 256, 1000, 4096, 65537]:
        magic, shift = orc.magicu64(d)
        ns = np.concatenate([np.arange(0, 5000), rng.integers(0, 2 ** 31 - 1, 2000), [2 ** 31 - 1]])
        for n in ns:
            assert orc.lib.orc_div64(int(n), magic, shift) == int(n) // d, (d, int(n))


def test_bf16_rounding_rules():
    rng = np.random.default_rng(1)
    # every bf16 value v, its successor, the midpoint and points either side
    for hi in rng.integers(0x0080, 0x7f00, 3000):
        lo_bits = np.uint32(int(hi) << 16)
        for frac, rne, away in ((0x7fff, 0, 0), (0x8000, None, 1), (0x8001, 1, 1), (0x0000, 0, 0)):
            u = np.uint32(lo_bits | frac)
            f = u.view(np.float32)
            got_rne = orc.lib.orc_f32_to_bf16_rne(float(f))
            got_away = orc.lib.orc_f32_to_bf16_half_away(float(f))
            want_rne = int(hi) + (rne if rne is not None else (int(hi) & 1))
            assert got_rne == want_rne
            assert got_away == int(hi) + away
            # negative mirror
            fn = np.uint32(u | 0x80000000).view(np.float32)
            assert orc.lib.orc_f32_to_bf16_rne(float(fn)) == (want_rne | 0x8000)
    x = rng.standard_normal(4096).astype(np.float32)
    import torch
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert (orc.round_bf16(x) == want).all()
