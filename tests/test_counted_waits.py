"""CPU model of the counted waits in the streaming kernels of the unfused trio (sdd_nt_stream_kernel,
sdd_softmax_stream_kernel, the bf16 path of dsd_nn_kernel in sf-bert_amd/csrc/unfused_attention.hip).

Vector memory operations of a wave complete in issue order, so `s_waitcnt vmcnt(N)` returns once all but the last N
issued have completed.  Each model replays, for one wave, the order in which its kernel issues loads and stores
(transcribed from the kernel's loop, with the counts the kernel itself uses, read from the host build of
tile_index.h) and asserts at every wait that the tile -- or register set -- the step is about to read was issued more
than N operations ago, and at every load that the LDS buffer it overwrites has no reader left.  A count one too lax
fails (tests at the end)."""
import pytest

from tile_index_lib import lib

ROW_LENGTHS = [1, 2, 3, 7, 8, 9, 64, 65]


class Wave:
    """Issue-ordered queue of one wave's vector memory operations."""

    def __init__(self):
        self.issued = 0
        self.retired = 0          # operations 0 .. retired-1 are known to have completed

    def issue(self, n):
        first = self.issued
        self.issued += n
        return (first, self.issued)          # the range of sequence numbers

    def wait(self, n):
        self.retired = max(self.retired, self.issued - n)

    def done(self, ops):
        return ops[1] <= self.retired


class Ring:
    """LDS buffers: which tile each holds (by the loads that fill it) and until which step it is read."""

    def __init__(self, n):
        self.loads = [None] * n
        self.tile = [None] * n
        self.read_until = [-1] * n

    def fill(self, buf, tile, ops, step):
        # the barrier at the top of `step` has passed: readers of earlier steps are done
        assert self.read_until[buf] < step, "tile %r overwritten while step %d still reads it" % (self.tile[buf], self.read_until[buf])
        self.loads[buf], self.tile[buf] = ops, tile

    def read(self, wave, buf, tile, step):
        assert self.tile[buf] == tile, "buffer %d holds %r, the step wants %r" % (buf, self.tile[buf], tile)
        assert wave.done(self.loads[buf]), "tile %r read before its loads have completed" % (tile,)
        self.read_until[buf] = step


def sdd_stream(rows, elem_bytes, count=None, loads=None):
    """sdd_nt_stream_kernel: `rows` = block-row of each of the group's n <= 8 look-up entries."""
    L = lib()
    LOADS, PASSES = L.ti_sdd_wait_loads(elem_bytes), L.ti_slab_passes(elem_bytes)
    COUNT = L.ti_sdd_wait_count(elem_bytes) if count is None else count
    n, last = len(rows), len(rows) - 1
    w, ring = Wave(), Ring(3)
    ring.fill(0, 0, w.issue(LOADS), 0)
    ring.fill(1, min(1, last), w.issue(LOADS), 0)
    cur_row = None
    for g in range(n):
        if rows[g] != cur_row:
            w.issue(4)            # the query fragments of a new block-row, waited for at once
            w.wait(0)
            cur_row = rows[g]
        w.wait(COUNT)
        # barrier: K(g) is in LDS for every wave, every wave is done with K(g-1)
        ring.fill((g + 2) % 3, min(g + 2, last), w.issue(LOADS), g)
        ring.read(w, g % 3, g, g)
        w.issue(PASSES)           # the block's rows leave through the slab
    w.wait(0)
    assert w.retired == w.issued


def sdd_softmax_stream(count_blocks, elem_bytes, count=None, first=None):
    """sdd_softmax_stream_kernel: two passes over a block-row of count_blocks key blocks."""
    L = lib()
    LOADS, PASSES = L.ti_sdd_wait_loads(elem_bytes), L.ti_slab_passes(elem_bytes)
    COUNT = L.ti_sdd_wait_count(elem_bytes) if count is None else count
    FIRST = LOADS if first is None else first
    last = count_blocks - 1
    w, ring = Wave(), Ring(3)
    step = 0
    for pas in range(2):
        # (second pass: a barrier -- every wave is done with the tiles of the first)
        ring.fill(0, (pas, 0), w.issue(LOADS), step)
        ring.fill(1, (pas, min(1, last)), w.issue(LOADS), step)
        for j in range(count_blocks):
            w.wait(FIRST if (pas == 0 or j < 2) else COUNT)
            ring.fill((j + 2) % 3, (pas, min(j + 2, last)), w.issue(LOADS), step)
            ring.read(w, j % 3, (pas, j), step)
            if pas == 1:
                w.issue(PASSES)
            step += 1
    w.wait(0)


def dsd_stream(count_blocks, count=None):
    """dsd_nn_kernel, bf16 P and V: V tiles through a ring of four LDS buffers, P in registers DEPTH blocks ahead."""
    L = lib()
    DEPTH, P_LOADS, V_LOADS = L.ti_dsd_depth(), L.ti_dsd_p_loads(), L.ti_dsd_v_loads()
    COUNT = L.ti_dsd_wait_count() if count is None else count
    last = count_blocks - 1
    w, ring = Wave(), Ring(4)
    ring.fill(0, 0, w.issue(V_LOADS), 0)
    ring.fill(1, min(1, last), w.issue(V_LOADS), 0)
    p_regs = [(min(d, last), w.issue(P_LOADS)) for d in range(DEPTH)]
    step = 0
    for j0 in range(0, count_blocks, DEPTH):
        for d in range(0, DEPTH, 2):
            j = j0 + d
            w.wait(COUNT)
            ring.fill((j + 2) % 4, min(j + 2, last), w.issue(V_LOADS), step)
            ring.fill((j + 3) % 4, min(j + 3, last), w.issue(V_LOADS), step)
            for e in range(2):
                if j + e < count_blocks:          # blocks past the row's end are multiplied by zeros: any tile will do
                    ring.read(w, (j + e) % 4, j + e, step)
                    blk, ops = p_regs[d + e]
                    assert blk == j + e and w.done(ops), "P(%d) read before its loads have completed" % (j + e)
            p_regs[d] = (min(j + DEPTH, last), w.issue(P_LOADS))
            p_regs[d + 1] = (min(j + DEPTH + 1, last), w.issue(P_LOADS))
            step += 1
    w.wait(0)


def group_rows(n, crossing):
    """Block-rows of a group of n look-up entries; `crossing`: index at which the next block-row begins."""
    return [0 if g < crossing else 1 for g in range(n)]


@pytest.mark.parametrize("elem_bytes", [2, 4])
@pytest.mark.parametrize("n", range(1, 9))
def test_sdd_stream_waits(n, elem_bytes):
    for crossing in range(0, n + 1):
        sdd_stream(group_rows(n, crossing), elem_bytes)
    sdd_stream(list(range(n)), elem_bytes)      # every entry a new block-row


@pytest.mark.parametrize("elem_bytes", [2, 4])
@pytest.mark.parametrize("blocks", ROW_LENGTHS)
def test_sdd_softmax_stream_waits(blocks, elem_bytes):
    sdd_softmax_stream(blocks, elem_bytes)


@pytest.mark.parametrize("blocks", ROW_LENGTHS)
def test_dsd_stream_waits(blocks):
    dsd_stream(blocks)


def test_counts_match_what_the_loops_issue():
    L = lib()
    for elem_bytes, passes in ((2, 4), (4, 8)):
        assert L.ti_slab_passes(elem_bytes) == passes
        assert L.ti_sdd_wait_loads(elem_bytes) == 4
        assert L.ti_sdd_wait_count(elem_bytes) == 4 + 2 * passes
    assert L.ti_dsd_wait_count() == 8 and L.ti_dsd_depth() == 4


def test_a_count_one_too_lax_is_caught():
    L = lib()
    for elem_bytes in (2, 4):
        with pytest.raises(AssertionError, match="before its loads"):
            sdd_stream([0] * 8, elem_bytes, count=L.ti_sdd_wait_count(elem_bytes) + 1)
        with pytest.raises(AssertionError, match="before its loads"):
            sdd_softmax_stream(9, elem_bytes, count=L.ti_sdd_wait_count(elem_bytes) + 1)
        with pytest.raises(AssertionError, match="before its loads"):
            sdd_softmax_stream(9, elem_bytes, first=L.ti_sdd_wait_loads(elem_bytes) + 1)
    with pytest.raises(AssertionError, match="before its loads"):
        dsd_stream(9, count=L.ti_dsd_wait_count() + 1)


def test_a_buffer_reused_too_early_is_caught():
    ring, w = Ring(3), Wave()
    ring.fill(0, 0, w.issue(4), 0)
    w.wait(0)
    ring.read(w, 0, 0, step=3)
    with pytest.raises(AssertionError, match="overwritten"):
        ring.fill(0, 3, w.issue(4), step=3)
