"""Host build of the kernels' index arithmetic (sf-bert_amd/csrc/tile_index.h) plus a lane-level model of the
gfx950 instructions that consume it, for the CPU tests.

The model states what each instruction does with 64 lanes' addresses and registers:

* ``global_load_lds_dwordx4``: lane l fetches 16 bytes from its own global address; the wave's 1 KiB lands in LDS at
  M0 + 16 l (lane order, whatever the global addresses were);
* ``ds_read_b128``: lane l reads 16 bytes at its own LDS address;
* ``ds_read_b64_tr_b16``: in every group of 16 lanes, lane 4j + q supplies the 4 consecutive 16-bit values at its
  address as columns 4q .. 4q+3 of row j of a 4 x 16 matrix; lane i of the group receives column i (4 values);
* ``v_mfma_f32_32x32x16_bf16``: lane l holds A[l % 32][8 (l / 32) + e] and B[8 (l / 32) + e][l % 32], e = 0..7, and
  receives D[8 (i / 4) + 4 (l / 32) + i % 4][l % 32] in accumulator element i = 0..15.
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SHIM = os.path.join(HERE, "tile_index_shim.cpp")
HEADER = os.path.join(ROOT, "sf-bert_amd", "csrc", "tile_index.h")
BUILD = os.path.join(HERE, "_build")
LIB = os.path.join(BUILD, "libtile_index.so")

_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    os.makedirs(BUILD, exist_ok=True)
    newest = max(os.path.getmtime(SHIM), os.path.getmtime(HEADER))
    if not os.path.exists(LIB) or os.path.getmtime(LIB) < newest:
        subprocess.check_call(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-Wall", "-Werror", "-o", LIB, SHIM])
    _lib = ctypes.CDLL(LIB)
    for name in dir(_Names):
        if name.startswith("ti_"):
            getattr(_lib, name).restype = ctypes.c_uint32
    return _lib


class _Names:
    ti_const = ti_swz = ti_lane_source = ti_lane_source_part = ti_lane_source_by_halves = None
    ti_load_group = ti_load_group_odd = ti_k_lane_base = ti_k_frag_offset = ti_v_lane_base = ti_v_frag_offset = None
    ti_slab_passes = ti_sdd_wait_count = ti_sdd_wait_loads = ti_dsd_wait_count = ti_dsd_depth = None
    ti_dsd_p_loads = ti_dsd_v_loads = None
    ti_once_inst_offset = ti_once_lane_offset = ti_once_base = ti_once_m0 = None
    ti_lane_source_ragged = ti_last_slice_chunks = ti_staged_source = ti_staged_lds_offset = None


class TileIndex:
    """TileIndex<BS, D> of the kernels, evaluated on the host."""

    def __init__(self, bs, d):
        self.bs, self.d, self._l = bs, d, lib()
        names = ["NW", "SLICES", "PARTIAL", "SLICE_BYTES", "TILE_BYTES", "GROUPS", "LOADS"]
        for which, name in enumerate(names):
            value = self._l.ti_const(bs, d, which)
            assert value != 0xFFFFFFFF, (bs, d)
            setattr(self, name, int(value))

    def swz(self, row):
        return int(self._l.ti_swz(self.bs, self.d, row))

    def lane_source(self, lane, odd, row_bytes):
        return int(self._l.ti_lane_source(self.bs, self.d, lane, odd, row_bytes))

    def lane_source_part(self, lane, odd, row_bytes):
        return int(self._l.ti_lane_source_part(self.bs, self.d, lane, odd, row_bytes))

    def lane_source_by_halves(self, lane, odd, row_bytes):
        return int(self._l.ti_lane_source_by_halves(self.bs, self.d, lane, odd, row_bytes))

    def lane_source_ragged(self, lane, odd, row_bytes, nch):
        return int(self._l.ti_lane_source_ragged(self.bs, self.d, lane, odd, row_bytes, nch))

    def last_slice_chunks(self, hd):
        return int(self._l.ti_last_slice_chunks(self.bs, self.d, hd))

    def load_group(self, i, wave):
        return int(self._l.ti_load_group(self.bs, self.d, i, wave))

    def load_group_odd(self, i, wave):
        return int(self._l.ti_load_group_odd(self.bs, self.d, i, wave))

    def once_inst_offset(self, i):
        return int(ctypes.c_int32(self._l.ti_once_inst_offset(self.bs, self.d, i)).value)

    def once_lane_offset(self, lane, i, wave, row_bytes):
        return int(self._l.ti_once_lane_offset(self.bs, self.d, lane, i, wave, row_bytes))

    def once_base(self, wave, row_bytes):
        return int(self._l.ti_once_base(self.bs, self.d, wave, row_bytes))

    def once_m0(self, wave):
        return int(self._l.ti_once_m0(self.bs, self.d, wave))

    def staged_source(self, lane, row_bytes):
        return int(self._l.ti_staged_source(self.bs, self.d, lane, row_bytes))

    def staged_lds_offset(self, lane, odd):
        return int(self._l.ti_staged_lds_offset(self.bs, self.d, lane, odd))

    def k_lane_base(self, qn, half):
        return int(self._l.ti_k_lane_base(self.bs, self.d, qn, half))

    def k_frag_offset(self, lane_base, kt, ks):
        return int(self._l.ti_k_frag_offset(self.bs, self.d, lane_base, kt, ks))

    def v_lane_base(self, lane):
        return int(self._l.ti_v_lane_base(self.bs, self.d, lane))

    def v_frag_offset(self, lane_base, mt, u, x):
        return int(self._l.ti_v_frag_offset(self.bs, self.d, lane_base, mt, u, x))


# ---------------------------------------------------------------------------------------------------------------
# instruction model
# ---------------------------------------------------------------------------------------------------------------
class Lds:
    """LDS of one work-group: bytes, plus how often each byte was written since the last clear."""

    def __init__(self, nbytes):
        self.mem = np.zeros(nbytes, np.uint8)
        self.writes = np.zeros(nbytes, np.int32)

    def global_load_lds_dwordx4(self, m0, glob, base, lane_offsets, allowed, inst_offset=0):
        """allowed: boolean array over glob's bytes -- the bytes this tile may read (its own rows).  The instruction
        offset (13 signed bits) goes into the global address and into the LDS address alike."""
        assert len(lane_offsets) == 64 and -4096 <= inst_offset <= 4095 and 0 <= m0 < 65536
        for lane, off in enumerate(lane_offsets):
            assert 0 <= off < 2 ** 32, "the lane offset is an unsigned 32-bit register"
            src, dst = base + off + inst_offset, m0 + inst_offset + 16 * lane
            assert 0 <= src and src + 16 <= glob.size, "lane %d reads outside the allocation" % lane
            assert allowed[src:src + 16].all(), "lane %d reads bytes outside its row" % lane
            assert 0 <= dst and dst + 16 <= self.mem.size, "LDS destination outside the tile"
            self.mem[dst:dst + 16] = glob[src:src + 16]
            self.writes[dst:dst + 16] += 1

    def ds_write_b128(self, addresses, data):
        """data: [64][16] bytes, lane l's 16 bytes go to its own address."""
        for lane, a in enumerate(addresses):
            assert a % 16 == 0 and 0 <= a and a + 16 <= self.mem.size, "b128 write misaligned or outside the tile"
            self.mem[a:a + 16] = data[lane]
            self.writes[a:a + 16] += 1

    def ds_read_b128(self, addresses):
        out = np.zeros((64, 8), np.uint16)
        for lane, a in enumerate(addresses):
            assert a % 16 == 0 and 0 <= a and a + 16 <= self.mem.size, "b128 read misaligned or outside the tile"
            assert (self.writes[a:a + 16] > 0).all(), "read of LDS bytes no load has written"
            out[lane] = self.mem[a:a + 16].view(np.uint16)
        return out

    def ds_read_b64_tr_b16(self, addresses):
        out = np.zeros((64, 4), np.uint16)
        for group in range(4):
            rows = np.zeros((4, 16), np.uint16)
            for s in range(16):
                a = addresses[16 * group + s]
                assert a % 8 == 0 and 0 <= a and a + 8 <= self.mem.size, "b64 read misaligned or outside the tile"
                assert (self.writes[a:a + 8] > 0).all(), "read of LDS bytes no load has written"
                j, q = s // 4, s % 4
                rows[j, 4 * q:4 * q + 4] = self.mem[a:a + 8].view(np.uint16)
            for i in range(16):
                out[16 * group + i] = rows[:, i]
        return out


def mfma_32x32x16(a_regs, b_regs, acc=None):
    """a_regs, b_regs: [64][8] (any numeric dtype); returns [64][16] float64 accumulators (+ acc)."""
    a_full = np.zeros((32, 16))
    b_full = np.zeros((16, 32))
    for lane in range(64):
        r, h = lane % 32, lane // 32
        a_full[r, 8 * h:8 * h + 8] = a_regs[lane]
        b_full[8 * h:8 * h + 8, r] = b_regs[lane]
    d_full = a_full @ b_full
    out = np.zeros((64, 16)) if acc is None else acc.copy()
    for lane in range(64):
        n, h = lane % 32, lane // 32
        for i in range(16):
            out[lane, i] += d_full[8 * (i // 4) + 4 * h + i % 4, n]
    return out


def accumulator_row(i, half):
    """Row (of the 32 x 32 result tile) that accumulator element i of a lane in half `half` holds."""
    return 8 * (i // 4) + 4 * half + i % 4
