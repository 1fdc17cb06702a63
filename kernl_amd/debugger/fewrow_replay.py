"""Replay of the stream-K few-row linear kernel's x stage (csrc/linear_splitk.hip, `FewRowStageMap` in
csrc/index_math.h) on the LDS model: the 512 threads store their 16-byte pieces of a group of units, then every lane of
a wave reads its MFMA operand fragments — each piece must be written exactly once, every read must return the x values
the instruction expects (k = 16 g + 8 s .. + 7 of row 16 mb + r of the unit), and neither side may conflict on banks."""
import struct
from typing import Tuple

from kernl_amd.debugger.index_lib import index_lib
from kernl_amd.debugger.lds import AccessStats, Lds

CONFIGS = ((1, 4), (2, 2), (4, 2), (8, 2))   # (16-row blocks of x, units per stage) as the kernel is launched
THREADS = 512


def replay_stage(row_blocks: int, units_per_stage: int) -> Tuple[AccessStats, AccessStats]:
    """Returns the (write, read) access statistics; raises AssertionError when a fragment holds the wrong values."""
    ix = index_lib()
    fr = lambda what, *a: ix.fewrow(row_blocks, units_per_stage, what, *a)
    rows = 16 * row_blocks
    unit_bytes = fr("unit_bytes")
    lds = Lds(units_per_stage * unit_bytes)
    # a piece carries (unit, row, first k) three times over plus padding: 16 bytes
    tag = lambda unit, row, k0: struct.pack("<4i", unit, row, k0, 0)
    for i in range(fr("pieces_per_thread")):
        for wave in range(THREADS // 64):
            tids = range(64 * wave, 64 * wave + 64)
            addrs = [fr("piece_dst", t, i) for t in tids]
            data = [tag(fr("piece_unit", t, i), fr("piece_row", t, i), 8 * fr("piece_index", t)) for t in tids]
            lds.wave_write(addrs, data, 16, "stage")
    if not lds.once_written(0, units_per_stage * unit_bytes):
        raise AssertionError("the staging stores do not cover the stage exactly once")
    for unit in range(units_per_stage):
        for mb in range(row_blocks):
            for s in range(2):
                addrs = [unit * unit_bytes + fr("frag_offset", mb, lane % 16, lane // 16, s) for lane in range(64)]
                got = lds.wave_read(addrs, 16, "fragment")
                for lane, piece in enumerate(got):
                    want = (unit, 16 * mb + lane % 16, 16 * (lane // 16) + 8 * s)
                    if struct.unpack("<4i", piece)[:3] != want:
                        raise AssertionError(f"lane {lane} block {mb} step {s} of unit {unit}: read {struct.unpack('<4i', piece)[:3]}, "
                                             f"the MFMA operand is {want}")
    assert rows * 8 * units_per_stage == THREADS * fr("pieces_per_thread")
    return lds.writes, lds.reads
