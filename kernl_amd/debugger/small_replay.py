"""Replay of an operand tile of the small-problem linear kernels (csrc/linear_small.hip, `SmallTileMap` in
csrc/index_math.h) on the LDS model.  Tile loads write LDS directly — a wave's load fills 64 consecutive 16-byte chunks,
each lane fetching from memory the chunk that belongs at its LDS position — and the MFMA operand fragments are read
back by 16 rows x 4 k-groups of lanes.  The loads must bring every (row, chunk) of the tile exactly once, every fragment
read must return the k-values the instruction expects (k = 32 s + 8 g .. + 7 of row 16 b + r), and the reads must not
conflict on banks."""
import struct

from kernl_amd.debugger.index_lib import index_lib
from kernl_amd.debugger.lds import AccessStats, Lds

TILE_ROWS = (16, 32, 64)   # x and w tiles of the kernels as built: 16 / 32 / 64 rows of 64 k-values


def replay_tile(rows: int) -> AccessStats:
    """Returns the access statistics of the fragment reads; raises AssertionError when a fragment holds the wrong values."""
    ix = index_lib()
    st = lambda what, *a: ix.small_tile(what, *a)
    chunks = rows * 8
    lds = Lds(chunks * 16)
    seen = set()
    for load in range(chunks // 64):                      # one 1 KB load instruction of a wave
        qs = range(64 * load, 64 * load + 64)
        cells = [(st("load_row", q), st("load_chunk", q)) for q in qs]
        seen.update(cells)
        lds.wave_write([16 * q for q in qs], [struct.pack("<4i", row, 8 * c, 0, 0) for row, c in cells], 16, "tile load")
    if len(seen) != chunks or not lds.once_written(0, chunks * 16):
        raise AssertionError("the tile loads do not bring every chunk of the tile exactly once")
    for block in range(rows // 16):
        for kstep in range(2):
            addrs = [st("frag_offset", 16 * block + lane % 16, kstep, lane // 16) for lane in range(64)]
            got = lds.wave_read(addrs, 16, "fragment")
            for lane, piece in enumerate(got):
                want = (16 * block + lane % 16, 32 * kstep + 8 * (lane // 16))
                if struct.unpack("<4i", piece)[:2] != want:
                    raise AssertionError(f"lane {lane} block {block} k-step {kstep}: read {struct.unpack('<4i', piece)[:2]}, "
                                         f"the MFMA operand is {want}")
    return lds.reads
