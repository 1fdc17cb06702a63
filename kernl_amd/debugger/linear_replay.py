"""Checks of the wide linear kernel's weight placement (csrc/linear_kernels.h; `wide_weight_row` in csrc/index_math.h): LDS row `row` of a weight
tile feeds MFMA row row % 16 of 16-row block row / 16, and carries a weight row chosen so that the four-element
results of a lane line up as consecutive output columns."""
from typing import Dict, List

from kernl_amd.debugger.index_lib import index_lib
from kernl_amd.debugger.wave_ops import mfma16_result_position


def lane_columns(layout: str, tile_rows: int) -> Dict[int, List[List[int]]]:
    """For every lane group g = lane / 16: the weight rows (= output columns inside the tile) its accumulators hold,
    one list per lane-contiguous group of blocks, in register order (block by block, element by element)."""
    ix = index_lib()
    blocks_per_group = 2 if layout == "192" else 4
    out: Dict[int, List[List[int]]] = {}
    for g in range(4):
        lane = 16 * g
        groups = []
        for first in range(0, tile_rows // 16, blocks_per_group):
            cols = []
            for j in range(first, first + blocks_per_group):
                for e in range(4):
                    r, _ = mfma16_result_position(lane, e)       # MFMA row inside block j
                    cols.append(ix.wide_weight_row(layout, 16 * j + r))
            groups.append(cols)
        out[g] = groups
    return out


def check_weight_placement(layout: str) -> None:
    ix = index_lib()
    tile_rows = 192 if layout == "192" else 256
    rows = [ix.wide_weight_row(layout, r) for r in range(tile_rows)]
    if sorted(rows) != list(range(tile_rows)):
        raise AssertionError(f"{layout}: the placement is not a permutation of the tile's weight rows")
    for g, groups in lane_columns(layout, tile_rows).items():
        for cols in groups:
            if layout == "gated":
                # gate columns 8 g' .. + 7 and the value columns 32 further on, g' within the 64-row group
                gate, value = cols[0:4] + cols[4:8], cols[8:12] + cols[12:16]
                if gate != list(range(gate[0], gate[0] + 8)) or value != [c + 32 for c in gate] or gate[0] % 8 != 0:
                    raise AssertionError(f"gated: lane group {g} holds {cols}, not 8 gate columns and their value columns")
            elif cols != list(range(cols[0], cols[0] + len(cols))) or cols[0] % len(cols) != 0:
                raise AssertionError(f"{layout}: lane group {g} holds {cols}, not consecutive output columns")
        if layout == "256":
            # the two groups of a wave's eight blocks follow each other: 32 consecutive columns, 64-byte aligned
            for first in range(0, len(groups), 2):
                both = groups[first] + groups[first + 1]
                if both != list(range(both[0], both[0] + 32)) or both[0] % 32 != 0:
                    raise AssertionError(f"256: lane group {g} holds {both}, not 32 consecutive output columns")
