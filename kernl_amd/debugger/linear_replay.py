"""Checks of the wide linear kernels' weight placement (csrc/linear_kernels.h; `wide_weight_row` in csrc/index_math.h).

The x fragment is the matrix instruction's A operand and the weight fragment its B operand, so lane l of a wave receives
column l % 16 of every 16 x 16 result block: the output column whose weight row sits in LDS row 16 j + l % 16 of the
wave's weight rows (block j).  The placement picks that weight row so that the lane's blocks line up as consecutive
output columns of one row."""
from typing import Dict, List

from kernl_amd.debugger.index_lib import index_lib
from kernl_amd.debugger.wave_ops import mfma16_result_position

ROWS_PER_WAVE = {"256": 128, "192": 96, "gated": 128}


def lane_columns(layout: str, tile_rows: int) -> Dict[int, List[List[int]]]:
    """For every lane l16 = 0 .. 15: the weight rows (= columns inside the tile; gated: rows of the fused weight) its
    accumulators hold, one list per wave of the tile's column split, in block order."""
    ix = index_lib()
    per_wave = ROWS_PER_WAVE[layout]
    out: Dict[int, List[List[int]]] = {}
    for l16 in range(16):
        _, col = mfma16_result_position(l16, 0)   # column of the result block = row of the B operand = LDS row in block
        out[l16] = [[ix.wide_weight_row(layout, first + 16 * j + col) for j in range(per_wave // 16)]
                    for first in range(0, tile_rows, per_wave)]
    return out


def check_weight_placement(layout: str) -> None:
    ix = index_lib()
    tile_rows = 192 if layout == "192" else 256
    per_wave = ROWS_PER_WAVE[layout]
    rows = [ix.wide_weight_row(layout, r) for r in range(tile_rows)]
    if sorted(rows) != list(range(tile_rows)):
        raise AssertionError(f"{layout}: the placement is not a permutation of the tile's weight rows")
    for l16, waves in lane_columns(layout, tile_rows).items():
        for w, cols in enumerate(waves):
            if layout == "gated":
                # output columns c .. c + 3 of the wave's 64, c = 4 l16: their gate rows (32 gate rows, then the 32 value
                # rows of the same columns, and so on), then their value rows 32 further on
                c = 4 * l16
                gate = [per_wave * w + 64 * (c // 32) + c % 32 + e for e in range(4)]
                if cols != gate + [r + 32 for r in gate]:
                    raise AssertionError(f"gated: lane {l16} holds {cols}, not 4 gate rows and their value rows")
            else:
                n = per_wave // 16
                if cols != list(range(per_wave * w + n * l16, per_wave * w + n * l16 + n)):
                    raise AssertionError(f"{layout}: lane {l16} holds {cols}, not {n} consecutive output columns")
