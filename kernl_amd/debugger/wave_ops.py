"""Register layouts of the wave64 instructions the kernels are built on, as gathers and scatters between per-lane
register arrays and ordinary matrices.

v_mfma_f32_32x32x16 (D[32x32] += A[32x16] B[16x32]): lane l holds row l % 32 of A and column l % 32 of B, both for
k = 8 (l / 32) .. + 7; element v (0..15) of lane l of D is row 8 (v / 4) + 4 (l / 32) + v % 4, column l % 32.
v_mfma_f32_16x16x32 (D[16x16] += A[16x32] B[32x16]): lane l holds row l % 16 of A and column l % 16 of B for
k = 8 (l / 16) .. + 7; element e (0..3) of lane l of D is row 4 (l / 16) + e, column l % 16.
ds_read_b64_tr_b16: in every group of 16 consecutive lanes, lane i hands in the address of 4 consecutive 16-bit values
M[i][0..3] and receives M[i / 4][i % 4], M[4 + i / 4][i % 4], M[8 + i / 4][i % 4], M[12 + i / 4][i % 4].
"""
from typing import List, Sequence

import numpy as np

from kernl_amd.debugger.lds import Lds


def mfma32_operand(frags: np.ndarray) -> np.ndarray:
    """Per-lane fragments [64, 8] -> the [32, 16] matrix (rows = lane % 32, k = 8 (lane / 32) + j)."""
    m = np.zeros((32, 16), dtype=np.float64)
    for lane in range(64):
        m[lane % 32, 8 * (lane // 32):8 * (lane // 32) + 8] = frags[lane]
    return m


def mfma32(a_frags: np.ndarray, b_frags: np.ndarray, acc: np.ndarray) -> np.ndarray:
    """acc [64 lanes, 16] += A B in the instruction's own layouts; A, B as per-lane fragments [64, 8]."""
    d = mfma32_operand(a_frags) @ mfma32_operand(b_frags).T          # [32 rows, 32 columns]
    out = acc.copy()
    for lane in range(64):
        for v in range(16):
            out[lane, v] += d[8 * (v // 4) + 4 * (lane // 32) + v % 4, lane % 32]
    return out


def mfma16_result_position(lane: int, e: int):
    """(row, column) of element e of lane `lane` of a 16x16 result."""
    return 4 * (lane // 16) + e, lane % 16


def transposing_read_b64(lds: Lds, addresses: Sequence[int], tag: str = "") -> List[np.ndarray]:
    """ds_read_b64_tr_b16 for a whole wave: returns, per lane, its 4 16-bit values as raw uint16."""
    raw = lds.wave_read(addresses, 8, tag)
    handed_in = [np.frombuffer(r, dtype=np.uint16) for r in raw]
    out = []
    for lane in range(64):
        g, i = lane // 16, lane % 16
        out.append(np.array([handed_in[16 * g + 4 * q + i // 4][i % 4] for q in range(4)], dtype=np.uint16))
    return out
