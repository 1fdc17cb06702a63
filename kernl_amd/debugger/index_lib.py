"""Loads `libkernl_index.so` (the index functions of csrc/index_math.h compiled for the host); builds it with g++ when
it is not there yet — a two-second compile of one file that needs neither ROCm nor a GPU."""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(os.path.dirname(_HERE), "csrc")
_PATH = os.path.join(os.path.dirname(_HERE), "libkernl_index.so")
_lib = None


class IndexLib:
    """Thin, typed view of the C entry points."""

    ATTN = {"stage_row": 0, "k_stage_chunk": 1, "v_stage_chunk": 2, "k_frag_offset": 3, "v_frag_offset": 4}
    MASK = {"stage_row": 0, "stage_chunk": 1, "read_offset": 2}
    WIDE = {"256": 0, "192": 1, "gated": 2}
    SMALL = {"load_row": 0, "load_chunk": 1, "frag_offset": 2}
    FEWROW = {"piece_unit": 0, "piece_row": 1, "piece_index": 2, "piece_dst": 3, "frag_offset": 4, "pieces_per_thread": 5,
              "unit_bytes": 6}

    def __init__(self, cdll):
        self._c = cdll
        for name, n in (("kernl_idx_rowperm16", 1), ("kernl_idx_swz_offset", 3), ("kernl_idx_attention", 5),
                        ("kernl_idx_mask", 5), ("kernl_idx_wide_weight_row", 2), ("kernl_idx_fewrow", 7),
                        ("kernl_idx_small_tile", 4), ("kernl_idx_xcd_contiguous", 2)):
            fn = getattr(cdll, name)
            fn.restype = ctypes.c_int
            fn.argtypes = [ctypes.c_int] * n

    def rowperm16(self, i: int) -> int:
        return self._c.kernl_idx_rowperm16(i)

    def swz_offset(self, row_bytes: int, row: int, chunk: int) -> int:
        return self._checked(self._c.kernl_idx_swz_offset(row_bytes, row, chunk))

    def attention(self, head_size: int, what: str, a: int, b: int = 0, c: int = 0) -> int:
        return self._checked(self._c.kernl_idx_attention(head_size, self.ATTN[what], a, b, c))

    def mask(self, element_size: int, what: str, a: int, b: int = 0, c: int = 0) -> int:
        return self._checked(self._c.kernl_idx_mask(element_size, self.MASK[what], a, b, c))

    def wide_weight_row(self, layout: str, row: int) -> int:
        return self._checked(self._c.kernl_idx_wide_weight_row(self.WIDE[layout], row))

    def fewrow(self, row_blocks: int, units_per_stage: int, what: str, a: int = 0, b: int = 0, c: int = 0, d: int = 0) -> int:
        return self._checked(self._c.kernl_idx_fewrow(row_blocks, units_per_stage, self.FEWROW[what], a, b, c, d))

    def xcd_contiguous(self, b: int, n: int) -> int:
        return self._checked(self._c.kernl_idx_xcd_contiguous(b, n))

    def small_tile(self, what: str, a: int, b: int = 0, c: int = 0) -> int:
        return self._checked(self._c.kernl_idx_small_tile(self.SMALL[what], a, b, c))

    @staticmethod
    def _checked(v: int) -> int:
        if v < 0:
            raise ValueError("index function called with a configuration the kernels are not built for")
        return v


def index_lib() -> IndexLib:
    global _lib
    if _lib is None:
        src = os.path.join(_CSRC, "index_math_host.cpp")
        hdr = os.path.join(_CSRC, "index_math.h")
        stale = not os.path.exists(_PATH) or os.path.getmtime(_PATH) < max(os.path.getmtime(src), os.path.getmtime(hdr))
        if stale:
            subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-o", _PATH, src], check=True)
        _lib = IndexLib(ctypes.CDLL(_PATH))
    return _lib
