"""A byte-addressed model of one workgroup's LDS with bank-conflict accounting.

Model (MI355X, measured with a read-rate probe: 256 bytes per clock and CU): 64 banks of 4 bytes.  A wave instruction
that moves `width` bytes per lane is served in passes of 256 / width consecutive lanes (16 lanes for 16-byte accesses,
32 for 8-byte, 64 for 4-byte).  In a pass every bank delivers one dword per cycle; lanes that want the same dword share
it.  A pass therefore takes as many cycles as the most wanted bank has DIFFERENT dwords requested, and an instruction
is conflict-free when its cycle count equals its number of passes.  The lane grouping of a pass is the assumption of
this model; what it is good for is comparing layouts, not predicting absolute time.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Sequence

import numpy as np

BANKS = 64


@dataclass
class AccessStats:
    instructions: int = 0
    passes: int = 0
    cycles: int = 0
    worst: int = 1                                   # most cycles any single pass took
    by_tag: Dict[str, List[int]] = field(default_factory=dict)   # tag -> [passes, cycles]

    @property
    def conflict_free(self) -> bool:
        return self.cycles == self.passes


class Lds:
    def __init__(self, size: int):
        self.mem = np.zeros(size, dtype=np.uint8)
        self.written = np.zeros(size, dtype=np.int32)     # how often each byte has been stored to
        self.reads = AccessStats()
        self.writes = AccessStats()

    # ---- accounting
    @staticmethod
    def _cost(addresses: Sequence[int], width: int):
        lanes_per_pass = max(1, 256 // width)
        passes = cycles = 0
        worst = 1
        for start in range(0, len(addresses), lanes_per_pass):
            wanted: Dict[int, set] = {}
            for a in addresses[start:start + lanes_per_pass]:
                if a is None:
                    continue
                for dword in range(a // 4, (a + width + 3) // 4):
                    wanted.setdefault(dword % BANKS, set()).add(dword)
            if not wanted:
                continue
            c = max(len(v) for v in wanted.values())
            passes += 1
            cycles += c
            worst = max(worst, c)
        return passes, cycles, worst

    def _account(self, stats: AccessStats, addresses, width, tag):
        p, c, w = self._cost(addresses, width)
        stats.instructions += 1
        stats.passes += p
        stats.cycles += c
        stats.worst = max(stats.worst, w)
        t = stats.by_tag.setdefault(tag, [0, 0])
        t[0] += p
        t[1] += c

    # ---- wave instructions: `addresses` has one byte address per lane (None = lane inactive)
    def wave_read(self, addresses: Sequence[int], width: int, tag: str = "") -> List[bytes]:
        """ds_read_b{32,64,128}: every lane gets `width` bytes from its own address."""
        out = []
        for a in addresses:
            if a is None:
                out.append(b"")
                continue
            if a % min(width, 16) != 0:
                raise ValueError(f"{tag}: address {a} is not aligned to the {width}-byte access")
            if a < 0 or a + width > self.mem.size:
                raise IndexError(f"{tag}: LDS read of {width} bytes at {a} is outside the {self.mem.size} bytes allocated")
            if (self.written[a:a + width] == 0).any():
                raise ValueError(f"{tag}: LDS read at {a} touches bytes nothing has written")
            out.append(self.mem[a:a + width].tobytes())
        self._account(self.reads, addresses, width, tag)
        return out

    def wave_write(self, addresses: Sequence[int], data: Sequence[bytes], width: int, tag: str = "") -> None:
        """ds_write_b{32,64,128}, or one direct-to-LDS load of `width` bytes per lane."""
        for a, d in zip(addresses, data):
            if a is None:
                continue
            if len(d) != width:
                raise ValueError(f"{tag}: {len(d)} bytes given for a {width}-byte store")
            if a < 0 or a + width > self.mem.size:
                raise IndexError(f"{tag}: LDS write of {width} bytes at {a} is outside the {self.mem.size} bytes allocated")
            self.mem[a:a + width] = np.frombuffer(d, dtype=np.uint8)
            self.written[a:a + width] += 1
        self._account(self.writes, addresses, width, tag)

    def once_written(self, start: int, size: int) -> bool:
        """Every byte of [start, start + size) has been stored to exactly once."""
        return bool((self.written[start:start + size] == 1).all())
