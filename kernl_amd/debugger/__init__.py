"""Host-side replay of the HIP kernels' index arithmetic (the counterpart of the reference's Triton debugger,
src/kernl/debugger/: run a kernel's addressing lane by lane on the CPU, over ordinary arrays).

The address functions replayed here are not re-typed in Python: they are the C++ functions of
`kernl_amd/csrc/index_math.h`, the header the kernels themselves are compiled from, built for the host into
`libkernl_index.so` and called through ctypes.  What this package adds is the machine around them — an LDS model with
bank-conflict accounting (`lds`), the operand layouts of the MFMA instructions and of the transposing LDS read
(`wave_ops`) — and replays of the kernels' tile steps that check, element by element, that every lane ends up with
the data the mathematics wants (`attention_replay`, `linear_replay`).  No GPU is needed.
"""
from kernl_amd.debugger.index_lib import index_lib  # noqa: F401
from kernl_amd.debugger.lds import Lds  # noqa: F401
