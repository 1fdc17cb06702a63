"""Static input memory for graph replay (reference: src/kernl/optimizer/pool_cuda_graphs.py:4-64).

A captured hipGraph reads its inputs from fixed device addresses.  `CudaGraphPool` is one flat byte buffer from which
input copies are carved with 8-byte aligned bump allocation; `reset()` rewinds it so the next call's inputs land at
the same addresses.  The class keeps the reference's name although the graphs here are hipGraphs.
"""
import torch


def get_aligned_size(t: torch.Tensor, alignment=8) -> int:
    """Bytes of `t`'s storage rounded up to `alignment` (known answers: test/test_cuda_graph.py:11-16)."""
    storage_len = t.untyped_storage().nbytes()
    return (storage_len + alignment - 1) // alignment * alignment


class CudaGraphPool:
    def __init__(self, size, device="cuda"):
        """`size` bytes, positive multiple of 8."""
        assert (size > 0) and (size % 8 == 0), f"Size must be positive and multiple of 8, got {size}"
        self.pool: torch.Tensor = torch.empty(size, dtype=torch.int8, device=device)
        self.size = self.pool.untyped_storage().nbytes()
        self.offset = 0

    def can_store(self, t: torch.Tensor) -> bool:
        return (self.pool.device == t.device) and (self.size - self.offset >= get_aligned_size(t))

    def copy_to_pool(self, t: torch.Tensor) -> torch.Tensor:
        """Copy `t` into the pool; returns a tensor of the same shape/stride/dtype viewing pool memory."""
        assert t.device == self.pool.device
        assert self.can_store(t)
        # a stride of 0 (expanded dim) would alias on write: the copy gets stride 1 there instead
        stride = tuple(s if s > 0 else 1 for s in t.stride())
        view = torch.as_strided(
            self.pool.view(t.dtype), size=t.size(), stride=stride, storage_offset=self.offset // t.element_size()
        )
        view.copy_(t)
        self.offset += get_aligned_size(t)
        return view

    def reset(self):
        self.offset = 0
