"""The entry point that allocates nothing (`kernl_attention_skinny_static_fwd`, partial results in a static device
array) against `kernl_attention_skinny_fwd` with a caller-provided workspace: bit-identical outputs, on two calls in
a row with the second on a smaller input (the array keeps the first call's contents), and against the oracle."""
import pytest
import torch

from kernl_amd import _lib
from oracle import attention_oracle

from conftest import check_close

pytestmark = pytest.mark.gpu


def _both(shape_q, n_keys, seed, causal=False, with_mask=False):
    gen = torch.Generator().manual_seed(seed)
    B, H, M, D = shape_q
    q = torch.randn(shape_q, generator=gen).half()
    k = torch.randn((B, H, n_keys, D), generator=gen).half()
    v = torch.randn((B, H, n_keys, D), generator=gen).half()
    mask = None
    if with_mask:
        mask = torch.zeros((B, 1, 1, n_keys))
        mask[..., n_keys - n_keys // 3:] = float("-inf")
    dev = torch.device("cuda:0")
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    md = None if mask is None else mask.to(dev)
    clamp = torch.finfo(torch.float32).min if mask is not None else 0.0
    nbytes = _lib.attention_skinny_workspace_bytes(B, H, M, n_keys, D)
    assert nbytes <= _lib.load().kernl_attention_skinny_static_max_bytes()
    ws = torch.empty((max(nbytes, 4) // 4,), dtype=torch.float32, device=dev)
    ref = torch.empty(shape_q, dtype=torch.float16, device=dev)
    _lib.attention_skinny_fwd(qd, kd, vd, ref, md, ws if nbytes > 0 else None, D ** -0.5, causal, clamp)
    out = torch.full(shape_q, float("nan"), dtype=torch.float16, device=dev)
    _lib.attention_skinny_static_fwd(qd, kd, vd, out, md, D ** -0.5, causal, clamp)
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), "static-buffer result differs from the workspace result"
    check_close(out, attention_oracle(q, k, v, D ** -0.5, causal, mask), torch.float16, what="skinny static")
    return nbytes


def test_static_buffer_entry_matches_workspace_entry_twice_in_a_row():
    big = _both((2, 8, 1, 128), 4096, seed=0, with_mask=True)
    small = _both((1, 4, 1, 64), 777, seed=1)
    assert big > small > 0  # both calls really split the keys, the second over a smaller part of the array
    _both((2, 8, 1, 128), 4096, seed=2, causal=True)


def test_static_buffer_entry_allocates_nothing_and_replays_from_a_graph():
    """The use the entry point is for: captured in a hipGraph (after the once-per-device lookup outside capture) and
    replayed on changed inputs, with torch's allocator untouched by the call; every replay is compared with the
    workspace entry on the same inputs, with eager work and synchronisations between the replays."""
    dev = torch.device("cuda:0")
    gen = torch.Generator().manual_seed(7)
    B, H, N, D = 2, 8, 2048, 128
    q = torch.randn((B, H, 1, D), generator=gen).half().to(dev)
    k = torch.randn((B, H, N, D), generator=gen).half().to(dev)
    v = torch.randn((B, H, N, D), generator=gen).half().to(dev)
    out = torch.empty_like(q)
    ref = torch.empty_like(q)
    nbytes = _lib.attention_skinny_workspace_bytes(B, H, 1, N, D)
    assert 0 < nbytes <= _lib.load().kernl_attention_skinny_static_max_bytes()
    ws = torch.empty((nbytes // 4,), dtype=torch.float32, device=dev)
    _lib.attention_skinny_static_init(dev)  # the address lookup, outside capture
    torch.cuda.synchronize()
    before = (torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev))
    _lib.attention_skinny_static_fwd(q, k, v, out, None, D ** -0.5, False, 0.0)
    torch.cuda.synchronize()
    assert (torch.cuda.memory_allocated(dev), torch.cuda.memory_reserved(dev)) == before
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        _lib.attention_skinny_static_fwd(q, k, v, out, None, D ** -0.5, False, 0.0)
    torch.cuda.synchronize()
    for r in range(3):
        q.copy_(torch.randn(q.shape, generator=gen).half())
        k[:, :, r::3].mul_(-0.5)
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        _lib.attention_skinny_fwd(q, k, v, ref, None, ws, D ** -0.5, False, 0.0)
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), f"replay {r} differs from the workspace entry"
        check_close(out, attention_oracle(q.cpu(), k.cpu(), v.cpu(), D ** -0.5, False, None), torch.float16, what=f"skinny static replay {r}")


def test_static_buffer_entry_refuses_what_does_not_fit():
    lib = _lib.load()
    B, H, M, N, D = 5, 80, 1, 4096, 256
    assert _lib.attention_skinny_workspace_bytes(B, H, M, N, D) > lib.kernl_attention_skinny_static_max_bytes()
    dev = torch.device("cuda:0")
    q = torch.zeros((1, 1, 1, 8), dtype=torch.float16, device=dev)  # never read: the size check comes first
    with pytest.raises(_lib.KernlLibraryError, match="static buffer holds"):
        import ctypes

        s4 = (ctypes.c_int64 * 4)(D * N, D * N, D, 1)
        st = lib.kernl_attention_skinny_static_fwd(q.data_ptr(), q.data_ptr(), q.data_ptr(), q.data_ptr(), None,
                                                   B, H, M, N, D, s4, s4, s4, s4, None, None, 2, 1.0, 0, 0.0, 0, None)
        _lib._check(st, "kernl_attention_skinny_static_fwd")
