"""GPU parity of the split-K single-query attention kernel against the CPU oracle.

Shapes follow the reference's skinny cross-attention cases (test/test_attention.py:176-208: batch 1 / 5, 6 / 16 / 20
heads, 1500 keys, head size 64, one query, sm_scale 0.3, inputs U(0, 1)), plus what the reference sends to eager
PyTorch instead (masks, the causal flag), other head sizes, strided keys and the dispatch inside attention_wrapper.
"""
import pytest
import torch

from kernl_amd import _lib
from kernl_amd.implementations.attention_skinny import skinny_attention_forward
from kernl_amd.optimizer.attention import attention_wrapper
from oracle import attention_oracle

pytestmark = pytest.mark.gpu


def _run(q, k, v, sm_scale, causal, mask):
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    out = torch.empty_like(qc)
    skinny_attention_forward(qc, kc, vc, out, sm_scale, is_causal=causal, attention_mask=None if mask is None else mask.cuda())
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize(
    "shape",
    [(1, 6, 1500, 64), (5, 6, 1500, 64), (1, 16, 1500, 64), (5, 16, 1500, 64), (1, 20, 1500, 64), (5, 20, 1500, 64)],
    ids=["tiny-beam-1", "tiny-beam-5", "medium-beam-1", "medium-beam-5", "large-beam-1", "large-beam-5"],
)
def test_skinny_cross_attention(shape, dtype, close):
    batch, heads, seqlen, dhead = shape
    gen = torch.Generator().manual_seed(0)
    q = torch.rand((batch, heads, 1, dhead), generator=gen).to(dtype)
    k = torch.rand((batch, heads, seqlen, dhead), generator=gen).to(dtype)
    v = torch.rand((batch, heads, seqlen, dhead), generator=gen).to(dtype)
    print(f"case shape={shape} dtype={dtype}", flush=True)
    out = _run(q, k, v, 0.3, False, None)
    close(out, attention_oracle(q, k, v, 0.3, False, None), dtype, what=f"skinny {shape}")


@pytest.mark.parametrize("mask_kind", ["padding", "bias_row", "bias_full", "all_masked"])
@pytest.mark.parametrize("shape", [(2, 4, 1, 777, 64), (1, 8, 1, 2048, 128), (3, 2, 1, 51, 32), (2, 2, 3, 300, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_skinny_masks(shape, mask_kind, close):
    B, H, M, N, D = shape
    gen = torch.Generator().manual_seed(1)
    q = torch.randn((B, H, M, D), generator=gen).half()
    k = torch.randn((B, H, N, D), generator=gen).half()
    v = torch.randn((B, H, N, D), generator=gen).half()
    if mask_kind == "padding":
        mask = torch.zeros((B, 1, 1, N))
        for b in range(B):
            mask[b, :, :, int(torch.randint(1, N + 1, (1,), generator=gen)):] = float("-inf")
    elif mask_kind == "bias_row":
        mask = torch.randn((1, H, 1, N), generator=gen).half()
    elif mask_kind == "bias_full":
        mask = torch.randn((B, H, M, N), generator=gen)
    else:
        mask = torch.full((B, 1, 1, N), float("-inf"))
    print(f"case shape={shape} mask={mask_kind}", flush=True)
    out = _run(q, k, v, D ** -0.5, False, mask)
    if mask_kind == "all_masked":
        # -inf entries are clamped to finfo.min (reference attention.py:380): a fully masked row is the plain average
        # of V, not NaN (the closed-form oracle does not model the clamp)
        ref = v.float().mean(dim=-2, keepdim=True).expand(-1, -1, M, -1)
    else:
        ref = attention_oracle(q, k, v, D ** -0.5, False, mask)
    close(out, ref, torch.float16, what=f"skinny {shape} {mask_kind}")


def test_skinny_causal_rows(close):
    # top-left aligned causal masking: query row m sees keys 0..m (reference attention.py:346-347)
    gen = torch.Generator().manual_seed(2)
    q = torch.randn((2, 3, 4, 64), generator=gen).half()
    k = torch.randn((2, 3, 200, 64), generator=gen).half()
    v = torch.randn((2, 3, 200, 64), generator=gen).half()
    out = _run(q, k, v, 0.125, True, None)
    close(out, attention_oracle(q, k, v, 0.125, True, None), torch.float16, what="skinny causal")
    # row 0 attends to key 0 only
    assert torch.equal(out[:, :, 0].cpu(), v[:, :, 0])


def test_skinny_strided_inputs(close):
    # K and V as permuted views of [B, N, H, D] buffers (how projections leave them), q sliced from a longer sequence
    gen = torch.Generator().manual_seed(3)
    B, H, N, D = 2, 6, 640, 64
    kbuf = torch.randn((B, N, H, D), generator=gen).half()
    vbuf = torch.randn((B, N, H, D), generator=gen).half()
    qbuf = torch.randn((B, H, 5, D), generator=gen).half()
    kc, vc, qc = kbuf.cuda().permute(0, 2, 1, 3), vbuf.cuda().permute(0, 2, 1, 3), qbuf.cuda()[:, :, 2:3]
    assert not kc.is_contiguous() and not qc.is_contiguous()
    out = torch.empty((B, H, 1, D), dtype=torch.half, device="cuda")
    skinny_attention_forward(qc, kc, vc, out, 0.125)
    torch.cuda.synchronize()
    ref = attention_oracle(qbuf[:, :, 2:3], kbuf.permute(0, 2, 1, 3), vbuf.permute(0, 2, 1, 3), 0.125, False, None)
    close(out, ref, torch.float16, what="skinny strided")


def test_skinny_small_workspace_only_costs_parallelism(close):
    # calling through the C ABI with no workspace: a single key range, same result
    gen = torch.Generator().manual_seed(4)
    q = torch.randn((1, 4, 1, 64), generator=gen).half()
    k = torch.randn((1, 4, 900, 64), generator=gen).half()
    v = torch.randn((1, 4, 900, 64), generator=gen).half()
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    out = torch.empty_like(qc)
    _lib.attention_skinny_fwd(qc, kc, vc, out, None, None, 0.125, False, 0.0)
    torch.cuda.synchronize()
    close(out, attention_oracle(q, k, v, 0.125, False, None), torch.float16, what="skinny no workspace")


def test_attention_wrapper_dispatches_single_query(monkeypatch, close):
    # reference dispatch: q_len == 1 and more than 50 keys go to the split-K kernel (optimizer/attention.py:45-49)
    import kernl_amd.optimizer.attention as opt

    calls = []
    real = opt.skinny_attention_forward
    monkeypatch.setattr(opt, "skinny_attention_forward", lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    gen = torch.Generator().manual_seed(5)
    for n_keys, expected_calls in ((1500, 1), (40, 1)):
        q = torch.randn((2, 4, 1, 64), generator=gen).half()
        k = torch.randn((2, 4, n_keys, 64), generator=gen).half()
        v = torch.randn((2, 4, n_keys, 64), generator=gen).half()
        out = torch.empty((2, 4, 1, 64), dtype=torch.half, device="cuda")
        attention_wrapper(q.cuda(), k.cuda(), v.cuda(), out, 0.125, False, None)
        torch.cuda.synchronize()
        close(out, attention_oracle(q, k, v, 0.125, False, None), torch.float16, what=f"wrapper q_len 1, {n_keys} keys")
        assert len(calls) == expected_calls


def test_attention_wrapper_keeps_very_large_decode_batches_on_the_tiled_kernel(monkeypatch, close):
    # more rows (batch x heads) than the split-K kernel's grid holds: the wrapper must not hand them over
    import kernl_amd.optimizer.attention as opt

    calls = []
    real = opt.skinny_attention_forward
    monkeypatch.setattr(opt, "skinny_attention_forward", lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    B, H, N, D = 2200, 32, 64, 64                       # 70400 rows
    gen = torch.Generator(device="cuda").manual_seed(11)
    q = torch.randn((B, H, 1, D), generator=gen, device="cuda", dtype=torch.half)
    k = torch.randn((B, H, N, D), generator=gen, device="cuda", dtype=torch.half)
    v = torch.randn((B, H, N, D), generator=gen, device="cuda", dtype=torch.half)
    out = torch.empty_like(q)
    attention_wrapper(q, k, v, out, 0.125, False, None)
    torch.cuda.synchronize()
    assert not calls
    for b in (0, 1099, B - 1):                          # the oracle on three batch entries, first to last
        sl = slice(b, b + 1)
        close(out[sl], attention_oracle(q[sl].cpu(), k[sl].cpu(), v[sl].cpu(), 0.125, False, None), torch.float16,
              what=f"70400-row decode, batch entry {b}")


def test_skinny_rejects_unsupported_head_size():
    q = torch.zeros((1, 1, 1, 48), dtype=torch.half, device="cuda")
    k = torch.zeros((1, 1, 64, 48), dtype=torch.half, device="cuda")
    with pytest.raises(_lib.KernlLibraryError, match="head size"):
        skinny_attention_forward(q, k, k.clone(), torch.empty_like(q), 1.0)


@pytest.mark.parametrize("storage", ["int8", "float8_e5m2"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 4, 1, 777, 64), (1, 8, 1, 4096, 128), (3, 2, 1, 51, 32), (2, 2, 3, 300, 64),
                                   (1, 2, 1, 9, 8)], ids=lambda s: "x".join(map(str, s)))
def test_skinny_fp8_keys_and_values(shape, dtype, storage, close):
    """Keys and values stored as fp8 e5m2 (reference: the int8 caches of experimental/llama-v2/kernel/
    fused_kernel_fp8.py:68-72, read by fused_kernel_attention.py:69-71,90-92): the kernel decodes the bytes and
    computes as before, so it must match the oracle run on the DECODED keys and values — and the storage conversion
    itself must match the oracle's decoder."""
    from kernl_amd.implementations.attention_skinny import from_e5m2, to_e5m2
    from oracle import e5m2_decode_oracle

    B, H, M, N, D = shape
    gen = torch.Generator().manual_seed(9)
    q = torch.randn((B, H, M, D), generator=gen).to(dtype)
    k = torch.randn((B, H, N, D), generator=gen)
    v = torch.randn((B, H, N, D), generator=gen)
    k8, v8 = to_e5m2(k), to_e5m2(v)
    assert k8.dtype == torch.int8 and k8.shape == k.shape
    k_dec, v_dec = e5m2_decode_oracle(k8), e5m2_decode_oracle(v8)
    assert torch.equal(from_e5m2(k8, torch.float32), k_dec)
    assert (k_dec - k).abs().max() <= 0.125 * k.abs().max()  # 2 mantissa bits: relative step 1/8 at most
    mask = torch.rand((B, 1, 1, N), generator=gen)
    if storage == "float8_e5m2":
        k8, v8 = k8.view(torch.float8_e5m2), v8.view(torch.float8_e5m2)
    qc = q.cuda()
    out = torch.empty_like(qc)
    skinny_attention_forward(qc, k8.cuda(), v8.cuda(), out, 0.25, is_causal=False, attention_mask=mask.cuda())
    torch.cuda.synchronize()
    close(out, attention_oracle(q, k_dec, v_dec, 0.25, False, mask), dtype, what=f"skinny fp8 kv {shape}")


def test_skinny_fp8_rejects_misaligned_rows():
    q = torch.randn((1, 1, 1, 64), device="cuda", dtype=torch.float16)
    kv = torch.zeros((1, 1, 16, 68), device="cuda", dtype=torch.int8)[..., 4:]  # rows start 4 bytes off an 8-byte boundary
    out = torch.empty_like(q)
    with pytest.raises(RuntimeError, match="8-byte aligned"):
        skinny_attention_forward(q, kv, kv, out, 1.0)
