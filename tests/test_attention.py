"""GPU parity of the fused attention kernel against the CPU oracle.

Shapes, mask kinds and stride cases follow the reference's test/test_attention.py:62-145 (tile-edge sequence lengths
8..512 and 1500, broadcast padding mask, full bias mask, mixed strides, cross-attention), sized so the fp32 oracle
finishes in seconds; BASELINE config 1 ([32,12,512,64] with padding lengths in [256,512]) runs at full size.
"""
import pytest
import torch

from kernl_amd import _lib
from kernl_amd.implementations.attention import attention_forward
from oracle import attention_oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["auto", "streaming", "pipelined", "split"])
def attention_kernel(request):
    """Every case runs four times: with the library's own choice between its MFMA kernels, with the streaming kernel
    forced, with the software-pipelined kernel forced wherever it applies (head size 64; no mask, per-key mask or
    causal) — by default that kernel only takes 1024 keys or more, which few of the shapes here have — and with the
    streaming kernel's small-grid form (32-row workgroups whose waves split the key tiles) forced wherever it applies
    (head size 64, non-causal, no mask or a per-key mask, up to 4096 keys), whatever the grid: one tile for four waves,
    ragged tiles, rows beyond M, fully masked rows and tiles all go through its merge."""
    lib = _lib.load()
    lib.kernl_attention_set_variant({"auto": 0, "streaming": 3, "pipelined": 4, "split": 5}[request.param])
    yield request.param
    lib.kernl_attention_set_variant(0)


def _mk(shape, dtype, gen, lo=None):
    if lo is None:
        t = torch.randn(shape, generator=gen)
    else:
        t = torch.rand(shape, generator=gen) * 2.0  # U(0, 2) as in the reference test
    return t.to(dtype)


def _run(q, k, v, sm_scale, causal, mask):
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    out = torch.empty_like(qc)
    attention_forward(qc, kc, vc, out, sm_scale, is_causal=causal, attention_mask=None if mask is None else mask.cuda())
    torch.cuda.synchronize()
    return out


SHAPES = [
    (1, 3, 8, 64), (2, 3, 16, 64), (1, 2, 33, 64), (2, 2, 128, 64), (1, 2, 257, 64), (2, 4, 384, 64),
    (1, 4, 512, 64), (1, 1, 1500, 64), (1, 2, 128, 128), (1, 2, 200, 128), (1, 1, 1024, 128),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("causal", [False, True], ids=["noncausal", "causal"])
@pytest.mark.parametrize("mask_kind", ["none", "padding", "bias"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_attention_vs_oracle(shape, mask_kind, causal, dtype, close):
    B, H, S, D = shape
    gen = torch.Generator().manual_seed(0)
    q, k, v = (_mk(shape, dtype, gen) for _ in range(3))
    sm_scale = 0.3 if D == 64 else 0.125
    mask = None
    if mask_kind == "padding":
        lengths = torch.randint(1, S + 1, (B,), generator=gen)
        mask = torch.zeros((B, 1, 1, S))
        for b in range(B):
            mask[b, :, :, lengths[b]:] = float("-inf")
    elif mask_kind == "bias":
        mask = torch.rand((B, H, S, S), generator=gen)
    print(f"case shape={shape} mask={mask_kind} causal={causal} dtype={dtype}", flush=True)
    out = _run(q, k, v, sm_scale, causal, mask)
    ref = attention_oracle(q, k, v, sm_scale, causal, mask)
    close(out, ref, dtype, what=f"attention {shape} {mask_kind} causal={causal}")


@pytest.mark.parametrize("mask_dtype", ["fp32", "same"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("keys", [200, 512, 1500])
def test_per_key_mask_of_every_dtype_and_length(keys, dtype, mask_dtype, close):
    """Per-key masks with ordinary values, a -inf tail and a fully masked batch entry, as fp32 and in the inputs' 16-bit
    type, on rows that one wave classifies by itself (up to 512 keys) and on longer ones, with enough (batch, head) pairs
    that the persistent kernel walks several items per workgroup (its next item's query and mask rows are prefetched
    into LDS while the current one finishes)."""
    B, H, D = 9, 16, 64
    gen = torch.Generator().manual_seed(keys)
    q, k, v = (_mk((B, H, keys, D), dtype, gen) for _ in range(3))
    mask = torch.randn((B, 1, 1, keys), generator=gen)
    lengths = torch.randint(1, keys + 1, (B,), generator=gen)
    for b in range(B):
        if b % 3 != 0:
            mask[b, :, :, : lengths[b]] = 0.0          # a plain padding mask: zeros, then -inf
        mask[b, :, :, lengths[b]:] = float("-inf")
    mask[4] = float("-inf")                            # nothing visible: the plain average of V
    mask = mask.to(torch.float32 if mask_dtype == "fp32" else dtype)
    print(f"case keys={keys} dtype={dtype} mask={mask.dtype}", flush=True)
    out = _run(q, k, v, 0.125, False, mask)
    ref = attention_oracle(q, k, v, 0.125, False, mask)
    # every key at -inf: the reference kernel replaces -inf by the most negative finite value of the MASK's dtype
    # (attention.py:380,516) and adds that to the fp32 scores — an fp32 minimum absorbs them (uniform softmax), a
    # half-precision one (-65504) leaves them their weight; the closed form above has no such row
    floor = torch.full((1, 1, 1, keys), torch.finfo(mask.dtype).min, dtype=torch.float32)
    ref[4] = attention_oracle(q[4:5], k[4:5], v[4:5], 0.125, False, floor)[0]
    close(out, ref, dtype, what=f"per-key mask {keys} {mask.dtype}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("keys", [512, 1536])
def test_padding_masks_in_the_model_dtype_drop_the_same_tiles(keys, dtype, close):
    """A padding mask built in the model's dtype with `finfo(dtype).min` beyond the length (what transformers' mask
    builders produce: -65504 for fp16) marks dead keys just as -inf in fp32 does: the key tiles it covers entirely are
    not visited, and the result is bit for bit the one the fp32 -inf mask gives (and close to the oracle's)."""
    B, H, D = 6, 12, 64
    gen = torch.Generator().manual_seed(keys + 1)
    q, k, v = (_mk((B, H, keys, D), dtype, gen) for _ in range(3))
    lengths = torch.tensor([keys, keys // 2 + 3, 64, 65, keys - 1, 200])
    visible = torch.arange(keys)[None, :] < lengths[:, None]
    m32 = torch.where(visible, 0.0, float("-inf"))[:, None, None, :]
    m16 = torch.where(visible, 0.0, torch.finfo(dtype).min).to(dtype)[:, None, None, :]
    out32 = _run(q, k, v, 0.125, False, m32)
    out16 = _run(q, k, v, 0.125, False, m16)
    assert torch.equal(out32, out16)
    close(out16, attention_oracle(q, k, v, 0.125, False, m16), dtype, what=f"model-dtype padding mask {keys} {dtype}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
def test_causal_attention_with_left_padding(dtype, close):
    """The causal flag together with a per-key padding mask whose hidden keys come FIRST (left-padded prompts): the rows
    inside the padding see hidden keys only and get their plain average of V (the mask holds the most negative fp32
    value, which absorbs every score), the rows behind it see the visible keys of their causal prefix — key tiles that
    hold hidden keys only are still visited wherever a row depends on them."""
    B, H, S, D = 4, 3, 512, 64
    gen = torch.Generator().manual_seed(21)
    q, k, v = (_mk((B, H, S, D), dtype, gen) for _ in range(3))
    pad = torch.tensor([0, 70, 130, 511])
    hidden = torch.arange(S)[None, :] < pad[:, None]
    mask = torch.where(hidden, torch.finfo(torch.float32).min, 0.0)[:, None, None, :]
    out = _run(q, k, v, 0.125, True, mask)
    ref = attention_oracle(q, k, v, 0.125, True, mask)
    assert torch.isfinite(out).all()
    close(out, ref, dtype, what=f"causal + left padding {dtype}")


def test_attention_u02_inputs_like_reference(close):
    # reference draws q, k, v from U(0, 2) with sm_scale 0.3 (test/test_attention.py:91-99): large positive logits
    gen = torch.Generator().manual_seed(1)
    shape = (2, 4, 256, 64)
    q, k, v = (_mk(shape, torch.float16, gen, lo=0) for _ in range(3))
    out = _run(q, k, v, 0.3, False, None)
    close(out, attention_oracle(q, k, v, 0.3), what="attention U(0,2)")


def test_attention_mixed_strides(close):
    # reference test/test_attention.py:110-129: column-major q, batch-interleaved k, transposed mask
    gen = torch.Generator().manual_seed(2)
    B, H, S, D = 2, 3, 96, 64
    q = torch.randn((B, H, D, S), generator=gen).half().transpose(-1, -2)  # feature stride != 1 -> scalar kernel
    k = torch.randn((H, B, S, D), generator=gen).half().transpose(0, 1)     # batch/head swapped strides
    v = torch.randn((B, H, S, D), generator=gen).half()
    mask = torch.rand((B, H, S, S), generator=gen).transpose(-1, -2)
    out = _run(q, k, v, 0.3, False, mask)
    close(out, attention_oracle(q, k, v, 0.3, False, mask), what="attention mixed strides")


def test_attention_bert_permuted_views(close):
    # q/k/v as BERT produces them: [B,S,H,D] linear outputs viewed as [B,H,S,D]
    gen = torch.Generator().manual_seed(3)
    B, H, S, D = 2, 12, 160, 64
    q, k, v = (torch.randn((B, S, H, D), generator=gen).half().permute(0, 2, 1, 3) for _ in range(3))
    lengths = torch.tensor([160, 97])
    mask = torch.zeros((B, 1, 1, S))
    for b in range(B):
        mask[b, :, :, lengths[b]:] = torch.finfo(torch.float32).min
    out = _run(q, k, v, 0.125, False, mask)
    close(out, attention_oracle(q, k, v, 0.125, False, mask), what="attention permuted views")


def test_attention_cross_attention_single_query(close):
    # reference test/test_attention.py:133-145: q_len 1, k_len 24, mask [1, 8, 1, 24]
    gen = torch.Generator().manual_seed(4)
    q = torch.randn((5, 8, 1, 64), generator=gen).half()
    k = torch.randn((5, 8, 24, 64), generator=gen).half()
    v = torch.randn((5, 8, 24, 64), generator=gen).half()
    mask = torch.randn((1, 8, 1, 24), generator=gen)
    out = _run(q, k, v, 1.0, False, mask)
    close(out, attention_oracle(q, k, v, 1.0, False, mask), what="cross attention")


def test_attention_scalar_kernel_matches(close):
    gen = torch.Generator().manual_seed(5)
    shape = (1, 2, 130, 64)
    q, k, v = (_mk(shape, torch.float16, gen) for _ in range(3))
    mask = torch.rand((1, 2, 130, 130), generator=gen)
    lib = _lib.load()
    lib.kernl_attention_force_scalar(1)
    try:
        for causal in (False, True):
            out = _run(q, k, v, 0.2, causal, mask)
            close(out, attention_oracle(q, k, v, 0.2, causal, mask), what=f"scalar kernel causal={causal}")
    finally:
        lib.kernl_attention_force_scalar(0)


def test_attention_head_size_not_mfma(close):
    gen = torch.Generator().manual_seed(6)
    shape = (1, 2, 70, 80)
    q, k, v = (_mk(shape, torch.float16, gen) for _ in range(3))
    out = _run(q, k, v, 0.1, True, None)
    close(out, attention_oracle(q, k, v, 0.1, True, None), what="head size 80")


def test_fully_masked_row_is_finite_uniform_average():
    # -inf mask entries are clamped to finfo.min (reference attention.py:380): a row whose keys are all masked
    # returns the plain average of V instead of NaN.
    gen = torch.Generator().manual_seed(7)
    shape = (2, 2, 128, 64)
    q, k, v = (_mk(shape, torch.float16, gen) for _ in range(3))
    mask = torch.zeros((2, 1, 1, 128))
    mask[1] = float("-inf")
    out = _run(q, k, v, 0.125, False, mask).float().cpu()
    assert torch.isfinite(out).all()
    expected = v[1].float().mean(dim=-2, keepdim=True).expand(-1, 128, -1)
    assert (out[1] - expected).abs().max().item() < 5e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("kind", ["all_very_negative", "growing", "shrinking", "first_tiles_masked", "huge_then_small", "small_then_huge",
                                  "half_min_bias"])
def test_softmax_reference_moves_with_the_scores(kind, dtype, close):
    """The kernel keeps scores relative to a per-row exponent reference that moves lazily: up when a score exceeds it
    by more than 2^8, down only while the row has accumulated nothing.  Each case drives one of those moves: scores
    that are all far below zero, that grow or shrink from key tile to key tile, rows whose first key tiles are fully
    masked, and one dominant key followed by ordinary ones."""
    gen = torch.Generator().manual_seed(21)
    B, H, S, D = 2, 2, 320, 64  # 5 key tiles of 64
    q = torch.randn((B, H, S, D), generator=gen)
    k = torch.randn((B, H, S, D), generator=gen)
    v = torch.randn((B, H, S, D), generator=gen)
    mask = None
    tile = torch.arange(S) // 64
    if kind == "all_very_negative":
        # every score near -60 (natural-log units): exp underflows in 16 bits unless the reference follows
        q = q * 0.1 + 1.0
        k = k * 0.1 - 7.5
    elif kind == "growing":
        k = k * (1.0 + 1.5 * tile.float())[None, None, :, None]
    elif kind == "shrinking":
        k = k * (7.0 - 1.5 * tile.float())[None, None, :, None]
    elif kind == "first_tiles_masked":
        mask = torch.rand((B, H, S, S), generator=gen)
        mask[:, :, ::2, :128] = float("-inf")   # even rows: the first two key tiles are masked out entirely
        mask[:, :, 1::3, 64:192] = float("-inf")
    elif kind == "half_min_bias":
        # additive masks of finfo(float16).min, as half-precision models build them: a masked prefix on some rows,
        # every key masked on others (those rows are a softmax over the masked keys, in the oracle too)
        mask = torch.zeros((B, H, S, S))
        mask[:, :, ::2, :150] = -65504.0
        mask[:, :, 7::16, :] = -65504.0
    elif kind == "huge_then_small":
        k[:, :, 5, :] = q[:, :, 40, :] * 4.0      # one dominant key in the first tile for row 40 (and large for others)
    elif kind == "small_then_huge":
        # a dominant key in the LAST tile (a later clean tile of its wave in the small-grid form too): row 40's score there
        # is ~46 octaves above everything in its first tile, so steps that trust the first tile's reference overflow 16
        # bits and the tiles have to be walked again in full
        k[:, :, 300, :] = q[:, :, 40, :] * 4.0
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    out = _run(q, k, v, 0.125, False, mask)
    ref = attention_oracle(q, k, v, 0.125, False, mask)
    assert torch.isfinite(out.float()).all()
    close(out, ref, dtype, what=f"attention reference moves: {kind}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("mask_kind", ["none", "bias"])
@pytest.mark.parametrize("case", [(1, 4, 1, 300, 64), (2, 3, 17, 64, 64), (1, 2, 130, 333, 64), (1, 2, 128, 128, 128),
                                  (1, 1, 300, 1000, 128), (2, 2, 64, 0, 64), (1, 2, 40, 700, 80)],
                         ids=lambda c: "x".join(map(str, c)))
def test_causal_attention_over_a_cache(case, mask_kind, dtype, close):
    """M new query rows at positions start.. against the start + M (+ a few unused) keys of a cache
    (reference: experimental/llama-v2/kernel/fused_kernel_attention.py, `start_position`; mask semantics
    llama/model.py:338-343).  Head size 80 takes the scalar kernel."""
    B, H, M, start, D = case
    N = start + M + (5 if start % 2 else 0)   # some cases carry keys beyond every row's horizon
    gen = torch.Generator().manual_seed(23)
    q = torch.randn((B, H, M, D), generator=gen).to(dtype)
    k = torch.randn((B, H, N, D), generator=gen).to(dtype)
    v = torch.randn((B, H, N, D), generator=gen).to(dtype)
    mask = torch.rand((B, H, M, N), generator=gen) if mask_kind == "bias" else None
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    out = torch.empty_like(qc)
    attention_forward(qc, kc, vc, out, 0.2, is_causal=True, attention_mask=None if mask is None else mask.cuda(),
                      start_position=start)
    torch.cuda.synchronize()
    ref = attention_oracle(q, k, v, 0.2, True, mask, start_position=start)
    close(out, ref, dtype, what=f"cached causal attention {case} {mask_kind}")


def test_attention_properties_full_size(close):
    # BASELINE config 1 at full size: [32,12,512,64], padding lengths U[256,512], scale 1/8.
    gen = torch.Generator().manual_seed(0)
    shape = (32, 12, 512, 64)
    q, k, v = (torch.randn(shape, generator=gen).half() for _ in range(3))
    lengths = torch.randint(256, 513, (32,), generator=gen)
    mask = torch.zeros((32, 1, 1, 512))
    for b in range(32):
        mask[b, :, :, lengths[b]:] = float("-inf")
    out = _run(q, k, v, 0.125, False, mask)
    ref = attention_oracle(q, k, v, 0.125, False, mask)
    close(out, ref, what="config 1")
    # V = 1 => O = 1 exactly representable
    ones = torch.ones_like(v)
    out1 = _run(q, k, ones, 0.125, False, mask).float().cpu()
    assert (out1 - 1.0).abs().max().item() <= 2e-3
    # keys beyond the padding length must not influence the output: scramble them
    k2, v2 = k.clone(), v.clone()
    for b in range(32):
        k2[b, :, lengths[b]:] = 7.0
        v2[b, :, lengths[b]:] = -9.0
    out2 = _run(q, k2, v2, 0.125, False, mask)
    assert torch.equal(out2.cpu(), out.cpu())


def test_attention_rejects_bad_arguments():
    q = torch.zeros((1, 2, 16, 64), dtype=torch.float16, device="cuda")
    out = torch.empty_like(q)
    with pytest.raises(AssertionError):
        attention_forward(q.float(), q.float(), q.float(), out.float(), 1.0)  # fp32 not supported
    with pytest.raises(AssertionError):
        attention_forward(q, q, q, out, 1.0, False, torch.zeros((3, 1, 1, 16), device="cuda"))  # bad batch broadcast
    with pytest.raises(AssertionError):
        attention_forward(q, q, q, out, 1.0, False, torch.zeros((1, 1, 1, 15), device="cuda"))  # bad key count


@pytest.mark.parametrize("n_keys", [4096, 4100, 6000], ids=lambda n: f"{n}keys")
@pytest.mark.parametrize("mask_kind", ["padding", "all_masked"])
def test_attention_long_key_sequences_with_vector_mask(n_keys, mask_kind, close):
    # up to 64 key tiles the per-key mask is classified tile by tile (clean / general / dropped sets kept in two
    # 64-bit words); longer sequences take every tile through the general body
    gen = torch.Generator().manual_seed(11)
    q = torch.randn((1, 2, 160, 64), generator=gen).half()
    k = torch.randn((1, 2, n_keys, 64), generator=gen).half()
    v = torch.randn((1, 2, n_keys, 64), generator=gen).half()
    mask = torch.zeros((1, 1, 1, n_keys))
    if mask_kind == "padding":
        mask[..., n_keys - 1500:] = float("-inf")
        mask[..., 100:300] = float("-inf")
        ref = attention_oracle(q, k, v, 0.125, False, mask)
    else:
        mask[:] = float("-inf")
        ref = v.float().mean(dim=-2, keepdim=True).expand(-1, -1, 160, -1)
    out = _run(q, k, v, 0.125, False, mask)
    close(out, ref, torch.float16, what=f"attention {n_keys} keys {mask_kind}")


@pytest.mark.parametrize("mask_dtype", ["fp32", "same"], ids=["mask-fp32", "mask-16bit"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize(
    "layout", ["per_batch", "per_head", "shared", "full", "rows_padded", "with_minus_inf", "cross", "ragged_keys"]
)
def test_matrix_masks_of_every_layout(layout, dtype, mask_dtype, close):
    """One additive value per (query, key): broadcast over heads (a BERT-style extended mask, [B,1,M,N]), over the
    batch (a T5 position bias, [1,H,M,N]), over both, over neither; rows with padding between them; -inf entries;
    more keys than queries; key counts that are no multiple of the 64-key tile.  Head size 64 stages these masks
    through LDS, 16 bytes at a time, so fp32 and 16-bit masks take different routes."""
    B, H, M, N, D = 3, 5, 200, 200, 64
    if layout == "cross":
        M, N = 130, 328
    if layout == "ragged_keys":
        M, N = 128, 456          # 456 = 7 * 64 + 8: the last tile has one 16-byte chunk of 16-bit values
    gen = torch.Generator().manual_seed(17)
    q = _mk((B, H, M, D), dtype, gen)
    k, v = _mk((B, H, N, D), dtype, gen), _mk((B, H, N, D), dtype, gen)
    mdt = torch.float32 if mask_dtype == "fp32" else dtype
    mshape = {"per_batch": (B, 1, M, N), "per_head": (1, H, M, N), "shared": (1, 1, M, N)}.get(layout, (B, H, M, N))
    mask = (torch.randn(mshape, generator=gen) * 2.0).to(mdt)
    if layout == "with_minus_inf":
        mask = mask.float().masked_fill(torch.rand(mshape, generator=gen) < 0.3, float("-inf")).to(mdt)
        mask[..., 0] = 0.0       # no fully masked row
    mask_gpu = mask.cuda()
    if layout == "rows_padded":  # rows 16-byte aligned but not back to back
        wide = torch.zeros(mshape[:3] + (N + 24,), dtype=mdt, device="cuda")
        wide[..., :N] = mask_gpu
        mask_gpu = wide[..., :N]
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    out = torch.empty_like(qc)
    print(f"case layout={layout} dtype={dtype} mask={mdt} mask shape={tuple(mask_gpu.shape)} strides={mask_gpu.stride()}", flush=True)
    attention_forward(qc, kc, vc, out, 0.2, is_causal=False, attention_mask=mask_gpu)
    torch.cuda.synchronize()
    close(out, attention_oracle(q, k, v, 0.2, False, mask.float()), dtype, what=f"matrix mask {layout}")


def test_matrix_mask_config1_size_properties(close):
    """[32,12,512,64] with a [32,1,512,512] fp32 mask (workgroups mapped to XCDs by batch entry) and with a
    [1,12,512,512] bias: a sample of rows against the oracle, and — size independent — a mask that is constant along
    the keys of every row changes nothing."""
    B, H, S, D = 32, 12, 512, 64
    gen = torch.Generator(device="cuda").manual_seed(5)
    q, k, v = (torch.randn((B, H, S, D), generator=gen, device="cuda", dtype=torch.half) for _ in range(3))
    plain = torch.empty_like(q)
    attention_forward(q, k, v, plain, 0.125, is_causal=False, attention_mask=None)
    for mshape in ((B, 1, S, S), (1, H, S, S)):
        mask = torch.randn(mshape, generator=gen, device="cuda")
        out = torch.empty_like(q)
        attention_forward(q, k, v, out, 0.125, is_causal=False, attention_mask=mask)
        row_constant = mask[..., :1].expand(mshape).contiguous()
        same = torch.empty_like(q)
        attention_forward(q, k, v, same, 0.125, is_causal=False, attention_mask=row_constant)
        torch.cuda.synchronize()
        assert (same.float() - plain.float()).abs().max().item() <= 2e-3, f"row-constant mask {mshape} changed the result"
        for b, h in ((0, 0), (B - 1, H - 1), (13, 7)):
            mb, mh = (b if mshape[0] > 1 else 0), (h if mshape[1] > 1 else 0)
            ref = attention_oracle(q[b:b + 1, h:h + 1].cpu(), k[b:b + 1, h:h + 1].cpu(), v[b:b + 1, h:h + 1].cpu(), 0.125, False,
                                   mask[mb:mb + 1, mh:mh + 1].cpu())
            close(out[b:b + 1, h:h + 1], ref, torch.float16, what=f"matrix mask {mshape} at batch {b} head {h}")


@pytest.mark.parametrize("storage", ["int8", "float8_e5m2"])
@pytest.mark.parametrize("mask_kind", ["none", "padding"])
@pytest.mark.parametrize(
    "case",
    [(2, 3, 200, 200, 64, False, 0), (1, 4, 130, 333, 64, True, 203), (2, 2, 128, 128, 128, True, 0),
     (1, 2, 96, 1100, 128, True, 1004), (1, 2, 17, 64, 64, False, 0), (2, 2, 512, 512, 64, True, 0)],
    ids=lambda c: "x".join(map(str, c)),
)
def test_attention_over_fp8_keys_and_values(case, mask_kind, storage, close):
    """Keys and values stored as fp8 e5m2 bytes (reference: the int8 key/value caches of experimental/llama-v2/kernel/
    fused_kernel_fp8.py:68-74, widened on load by fused_kernel_attention.py:66-70, :90-94): the tiled kernel must give
    what the oracle gives on the DECODED keys and values — prefill over such a cache, with and without the causal
    diagonal shifted by `start_position`, ragged tiles, both head sizes."""
    from kernl_amd.implementations.attention_skinny import to_e5m2
    from oracle import e5m2_decode_oracle

    B, H, M, N, D, causal, start = case
    gen = torch.Generator().manual_seed(23)
    q = torch.randn((B, H, M, D), generator=gen).half()
    k8, v8 = to_e5m2(torch.randn((B, H, N, D), generator=gen)), to_e5m2(torch.randn((B, H, N, D), generator=gen))
    k_dec, v_dec = e5m2_decode_oracle(k8), e5m2_decode_oracle(v8)
    mask = None
    if mask_kind == "padding":
        lengths = torch.randint(max(1, N // 2), N + 1, (B,), generator=gen)
        mask = torch.zeros((B, 1, 1, N))
        for b in range(B):
            mask[b, :, :, lengths[b]:] = float("-inf")
    if storage == "float8_e5m2":
        k8, v8 = k8.view(torch.float8_e5m2), v8.view(torch.float8_e5m2)
    qc = q.cuda()
    out = torch.empty_like(qc)
    print(f"case {case} mask={mask_kind} storage={storage}", flush=True)
    attention_forward(qc, k8.cuda(), v8.cuda(), out, 0.2, is_causal=causal, attention_mask=None if mask is None else mask.cuda(),
                      start_position=start)
    torch.cuda.synchronize()
    ref = attention_oracle(q, k_dec, v_dec, 0.2, causal, mask, start)
    close(out, ref, torch.float16, what=f"fp8 keys/values {case} {mask_kind}")


def test_attention_fp8_keys_and_values_rejections():
    q = torch.zeros((1, 1, 64, 64), dtype=torch.bfloat16, device="cuda")
    kv = torch.zeros((1, 1, 64, 64), dtype=torch.int8, device="cuda")
    with pytest.raises(AssertionError, match="float16"):
        attention_forward(q, kv, kv, torch.empty_like(q), 1.0)
    q = q.half()
    with pytest.raises(_lib.KernlLibraryError, match="per-key"):
        attention_forward(q, kv, kv, torch.empty_like(q), 1.0, attention_mask=torch.zeros((1, 1, 64, 64), device="cuda"))
    q48, kv48 = torch.zeros((1, 1, 64, 48), dtype=torch.half, device="cuda"), torch.zeros((1, 1, 64, 48), dtype=torch.int8, device="cuda")
    with pytest.raises(_lib.KernlLibraryError, match="head size"):
        attention_forward(q48, kv48, kv48, torch.empty_like(q48), 1.0)
