"""GPU parity of LayerNorm / RMSNorm against the CPU oracle.

Cases follow the reference's test/test_layer_norm.py:47-123 (square shapes 128..4096, large-mean input
-20 + 0.5·randn, RMSNorm, transposed 250x250 input) plus BASELINE config 2's [16384, 768] at full size.
"""
import pytest
import torch

from kernl_amd.implementations.layer_norm import add_layer_norm, layer_norm
from oracle import effective_eps, embedding_layer_norm_oracle, layer_norm_oracle, rms_norm_oracle

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=["fp16", "bf16", "fp32"])
@pytest.mark.parametrize("shape", [128, 512, 1024, 2048, 4096], ids=lambda s: f"{s}x{s}")
def test_layer_norm_vs_oracle(shape, dtype, close):
    gen = torch.Generator().manual_seed(0)
    M = N = shape
    x = (-20 + 0.5 * torch.randn((M, N), generator=gen)).to(dtype)
    w = torch.rand((N,), generator=gen).to(dtype)
    b = torch.randn((N,), generator=gen).to(dtype)
    eps = 1e-5
    print(f"case {M}x{N} {dtype}", flush=True)
    out = layer_norm(x.cuda(), w.cuda(), b.cuda(), eps)
    torch.cuda.synchronize()
    ref = layer_norm_oracle(x, w, b, effective_eps(eps, dtype))
    close(out, ref, dtype, scale="magnitude", what=f"layernorm {shape}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(64, 128), (100, 768), (33, 1000), (7, 4096), (5, 8192), (3, 10000), (9, 250)],
                         ids=lambda s: "x".join(map(str, s)))
def test_rms_norm_vs_oracle(shape, dtype, close):
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(shape, generator=gen).to(dtype)
    w = (1 + 0.1 * torch.randn((shape[1],), generator=gen)).to(dtype)
    out = layer_norm(x.cuda(), w.cuda(), None, 1e-5, use_rms_norm=True)
    torch.cuda.synchronize()
    close(out, rms_norm_oracle(x, w, effective_eps(1e-5, dtype)), dtype, scale="magnitude", what=f"rmsnorm {shape}")


def test_layer_norm_odd_sizes_and_3d(close):
    gen = torch.Generator().manual_seed(2)
    for shape in [(3, 7, 768), (2, 5, 100), (4, 1, 8192), (2, 3, 9000), (1, 2, 3, 64)]:
        x = torch.randn(shape, generator=gen).half()
        w = (1 + 0.1 * torch.randn((shape[-1],), generator=gen)).half()
        b = (0.1 * torch.randn((shape[-1],), generator=gen)).half()
        out = layer_norm(x.cuda(), w.cuda(), b.cuda(), 1e-12)
        torch.cuda.synchronize()
        assert out.shape == x.shape
        close(out, layer_norm_oracle(x, w, b, effective_eps(1e-12, torch.float16)), scale="magnitude", what=f"layernorm {shape}")


def test_layer_norm_transposed_input(close):
    # reference test/test_layer_norm.py:110-123
    gen = torch.Generator().manual_seed(3)
    x = torch.randn((250, 250), generator=gen).half().t()
    w = torch.rand((250,), generator=gen).half()
    b = torch.randn((250,), generator=gen).half()
    assert not x.is_contiguous()
    xc = x.cuda()
    assert xc.stride() == x.stride() and not xc.is_contiguous()
    out = layer_norm(xc, w.cuda(), b.cuda(), 1e-5)
    torch.cuda.synchronize()
    close(out, layer_norm_oracle(x, w, b, 1.6e-5), scale="magnitude", what="layernorm transposed")


def test_layer_norm_config2_full_size(close):
    gen = torch.Generator().manual_seed(0)
    x = torch.randn((16384, 768), generator=gen).half()
    w = (1 + 0.1 * torch.randn((768,), generator=gen)).half()
    b = (0.1 * torch.randn((768,), generator=gen)).half()
    out = layer_norm(x.cuda(), w.cuda(), b.cuda(), 1e-12)
    torch.cuda.synchronize()
    close(out, layer_norm_oracle(x, w, b, effective_eps(1e-12, torch.float16)), scale="magnitude", what="config 2 layernorm")
    # size-independent properties: with w = 1, b = 0 every output row has mean 0 and mean square 1 - eps·rstd²
    ones, zeros = torch.ones((768,), dtype=torch.float16), torch.zeros((768,), dtype=torch.float16)
    y = layer_norm(x.cuda(), ones.cuda(), zeros.cuda(), 1e-12).float().cpu()
    assert y.mean(dim=-1).abs().max().item() < 2e-3
    assert (y.pow(2).mean(dim=-1) - 1).abs().max().item() < 5e-3
    # shifting a row by a constant does not change LayerNorm (up to the fp16 rounding of the shifted input)
    y2 = layer_norm((x.float() + 0.5).half().cuda(), ones.cuda(), zeros.cuda(), 1e-12).float().cpu()
    assert (y2 - y).abs().max().item() < 1e-2


@pytest.mark.parametrize("dtype,n", [(torch.float16, 768), (torch.bfloat16, 256), (torch.float32, 384),
                                     (torch.float16, 136), (torch.float32, 128), (torch.float16, 520)],
                         ids=["fp16-768", "bf16-256", "fp32-384", "fp16-136", "fp32-128", "fp16-520"])
def test_rows_that_share_a_wave(dtype, n, close):
    # rows of up to 32 or of 65..96 sixteen-byte chunks are taken two to a wave: odd row counts leave the last wave
    # with one row, and more rows than the grid holds make every wave walk several pairs
    from kernl_amd import _lib

    gen = torch.Generator().manual_seed(7)
    for rows in (1, 2, 7, 8, 9, 8201):
        x = (3 + 2 * torch.randn((rows, n), generator=gen)).to(dtype)
        r = torch.randn((rows, n), generator=gen).to(dtype)
        w = (1 + 0.1 * torch.randn((n,), generator=gen)).to(dtype)
        b = (0.1 * torch.randn((n,), generator=gen)).to(dtype)
        eps = effective_eps(1e-5, dtype)
        tol = dtype
        print(f"case rows={rows} n={n} {dtype}", flush=True)
        out = layer_norm(x.cuda(), w.cuda(), b.cuda(), 1e-5)
        close(out, layer_norm_oracle(x, w, b, eps), tol, scale="magnitude", what=f"layernorm {rows}x{n}")
        out = layer_norm(x.cuda(), w.cuda(), None, 1e-5, use_rms_norm=True)
        close(out, rms_norm_oracle(x, w, eps), tol, scale="magnitude", what=f"rmsnorm {rows}x{n}")
        out = add_layer_norm(x.cuda(), r.cuda(), w.cuda(), b.cuda(), 1e-5)
        close(out, layer_norm_oracle(x.float() + r.float(), w, b, eps), tol, scale="magnitude", what=f"add+layernorm {rows}x{n}")
        # the saved statistics of every row, those of a lone last row included
        xg, o = x.cuda(), torch.empty((rows, n), dtype=dtype, device="cuda")
        mean = torch.full((rows,), float("nan"), device="cuda")
        rstd = torch.full((rows,), float("nan"), device="cuda")
        _lib.layernorm_fwd(xg, w.cuda(), b.cuda(), o, mean, rstd, eps, False, None)
        torch.cuda.synchronize()
        xd = x.double()
        assert (mean.cpu().double() - xd.mean(dim=-1)).abs().max().item() < 1e-4
        want = (xd.var(dim=-1, unbiased=False) + eps).rsqrt()
        assert ((rstd.cpu().double() - want).abs() / want).max().item() < 1e-4


def test_add_layer_norm_matches_separate_add(close):
    gen = torch.Generator().manual_seed(4)
    for shape in [(512, 768), (4, 40, 768), (30, 1000)]:
        x = torch.randn(shape, generator=gen).half()
        r = torch.randn(shape, generator=gen).half()
        w = (1 + 0.1 * torch.randn((shape[-1],), generator=gen)).half()
        b = (0.1 * torch.randn((shape[-1],), generator=gen)).half()
        out = add_layer_norm(x.cuda(), r.cuda(), w.cuda(), b.cuda(), 1e-12)
        torch.cuda.synchronize()
        ref = layer_norm_oracle(x.float() + r.float(), w, b, 1.6e-5)
        close(out, ref, scale="magnitude", what=f"add+layernorm {shape}")


def test_layer_norm_rejects_bad_arguments():
    x = torch.zeros((4, 64), dtype=torch.float16, device="cuda")
    w = torch.ones((64,), dtype=torch.float16, device="cuda")
    with pytest.raises(AssertionError):
        layer_norm(x, w.float(), None, 1e-5)
    with pytest.raises(AssertionError):
        layer_norm(x, w, w.float(), 1e-5)


@pytest.mark.parametrize("form", ["two_dims", "no_affine", "two_dims_add", "no_affine_add", "broadcast_add"])
def test_functional_layer_norm_forms_all_reach_the_kernel(form, close, monkeypatch):
    """`F.layer_norm` over two trailing dimensions (= LayerNorm over their flattening), without weight and bias, and with
    an addition in front: every form runs on the LayerNorm kernel, none on PyTorch's."""
    import kernl_amd.optimizer.layer_norm as opt
    from oracle import layer_norm_oracle

    def forbidden(*a, **k):
        raise AssertionError("F.layer_norm was called")

    monkeypatch.setattr(torch.nn.functional, "layer_norm", forbidden)
    gen = torch.Generator().manual_seed(3)
    x = torch.randn((6, 10, 4, 64), generator=gen).half()
    y = torch.randn((6, 10, 4, 64), generator=gen).half()
    eps = 1.6e-5
    if form.startswith("two_dims"):
        w, b = (1 + 0.1 * torch.randn((4, 64), generator=gen)).half(), (0.1 * torch.randn((4, 64), generator=gen)).half()
        shape = (4, 64)
    else:
        w = b = None
        shape = (64,)
    wc, bc = (None if w is None else w.cuda()), (None if b is None else b.cuda())
    if form == "broadcast_add":
        out = opt.add_layer_norm_wrapper_functional(x.cuda(), y[:1].cuda(), shape, wc, bc, eps)
        src = x.float() + y[:1].float()
    elif form.endswith("_add"):
        out = opt.add_layer_norm_wrapper_functional(x.cuda(), y.cuda(), shape, wc, bc, eps)
        src = x.float() + y.float()
    else:
        out = opt.layer_norm_wrapper_functional(x.cuda(), shape, wc, bc, eps)
        src = x.float()
    torch.cuda.synchronize()
    n = 1
    for d in shape:
        n *= d
    flat = src.reshape(-1, n)
    if form == "broadcast_add":
        flat = (x + y[:1]).float().reshape(-1, n)   # the addition of two fp16 tensors rounds to fp16 first
    wf = torch.ones(n) if w is None else w.float().reshape(n)
    bf = None if b is None else b.float().reshape(n)
    ref = layer_norm_oracle(flat, wf, bf, eps).reshape(x.shape)
    assert out.shape == x.shape and out.dtype == torch.half
    close(out, ref, scale="magnitude", what=f"functional layer norm, {form}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("case", [(32, 512, 768, 3), (1, 16, 768, 3), (3, 77, 264, 2), (2, 5, 2048, 1), (5, 130, 1024, 3)],
                         ids=lambda c: "x".join(map(str, c)))
def test_embedding_lookups_summed_and_normalised(case, dtype, close):
    """`embedding_layer_norm`: word + token-type + position rows and their LayerNorm in one launch, against the oracle
    (gathers, additions rounded to the tables' dtype, fp32 LayerNorm).  32 x 512 x 768 is BERT-base's embedding stage at
    BASELINE config 3; the others put ragged widths, one and two tables, broadcast position ids (stride 0) and a
    token-type view with stride 0 in both dimensions behind the same kernel."""
    from kernl_amd.implementations.layer_norm import embedding_layer_norm

    batch, seq, n, n_tables = case
    gen = torch.Generator().manual_seed(9)
    rows = (1000, 2, 600)[:n_tables]
    tables = [(torch.randn((r, n), generator=gen) * (0.5, 0.1, 0.2)[k]).to(dtype) for k, r in enumerate(rows)]
    ids = [torch.randint(0, 1000, (batch, seq), generator=gen)]
    if n_tables > 1:
        ids.append(torch.zeros((1, 1), dtype=torch.int64).expand(batch, seq) if batch == 1 else torch.randint(0, 2, (batch, seq), generator=gen))
    if n_tables > 2:
        ids.append(torch.arange(seq)[None, :])                      # shared by all sequences
    w = (1.0 + 0.2 * torch.randn((n,), generator=gen)).to(dtype)
    b = (0.1 * torch.randn((n,), generator=gen)).to(dtype) if n != 264 else None
    out = embedding_layer_norm([t.cuda() for t in tables], [i.cuda() for i in ids], w.cuda(), None if b is None else b.cuda(), 1e-12)
    torch.cuda.synchronize()
    assert out.shape == (batch, seq, n) and out.dtype == dtype
    ref = embedding_layer_norm_oracle(tables, ids, w, b, effective_eps(1e-12, dtype))
    close(out, ref, dtype, scale="magnitude", what=f"embedding + layernorm {case}")


def test_embedding_ids_outside_the_table_are_clamped():
    from kernl_amd.implementations.layer_norm import embedding_layer_norm

    gen = torch.Generator().manual_seed(1)
    table = torch.randn((10, 64), generator=gen).half().cuda()
    w = torch.ones(64).half().cuda()
    ids = torch.tensor([[0, 9, 10, 12345, -1, -99]]).cuda()
    out = embedding_layer_norm([table], [ids], w, None, 1e-5)
    want = embedding_layer_norm([table], [ids.clamp(0, 9)], w, None, 1e-5)
    assert torch.equal(out, want)
