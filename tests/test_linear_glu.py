"""GPU parity of the gated linear unit (SwiGLU / GeGLU feed-forward entry) against the CPU oracle.

The reference tests its fused feed-forward against the eager `silu(w1(x)) * w3(x)` at M = 1..128, 4096 -> 11008
(experimental/llama-v2/test/test_ff.py); the cases here cover that shape class, every tile shape of the gated path,
ragged edges (M not a multiple of the tile, output width a multiple of 32 only), biases, bf16, strided inputs, the
fallback for widths the kernel does not take, and the Llama-7B prefill shape at full size.
"""
import pytest
import torch

from kernl_amd import _lib
from kernl_amd.implementations.linear_layer import interleave_glu_rows, linear_glu_layer
from kernl_amd.optimizer.linear import glu_linear_wrapper
from oracle import glu_oracle

pytestmark = pytest.mark.gpu


def _case(M, N, K, dtype, bias, seed=0):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn((M, K), generator=gen).to(dtype)
    wg = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
    wv = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
    bg = bv = None
    if bias:
        bg, bv = (0.5 * torch.randn((N,), generator=gen)).to(dtype), (0.5 * torch.randn((N,), generator=gen)).to(dtype)
    return x, wg, bg, wv, bv


def _run(x, wg, bg, wv, bv, activation):
    w = interleave_glu_rows(wg, wv).cuda()
    b = None if bg is None else interleave_glu_rows(bg, bv).cuda()
    out = linear_glu_layer(x.cuda(), w, b, activation)
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("bias", [False, True], ids=["nobias", "bias"])
@pytest.mark.parametrize("activation", ["silu", "fast_gelu", "gelu", "relu", "tanh", ""])
@pytest.mark.parametrize("shape", [(1, 32, 64), (16, 11008, 4096), (128, 256, 512), (300, 96, 200), (257, 160, 72)],
                         ids=lambda s: "x".join(map(str, s)))
def test_glu_vs_oracle(shape, activation, bias, dtype, close):
    M, N, K = shape
    if K == 4096 and (bias or dtype == torch.bfloat16 or activation not in ("silu", "fast_gelu")):
        pytest.skip("large case runs once per activation family")
    x, wg, bg, wv, bv = _case(M, N, K, dtype, bias)
    print(f"case {shape} {activation!r} bias={bias} {dtype}", flush=True)
    out = _run(x, wg, bg, wv, bv, activation)
    assert out.shape == (M, N) and out.dtype == dtype
    close(out, glu_oracle(x, wg, bg, wv, bv, activation), dtype, scale="magnitude", what=f"glu {shape} {activation}")


@pytest.mark.parametrize("tile", [1, 3, 5])
@pytest.mark.parametrize("shape", [(700, 544, 1024), (256, 256, 64), (513, 1056, 320)], ids=lambda s: "x".join(map(str, s)))
def test_glu_every_tile_shape(shape, tile, close):
    M, N, K = shape
    x, wg, bg, wv, bv = _case(M, N, K, torch.float16, True, seed=tile)
    lib = _lib.load()
    lib.kernl_linear_force_tile(tile)
    try:
        out = _run(x, wg, bg, wv, bv, "silu")
    finally:
        lib.kernl_linear_force_tile(0)
    close(out, glu_oracle(x, wg, bg, wv, bv, "silu"), scale="magnitude", what=f"glu tile {tile} {shape}")


def test_glu_3d_and_strided_input(close):
    x, wg, _, wv, _ = _case(2 * 50, 64, 128, torch.float16, False, seed=5)
    wide = torch.zeros((100, 256), dtype=torch.float16)
    wide[:, :128] = x
    w = interleave_glu_rows(wg, wv).cuda()
    out = linear_glu_layer(wide.cuda()[:, :128].view(2, 50, 128), w, None, "silu")  # row stride 256, 3-D
    torch.cuda.synchronize()
    assert out.shape == (2, 50, 64)
    close(out.view(100, 64), glu_oracle(x, wg, None, wv, None, "silu"), scale="magnitude", what="glu strided")
    xt = torch.randn((128, 40), generator=torch.Generator().manual_seed(6)).half()
    out = linear_glu_layer(xt.cuda().t(), w, None, "silu")  # feature stride 40: copied to a dense layout first
    torch.cuda.synchronize()
    close(out, glu_oracle(xt.t(), wg, None, wv, None, "silu"), scale="magnitude", what="glu transposed")


def test_glu_wrapper_caches_and_falls_back(close):
    x, wg, bg, wv, bv = _case(64, 96, 64, torch.float16, True, seed=7)
    xg, params = x.cuda(), [t.cuda() for t in (wg, bg, wv, bv)]
    out1 = glu_linear_wrapper(xg, *params, "silu")
    out2 = glu_linear_wrapper(xg, *params, "silu")
    torch.cuda.synchronize()
    assert torch.equal(out1, out2)
    close(out1, glu_oracle(x, wg, bg, wv, bv, "silu"), scale="magnitude", what="glu wrapper")
    # an output width that is no multiple of 32 runs as two linears and a product, with the same result
    x, wg, bg, wv, bv = _case(64, 40, 64, torch.float16, True, seed=8)
    out = glu_linear_wrapper(x.cuda(), wg.cuda(), bg.cuda(), wv.cuda(), bv.cuda(), "silu")
    torch.cuda.synchronize()
    close(out, glu_oracle(x, wg, bg, wv, bv, "silu"), scale="magnitude", what="glu fallback width")
    # fp32 parameters with fp16 activations are cast once, as for the plain linear wrapper
    x, wg, _, wv, _ = _case(32, 64, 64, torch.float32, False, seed=9)
    wg_g, wv_g = wg.cuda(), wv.cuda()
    out = glu_linear_wrapper(x.half().cuda(), wg_g, None, wv_g, None, "silu")
    torch.cuda.synchronize()
    assert wg_g.dtype == torch.float16 and out.dtype == torch.float16
    close(out, glu_oracle(x.half(), wg.half(), None, wv.half(), None, "silu"), scale="magnitude", what="glu cast")


def test_glu_llama_7b_prefill_shape(close):
    """[2048, 4096] -> 11008 at full size: oracle on a sample of rows (the CPU product of the whole case takes
    minutes), plus two size-independent properties on all rows: a zero gate weight gives exactly zero, and scaling the
    value weight by 2 doubles the output exactly (a power of two commutes with every rounding of a normal number)."""
    M, N, K = 2048, 11008, 4096
    x, wg, _, wv, _ = _case(M, N, K, torch.float16, False, seed=10)
    out = _run(x, wg, None, wv, None, "silu")
    rows = torch.arange(0, M, 41)
    close(out[rows.cuda()], glu_oracle(x[rows], wg, None, wv, None, "silu"), scale="magnitude", what="glu 7b sample")
    doubled = _run(x, wg, None, wv * 2, None, "silu")
    normal = out.abs() >= 2.0 ** -13  # below that fp16 is subnormal and rounding no longer commutes with doubling
    assert torch.equal(doubled[normal], (out * 2)[normal])
    assert (doubled.float() - 2 * out.float()).abs().max().item() <= 2.0 ** -23
    zero = _run(x, torch.zeros_like(wg), None, wv, None, "silu")
    assert not zero.any()


def test_glu_argument_errors():
    x = torch.zeros((8, 64), dtype=torch.float16, device="cuda")
    w = torch.zeros((64, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(AssertionError):
        linear_glu_layer(x, w[:48], None, "silu")  # interleaved rows must come in blocks of 64
    with pytest.raises(AssertionError):
        linear_glu_layer(x.float(), w.float(), None, "silu")
    with pytest.raises(AssertionError):
        linear_glu_layer(x[:, :32], w, None, "silu")
    out = torch.empty((8, 48), dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        _lib.linear_glu_fwd(x, w[:48].repeat(2, 1), None, out, _lib.ACT_SILU)  # N = 48


def test_glu_more_tiles_than_compute_units(close):
    M, N, K = 4352, 2208, 128  # 17 x 18 tiles of the interleaved weight: workgroups walk two tiles each
    x, wg, bg, wv, bv = _case(M, N, K, torch.float16, True, seed=12)
    lib = _lib.load()
    lib.kernl_linear_force_tile(5)
    try:
        out = _run(x, wg, bg, wv, bv, "silu")
    finally:
        lib.kernl_linear_force_tile(0)
    close(out, glu_oracle(x, wg, bg, wv, bv, "silu"), scale="magnitude", what="glu persistent")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("bias", [False, True], ids=["nobias", "bias"])
@pytest.mark.parametrize("shape", [(1, 11008, 4096), (7, 96, 64), (16, 160, 320), (40, 1024, 192), (64, 352, 4096),
                                   (33, 8224, 256), (64, 8192, 64), (16, 11008, 128), (32, 8992, 192), (24, 13824, 64),
                                   (9, 12320, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_glu_few_rows_streams_the_weight(shape, bias, dtype, close):
    """M <= 64 (reference experimental/llama-v2/test/test_ff.py runs M = 1..128): every workgroup takes 16 gate rows
    and their 16 value rows of the interleaved weight (48 or 64 of each where 8..32 rows of x meet more than 8192
    output columns), the waves split K."""
    M, N, K = shape
    x, wg, bg, wv, bv = _case(M, N, K, dtype, bias, seed=5)
    out = _run(x, wg, bg, wv, bv, "silu")
    close(out, glu_oracle(x, wg, bg, wv, bv, "silu"), dtype, what=f"gated, few rows {shape}")
