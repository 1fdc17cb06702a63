"""GPU parity of the fused linear layer against the CPU oracle.

Cases follow the reference's test/test_linear_layer.py:48-99 (shapes (bs, M, 768, 768), bias on/off, activations
"", tanh, gelu, relu, contiguous and `.mT` inputs, fp16 and fp32) plus BASELINE config 2 at full size.
"""
import pytest
import torch

from kernl_amd import _lib
from kernl_amd.implementations.linear_layer import linear_layer
from oracle import linear_oracle

pytestmark = pytest.mark.gpu


def _inputs(M, N, K, dtype, gen, w_std=1.0, bias=True, batch=None):
    xs = (M, K) if batch is None else (batch, M, K)
    x = torch.randn(xs, generator=gen).to(dtype)
    w = (torch.randn((N, K), generator=gen) * w_std).to(dtype)
    b = (torch.randn((N,), generator=gen) * w_std).to(dtype) if bias else None
    return x, w, b


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=["fp16", "bf16", "fp32"])
@pytest.mark.parametrize("activation", ["", "tanh", "gelu", "fast_gelu", "relu", "silu"])
@pytest.mark.parametrize("bias", [True, False], ids=["bias", "nobias"])
@pytest.mark.parametrize("shape", [(1, 8, 8, 8), (1, 8, 768, 768), (16, 16, 768, 768), (1, 128, 768, 768),
                                   (16, 512, 768, 768), (1, 300, 520, 264)], ids=lambda s: "x".join(map(str, s)))
def test_linear_vs_oracle(shape, bias, activation, dtype, close):
    bs, M, N, K = shape
    gen = torch.Generator().manual_seed(0)
    # weights ~ N(0, 1/K) keep outputs at unit scale so the absolute tolerance is meaningful
    x, w, b = _inputs(M, N, K, dtype, gen, w_std=K ** -0.5, bias=bias, batch=bs)
    print(f"case shape={shape} bias={bias} act={activation!r} dtype={dtype}", flush=True)
    out = linear_layer(x.cuda(), w.cuda(), None if b is None else b.cuda(), activation=activation)
    torch.cuda.synchronize()
    assert out.shape == (bs, M, N) and out.dtype == dtype
    ref = linear_oracle(x, w, b, activation)
    close(out, ref, dtype, what=f"linear {shape} {activation!r}")


TILE_IDS = ["256x256", "256x192", "128x128", "256x128k32", "wide256x256", "wide256x192", "wide128x256", "wide128x192"]
# tiles over the whole K: 32 x 64, 64 x 64 (shared by the waves), 16 / 32 / 64 x 32 (k-tiles dealt), 64 x 128 (shared)
SMALL_TILES = [10, 11, 12, 13, 14, 15]
SMALL_IDS = ["small32x64", "small64x64", "dealt16x32", "dealt32x32", "dealt64x32", "small64x128"]


@pytest.mark.parametrize("tile", list(range(1, 9)) + SMALL_TILES, ids=TILE_IDS + SMALL_IDS)
@pytest.mark.parametrize(
    "shape",
    [(1000, 600, 776), (256, 256, 64), (513, 385, 1032), (700, 520, 1024), (300, 260, 32), (257, 513, 96), (640, 512, 160),
     (513, 385, 128), (384, 640, 192), (130, 200, 320)],
    ids=lambda s: "x".join(map(str, s))
)
def test_linear_every_tile_shape(shape, tile, close):
    M, N, K = shape
    gen = torch.Generator().manual_seed(1)
    x, w, b = _inputs(M, N, K, torch.float16, gen, w_std=K ** -0.5)
    lib = _lib.load()
    lib.kernl_linear_force_tile(tile)
    try:
        out = linear_layer(x.cuda(), w.cuda(), b.cuda(), activation="gelu")
        torch.cuda.synchronize()
    finally:
        lib.kernl_linear_force_tile(0)
    close(out, linear_oracle(x, w, b, "gelu"), what=f"linear tile {tile} {shape}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("tile", [0, 5, 6, 7, 8] + SMALL_TILES, ids=["heuristic"] + TILE_IDS[4:] + SMALL_IDS)
@pytest.mark.parametrize("shape", [(300, 520, 8), (300, 520, 40), (513, 385, 72), (700, 520, 136), (1000, 600, 520),
                                   (2050, 1030, 776), (4352, 4300, 1992)], ids=lambda s: "x".join(map(str, s)))
def test_linear_ragged_last_k_tile(shape, tile, dtype, close):
    """K a multiple of 8 but not of 64 on the wide kernels: the last k-tile of every output tile is partly
    outside the rows.  One, two, an odd and an even number of k-tiles; more output tiles than compute units, so the
    stream of k-tiles crosses tile boundaries.  What follows a row in memory must not leak into it: the row after
    row 4 starts with infinities, and row 4 (like every other row) still has to match the oracle."""
    M, N, K = shape
    gen = torch.Generator().manual_seed(31)
    x, w, b = _inputs(M, N, K, dtype, gen, w_std=K ** -0.5)
    x[5, :8] = float("inf")
    lib = _lib.load()
    lib.kernl_linear_force_tile(tile)
    try:
        out = linear_layer(x.cuda(), w.cuda(), b.cuda(), activation="tanh")
        torch.cuda.synchronize()
    finally:
        lib.kernl_linear_force_tile(0)
    keep = torch.arange(M) != 5
    assert torch.isfinite(out[keep.cuda()].float()).all(), "a neighbouring row leaked into the ragged k-tile"
    x[5, :8] = 0.0
    ref = linear_oracle(x, w, b, "tanh")
    close(out[keep.cuda()], ref[keep], dtype, what=f"ragged K {shape} tile {tile}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("activation", ["", "fast_gelu"])
@pytest.mark.parametrize("shape", [(65, 768, 768), (128, 2304, 768), (128, 3072, 768), (200, 1000, 448), (500, 520, 64),
                                   (512, 1024, 1024), (1024, 700, 1480), (1000, 960, 520), (130, 70, 8),
                                   (8, 768, 3072), (16, 2304, 768), (16, 8192, 1024), (33, 768, 3080), (128, 768, 3072),
                                   (256, 1024, 4096), (100, 2048, 2048), (20, 1000, 8192), (40, 96, 72), (512, 768, 3072), (300, 1000, 2056), (96, 5440, 768),
                                   (512, 3072, 768), (500, 2300, 776), (1024, 768, 1536), (700, 1000, 2056)],
                         ids=lambda s: "x".join(map(str, s)))
def test_linear_small_problem_kernels_are_what_small_problems_run(shape, activation, dtype, close):
    """A few hundred rows at most against a weight of a few million elements: the library's own choice is one of the
    small-problem kernels (one launch, whole K per workgroup; `kernl_linear_small_kind` names it).  Forcing that kernel
    must give the same bits as the heuristic, every one of the six must match the oracle, and so must the operator,
    which must not hand such a shape to the stream-K or split-K entry points.  Tiles ragged in rows, columns and K, fewer
    k-tiles than ring stages or waves, strided output."""
    M, N, K = shape
    gen = torch.Generator().manual_seed(57)
    x, w, b = _inputs(M, N, K, dtype, gen, w_std=K ** -0.5)
    ref = linear_oracle(x, w, b, activation)
    lib = _lib.load()
    picked = _lib.linear_small_kind(M, N, K)
    assert picked in SMALL_TILES
    outs = {}
    for tile in [0] + SMALL_TILES:
        out = torch.empty((M, N), dtype=dtype, device="cuda")
        lib.kernl_linear_force_tile(tile)
        try:
            _lib.linear_fwd(x.cuda(), w.cuda(), b.cuda(), out, None, {"": _lib.ACT_NONE, "fast_gelu": _lib.ACT_GELU_TANH}[activation])
            torch.cuda.synchronize()
        finally:
            lib.kernl_linear_force_tile(0)
        outs[tile] = out
        close(out, ref, dtype, what=f"small problem {shape} {activation!r} tile {tile}")
    assert torch.equal(outs[0], outs[picked]), "the heuristic did not run the kernel kernl_linear_small_kind names"
    assert torch.equal(linear_layer(x.cuda(), w.cuda(), b.cuda(), activation=activation), outs[0])
    # a column slice of a wider buffer as the output's home: row stride != N
    wide = torch.zeros((M, N + 24), dtype=dtype, device="cuda")
    _lib.linear_fwd(x.cuda(), w.cuda(), b.cuda(), wide[:, 8:8 + N], None, _lib.ACT_NONE)
    torch.cuda.synchronize()
    close(wide[:, 8:8 + N], linear_oracle(x, w, b, ""), dtype, what=f"small problem {shape} strided output")
    assert (wide[:, :8] == 0).all() and (wide[:, 8 + N:] == 0).all()


@pytest.mark.parametrize("tile", SMALL_TILES, ids=SMALL_IDS)
def test_linear_small_problem_kernels_take_any_bias_alignment(tile, close):
    """The small-problem kernels fetch a lane's four bias values as one 8-byte load where they can: a bias that starts 2
    bytes into an allocation, and one whose last group of four crosses N, take the element-wise route."""
    gen = torch.Generator().manual_seed(61)
    M, N, K = 70, 330, 200
    x, w, _ = _inputs(M, N, K, torch.float16, gen, w_std=K ** -0.5)
    holder = torch.randn((N + 1,), generator=gen).half().cuda()
    lib = _lib.load()
    for b in (holder[1:], holder[:N].clone()):
        assert b.is_contiguous() and b.shape == (N,)
        out = torch.empty((M, N), dtype=torch.float16, device="cuda")
        lib.kernl_linear_force_tile(tile)
        try:
            _lib.linear_fwd(x.cuda(), w.cuda(), b, out, None, _lib.ACT_NONE)
            torch.cuda.synchronize()
        finally:
            lib.kernl_linear_force_tile(0)
        close(out, linear_oracle(x, w, b.cpu(), ""), what=f"tile {tile}, bias at offset {b.data_ptr() % 8}")


def test_linear_non_contiguous_input(close):
    # reference test/test_linear_layer.py:73-78: x.mT of a contiguous [K, M] matrix
    gen = torch.Generator().manual_seed(2)
    M, N, K = 256, 768, 768
    xt = torch.randn((4, K, M), generator=gen).half()
    w = (torch.randn((N, K), generator=gen) * K ** -0.5).half()
    b = torch.randn((N,), generator=gen).half()
    x = xt.mT
    assert not x.is_contiguous()
    out = linear_layer(x.cuda(), w.cuda(), b.cuda(), activation="tanh")
    torch.cuda.synchronize()
    close(out, linear_oracle(x, w, b, "tanh"), what="linear x.mT")
    # 2-D column-major input goes through the strided kernel without a copy
    x2 = xt[0].mT
    x2c = x2.cuda()
    assert x2c.stride() == x2.stride() and x2c.stride(1) != 1
    out2 = linear_layer(x2c, w.cuda(), b.cuda())
    torch.cuda.synchronize()
    close(out2, linear_oracle(x2, w, b, ""), what="linear 2-D column-major x")


def test_linear_saves_activation_inputs(close):
    gen = torch.Generator().manual_seed(3)
    M, N, K = 384, 512, 256
    x, w, b = _inputs(M, N, K, torch.float16, gen, w_std=K ** -0.5)
    act_in = torch.empty((M, N), dtype=torch.float16, device="cuda")
    out = linear_layer(x.cuda(), w.cuda(), b.cuda(), activation="gelu", act_inputs=act_in)
    torch.cuda.synchronize()
    ref, pre = linear_oracle(x, w, b, "gelu", return_act_inputs=True)
    close(out, ref, what="linear out")
    close(act_in, pre, what="linear act_inputs")


@pytest.mark.parametrize("tile", [5, 6, 7, 8] + SMALL_TILES, ids=TILE_IDS[4:] + SMALL_IDS)
def test_linear_wide_tiles_save_activation_inputs(tile, close):
    gen = torch.Generator().manual_seed(13)
    M, N, K = 300, 520, 448
    x, w, b = _inputs(M, N, K, torch.bfloat16, gen, w_std=K ** -0.5)
    act_in = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    lib = _lib.load()
    lib.kernl_linear_force_tile(tile)
    try:
        out = linear_layer(x.cuda(), w.cuda(), b.cuda(), activation="relu", act_inputs=act_in)
        torch.cuda.synchronize()
    finally:
        lib.kernl_linear_force_tile(0)
    ref, pre = linear_oracle(x, w, b, "relu", return_act_inputs=True)
    close(out, ref, torch.bfloat16, what=f"tile {tile} out")
    close(act_in, pre, torch.bfloat16, what=f"tile {tile} act_inputs")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("activation", ["", "gelu", "silu"])
@pytest.mark.parametrize("shape", [(1, 4096, 512), (5, 80, 64), (16, 1000, 192), (17, 768, 3072), (33, 2304, 768),
                                   (64, 4096, 1024), (3, 24, 4096), (5, 8200, 128), (33, 9000, 192), (64, 8192, 128),
                                   (9, 12300, 64), (20, 16400, 64), (64, 16400, 128), (40, 11008, 320)],
                         ids=lambda s: "x".join(map(str, s)))
def test_linear_few_rows_streams_the_weight(shape, activation, dtype, close):
    """At most 64 rows of x (decoding steps): the kernel that streams the weight once, 16 output columns per workgroup.
    Shapes cover one to four 16-row blocks of x, output widths that are not a multiple of 16, chunk counts that do
    not divide by the waves of a workgroup, outputs wide enough for 32, 48 and 64 columns per workgroup (with widths
    that leave the last workgroup partly empty), and the saved pre-activation."""
    M, N, K = shape
    gen = torch.Generator().manual_seed(17)
    x, w, b = _inputs(M, N, K, dtype, gen, w_std=K ** -0.5)
    act_in = torch.empty((M, N), dtype=dtype, device="cuda")
    lib = _lib.load()
    lib.kernl_linear_force_tile(9)
    try:
        out = linear_layer(x.cuda(), w.cuda(), b.cuda(), activation=activation, act_inputs=act_in)
        out_nobias = linear_layer(x.cuda(), w.cuda(), None, activation=activation)
        torch.cuda.synchronize()
    finally:
        lib.kernl_linear_force_tile(0)
    ref, pre = linear_oracle(x, w, b, activation, return_act_inputs=True)
    close(out, ref, dtype, what=f"few rows {shape} {activation!r}")
    close(act_in, pre, dtype, what=f"few rows {shape} pre-activation")
    close(out_nobias, linear_oracle(x, w, None, activation), dtype, what=f"few rows {shape} no bias")


@pytest.mark.parametrize("activation", ["", "silu"])
@pytest.mark.parametrize("shape", [(1, 4096, 4096), (5, 80, 64), (16, 1000, 192), (33, 9000, 192), (64, 512, 1024),
                                   (100, 256, 128), (4, 96, 72), (65, 200, 136), (300, 1000, 328), (2048, 2304, 768),
                                   (1024, 4096, 1024), (7, 64, 100), (520, 4096, 1024), (2050, 1100, 512), (300, 700, 192)],
                         ids=lambda s: "x".join(map(str, s)))
def test_linear_fp8_weight_storage(shape, activation, close):
    """Weight stored as fp8 e5m2 (reference: `get_model_fp8`, experimental/llama-v2/kernel/fused_kernel_fp8.py:75-84):
    the result must be the oracle's on the DECODED weight.  Up to 64 rows with K % 64 == 0 stream the bytes; more rows,
    with K % 64 == 0, take the wide kernels (bytes staged into LDS by the loads themselves, widened at the fragment
    reads: 256-row and 128-row tiles, ragged edges in both dimensions); another K that is a multiple of 8 takes the
    8-wave kernel that widens the bytes on their way into LDS; K = 100 goes through a widened copy."""
    from oracle import e5m2_decode_oracle

    M, N, K = shape
    gen = torch.Generator().manual_seed(29)
    x, w, b = _inputs(M, N, K, torch.float16, gen, w_std=K ** -0.5)
    w8 = w.to(torch.float8_e5m2).view(torch.int8)
    w_dec = e5m2_decode_oracle(w8)
    act_in = torch.empty((M, N), dtype=torch.float16, device="cuda")
    out = linear_layer(x.cuda(), w8.cuda(), b.cuda(), activation=activation, act_inputs=act_in)
    torch.cuda.synchronize()
    ref, pre = linear_oracle(x, w_dec, b, activation, return_act_inputs=True)
    close(out, ref, what=f"fp8 weight {shape} {activation!r}")
    close(act_in, pre, what=f"fp8 weight {shape} pre-activation")


@pytest.mark.parametrize("shape", [(20, 1000, 320), (33, 2304, 2048), (128, 4096, 1024), (64, 26300, 256)],
                         ids=lambda s: "x".join(map(str, s)))
def test_linear_fp8_weight_stream_k(shape, close, monkeypatch):
    """fp8 e5m2 weights on the stream-K few-row kernel (a lane's 16 weight bytes of a unit are one load, widened by byte
    permutes): plain with bias + activation and the gated form with the RMSNorm prologue, against the oracle on the
    decoded weight; 17 to 128 rows against a large weight reach it through `linear_layer`."""
    from kernl_amd.implementations.linear_layer import interleave_glu_rows
    from oracle import e5m2_decode_oracle, glu_oracle, rms_norm_oracle

    M, N, K = shape
    gen = torch.Generator().manual_seed(73)
    x, w, b = _inputs(M, N, K, torch.float16, gen, w_std=K ** -0.5)
    w8 = w.to(torch.float8_e5m2).view(torch.int8)
    out = torch.empty((M, N), dtype=torch.float16, device="cuda")
    _lib.linear_fewrow_fwd(x.cuda(), w8.cuda(), b.cuda(), None, out, _lib.ACT_GELU_TANH)
    torch.cuda.synchronize()
    close(out, linear_oracle(x, e5m2_decode_oracle(w8), b, "fast_gelu"), what=f"stream-K fp8 weight {shape}")
    calls = []
    real = _lib.linear_fewrow_fwd
    monkeypatch.setattr(_lib, "linear_fewrow_fwd", lambda *a, **k: (calls.append(a[1].dtype), real(*a, **k))[1])
    routed = linear_layer(x.cuda(), w8.cuda(), b.cuda(), "fast_gelu")
    assert calls == ([torch.int8] if N * K >= (1 << 22) else [])
    close(routed, linear_oracle(x, e5m2_decode_oracle(w8), b, "fast_gelu"), what=f"fp8 weight {shape} through linear_layer")
    if N % 32 == 0:
        wv = (torch.randn((N, K), generator=gen) * K ** -0.5).half()
        g = (1.0 + 0.2 * torch.randn((K,), generator=gen)).half()
        wi8 = interleave_glu_rows(w, wv).to(torch.float8_e5m2).view(torch.int8)
        dec = e5m2_decode_oracle(wi8).reshape(N // 32, 2, 32, K)
        out = torch.empty((M, N), dtype=torch.float16, device="cuda")
        real(x.cuda(), wi8.cuda(), None, None, out, _lib.ACT_SILU, rms_weight=g.cuda(), eps=1.6e-5, gated=True)
        torch.cuda.synchronize()
        ref = glu_oracle(rms_norm_oracle(x, g, 1.6e-5), dec[:, 0].reshape(N, K), None, dec[:, 1].reshape(N, K), None, "silu")
        close(out, ref, scale="magnitude", what=f"stream-K fp8 gated + norm {shape}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("kind", ["plain", "plain_bias", "gated", "gated_bias"])
@pytest.mark.parametrize("shape", [(2048, 12288, 4096), (2048, 11008, 4096), (300, 768, 512), (1000, 1056, 776), (129, 256, 264),
                                   (4100, 192, 64)], ids=lambda s: "x".join(map(str, s)))
def test_rms_norm_folded_into_the_weight_for_prompts(shape, kind, dtype, close):
    """Prompts: rms_norm(x) @ w^T as rstd * (x @ (w * g)^T) with the row factor applied in the wide kernels' epilogue
    (`kernl_linear_scaled_fwd`) and the statistics from `kernl_add_rms_stats_fwd` — against the composition of the RMSNorm
    and linear / gated oracles on the UNFOLDED weights.  2048 x 4096 -> 12288 and -> 2 x 11008 are a Llama-7B prompt's
    query/key/value and feed-forward entry projections (oracle on a sample of rows there); the others put ragged rows,
    ragged columns, a ragged last k-tile and every tile shape of the wide kernels behind the same epilogue."""
    from kernl_amd.implementations.linear_layer import interleave_glu_rows, rms_linear_layer, rms_stats
    from oracle import glu_oracle, rms_norm_oracle

    M, N, K = shape
    gated, with_bias = kind.startswith("gated"), kind.endswith("bias")
    if gated and N % 32 != 0:
        pytest.skip("gated outputs come in blocks of 32")
    gen = torch.Generator().manual_seed(43)
    x = (torch.randn((M, K), generator=gen) * 3.0 + 0.5).to(dtype)       # rows far from unit RMS
    x[::7] *= 0.05                                                       # and far from each other
    g = (1.0 + 0.2 * torch.randn((K,), generator=gen)).to(dtype)
    eps = 1e-5 if dtype == torch.bfloat16 else 1.6e-5
    rows = torch.arange(0, M, 37 if M >= 2048 else 1)
    normed = rms_norm_oracle(x[rows], g, eps)

    def fold(w):
        return (w.float() * g.float()[None, :]).to(dtype)

    rstd = rms_stats(x.cuda(), eps, clamp=False)
    torch.testing.assert_close(rstd.cpu(), torch.rsqrt(x.float().pow(2).mean(-1) + eps), rtol=2e-6, atol=0)
    if gated:
        wg = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
        wv = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
        bg, bv = ((0.5 * torch.randn((N,), generator=gen)).to(dtype) for _ in range(2)) if with_bias else (None, None)
        bias = interleave_glu_rows(bg, bv).cuda() if with_bias else None
        out = rms_linear_layer(x.cuda(), g.cuda(), eps, interleave_glu_rows(wg, wv).cuda(), bias, "silu", gated=True,
                               folded_weight=interleave_glu_rows(fold(wg), fold(wv)).cuda(), rstd=rstd)
        ref = glu_oracle(normed, wg, bg, wv, bv, "silu")
    else:
        w = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
        b = (0.5 * torch.randn((N,), generator=gen)).to(dtype) if with_bias else None
        out = rms_linear_layer(x.cuda(), g.cuda(), eps, w.cuda(), None if b is None else b.cuda(), "",
                               folded_weight=fold(w).cuda(), rstd=None if M == 300 else rstd)   # one case computes them itself
        ref = linear_oracle(normed, w, b, "")
    torch.cuda.synchronize()
    assert out.shape == (M, N) and out.dtype == dtype
    close(out[rows.cuda()], ref, dtype, scale="magnitude", what=f"folded rms + linear {shape} {kind}")


def test_prompt_route_of_the_rms_projections_calls_the_scaled_kernel(monkeypatch):
    """Which shapes take the folded route: more rows than the few-row kernels take, where the plain product would run the
    wide tile kernels; fewer rows, or a missing folded weight, keep the kernels they had."""
    from kernl_amd.implementations import linear_layer as ll

    calls = []
    real = _lib.linear_scaled_fwd
    monkeypatch.setattr(_lib, "linear_scaled_fwd", lambda *a, **k: (calls.append(a[0].shape[0]), real(*a, **k))[1])
    gen = torch.Generator().manual_seed(3)
    w = (torch.randn((4096, 2048), generator=gen) * 0.02).half().cuda()
    g = torch.ones(2048).half().cuda()
    # (256 rows: too few tiles for the chip, the plain product splits K instead)
    for rows, expect in ((2048, True), (4096, True), (256, False), (100, False), (16, False)):
        x = torch.randn((rows, 2048), generator=gen).half().cuda()
        n = len(calls)
        a = ll.rms_linear_layer(x, g, 1e-5, w, None, "", folded_weight=w)
        b = ll.rms_linear_layer(x, g, 1e-5, w, None, "")
        assert (len(calls) > n) == expect, (rows, calls)
        assert len(calls) <= n + 1            # never without the folded weight
        torch.testing.assert_close(a.float(), b.float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("tile", [0, 5, 6, 7, 8], ids=["heuristic", "wide256x256", "wide256x192", "wide128x256", "wide128x192"])
@pytest.mark.parametrize("shape", [(16384, 768, 768), (2048, 4096, 4096), (1000, 1056, 776), (513, 390, 264), (300, 768, 3072),
                                   (129, 200, 72)], ids=lambda s: "x".join(map(str, s)))
def test_linear_with_the_residual_added_in_the_epilogue(shape, tile, dtype, close):
    """`kernl_linear_residual_fwd`: round(x @ w^T + bias) + residual from the wide kernels' epilogue — bit for bit the
    linear kernel followed by an addition of the two 16-bit tensors, and the oracle's product plus the residual within
    tolerance.  16384 x 768 -> 768 is BERT-base's attention-output projection at batch 32 x 512 and 2048 x 4096 -> 4096 a
    Llama-7B prompt's; the others put ragged rows, ragged columns (scalar residual reads), a ragged last k-tile and a
    residual with padded rows behind every tile shape."""
    M, N, K = shape
    if tile == 0 and M * N * K > 2 ** 33:
        pytest.skip("the large shapes run once per forced tile")
    gen = torch.Generator().manual_seed(11)
    x, w, b = _inputs(M, N, K, dtype, gen, w_std=K ** -0.5, bias=(N % 2 == 0))
    res_full = (torch.randn((M, N + 24), generator=gen) * 2.0).to(dtype).cuda()
    res = res_full[:, 8:8 + N] if M < 1000 else res_full[:, :N].contiguous()    # (padded rows; 16-byte aligned only if N % 8 == 0)
    xd, wd, bd = x.cuda(), w.cuda(), None if b is None else b.cuda()
    out = torch.full((M, N), float("nan"), dtype=dtype, device="cuda")
    lib = _lib.load()
    lib.kernl_linear_force_tile(tile)
    try:
        _lib.linear_residual_fwd(xd, wd, bd, res, out)
        plain = torch.empty_like(out)
        _lib.linear_fwd(xd, wd, bd, plain, None, _lib.ACT_NONE)
        torch.cuda.synchronize()
    finally:
        lib.kernl_linear_force_tile(0)
    # (left to the heuristic the plain product may run another kernel, whose sums differ in the last bit)
    if tile != 0 or _lib.linear_wide_kind(M, N, K) != 0:
        assert torch.equal(out, plain + res), f"linear + residual {shape} tile {tile}: differs from product, then addition"
    rows = torch.arange(0, M, 29 if M >= 2048 else 1)
    ref = linear_oracle(x[rows], w, b, "") + res.cpu()[rows].float()
    close(out[rows.cuda()], ref, dtype, scale="magnitude", what=f"linear + residual {shape} tile {tile}")


def test_which_shapes_add_the_residual_in_the_epilogue():
    """`residual_linear_supported`: 16-bit problems that the plain product runs on the wide tile kernels — encoder batches
    and prompts — and nothing else (few rows, small problems, split K, fp32, mismatched residuals)."""
    from kernl_amd.implementations.linear_layer import residual_linear_layer, residual_linear_supported

    def case(rows, n, k, dtype=torch.float16, res_shape=None, res_dtype=None):
        x = torch.zeros((rows, k), dtype=dtype, device="cuda")
        w = torch.zeros((n, k), dtype=dtype, device="cuda")
        r = torch.zeros(res_shape or (rows, n), dtype=res_dtype or dtype, device="cuda")
        return residual_linear_supported(x, w, None, r)

    assert case(16384, 768, 768) and case(16384, 768, 3072) and case(2048, 4096, 4096) and case(2048, 4096, 11008)
    assert case(8192, 768, 768, torch.bfloat16)
    assert not case(64, 4096, 4096) and not case(128, 768, 768)          # decoding steps: the few-row kernels
    assert not case(512, 768, 768) and not case(256, 768, 3072)          # small problems / split K
    assert not case(16384, 768, 768, torch.float32)
    assert not case(16384, 768, 768, res_dtype=torch.float32) and not case(16384, 768, 768, res_shape=(16384, 1))
    gen = torch.Generator().manual_seed(2)
    x = torch.randn((8, 1024, 768), generator=gen).half().cuda()
    w = (torch.randn((768, 768), generator=gen) * 0.03).half().cuda()
    r = torch.randn((8, 1024, 768), generator=gen).half().cuda()
    out = residual_linear_layer(x, w, None, r)
    assert out.shape == r.shape and torch.equal(out, linear_layer(x, w, None) + r)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape", [(8, 1024, 768, 768), (4, 2048, 768, 3072), (2, 128, 768, 768), (1, 16, 264, 520)],
                         ids=lambda s: "x".join(map(str, s)))
def test_projection_with_the_addition_and_layer_norm_behind_it(shape, dtype, close, monkeypatch):
    """`linear_add_layer_norm_wrapper` = layer_norm(residual + linear(v)), an encoder layer's attention-output and
    feed-forward-down projections: against the composition of the oracles, whichever kernel the addition ends up in (the
    projection's epilogue for the first two shapes, the add + LayerNorm kernel for the others), and the two routes agree."""
    from kernl_amd.optimizer import linear as ol
    from oracle import effective_eps, layer_norm_oracle

    bs, M, N, K = shape
    gen = torch.Generator().manual_seed(17)
    v = torch.randn((bs, M, K), generator=gen).to(dtype)
    w = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
    b = (0.3 * torch.randn((N,), generator=gen)).to(dtype)
    res = (2.0 * torch.randn((bs, M, N), generator=gen)).to(dtype)
    g = (1.0 + 0.2 * torch.randn((N,), generator=gen)).to(dtype)
    be = (0.1 * torch.randn((N,), generator=gen)).to(dtype)
    calls = []
    real = _lib.linear_residual_fwd
    monkeypatch.setattr(_lib, "linear_residual_fwd", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    args = (v.cuda(), w.cuda(), b.cuda(), res.cuda(), (N,), g.cuda(), be.cuda(), 1e-12)
    out = ol.linear_add_layer_norm_wrapper(*args)
    assert len(calls) == (1 if bs * M >= 8192 else 0)
    monkeypatch.setattr(ol, "WIDE_RESIDUAL_EPILOGUE", False)
    other = ol.linear_add_layer_norm_wrapper(*args)
    torch.cuda.synchronize()
    assert len(calls) <= 1 and out.shape == res.shape and out.dtype == dtype
    summed = res.float() + linear_oracle(v, w, b, "").to(dtype).float()   # the projection is rounded before the addition
    ref = layer_norm_oracle(summed, g, be, effective_eps(1e-12, dtype))
    close(out, ref, dtype, scale="magnitude", what=f"projection + add + layernorm {shape}")
    close(other, ref, dtype, scale="magnitude", what=f"projection, then add + layernorm {shape}")


def test_residual_addition_with_row_statistics(close):
    """`add_rms_stats`: the sum is the fp16 / bf16 rounding of the fp32 sum (what `a + b` gives), the statistics are those
    of the ROUNDED sum; ragged row counts, 3-D inputs, non-contiguous operands."""
    from kernl_amd.implementations.linear_layer import add_rms_stats

    gen = torch.Generator().manual_seed(5)
    for dtype in (torch.float16, torch.bfloat16):
        for shape in ((3, 701, 1024), (2050, 4096), (130, 8), (5, 33, 776)):
            a = (torch.randn(shape, generator=gen) * 4).to(dtype)
            b = (torch.randn(shape, generator=gen) * 0.3).to(dtype)
            total, rstd = add_rms_stats(a.cuda(), b.cuda(), 1e-5)
            want = (a.float() + b.float()).to(dtype)
            assert torch.equal(total.cpu(), want), (dtype, shape)
            torch.testing.assert_close(rstd.cpu(), torch.rsqrt(want.float().pow(2).mean(-1) + 1e-5).reshape(-1), rtol=3e-6, atol=0)
    a = torch.randn((400, 2048), generator=gen).half().cuda()[:, ::2]          # strided rows: copied before the launch
    b = torch.randn((400, 1024), generator=gen).half().cuda()
    total, rstd = add_rms_stats(a, b, 1e-5)
    assert torch.equal(total, a + b)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("kind", ["plain", "plain_bias_silu", "gated"])
@pytest.mark.parametrize("shape", [(1, 4096, 4096), (5, 96, 64), (16, 1024, 192), (33, 2304, 768), (64, 512, 1024),
                                   (100, 256, 128), (4, 96, 72)], ids=lambda s: "x".join(map(str, s)))
def test_rms_norm_fused_into_the_linear_layer(shape, kind, dtype, close):
    """out = act(rms_norm(x) @ wᵀ + b) in one launch for decoding steps (reference: `rms_matmul_rbe` without the rotary
    epilogue, experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:116-183; gated: `ff_llama`, fused_kernel_ff.py:10-79),
    against the composition of the RMSNorm and linear oracles.  100 rows and K = 72 take the two-kernel route."""
    from kernl_amd.implementations.linear_layer import interleave_glu_rows, rms_linear_layer
    from oracle import glu_oracle, rms_norm_oracle

    M, N, K = shape
    gen = torch.Generator().manual_seed(41)
    x = (torch.randn((M, K), generator=gen) * 3.0 + 0.5).to(dtype)       # rows far from unit RMS
    g = (1.0 + 0.2 * torch.randn((K,), generator=gen)).to(dtype)
    eps = 1e-5 if dtype == torch.bfloat16 else 1.6e-5
    normed = rms_norm_oracle(x, g, eps)
    if kind == "gated":
        wg = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
        wv = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
        out = rms_linear_layer(x.cuda(), g.cuda(), eps, interleave_glu_rows(wg, wv).cuda(), None, "silu", gated=True)
        ref = glu_oracle(normed, wg, None, wv, None, "silu")
    else:
        w = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
        b = (0.5 * torch.randn((N,), generator=gen)).to(dtype) if kind == "plain_bias_silu" else None
        act = "silu" if kind == "plain_bias_silu" else ""
        out = rms_linear_layer(x.cuda(), g.cuda(), eps, w.cuda(), None if b is None else b.cuda(), act)
        ref = linear_oracle(normed, w, b, act)
    torch.cuda.synchronize()
    assert out.shape == (M, N) and out.dtype == dtype
    close(out, ref, dtype, what=f"rms + linear {shape} {kind}")


def test_linear_few_rows_strided_output_and_batched_input(close):
    gen = torch.Generator().manual_seed(18)
    x, w, b = _inputs(2, 640, 256, torch.float16, gen, w_std=1 / 16, batch=3)  # [3, 2, 256] -> 6 rows
    out = linear_layer(x.cuda(), w.cuda(), b.cuda(), activation="tanh")
    torch.cuda.synchronize()
    close(out, linear_oracle(x, w, b, "tanh"), what="few rows, batched")
    assert out.shape == (3, 2, 640)


@pytest.mark.parametrize("which", ["up", "down"])
def test_linear_config2_full_size(which, close):
    # BASELINE config 2: up-projection [16384,768]x[3072,768]ᵀ + bias + tanh-GELU; down-projection back, no activation
    gen = torch.Generator().manual_seed(0)
    if which == "up":
        M, N, K, act = 16384, 3072, 768, "fast_gelu"
    else:
        M, N, K, act = 16384, 768, 3072, ""
    x = torch.randn((M, K), generator=gen).half()
    w = (torch.randn((N, K), generator=gen) * 0.02).half()
    b = (torch.randn((N,), generator=gen) * 0.02).half()
    out = linear_layer(x.cuda(), w.cuda(), b.cuda(), activation=act)
    torch.cuda.synchronize()
    ref = linear_oracle(x, w, b, act)
    close(out, ref, scale=max(1.0, ref.abs().max().item() / 4), what=f"config 2 {which}")
    # linearity in x (size independent): without bias and activation f(2x) = 2 f(x); scaling by 2 is exact in
    # fp32 and in fp16, except that a subnormal fp16 result gains one bit when doubled (spacing 2^-24)
    if act == "":
        nb = linear_layer(x.cuda(), w.cuda(), None)
        nb2 = linear_layer((x * 2).cuda(), w.cuda(), None)
        torch.cuda.synchronize()
        assert (nb2.float() - nb.float() * 2).abs().max().item() <= 2.0 ** -23


def test_linear_rejects_bad_arguments():
    x = torch.zeros((4, 8), dtype=torch.float16, device="cuda")
    w = torch.zeros((16, 8), dtype=torch.float16, device="cuda")
    with pytest.raises(AssertionError):
        linear_layer(x, w.float(), None)  # dtype mismatch
    with pytest.raises(AssertionError):
        linear_layer(x, torch.zeros((16, 9), dtype=torch.float16, device="cuda"), None)  # K mismatch
    with pytest.raises(AssertionError):
        linear_layer(x, w.t().contiguous().t(), None)  # weight must be contiguous
    with pytest.raises(AssertionError):
        linear_layer(x, w, torch.zeros((15,), dtype=torch.float16, device="cuda"))  # bias size


def test_unknown_activation_is_identity(close):
    gen = torch.Generator().manual_seed(4)
    x, w, b = _inputs(64, 64, 64, torch.float16, gen, w_std=0.125)
    out = linear_layer(x.cuda(), w.cuda(), b.cuda(), activation="swish-not-a-name")
    torch.cuda.synchronize()
    close(out, linear_oracle(x, w, b, ""), what="unknown activation")


@pytest.mark.parametrize("shape", [(4352, 4352, 128), (4352, 4300, 192), (4400, 4352, 64), (8200, 2304, 256)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("tile", [5, 6, 7, 8], ids=TILE_IDS[4:])
def test_linear_more_tiles_than_compute_units(shape, tile, close):
    """More than 256 output tiles of 256x256: workgroups of the persistent kernel walk several tiles each, with the
    operand stream running through the tile boundaries (even k-tile counts) or one tile per workgroup (odd counts)."""
    M, N, K = shape
    gen = torch.Generator().manual_seed(11)
    x, w, b = _inputs(M, N, K, torch.float16, gen, w_std=K ** -0.5)
    lib = _lib.load()
    lib.kernl_linear_force_tile(tile)
    try:
        out = linear_layer(x.cuda(), w.cuda(), b.cuda(), activation="relu")
        torch.cuda.synchronize()
    finally:
        lib.kernl_linear_force_tile(0)
    close(out, linear_oracle(x, w, b, "relu"), what=f"linear persistent {shape}")


@pytest.mark.parametrize("activation", ["gelu", "fast_gelu", "silu", "tanh"])
def test_activation_curve_through_identity_weights(activation):
    """The epilogue's activation sampled on a grid (identity weight, no bias): the fp16 kernels use short
    sigmoid-form approximations (erf-GELU: |error| <= 2.6e-5 by construction), which must hold over the whole range,
    saturate cleanly for large |x| and stay within an fp16 rounding of the fp32 closed form."""
    K = 64
    grid = torch.cat((torch.linspace(-12, 12, 64 * 255), torch.tensor([0.0, -0.0, 30.0, -30.0, 1000.0, -1000.0, 60000.0, -60000.0] * 8)))
    x = grid.reshape(-1, K).half()
    w = torch.eye(K).half()
    out = linear_layer(x.cuda(), w.cuda(), None, activation=activation)
    torch.cuda.synchronize()
    ref = linear_oracle(x, w, None, activation)
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    err = (got - ref).abs()
    bound = 4e-5 + 1.0e-3 * ref.abs()  # approximation error + one fp16 rounding (2^-11 relative, with slack)
    worst = (err - bound).max().item()
    assert worst <= 0, f"{activation}: error exceeds bound by {worst:.3e} at x={x.float().flatten()[(err - bound).argmax()].item()}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("table_dtype", ["same", "fp32"])
@pytest.mark.parametrize(
    "case",
    # batch, positions, K, heads (query + key + value), head size, rotated heads, bias, residual
    [(1, 1, 4096, 96, 128, 64, False, False), (4, 1, 512, 12, 64, 8, True, False), (2, 3, 256, 6, 128, 4, False, True),
     (33, 1, 320, 9, 32, 9, True, True), (1, 64, 128, 3, 64, 2, False, False), (5, 2, 192, 4, 96, 0, True, True)],
    ids=lambda c: "x".join(str(int(v)) for v in c),
)
def test_decode_projection_with_norm_rotation_and_residual(case, table_dtype, dtype, close):
    """A decoding step's query/key/value projection in one launch: RMSNorm prologue, the product, rotation of the query
    and key heads, residual (reference: `rms_matmul_rbe_qkv`, experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:250-347)
    against the composition of the RMSNorm, linear and rotary oracles."""
    from kernl_amd.implementations.linear_layer import decode_linear_layer
    from oracle import rms_norm_oracle, rotary_oracle

    B, S, K, heads, D, rot_heads, with_bias, with_residual = case
    N = heads * D
    gen = torch.Generator().manual_seed(43)
    x = (torch.randn((B, S, K), generator=gen) * 2.0 + 0.3).to(dtype)
    g = (1.0 + 0.2 * torch.randn((K,), generator=gen)).to(dtype)
    w = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
    b = (0.5 * torch.randn((N,), generator=gen)).to(dtype) if with_bias else None
    res = torch.randn((B, S, N), generator=gen).to(dtype) if with_residual else None
    tdt = dtype if table_dtype == "same" else torch.float32
    angles = torch.rand((B, S, D), generator=gen) * 6.28          # per batch entry AND position, both halves independent
    cos, sin = angles.cos().to(tdt), angles.sin().to(tdt)
    eps = 1e-5 if dtype == torch.bfloat16 else 1.6e-5
    out = decode_linear_layer(x.cuda(), w.cuda(), None if b is None else b.cuda(), g.cuda(), eps,
                              None if res is None else res.cuda(), cos.cuda(), sin.cuda(), head_dim=D, rope_cols=rot_heads * D)
    torch.cuda.synchronize()
    y = linear_oracle(rms_norm_oracle(x, g, eps), w, b, "")                        # [B, S, N] fp32
    heads_view = y.reshape(B, S, heads, D)
    rotated = rotary_oracle(heads_view[:, :, :rot_heads], cos[:, :, None, :], sin[:, :, None, :])
    ref = torch.cat((rotated, heads_view[:, :, rot_heads:]), dim=2).reshape(B, S, N)
    if res is not None:
        ref = ref + res.float()
    assert out.shape == (B, S, N) and out.dtype == dtype
    close(out, ref, dtype, scale="magnitude", what=f"decode projection {case}")
    # tables shared by the batch ([1, S, D]) are read with a zero batch stride
    out1 = decode_linear_layer(x.cuda(), w.cuda(), None if b is None else b.cuda(), g.cuda(), eps,
                               None if res is None else res.cuda(), cos[:1].cuda(), sin[:1].cuda(), head_dim=D, rope_cols=rot_heads * D)
    torch.cuda.synchronize()
    rotated1 = rotary_oracle(heads_view[:, :, :rot_heads], cos[:1, :, None, :], sin[:1, :, None, :])
    ref1 = torch.cat((rotated1, heads_view[:, :, rot_heads:]), dim=2).reshape(B, S, N)
    close(out1, ref1 if res is None else ref1 + res.float(), dtype, scale="magnitude", what=f"decode projection, shared tables {case}")


@pytest.mark.parametrize("with_norm", [False, True], ids=["plain", "rms"])
@pytest.mark.parametrize("shape", [(1, 4096, 11008), (7, 768, 3072), (40, 8192, 512), (64, 96, 64)], ids=lambda s: "x".join(map(str, s)))
def test_decode_projection_with_residual_only(shape, with_norm, close):
    """out = residual + linear(x) (the attention-output and feed-forward-down projections of a decoding step), with and
    without the RMSNorm prologue; every grid rule of the few-row kernel is in the list."""
    from kernl_amd.implementations.linear_layer import decode_linear_layer
    from oracle import rms_norm_oracle

    M, N, K = shape
    gen = torch.Generator().manual_seed(47)
    x, w, b = _inputs(M, N, K, torch.float16, gen, w_std=K ** -0.5)
    res = torch.randn((M, N), generator=gen).half()
    g = (1.0 + 0.2 * torch.randn((K,), generator=gen)).half() if with_norm else None
    out = decode_linear_layer(x.cuda(), w.cuda(), b.cuda(), None if g is None else g.cuda(), 1.6e-5, res.cuda())
    torch.cuda.synchronize()
    xin = rms_norm_oracle(x, g, 1.6e-5) if with_norm else x
    close(out, linear_oracle(xin, w, b, "") + res.float(), scale="magnitude", what=f"residual projection {shape}")


def test_decode_projection_rejections():
    from kernl_amd import _lib
    from kernl_amd.implementations.linear_layer import decode_linear_layer, decode_linear_supported

    x = torch.zeros((65, 128), dtype=torch.half, device="cuda")
    w = torch.zeros((128, 128), dtype=torch.half, device="cuda")
    assert not decode_linear_supported(x, w) and decode_linear_supported(x[:64], w) and not decode_linear_supported(x[:4, :96], w[:, :96])
    with pytest.raises(AssertionError):
        decode_linear_layer(x, w)
    g = torch.ones((128,), dtype=torch.half, device="cuda")
    t = torch.zeros((1, 4, 48), dtype=torch.half, device="cuda")
    with pytest.raises(AssertionError):   # head size 48 is no multiple of 32
        decode_linear_layer(x[:4], w, None, g, 1e-5, None, t, t, head_dim=48, rope_cols=96)
    out = torch.empty((4, 128), dtype=torch.half, device="cuda")
    t64 = torch.zeros((1, 4, 64), dtype=torch.half, device="cuda")
    with pytest.raises(_lib.KernlLibraryError, match="RMSNorm prologue"):
        _lib.linear_decode_fwd(x[:4], None, 0.0, w, None, None, out, t64, t64, 64, 64, 4)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("activation", ["", "fast_gelu"])
@pytest.mark.parametrize("shape", [(129, 768, 3072), (200, 1000, 2048), (256, 4096, 4096), (300, 4100, 2112), (640, 400, 2112)],
                         ids=lambda s: "x".join(map(str, s)))
def test_linear_split_over_k(shape, activation, dtype, close):
    """Row counts whose 128-row tiles are too few for the chip: `linear_layer` hands them to `kernl_linear_splitk_fwd`
    (ranges of K per tile, partial tiles added by a second launch).  Ragged last tiles in both directions, ranges of
    unequal length (33 k-tiles in 2), the saved pre-activation, and a workspace full of NaNs."""
    M, N, K = shape
    gen = torch.Generator().manual_seed(71)
    x, w, b = _inputs(M, N, K, dtype, gen, w_std=K ** -0.5)
    xd, wd, bd = x.cuda(), w.cuda(), b.cuda()
    need = _lib.linear_splitk_workspace_bytes(xd, wd)
    assert need > 0, "the shape list is meant for the split form"
    ws = torch.full((need // 4,), float("nan"), dtype=torch.float32, device="cuda")
    out = torch.empty((M, N), dtype=dtype, device="cuda")
    act_in = torch.empty((M, N), dtype=dtype, device="cuda")
    _lib.linear_splitk_fwd(xd, wd, bd, out, act_in, _lib.ACT_GELU_TANH if activation else _lib.ACT_NONE, ws)
    routed = linear_layer(xd, wd, None, activation)
    torch.cuda.synchronize()
    ref, pre = linear_oracle(x, w, b, activation, return_act_inputs=True)
    close(out, ref, dtype, what=f"split K {shape} {activation!r}")
    close(act_in, pre, dtype, what=f"split K {shape} pre-activation")
    close(routed, linear_oracle(x, w, None, activation), dtype, what=f"split K {shape} through linear_layer")


def test_linear_split_over_k_rule():
    """The library splits only where it pays: few tiles and a long K."""
    rows = lambda m, k: torch.empty((m, k), dtype=torch.float16, device="cuda")
    weight = lambda n, k: torch.empty((n, k), dtype=torch.float16, device="cuda")
    assert _lib.linear_splitk_workspace_bytes(rows(256, 4096), weight(4096, 4096)) > 0
    assert _lib.linear_splitk_workspace_bytes(rows(256, 768), weight(3072, 768)) == 0      # short K
    assert _lib.linear_splitk_workspace_bytes(rows(2048, 4096), weight(4096, 4096)) == 0   # tiles enough
    assert _lib.linear_splitk_workspace_bytes(rows(256, 4104), weight(4096, 4104)) == 0    # K % 64 != 0
    with pytest.raises(_lib.KernlLibraryError, match="nothing to split"):
        _lib.linear_splitk_fwd(rows(2048, 4096), weight(4096, 4096), None, rows(2048, 4096), None, _lib.ACT_NONE,
                               torch.empty(1024, dtype=torch.uint8, device="cuda"))
    with pytest.raises(_lib.KernlLibraryError, match="workspace"):
        _lib.linear_splitk_fwd(rows(256, 4096), weight(4096, 4096), None, rows(256, 4096), None, _lib.ACT_NONE,
                               torch.empty(1024, dtype=torch.uint8, device="cuda"))


FEW_ROW_SHAPES = [
    (33, 200, 256),      # two tiles, the second ragged; a run is exactly one tile: no partial sums
    (17, 1000, 320),     # five chunks per tile, runs of four: every run crosses into the next tile
    (64, 777, 704),      # width that is no multiple of 4 (element stores), eleven chunks per tile
    (20, 384, 1024),     # runs that divide a tile evenly
    (5, 1000, 320),      # one 16-row block of x
    (48, 5120, 5120),    # 247 workgroups with runs of 13 units against 80 chunks per tile
    (64, 4096, 11008),   # long K
    (33, 11008, 4096),   # 86 tiles
    (30, 26300, 256),    # 206 tiles: whole tiles per workgroup, the last one ragged
    (64, 40000, 256),    # more tiles than workgroups: runs of 5 units against 4 chunks per tile
    (18, 80000, 256),    # runs of 10 units: a workgroup finishes a tile, covers one whole and starts a third
    (128, 1000, 320),    # eight 16-row blocks of x
    (100, 5120, 1024),
    (70, 26300, 256),    # whole tiles per workgroup with 128 rows of x
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("shape", FEW_ROW_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_linear_few_rows_stream_k(shape, dtype, close):
    """`kernl_linear_fewrow_fwd` (units of one tile and one k chunk dealt in equal runs to the workgroups, partial tiles
    added by a second launch) against the oracle: plain, with bias + activation, and with bias + residual; the
    workspace is filled with NaNs first, so a partial tile that is read without having been written shows."""
    M, N, K = shape
    gen = torch.Generator().manual_seed(53)
    x, w, b = _inputs(M, N, K, dtype, gen, w_std=K ** -0.5)
    res = torch.randn((M, N), generator=gen).to(dtype)
    xd, wd, bd, rd = x.cuda(), w.cuda(), b.cuda(), res.cuda()
    assert _lib.linear_fewrow_supported(xd, wd)
    need = _lib.linear_fewrow_workspace_bytes(M, N, K)
    ws = torch.full((max(need, 16) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    outs = [torch.empty((M, N), dtype=dtype, device="cuda") for _ in range(3)]
    _lib.linear_fewrow_fwd(xd, wd, None, None, outs[0], _lib.ACT_NONE, ws)
    _lib.linear_fewrow_fwd(xd, wd, bd, None, outs[1], _lib.ACT_GELU_TANH, ws)
    _lib.linear_fewrow_fwd(xd, wd, bd, rd, outs[2], _lib.ACT_NONE)   # workspace allocated by the binding
    torch.cuda.synchronize()
    close(outs[0], linear_oracle(x, w, None, ""), dtype, what=f"stream-K {shape} plain")
    close(outs[1], linear_oracle(x, w, b, "fast_gelu"), dtype, what=f"stream-K {shape} bias + gelu")
    close(outs[2], linear_oracle(x, w, b, "") + res.float(), dtype, scale="magnitude", what=f"stream-K {shape} residual")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize(
    "case",
    # batch, positions, K, heads (query + key + value), head size, rotated heads, bias, residual
    [(5, 4, 320, 6, 128, 4, True, True), (33, 1, 256, 10, 64, 10, False, False), (2, 32, 704, 12, 32, 8, True, True),
     (40, 1, 4096, 96, 128, 64, False, False), (16, 1, 512, 4, 128, 2, False, True), (3, 7, 1024, 7, 64, 0, True, False),
     (64, 2, 512, 6, 128, 4, True, True), (97, 1, 256, 10, 64, 6, False, True)],
    ids=lambda c: "x".join(str(int(v)) for v in c),
)
def test_few_rows_stream_k_with_norm_rotation_and_residual(case, dtype, close):
    """The batched decoding step's query/key/value projection on the stream-K kernel: RMSNorm on the way in (the row sums
    of squares travel with the partial tiles of tile 0), rotation of the query and key heads and residual in the second
    launch's epilogue; against the composition of the RMSNorm, linear and rotary oracles, as for the 64-row kernel."""
    from oracle import rms_norm_oracle, rotary_oracle

    B, S, K, heads, D, rot_heads, with_bias, with_residual = case
    N, M = heads * D, B * S
    gen = torch.Generator().manual_seed(61)
    x = (torch.randn((B, S, K), generator=gen) * 2.0 + 0.3).to(dtype)
    g = (1.0 + 0.2 * torch.randn((K,), generator=gen)).to(dtype)
    w = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
    b = (0.5 * torch.randn((N,), generator=gen)).to(dtype) if with_bias else None
    res = torch.randn((M, N), generator=gen).to(dtype) if with_residual else None
    angles = torch.rand((B, S, D), generator=gen) * 6.28
    cos, sin = angles.cos(), angles.sin()                       # fp32 tables
    eps = 1e-5 if dtype == torch.bfloat16 else 1.6e-5
    out = torch.empty((M, N), dtype=dtype, device="cuda")
    need = _lib.linear_fewrow_workspace_bytes(M, N, K, False, True)
    ws = torch.full((max(need, 16) // 4,), float("nan"), dtype=torch.float32, device="cuda")
    _lib.linear_fewrow_fwd(x.reshape(M, K).cuda(), w.cuda(), None if b is None else b.cuda(), None if res is None else res.cuda(),
                           out, _lib.ACT_NONE, ws, rms_weight=g.cuda(), eps=eps, cos=cos.cuda(), sin=sin.cuda(), head_dim=D,
                           rope_cols=rot_heads * D, rows_per_batch=S)
    torch.cuda.synchronize()
    y = linear_oracle(rms_norm_oracle(x, g, eps), w, b, "")
    heads_view = y.reshape(B, S, heads, D)
    rotated = rotary_oracle(heads_view[:, :, :rot_heads], cos[:, :, None, :], sin[:, :, None, :])
    ref = torch.cat((rotated, heads_view[:, :, rot_heads:]), dim=2).reshape(M, N)
    if res is not None:
        ref = ref + res.float()
    close(out, ref, dtype, scale="magnitude", what=f"stream-K decode projection {case}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("with_norm", [False, True], ids=["plain", "rms"])
@pytest.mark.parametrize("shape", [(20, 352, 320), (33, 96, 256), (64, 11008, 4096), (10, 14336, 256), (48, 1000, 512),
                                   (100, 352, 320), (128, 14336, 256)],
                         ids=lambda s: "x".join(map(str, s)))
def test_few_rows_stream_k_gated_and_normalised(shape, with_norm, dtype, close):
    """The gated linear unit on interleaved weights (the second launch multiplies act(gate) by the value two waves
    further on) and the plain form with bias + activation, each with and without the RMSNorm prologue; 14336 outputs
    against K = 256 are 224 tiles (whole tiles per workgroup for the plain form, which then computes the norm's row
    sums itself)."""
    from kernl_amd.implementations.linear_layer import interleave_glu_rows
    from oracle import glu_oracle, rms_norm_oracle

    M, N, K = shape
    gen = torch.Generator().manual_seed(67)
    x = (torch.randn((M, K), generator=gen) * 3.0 + 0.5).to(dtype)
    g = (1.0 + 0.2 * torch.randn((K,), generator=gen)).to(dtype)
    eps = 1e-5 if dtype == torch.bfloat16 else 1.6e-5
    xin = rms_norm_oracle(x, g, eps) if with_norm else x
    kw = dict(rms_weight=g.cuda(), eps=eps) if with_norm else {}
    w = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
    b = (0.5 * torch.randn((N,), generator=gen)).to(dtype)
    out = torch.empty((M, N), dtype=dtype, device="cuda")
    _lib.linear_fewrow_fwd(x.cuda(), w.cuda(), b.cuda(), None, out, _lib.ACT_SILU, **kw)
    torch.cuda.synchronize()
    close(out, linear_oracle(xin, w, b, "silu"), dtype, scale="magnitude", what=f"stream-K {shape} bias + silu, norm {with_norm}")
    if N % 32 == 0:
        wv = (torch.randn((N, K), generator=gen) * K ** -0.5).to(dtype)
        bv = (0.5 * torch.randn((N,), generator=gen)).to(dtype)
        out = torch.empty((M, N), dtype=dtype, device="cuda")
        _lib.linear_fewrow_fwd(x.cuda(), interleave_glu_rows(w, wv).cuda(), interleave_glu_rows(b, bv).cuda(), None, out,
                               _lib.ACT_SILU, gated=True, **kw)
        torch.cuda.synchronize()
        close(out, glu_oracle(xin, w, b, wv, bv, "silu"), dtype, scale="magnitude", what=f"stream-K gated {shape}, norm {with_norm}")


def test_linear_few_rows_stream_k_is_what_the_operators_run(close, monkeypatch):
    """17 to 128 rows against a large weight: `linear_layer` and the residual form of `decode_linear_layer` take the
    stream-K kernel; fewer rows, small weights and a saved pre-activation keep the other kernels.  Strided rows of x
    and a 3-D input go through unchanged."""
    from kernl_amd.implementations.linear_layer import decode_linear_layer

    calls = []
    real = _lib.linear_fewrow_fwd
    monkeypatch.setattr(_lib, "linear_fewrow_fwd", lambda *a, **k: (calls.append(a[0].shape[0]), real(*a, **k))[1])
    gen = torch.Generator().manual_seed(59)
    N, K = 4608, 2048   # 9.4 M weights: beyond what the small-problem kernels take
    w = (torch.randn((N, K), generator=gen) * K ** -0.5).half()
    b = torch.randn((N,), generator=gen).half()
    for rows, expected in ((16, 0), (17, 1), (64, 1), (65, 1), (128, 1), (129, 0)):
        calls.clear()
        x = torch.randn((rows, K), generator=gen).half()
        out = linear_layer(x.cuda(), w.cuda(), b.cuda(), "relu")
        assert len(calls) == expected, (rows, calls)
        close(out, linear_oracle(x, w, b, "relu"), torch.float16, what=f"{rows} rows")
    calls.clear()
    x = torch.randn((40, K), generator=gen).half()
    linear_layer(x.cuda(), w.cuda(), b.cuda(), "", act_inputs=torch.empty((40, N), dtype=torch.float16, device="cuda"))
    linear_layer(x[:, :256].contiguous().cuda(), w[:, :256].contiguous().cuda(), b.cuda(), "")   # a small weight
    assert calls == []
    wide = torch.randn((2, 20, 2 * K), generator=gen).half()
    xs = wide[:, :, :K]                                    # rows 2 K apart, batch of 2 x 20
    res = torch.randn((2, 20, N), generator=gen).half()
    out = decode_linear_layer(xs.cuda(), w.cuda(), b.cuda(), residual=res.cuda())
    assert calls == [40] and out.shape == (2, 20, N)
    close(out, linear_oracle(xs, w, b, "") + res.float(), torch.float16, scale="magnitude", what="residual form, strided x")


@pytest.mark.parametrize("tile", [1, 3, 5, 7], ids=["8wave-256", "8wave-128", "wide-256", "wide-128"])
def test_linear_fp8_weight_every_kernel(tile, close):
    """Each of the four kernels that take one-byte weights beyond 64 rows, forced in turn on a shape with ragged edges."""
    from oracle import e5m2_decode_oracle

    M, N, K = 700, 1300, 384
    gen = torch.Generator().manual_seed(31)
    x, w, b = _inputs(M, N, K, torch.float16, gen, w_std=K ** -0.5)
    w8 = w.to(torch.float8_e5m2).view(torch.int8)
    lib = _lib.load()
    lib.kernl_linear_force_tile(tile)
    try:
        out = linear_layer(x.cuda(), w8.cuda(), b.cuda(), activation="fast_gelu")
        torch.cuda.synchronize()
    finally:
        lib.kernl_linear_force_tile(0)
    close(out, linear_oracle(x, e5m2_decode_oracle(w8), b, "fast_gelu"), what=f"fp8 weight, kernel choice {tile}")
