"""Fused linear layer — host side of `kernl_linear_fwd`.

Mirrors the reference operator (src/kernl/implementations/linear_layer.py:213-292): `linear_layer(x, weight, bias,
activation, act_inputs)` computes activation(x @ weightᵀ + bias) with weight laid out [out_features, in_features].
"""
from typing import Optional

import torch
from torch.amp import custom_fwd

from kernl_amd import _lib

# activation names of the reference (linear_layer.py:198-205) -> epilogue codes of the C ABI.
# "silu" is an addition (SwiGLU gate projections).  As in the reference, an unknown name means "no activation".
ACTIVATIONS = {
    "": _lib.ACT_NONE,
    "relu": _lib.ACT_RELU,
    "tanh": _lib.ACT_TANH,
    "gelu": _lib.ACT_GELU_ERF,
    "fast_gelu": _lib.ACT_GELU_TANH,
    "silu": _lib.ACT_SILU,
}


ONE_BYTE_WEIGHT_DTYPES = (torch.int8, torch.uint8, torch.float8_e5m2)


FEW_ROW_MIN_ROWS = 17          # up to 16 rows the kernel that gives a workgroup 16 columns and all of K is as fast or faster
FEW_ROW_MAX_ROWS = 128         # what `kernl_linear_fewrow_fwd` takes
SPLIT_K_MAX_ROWS = 2048        # beyond that the tiled kernels always have tiles enough; the library decides below it
FEW_ROW_MIN_WEIGHT = 1 << 22   # elements: below that (2048 x 2048) launch latency decides and one launch beats two ...


FEW_ROW_LONG_K = 1536          # ... unless K is long and there are more than 32 rows


def few_row_rule(rows: int, n: int, k: int) -> bool:
    """Where the stream-K kernel is the faster one (measured, graph replay): 17 to 128 rows against a weight of 4 M
    elements or more (5120 x 5120 at 32 / 64 rows: 18 / 21 us against 34 / 35 on the weight-streaming kernel of
    `kernl_linear_fwd`; 4096 x 11008: 25 / 30 against 35 / 53; at 128 rows 28 against 63 and 38 against 130 on its tile
    kernels), and 33 rows or more against smaller weights with a long K (768 x 3072 at 48 / 128 rows: 11 / 14 us against
    15 / 27).  Short K and few rows stay where they were (3072 x 768 at 48 rows: 8.9 against 7.2)."""
    if not FEW_ROW_MIN_ROWS <= rows <= FEW_ROW_MAX_ROWS or k < 256 or k % 64 != 0:
        return False
    return n * k >= FEW_ROW_MIN_WEIGHT or (k >= FEW_ROW_LONG_K and rows > 32)


SMALL_PROBLEM_KERNELS = True   # tuning hook: False keeps such shapes on the stream-K / split-K / tile kernels


def takes_small_problem_kernel(x2d: torch.Tensor, weight: torch.Tensor) -> bool:
    """Whether `kernl_linear_fwd` runs this product on one of its small-problem kernels (one launch of small tiles over
    the whole K: a few hundred rows at most against a weight of a few million elements) — such shapes are not handed
    to the stream-K or split-K entry points, which they would otherwise qualify for."""
    M, K = x2d.shape
    return (
        SMALL_PROBLEM_KERNELS
        and x2d.dtype in (torch.float16, torch.bfloat16) and weight.dtype == x2d.dtype
        and x2d.stride(1) == 1 and x2d.stride(0) % 8 == 0 and x2d.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0
        and _lib.linear_small_kind(M, weight.shape[0], K) != 0
    )


def takes_few_row_kernel(x2d: torch.Tensor, weight: torch.Tensor) -> bool:
    return few_row_rule(x2d.shape[0], weight.shape[0], weight.shape[1]) and _lib.linear_fewrow_supported(x2d, weight)


class LinearLayer(torch.autograd.Function):
    @staticmethod
    @custom_fwd(device_type="cuda", cast_inputs=torch.float16)
    def forward(
        ctx,
        x: torch.Tensor,
        weight: torch.Tensor,
        bias: Optional[torch.Tensor],
        activation: str,
        act_inputs: Optional[torch.Tensor],
    ) -> torch.Tensor:
        """e = activation(x @ weightᵀ + bias); `act_inputs` (optional, [M, N]) receives the pre-activation."""
        x_ = x if x.ndim == 2 else x.reshape(-1, x.shape[-1])

        if weight.dtype in ONE_BYTE_WEIGHT_DTYPES:
            # fp8 e5m2 weight storage (reference: experimental/llama-v2/kernel/fused_kernel_fp8.py:75-84): decoding
            # steps stream the bytes, larger inputs take a tiled kernel that widens them on their way into LDS; only
            # a K that is no multiple of 8 widens the whole weight first
            assert x.dtype == torch.float16, f"fp8 weights go with float16 activations, got {x.dtype}"
            assert weight.is_contiguous() and x_.shape[1] == weight.shape[1]
            if x_.stride(-1) != 1 or x_.stride(0) % 8 != 0 or x_.data_ptr() % 16 != 0:
                x_ = x_.contiguous()
            if _lib.linear_w8_supported(x_, weight):
                M, N = x_.shape[0], weight.shape[0]
                outputs = torch.empty((M, N), device=x.device, dtype=x.dtype)
                if act_inputs is None and takes_few_row_kernel(x_, weight):
                    _lib.linear_fewrow_fwd(x_, weight, bias, None, outputs, ACTIVATIONS.get(activation, _lib.ACT_NONE))
                else:
                    _lib.linear_w8_fwd(x_, weight, bias, outputs, act_inputs, ACTIVATIONS.get(activation, _lib.ACT_NONE))
                return outputs if x.ndim == 2 else outputs.reshape(*x.shape[:-1], N)
            weight = weight.view(torch.float8_e5m2).to(torch.float16)

        assert x.dtype == weight.dtype, f"Input and weight must have the same dtype, got {x.dtype} and {weight.dtype}"
        if bias is not None:
            assert x.dtype == bias.dtype, f"Input and bias must have the same dtype, got {x.dtype} and {bias.dtype}"
        assert x_.shape[1] == weight.shape[1], f"Incompatible dimensions: {x_.shape} - {weight.shape}"
        assert bias is None or bias.is_contiguous()
        assert bias is None or bias.shape[0] == weight.shape[0], "Incompatible dimensions in between weight and bias"
        assert weight.is_contiguous()
        assert x.dtype in _lib.DTYPE_CODE, f"Unsupported dtype {x.dtype}"

        M, K = x_.shape
        N, K = weight.shape
        outputs = torch.empty((M, N), device=x.device, dtype=x.dtype)
        if act_inputs is not None:
            assert act_inputs.shape == (M, N) and act_inputs.dtype == x.dtype
        small = takes_small_problem_kernel(x_, weight)
        split_bytes = 0
        if not small and FEW_ROW_MAX_ROWS < M <= SPLIT_K_MAX_ROWS:
            split_bytes = _lib.linear_splitk_workspace_bytes(x_, weight)
        if small:
            _lib.linear_fwd(x_, weight, bias, outputs, act_inputs, ACTIVATIONS.get(activation, _lib.ACT_NONE))
        elif act_inputs is None and takes_few_row_kernel(x_, weight):
            _lib.linear_fewrow_fwd(x_, weight, bias, None, outputs, ACTIVATIONS.get(activation, _lib.ACT_NONE))
        elif split_bytes:
            # too few 128-row tiles to occupy the chip: ranges of K per tile, added by a second launch
            workspace = torch.empty(split_bytes, dtype=torch.uint8, device=x.device)
            _lib.linear_splitk_fwd(x_, weight, bias, outputs, act_inputs, ACTIVATIONS.get(activation, _lib.ACT_NONE), workspace)
        else:
            _lib.linear_fwd(x_, weight, bias, outputs, act_inputs, ACTIVATIONS.get(activation, _lib.ACT_NONE))
        return outputs if x.ndim == 2 else outputs.reshape(*x.shape[:-1], N)


def linear_layer(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    activation="",
    act_inputs: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Reference: linear_layer.py:285-292."""
    return LinearLayer.apply(x, weight, bias, activation, act_inputs)


GLU_BLOCK = 32  # rows per interleaving block of `kernl_linear_glu_fwd`


def interleave_glu_rows(gate: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
    """[N, ...] gate and value parameters -> [2N, ...] with 32-row blocks alternating gate, value."""
    assert gate.shape == value.shape and gate.shape[0] % GLU_BLOCK == 0
    g = gate.reshape(gate.shape[0] // GLU_BLOCK, 1, GLU_BLOCK, *gate.shape[1:])
    v = value.reshape(value.shape[0] // GLU_BLOCK, 1, GLU_BLOCK, *value.shape[1:])
    return torch.cat((g, v), dim=1).reshape(2 * gate.shape[0], *gate.shape[1:]).contiguous()


def glu_supported(x: torch.Tensor, out_features: int) -> bool:
    """What the gated kernel needs; callers run the two projections separately otherwise."""
    return (
        x.dtype in (torch.float16, torch.bfloat16)
        and out_features % GLU_BLOCK == 0
        and x.shape[-1] % 8 == 0
    )


class LinearGLU(torch.autograd.Function):
    @staticmethod
    @custom_fwd(device_type="cuda", cast_inputs=torch.float16)
    def forward(ctx, x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], activation: str) -> torch.Tensor:
        assert x.dtype == weight.dtype, f"Input and weight must have the same dtype, got {x.dtype} and {weight.dtype}"
        assert x.dtype in (torch.float16, torch.bfloat16), f"Unsupported dtype {x.dtype}"
        assert weight.is_contiguous() and weight.shape[0] % (2 * GLU_BLOCK) == 0
        assert x.shape[-1] == weight.shape[1], f"Incompatible dimensions: {x.shape} - {weight.shape}"
        assert bias is None or (bias.is_contiguous() and bias.dtype == x.dtype and bias.shape[0] == weight.shape[0])
        x_ = x if x.ndim == 2 else x.reshape(-1, x.shape[-1])
        if x_.stride(-1) != 1 or x_.stride(0) % 8 != 0 or x_.data_ptr() % 16 != 0:
            x_ = x_.contiguous()
        M, N = x_.shape[0], weight.shape[0] // 2
        out = torch.empty((M, N), device=x.device, dtype=x.dtype)
        if takes_few_row_kernel(x_, weight):
            _lib.linear_fewrow_fwd(x_, weight, bias, None, out, ACTIVATIONS.get(activation, _lib.ACT_NONE), gated=True)
        else:
            _lib.linear_glu_fwd(x_, weight, bias, out, ACTIVATIONS.get(activation, _lib.ACT_NONE))
        return out if x.ndim == 2 else out.reshape(*x.shape[:-1], N)


def linear_glu_layer(x: torch.Tensor, weight_interleaved: torch.Tensor, bias_interleaved: Optional[torch.Tensor], activation="silu") -> torch.Tensor:
    """activation(x @ w_gateᵀ + b_gate) * (x @ w_valueᵀ + b_value) with the parameters interleaved by
    `interleave_glu_rows`.  Reference: `kernel_ff` (experimental/llama-v2/kernel/fused_kernel_ff.py:82-117), without
    its RMSNorm prologue."""
    return LinearGLU.apply(x, weight_interleaved, bias_interleaved, activation)


def rms_linear_layer(
    x: torch.Tensor,
    rms_weight: torch.Tensor,
    eps: float,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    activation: str = "",
    gated: bool = False,
    folded_weight: Optional[torch.Tensor] = None,
    rstd: Optional[torch.Tensor] = None,
    unfolded=None,
) -> torch.Tensor:
    """activation(linear(rms_norm(x, rms_weight, eps), weight, bias)) — or, with `gated`, the gated linear unit of the
    normalised input (weight and bias interleaved by `interleave_glu_rows`) — in one launch for decoding steps.

    Prompts (more rows than the few-row kernels take) run the norm folded away when the caller hands in `folded_weight`
    = weight * rms_weight[None, :]: rms_norm(x) @ w^T = rstd[:, None] * (x @ folded_weight^T), the factor applied in the
    tile kernels' epilogue (`scaled_linear_layer`).  `rstd` [rows] fp32 = 1 / sqrt(mean(x^2) + eps) comes from whoever
    produced x (`add_rms_stats`) or is computed here in one pass over x.  A caller that passes the folded weight as
    `weight` too (it keeps no other arrangement) gives `unfolded`, a function returning the plain one, for the shapes that
    end up on the two-launch path.

    Reference: `rms_matmul_rbe_wrapper` without the rotary epilogue (experimental/llama-v2/kernel/
    fused_kernel_proj_qkv.py:186-213) and `kernel_ff` (fused_kernel_ff.py:82-117), whose kernels normalise inside the
    product.  Inputs the fused kernel does not take (more than 64 rows, K not a multiple of 64) are normalised by the
    RMSNorm kernel and multiplied by the linear kernels."""
    from kernl_amd.implementations.layer_norm import layer_norm

    assert x.dtype == weight.dtype == rms_weight.dtype and x.dtype in (torch.float16, torch.bfloat16)
    assert weight.is_contiguous() and rms_weight.is_contiguous() and rms_weight.shape[0] == x.shape[-1]
    x_ = x if x.ndim == 2 else x.reshape(-1, x.shape[-1])
    if x_.stride(-1) != 1 or x_.stride(0) % 8 != 0 or x_.data_ptr() % 16 != 0:
        x_ = x_.contiguous()
    n_out = weight.shape[0] // 2 if gated else weight.shape[0]
    if x.dtype == torch.float16:
        eps = max(eps, 1.6e-5)  # the fp16 policy of the RMSNorm operator (reference: layer_norm.py:295-296)
    if takes_few_row_kernel(x_, weight) and (not gated or n_out % GLU_BLOCK == 0):
        out = torch.empty((x_.shape[0], n_out), device=x.device, dtype=x.dtype)
        _lib.linear_fewrow_fwd(x_, weight, bias, None, out, ACTIVATIONS.get(activation, _lib.ACT_NONE),
                               rms_weight=rms_weight, eps=eps, gated=gated)
        return out if x.ndim == 2 else out.reshape(*x.shape[:-1], n_out)
    if _lib.linear_rms_supported(x_) and (not gated or n_out % GLU_BLOCK == 0):
        out = torch.empty((x_.shape[0], n_out), device=x.device, dtype=x.dtype)
        _lib.linear_rms_fwd(x_, rms_weight, eps, weight, bias, out, ACTIVATIONS.get(activation, _lib.ACT_NONE), gated)
        return out if x.ndim == 2 else out.reshape(*x.shape[:-1], n_out)
    if (
        folded_weight is not None
        and activation == ("silu" if gated else "")
        and (not gated or n_out % GLU_BLOCK == 0)
        and x_.shape[0] > FEW_ROW_MAX_ROWS
        and _lib.linear_scaled_supported(x_, folded_weight)
        and (bias is None or bias.dtype == x.dtype)
        # only where the plain product would run the wide tile kernels anyway (not the small-tile or split-K forms)
        and not takes_small_problem_kernel(x_, folded_weight)
        and (x_.shape[0] > SPLIT_K_MAX_ROWS or _lib.linear_splitk_workspace_bytes(x_, folded_weight) == 0)
    ):
        if rstd is None:
            rstd = rms_stats(x_, eps, clamp=False)
        out = scaled_linear_layer(x_, folded_weight, bias, rstd, activation, gated)
        return out if x.ndim == 2 else out.reshape(*x.shape[:-1], n_out)
    normed = layer_norm(x, rms_weight, None, eps, use_rms_norm=True)
    if unfolded is not None:
        weight = unfolded()
    if gated:
        return linear_glu_layer(normed, weight, bias, activation)
    return linear_layer(normed, weight, bias, activation)


def rms_eps(dtype: torch.dtype, eps: float) -> float:
    """The eps the RMSNorm operator uses for `dtype`: fp16 inputs clamp it to 1.6e-5 (reference: layer_norm.py:295-296)."""
    return max(eps, 1.6e-5) if dtype == torch.float16 else eps


def rms_stats(x: torch.Tensor, eps: float, clamp: bool = True) -> torch.Tensor:
    """rstd [rows] fp32 = 1 / sqrt(mean(x^2, -1) + eps) of a 16-bit tensor, one pass over x."""
    x_ = x if x.ndim == 2 else x.reshape(-1, x.shape[-1])
    if x_.stride(-1) != 1 or x_.stride(0) % 8 != 0 or x_.data_ptr() % 16 != 0:
        x_ = x_.contiguous()
    rstd = torch.empty((x_.shape[0],), device=x.device, dtype=torch.float32)
    _lib.add_rms_stats_fwd(x_, None, None, rstd, rms_eps(x.dtype, eps) if clamp else eps)
    return rstd


def add_rms_stats_supported(a: torch.Tensor, b: torch.Tensor) -> bool:
    return (
        a.is_cuda and a.dtype in (torch.float16, torch.bfloat16) and b.dtype == a.dtype and a.shape == b.shape
        and a.ndim >= 2 and a.shape[-1] % 8 == 0 and a.numel() > 0
    )


def add_rms_stats(a: torch.Tensor, b: torch.Tensor, eps: float):
    """(a + b, rstd): the sum rounded to the inputs' dtype and, per row, 1 / sqrt(mean(sum^2) + eps) of the rounded sum
    in fp32 — a residual addition together with the row statistics of the RMSNorm that follows it, in one pass.
    `eps` is used as given (`rms_eps` holds the operator's fp16 policy)."""
    assert add_rms_stats_supported(a, b)
    rows = a.numel() // a.shape[-1]

    def rows_of(t):
        t2 = t.reshape(rows, t.shape[-1])
        return t2 if t2.stride(-1) == 1 and t2.stride(0) % 8 == 0 and t2.data_ptr() % 16 == 0 else t2.contiguous()

    out = torch.empty(a.shape, device=a.device, dtype=a.dtype)
    rstd = torch.empty((rows,), device=a.device, dtype=torch.float32)
    _lib.add_rms_stats_fwd(rows_of(a), rows_of(b), out.view(rows, a.shape[-1]), rstd, eps)
    return out, rstd


def scaled_linear_layer(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], row_scale: torch.Tensor,
                        activation: str = "", gated: bool = False) -> torch.Tensor:
    """act((x @ weight^T) * row_scale[:, None] + bias) for 2-D x; gated: silu(gate) * value of the interleaved weight.
    The tile kernels' epilogue applies the factor: see `kernl_linear_scaled_fwd`."""
    assert x.ndim == 2 and row_scale.dtype == torch.float32 and row_scale.numel() == x.shape[0]
    n_out = weight.shape[0] // 2 if gated else weight.shape[0]
    out = torch.empty((x.shape[0], n_out), device=x.device, dtype=x.dtype)
    _lib.linear_scaled_fwd(x, weight, bias, row_scale, out, ACTIVATIONS.get(activation, _lib.ACT_NONE), gated)
    return out


def residual_linear_supported(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], residual: torch.Tensor) -> bool:
    """Whether `residual_linear_layer` takes this input: a 16-bit problem that `linear_layer` would run on the wide tile
    kernels (they alone add a residual in their epilogue), a residual of the output's shape and dtype."""
    if not (x.is_cuda and x.dtype in (torch.float16, torch.bfloat16) and weight.dtype == x.dtype and residual.dtype == x.dtype):
        return False
    if bias is not None and bias.dtype != x.dtype:
        return False
    if x.numel() == 0 or residual.shape != (*x.shape[:-1], weight.shape[0]) or torch.is_autocast_enabled("cuda"):
        return False
    rows = x.numel() // x.shape[-1]
    if rows <= FEW_ROW_MAX_ROWS or weight.shape[0] % 8 != 0:
        return False
    x_ = x if x.ndim == 2 else x.reshape(-1, x.shape[-1])
    if not _lib.linear_scaled_supported(x_, weight):
        return False
    if rows <= SPLIT_K_MAX_ROWS and _lib.linear_splitk_workspace_bytes(x_, weight) != 0:
        return False
    return _lib.linear_wide_kind(rows, weight.shape[0], weight.shape[1]) != 0


def residual_linear_layer(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], residual: torch.Tensor) -> torch.Tensor:
    """residual + linear(x, weight, bias) in one launch: the addition happens in the tile kernels' epilogue, on the rounded
    projection (bit for bit the two-step result).  See `kernl_linear_residual_fwd`; no counterpart in the reference."""
    assert residual_linear_supported(x, weight, bias, residual)
    rows, n_out = x.numel() // x.shape[-1], weight.shape[0]
    x_ = x if x.ndim == 2 else x.reshape(rows, x.shape[-1])
    res_ = residual.reshape(rows, n_out)
    out = torch.empty((rows, n_out), device=x.device, dtype=x.dtype)
    _lib.linear_residual_fwd(x_, weight, bias, res_, out)
    return out.reshape(residual.shape)


def decode_linear_supported(x: torch.Tensor, weight: torch.Tensor, head_dim: Optional[int] = None) -> bool:
    """Whether `decode_linear_layer` takes this input: 16-bit, K a multiple of 64, at most 64 rows in all — or up to 128
    against a weight large enough for the stream-K kernel (whose rotation wants a head size of 32, 64 or 128)."""
    if x.dtype not in (torch.float16, torch.bfloat16) or weight.dtype != x.dtype or x.shape[-1] % 64 != 0:
        return False
    rows = x.numel() // x.shape[-1]
    if not (weight.is_contiguous() and weight.data_ptr() % 16 == 0):
        return False
    if 0 < rows <= 64:
        return True
    return few_row_rule(rows, weight.shape[0], weight.shape[1]) and (head_dim is None or head_dim in (32, 64, 128))


def decode_linear_layer(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor] = None,
    rms_weight: Optional[torch.Tensor] = None,
    eps: float = 0.0,
    residual: Optional[torch.Tensor] = None,
    cos: Optional[torch.Tensor] = None,
    sin: Optional[torch.Tensor] = None,
    head_dim: int = 0,
    rope_cols: int = 0,
) -> torch.Tensor:
    """One launch for a decoding step's projection and what surrounds it:

        y = linear(rms_norm(x, rms_weight, eps) if rms_weight is given else x, weight, bias)
        y[..., :rope_cols] rotated head by head (half-split rotary embedding) when cos / sin are given
        out = y + residual when a residual is given

    x [batch, positions, K] or [rows, K], at most 64 rows in all (128 against large weights); cos / sin [batch | 1, positions, head_dim] (a 2-D x
    counts as one batch entry); residual of the output's shape.  Reference: `rms_matmul_rbe_qkv_wrapper`,
    experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:289-344 (RMSNorm prologue + query/key/value projection +
    rotation of the query and key columns in one kernel)."""
    assert decode_linear_supported(x, weight, head_dim if cos is not None else None), \
        "decode_linear_layer: at most 64 rows of 16-bit x (128 against a large weight), K a multiple of 64"
    assert (cos is None) == (sin is None)
    K, N = x.shape[-1], weight.shape[0]
    x_ = x if x.ndim == 2 else x.reshape(-1, K)
    if x_.stride(-1) != 1 or x_.stride(0) % 8 != 0 or x_.data_ptr() % 16 != 0:
        x_ = x_.contiguous()
    rows_per_batch = x.shape[-2] if x.ndim == 3 else x_.shape[0]
    if rms_weight is not None:
        assert rms_weight.dtype == x.dtype and rms_weight.is_contiguous() and rms_weight.shape[0] == K
        if x.dtype == torch.float16:
            eps = max(eps, 1.6e-5)  # the fp16 policy of the RMSNorm operator (reference: layer_norm.py:295-296)
    if cos is not None:
        assert rms_weight is not None, "the rotating form comes with the RMSNorm prologue"
        assert cos.shape == sin.shape and cos.dtype == sin.dtype and cos.dim() == 3 and cos.shape[-1] == head_dim
        assert cos.shape[1] == rows_per_batch and cos.shape[0] in (1, x_.shape[0] // rows_per_batch)
        assert cos.stride(-1) == 1 and sin.stride() == cos.stride(), "tables need unit feature stride and equal layouts"
        assert head_dim % 32 == 0 and N % head_dim == 0 and rope_cols % head_dim == 0 and 0 <= rope_cols <= N
    res_ = None
    if residual is not None:
        assert residual.dtype == x.dtype and residual.numel() == x_.shape[0] * N
        res_ = residual.reshape(-1, N)
    out = torch.empty((x_.shape[0], N), device=x.device, dtype=x.dtype)
    if takes_few_row_kernel(x_, weight) and (cos is None or head_dim in (32, 64, 128)):
        _lib.linear_fewrow_fwd(x_, weight, bias, res_, out, _lib.ACT_NONE, rms_weight=rms_weight, eps=eps, cos=cos, sin=sin,
                               head_dim=head_dim, rope_cols=rope_cols, rows_per_batch=rows_per_batch)
    else:
        _lib.linear_decode_fwd(x_, rms_weight, eps, weight, bias, res_, out, cos, sin, head_dim, rope_cols, rows_per_batch)
    return out if x.ndim == 2 else out.reshape(*x.shape[:-1], N)
