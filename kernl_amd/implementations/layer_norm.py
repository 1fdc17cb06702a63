"""LayerNorm / RMSNorm forward — host side of `kernl_layernorm_fwd` and `kernl_add_layernorm_fwd`.

Mirrors the reference operator (src/kernl/implementations/layer_norm.py:279-346).  The reference's
`implementation` argument selected one of several Triton kernels; there is a single HIP implementation here, so the
argument is accepted and ignored.
"""
from typing import Optional

import torch
from torch.amp import custom_fwd

from kernl_amd import _lib


def _as_rows(t: torch.Tensor) -> torch.Tensor:
    return t if t.ndim == 2 else t.reshape(-1, t.shape[-1])


class LayerNorm(torch.autograd.Function):
    @staticmethod
    @custom_fwd(device_type="cuda", cast_inputs=torch.float16)
    def forward(
        ctx,
        x: torch.Tensor,
        weight: torch.Tensor,
        bias: Optional[torch.Tensor],
        eps: float,
        implementation,
        use_rms_norm: bool,
        residual: Optional[torch.Tensor] = None,
    ):
        assert x.dtype == weight.dtype, f"input and weight bias must have the same dtype: {x.dtype}, {weight.dtype}"
        if bias is not None:
            assert x.dtype == bias.dtype, f"input and bias must have the same dtype: {x.dtype}, {bias.dtype}"
        assert x.dtype in _lib.DTYPE_CODE, f"Unsupported dtype {x.dtype}"
        assert weight.is_contiguous() and (bias is None or bias.is_contiguous())
        assert weight.numel() == x.shape[-1]
        # eps too small to be represented next to an fp16 variance (reference: layer_norm.py:295-296)
        if x.dtype == torch.float16:
            eps = max(eps, 1.6e-5)
        if residual is not None:
            assert residual.shape == x.shape and residual.dtype == x.dtype
        if x.ndim == 2:
            out = torch.empty_like(x)  # keeps the strides of a dense input, e.g. a transposed matrix
            x2d, out2d = x, out
            if out.stride() != x.stride():
                out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
                out2d = out
        else:
            out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
            x2d, out2d = _as_rows(x), out.view(-1, x.shape[-1])
        res2d = None if residual is None else _as_rows(residual)
        M = x2d.shape[0]
        # side outputs the reference keeps for a backward pass (layer_norm.py:303-304)
        mean = torch.empty((M,), dtype=torch.float32, device=x.device)
        rstd = torch.empty((M,), dtype=torch.float32, device=x.device)
        _lib.layernorm_fwd(x2d, weight, bias, out2d, mean, rstd, eps, use_rms_norm, res2d)
        ctx.mean, ctx.rstd = mean, rstd
        return out


def layer_norm(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    eps: float,
    implementation=None,
    use_rms_norm: bool = False,
):
    """Reference: layer_norm.py:338-346."""
    return LayerNorm.apply(x, weight, bias, eps, implementation, use_rms_norm)


def add_layer_norm(
    x: torch.Tensor,
    residual: torch.Tensor,
    weight: torch.Tensor,
    bias: Optional[torch.Tensor],
    eps: float,
    use_rms_norm: bool = False,
):
    """LayerNorm(x + residual) in one pass over HBM.  No reference counterpart: there the add is a separate
    eager op in front of every LayerNorm."""
    return LayerNorm.apply(x, weight, bias, eps, None, use_rms_norm, residual)


def embedding_layer_norm_supported(tables, ids, weight, bias) -> bool:
    """What `embedding_layer_norm` takes: 1 to 3 fp16 / bf16 tables of one width (a multiple of 8, at most 2048) on the
    GPU, int64 ids that broadcast to one [batch, seq] shape, LayerNorm parameters of the tables' dtype."""
    if not 1 <= len(tables) <= 3 or len(ids) != len(tables):
        return False
    t0 = tables[0]
    if not (t0.is_cuda and t0.dtype in (torch.float16, torch.bfloat16) and t0.dim() == 2 and t0.shape[1] % 8 == 0 and t0.shape[1] <= 2048):
        return False
    if any(t.dim() != 2 or t.dtype != t0.dtype or t.shape[1] != t0.shape[1] or not t.is_contiguous() or t.data_ptr() % 16 != 0 for t in tables):
        return False
    if any(i.dtype != torch.int64 or i.dim() > 2 or not i.is_cuda for i in ids):
        return False
    try:
        shape = torch.broadcast_shapes(*[tuple(i.shape) for i in ids])
    except RuntimeError:
        return False
    if len(shape) != 2 or shape[0] * shape[1] == 0:
        return False
    params_ok = weight is not None and weight.dtype == t0.dtype and weight.is_contiguous() and weight.numel() == t0.shape[1]
    return bool(params_ok and (bias is None or (bias.dtype == t0.dtype and bias.is_contiguous() and bias.numel() == t0.shape[1])))


def embedding_layer_norm(tables, ids, weight: torch.Tensor, bias: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """LayerNorm(tables[0][ids[0]] + tables[1][ids[1]] + tables[2][ids[2]]) in one launch: the embedding stage of an
    encoder (word, token-type and position embeddings; the rows are added in the tables' dtype, in that order, as the
    eager model adds them).  The fp16 eps policy is the LayerNorm operator's.  No counterpart in the reference, which
    leaves the lookups and additions to PyTorch in front of its LayerNorm kernel (implementations/layer_norm.py:279-335)."""
    assert embedding_layer_norm_supported(tables, ids, weight, bias)
    shape = torch.broadcast_shapes(*[tuple(i.shape) for i in ids])
    t0 = tables[0]
    if t0.dtype == torch.float16:
        eps = max(eps, 1.6e-5)
    out = torch.empty((shape[0], shape[1], t0.shape[1]), device=t0.device, dtype=t0.dtype)
    _lib.embedding_layernorm_fwd(list(tables), [i.expand(shape) for i in ids], weight, bias, out, eps)
    return out
