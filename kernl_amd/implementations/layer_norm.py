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
