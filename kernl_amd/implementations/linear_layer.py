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
