"""Rotary position embedding — host side of `kernl_rope_fwd`.

out = x·cos + rotate_half(x)·sin in the half-split convention of Hugging Face decoders.  The reference fuses the
same rotation, in Meta's interleaved-pair convention, into its query/key projection kernel
(experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:69-100; eager form experimental/llama-v2/llama/model.py:78-88).
"""
import torch

from kernl_amd import _lib


def rotary_forward(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [B,H,S,D]; cos, sin broadcastable to it with sizes [B|1, H|1, S, D].  The result has the dtype PyTorch's
    type promotion gives `x * cos` and the strides of x."""
    assert x.dim() == 4, f"expected [batch, heads, positions, features], got {tuple(x.shape)}"
    assert cos.shape == sin.shape and cos.dtype == sin.dtype, "cos and sin must agree in shape and dtype"
    while cos.dim() < 4:
        cos, sin = cos.unsqueeze(0), sin.unsqueeze(0)
    assert x.shape[-1] % 2 == 0, "feature size must be even"
    assert cos.dtype in _lib.DTYPE_CODE, f"Unsupported table dtype {cos.dtype}"
    out_dtype = torch.result_type(x, cos)
    assert out_dtype in _lib.DTYPE_CODE, f"Unsupported dtype {out_dtype}"
    if x.dtype != out_dtype:
        x = x.to(out_dtype)
    out = torch.empty_like(x)
    _lib.rope_fwd(x, cos, sin, out)
    return out
