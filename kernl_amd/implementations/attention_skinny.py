"""Split-K attention for single-query decoding — host side of `kernl_attention_skinny_fwd`.

Mirrors the operator interface of the reference (src/kernl/implementations/attention_skinny.py:368-548): same
function name, argument meaning, asserts and autocast behaviour.  The reference allocates its partial maxima, sums
and products with torch before the two Triton launches (:416-441); here the same role is played by one fp32
workspace tensor whose size the library reports.
"""
from typing import Optional

import torch
from torch.amp import custom_fwd

from kernl_amd import _lib


ONE_BYTE_KV_DTYPES = (torch.int8, torch.uint8, torch.float8_e5m2)


def to_e5m2(x: torch.Tensor) -> torch.Tensor:
    """fp16 / bf16 / fp32 -> fp8 e5m2 (round to nearest even) as an int8 tensor of the same shape: the storage format
    of the reference's key/value caches (`f16_to_f8`, experimental/llama-v2/kernel/fused_kernel_fp8.py:40-56)."""
    return x.to(torch.float8_e5m2).view(torch.int8)


def from_e5m2(x: torch.Tensor, dtype: torch.dtype = torch.float16) -> torch.Tensor:
    """int8 / uint8 / float8_e5m2 storage -> `dtype` (reference: `f8_to_f16`, fused_kernel_fp8.py:20-37)."""
    return x.view(torch.float8_e5m2).to(dtype)


class SkinnyAttention(torch.autograd.Function):
    @staticmethod
    @custom_fwd(device_type="cuda", cast_inputs=torch.float16)
    def forward(
        ctx,
        q: torch.Tensor,
        k: torch.Tensor,
        v: torch.Tensor,
        output: torch.Tensor,
        sm_scale: float,
        is_causal: bool,
        attention_mask: Optional[torch.Tensor] = None,
    ):
        """out = softmax(q·kᵀ·sm_scale + causal + attention_mask)·v for very few query rows, written into `output`.

        q [batch, heads, m, d] with small m (decoding: 1); k, v [batch, heads, n, d]; attention_mask additive,
        broadcastable as [batch|1, heads|1, m|1, n] (reference asserts: attention_skinny.py:401-454).  k and v may
        be fp8 e5m2 storage (see `to_e5m2`): half the bytes to stream, same arithmetic on the decoded values.
        """
        assert q.shape[-1] == k.shape[-1]
        # keys and values either share the dtype of q, or are both stored as fp8 e5m2 (int8 / uint8 / float8_e5m2
        # tensors; reference: `assert k.dtype == v.dtype and k.dtype in [torch.float16, torch.int8]`,
        # experimental/llama-v2/kernel/fused_kernel_attention.py:115)
        assert k.dtype == v.dtype and q.dtype == output.dtype and (
            k.dtype == q.dtype or k.dtype in ONE_BYTE_KV_DTYPES
        ), f"Incompatible dtypes: {q.dtype}, {k.dtype}, {v.dtype}, {output.dtype}"
        assert q.dtype in [torch.float16, torch.bfloat16], f"Only float16 and bfloat16 are supported, got {q.dtype}"
        batch, heads, m_size, dhead = q.size()
        n_size = k.size(2)
        assert k.size(0) == batch and v.size(0) == batch and k.size(1) == heads and v.size(1) == heads
        assert v.size(2) == n_size and v.size(3) == dhead and output.size() == q.size()
        min_clamp = 0.0
        if attention_mask is not None:
            assert attention_mask.dim() == 4, "Mask must have 4 dimensions"
            assert attention_mask.size(0) in (batch, 1), "Incompatible broadcast batch dimension"
            assert attention_mask.size(1) in (heads, 1), "Incompatible broadcast heads dimension"
            assert attention_mask.size(2) in (m_size, 1), "Incompatible broadcast m_size dimension"
            assert attention_mask.size(3) == n_size, "Last size of mask must broadcast on QK^t"
            assert attention_mask.dtype in _lib.DTYPE_CODE, f"Mask must be a floating tensor, got {attention_mask.dtype}"
            min_clamp = torch.finfo(attention_mask.dtype).min
        nbytes = _lib.attention_skinny_workspace_bytes(batch, heads, m_size, n_size, dhead)
        workspace = torch.empty((nbytes // 4,), dtype=torch.float32, device=q.device) if nbytes > 0 else None
        _lib.attention_skinny_fwd(q, k, v, output, attention_mask, workspace, sm_scale, is_causal, min_clamp)
        return output


def skinny_attention_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    output: torch.Tensor,
    sm_scale: float,
    is_causal: bool = False,
    attention_mask: Optional[torch.Tensor] = None,
):
    """Reference: attention_skinny.py:539-548."""
    return SkinnyAttention.apply(q, k, v, output, sm_scale, is_causal, attention_mask)
