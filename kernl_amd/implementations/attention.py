"""Fused attention forward — host side of `kernl_attention_fwd`.

Mirrors the operator interface of the reference (src/kernl/implementations/attention.py:438-541): same function
names, argument meaning, asserts and autocast behaviour.  The Triton launch is replaced by one call through the
C ABI into the gfx950 flash-attention kernel; nothing here computes attention on the host.
"""
import math
from typing import List, Optional, Union

import torch
from torch.amp import custom_fwd

from kernl_amd import _lib

ONE_BYTE_KV_DTYPES = (torch.int8, torch.uint8, torch.float8_e5m2)  # fp8 e5m2 storage of keys and values


def attention_reference(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    output: torch.Tensor,
    sm_scale: float,
    is_causal: bool,
    attention_mask: Union[torch.Tensor, None],
) -> torch.Tensor:
    """Eager attention on the tensors' own device and dtype (reference: attention.py:29-61).

    Kept because the reference exposes it and dispatches to it for masked single-query attention
    (src/kernl/optimizer/attention.py:45-49).  `attention_mask` is ADDED to q·kᵀ·sm_scale, it is not a binary mask.
    """
    p = torch.matmul(q, k.transpose(2, 3)) * sm_scale
    if attention_mask is not None:
        p = p + attention_mask
    if is_causal:
        m_size, n_size = q.size(2), k.size(2)
        keep = torch.tril(torch.ones((m_size, n_size), device=q.device, dtype=torch.bool))
        p = torch.where(keep, p, float("-inf"))
    p = torch.nn.functional.softmax(p, dim=-1)
    return torch.matmul(p.to(v.dtype), v, out=output)


def closest_power_of_2(n: int, min_range: int = 16, max_range: int = 128) -> List[int]:
    """Powers of two around `n` clamped to [min_range, max_range] (reference: attention.py:64-70; known answers
    in test/test_attention.py:148-157).  The reference used it to prune autotune candidates; this build has fixed
    tile shapes and keeps the helper only as part of the public surface."""
    n = max(min(n, max_range), min_range)
    lo = math.floor(math.log2(n - 1))
    hi = math.ceil(math.log2(n + 1))
    return [2**i for i in range(lo, hi + 1)]


class Attention(torch.autograd.Function):
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
        start_position: int = 0,
    ):
        """out = softmax(q·kᵀ·sm_scale + causal + attention_mask)·v, written into `output` (caller allocated).

        With `is_causal`, query row m sees keys 0 .. m + start_position: `start_position` > 0 is the causal attention
        of new tokens over a key/value cache (reference: experimental/llama-v2/kernel/fused_kernel_attention.py:59-76).

        q [batch, heads, m, d]; k, v [batch, heads, n, d]; attention_mask additive, broadcastable as
        [batch|1, heads|1, m|1, n].  fp32 inputs are not supported (reference: attention.py:455-497); under
        autocast every floating argument, mask included, is cast to fp16 first, as `custom_fwd` does there.
        """
        assert q.shape[-1] == k.shape[-1]
        # keys and values stored as fp8 e5m2 bytes (reference: `get_model_fp8` on `cache_k` / `cache_v`,
        # experimental/llama-v2/kernel/fused_kernel_fp8.py:68-74): the kernel widens them on their way into LDS
        one_byte_kv = k.dtype in ONE_BYTE_KV_DTYPES and v.dtype in ONE_BYTE_KV_DTYPES
        if one_byte_kv:
            assert q.dtype == output.dtype == torch.float16, f"fp8 keys/values go with float16 queries, got {q.dtype}"
        else:
            assert (
                q.dtype == k.dtype == v.dtype == output.dtype
            ), f"All tensors must have the same dtype: {q.dtype}, {k.dtype}, {v.dtype}, {output.dtype}"
        assert q.dtype in [torch.float16, torch.bfloat16], f"Only float16 and bfloat16 are supported, got {q.dtype}"
        batch, head_size, m_size, dhead = q.size()
        n_size = k.size(2)
        assert k.size(0) == batch and v.size(0) == batch and k.size(1) == head_size and v.size(1) == head_size
        assert v.size(2) == n_size and v.size(3) == dhead and output.size() == q.size()

        min_clamp = 0.0
        if attention_mask is not None:
            assert attention_mask.dim() == 4, "Mask must have 4 dimensions"
            assert (
                attention_mask.size(0) == batch or attention_mask.size(0) == 1
            ), "Incompatible broadcast batch dimension"
            assert (
                attention_mask.size(1) == head_size or attention_mask.size(1) == 1
            ), "Incompatible broadcast heads dimension"
            assert (
                attention_mask.size(2) == m_size or attention_mask.size(2) == 1
            ), "Incompatible broadcast m_size dimension"
            assert attention_mask.size(3) == n_size, "Last size of mask must broadcast on QK^t"
            assert attention_mask.dtype in _lib.DTYPE_CODE, f"Mask must be a floating tensor, got {attention_mask.dtype}"
            min_clamp = torch.finfo(attention_mask.dtype).min

        if one_byte_kv:
            _lib.attention_kv8_fwd(q, k, v, output, attention_mask, sm_scale, is_causal, int(start_position), min_clamp)
        elif is_causal and start_position:
            _lib.attention_cached_fwd(q, k, v, output, attention_mask, sm_scale, int(start_position), min_clamp)
        else:
            _lib.attention_fwd(q, k, v, output, attention_mask, sm_scale, is_causal, min_clamp)
        return output


def attention_forward(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    output: torch.Tensor,
    sm_scale: float,
    is_causal: bool = False,
    attention_mask: Optional[torch.Tensor] = None,
    start_position: int = 0,
):
    """Reference: attention.py:532-541; `start_position` as in `triton_fa` of
    experimental/llama-v2/kernel/fused_kernel_attention.py:113-146."""
    return Attention.apply(q, k, v, output, sm_scale, is_causal, attention_mask, start_position)
