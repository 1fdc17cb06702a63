"""Attention graph patterns (reference: src/kernl/optimizer/attention.py:24-112).

`attention_wrapper` is the fx leaf the rewritten graph calls.  Patterns 1-3 are the reference's (BERT `/ 8.0 + mask`,
T5 `+ position_bias` with float softmax, Whisper bmm); the wildcard-scale and `scaled_dot_product_attention` patterns
cover what current transformers versions emit.
"""
from typing import Optional

import torch

from kernl_amd.implementations.attention import attention_forward
from kernl_amd.implementations.attention_skinny import skinny_attention_forward
from kernl_amd.utils.extended_matcher import replace_pattern


def _per_key_view(mask: torch.Tensor) -> torch.Tensor:
    """A mask that was `expand`ed over the query dimension carries one value per key: look at a single row."""
    if mask.dim() == 4 and mask.size(2) > 1 and mask.stride(2) == 0:
        return mask[:, :, :1, :]
    return mask


def _rows_aligned(*tensors: torch.Tensor) -> bool:
    """Unit feature stride and 16-byte aligned rows (what the split-K kernel's vector loads need)."""
    for t in tensors:
        if t.stride(-1) != 1 or t.data_ptr() % 16 != 0 or any(st % 8 != 0 for st in t.stride()[:-1]):
            return False
    return True


SPLIT_K_MAX_ROWS = 65535  # batch x heads x queries the split-K kernel's launch grid can hold


def takes_split_k_kernel(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> bool:
    """Whether a [batch, heads, queries, dhead] problem goes to the split-K (single-query) kernel: one query per
    row over more than 50 keys (reference: optimizer/attention.py:45), a head size that kernel is built for, rows it
    can load 16 bytes at a time, and no more rows than its grid holds — larger decode batches stay on the tiled
    kernel, which takes one-query tiles too."""
    dhead = q.size(-1)
    return (
        q.size(-2) == 1
        and k.size(-2) > 50
        and 8 <= dhead <= 256
        and (dhead & (dhead - 1)) == 0
        and q.size(0) * q.size(1) * q.size(2) <= SPLIT_K_MAX_ROWS
        and _rows_aligned(q, k, v)
    )


def attention_wrapper(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    output: torch.Tensor,
    sm_scale: float,
    is_causal: bool,
    attention_mask: Optional[torch.Tensor],
) -> torch.Tensor:
    # bmm-shaped tensors use their first dimension for batch and heads together; the kernel wants 4 dimensions
    extend_head = q.dim() == 3
    if extend_head:
        q, k, v, output = q.unsqueeze(1), k.unsqueeze(1), v.unsqueeze(1), output.unsqueeze(1)
        if attention_mask is not None and attention_mask.dim() == 3:
            attention_mask = attention_mask.unsqueeze(1)
    if attention_mask is not None:
        attention_mask = _per_key_view(attention_mask)
    # Single-query attention over long keys has no parallelism over rows: like the reference
    # (optimizer/attention.py:45-49) hand it to the split-K kernel — which here also takes masks and the causal
    # flag, where the reference falls back to eager PyTorch.  Head sizes it does not cover stay on the tiled kernel.
    if takes_split_k_kernel(q, k, v):
        skinny_attention_forward(q, k, v, output, sm_scale, is_causal=is_causal, attention_mask=attention_mask)
    else:
        attention_forward(q, k, v, output, sm_scale, is_causal=is_causal, attention_mask=attention_mask)
    if extend_head:
        output = output.squeeze(1)
    return output


def additive_mask(mask: torch.Tensor) -> torch.Tensor:
    """A boolean attention mask (True = attend) as the additive 0 / -inf mask the kernels take, one value per key
    where the query dimension was only `expand`ed.  Any other mask passes through."""
    if mask.dtype != torch.bool:
        return mask
    while mask.dim() < 4:
        mask = mask.unsqueeze(0)
    return torch.where(_per_key_view(mask), 0.0, float("-inf"))


def sdpa_wrapper(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    attn_mask: Optional[torch.Tensor],
    scale: Optional[float],
    is_causal: bool,
    assume_causal: bool,
) -> torch.Tensor:
    """`F.scaled_dot_product_attention(q, k, v, attn_mask, 0.0, is_causal, scale)` on the fused kernel.  A boolean
    mask (True = attend) becomes the additive 0 / -inf mask the kernel takes."""
    if scale is None:
        scale = q.size(-1) ** -0.5
    mask = attn_mask
    if mask is not None:
        while mask.dim() < 4:
            mask = mask.unsqueeze(0)
        mask = _per_key_view(additive_mask(mask))
    output = torch.empty_like(q)
    return attention_wrapper(q, k, v, output, float(scale), bool(is_causal) or assume_causal, mask)


torch.fx.wrap("attention_wrapper")
torch.fx.wrap("sdpa_wrapper")
torch.fx.wrap("additive_mask")


def fuse_attention_pattern_1(gm: torch.fx.GraphModule, is_causal: bool):
    """BERT as the reference saw it: softmax(q·kᵀ / 8.0 + mask)·v."""

    def pattern(q, k, attention_mask, v):
        scores = torch.matmul(q, k.transpose(-1, -2)) / 8.0
        probs = torch.nn.functional.softmax(scores + attention_mask, dim=-1)
        return torch.matmul(probs, v)

    def replace(q, k, attention_mask, v):
        return attention_wrapper(q, k, v, torch.empty_like(q), 1 / 8.0, is_causal, attention_mask)

    replace_pattern(gm, pattern, replace)


def fuse_attention_pattern_2(gm: torch.fx.GraphModule, is_causal: bool):
    """T5: scores + position_bias, softmax in float, cast back; no scaling."""

    def pattern(q, k, position_bias, v):
        biased = torch.add(torch.matmul(q, k.transpose(3, 2)), position_bias)
        probs = torch.nn.functional.softmax(biased.float(), dim=-1).type_as(biased)
        return torch.matmul(probs, v)

    def replace(q, k, position_bias, v):
        return attention_wrapper(q, k, v, torch.empty_like(q), 1.0, is_causal, position_bias)

    replace_pattern(gm, pattern, replace)


def fuse_attention_pattern_3(gm: torch.fx.GraphModule, is_causal: bool):
    """Whisper: bmm-shaped, pre-scaled q, no mask."""

    def pattern(q, k, v):
        probs = torch.nn.functional.softmax(torch.bmm(q, k.transpose(1, 2)), dim=-1)
        return torch.bmm(probs, v)

    def replace(q, k, v):
        return attention_wrapper(q, k, v, torch.empty_like(q), 1.0, is_causal, None)

    replace_pattern(gm, pattern, replace)


_TRANSPOSES = ((-1, -2), (-2, -1), (2, 3), (3, 2))


def _scaled_patterns(d0: int, d1: int, is_causal: bool):
    """(pattern, replacement) pairs for one spelling of the key transposition.  `literal_scale` only binds to a python
    number in the graph (the kernel takes the scale as a host float)."""

    def pattern_mul_mask(q, k, literal_scale, attention_mask, v):
        scores = torch.matmul(q, k.transpose(d0, d1)) * literal_scale
        probs = torch.nn.functional.softmax(scores + attention_mask, dim=-1)
        return torch.matmul(probs, v)

    def replace_mul_mask(q, k, literal_scale, attention_mask, v):
        output = torch.empty_like(q)
        return attention_wrapper(q, k, v, output, literal_scale, is_causal, attention_mask)

    def pattern_div_mask(q, k, literal_scale, attention_mask, v):
        scores = torch.matmul(q, k.transpose(d0, d1)) / literal_scale
        probs = torch.nn.functional.softmax(scores + attention_mask, dim=-1)
        return torch.matmul(probs, v)

    def replace_div_mask(q, k, literal_scale, attention_mask, v):
        output = torch.empty_like(q)
        return attention_wrapper(q, k, v, output, 1.0 / literal_scale, is_causal, attention_mask)

    def pattern_mul(q, k, literal_scale, v):
        scores = torch.matmul(q, k.transpose(d0, d1)) * literal_scale
        probs = torch.nn.functional.softmax(scores, dim=-1)
        return torch.matmul(probs, v)

    def replace_mul(q, k, literal_scale, v):
        output = torch.empty_like(q)
        return attention_wrapper(q, k, v, output, literal_scale, is_causal, None)

    def pattern_div(q, k, literal_scale, v):
        scores = torch.matmul(q, k.transpose(d0, d1)) / literal_scale
        probs = torch.nn.functional.softmax(scores, dim=-1)
        return torch.matmul(probs, v)

    def replace_div(q, k, literal_scale, v):
        output = torch.empty_like(q)
        return attention_wrapper(q, k, v, output, 1.0 / literal_scale, is_causal, None)

    # softmax evaluated in fp32 and cast back (Llama-style eager attention); the fused kernel always keeps its
    # softmax statistics in fp32, so the casts disappear
    def pattern_mul_mask_f32(q, k, literal_scale, attention_mask, v, literal_dtype):
        scores = torch.matmul(q, k.transpose(d0, d1)) * literal_scale
        probs = torch.nn.functional.softmax(scores + attention_mask, dim=-1, dtype=torch.float32).to(literal_dtype)
        return torch.matmul(probs, v)

    def replace_mul_mask_f32(q, k, literal_scale, attention_mask, v, literal_dtype):
        output = torch.empty_like(q)
        return attention_wrapper(q, k, v, output, literal_scale, is_causal, attention_mask)

    def pattern_mul_f32(q, k, literal_scale, v, literal_dtype):
        scores = torch.matmul(q, k.transpose(d0, d1)) * literal_scale
        probs = torch.nn.functional.softmax(scores, dim=-1, dtype=torch.float32).to(literal_dtype)
        return torch.matmul(probs, v)

    def replace_mul_f32(q, k, literal_scale, v, literal_dtype):
        output = torch.empty_like(q)
        return attention_wrapper(q, k, v, output, literal_scale, is_causal, None)

    return (
        (pattern_mul_mask, replace_mul_mask),
        (pattern_div_mask, replace_div_mask),
        (pattern_mul_mask_f32, replace_mul_mask_f32),
        (pattern_mul, replace_mul),
        (pattern_div, replace_div),
        (pattern_mul_f32, replace_mul_f32),
    )


def fuse_attention_scaled(gm: torch.fx.GraphModule, is_causal: bool):
    """softmax(q·kᵀ {*, /} s (+ mask))·v for ANY literal scale `s`: what eager attention of current transformers models
    traces to (`matmul(q, k.transpose(2, 3)) * scaling + mask`).  The scale is a wildcard bound to the graph's literal."""
    for d0, d1 in _TRANSPOSES:
        for pattern, replacement in _scaled_patterns(d0, d1, is_causal):
            replace_pattern(gm, pattern, replacement)


def fuse_attention_sdpa(gm: torch.fx.GraphModule, is_causal: bool):
    """`F.scaled_dot_product_attention` without dropout."""
    sdpa = torch.nn.functional.scaled_dot_product_attention
    for node in list(gm.graph.nodes):
        if node.op != "call_function" or node.target is not sdpa:
            continue
        pair = node.normalized_arguments(gm, normalize_to_only_use_kwargs=True)
        kwargs = dict(pair.kwargs) if pair is not None else None
        if kwargs is None:
            names = ("query", "key", "value", "attn_mask", "dropout_p", "is_causal", "scale", "enable_gqa")
            kwargs = dict(zip(names, node.args))
            kwargs.update(node.kwargs)
        if kwargs.get("dropout_p", 0.0) != 0.0 or kwargs.get("enable_gqa", False):
            continue
        scale, causal = kwargs.get("scale"), kwargs.get("is_causal", False)
        if isinstance(scale, torch.fx.Node) or isinstance(causal, torch.fx.Node):
            continue
        with gm.graph.inserting_before(node):
            new = gm.graph.call_function(
                sdpa_wrapper,
                (kwargs["query"], kwargs["key"], kwargs["value"], kwargs.get("attn_mask"), scale, causal, is_causal),
            )
        node.replace_all_uses_with(new)
        gm.graph.erase_node(node)
    gm.graph.lint()
    gm.recompile()


def share_mask_conversion(gm: torch.fx.GraphModule):
    """Every layer of an encoder receives the same mask node; converting a boolean mask inside each fused call costs
    a few small kernels per layer, which is most of a short sequence's forward.  One `additive_mask` node per
    distinct mask feeds all the calls that use it."""
    converted = {}
    for node in list(gm.graph.nodes):
        if node.op != "call_function" or node.target is not sdpa_wrapper:
            continue
        mask = node.args[3]
        if not isinstance(mask, torch.fx.Node) or (mask.op == "call_function" and mask.target is additive_mask):
            continue
        if mask not in converted:
            with gm.graph.inserting_after(mask):
                converted[mask] = gm.graph.call_function(additive_mask, (mask,))
        args = list(node.args)
        args[3] = converted[mask]
        node.args = tuple(args)
    if converted:
        gm.graph.lint()
        gm.recompile()
