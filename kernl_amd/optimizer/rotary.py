"""Fuse the rotary position embedding of Hugging Face decoders into one kernel per tensor.

`apply_rotary_pos_emb` traces to, per tensor,

    x * cos + cat((-x[..., D/2:], x[..., :D/2]), dim=-1) * sin

i.e. two slices, a negation, a concatenation, two multiplications and an addition: seven element-wise kernels and six
intermediate tensors for what is one read and one write of x.  The reference removes the same overhead in its Llama
experiment by rotating inside the query/key projection (experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:69-100).
The slice bound is a literal that differs per model, so the sub-graph is matched by walking it rather than by
`replace_pattern`.
"""
import operator

import torch
from torch.fx import Node

from kernl_amd.implementations.rotary import rotary_forward


def rotary_wrapper(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    return rotary_forward(x, cos, sin)


torch.fx.wrap("rotary_wrapper")

_MUL = (operator.mul, torch.mul)
_ADD = (operator.add, torch.add)
_NEG = (operator.neg, torch.neg)


def _is_call(node, targets) -> bool:
    return isinstance(node, Node) and node.op == "call_function" and node.target in targets


def _last_dim_slice(node):
    """(source, start, stop) for `source[..., start:stop]`, else None."""
    if not _is_call(node, (operator.getitem,)) or len(node.args) != 2:
        return None
    source, index = node.args
    if not (isinstance(index, tuple) and len(index) == 2 and index[0] is Ellipsis and isinstance(index[1], slice)):
        return None
    sl = index[1]
    if sl.step not in (None, 1):
        return None
    return source, sl.start, sl.stop


def _rotate_half_source(cat: Node):
    """x and the split point h if `cat` is cat((-x[..., h:], x[..., :h]), dim=-1), else None."""
    if not _is_call(cat, (torch.cat,)) or not cat.args:
        return None
    operands = cat.args[0]
    dim = cat.kwargs.get("dim", cat.args[1] if len(cat.args) > 1 else 0)
    if dim != -1 or not isinstance(operands, (list, tuple)) or len(operands) != 2:
        return None
    neg, low = operands
    if not _is_call(neg, _NEG):
        return None
    high_slice, low_slice = _last_dim_slice(neg.args[0]), _last_dim_slice(low)
    if high_slice is None or low_slice is None:
        return None
    (xa, start_a, stop_a), (xb, start_b, stop_b) = high_slice, low_slice
    if xa is not xb or stop_a is not None or start_b not in (None, 0) or not isinstance(start_a, int) or start_a != stop_b:
        return None
    return xa, start_a


def fuse_rotary_embedding(gm: torch.fx.GraphModule):
    changed = False
    for add in list(gm.graph.nodes):
        if not _is_call(add, _ADD) or len(add.args) != 2 or add.kwargs:
            continue
        for direct, rotated in (add.args, add.args[::-1]):
            if not (_is_call(direct, _MUL) and _is_call(rotated, _MUL)):
                continue
            found = None
            for cat, sin in (rotated.args, rotated.args[::-1]):
                src = _rotate_half_source(cat) if isinstance(cat, Node) else None
                if src is None or not isinstance(sin, Node):
                    continue
                x, half = src
                for xx, cos in (direct.args, direct.args[::-1]):
                    if xx is x and isinstance(cos, Node):
                        found = (x, cos, sin, half)
                        break
                if found:
                    break
            if not found:
                continue
            x, cos, sin, half = found
            # the split must be at the middle of the feature dimension: known only when the tracer recorded shapes
            example = x.meta.get("example_value")
            if example is None or example.dim() != 4 or example.shape[-1] != 2 * half:
                continue
            with gm.graph.inserting_before(add):
                fused = gm.graph.call_function(rotary_wrapper, (x, cos, sin))
            fused.meta = dict(add.meta)
            add.replace_all_uses_with(fused)
            changed = True
            break
    if changed:
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()
