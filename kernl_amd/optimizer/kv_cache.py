"""Drop the copies a fresh key/value cache costs.

A forward pass that starts from an empty cache updates it with `torch.cat([torch.tensor([]), states], dim=-2)`:
concatenating an EMPTY tensor, i.e. a plain copy of the keys and of the values of every layer (17 MB each at the
Llama-7B prefill shape, two extra kernels per layer).  `torch.cat` skips empty 1-d operands by definition, so the
node can be replaced by its only real operand.  No counterpart in the reference, whose Llama experiment kept its own
cache tensors (experimental/llama-v2/llama/model.py:208-211).
"""
import torch
from torch.fx import Node


def _is_empty_tensor_literal(value) -> bool:
    return (
        isinstance(value, Node)
        and value.op == "call_function"
        and value.target is torch.tensor
        and len(value.args) == 1
        and isinstance(value.args[0], (list, tuple))
        and len(value.args[0]) == 0
    )


def drop_empty_cat_operands(gm: torch.fx.GraphModule):
    changed = False
    for node in list(gm.graph.nodes):
        if node.op != "call_function" or node.target is not torch.cat or not node.args:
            continue
        operands = node.args[0]
        if not isinstance(operands, (list, tuple)):
            continue
        kept = [o for o in operands if not _is_empty_tensor_literal(o)]
        if len(kept) == len(operands) or len(kept) == 0:
            continue
        if len(kept) == 1:
            node.replace_all_uses_with(kept[0])
            gm.graph.erase_node(node)
        else:
            node.args = (type(operands)(kept),) + tuple(node.args[1:])
        changed = True
    if changed:
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()
