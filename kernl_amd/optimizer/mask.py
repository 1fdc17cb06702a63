"""Keep broadcast attention masks small.

Current transformers versions build the additive mask of eager attention as
`torch.where(bool_mask.expand(B, -1, S, S), 0.0, finfo.min)`: `where` materialises the expanded [B,1,S,S] matrix
although every query row is identical (33 MB at batch 32, sequence 512, re-read by every head of every layer).
`where(expand(c), x, y)` with scalar x, y equals `expand(where(c, x, y))`, so this pass moves the `expand` below the
`where`; the mask the attention kernel then receives is a stride-0 view of a [B,1,1,S] tensor and is consumed as one
value per key.  No counterpart in the reference, whose BERT graphs carried a [B,1,1,S] mask already.
"""
import torch
from torch.fx import Node


def _is_scalar(value) -> bool:
    if isinstance(value, (int, float)):
        return True
    if isinstance(value, Node):
        if value.op == "call_function" and value.target is torch.tensor and value.args and isinstance(value.args[0], (int, float)):
            return True
        if value.op == "call_function" and value.target is torch.full and len(value.args) >= 2 and value.args[0] == ():
            return True
    return False


def scalar_tensors_to_full(gm: torch.fx.GraphModule):
    """`torch.tensor(<python number>, device=gpu)` is a copy from pageable host memory, which stream capture refuses;
    `torch.full((), number, ...)` builds the same 0-d tensor with a fill kernel."""
    changed = False
    for node in list(gm.graph.nodes):
        if node.op != "call_function" or node.target is not torch.tensor:
            continue
        if len(node.args) != 1 or not isinstance(node.args[0], (int, float)) or isinstance(node.args[0], bool):
            continue
        kwargs = {k: v for k, v in node.kwargs.items() if k in ("dtype", "device")}
        if set(node.kwargs) - {"dtype", "device", "requires_grad"}:
            continue
        if "dtype" not in kwargs:
            kwargs["dtype"] = torch.get_default_dtype() if isinstance(node.args[0], float) else torch.int64
        with gm.graph.inserting_before(node):
            full = gm.graph.call_function(torch.full, ((), node.args[0]), kwargs)
        node.replace_all_uses_with(full)
        gm.graph.erase_node(node)
        changed = True
    if changed:
        gm.graph.lint()
        gm.recompile()


def sink_expand_below_where(gm: torch.fx.GraphModule):
    changed = False
    for node in list(gm.graph.nodes):
        if node.op != "call_function" or node.target is not torch.where or len(node.args) != 3 or node.kwargs:
            continue
        cond, a, b = node.args
        if not (isinstance(cond, Node) and cond.op == "call_method" and cond.target == "expand"):
            continue
        if not (_is_scalar(a) and _is_scalar(b)) or len(cond.users) != 1:
            continue
        source = cond.args[0]
        with gm.graph.inserting_before(node):
            small = gm.graph.call_function(torch.where, (source, a, b))
            expanded = gm.graph.call_method("expand", (small,) + tuple(cond.args[1:]), dict(cond.kwargs))
        node.replace_all_uses_with(expanded)
        gm.graph.erase_node(node)
        gm.graph.erase_node(cond)
        changed = True
    if changed:
        gm.graph.lint()
        gm.recompile()
