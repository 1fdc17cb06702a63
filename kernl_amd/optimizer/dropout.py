"""Remove dropout from an inference graph (reference: src/kernl/optimizer/dropout.py:19-33): every
`nn.Dropout` module call and every `F.dropout` call is replaced by its input."""
import torch


def remove_dropout(gm: torch.fx.GraphModule):
    modules = dict(gm.named_modules())
    changed = False
    for node in list(gm.graph.nodes):
        is_module = node.op == "call_module" and isinstance(modules.get(node.target), torch.nn.Dropout)
        is_function = node.op == "call_function" and node.target is torch.nn.functional.dropout
        if is_module or is_function:
            source = node.args[0] if node.args else node.kwargs["input"]
            node.replace_all_uses_with(source)
            gm.graph.erase_node(node)
            changed = True
    if changed:
        gm.recompile()
