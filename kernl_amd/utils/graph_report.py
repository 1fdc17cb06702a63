"""Tabulated dump of an fx graph (reference: src/kernl/utils/graph_report.py:20-35) — debugging aid for writing
replacement patterns."""
import torch
from tabulate import tabulate


def graph_report(gm: torch.fx.GraphModule) -> str:
    modules = dict(gm.named_modules())
    rows = []
    for n in gm.graph.nodes:
        kind = type(modules[n.target]).__name__ if n.op == "call_module" and n.target in modules else ""
        target = getattr(n.target, "__name__", str(n.target))
        rows.append([n.op, n.name, target, kind, ", ".join(str(a) for a in n.args), str(dict(n.kwargs)) if n.kwargs else ""])
    return tabulate(rows, headers=["opcode", "name", "target", "module", "args", "kwargs"])
