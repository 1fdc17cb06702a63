"""Rewrite in-place python operators (`x += y`) as their functional torch equivalents so that later patterns see one
spelling (reference: src/kernl/optimizer/normalizer.py:7-29)."""
import operator

import torch

NORMALIZED_OPERATORS = {
    operator.iadd: torch.add,
    operator.iand: torch.bitwise_and,
    operator.ifloordiv: torch.floor_divide,
    operator.imod: torch.remainder,
    operator.imul: torch.mul,
    operator.imatmul: torch.matmul,
    operator.ior: torch.bitwise_or,
    operator.ipow: torch.pow,
    operator.isub: torch.sub,
    operator.itruediv: torch.div,
    operator.ixor: torch.bitwise_xor,
}


def normalize_operators(gm: torch.fx.GraphModule):
    changed = False
    for node in list(gm.graph.nodes):
        if node.op == "call_function" and node.target in NORMALIZED_OPERATORS:
            node.target = NORMALIZED_OPERATORS[node.target]
            changed = True
    if changed:
        gm.recompile()
