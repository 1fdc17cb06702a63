"""Literal-argument comparison of two fx nodes (reference: src/kernl/utils/fx.py:21-39).

`kernl_amd.utils.extended_matcher` performs this comparison as part of matching; the helper is kept as a public
function because graph passes written against the reference call it directly.
"""
from typing import Any

from torch.fx import Node


def _same(a: Any, b: Any) -> bool:
    if isinstance(a, Node) and isinstance(b, Node):
        return True  # tensors are matched structurally elsewhere; only literals are compared here
    if type(a) is not type(b):
        return False
    if isinstance(a, (tuple, list)):
        return len(a) == len(b) and all(_same(x, y) for x, y in zip(a, b))
    return a == b


def static_args_are_equal(pn: Node, gn: Node) -> bool:
    """True when the positional arguments of `pn` and `gn` agree wherever they are literals."""
    if len(pn.args) != len(gn.args):
        return False
    return all(_same(a, b) for a, b in zip(pn.args, gn.args))
