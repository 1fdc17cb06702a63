"""Sub-graph matching and replacement on torch.fx graphs.

Same contract as the reference's `replace_pattern(gm, pattern, replacement)`
(src/kernl/utils/extended_matcher.py:343-523, itself a fork of torch.fx's subgraph rewriter): every non-overlapping
occurrence of `pattern` in `gm` is replaced by `replacement`, matching on use-def structure rather than on names.
The three behaviours the reference adds on top of stock torch.fx are kept:

  * literal arguments take part in the match (`x / 8.0` does not match `x / 4.0`; reference :112-115 and
    src/kernl/utils/fx.py:21-39);
  * a `call_module` node matches on the TYPE of the module, and the replacement's module nodes are re-pointed to
    the module instance that was matched in `gm` (reference :116-126 and :458-467);
  * `get_attr` nodes of the replacement are resolved the same way (reference :301-308).

This implementation is written from scratch as a small backtracking matcher.  Two extensions the graphs produced by
current PyTorch / transformers need:

  * a pattern placeholder may bind to a LITERAL of the graph (e.g. the softmax scale `0.125`, the LayerNorm eps or
    `normalized_shape`), the replacement then receives that literal — one pattern covers every head size; a
    placeholder whose name starts with `literal_` binds ONLY to literals;
  * `call_function` arguments are compared after normalisation to keyword form, so `softmax(x, dim=-1)` written with
    or without the defaulted `_stacklevel` / `dtype` arguments is the same node.
"""
from typing import Any, Callable, Dict, List, NamedTuple, Optional, Set, Union

import torch
from torch.fx import Graph, GraphModule, Node, symbolic_trace

_IGNORED_KWARGS = {"_stacklevel"}


class Match(NamedTuple):
    # Node of `gm` the match was found from (it produced the pattern's returned value)
    anchor: Node
    # Maps nodes of the pattern graph to nodes of `gm` (placeholders may map to literals)
    nodes_map: Dict[Node, Any]
    # Maps module / attribute names used by the pattern to the names they were matched to in `gm`
    module_map: Dict[str, str]


def _as_graph_module(fn: Union[Callable, torch.nn.Module, GraphModule]) -> GraphModule:
    if isinstance(fn, GraphModule):
        return fn
    return symbolic_trace(fn)


def _normalized(node: Node, root: torch.nn.Module):
    """(args, kwargs) in a canonical form: keyword-only with defaults where torch.fx can work the signature out."""
    if node.op == "call_function":
        try:
            pair = node.normalized_arguments(root, normalize_to_only_use_kwargs=True)
        except Exception:
            pair = None
        if pair is not None:
            return tuple(pair.args), {k: v for k, v in pair.kwargs.items() if k not in _IGNORED_KWARGS}
    return tuple(node.args), {k: v for k, v in node.kwargs.items() if k not in _IGNORED_KWARGS}


class _Matcher:
    def __init__(self, pattern: GraphModule, gm: GraphModule):
        self.pattern, self.gm = pattern, gm
        self.p_modules = dict(pattern.named_modules())
        self.g_modules = dict(gm.named_modules())
        self.p_placeholders = [n for n in pattern.graph.nodes if n.op == "placeholder"]
        self.p_output = next(n for n in pattern.graph.nodes if n.op == "output")
        anchors = self.p_output.args[0]
        self.p_anchors: List[Node] = list(anchors) if isinstance(anchors, (tuple, list)) else [anchors]
        self.p_internal = [n for n in pattern.graph.nodes if n.op not in ("placeholder", "output")]

    # --- node-level compatibility -------------------------------------------------------------------------------
    def _same_target(self, pn: Node, gn: Node, module_map: Dict[str, str]) -> bool:
        if pn.op != gn.op:
            return False
        if pn.op == "call_module":
            p_mod, g_mod = self.p_modules.get(pn.target), self.g_modules.get(gn.target)
            if p_mod is None or g_mod is None or type(p_mod) is not type(g_mod):
                return False
            bound = module_map.get(pn.target)
            if bound is not None and bound != gn.target:
                return False
            module_map[pn.target] = gn.target
            return True
        if pn.op == "get_attr":
            bound = module_map.get(pn.target)
            if bound is not None and bound != gn.target:
                return False
            module_map[pn.target] = gn.target
            return True
        return pn.target == gn.target

    def _match_value(self, pv: Any, gv: Any, nodes_map: Dict[Node, Any], module_map: Dict[str, str]) -> bool:
        if isinstance(pv, Node):
            return self._match_node(pv, gv, nodes_map, module_map)
        if isinstance(gv, Node):
            return False  # literal in the pattern, tensor in the graph
        if isinstance(pv, (tuple, list)):
            if not isinstance(gv, (tuple, list)) or len(pv) != len(gv):
                return False
            return all(self._match_value(a, b, nodes_map, module_map) for a, b in zip(pv, gv))
        if isinstance(pv, dict):
            if not isinstance(gv, dict) or pv.keys() != gv.keys():
                return False
            return all(self._match_value(pv[k], gv[k], nodes_map, module_map) for k in pv)
        if isinstance(pv, slice):
            return isinstance(gv, slice) and (pv.start, pv.stop, pv.step) == (gv.start, gv.stop, gv.step)
        if type(pv) is not type(gv) and not (isinstance(pv, (int, float)) and isinstance(gv, (int, float))):
            return False
        if isinstance(pv, (int, float)) and (isinstance(pv, bool) != isinstance(gv, bool)):
            return False
        try:
            return bool(pv == gv)
        except Exception:
            return False

    def _match_node(self, pn: Node, gv: Any, nodes_map: Dict[Node, Any], module_map: Dict[str, str]) -> bool:
        if pn in nodes_map:
            bound = nodes_map[pn]
            return bound is gv if isinstance(bound, Node) or isinstance(gv, Node) else self._literal_eq(bound, gv)
        if pn.op == "placeholder":
            if str(pn.target).startswith("literal_") and isinstance(gv, Node):
                return False  # this parameter only stands for a python literal
            nodes_map[pn] = gv  # wildcard: a node of the graph, or a literal
            return True
        if not isinstance(gv, Node):
            return False
        gn = gv
        if gn in self._claimed or gn.op in ("placeholder", "output"):
            return False
        if gn in [v for v in nodes_map.values() if isinstance(v, Node)]:
            return False  # one graph node cannot play two pattern roles
        if not self._same_target(pn, gn, module_map):
            return False
        p_args, p_kwargs = _normalized(pn, self.pattern)
        g_args, g_kwargs = _normalized(gn, self.gm)
        if len(p_args) != len(g_args) or p_kwargs.keys() != g_kwargs.keys():
            return False
        nodes_map[pn] = gn
        for a, b in zip(p_args, g_args):
            if not self._match_value(a, b, nodes_map, module_map):
                return False
        for key in p_kwargs:
            if not self._match_value(p_kwargs[key], g_kwargs[key], nodes_map, module_map):
                return False
        return True

    @staticmethod
    def _literal_eq(a: Any, b: Any) -> bool:
        try:
            return type(a) is type(b) and bool(a == b)
        except Exception:
            return False

    # --- whole-pattern match anchored at one graph node ----------------------------------------------------------
    def _try_anchor(self, gn: Node) -> Optional[Match]:
        if len(self.p_anchors) != 1:
            return None  # patterns here return a single value
        nodes_map: Dict[Node, Any] = {}
        module_map: Dict[str, str] = {}
        if not self._match_node(self.p_anchors[0], gn, nodes_map, module_map):
            return None
        if any(pn not in nodes_map for pn in self.p_internal):
            return None  # dead code in the pattern: nothing sensible to do
        if any(ph not in nodes_map for ph in self.p_placeholders):
            return None
        # values computed inside the match must not be needed outside of it, except the returned one
        matched: Set[Node] = {nodes_map[pn] for pn in self.p_internal}
        for pn in self.p_internal:
            g = nodes_map[pn]
            if pn in self.p_anchors:
                continue
            if any(user not in matched for user in g.users):
                return None
        return Match(anchor=gn, nodes_map=nodes_map, module_map=module_map)

    def find_all(self) -> List[Match]:
        self._claimed: Set[Node] = set()
        matches: List[Match] = []
        for gn in list(self.gm.graph.nodes):
            if gn.op in ("placeholder", "output") or gn in self._claimed:
                continue
            m = self._try_anchor(gn)
            if m is None:
                continue
            matches.append(m)
            self._claimed.update(m.nodes_map[pn] for pn in self.p_internal)
        return matches


def _copy_missing_attrs(gm: GraphModule, replacement: GraphModule, target: str) -> None:
    """Make `target` (a module path or attribute path used by the replacement) resolvable on `gm`."""
    obj: Any = gm
    for part in target.split("."):
        if not hasattr(obj, part):
            break
        obj = getattr(obj, part)
    else:
        return  # already there: the graph's own object wins
    src: Any = replacement
    for part in target.split("."):
        src = getattr(src, part)
    if isinstance(src, torch.nn.Module):
        gm.add_submodule(target, src)
    else:
        owner: Any = gm
        parts = target.split(".")
        for part in parts[:-1]:
            if not hasattr(owner, part):
                owner.add_module(part, torch.nn.Module())
            owner = getattr(owner, part)
        setattr(owner, parts[-1], src)


def replace_pattern(
    gm: GraphModule,
    pattern: Union[Callable, torch.nn.Module, GraphModule],
    replacement: Union[Callable, torch.nn.Module, GraphModule],
) -> List[Match]:
    """Replace every non-overlapping occurrence of `pattern` in `gm` by `replacement`; returns the matches.

    `pattern` and `replacement` take the same parameters, in the same order; both are symbolically traced.  Module
    attributes the replacement uses under the same name as the pattern (`self.linear`) are re-pointed to the module
    the pattern matched in `gm`.
    """
    pattern_gm = _as_graph_module(pattern)
    replacement_gm = _as_graph_module(replacement)
    matcher = _Matcher(pattern_gm, gm)
    matches = matcher.find_all()
    if not matches:
        return matches

    r_placeholders = [n for n in replacement_gm.graph.nodes if n.op == "placeholder"]
    assert len(r_placeholders) == len(matcher.p_placeholders), "pattern and replacement must take the same parameters"
    graph: Graph = gm.graph
    order = {n: i for i, n in enumerate(graph.nodes)}
    replaced: Dict[Node, Node] = {}  # anchors of earlier matches -> the node that now stands for them

    for m in matches:
        def live(v: Any) -> Any:
            while isinstance(v, Node) and v in replaced:
                v = replaced[v]
            return v

        val_map: Dict[Node, Any] = {}
        for rp, pp in zip(r_placeholders, matcher.p_placeholders):
            val_map[rp] = live(m.nodes_map[pp])
        matched_nodes = [m.nodes_map[pn] for pn in matcher.p_internal]
        last = max(matched_nodes, key=lambda n: order[n])

        new_out: Any = None
        with graph.inserting_before(last):
            for rn in replacement_gm.graph.nodes:
                if rn.op == "placeholder":
                    continue
                if rn.op == "output":
                    new_out = torch.fx.node.map_arg(rn.args[0], lambda n: val_map[n])
                    continue
                copied = graph.node_copy(rn, lambda n: val_map[n])
                if rn.op in ("call_module", "get_attr"):
                    head = rn.target.split(".")[0]
                    if rn.target in m.module_map:
                        copied.target = m.module_map[rn.target]
                    elif head in m.module_map:
                        copied.target = m.module_map[head] + rn.target[len(head):]
                    else:
                        _copy_missing_attrs(gm, replacement_gm, rn.target)
                val_map[rn] = copied
        assert isinstance(new_out, Node), "replacement must return a single tensor value"
        m.anchor.replace_all_uses_with(new_out)
        replaced[m.anchor] = new_out
        for n in sorted(matched_nodes, key=lambda n: order[n], reverse=True):
            if len(n.users) == 0:
                graph.erase_node(n)

    graph.lint()
    gm.recompile()
    return matches
