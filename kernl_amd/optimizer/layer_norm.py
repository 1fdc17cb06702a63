"""LayerNorm / RMSNorm graph patterns (reference: src/kernl/optimizer/layer_norm.py:22-74).

Module-form patterns are the reference's.  The functional forms are what torch.compile hands to a backend today
(`F.layer_norm(x, shape, weight, bias, eps)` on lifted parameters); eps and the RMSNorm epsilon are wildcards bound to
the graph's literal, so a Llama norm with eps 1e-5 matches as well as T5's 1e-6.  A LayerNorm whose input is
`a + b` with no other consumer is rewritten to the fused add+LayerNorm kernel.
"""
import torch

from kernl_amd.implementations.layer_norm import add_layer_norm, layer_norm
from kernl_amd.utils.extended_matcher import replace_pattern


def _half_params_once(v: torch.Tensor, *params) -> None:
    # one-time in-place down-cast, as the reference does (optimizer/layer_norm.py:24-27)
    if v.dtype == torch.float16 or torch.is_autocast_enabled("cuda"):
        for p in params:
            if p is not None and p.dtype == torch.float32:
                p.data = p.data.half()


def layer_norm_wrapper(v: torch.Tensor, layernorm: torch.nn.LayerNorm):
    _half_params_once(v, layernorm.weight, layernorm.bias)
    return layer_norm(v, layernorm.weight, layernorm.bias, layernorm.eps)


_unit_weights = {}


def _flat_affine(v: torch.Tensor, normalized_shape, weight, bias):
    """F.layer_norm over the last len(normalized_shape) dimensions is a LayerNorm over their flattening; a missing
    weight is a weight of ones (kept per size, dtype and device: built once, before graph capture)."""
    n = 1
    for d in normalized_shape:
        n *= int(d)
    if weight is None:
        key = (n, v.dtype, v.device)
        if key not in _unit_weights:
            _unit_weights[key] = torch.ones(n, dtype=v.dtype, device=v.device)
        weight = _unit_weights[key]
    lead = v.shape[: v.dim() - len(normalized_shape)]
    return lead, n, weight.reshape(n), None if bias is None else bias.reshape(n)


def layer_norm_wrapper_functional(v: torch.Tensor, normalized_shape, weight, bias, eps: float):
    _half_params_once(v, weight, bias)
    if len(normalized_shape) == 1 and weight is not None:
        return layer_norm(v, weight, bias, eps)
    lead, n, w, b = _flat_affine(v, normalized_shape, weight, bias)
    return layer_norm(v.reshape(*lead, n), w, b, eps).reshape(v.shape)


def add_layer_norm_wrapper_functional(a: torch.Tensor, b: torch.Tensor, normalized_shape, weight, bias, eps: float):
    if not isinstance(a, torch.Tensor) or not isinstance(b, torch.Tensor) or a.shape != b.shape or a.dtype != b.dtype:
        # a python scalar (on either side) or a broadcast operand: add first (one element-wise kernel), then the
        # LayerNorm kernel, which also casts the parameters once to the dtype of the sum
        return layer_norm_wrapper_functional(a + b, normalized_shape, weight, bias, eps)
    _half_params_once(a, weight, bias)
    if len(normalized_shape) == 1 and weight is not None:
        return add_layer_norm(a, b, weight, bias, eps)
    lead, n, w, bb = _flat_affine(a, normalized_shape, weight, bias)
    return add_layer_norm(a.reshape(*lead, n), b.reshape(*lead, n), w, bb, eps).reshape(a.shape)


def layer_norm_rms_wrapper(v: torch.Tensor, weight: torch.Tensor, eps: float):
    if weight.dtype != v.dtype:
        weight = weight.to(v.dtype)
    return layer_norm(v, weight, None, eps, None, use_rms_norm=True)


def embedding_layer_norm_wrapper(ids0, table0, ids1, table1, ids2, table2, normalized_shape, weight, bias, eps: float):
    """layer_norm((embedding(ids0, table0) + embedding(ids1, table1)) + embedding(ids2, table2)) — the third pair may be
    None — as one launch where the kernel takes the operands (`embedding_layer_norm`), as the lookups, additions and the
    LayerNorm kernel they were otherwise."""
    from kernl_amd.implementations.layer_norm import embedding_layer_norm, embedding_layer_norm_supported

    pairs = [(i, t) for i, t in ((ids0, table0), (ids1, table1), (ids2, table2)) if t is not None]
    tables, ids = [t for _, t in pairs], [i for i, _ in pairs]
    if all(t.dtype == torch.float16 for t in tables):
        _half_params_once(tables[0], weight, bias)
    if len(normalized_shape) == 1 and not torch.is_autocast_enabled("cuda") and embedding_layer_norm_supported(tables, ids, weight, bias):
        return embedding_layer_norm(tables, ids, weight, bias, eps)
    total = torch.nn.functional.embedding(ids[0], tables[0])
    for i, t in zip(ids[1:-1], tables[1:-1]):
        total = total + torch.nn.functional.embedding(i, t)
    return add_layer_norm_wrapper_functional(total, torch.nn.functional.embedding(ids[-1], tables[-1]), normalized_shape, weight, bias, eps)


torch.fx.wrap("embedding_layer_norm_wrapper")
torch.fx.wrap("layer_norm_wrapper")
torch.fx.wrap("layer_norm_wrapper_functional")
torch.fx.wrap("add_layer_norm_wrapper_functional")
torch.fx.wrap("layer_norm_rms_wrapper")


def replace_layer_norm(gm: torch.fx.GraphModule):
    class Pattern(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.layernorm = torch.nn.LayerNorm((1, 1))

        def forward(self, v):
            return self.layernorm(v)

    class Replacement(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.layernorm = torch.nn.LayerNorm((1, 1))

        def forward(self, v):
            return layer_norm_wrapper(v, self.layernorm)

    replace_pattern(gm, Pattern(), Replacement())


def replace_layer_norm_fn(gm: torch.fx.GraphModule):
    def pattern_add(a, b, literal_shape, weight, bias, literal_eps):
        return torch.nn.functional.layer_norm(a + b, literal_shape, weight, bias, literal_eps)

    def replace_add(a, b, literal_shape, weight, bias, literal_eps):
        return add_layer_norm_wrapper_functional(a, b, literal_shape, weight, bias, literal_eps)

    def pattern(v, literal_shape, weight, bias, literal_eps):
        return torch.nn.functional.layer_norm(v, literal_shape, weight, bias, literal_eps)

    def replace(v, literal_shape, weight, bias, literal_eps):
        return layer_norm_wrapper_functional(v, literal_shape, weight, bias, literal_eps)

    replace_pattern(gm, pattern_add, replace_add)
    replace_pattern(gm, pattern, replace)


def replace_layer_norm_rms(gm: torch.fx.GraphModule):
    # T5 spelling (reference pattern, eps generalised from the literal 1e-06)
    def pattern(v, weight, literal_eps):
        mean_square = v.to(torch.float32).pow(2).mean(-1, keepdim=True)
        return weight * (v * torch.rsqrt(mean_square + literal_eps))

    def replace(v, weight, literal_eps):
        return layer_norm_rms_wrapper(v, weight, literal_eps)

    replace_pattern(gm, pattern, replace)

    # Llama spelling: normalise the fp32 copy, cast back to the input dtype, then scale
    for dtype in (torch.float16, torch.bfloat16, torch.float32):

        def make(dtype):
            def pattern_llama(v, weight, literal_eps):
                h = v.to(torch.float32)
                variance = h.pow(2).mean(-1, keepdim=True)
                h2 = h * torch.rsqrt(variance + literal_eps)
                return weight * h2.to(dtype)

            return pattern_llama

        replace_pattern(gm, make(dtype), replace)


def fuse_embeddings_into_layer_norm(gm: torch.fx.GraphModule):
    """`add_layer_norm_wrapper_functional(embedding(i0, t0) + embedding(i1, t1), embedding(i2, t2), ...)` — or two lookups —
    becomes one `embedding_layer_norm_wrapper` call (BertEmbeddings: word + token type, + position, LayerNorm).  Only sums
    taken left to right are rewritten (the kernel adds in that order, rounding after each addition as the model does), and
    only lookups and partial sums nothing else reads.  Runs after the LayerNorm passes."""
    import operator

    def lookup(n):
        if not (isinstance(n, torch.fx.Node) and n.op == "call_function" and n.target is torch.nn.functional.embedding and len(n.users) == 1):
            return None
        args = list(n.args) + [None] * 7
        max_norm = n.kwargs.get("max_norm", args[3])
        if max_norm is not None or len(n.args) < 2:
            return None
        return (n.args[0], n.args[1])

    changed = False
    for node in list(gm.graph.nodes):
        if not (node.op == "call_function" and node.target is add_layer_norm_wrapper_functional and len(node.args) == 6 and not node.kwargs):
            continue
        a, b = node.args[:2]
        last = lookup(b)
        if last is None:
            continue
        first = lookup(a)
        if first is not None:
            pairs = [first, last]
        elif (isinstance(a, torch.fx.Node) and a.op == "call_function" and a.target in (operator.add, torch.add) and len(a.args) == 2
              and not a.kwargs and len(a.users) == 1 and lookup(a.args[0]) is not None and lookup(a.args[1]) is not None):
            pairs = [lookup(a.args[0]), lookup(a.args[1]), last]
        else:
            continue
        flat = [x for pair in pairs for x in pair] + [None, None] * (3 - len(pairs))
        with gm.graph.inserting_before(node):
            fused = gm.graph.call_function(embedding_layer_norm_wrapper, tuple(flat) + tuple(node.args[2:]))
        node.replace_all_uses_with(fused)
        gm.graph.erase_node(node)
        changed = True
    if changed:
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()
