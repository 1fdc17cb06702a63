"""Keep broadcast attention masks small.

Current transformers versions build the additive mask of eager attention as
`torch.where(bool_mask.expand(B, -1, S, S), 0.0, finfo.min)`: `where` materialises the expanded [B,1,S,S] matrix
although every query row is identical (33 MB at batch 32, sequence 512, re-read by every head of every layer).
`where(expand(c), x, y)` with scalar x, y equals `expand(where(c, x, y))`, so this pass moves the `expand` below the
`where`; the mask the attention kernel then receives is a stride-0 view of a [B,1,1,S] tensor and is consumed as one
value per key.  No counterpart in the reference, whose BERT graphs carried a [B,1,1,S] mask already.
"""
import operator

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


# Pure, shape-static ops that may be evaluated while compiling when every tensor operand is itself a constant.
_FOLDABLE_FUNCTIONS = {
    torch.arange, torch.ones, torch.zeros, torch.full, torch.tril, torch.triu, torch.where,
    operator.add, operator.sub, operator.mul, operator.and_, operator.or_, operator.getitem,
    operator.ge, operator.gt, operator.le, operator.lt, operator.eq, operator.ne,
    torch.add, torch.sub, torch.mul, torch.bitwise_and, torch.bitwise_or,
    # (the packed-sequence test transformers makes on position ids when no key/value cache is in use: position
    # differences, a running count of restarts, and a comparison of the counts of query and key)
    torch.diff, torch.cumsum, torch.eq, torch.ne,
}
_FOLDABLE_METHODS = {"new_ones", "new_zeros", "to", "expand", "view", "reshape", "unsqueeze", "squeeze", "bool", "long", "int",
                     "cumsum", "diff", "__eq__", "__ne__", "__and__", "__or__", "__ge__", "__gt__", "__le__", "__lt__"}
_FOLD_LIMIT = 1 << 22  # elements


def _fold_constants(gm: torch.fx.GraphModule):
    """node -> tensor value, for nodes computable from literals alone (index grids and the like)."""
    values = {}

    def materialize(arg):
        return torch.fx.node.map_arg(arg, lambda n: values[n])

    for node in gm.graph.nodes:
        if node.op == "get_attr" and str(node.target).startswith("_tensor_constant"):
            # literal tensors the tracer lifted into attributes of the graph module
            const = getattr(gm, node.target, None)
            if isinstance(const, torch.Tensor) and const.numel() <= _FOLD_LIMIT:
                values[node] = const
            continue
        if node.op == "call_function" and node.target in _FOLDABLE_FUNCTIONS:
            pass
        elif node.op == "call_method" and node.target in _FOLDABLE_METHODS:
            pass
        else:
            continue
        if not all(n in values for n in node.all_input_nodes):
            continue
        if node.op == "call_method" and not node.all_input_nodes:
            continue
        try:
            args, kwargs = materialize(node.args), materialize(node.kwargs)
            out = node.target(*args, **kwargs) if node.op == "call_function" else getattr(args[0], node.target)(*args[1:], **kwargs)
        except Exception:
            continue
        if isinstance(out, torch.Tensor) and out.numel() <= _FOLD_LIMIT:
            values[node] = out
    return values


def drop_all_true_conjuncts(gm: torch.fx.GraphModule):
    """`c & x` where `c` folds to an all-True constant is `x` broadcast to the result shape.

    transformers builds attention masks as `mask_function(q_idx, kv_idx) & padding[b, kv_idx]`; for an encoder the
    first conjunct is the constant grid `q_idx >= 0`, whose only effect is to blow the per-key padding mask up to a
    [B,1,S,S] matrix.  Removing it leaves an `expand` of the [B,1,1,S] padding mask."""
    values = _fold_constants(gm)
    changed = False
    for node in list(gm.graph.nodes):
        if node.op != "call_function" or node.target not in (operator.and_, torch.bitwise_and) or len(node.args) != 2:
            continue
        a, b = node.args
        for const, other in ((a, b), (b, a)):
            if not (isinstance(const, Node) and const in values and isinstance(other, Node) and other not in values):
                continue
            cval = values[const]
            if cval.dtype != torch.bool or not bool(cval.all()):
                continue
            other_val = other.meta.get("example_value")
            if other_val is None or other_val.dtype != torch.bool:
                continue
            out_shape = tuple(torch.broadcast_shapes(tuple(cval.shape), tuple(other_val.shape)))
            if not all(isinstance(d, int) for d in out_shape):
                continue
            with gm.graph.inserting_before(node):
                if len(out_shape) == other_val.dim():
                    new = gm.graph.call_method("expand", (other,) + out_shape)
                else:
                    continue
            new.meta["example_value"] = other_val.expand(out_shape)
            node.replace_all_uses_with(new)
            gm.graph.erase_node(node)
            changed = True
            break
    if changed:
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()


def full_range_index_to_view(gm: torch.fx.GraphModule):
    """`x[i0, i1, ...]` with one constant index tensor per dimension of x, each an `arange` over the whole dimension laid
    along an axis of its own (`padding[batch_idx[:, None, None, None], kv_idx[None, None, None, :]]`, what transformers'
    mask builders index the [B, S] padding mask with), is `x` reshaped with those axes in place and ones elsewhere: a view
    instead of two aranges, an addition and a gather launch per forward."""
    values = _fold_constants(gm)
    changed = False
    for node in list(gm.graph.nodes):
        if node.op != "call_function" or node.target is not operator.getitem or len(node.args) != 2:
            continue
        x, index = node.args
        if not (isinstance(x, Node) and isinstance(index, tuple) and index and all(isinstance(i, Node) and i in values for i in index)):
            continue
        xv = x.meta.get("example_value")
        if x in values or not isinstance(xv, torch.Tensor) or xv.dim() != len(index) or not all(isinstance(d, int) for d in xv.shape):
            continue
        idx = [values[i] for i in index]
        rank = max(t.dim() for t in idx)
        if rank == 0 or any(t.dtype not in (torch.int64, torch.int32) for t in idx):
            continue
        target, last_axis, ok = [1] * rank, -1, True
        for k, t in enumerate(idx):
            shape = (1,) * (rank - t.dim()) + tuple(t.shape)
            axes = [a for a, d in enumerate(shape) if d != 1]
            if xv.shape[k] == 1 and not axes:
                axes = [last_axis + 1] if last_axis + 1 < rank else []
            if len(axes) != 1 or axes[0] <= last_axis or shape[axes[0]] != xv.shape[k]:
                ok = False
                break
            if not torch.equal(t.reshape(-1).cpu().long(), torch.arange(xv.shape[k])):
                ok = False
                break
            last_axis = axes[0]
            target[last_axis] = xv.shape[k]
        if not ok:
            continue
        with gm.graph.inserting_before(node):
            view = gm.graph.call_method("reshape", (x,) + tuple(target))
        view.meta["example_value"] = xv.reshape(target)
        node.replace_all_uses_with(view)
        gm.graph.erase_node(node)
        changed = True
    if changed:
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()


def merge_nested_expands(gm: torch.fx.GraphModule):
    """x.expand(s1).expand(s2) -> x.expand(s2) when the ranks agree (keeps stride-0 dims visible to later passes)."""
    changed = False
    for node in list(gm.graph.nodes):
        if not (node.op == "call_method" and node.target == "expand" and not node.kwargs):
            continue
        inner = node.args[0]
        if not (isinstance(inner, Node) and inner.op == "call_method" and inner.target == "expand" and not inner.kwargs):
            continue
        if len(inner.args) != len(node.args) or len(inner.users) != 1:
            continue
        inner_shape, outer_shape = inner.args[1:], node.args[1:]
        if not all(isinstance(d, int) for d in inner_shape + outer_shape):
            continue
        merged = tuple(i if o == -1 else o for i, o in zip(inner_shape, outer_shape))
        node.args = (inner.args[0],) + merged
        changed = True
    if changed:
        gm.graph.eliminate_dead_code()
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


def constant_causal_masks_to_flag(gm: torch.fx.GraphModule):
    """An attention mask that is a compile-time constant and exactly the lower-triangular (causal) pattern is
    dropped in favour of the kernel's `is_causal` flag: no [1,1,S,S] matrix is built, read or added.

    Applies to the fused calls produced by `kernl_amd.optimizer.attention` (run after them).  A boolean mask must
    equal tril; an additive mask must be 0 on and below the diagonal and <= -1e4 above it.  Only square masks
    qualify (the kernel's causal mode is top-left aligned)."""
    from kernl_amd.optimizer.attention import attention_wrapper, sdpa_wrapper

    values = None
    changed = False
    for node in list(gm.graph.nodes):
        if node.op != "call_function" or node.target not in (attention_wrapper, sdpa_wrapper):
            continue
        mask_idx = 6 if node.target is attention_wrapper else 3
        mask = node.args[mask_idx]
        if not isinstance(mask, Node):
            continue
        if values is None:
            values = _fold_constants(gm)
        val = values.get(mask)
        if val is None or val.dim() < 2 or val.shape[-1] != val.shape[-2] or val.shape[-1] < 2:
            continue
        flat = val.reshape(-1, val.shape[-2], val.shape[-1])
        tril = torch.tril(torch.ones(val.shape[-2:], dtype=torch.bool, device=val.device))
        if val.dtype == torch.bool:
            is_causal = bool((flat == tril).all())
        else:
            f = flat.float()
            is_causal = bool(((f == 0) == tril).all()) and bool((f[:, ~tril] <= -1e4).all())
        if not is_causal:
            continue
        args = list(node.args)
        args[mask_idx] = None
        args[5] = True  # is_causal, same position in both wrappers
        node.args = tuple(args)
        changed = True
    if changed:
        gm.graph.eliminate_dead_code()
        gm.graph.lint()
        gm.recompile()
