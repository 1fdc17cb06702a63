"""Linear-layer graph patterns (reference: src/kernl/optimizer/linear.py:24-115).

`linear_wrapper` (module form) and `linear_wrapper_functional` are the fx leaves the rewritten graph calls.  Fused
activation patterns run before the bare ones, as in the reference (:109-115).  torch.compile now hands `nn.Linear`
to a backend as `F.linear(x, weight, bias)` on lifted parameters, so the functional patterns carry the same set of
activations as the module ones.
"""
from typing import Callable

import torch

from kernl_amd.implementations.linear_layer import GLU_BLOCK, interleave_glu_rows, linear_glu_layer, linear_layer
from kernl_amd.utils.extended_matcher import replace_pattern


def linear_wrapper(v: torch.Tensor, linear: torch.nn.Linear, activation=""):
    return linear_wrapper_functional(v, linear.weight, linear.bias, activation=activation)


torch.fx.wrap("linear_wrapper")


def linear_wrapper_functional(v: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, activation=""):
    # One-time, in-place down-cast of fp32 parameters so they are not converted on every call
    # (reference: optimizer/linear.py:33-36).  Only when the activations already are fp16 or autocast will make them so.
    if weight.dtype == torch.float32 and (v.dtype == torch.float16 or torch.is_autocast_enabled("cuda")):
        weight.data = weight.data.half()
    if bias is not None and bias.dtype == torch.float32 and (v.dtype == torch.float16 or torch.is_autocast_enabled("cuda")):
        bias.data = bias.data.half()
    if not weight.is_contiguous():
        weight = weight.contiguous()
    return linear_layer(v, weight, bias, activation=activation)


torch.fx.wrap("linear_wrapper_functional")


def replace_linear_activation(gm: torch.fx.GraphModule, activation_module: Callable, activation: str):
    class Pattern(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.linear = torch.nn.Linear(1, 1)
            self.activation = activation_module

        def forward(self, v):
            return self.activation(self.linear(v))

    class Replacement(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.linear = torch.nn.Linear(1, 1)
            self.activation = activation_module

        def forward(self, v):
            return linear_wrapper(v, self.linear, activation=activation)

    replace_pattern(gm, Pattern(), Replacement())


def replace_linear(gm: torch.fx.GraphModule):
    class Pattern(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.linear = torch.nn.Linear(1, 1)

        def forward(self, v):
            return self.linear(v)

    class Replacement(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.linear = torch.nn.Linear(1, 1)

        def forward(self, v):
            return linear_wrapper(v, self.linear)

    replace_pattern(gm, Pattern(), Replacement())


def _functional_activation_patterns():
    F = torch.nn.functional
    return (
        (lambda t: F.gelu(t), "gelu"),
        (lambda t: F.gelu(t, approximate="tanh"), "fast_gelu"),
        (lambda t: torch.tanh(t), "tanh"),
        (lambda t: F.tanh(t), "tanh"),
        (lambda t: t.tanh(), "tanh"),
        (lambda t: F.relu(t), "relu"),
        (lambda t: torch.relu(t), "relu"),
        (lambda t: F.silu(t), "silu"),
    )


def replace_linear_fn_activation(gm: torch.fx.GraphModule):
    """activation(F.linear(v, weight, bias)) -> one fused call.  `bias` also binds to the literal None."""
    for act_fn, name in _functional_activation_patterns():

        def make(act_fn, name):
            def pattern(v, weight, bias):
                return act_fn(torch.nn.functional.linear(v, weight, bias))

            def replace(v, weight, bias):
                return linear_wrapper_functional(v, weight, bias, activation=name)

            return pattern, replace

        pat, rep = make(act_fn, name)
        replace_pattern(gm, pat, rep)


def replace_linear_fn(gm: torch.fx.GraphModule):
    def pattern(v, weight, bias):
        return torch.nn.functional.linear(v, weight, bias)

    def replace(v, weight, bias):
        output = linear_wrapper_functional(v, weight, bias)
        return output

    replace_pattern(gm, pattern, replace)


def replace_linear_fn_constant_match(gm: torch.fx.GraphModule):
    """F.linear(v, weight, None) spelled with a literal None (reference: optimizer/linear.py:97-106).  The wildcard
    `bias` of `replace_linear_fn` already binds to None; kept so the reference's pass list maps one to one."""

    def pattern(v, weight):
        return torch.nn.functional.linear(v, weight, None)

    def replace(v, weight):
        output = linear_wrapper_functional(v, weight, None)
        return output

    replace_pattern(gm, pattern, replace)


class _DerivedParams:
    """Tensors derived from a group of parameters (concatenated or interleaved weights), kept for as long as the
    parameters they were made from are alive and stay where they are.

    Two kinds of entry:

    * aliased — the derived tensor IS the parameters' memory: after the concatenation every original is re-pointed at
      its slice of the fused buffer, so any in-place update of a parameter (optimizer step, `load_state_dict`,
      `w.data.copy_(...)`) lands in the fused buffer, in eager calls and under hipGraph replays alike;
    * copied — the derived tensor is a separate arrangement of the values (block-interleaved gate / value rows, which
      no strided view of the originals can express).  Its entry remembers the originals' version counters; a lookup
      that finds them changed rebuilds the derived tensor IN PLACE, so graphs captured on its address stay valid.
      Writes that bypass the version counter (`w.data.copy_(...)`) need `refresh_fused_parameters()`.

    The key is the originals' storage addresses and dtypes; an address alone is not an identity — once a model is
    freed the allocator hands the same addresses to the next one — so every entry also holds weak references to the
    original tensors and is dropped as soon as one of them has died or moved."""

    class _Entry:
        __slots__ = ("refs", "value", "versions", "rebuild")

        def __init__(self, refs, value, versions, rebuild):
            self.refs, self.value, self.versions, self.rebuild = refs, value, versions, rebuild

    def __init__(self):
        self._entries = {}

    @staticmethod
    def key_of(params):
        return tuple((0, None) if p is None else (p.data_ptr(), p.dtype) for p in params)

    @staticmethod
    def _versions(params):
        return tuple(-1 if p is None else p._version for p in params)

    def get(self, params):
        key = self.key_of(params)
        entry = self._entries.get(key)
        if entry is None:
            return None
        originals = []
        for ref, p in zip(entry.refs, params):
            if p is None:
                originals.append(None)
                continue
            alive = ref()
            # the tensor passed in may be an alias of the original (same storage); what matters is that the original
            # still owns that memory
            if alive is None or alive.data_ptr() != p.data_ptr():
                del self._entries[key]
                return None
            originals.append(alive)
        if entry.rebuild is not None:
            versions = self._versions(originals)
            if versions != entry.versions:
                entry.rebuild(entry.value, originals)
                entry.versions = versions
        return entry.value

    def put(self, params, value, rebuild=None):
        """`rebuild(value, originals)` rewrites `value` in place from the originals; None for aliased entries."""
        import weakref

        self._drop_dead()
        refs = [None if p is None else weakref.ref(p) for p in params]
        self._entries[self.key_of(params)] = self._Entry(refs, value, self._versions(params), rebuild)

    def _drop_dead(self):
        self._entries = {
            k: e for k, e in self._entries.items() if all(r is None or r() is not None for r in e.refs)
        }

    def refresh(self, only_changed: bool) -> int:
        """Rebuild copied entries in place from their live originals; returns how many were rebuilt.  With
        `only_changed` this is the check in front of every graph replay: a walk over the copied entries that compares
        version counters and touches nothing else."""
        if not only_changed:
            self._drop_dead()
        n = 0
        for entry in self._entries.values():
            if entry.rebuild is None:
                continue
            originals = [None if r is None else r() for r in entry.refs]
            if any(o is None and r is not None for o, r in zip(originals, entry.refs)):
                continue  # an original has died: the entry goes with the next sweep
            versions = self._versions(originals)
            if only_changed and versions == entry.versions:
                continue
            entry.rebuild(entry.value, originals)
            entry.versions = versions
            n += 1
        return n

    def __len__(self):
        return len(self._entries)


# concatenated / interleaved parameters of fused projections
_fused_params = _DerivedParams()


def refresh_fused_parameters(only_changed: bool = False) -> int:
    """Re-derive, in place, every fused weight that is a re-arranged COPY of model parameters (the block-interleaved
    gate / value weights of gated feed-forward layers) and return how many were rewritten.

    Concatenated query / key / value weights need no refresh: the parameters alias the fused buffer.  Copied ones are
    refreshed by themselves whenever a parameter's version counter has moved (optimizer steps, `load_state_dict`,
    `param.copy_()`), in eager calls and before every hipGraph replay; call this after writes the counter does not
    see (`param.data.copy_(...)`, `param.data.mul_(...)`).  Re-assigning `param.data` to new memory is not supported
    under a captured graph, as for any other parameter: the graph keeps reading the old address."""
    return _fused_params.refresh(only_changed)


def fused_linear_wrapper(v: torch.Tensor, weights, biases):
    """Several activation-free linears of the SAME input (BERT's query/key/value projections) as ONE GEMM against
    the row-concatenated weights; returns the outputs as column slices of the single result.

    The concatenated weight is built on the first call (the warm-up call that precedes graph capture) and kept for as
    long as the original parameters live unchanged, so capture and replays neither allocate nor copy.  No counterpart in the
    reference, which launches one Triton GEMM per projection."""
    weight, bias, sizes = _concatenated_params(v, weights, biases)
    out = linear_layer(v, weight, bias, activation="")
    return tuple(torch.split(out, sizes, dim=-1))


def _concatenated_params(v: torch.Tensor, weights, biases):
    """Row-concatenated weight (and bias) of sibling projections, built once per group of parameters.  The originals
    are re-pointed at their slices of the fused buffers, so there is ONE copy of the values and updates of a
    parameter are updates of the fused weight."""
    originals = tuple(weights) + tuple(biases)
    cached = _fused_params.get(originals)
    if cached is None:
        for w, b in zip(weights, biases):
            # same one-time down-cast as linear_wrapper_functional
            if w.dtype == torch.float32 and (v.dtype == torch.float16 or torch.is_autocast_enabled("cuda")):
                w.data = w.data.half()
            if b is not None and b.dtype == torch.float32 and (v.dtype == torch.float16 or torch.is_autocast_enabled("cuda")):
                b.data = b.data.half()
        sizes = [w.shape[0] for w in weights]
        weight = torch.cat([w.detach() for w in weights], dim=0).contiguous()
        bias = None
        if any(b is not None for b in biases):
            bias = torch.cat(
                [torch.zeros(w.shape[0], dtype=w.dtype, device=w.device) if b is None else b.detach() for w, b in zip(weights, biases)]
            ).contiguous()
        cached = (weight, bias, sizes)
        if any(_is_view_of_larger_storage(p) for p in originals):
            # Some parameter is already a slice of a larger buffer — the fused weight of ANOTHER group it belongs to
            # (tied or shared projections), or a flat parameter buffer.  Re-pointing it a second time would move it out
            # of the first group's buffer, whose entry would then be dropped and its memory freed under graphs that
            # still read it.  This group keeps a copy instead, rewritten in place when a parameter's version moves.
            _fused_params.put(originals, cached, rebuild=_rebuild_concatenated)
        else:
            row = 0
            for w, b, n in zip(weights, biases, sizes):
                w.data = weight[row : row + n]
                if b is not None:
                    b.data = bias[row : row + n]
                row += n
            _fused_params.put(originals, cached)  # keyed by the addresses the parameters now have inside the fused buffers
    return cached


def _is_view_of_larger_storage(p) -> bool:
    return p is not None and p.untyped_storage().nbytes() != p.numel() * p.element_size()


def _rebuild_concatenated(value, originals):
    """In-place refresh of a COPIED concatenation (see `_concatenated_params`) from its live parameters."""
    weight, bias, sizes = value
    count = len(sizes)
    row = 0
    for w, b, n in zip(originals[:count], originals[count:], sizes):
        weight[row : row + n].copy_(w.detach())
        if bias is not None:
            if b is None:
                bias[row : row + n].zero_()
            else:
                bias[row : row + n].copy_(b.detach())
        row += n


torch.fx.wrap("fused_linear_wrapper")


def fuse_sibling_linears(gm: torch.fx.GraphModule):
    """`linear_wrapper_functional(v, w_i, b_i)` calls without activation that share the input `v` and whose weights
    are graph inputs or attributes (i.e. parameters, not computed tensors) become one `fused_linear_wrapper` call."""
    import operator

    groups = {}
    for node in gm.graph.nodes:
        if node.op != "call_function" or node.target is not linear_wrapper_functional:
            continue
        if node.kwargs.get("activation", "") != "" or len(node.args) != 3:
            continue
        v, w, b = node.args
        if not isinstance(v, torch.fx.Node) or not isinstance(w, torch.fx.Node) or w.op not in ("placeholder", "get_attr"):
            continue
        if b is not None and not (isinstance(b, torch.fx.Node) and b.op in ("placeholder", "get_attr")):
            continue
        shape = getattr(w.meta.get("example_value"), "shape", None)
        groups.setdefault((v, None if shape is None else tuple(shape[1:])), []).append(node)
    changed = False
    for (v, _), nodes in groups.items():
        if len(nodes) < 2:
            continue
        first = nodes[0]
        with gm.graph.inserting_before(first):
            fused = gm.graph.call_function(
                fused_linear_wrapper, (v, [n.args[1] for n in nodes], [n.args[2] for n in nodes])
            )
            parts = [gm.graph.call_function(operator.getitem, (fused, i)) for i in range(len(nodes))]
        for n, part in zip(nodes, parts):
            n.replace_all_uses_with(part)
            gm.graph.erase_node(n)
        changed = True
    if changed:
        gm.graph.lint()
        gm.recompile()


def glu_linear_wrapper(v: torch.Tensor, w_gate, b_gate, w_value, b_value, activation: str):
    """activation(linear(v, w_gate, b_gate)) * linear(v, w_value, b_value) as one GEMM with a gated epilogue: the
    feed-forward entry of SwiGLU / GeGLU decoders (reference: `kernel_ff`,
    experimental/llama-v2/kernel/fused_kernel_ff.py:82-117).

    The block-interleaved weight the kernel takes is built on the first call (before graph capture) and cached like
    the fused sibling projections above.  Shapes or dtypes the gated kernel does not cover run as the two fused
    linears and the multiplication they were in the original graph."""
    usable, half = _glu_usable(v, w_gate, b_gate, w_value, b_value)
    if not usable:
        gate = linear_wrapper_functional(v, w_gate, b_gate, activation=activation)
        return gate * linear_wrapper_functional(v, w_value, b_value)
    weight, bias = _interleaved_params(half, w_gate, b_gate, w_value, b_value)
    return linear_glu_layer(v, weight, bias, activation=activation)


def _glu_usable(v: torch.Tensor, w_gate, b_gate, w_value, b_value):
    half = v.dtype == torch.float16 or torch.is_autocast_enabled("cuda")
    dtype = torch.float16 if half else v.dtype
    usable = (
        dtype in (torch.float16, torch.bfloat16)
        and w_gate.shape == w_value.shape
        and w_gate.shape[0] % GLU_BLOCK == 0
        and w_gate.shape[1] % 8 == 0
        and (b_gate is None) == (b_value is None)
    )
    return usable, half


def _interleaved_params(half: bool, w_gate, b_gate, w_value, b_value):
    """Block-interleaved weight (and bias) of a gated linear unit, built once per group of parameters and rewritten in
    place when the parameters' version counters move."""
    params = (w_gate, w_value) + (() if b_gate is None else (b_gate, b_value))
    cached = _fused_params.get(params)
    if cached is None:
        for p in params:
            if p.dtype == torch.float32 and half:
                p.data = p.data.half()
        weight = interleave_glu_rows(w_gate.detach(), w_value.detach())
        bias = None if b_gate is None else interleave_glu_rows(b_gate.detach(), b_value.detach())
        cached = (weight, bias)

        def rebuild(value, originals):
            value[0].copy_(interleave_glu_rows(originals[0].detach(), originals[1].detach()))
            if value[1] is not None:
                value[1].copy_(interleave_glu_rows(originals[2].detach(), originals[3].detach()))

        _fused_params.put(params, cached, rebuild)
    return cached


torch.fx.wrap("glu_linear_wrapper")

_GLU_ACTIVATIONS = ("silu", "gelu", "fast_gelu", "relu", "tanh")


def fuse_gated_linears(gm: torch.fx.GraphModule):
    """`linear(v, w_gate, activation=act) * linear(v, w_value)` — both products consumed only by the multiplication,
    the same input, parameters as weights — becomes one `glu_linear_wrapper` call."""
    import operator

    def is_param(n):
        return n is None or (isinstance(n, torch.fx.Node) and n.op in ("placeholder", "get_attr"))

    def as_linear(n, want_activation):
        if not (isinstance(n, torch.fx.Node) and n.op == "call_function" and n.target is linear_wrapper_functional):
            return None
        if len(n.args) != 3 or len(n.users) != 1 or set(n.kwargs) - {"activation"}:
            return None
        act = n.kwargs.get("activation", "")
        if (act in _GLU_ACTIVATIONS) != want_activation or (not want_activation and act != ""):
            return None
        v, w, b = n.args
        if not isinstance(v, torch.fx.Node) or w is None or not is_param(w) or not is_param(b):
            return None
        return v, w, b, act

    changed = False
    for node in list(gm.graph.nodes):
        if not (node.op == "call_function" and node.target in (operator.mul, torch.mul) and len(node.args) == 2 and not node.kwargs):
            continue
        for gate_n, value_n in (node.args, node.args[::-1]):
            gate, value = as_linear(gate_n, True), as_linear(value_n, False)
            if gate is None or value is None or gate[0] is not value[0] or gate_n is value_n:
                continue
            with gm.graph.inserting_before(node):
                fused = gm.graph.call_function(
                    glu_linear_wrapper, (gate[0], gate[1], gate[2], value[1], value[2], gate[3])
                )
            fused.meta = dict(node.meta)
            node.replace_all_uses_with(fused)
            gm.graph.erase_node(node)
            gm.graph.erase_node(gate_n)
            gm.graph.erase_node(value_n)
            changed = True
            break
    if changed:
        gm.graph.lint()
        gm.recompile()


# ---------------------------------------------------------------------------------------------------------------------
# RMSNorm fused into the projections that consume it (decoding steps)
# ---------------------------------------------------------------------------------------------------------------------
def _rms_fusable(x: torch.Tensor, rms_weight: torch.Tensor) -> bool:
    """The fused kernel takes at most 64 rows of 16-bit x with K a multiple of 64; more rows are normalised once by
    the RMSNorm kernel instead of once per workgroup."""
    rows = x.numel() // x.shape[-1] if x.numel() else 0
    return (
        x.is_cuda
        and x.dtype in (torch.float16, torch.bfloat16)
        and 0 < rows <= 64
        and x.shape[-1] % 64 == 0
        and rms_weight.shape == (x.shape[-1],)
    )


def _rms_weight_like(x: torch.Tensor, rms_weight: torch.Tensor) -> torch.Tensor:
    if rms_weight.dtype == torch.float32 and x.dtype == torch.float16:
        rms_weight.data = rms_weight.data.half()  # one-time, as for the other parameters
    return rms_weight if rms_weight.dtype == x.dtype else rms_weight.to(x.dtype)


RMS_PROMPT_FOLDING = True   # tuning hook: False keeps prompts on the RMSNorm kernel followed by the plain products
WIDE_RESIDUAL_EPILOGUE = True   # tuning hook: False keeps `residual + linear(...)` of many rows as product and addition


def _rms_prompt_foldable(x: torch.Tensor, rms_weight: torch.Tensor) -> bool:
    """Prompts: more rows than the few-row kernels take, 16-bit, no autocast — the norm is folded into the weight and
    the row statistics into the product's epilogue (`rms_linear_layer` decides whether the shape runs that way)."""
    from kernl_amd.implementations.linear_layer import FEW_ROW_MAX_ROWS

    rows = x.numel() // x.shape[-1] if x.numel() else 0
    return (
        RMS_PROMPT_FOLDING
        and x.is_cuda
        and x.dtype in (torch.float16, torch.bfloat16)
        and rows > FEW_ROW_MAX_ROWS
        and x.shape[-1] % 8 == 0
        and rms_weight.shape == (x.shape[-1],)
        and not torch.is_autocast_enabled("cuda")
    )


def _folded(weight: torch.Tensor, rms_weight: torch.Tensor) -> torch.Tensor:
    # the product is formed in fp32 and rounded once
    return (weight.float() * rms_weight.float()[None, :]).to(weight.dtype)


def _folded_weight(weight: torch.Tensor, rms_weight: torch.Tensor) -> torch.Tensor:
    """weight * rms_weight[None, :] of ONE parameter (a copy, rewritten in place when either version counter moves)."""
    params = (weight, rms_weight)
    cached = _fused_params.get(params)
    if cached is None:
        cached = _folded(weight.detach(), rms_weight.detach()).contiguous()
        _fused_params.put(params, cached, lambda value, originals: value.copy_(_folded(originals[0].detach(), originals[1].detach())))
    return cached


def _folded_concatenated_weight(weights, rms_weight: torch.Tensor) -> torch.Tensor:
    """Row-concatenated weights of sibling projections with the norm's weight multiplied into their columns: a second
    copy beside the concatenation the parameters alias (which decoding steps keep using), rewritten in place when a
    version counter moves."""
    params = tuple(weights) + (rms_weight,)
    cached = _fused_params.get(params)
    if cached is None:
        def build(originals):
            return _folded(torch.cat([w.detach() for w in originals[:-1]], dim=0), originals[-1].detach())

        cached = build(params).contiguous()
        _fused_params.put(params, cached, lambda value, originals: value.copy_(build(originals)))
    return cached


def _folded_interleaved_params(half: bool, w_gate, b_gate, w_value, b_value, rms_weight: torch.Tensor):
    """`_interleaved_params` with the norm's weight multiplied into the columns of both weights."""
    params = (w_gate, w_value, rms_weight) + (() if b_gate is None else (b_gate, b_value))
    cached = _fused_params.get(params)
    if cached is None:
        for p in params:
            if p.dtype == torch.float32 and half:
                p.data = p.data.half()

        def build_weight(originals):
            g = originals[2].detach()
            return interleave_glu_rows(_folded(originals[0].detach(), g), _folded(originals[1].detach(), g))

        weight = build_weight(params)
        bias = None if b_gate is None else interleave_glu_rows(b_gate.detach(), b_value.detach())
        cached = (weight, bias)

        def rebuild(value, originals):
            value[0].copy_(build_weight(originals))
            if value[1] is not None:
                value[1].copy_(interleave_glu_rows(originals[3].detach(), originals[4].detach()))

        _fused_params.put(params, cached, rebuild)
    return cached


def rms_linear_wrapper(x: torch.Tensor, rms_weight, eps: float, weight, bias, activation="", rstd=None):
    """linear_wrapper_functional(layer_norm_rms_wrapper(x, rms_weight, eps), weight, bias, activation) — one launch
    for decoding steps (reference: `rms_matmul_rbe_wrapper`, experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:186-213)."""
    from kernl_amd.implementations.linear_layer import rms_linear_layer
    from kernl_amd.optimizer.layer_norm import layer_norm_rms_wrapper

    prompt = activation == "" and _rms_prompt_foldable(x, rms_weight)
    if not (_rms_fusable(x, rms_weight) or prompt) or weight.dtype not in (x.dtype, torch.float32):
        return linear_wrapper_functional(layer_norm_rms_wrapper(x, rms_weight, eps), weight, bias, activation=activation)
    if weight.dtype == torch.float32:
        weight.data = weight.data.half()
    if bias is not None and bias.dtype == torch.float32:
        bias.data = bias.data.half()
    if weight.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        return linear_wrapper_functional(layer_norm_rms_wrapper(x, rms_weight, eps), weight, bias, activation=activation)
    w = weight if weight.is_contiguous() else weight.contiguous()
    g = _rms_weight_like(x, rms_weight)
    return rms_linear_layer(x, g, eps, w, bias, activation, folded_weight=_folded_weight(w, g) if prompt else None,
                            rstd=rstd if prompt else None)


def rms_fused_linear_wrapper(x: torch.Tensor, rms_weight, eps: float, weights, biases, rstd=None):
    """fused_linear_wrapper(layer_norm_rms_wrapper(x, rms_weight, eps), weights, biases): the query / key / value
    projections of a decoder layer with the RMSNorm in front of them (reference: `rms_matmul_rbe_qkv_wrapper`,
    experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:289-344, without its rotary epilogue)."""
    from kernl_amd.implementations.linear_layer import rms_linear_layer
    from kernl_amd.optimizer.layer_norm import layer_norm_rms_wrapper

    prompt = _rms_prompt_foldable(x, rms_weight)
    if not (_rms_fusable(x, rms_weight) or prompt):
        return fused_linear_wrapper(layer_norm_rms_wrapper(x, rms_weight, eps), weights, biases)
    weight, bias, sizes = _concatenated_params(x, weights, biases)
    if weight.dtype != x.dtype:
        return fused_linear_wrapper(layer_norm_rms_wrapper(x, rms_weight, eps), weights, biases)
    g = _rms_weight_like(x, rms_weight)
    out = rms_linear_layer(x, g, eps, weight, bias, "", folded_weight=_folded_concatenated_weight(weights, g) if prompt else None,
                           rstd=rstd if prompt else None)
    return tuple(torch.split(out, sizes, dim=-1))


def rms_glu_linear_wrapper(x: torch.Tensor, rms_weight, eps: float, w_gate, b_gate, w_value, b_value, activation: str, rstd=None):
    """glu_linear_wrapper(layer_norm_rms_wrapper(x, rms_weight, eps), ...): the feed-forward entry of a SwiGLU decoder
    with its RMSNorm (reference: `kernel_ff`, experimental/llama-v2/kernel/fused_kernel_ff.py:82-117, whose kernel
    normalises inside the product, :10-79)."""
    from kernl_amd.implementations.linear_layer import rms_linear_layer
    from kernl_amd.optimizer.layer_norm import layer_norm_rms_wrapper

    usable, half = _glu_usable(x, w_gate, b_gate, w_value, b_value)
    prompt = activation == "silu" and _rms_prompt_foldable(x, rms_weight)
    if not usable or not (_rms_fusable(x, rms_weight) or prompt):
        return glu_linear_wrapper(layer_norm_rms_wrapper(x, rms_weight, eps), w_gate, b_gate, w_value, b_value, activation)
    g = _rms_weight_like(x, rms_weight)
    if prompt:
        # prompts read the weight with the norm's weight folded in: the un-folded arrangement is only built if decoding
        # steps (which apply the norm's weight to x) ever run through this layer
        folded, bias = _folded_interleaved_params(half, w_gate, b_gate, w_value, b_value, g)
        if folded.dtype == x.dtype:
            return rms_linear_layer(x, g, eps, folded, bias, activation, gated=True, folded_weight=folded, rstd=rstd,
                                    unfolded=lambda: _interleaved_params(half, w_gate, b_gate, w_value, b_value)[0])
    weight, bias = _interleaved_params(half, w_gate, b_gate, w_value, b_value)
    if weight.dtype != x.dtype:
        return glu_linear_wrapper(layer_norm_rms_wrapper(x, rms_weight, eps), w_gate, b_gate, w_value, b_value, activation)
    return rms_linear_layer(x, g, eps, weight, bias, activation, gated=True)


def linear_residual_wrapper(v: torch.Tensor, weight: torch.Tensor, bias, residual: torch.Tensor):
    """residual + linear(v, weight, bias): the attention-output and feed-forward-down projections of a decoder layer with
    the addition that follows them.  Decoding steps (at most 64 rows) run it as one launch; larger inputs as the linear
    kernel and the addition they were.  No counterpart in the reference, whose model adds in eager PyTorch
    (experimental/llama-v2/llama/model.py:262-264)."""
    from kernl_amd.implementations.linear_layer import decode_linear_layer, decode_linear_supported, takes_small_problem_kernel

    if weight.dtype == torch.float32 and (v.dtype == torch.float16 or torch.is_autocast_enabled("cuda")):
        weight.data = weight.data.half()
    if bias is not None and bias.dtype == torch.float32 and (v.dtype == torch.float16 or torch.is_autocast_enabled("cuda")):
        bias.data = bias.data.half()
    x2d = v if v.dim() == 2 else v.reshape(-1, v.shape[-1])
    if (
        decode_linear_supported(v, weight)
        # small weights: the one-launch small-tile kernels beat the weight-streaming kernel by more than the separate
        # addition costs (64 x 768 x 3072: 8.0 us against 11.6), so such shapes keep the addition
        and not takes_small_problem_kernel(x2d, weight)
        and residual.dtype == v.dtype
        and residual.shape[:-1] == v.shape[:-1]
        and residual.shape[-1] == weight.shape[0]
        and (bias is None or bias.dtype == v.dtype)
        and not torch.is_autocast_enabled("cuda")
    ):
        return decode_linear_layer(v, weight, bias, residual=residual)
    fused = _wide_residual_linear(v, weight, bias, residual)
    if fused is not None:
        return fused
    return residual + linear_wrapper_functional(v, weight, bias)


def _wide_residual_linear(v: torch.Tensor, weight: torch.Tensor, bias, residual: torch.Tensor):
    """residual + linear(v) with the addition in the epilogue of the wide tile kernels, for the shapes those kernels run
    anyway (prompts, encoder batches); None otherwise."""
    from kernl_amd.implementations.linear_layer import residual_linear_layer, residual_linear_supported

    if not (WIDE_RESIDUAL_EPILOGUE and residual.is_cuda):
        return None
    if weight.dtype == torch.float32 and v.dtype == torch.float16:
        weight.data = weight.data.half()
    if bias is not None and bias.dtype == torch.float32 and v.dtype == torch.float16:
        bias.data = bias.data.half()
    if not residual_linear_supported(v, weight, bias, residual):
        return None
    return residual_linear_layer(v, weight, bias, residual)


def linear_residual_stats_wrapper(v: torch.Tensor, weight: torch.Tensor, bias, residual: torch.Tensor, eps: float):
    """(residual + linear(v, weight, bias), rstd): `linear_residual_wrapper` whose addition also leaves, for prompts, the
    row statistics 1 / sqrt(mean(sum^2) + eps) of the RMSNorm that follows — the projections behind that norm take them
    (`rstd=` of the `rms_*` wrappers) and never see a normalised tensor.  rstd is None where the statistics are not
    wanted (decoding steps, whose one-launch kernels normalise inside the product; dtypes the kernel does not take)."""
    from kernl_amd.implementations.linear_layer import add_rms_stats, add_rms_stats_supported, rms_eps, rms_stats

    from kernl_amd.implementations.linear_layer import FEW_ROW_MAX_ROWS

    rows = v.numel() // v.shape[-1] if v.numel() else 0
    prompt = (
        RMS_PROMPT_FOLDING and residual.is_cuda and rows > FEW_ROW_MAX_ROWS and not torch.is_autocast_enabled("cuda")
        and residual.dtype in (torch.float16, torch.bfloat16) and residual.dtype == v.dtype
        and residual.shape[:-1] == v.shape[:-1] and residual.shape[-1] == weight.shape[0] and weight.shape[0] % 8 == 0
    )
    if not prompt:
        return linear_residual_wrapper(v, weight, bias, residual), None
    fused = _wide_residual_linear(v, weight, bias, residual)
    if fused is not None:
        # the addition rode in the projection: one pass over the sum for its row statistics
        return fused, rms_stats(fused, eps)
    y = linear_wrapper_functional(v, weight, bias)
    if y.dtype != residual.dtype or not add_rms_stats_supported(residual, y):
        return residual + y, None
    return add_rms_stats(residual, y, rms_eps(residual.dtype, eps))


def rms_fused_linear_rope_wrapper(x: torch.Tensor, rms_weight, eps: float, weights, biases, cos, sin, n_rotated: int, head_dim: int,
                                  rstd=None):
    """rms_fused_linear_wrapper(x, ...) with the rotary embedding of its first `n_rotated` outputs (query and key) applied
    head by head: outputs [.., heads_i * head_dim] as before, the rotated ones already rotated.  A decoding step runs
    norm, product and rotation as ONE launch (reference: `rms_matmul_rbe_qkv_wrapper`,
    experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:289-344); larger inputs run the kernels they ran before.
    cos, sin: [batch | 1, 1, positions, head_dim] as Hugging Face decoders hand them to `apply_rotary_pos_emb`."""
    from kernl_amd.implementations.linear_layer import decode_linear_layer, decode_linear_supported
    from kernl_amd.implementations.rotary import rotary_forward

    weight, bias, sizes = _concatenated_params(x, weights, biases)
    fast = (
        x.dim() == 3
        and _rms_fusable(x, rms_weight)
        and decode_linear_supported(x, weight, head_dim)
        and (bias is None or bias.dtype == x.dtype)
        and cos.dim() == 4 and cos.shape == sin.shape and cos.dtype == sin.dtype and cos.shape[1] == 1
        and cos.shape[2] == x.shape[1] and cos.shape[3] == head_dim and cos.shape[0] in (1, x.shape[0])
        and cos.stride(-1) == 1 and sin.stride() == cos.stride()
        and cos.dtype in (torch.float16, torch.bfloat16, torch.float32)
        and head_dim % 32 == 0 and all(n % head_dim == 0 for n in sizes)
    )
    if fast:
        out = decode_linear_layer(x, weight, bias, _rms_weight_like(x, rms_weight), eps, None, cos.squeeze(1), sin.squeeze(1),
                                  head_dim=head_dim, rope_cols=sum(sizes[:n_rotated]))
        return tuple(torch.split(out, sizes, dim=-1))
    outs = list(rms_fused_linear_wrapper(x, rms_weight, eps, weights, biases, rstd=rstd))
    first = outs[0]
    rot_cols = sum(sizes[:n_rotated])
    adjacent = (
        n_rotated > 1 and first.dim() == 3 and first.stride(-1) == 1
        and all(sizes[i] % head_dim == 0 for i in range(n_rotated))
        and all(outs[i].stride() == first.stride() for i in range(n_rotated))
        and all(outs[i].data_ptr() == first.data_ptr() + sum(sizes[:i]) * first.element_size() for i in range(n_rotated))
    )
    if adjacent:
        # the rotated outputs are neighbouring column ranges of one buffer: one launch over all their heads
        both = first.as_strided((first.shape[0], first.shape[1], rot_cols), first.stride())
        heads = both.reshape(first.shape[0], first.shape[1], -1, head_dim).transpose(1, 2)
        rotated = rotary_forward(heads, cos, sin).transpose(1, 2).reshape(first.shape[0], first.shape[1], rot_cols)
        outs[:n_rotated] = torch.split(rotated, sizes[:n_rotated], dim=-1)
        return tuple(outs)
    for i in range(n_rotated):
        o = outs[i]
        heads = o.reshape(*o.shape[:-1], -1, head_dim).transpose(-3, -2)        # [.., heads, positions, head_dim], a view
        outs[i] = rotary_forward(heads, cos, sin).transpose(-3, -2).reshape(o.shape)
    return tuple(outs)


def linear_add_layer_norm_wrapper(v: torch.Tensor, weight: torch.Tensor, bias, residual: torch.Tensor, normalized_shape,
                                  ln_weight, ln_bias, eps: float):
    """layer_norm(residual + linear(v, weight, bias)): the attention-output and feed-forward-down projections of an
    encoder layer with the addition and LayerNorm behind them.  Where the projection runs the wide tile kernels the
    addition rides in their epilogue and the LayerNorm reads one tensor (16384 x 768, fp16: 15 us -> 11 us per norm);
    elsewhere the projection is followed by the fused add + LayerNorm kernel, as before.  No counterpart in the
    reference, whose graphs add in eager PyTorch in front of every LayerNorm."""
    from kernl_amd.optimizer.layer_norm import add_layer_norm_wrapper_functional, layer_norm_wrapper_functional

    if isinstance(residual, torch.Tensor):
        fused = _wide_residual_linear(v, weight, bias, residual)
        if fused is not None:
            return layer_norm_wrapper_functional(fused, normalized_shape, ln_weight, ln_bias, eps)
    return add_layer_norm_wrapper_functional(linear_wrapper_functional(v, weight, bias), residual, normalized_shape, ln_weight,
                                             ln_bias, eps)


torch.fx.wrap("linear_add_layer_norm_wrapper")
torch.fx.wrap("rms_linear_wrapper")
torch.fx.wrap("rms_fused_linear_wrapper")
torch.fx.wrap("rms_glu_linear_wrapper")
torch.fx.wrap("linear_residual_wrapper")
torch.fx.wrap("linear_residual_stats_wrapper")
torch.fx.wrap("rms_fused_linear_rope_wrapper")


def fuse_residual_into_linears(gm: torch.fx.GraphModule):
    """`residual + linear_wrapper_functional(v, w, b)` (either operand order, no activation, the product consumed by the
    addition only) becomes one `linear_residual_wrapper` call.  Runs after the linear passes."""
    import operator

    changed = False
    for node in list(gm.graph.nodes):
        if not (node.op == "call_function" and node.target in (operator.add, torch.add) and len(node.args) == 2 and not node.kwargs):
            continue
        for lin, res in (node.args, node.args[::-1]):
            if not (isinstance(lin, torch.fx.Node) and isinstance(res, torch.fx.Node)):
                continue
            if not (lin.op == "call_function" and lin.target is linear_wrapper_functional and len(lin.users) == 1):
                continue
            if len(lin.args) != 3 or lin.kwargs.get("activation", "") != "" or set(lin.kwargs) - {"activation"}:
                continue
            if res is lin:
                continue
            with gm.graph.inserting_before(node):
                fused = gm.graph.call_function(linear_residual_wrapper, tuple(lin.args) + (res,))
            fused.meta = dict(node.meta)
            node.replace_all_uses_with(fused)
            gm.graph.erase_node(node)
            gm.graph.erase_node(lin)
            changed = True
            break
    if changed:
        gm.graph.lint()
        gm.recompile()


def fuse_linears_into_add_layer_norms(gm: torch.fx.GraphModule):
    """`add_layer_norm_wrapper_functional(linear_wrapper_functional(v, w, b), residual, ...)` (either operand order, no
    activation, the product consumed by the addition only) becomes one `linear_add_layer_norm_wrapper` call, which decides
    per shape where the addition happens.  Runs after the linear and LayerNorm passes."""
    from kernl_amd.optimizer.layer_norm import add_layer_norm_wrapper_functional

    changed = False
    for node in list(gm.graph.nodes):
        if not (node.op == "call_function" and node.target is add_layer_norm_wrapper_functional and len(node.args) == 6 and not node.kwargs):
            continue
        for lin, res in (node.args[:2], node.args[1::-1]):
            if not (isinstance(lin, torch.fx.Node) and isinstance(res, torch.fx.Node)) or res is lin:
                continue
            if not (lin.op == "call_function" and lin.target is linear_wrapper_functional and len(lin.users) == 1):
                continue
            if len(lin.args) != 3 or lin.kwargs.get("activation", "") != "" or set(lin.kwargs) - {"activation"}:
                continue
            with gm.graph.inserting_before(node):
                fused = gm.graph.call_function(linear_add_layer_norm_wrapper, tuple(lin.args) + (res,) + tuple(node.args[2:]))
            node.replace_all_uses_with(fused)
            gm.graph.erase_node(node)
            gm.graph.erase_node(lin)
            changed = True
            break
    if changed:
        gm.graph.lint()
        gm.recompile()


def fuse_rms_stats_into_residual_adds(gm: torch.fx.GraphModule):
    """A `linear_residual_wrapper` whose sum feeds `rms_*` projections (the residual stream of a decoder layer in front
    of the next RMSNorm) becomes `linear_residual_stats_wrapper`: element 0 replaces the sum everywhere, element 1 — the
    row statistics of that norm — goes to those projections as `rstd=`.  All of them must use the same eps.  Runs after
    the residual, RMSNorm and rotary passes."""
    import operator

    rms_forms = (rms_linear_wrapper, rms_fused_linear_wrapper, rms_glu_linear_wrapper, rms_fused_linear_rope_wrapper)
    changed = False
    for node in list(gm.graph.nodes):
        if not (node.op == "call_function" and node.target is linear_residual_wrapper and len(node.args) == 4 and not node.kwargs):
            continue
        takers = [u for u in node.users if u.op == "call_function" and u.target in rms_forms and len(u.args) >= 3
                  and u.args[0] is node and "rstd" not in u.kwargs and isinstance(u.args[2], (int, float))]
        if not takers or len({float(u.args[2]) for u in takers}) != 1:
            continue
        with gm.graph.inserting_after(node):
            both = gm.graph.call_function(linear_residual_stats_wrapper, tuple(node.args) + (float(takers[0].args[2]),))
        with gm.graph.inserting_after(both):
            total = gm.graph.call_function(operator.getitem, (both, 0))
        with gm.graph.inserting_after(total):
            rstd = gm.graph.call_function(operator.getitem, (both, 1))
        total.meta = dict(node.meta)
        node.replace_all_uses_with(total)
        gm.graph.erase_node(node)
        for u in takers:
            u.kwargs = {**u.kwargs, "rstd": rstd}
        changed = True
    if changed:
        gm.graph.lint()
        gm.recompile()


def fuse_rotary_into_projections(gm: torch.fx.GraphModule):
    """The rotary embedding of the query and key projections moves into the fused projection that produces them:

        f = rms_fused_linear_wrapper(x, g, eps, [wq, wk, wv], biases);  q = f[0].view(B, S, -1, D).transpose(1, 2)
        rotary_wrapper(q, cos, sin), rotary_wrapper(k, cos, sin)

    becomes `rms_fused_linear_rope_wrapper(x, g, eps, weights, biases, cos, sin, 2, D)` with the views reading its
    outputs directly.  The rotated outputs must be a leading run of the projection's outputs, each consumed only
    through that view / transpose chain, all with the same tables.  Runs after `fuse_rms_norm_into_linears`."""
    import operator

    from kernl_amd.optimizer.rotary import rotary_wrapper

    def chain_of(part: torch.fx.Node):
        """part = f[i] -> view(.., D) -> transpose(1, 2) -> rotary_wrapper: returns (rotary node, cos, sin, D) or None."""
        if len(part.users) != 1:
            return None
        view = next(iter(part.users))
        if not (view.op == "call_method" and view.target in ("view", "reshape") and view.args[0] is part and len(view.users) == 1):
            return None
        shape = view.args[1] if len(view.args) == 2 and isinstance(view.args[1], (tuple, list)) else view.args[1:]
        if len(shape) != 4 or not isinstance(shape[-1], int) or shape[-1] <= 0:
            return None
        tr = next(iter(view.users))
        if not (tr.op == "call_method" and tr.target == "transpose" and tuple(tr.args[1:]) in ((1, 2), (2, 1)) and len(tr.users) == 1):
            return None
        rot = next(iter(tr.users))
        if not (rot.op == "call_function" and rot.target is rotary_wrapper and rot.args[0] is tr and len(rot.args) == 3):
            return None
        return rot, rot.args[1], rot.args[2], shape[-1]

    changed = False
    for node in list(gm.graph.nodes):
        if not (node.op == "call_function" and node.target is rms_fused_linear_wrapper and len(node.args) == 5):
            continue
        parts = {}
        for user in node.users:
            if user.op == "call_function" and user.target is operator.getitem and isinstance(user.args[1], int):
                parts[user.args[1]] = user
        if len(parts) != len(node.users):
            continue
        chains = []
        for i in range(len(parts)):
            c = chain_of(parts[i]) if i in parts else None
            if c is None:
                break
            if chains and (c[1] is not chains[0][1] or c[2] is not chains[0][2] or c[3] != chains[0][3]):
                break
            chains.append(c)
        if not chains:
            continue
        _, cos, sin, head_dim = chains[0]
        # the tables must be computed before the projection for the fused call to take them: a table node that follows
        # the projection (Hugging Face unsqueezes them after it) moves up when its own inputs allow that
        order = {n: i for i, n in enumerate(gm.graph.nodes)}
        movable = all(
            order[t] < order[node] or all(order[inp] < order[node] for inp in t.all_input_nodes) for t in (cos, sin)
        )
        if not movable:
            continue
        for t in dict.fromkeys((cos, sin)):
            if order[t] > order[node]:
                node.prepend(t)
        with gm.graph.inserting_before(node):
            fused = gm.graph.call_function(rms_fused_linear_rope_wrapper, tuple(node.args) + (cos, sin, len(chains), head_dim))
        fused.meta = dict(node.meta)
        node.replace_all_uses_with(fused)
        gm.graph.erase_node(node)
        for rot, _, _, _ in chains:
            rot.replace_all_uses_with(rot.args[0])
            gm.graph.erase_node(rot)
        changed = True
    if changed:
        gm.graph.lint()
        gm.recompile()


def fuse_rms_norm_into_linears(gm: torch.fx.GraphModule):
    """An RMSNorm whose only consumers are linear layers taking it as their input is folded into them: every such
    consumer becomes its `rms_*` form on the un-normalised tensor and the norm node goes away.  Whether the one-launch
    kernel runs is decided per call from the number of rows (decoding steps: yes; prefill: the RMSNorm kernel once,
    then the ordinary linear kernels).  Runs after the linear and layer-norm passes."""
    from kernl_amd.optimizer.layer_norm import layer_norm_rms_wrapper

    fused_form = {
        linear_wrapper_functional: rms_linear_wrapper,
        fused_linear_wrapper: rms_fused_linear_wrapper,
        glu_linear_wrapper: rms_glu_linear_wrapper,
    }
    changed = False
    for node in list(gm.graph.nodes):
        if node.op != "call_function" or node.target is not layer_norm_rms_wrapper or len(node.args) != 3 or node.kwargs:
            continue
        users = list(node.users)
        if not users or not all(
            u.op == "call_function" and u.target in fused_form and len(u.args) >= 1 and u.args[0] is node
            and sum(1 for inp in u.all_input_nodes if inp is node) == 1
            for u in users
        ):
            continue
        x, rms_weight, eps = node.args
        for u in users:
            with gm.graph.inserting_before(u):
                new = gm.graph.call_function(fused_form[u.target], (x, rms_weight, eps) + tuple(u.args[1:]), dict(u.kwargs))
            u.replace_all_uses_with(new)
            gm.graph.erase_node(u)
        gm.graph.erase_node(node)
        changed = True
    if changed:
        gm.graph.lint()
        gm.recompile()


def replace_all_linear(gm: torch.fx.GraphModule):
    replace_linear_activation(gm, torch.nn.Tanh(), "tanh")
    replace_linear_activation(gm, torch.nn.ReLU(), "relu")
    replace_linear_activation(gm, torch.nn.functional.gelu, "gelu")
    replace_linear_fn_activation(gm)
    replace_linear(gm)
    replace_linear_fn(gm)
    replace_linear_fn_constant_match(gm)
    fuse_gated_linears(gm)
    fuse_sibling_linears(gm)
