"""Host-side logic on the CPU: static input pool, sub-graph matcher, rewrite passes.

Known answers come from the reference's own tests and docs: test/test_cuda_graph.py:7-40 (argsort, aligned sizes,
pool placement), test/test_attention.py:148-157 (closest_power_of_2) and the worked `replace_pattern` example of
docs/how-to-guides/support-new-model.md:139-246.
"""
import operator

import pytest
import torch

from kernl_amd.implementations.attention import closest_power_of_2
from kernl_amd.optimizer.cuda_graph import argsort, get_pool_size, prepare_inputs
from kernl_amd.optimizer.dynamo_backend import dynamo_backend_ofi
from kernl_amd.optimizer.pool_cuda_graphs import CudaGraphPool, get_aligned_size
from kernl_amd.utils.extended_matcher import replace_pattern
from kernl_amd.utils.fx import static_args_are_equal


def _targets(gm):
    return [getattr(n.target, "__name__", str(n.target)) for n in gm.graph.nodes if n.op in ("call_function", "call_method", "call_module")]


# ------------------------------------------------------------------------------------------------ pool (known answers)
def test_argsort():
    assert argsort(iterable=[1, 5, 3, 4, 5], key=lambda x: x) == [0, 2, 3, 1, 4]


def test_aligned_size():
    t = torch.ones((33,))
    assert get_aligned_size(t, alignment=16) == 144
    assert get_aligned_size(t, alignment=32) == 160
    assert get_aligned_size(torch.ones((1,)), alignment=8) == 8


def test_cuda_graph_pool_e2e():
    all_inputs = [
        torch.tensor([1, 2, 3]),
        torch.tensor([4, 5, 6, 7], dtype=torch.bfloat16),
        torch.tensor([8]),
        torch.tensor([9, 10, 11, 12], dtype=torch.double),
        torch.tensor([13, 14], dtype=torch.int8),
        torch.tensor([15], dtype=torch.float32),
        torch.tensor([16], dtype=torch.int64),
    ]
    all_pools = [CudaGraphPool(32, device="cpu"), CudaGraphPool(48, device="cpu")]
    new_tensors = prepare_inputs(inputs=all_inputs, pools=all_pools)
    assert len(new_tensors) == len(all_inputs)
    assert len(all_pools) == 3
    for original, copy in zip(all_inputs, new_tensors):
        assert original.shape == copy.shape
        assert original.stride() == copy.stride()
        assert original.dtype == copy.dtype
        assert original.device == copy.device
        assert torch.all(original == copy)
        assert original.data_ptr() != copy.data_ptr()
    # placement is deterministic: the same inputs land on the same addresses (what graph replay needs)
    again = prepare_inputs(inputs=[t + 1 for t in all_inputs], pools=all_pools)
    assert len(all_pools) == 3
    assert [t.data_ptr() for t in again] == [t.data_ptr() for t in new_tensors]
    assert all(torch.all(a == t + 1) for a, t in zip(again, all_inputs))


def test_cuda_graph_pool():
    c = CudaGraphPool(8, device="cpu")
    assert not c.can_store(torch.ones((16,), dtype=torch.int64))
    t = torch.ones((1,), dtype=torch.int8)
    assert c.can_store(t)
    assert c.offset == 0
    c.copy_to_pool(t)
    assert c.offset > 0
    c.reset()
    assert c.offset == 0
    exact = CudaGraphPool(16, device="cpu")
    exact.copy_to_pool(torch.tensor([1, 1, 1, 1], dtype=torch.float32))  # 16 bytes fit exactly
    assert exact.offset == 16 and not exact.can_store(t)


def test_pool_removes_zero_strides_and_sizes_to_power_of_two():
    pool = CudaGraphPool(64, device="cpu")
    expanded = torch.tensor([[1.0, 2.0]]).expand(3, 2)  # stride (0, 1)
    copy = pool.copy_to_pool(expanded)
    assert copy.stride() == (1, 1) and copy.shape == (3, 2)
    assert get_pool_size([torch.ones(5), torch.ones(9)], []) == 64  # 24 + 40 = 64
    assert get_pool_size([torch.ones(5)], [CudaGraphPool(256, device="cpu")]) == 256
    assert get_pool_size([torch.ones(33)], []) == 256  # 136 -> next power of two


def test_closest_power_of_2():
    assert closest_power_of_2(1, min_range=16, max_range=128) == [8, 16, 32]
    assert closest_power_of_2(20, min_range=16, max_range=128) == [16, 32]
    assert closest_power_of_2(257, min_range=16, max_range=128) == [64, 128, 256]
    assert closest_power_of_2(1, min_range=4, max_range=128) == [2, 4, 8]


# ------------------------------------------------------------------------------------------------ matcher
class _FeedForward(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1 = torch.nn.Linear(5, 10)
        self.tanh = torch.nn.Tanh()
        self.fc2 = torch.nn.Linear(10, 1)
        self.sigmoid = torch.nn.Sigmoid()

    def forward(self, x):
        return self.sigmoid(self.fc2(self.tanh(self.fc1(x))))


def test_replace_pattern_worked_example_from_the_docs():
    class Pattern(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.linear = torch.nn.Linear(1, 1)
            self.activation = torch.nn.Tanh()

        def forward(self, v):
            return self.activation(self.linear(v))

    class Replacement(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.linear = torch.nn.Linear(1, 1)
            self.relu = torch.nn.ReLU()

        def forward(self, v):
            return self.relu(self.linear(v))

    m = _FeedForward()
    gm = torch.fx.symbolic_trace(m)
    matches = replace_pattern(gm, Pattern(), Replacement())
    assert len(matches) == 1
    nodes = [(n.op, n.target) for n in gm.graph.nodes]
    assert nodes == [("placeholder", "x"), ("call_module", "fc1"), ("call_module", "relu"), ("call_module", "fc2"),
                     ("call_module", "sigmoid"), ("output", "output")]
    x = torch.randn(3, 5)
    assert torch.allclose(gm(x), torch.sigmoid(m.fc2(torch.relu(m.fc1(x)))))  # fc1 is the ORIGINAL module


def test_literal_arguments_take_part_in_the_match():
    def model(x, y):
        return torch.softmax(x / 8.0 + y, dim=-1), torch.softmax(x / 4.0 + y, dim=-1)

    def pattern(a, b):
        return torch.softmax(a / 8.0 + b, dim=-1)

    def replacement(a, b):
        return torch.sigmoid(a - b)

    gm = torch.fx.symbolic_trace(model)
    assert len(replace_pattern(gm, pattern, replacement)) == 1
    x, y = torch.randn(2, 4), torch.randn(2, 4)
    out = gm(x, y)
    assert torch.allclose(out[0], torch.sigmoid(x - y)) and torch.allclose(out[1], torch.softmax(x / 4.0 + y, -1))
    div8 = next(n for n in torch.fx.symbolic_trace(pattern).graph.nodes if n.target is operator.truediv)
    div4 = next(n for n in gm.graph.nodes if n.target is operator.truediv)
    assert not static_args_are_equal(div8, div4)


def test_wildcard_binds_literals_and_overlaps_are_not_double_counted():
    def model(x):
        a = torch.relu(x * 0.125)
        b = torch.relu(a * 3.0)
        return b + a  # `a` escapes: the first relu/mul pair must stay

    def pattern(t, literal_s):
        return torch.relu(t * literal_s)

    def replacement(t, literal_s):
        return torch.clamp_min(t, 0.0) * literal_s

    gm = torch.fx.symbolic_trace(model)
    matches = replace_pattern(gm, pattern, replacement)
    assert len(matches) == 2
    x = torch.randn(7)
    assert torch.allclose(gm(x), model(x))

    def model2(x, s):
        return torch.relu(x * s)

    gm2 = torch.fx.symbolic_trace(model2)
    assert replace_pattern(gm2, pattern, replacement) == []  # `literal_` placeholders refuse tensors


def test_internal_value_used_elsewhere_blocks_the_match():
    def model(x):
        inner = x * 2.0
        return torch.relu(inner), inner

    def pattern(t):
        return torch.relu(t * 2.0)

    def replacement(t):
        return torch.sigmoid(t)

    gm = torch.fx.symbolic_trace(model)
    assert replace_pattern(gm, pattern, replacement) == []


# ------------------------------------------------------------------------------------------------ passes
class _Block(torch.nn.Module):
    """One post-LN encoder block written the way BERT was traced in the reference's day (module calls, `/ 8.0`)."""

    def __init__(self, d=64, heads=1):
        super().__init__()
        self.q, self.k, self.v, self.o = (torch.nn.Linear(d, d) for _ in range(4))
        self.ln1, self.ln2 = torch.nn.LayerNorm(d, eps=1e-12), torch.nn.LayerNorm(d, eps=1e-12)
        self.up, self.down = torch.nn.Linear(d, 4 * d), torch.nn.Linear(4 * d, d)
        self.drop = torch.nn.Dropout(0.1)
        self.heads, self.d = heads, d

    def forward(self, x, mask):
        B, S, _ = x.shape
        split = lambda t: t.view(B, S, self.heads, -1).permute(0, 2, 1, 3)  # noqa: E731
        q, k, v = split(self.q(x)), split(self.k(x)), split(self.v(x))
        scores = torch.matmul(q, k.transpose(-1, -2))
        scores = scores / 8.0
        scores = scores + mask
        probs = torch.nn.functional.softmax(scores, dim=-1)
        probs = self.drop(probs)
        ctx = torch.matmul(probs, v).permute(0, 2, 1, 3).reshape(B, S, -1)
        h = self.ln1(self.drop(self.o(ctx)) + x)
        ff = self.down(torch.nn.functional.gelu(self.up(h)))
        ff += h
        return self.ln2(ff)


def test_backend_rewrites_reference_style_graph():
    gm = torch.fx.symbolic_trace(_Block())
    dynamo_backend_ofi(gm)
    t = _targets(gm)
    assert t.count("attention_wrapper") == 1
    assert t.count("linear_wrapper") == 6
    assert t.count("layer_norm_wrapper") == 2
    assert "softmax" not in t and "matmul" not in t and "drop" not in t and "gelu" not in t and "iadd" not in t
    # the fused gelu went into the up-projection
    up = next(n for n in gm.graph.nodes if n.op == "call_function" and n.target.__name__ == "linear_wrapper" and n.kwargs.get("activation") == "gelu")
    assert up.args[1].target == "up"
    attn = next(n for n in gm.graph.nodes if n.op == "call_function" and n.target.__name__ == "attention_wrapper")
    assert attn.args[4] == 1 / 8.0 and attn.args[5] is False


def test_backend_rewrites_dynamo_graph_of_bert():
    """What TorchDynamo hands over today: F.linear / F.layer_norm on lifted parameters, `* scaling`, a [B,1,S,S] mask."""
    from transformers import BertConfig, BertModel

    for attn_impl, fused in (("eager", "attention_wrapper"), ("sdpa", "sdpa_wrapper")):
        torch.manual_seed(0)
        cfg = BertConfig(num_hidden_layers=2, hidden_size=128, num_attention_heads=2, intermediate_size=256, vocab_size=100)
        cfg._attn_implementation = attn_impl
        model = BertModel(cfg).eval()
        graphs = []

        def backend(gm, example_inputs):
            dynamo_backend_ofi(gm)
            graphs.append(gm)
            return lambda *a: None  # never executed: the rewritten graph needs the GPU library

        torch._dynamo.reset()
        ids = torch.randint(0, 100, (2, 16))
        mask = torch.ones(2, 16, dtype=torch.long)
        try:
            with torch.inference_mode():
                torch._dynamo.optimize(backend, dynamic=False)(model.forward)(input_ids=ids, attention_mask=mask)
        except Exception:
            pass  # the dummy callable returns None
        assert len(graphs) == 1
        t = _targets(graphs[0])
        assert t.count(fused) == 2
        # query/key/value projections share their input: one fused GEMM per layer, 3 + pooler stay separate
        assert t.count("fused_linear_wrapper") == 2
        # the attention-output and feed-forward-down projections go with the addition and LayerNorm behind them (the call
        # decides per shape whether the addition rides in the projection or in the norm); the up-projections and the
        # pooler stay on their own, and so does the add + LayerNorm of the embeddings
        assert t.count("linear_add_layer_norm_wrapper") == 2 * 2
        assert t.count("linear_wrapper_functional") == 2 * 1 + 1
        assert t.count("add_layer_norm_wrapper_functional") == 0
        # the three embedding lookups, their two additions and the LayerNorm behind them are one call
        assert t.count("embedding_layer_norm_wrapper") == 1 and "embedding" not in t
        emb = next(n for n in graphs[0].graph.nodes if n.op == "call_function" and n.target.__name__ == "embedding_layer_norm_wrapper")
        assert [a.name for a in emb.args[1:6:2]] == [
            "l_self_modules_embeddings_modules_word_embeddings_parameters_weight_",
            "l_self_modules_embeddings_modules_token_type_embeddings_parameters_weight_",
            "l_self_modules_embeddings_modules_position_embeddings_parameters_weight_"]
        # the padding mask is reshaped, not gathered with index grids
        assert "arange" not in t
        assert "softmax" not in t and "dropout" not in t and "gelu" not in t and "layer_norm" not in t and "linear" not in t
        # the padding mask reaches the kernel as a broadcast of a per-key tensor, not as a [B,1,S,S] matrix
        attn = next(n for n in graphs[0].graph.nodes if n.op == "call_function" and n.target.__name__ == fused)
        mask_node = attn.args[6] if fused == "attention_wrapper" else attn.args[3]
        if fused == "sdpa_wrapper":
            # the boolean mask is turned into an additive one once, for every layer
            assert mask_node.target.__name__ == "additive_mask" and t.count("additive_mask") == 1
            assert len(mask_node.users) == 2
            mask_node = mask_node.args[0]
        assert mask_node.op == "call_method" and mask_node.target == "expand"
        assert "and_" not in t
    torch._dynamo.reset()


def test_boolean_masks_become_additive_per_key():
    from kernl_amd.optimizer.attention import additive_mask

    keep = torch.tensor([[True, True, False, True]])
    m = additive_mask(keep[:, None, None, :].expand(1, 1, 4, 4))
    assert m.shape == (1, 1, 1, 4) and m.dtype == torch.float32
    assert m.flatten().tolist() == [0.0, 0.0, float("-inf"), 0.0]
    m = additive_mask(torch.tril(torch.ones(3, 3, dtype=torch.bool)))
    assert m.shape == (1, 1, 3, 3) and m[0, 0, 0].tolist() == [0.0, float("-inf"), float("-inf")]
    f = torch.zeros(1, 1, 1, 4)
    assert additive_mask(f) is f


def test_rms_norm_and_swiglu_patterns():
    class LlamaNorm(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.ones(32))

        def forward(self, hidden_states, gate_w, up_w):
            h = hidden_states.to(torch.float32)
            variance = h.pow(2).mean(-1, keepdim=True)
            h = h * torch.rsqrt(variance + 1e-05)
            normed = self.weight * h.to(torch.float16)
            gate = torch.nn.functional.silu(torch.nn.functional.linear(normed, gate_w, None))
            return gate * torch.nn.functional.linear(normed, up_w)

    gm = torch.fx.symbolic_trace(LlamaNorm())
    dynamo_backend_ofi(gm)
    t = _targets(gm)
    assert "rsqrt" not in t and "pow" not in t
    # silu(linear) * linear on the same input with graph-input weights: one gated GEMM — and the RMSNorm, whose only
    # consumer that GEMM is, folded into it: (x, norm weight, eps, gate weight, gate bias, up weight, up bias, act)
    assert "layer_norm_rms_wrapper" not in t and "glu_linear_wrapper" not in t
    glu = [n for n in gm.graph.nodes if n.op == "call_function" and n.target.__name__ == "rms_glu_linear_wrapper"]
    assert len(glu) == 1 and glu[0].args[7] == "silu" and "linear_wrapper_functional" not in t and "mul" not in t
    assert glu[0].args[0].name == "hidden_states" and glu[0].args[1].target == "weight" and glu[0].args[2] == 1e-05
    assert glu[0].args[3].name == "gate_w" and glu[0].args[5].name == "up_w"


def test_rms_norm_with_another_consumer_is_not_folded():
    """The norm's output also feeds something that is not a linear layer (here it is returned): it has to exist."""
    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.ones(32))
            self.proj = torch.nn.Linear(32, 16, bias=False)

        def forward(self, hidden_states):
            h = hidden_states.to(torch.float32)
            variance = h.pow(2).mean(-1, keepdim=True)
            h = h * torch.rsqrt(variance + 1e-05)
            normed = self.weight * h.to(torch.float16)
            return self.proj(normed), normed

    gm = torch.fx.symbolic_trace(Block())
    dynamo_backend_ofi(gm)
    t = _targets(gm)
    assert t.count("layer_norm_rms_wrapper") == 1 and "rms_linear_wrapper" not in t


def test_llama_graph_rewrite_and_constant_causal_mask():
    """HF Llama: Llama-spelled RMSNorm (eps wildcard), SiLU fused into the gate projection, query/key/value fused
    into one GEMM, and the constant causal mask replaced by the kernel's is_causal flag."""
    from transformers import LlamaConfig, LlamaModel

    # (without a key/value cache transformers also derives a packed-sequence mask from the position ids: constants too)
    for attn_impl, fused, mask_idx, call_kwargs in (("eager", "attention_wrapper", 6, {}), ("sdpa", "sdpa_wrapper", 3, {}),
                                                    ("sdpa", "sdpa_wrapper", 3, {"use_cache": False})):
        torch.manual_seed(0)
        cfg = LlamaConfig(num_hidden_layers=2, hidden_size=128, num_attention_heads=2, num_key_value_heads=2,
                          intermediate_size=256, vocab_size=100, rms_norm_eps=1e-5)
        cfg._attn_implementation = attn_impl
        model = LlamaModel(cfg).eval()
        graphs = []

        def backend(gm, example_inputs):
            dynamo_backend_ofi(gm)
            graphs.append(gm)
            return lambda *a: None

        torch._dynamo.reset()
        try:
            with torch.inference_mode():
                torch._dynamo.optimize(backend, dynamic=False)(model.forward)(input_ids=torch.randint(0, 100, (1, 16)), **call_kwargs)
        except Exception:
            pass
        assert len(graphs) == 1
        t = _targets(graphs[0])
        assert t.count(fused) == 2
        # the two norms of every layer are folded into the projections they feed; the final norm stays
        assert t.count("layer_norm_rms_wrapper") == 1 and "rsqrt" not in t
        assert "silu" not in t and "softmax" not in t
        # SwiGLU: gate and up projections and their product are one gated GEMM per layer
        assert t.count("rms_glu_linear_wrapper") == 2
        assert "fused_linear_wrapper" not in t and "glu_linear_wrapper" not in t
        # rotary embedding: rotated inside the query/key/value projection (two of its three outputs, head size 64),
        # nothing left of rotate_half nor of a rotation kernel of its own
        assert t.count("rms_fused_linear_rope_wrapper") == 2 and "rms_fused_linear_wrapper" not in t
        assert "rotary_wrapper" not in t and "neg" not in t
        # the additions after the attention-output and feed-forward-down projections ride in those projections; the
        # three whose sum feeds the projections behind the next RMSNorm also leave that norm's row statistics (the
        # last one feeds the final norm, which stays a kernel of its own)
        assert t.count("linear_residual_stats_wrapper") == 3 and t.count("linear_residual_wrapper") == 1
        assert "linear_wrapper_functional" not in t
        for node in graphs[0].graph.nodes:
            if node.op == "call_function" and node.target.__name__ in ("rms_glu_linear_wrapper", "rms_fused_linear_rope_wrapper"):
                fed_by_sum = node.args[0].target.__name__ == "getitem" and node.args[0].args[1] == 0
                if fed_by_sum:
                    rstd = node.kwargs["rstd"]
                    assert rstd.target.__name__ == "getitem" and rstd.args == (node.args[0].args[0], 1)
                    assert rstd.args[0].target.__name__ == "linear_residual_stats_wrapper" and rstd.args[0].args[4] == 1e-5
                else:
                    assert "rstd" not in node.kwargs            # the first layer reads the embeddings
        assert t.count("add") == 1                      # position ids; no residual addition is left
        # the fresh key/value cache no longer copies: the only cat left builds the angle table
        assert t.count("cat") == 1
        for node in graphs[0].graph.nodes:
            if node.op == "call_function" and node.target.__name__ == "rms_fused_linear_rope_wrapper":
                assert node.args[7:] == (2, 64) and node.args[5].target == "unsqueeze" and node.args[6].target == "unsqueeze"
            if node.op == "call_function" and node.target.__name__ == fused:
                assert node.args[mask_idx] is None and node.args[5] is True
                assert node.args[0].target == "transpose" and node.args[1].target == "transpose"
    torch._dynamo.reset()


def test_empty_cat_operands_are_dropped():
    from kernl_amd.optimizer.kv_cache import drop_empty_cat_operands

    # TorchDynamo records the literal as a call of torch.tensor (symbolic_trace would fold it into an attribute)
    g = torch.fx.Graph()
    a_n, b_n = g.placeholder("a"), g.placeholder("b")
    empty = g.call_function(torch.tensor, ([],))
    one = g.call_function(torch.cat, ([empty, a_n],), {"dim": -2})
    empty2 = g.call_function(torch.tensor, ([],))
    two = g.call_function(torch.cat, ([empty2, a_n, b_n],), {"dim": -2})
    keep = g.call_function(torch.cat, ([a_n, b_n],), {"dim": -1})
    g.output((one, two, keep))
    gm = torch.fx.GraphModule(torch.nn.Module(), g)
    a, b = torch.randn(2, 3, 4), torch.randn(2, 3, 4)
    expect = gm(a, b)
    drop_empty_cat_operands(gm)
    cats = [n for n in gm.graph.nodes if n.op == "call_function" and n.target is torch.cat]
    assert len(cats) == 2 and all(len(n.args[0]) == 2 for n in cats)
    assert not any(n.op == "call_function" and n.target is torch.tensor for n in gm.graph.nodes)
    for got, want in zip(gm(a, b), expect):
        assert torch.equal(got, want)


def test_rotary_pass_only_fires_on_a_mid_split():
    from kernl_amd.optimizer.rotary import fuse_rotary_embedding

    def trace(split):
        class M(torch.nn.Module):
            def forward(self, x, cos, sin):
                x1, x2 = x[..., :split], x[..., split:]
                return x * cos + torch.cat((-x2, x1), dim=-1) * sin

        gm = torch.fx.symbolic_trace(M())
        for n in gm.graph.nodes:
            if n.op == "placeholder" and n.name == "x":
                n.meta["example_value"] = torch.empty(1, 2, 4, 8)
        return gm

    gm = trace(4)
    fuse_rotary_embedding(gm)
    assert _targets(gm).count("rotary_wrapper") == 1 and "cat" not in _targets(gm)
    gm = trace(2)  # not a rotation by halves: left alone
    fuse_rotary_embedding(gm)
    assert "rotary_wrapper" not in _targets(gm) and "cat" in _targets(gm)
    # sin and cos swapped between the operands is still the same expression; a different source tensor is not
    class Other(torch.nn.Module):
        def forward(self, x, y, cos, sin):
            return x * cos + torch.cat((-y[..., 4:], y[..., :4]), dim=-1) * sin

    gm = torch.fx.symbolic_trace(Other())
    for n in gm.graph.nodes:
        if n.op == "placeholder" and n.name in ("x", "y"):
            n.meta["example_value"] = torch.empty(1, 2, 4, 8)
    fuse_rotary_embedding(gm)
    assert "rotary_wrapper" not in _targets(gm)


def test_glu_row_interleaving_and_pass():
    from kernl_amd.implementations.linear_layer import interleave_glu_rows
    from kernl_amd.optimizer.linear import replace_all_linear
    F = torch.nn.functional

    gate = torch.arange(96 * 3).reshape(96, 3)
    value = -torch.arange(96 * 3).reshape(96, 3)
    w = interleave_glu_rows(gate, value)
    assert w.shape == (192, 3)
    for b in range(3):
        assert torch.equal(w[64 * b: 64 * b + 32], gate[32 * b: 32 * b + 32])
        assert torch.equal(w[64 * b + 32: 64 * b + 64], value[32 * b: 32 * b + 32])
    assert torch.equal(interleave_glu_rows(gate[:, 0], value[:, 0]), w[:, 0])

    class Mlp(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.g, self.u, self.d = torch.nn.Linear(8, 32, bias=False), torch.nn.Linear(8, 32, bias=False), torch.nn.Linear(32, 8, bias=False)

        def forward(self, x):
            gate = F.silu(F.linear(x, self.g.weight, None))
            up = F.linear(x, self.u.weight, None)
            return F.linear(gate * up, self.d.weight, None)

    gm = torch.fx.symbolic_trace(Mlp())
    replace_all_linear(gm)
    t = _targets(gm)
    assert t.count("glu_linear_wrapper") == 1 and t.count("linear_wrapper_functional") == 1 and "mul" not in t
    glu = next(n for n in gm.graph.nodes if n.op == "call_function" and n.target.__name__ == "glu_linear_wrapper")
    assert glu.args[1].target == "g.weight" and glu.args[3].target == "u.weight" and glu.args[5] == "silu"

    class Shared(torch.nn.Module):  # the gate is also used elsewhere: must stay
        def __init__(self):
            super().__init__()
            self.g, self.u = torch.nn.Linear(8, 32, bias=False), torch.nn.Linear(8, 32, bias=False)

        def forward(self, x):
            gate = F.silu(F.linear(x, self.g.weight, None))
            return gate * F.linear(x, self.u.weight, None), gate

    gm = torch.fx.symbolic_trace(Shared())
    replace_all_linear(gm)
    assert "glu_linear_wrapper" not in _targets(gm)


def test_derived_parameter_cache_follows_the_life_of_its_parameters():
    """Concatenated / interleaved weights are kept per group of original parameters.  A storage address is not an
    identity (the allocator hands a freed model's addresses to the next model), so an entry must stop matching as soon
    as one of its originals has died or moved — also when another tensor then shows the same address — and an entry
    that is a re-arranged copy is rewritten in place when an original has been written to."""
    import gc

    from kernl_amd.optimizer.linear import _DerivedParams

    cache = _DerivedParams()
    a, b = torch.zeros(8), torch.ones(4)
    assert cache.get((a, None, b)) is None
    derived = torch.zeros(12)

    def rebuild(value, originals):
        value.copy_(torch.cat([originals[0], originals[2]]))

    cache.put((a, None, b), derived, rebuild)
    assert cache.get((a, None, b)) is derived
    alias = torch.empty(0).set_(a.untyped_storage(), 0, (8,))   # same storage and address, no reference to `a`
    a.add_(1)                                 # written to: the same tensor comes back, rewritten in place
    again = cache.get((a, None, b))
    assert again is derived and again.tolist() == [1.0] * 12
    a.data.add_(1)                            # a write the version counter does not see
    assert cache.get((a, None, b)).tolist() == [1.0] * 12
    assert cache.refresh(only_changed=True) == 0 and cache.refresh(only_changed=False) == 1
    assert cache.get((a, None, b)).tolist() == [2.0] * 8 + [1.0] * 4
    assert _DerivedParams.key_of((alias, None, b)) == _DerivedParams.key_of((a, None, b))  # address and dtype
    del a
    gc.collect()
    # `alias` keeps the memory alive at the same address, as a new model's parameter would after the allocator
    # recycled it — but the tensor the entry was made from is gone
    assert cache.get((alias, None, b)) is None
    # entries of dead parameters are swept when something new is stored
    c = torch.zeros(3)
    cache.put((c,), 1)
    del c
    gc.collect()
    d = torch.zeros(5)
    cache.put((d,), 2)
    assert len(cache) == 1 and cache.get((d,)) == 2


def test_concatenated_projection_weights_alias_their_parameters():
    """After the first fused call the query / key / value parameters ARE slices of the fused weight: a write through
    any route, `param.data.copy_()` included, reaches the fused buffer without a rebuild, and the buffer's address (the
    one a captured graph replays on) never changes."""
    from kernl_amd.optimizer.linear import _concatenated_params

    torch.manual_seed(0)
    lins = [torch.nn.Linear(16, n) for n in (8, 8, 24)]
    before = [(l.weight.detach().clone(), l.bias.detach().clone()) for l in lins]
    x = torch.zeros(2, 16)
    weights, biases = [l.weight for l in lins], [l.bias for l in lins]
    weight, bias, sizes = _concatenated_params(x, weights, biases)
    assert sizes == [8, 8, 24] and weight.shape == (40, 16) and bias.shape == (40,)
    row = 0
    for l, (w0, b0) in zip(lins, before):
        assert isinstance(l.weight, torch.nn.Parameter) and l.weight.is_contiguous()
        assert l.weight.data_ptr() == weight[row].data_ptr() and l.bias.data_ptr() == bias[row:].data_ptr()
        assert torch.equal(l.weight, w0) and torch.equal(l.bias, b0)   # values survive the move
        row += l.weight.shape[0]
    lins[1].weight.data.copy_(torch.full((8, 16), 3.0))                  # not seen by the version counter
    with torch.no_grad():
        lins[2].bias.mul_(0.0)
    again = _concatenated_params(x, weights, biases)
    assert again[0] is weight and again[1] is bias
    assert torch.equal(weight[8:16], torch.full((8, 16), 3.0)) and torch.equal(bias[16:], torch.zeros(24))
    # a state dict loaded into the modules lands in the fused buffers too
    lins[0].load_state_dict({"weight": torch.ones(8, 16), "bias": torch.ones(8)})
    assert torch.equal(weight[:8], torch.ones(8, 16)) and torch.equal(bias[:8], torch.ones(8))
    # no bias on one projection: zeros in its place, the others still alias
    lin_nb = torch.nn.Linear(16, 8, bias=False)
    lin_b = torch.nn.Linear(16, 8)
    w2, b2, _ = _concatenated_params(x, [lin_nb.weight, lin_b.weight], [None, lin_b.bias])
    assert torch.equal(b2[:8], torch.zeros(8)) and lin_b.bias.data_ptr() == b2[8:].data_ptr()


def test_overlapping_projection_groups_do_not_move_each_others_parameters():
    """A weight that belongs to two sibling groups (shared or tied projections): the first group's fused buffer keeps
    its address and values — a captured graph reads it —, the second group keeps a copy that follows the parameters'
    version counters in place."""
    from kernl_amd.optimizer.linear import _concatenated_params, _fused_params

    torch.manual_seed(0)
    q, k, v = (torch.nn.Linear(16, 8) for _ in range(3))
    x = torch.zeros(2, 16)
    first = _concatenated_params(x, [q.weight, k.weight, v.weight], [q.bias, k.bias, v.bias])
    ptr, snapshot = first[0].data_ptr(), first[0].clone()
    second = _concatenated_params(x, [k.weight, v.weight], [k.bias, v.bias])
    # the second group did not re-point k and v: they still live in the first group's buffer
    assert k.weight.data_ptr() == first[0][8].data_ptr() and v.weight.data_ptr() == first[0][16].data_ptr()
    assert second[0].data_ptr() != k.weight.data_ptr() and torch.equal(second[0], first[0][8:])
    again = _concatenated_params(x, [q.weight, k.weight, v.weight], [q.bias, k.bias, v.bias])
    assert again[0] is first[0] and again[0].data_ptr() == ptr and torch.equal(again[0], snapshot)
    assert _concatenated_params(x, [k.weight, v.weight], [k.bias, v.bias])[0] is second[0]
    # a version-counted write reaches both: the aliased buffer directly, the copy on its next lookup, in place
    with torch.no_grad():
        k.weight.fill_(2.0)
        v.bias.fill_(-1.0)
    assert torch.equal(first[0][8:16], torch.full((8, 16), 2.0))
    refreshed = _concatenated_params(x, [k.weight, v.weight], [k.bias, v.bias])
    assert refreshed[0] is second[0] and torch.equal(second[0][:8], torch.full((8, 16), 2.0))
    assert torch.equal(second[1][8:], torch.full((8,), -1.0))
    assert len(_fused_params) >= 2


def test_add_layer_norm_with_a_scalar_on_either_side_reaches_the_kernel():
    """`layer_norm(1.0 + x)` traces to add(scalar, tensor): the wrapper must add first and call the LayerNorm kernel
    (which refuses CPU tensors here), not look for a dtype on the scalar."""
    from kernl_amd._lib import KernlLibraryError
    from kernl_amd.optimizer.layer_norm import add_layer_norm_wrapper_functional

    x = torch.zeros(2, 8, dtype=torch.float16)
    w, b = torch.ones(8), torch.zeros(8)
    for a, c in ((1.0, x), (x, 1.0), (x[:1], x)):
        with pytest.raises(KernlLibraryError):
            add_layer_norm_wrapper_functional(a, c, (8,), w, b, 1e-5)
    assert w.dtype == torch.float16  # parameters were cast once on the way


def test_interleaved_gate_weights_are_refreshed_in_place():
    """The block-interleaved weight of a gated linear unit is a copy: version-counted writes refresh it on the next
    lookup, other writes through `refresh_fused_parameters()`, always at the same address."""
    from kernl_amd.implementations.linear_layer import interleave_glu_rows
    from kernl_amd.optimizer.linear import _interleaved_params, refresh_fused_parameters

    torch.manual_seed(0)
    gate, value = torch.nn.Linear(16, 64, bias=False), torch.nn.Linear(16, 64, bias=False)
    weight, bias = _interleaved_params(False, gate.weight, None, value.weight, None)
    assert bias is None and torch.equal(weight, interleave_glu_rows(gate.weight.detach(), value.weight.detach()))
    ptr = weight.data_ptr()
    with torch.no_grad():
        gate.weight.mul_(2.0)
    again, _ = _interleaved_params(False, gate.weight, None, value.weight, None)
    assert again is weight and again.data_ptr() == ptr
    assert torch.equal(weight, interleave_glu_rows(gate.weight.detach(), value.weight.detach()))
    value.weight.data.add_(1.0)               # bypasses the version counter
    stale, _ = _interleaved_params(False, gate.weight, None, value.weight, None)
    assert not torch.equal(stale, interleave_glu_rows(gate.weight.detach(), value.weight.detach()))
    assert refresh_fused_parameters() >= 1
    assert weight.data_ptr() == ptr
    assert torch.equal(weight, interleave_glu_rows(gate.weight.detach(), value.weight.detach()))


def test_split_k_dispatch_rule():
    """Single-query attention goes to the split-K kernel only for what that kernel takes: more than 50 keys
    (reference: optimizer/attention.py:45), a power-of-two head size from 8 to 256, 16-byte aligned rows and at most
    65535 rows; everything else stays on the tiled kernel."""
    from kernl_amd.optimizer.attention import SPLIT_K_MAX_ROWS, takes_split_k_kernel

    def qkv(b, h, m, n, d, dtype=torch.float16):
        # one batch entry of memory, expanded over the batch: the real shapes without the gigabytes
        q = torch.zeros((1, h, m, d), dtype=dtype).expand(b, h, m, d)
        k = torch.zeros((1, h, n, d), dtype=dtype).expand(b, h, n, d)
        return q, k, k

    assert takes_split_k_kernel(*qkv(2, 4, 1, 51, 64))
    assert not takes_split_k_kernel(*qkv(2, 4, 1, 50, 64))          # few keys
    assert not takes_split_k_kernel(*qkv(2, 4, 2, 4096, 64))        # more than one query per row
    assert not takes_split_k_kernel(*qkv(2, 4, 1, 4096, 80))        # head size not a power of two
    assert not takes_split_k_kernel(*qkv(2, 4, 1, 4096, 512))       # head size too large
    assert takes_split_k_kernel(*qkv(2047, 32, 1, 128, 128)) and 2047 * 32 <= SPLIT_K_MAX_ROWS
    assert not takes_split_k_kernel(*qkv(2048, 32, 1, 128, 128))    # 65536 rows: beyond the kernel's grid
    q, k, v = qkv(2, 4, 1, 128, 64)
    assert not takes_split_k_kernel(q[..., 1:], k[..., 1:], v[..., 1:])   # rows no longer 16-byte aligned


def test_residual_additions_fold_into_the_projection_before_them():
    """`res + linear(...)` in either operand order becomes one call; a projection with an activation, or one whose
    result is used elsewhere too, keeps its addition."""
    from kernl_amd.optimizer.linear import fuse_residual_into_linears, replace_all_linear

    F = torch.nn.functional

    class Block(torch.nn.Module):
        """Parameters used through F.linear, the form torch.compile hands to a backend."""

        def __init__(self):
            super().__init__()
            self.wa, self.wb, self.wc, self.wd = (torch.nn.Parameter(torch.randn(8, 8)) for _ in range(4))
            self.ba = torch.nn.Parameter(torch.randn(8))

        def forward(self, x, r):
            y = r + F.linear(x, self.wa, self.ba)              # fused
            y = F.linear(y, self.wb, None) + y                 # fused, projection on the left
            y = y + F.relu(F.linear(y, self.wc, None))         # activation in between: stays
            z = F.linear(y, self.wd, None)
            return z + y, z                                    # the projection has a second user: stays

    torch.manual_seed(0)
    m = Block().eval()
    gm = torch.fx.symbolic_trace(m)
    replace_all_linear(gm)
    fuse_residual_into_linears(gm)
    t = _targets(gm)
    assert t.count("linear_residual_wrapper") == 2 and t.count("add") == 2
    nodes = [n for n in gm.graph.nodes if n.op == "call_function" and n.target.__name__ == "linear_residual_wrapper"]
    assert [n.args[3].name for n in nodes] == ["r", nodes[0].name]       # the residual operand of each


def test_row_statistics_ride_in_the_residual_addition_only_where_every_taker_agrees():
    """`fuse_rms_stats_into_residual_adds`: the sum of a residual projection that feeds `rms_*` projections becomes
    element 0 of `linear_residual_stats_wrapper` for ALL its users and element 1 goes to those projections as `rstd=`;
    takers with different eps leave the graph alone; a sum no `rms_*` projection reads keeps its plain wrapper."""
    import operator

    from kernl_amd.optimizer.linear import (fuse_rms_stats_into_residual_adds, linear_residual_wrapper, rms_glu_linear_wrapper,
                                            rms_linear_wrapper)

    def graph(eps_a, eps_b):
        g = torch.fx.Graph()
        x, r, w, gam = (g.placeholder(n) for n in ("x", "r", "w", "gam"))
        h = g.call_function(linear_residual_wrapper, (x, w, None, r))
        a = g.call_function(rms_linear_wrapper, (h, gam, eps_a, w, None))
        b = g.call_function(rms_glu_linear_wrapper, (h, gam, eps_b, w, None, w, None, "silu"))
        plain = g.call_function(linear_residual_wrapper, (a, w, None, h))      # reads the sum as its residual; feeds no norm
        g.output((plain, b))
        return torch.fx.GraphModule(torch.nn.Module(), g)

    gm = graph(1e-6, 1e-6)
    fuse_rms_stats_into_residual_adds(gm)
    nodes = {n.name: n for n in gm.graph.nodes}
    stats = [n for n in gm.graph.nodes if n.op == "call_function" and n.target.__name__ == "linear_residual_stats_wrapper"]
    assert len(stats) == 1 and stats[0].args[4] == 1e-6
    total, rstd = [n for n in gm.graph.nodes if n.op == "call_function" and n.target is operator.getitem]
    assert total.args == (stats[0], 0) and rstd.args == (stats[0], 1)
    takers = [n for n in gm.graph.nodes if n.op == "call_function" and n.target.__name__ in ("rms_linear_wrapper", "rms_glu_linear_wrapper")]
    assert all(n.args[0] is total and n.kwargs["rstd"] is rstd for n in takers) and len(takers) == 2
    plain = [n for n in gm.graph.nodes if n.op == "call_function" and n.target.__name__ == "linear_residual_wrapper"]
    assert len(plain) == 1 and plain[0].args[3] is total
    assert nodes  # (graph still lints)
    gm.graph.lint()

    gm = graph(1e-6, 1e-5)
    fuse_rms_stats_into_residual_adds(gm)
    assert "linear_residual_stats_wrapper" not in _targets(gm)


def test_folded_norm_weights_follow_their_parameters():
    """The prompt path's weights with the RMSNorm weight multiplied into their columns are copies: built once, rewritten
    in place when the projection weight OR the norm weight changes, and dropped with their parameters."""
    from kernl_amd.optimizer.linear import _folded_concatenated_weight, _folded_weight, _fused_params

    w = torch.nn.Parameter(torch.randn(6, 4))
    w2 = torch.nn.Parameter(torch.randn(2, 4))
    g = torch.nn.Parameter(torch.rand(4) + 0.5)
    f1 = _folded_weight(w, g)
    assert torch.equal(f1, w.detach() * g.detach()[None, :]) and _folded_weight(w, g) is f1
    fc = _folded_concatenated_weight([w, w2], g)
    assert fc.shape == (8, 4) and torch.equal(fc, torch.cat([w, w2]).detach() * g.detach()[None, :])
    with torch.no_grad():
        g.mul_(2.0)
    assert _folded_weight(w, g) is f1 and torch.equal(f1, w.detach() * g.detach()[None, :])
    with torch.no_grad():
        w2.add_(1.0)
    assert _folded_concatenated_weight([w, w2], g) is fc and torch.equal(fc, torch.cat([w, w2]).detach() * g.detach()[None, :])
    keys = [_fused_params.key_of((w, g)), _fused_params.key_of((w, w2, g))]
    assert all(k in _fused_params._entries for k in keys)
    del w, w2, g
    import gc

    gc.collect()
    _fused_params._drop_dead()
    assert not any(k in _fused_params._entries for k in keys)


def test_residual_projection_keeps_the_addition_where_the_small_tile_kernels_are_faster(monkeypatch):
    """A residual projection of a decoding step runs as one launch of the weight-streaming kernel — except against a
    small weight, where `kernl_linear_fwd`'s one-launch small-tile kernels win by more than the addition costs."""
    import kernl_amd.implementations.linear_layer as impl
    import kernl_amd.optimizer.linear as opt

    taken = []
    monkeypatch.setattr(impl, "decode_linear_layer", lambda v, w, b, residual=None: taken.append("fused") or residual)
    monkeypatch.setattr(opt, "linear_wrapper_functional", lambda v, w, b: taken.append("separate") or torch.zeros(v.shape[0], w.shape[0], dtype=v.dtype))
    for rows, n, k in ((64, 768, 3072), (1, 4096, 4096), (32, 4096, 4096), (1, 768, 768)):
        x = torch.zeros((rows, k), dtype=torch.float16)
        w = torch.zeros((n, k), dtype=torch.float16)
        opt.linear_residual_wrapper(x, w, None, torch.zeros((rows, n), dtype=torch.float16))
        small = impl.takes_small_problem_kernel(x, w)
        assert taken[-1] == ("separate" if small else "fused"), (rows, n, k)
    assert taken[0] == "separate" and taken[1] == "fused"


def test_few_row_kernel_routing_rule():
    """17 to 128 rows against a weight of at least 2048 x 2048 elements go to the stream-K kernel; fewer rows, small
    weights, a K that is no multiple of 64 and rows that are not 16-byte aligned do not."""
    from kernl_amd.implementations.linear_layer import takes_few_row_kernel

    w = torch.zeros((2048, 2048), dtype=torch.float16)
    rows = lambda m, k=2048: torch.zeros((m, k), dtype=torch.float16)
    assert [takes_few_row_kernel(rows(m), w) for m in (1, 16, 17, 64, 128, 129)] == [False, False, True, True, True, False]
    assert not takes_few_row_kernel(rows(32, 1024), torch.zeros((2048, 1024), dtype=torch.float16))      # small weight
    assert not takes_few_row_kernel(rows(32, 3072), torch.zeros((768, 3072), dtype=torch.float16))       # ... few rows
    assert takes_few_row_kernel(rows(33, 3072), torch.zeros((768, 3072), dtype=torch.float16))           # long K
    assert not takes_few_row_kernel(rows(64, 768), torch.zeros((3072, 768), dtype=torch.float16))        # short K
    assert not takes_few_row_kernel(rows(32, 4104), torch.zeros((2048, 4104), dtype=torch.float16))      # K % 64 != 0
    assert not takes_few_row_kernel(torch.zeros((32, 2052), dtype=torch.float16)[:, :2048], w)           # row stride
    assert not takes_few_row_kernel(rows(32).to(torch.float32), w.to(torch.float32))
    assert takes_few_row_kernel(rows(32).to(torch.bfloat16), w.to(torch.bfloat16))


def test_small_problem_rule_of_the_library():
    """`kernl_linear_small_kind` (no GPU needed): which shapes the linear entry point runs on its small-problem kernels.
    One round of workgroups is the condition throughout; big weights, single rows and long K with many rows are not
    their kind."""
    from kernl_amd import _lib

    kind = _lib.linear_small_kind
    assert kind(16, 768, 3072) == 12 and kind(8, 8192, 1024) == 12      # 16 x 32 tiles, up to 256 of them
    assert kind(8, 8224, 1024) == 0 and kind(7, 768, 3072) == 0 and kind(1, 768, 768) == 0
    assert kind(128, 768, 3072) == 13 and kind(64, 2304, 768) == 13     # 32 x 32 tiles, k-tiles dealt to the waves
    assert kind(256, 1024, 4096) == 13 and kind(288, 1024, 4096) == 14  # 8 x 32 tiles of 32 rows fit, 9 x 32 do not: 64 rows
    assert kind(512, 768, 3072) == 14 and kind(128, 2304, 768) == 14    # 64 x 32 tiles, k-tiles dealt
    assert kind(96, 5440, 768) == 10 and kind(384, 2304, 768) == 11     # shared 32 x 64 / 64 x 64 tiles where those need a second round
    assert kind(256, 3072, 768) == 11 and kind(1024, 1024, 1024) == 11  # 64 x 64 tiles
    assert kind(512, 3072, 768) == 15 and kind(2048, 768, 768) == 15    # short K: 64 x 128 tiles where 64 x 64 need a second round
    assert kind(768, 3072, 768) == 0 and kind(1024, 3072, 768) == 0     # more than 256 tiles of any kind
    assert kind(32, 4096, 4096) == 0 and kind(128, 11008, 4096) == 0    # big weights stay with the streaming kernels
    assert kind(768, 768, 3072) == 11 and kind(1024, 768, 1536) == 11   # long K: one round of 64 x 64 tiles where the dealt ones need two
    assert kind(2048, 1024, 4096) == 0                                  # long K and more than 256 tiles of 64 x 64: split-K
    assert kind(128, 768, 3076) == 0 and kind(0, 768, 768) == 0         # K no multiple of 8: not the MFMA path at all


def test_full_range_index_grids_become_a_view():
    """`x[arange(B)[:, None, None, None], arange(S)[None, None, None, :]]` is x reshaped to [B, 1, 1, S]; partial ranges,
    permuted axes and shifted grids stay gathers."""
    from kernl_amd.optimizer.mask import full_range_index_to_view

    def build(fn):
        gm = torch.fx.symbolic_trace(fn)
        for n in gm.graph.nodes:
            if n.op == "placeholder":
                n.meta["example_value"] = torch.zeros(3, 5, dtype=torch.bool)
        full_range_index_to_view(gm)
        return gm

    def whole(x):
        return x[torch.arange(3)[:, None, None, None], (torch.arange(5) + 0)[None, None, None, :]]

    def partial(x):
        return x[torch.arange(2)[:, None, None, None], torch.arange(5)[None, None, None, :]]

    def swapped(x):
        return x[torch.arange(3)[None, None, None, :], torch.arange(5)[:, None, None, None]]

    def shifted(x):
        return x[torch.arange(3)[:, None], (torch.arange(5) + 1).clamp(max=4)[None, :]]

    x = torch.rand(3, 5) > 0.5
    gm = build(whole)
    assert "reshape" in _targets(gm) and "arange" not in _targets(gm)
    assert torch.equal(gm(x), whole(x)) and gm(x).shape == (3, 1, 1, 5)
    for fn in (partial, swapped, shifted):
        gm = build(fn)
        assert "reshape" not in _targets(gm)
        assert torch.equal(gm(x), fn(x))


def test_embedding_oracle_against_the_library_routines():
    """The oracle of the fused embedding stage is gathers, additions and the LayerNorm oracle: with fp32 tables (no
    rounding between the additions) it must equal F.embedding + F.layer_norm; with fp16 tables the additions round."""
    from oracle import embedding_layer_norm_oracle

    gen = torch.Generator().manual_seed(4)
    tables = [torch.randn((r, 24), generator=gen) for r in (50, 2, 16)]
    ids = [torch.randint(0, 50, (3, 16), generator=gen), torch.randint(0, 2, (3, 16), generator=gen), torch.arange(16)[None, :]]
    w, b = torch.randn(24, generator=gen), torch.randn(24, generator=gen)
    want = torch.nn.functional.layer_norm(sum(torch.nn.functional.embedding(i, t) for i, t in zip(ids, tables)), (24,), w, b, 1e-5)
    torch.testing.assert_close(embedding_layer_norm_oracle(tables, ids, w, b, 1e-5), want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(embedding_layer_norm_oracle(tables[:1], ids[:1], w, None, 1e-5),
                               torch.nn.functional.layer_norm(tables[0][ids[0]], (24,), w, None, 1e-5), rtol=1e-5, atol=1e-5)
    half = [t.half() for t in tables]
    rounded = ((half[0][ids[0]] + half[1][ids[1]]) + half[2][ids[2].expand(3, 16)]).float()   # fp16 additions round each time
    torch.testing.assert_close(embedding_layer_norm_oracle(half, ids, w, b, 1e-5),
                               torch.nn.functional.layer_norm(rounded, (24,), w, b, 1e-5), rtol=1e-5, atol=1e-5)
