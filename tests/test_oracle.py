"""Pins the CPU oracle (no GPU): closed forms against torch library routines, algorithm restatements against the
closed forms, and the invariants / known answers that a dropped term, wrong sign or transposed operand would break.
The reference holds no stored numeric vectors for this path (its tests recompute expectations with torch at run
time); its known-answer material is `closest_power_of_2` (test/test_attention.py:148-157) and the graph-pool answers
(test/test_cuda_graph.py), covered in test_host_logic.py."""
import math

import numpy as np
import pytest
import torch

from oracle import (
    activation_oracle,
    attention_oracle,
    attention_tiled_oracle,
    effective_eps,
    glu_oracle,
    layer_norm_oracle,
    layer_norm_welford_oracle,
    linear_oracle,
    rms_norm_oracle,
    rotary_complex_oracle,
    rotary_oracle,
)


def _qkv(shape, seed=0, n=None):
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(shape, generator=gen)
    kshape = shape if n is None else (shape[0], shape[1], n, shape[3])
    return q, torch.randn(kshape, generator=gen), torch.randn(kshape, generator=gen)


def _brute_force_attention(q, k, v, scale, causal, mask):
    B, H, M, D = q.shape
    N = k.shape[2]
    out = torch.zeros((B, H, M, D), dtype=torch.float64)
    for b in range(B):
        for h in range(H):
            for m in range(M):
                logits = []
                for n in range(N):
                    s = sum(float(q[b, h, m, d]) * float(k[b, h, n, d]) for d in range(D)) * scale
                    if mask is not None:
                        s += float(mask[b if mask.shape[0] > 1 else 0, h if mask.shape[1] > 1 else 0,
                                        m if mask.shape[2] > 1 else 0, n])
                    if causal and n > m:
                        s = -math.inf
                    logits.append(s)
                mx = max(logits)
                w = [math.exp(x - mx) for x in logits]
                z = sum(w)
                for d in range(D):
                    out[b, h, m, d] = sum(w[n] * float(v[b, h, n, d]) for n in range(N)) / z
    return out


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("masked", [False, True])
def test_attention_closed_form_vs_brute_force(causal, masked):
    q, k, v = _qkv((2, 2, 5, 4), seed=1, n=7 if not causal else 5)
    mask = torch.randn((2, 1, 5, k.shape[2]), generator=torch.Generator().manual_seed(2)) if masked else None
    got = attention_oracle(q, k, v, 0.7, causal, mask)
    want = _brute_force_attention(q, k, v, 0.7, causal, mask)
    assert torch.allclose(got.double(), want, atol=1e-5)


def test_attention_matches_torch_sdpa():
    q, k, v = _qkv((2, 3, 33, 16), seed=3)
    got = attention_oracle(q, k, v, 0.25, False, None)
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, scale=0.25)
    assert torch.allclose(got, want, atol=1e-5)
    got_c = attention_oracle(q, k, v, 0.25, True, None)
    want_c = torch.nn.functional.scaled_dot_product_attention(q, k, v, scale=0.25, is_causal=True)
    assert torch.allclose(got_c, want_c, atol=1e-5)


def test_attention_invariants():
    q, k, v = _qkv((1, 2, 40, 8), seed=4)
    # V = 1 => O = 1
    assert torch.allclose(attention_oracle(q, k, torch.ones_like(v), 0.3), torch.ones_like(q), atol=1e-6)
    # causal row 0 attends key 0 only
    assert torch.allclose(attention_oracle(q, k, v, 0.3, True)[:, :, 0], v[:, :, 0], atol=1e-6)
    # permuting the keys (and values with them) changes nothing without a causal mask
    perm = torch.randperm(40, generator=torch.Generator().manual_seed(5))
    assert torch.allclose(attention_oracle(q, k[:, :, perm], v[:, :, perm], 0.3), attention_oracle(q, k, v, 0.3), atol=1e-5)
    # keys behind a -inf padding mask are as good as absent
    mask = torch.zeros((1, 1, 1, 40))
    mask[..., 25:] = float("-inf")
    assert torch.allclose(attention_oracle(q, k, v, 0.3, False, mask), attention_oracle(q, k[:, :, :25], v[:, :, :25], 0.3), atol=1e-5)
    # the mask is ADDED (sign check): a large positive bias on one key makes the output that key's value
    bias = torch.zeros((1, 1, 1, 40))
    bias[..., 7] = 200.0
    assert torch.allclose(attention_oracle(q, k, v, 0.3, False, bias), v[:, :, 7:8].expand_as(q), atol=1e-4)


@pytest.mark.parametrize("seq", [8, 16, 33, 128, 257])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("mask_kind", ["none", "vector", "matrix"])
def test_tiled_restatement_equals_closed_form(seq, causal, mask_kind):
    q, k, v = _qkv((2, 2, seq, 8), seed=seq)
    gen = torch.Generator().manual_seed(seq + 1)
    mask = None
    if mask_kind == "vector":
        mask = torch.zeros((2, 1, 1, seq))
        mask[1, ..., seq // 2 + 1:] = float("-inf")
    elif mask_kind == "matrix":
        mask = torch.rand((1, 2, seq, seq), generator=gen)
    got = attention_tiled_oracle(q.numpy(), k.numpy(), v.numpy(), 0.3, causal, None if mask is None else mask.numpy())
    want = attention_oracle(q, k, v, 0.3, causal, mask)
    assert np.allclose(got, want.double().numpy(), atol=1e-5)


def test_tiled_restatement_fully_masked_row_is_uniform_average():
    q, k, v = _qkv((1, 1, 4, 8), seed=9, n=20)
    mask = np.full((1, 1, 1, 20), -np.inf, dtype=np.float32)
    got = attention_tiled_oracle(q.numpy(), k.numpy(), v.numpy(), 0.5, False, mask)
    assert np.isfinite(got).all()
    assert np.allclose(got, v.double().mean(dim=2, keepdim=True).expand(-1, -1, 4, -1).numpy(), atol=1e-6)
    # fp16 clamp value: the add does not absorb q·kᵀ, so the result is the ordinary softmax over all keys
    got16 = attention_tiled_oracle(q.numpy(), k.numpy(), v.numpy(), 0.5, False, mask.astype(np.float16))
    assert np.allclose(got16, attention_oracle(q, k, v, 0.5).double().numpy(), atol=1e-6)


def test_activation_known_points():
    x = torch.tensor([0.0, -1.0, 1.0, 3.0, -3.0])
    assert torch.equal(activation_oracle(x, "relu"), torch.tensor([0.0, 0.0, 1.0, 3.0, 0.0]))
    gelu = activation_oracle(x, "gelu")
    assert gelu[0] == 0 and abs(gelu[2].item() - 0.8413447) < 1e-6 and abs(gelu[1].item() + 0.1586553) < 1e-6
    fast = activation_oracle(x, "fast_gelu")
    assert fast[0] == 0 and abs(fast[2].item() - 0.8411920) < 1e-6
    assert torch.allclose(activation_oracle(x, "tanh"), torch.tanh(x))
    assert torch.allclose(activation_oracle(x, "gelu"), torch.nn.functional.gelu(x), atol=1e-6)
    assert torch.allclose(activation_oracle(x, "fast_gelu"), torch.nn.functional.gelu(x, approximate="tanh"), atol=1e-6)
    assert torch.allclose(activation_oracle(x, "silu"), torch.nn.functional.silu(x), atol=1e-6)
    assert torch.equal(activation_oracle(x, "no-such-activation"), x)


def test_linear_closed_form():
    gen = torch.Generator().manual_seed(0)
    x, w, b = torch.randn((3, 7, 16), generator=gen), torch.randn((5, 16), generator=gen), torch.randn((5,), generator=gen)
    assert torch.allclose(linear_oracle(x, w, b), torch.nn.functional.linear(x, w, b), atol=1e-5)
    assert torch.allclose(linear_oracle(x, w, None, "relu"), torch.relu(torch.nn.functional.linear(x, w)), atol=1e-5)
    # weight is [N, K] (a transposed operand would not even have the right shape here) and strided x works
    xt = torch.randn((16, 7), generator=gen)
    assert torch.allclose(linear_oracle(xt.mT, w, b), torch.nn.functional.linear(xt.t(), w, b), atol=1e-5)
    out, pre = linear_oracle(x, w, b, "gelu", return_act_inputs=True)
    assert torch.allclose(pre, torch.nn.functional.linear(x, w, b), atol=1e-5)
    assert torch.allclose(out, torch.nn.functional.gelu(pre), atol=1e-6)
    # hand-computed 2x2 case: x = [[1, 2]], w = [[3, 4], [5, 6]], b = [1, -1] -> [[12, 16]]
    assert torch.equal(linear_oracle(torch.tensor([[1.0, 2.0]]), torch.tensor([[3.0, 4.0], [5.0, 6.0]]), torch.tensor([1.0, -1.0])),
                       torch.tensor([[12.0, 16.0]]))


def test_layer_norm_closed_form_and_large_mean():
    gen = torch.Generator().manual_seed(0)
    x = -20 + 0.5 * torch.randn((64, 1024), generator=gen)  # reference test/test_layer_norm.py:58
    w, b = torch.rand((1024,), generator=gen), torch.randn((1024,), generator=gen)
    assert torch.allclose(layer_norm_oracle(x, w, b, 1e-5), torch.nn.functional.layer_norm(x, (1024,), w, b, 1e-5), atol=2e-5)
    # known answer: row [1, 2, 3, 4], unit weight, eps 0 -> (x - 2.5) / sqrt(1.25)
    row = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    want = (row - 2.5) / math.sqrt(1.25)
    assert torch.allclose(layer_norm_oracle(row, torch.ones(4), None, 0.0), want, atol=1e-6)


def test_rms_norm_closed_form():
    gen = torch.Generator().manual_seed(1)
    x, w = torch.randn((8, 300), generator=gen), torch.rand((300,), generator=gen)
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-6) * w
    assert torch.allclose(rms_norm_oracle(x, w, 1e-6), want, atol=1e-6)
    # constant row c: x / |c| (eps 0)
    assert torch.allclose(rms_norm_oracle(torch.full((1, 16), -3.0), torch.ones(16), 0.0), torch.full((1, 16), -1.0), atol=1e-6)
    assert torch.allclose(rms_norm_oracle(x, w, 1e-6), torch.nn.functional.rms_norm(x, (300,), w, 1e-6), atol=1e-5)


@pytest.mark.parametrize("n", [128, 512, 1024, 4096, 5000, 9000])
@pytest.mark.parametrize("rms", [False, True])
def test_welford_restatement_equals_closed_form(n, rms):
    gen = torch.Generator().manual_seed(n)
    x = -20 + 0.5 * torch.randn((6, n), generator=gen)
    w, b = torch.rand((n,), generator=gen), torch.randn((n,), generator=gen)
    out, mean, rstd = layer_norm_welford_oracle(x.numpy(), w.numpy(), None if rms else b.numpy(), 1e-5, rms)
    want = rms_norm_oracle(x, w, 1e-5) if rms else layer_norm_oracle(x, w, b, 1e-5)
    assert np.allclose(out, want.numpy(), atol=2e-3, rtol=1e-4)
    if rms:
        assert np.all(mean == 0)
    else:
        assert np.allclose(mean, x.mean(-1).numpy(), atol=1e-4)
        assert np.allclose(rstd, (1 / torch.sqrt(x.var(-1, unbiased=False) + 1e-5)).numpy(), rtol=2e-3)


def test_effective_eps():
    assert effective_eps(1e-12, torch.float16) == 1.6e-5
    assert effective_eps(1e-3, torch.float16) == 1e-3
    assert effective_eps(1e-12, torch.bfloat16) == 1e-12
    assert effective_eps(1e-12, torch.float32) == 1e-12


def _angles(S, D, theta=10000.0):
    inv_freq = 1.0 / (theta ** (torch.arange(0, D, 2).float() / D))
    return torch.outer(torch.arange(S).float(), inv_freq)  # [S, D/2]


def _tables(angles):
    emb = torch.cat((angles, angles), dim=-1)
    return emb.cos(), emb.sin()


def test_rotary_half_split_equals_reference_complex_product():
    """The half-split form on features permuted [even..., odd...] is the reference's complex multiplication."""
    gen = torch.Generator().manual_seed(0)
    B, H, S, D = 2, 3, 17, 16
    x = torch.randn((B, H, S, D), generator=gen)
    ang = _angles(S, D)
    ref = rotary_complex_oracle(x, ang)  # interleaved layout
    to_half = torch.cat((torch.arange(0, D, 2), torch.arange(1, D, 2)))
    cos, sin = _tables(ang)
    out = rotary_oracle(x[..., to_half], cos, sin)
    assert torch.allclose(out, ref[..., to_half], atol=1e-6, rtol=1e-6)


def test_rotary_known_answers():
    gen = torch.Generator().manual_seed(1)
    S, D = 5, 8
    x = torch.randn((1, 2, S, D), generator=gen)
    zero = torch.zeros((S, D // 2))
    assert torch.equal(rotary_oracle(x, *_tables(zero)), x)
    assert torch.allclose(rotary_complex_oracle(x, zero), x)
    # quarter turn: the unit vector on feature 0 moves to its partner, with a plus sign; the partner moves to minus
    quarter = torch.full((S, D // 2), math.pi / 2)
    e0 = torch.zeros((1, 1, S, D))
    e0[..., 0] = 1.0
    out = rotary_oracle(e0, *_tables(quarter))
    expect = torch.zeros_like(e0)
    expect[..., D // 2] = 1.0
    assert torch.allclose(out, expect, atol=1e-6)
    eh = torch.zeros((1, 1, S, D))
    eh[..., D // 2] = 1.0
    expect = torch.zeros_like(eh)
    expect[..., 0] = -1.0
    assert torch.allclose(rotary_oracle(eh, *_tables(quarter)), expect, atol=1e-6)
    ec = torch.zeros((1, 1, S, D))
    ec[..., 0] = 1.0  # real part of pair 0 -> imaginary part of pair 0
    expect = torch.zeros_like(ec)
    expect[..., 1] = 1.0
    assert torch.allclose(rotary_complex_oracle(ec, quarter), expect, atol=1e-6)
    # angles add, norms of each pair are preserved
    a, b = _angles(S, D), 0.37 * _angles(S, D) + 0.1
    twice = rotary_oracle(rotary_oracle(x, *_tables(a)), *_tables(b))
    assert torch.allclose(twice, rotary_oracle(x, *_tables(a + b)), atol=1e-5)
    out = rotary_oracle(x, *_tables(a))
    pair_norm = lambda t: t[..., : D // 2] ** 2 + t[..., D // 2:] ** 2
    assert torch.allclose(pair_norm(out), pair_norm(x), atol=1e-5)


def test_glu_closed_form_and_known_answers():
    gen = torch.Generator().manual_seed(4)
    x = torch.randn((9, 24), generator=gen)
    wg, wv = torch.randn((16, 24), generator=gen), torch.randn((16, 24), generator=gen)
    bg, bv = torch.randn((16,), generator=gen), torch.randn((16,), generator=gen)
    F = torch.nn.functional
    out = glu_oracle(x, wg, bg, wv, bv, "silu")
    assert torch.allclose(out, F.silu(F.linear(x, wg, bg)) * F.linear(x, wv, bv), atol=1e-5, rtol=1e-5)
    a, b = x @ wg.T + bg, x @ wv.T + bv  # the two accumulators of the reference kernel
    assert torch.allclose(out, (a * torch.sigmoid(a)) * b, atol=1e-5, rtol=1e-5)
    assert torch.allclose(glu_oracle(x, wg, None, wv, None, "fast_gelu"),
                          F.gelu(F.linear(x, wg), approximate="tanh") * F.linear(x, wv), atol=1e-5, rtol=1e-5)
    # a zero gate silences the unit; a constant value of one leaves act(gate)
    assert torch.equal(glu_oracle(x, torch.zeros_like(wg), None, wv, bv, "silu"), torch.zeros((9, 16)))
    ones = glu_oracle(x, wg, bg, torch.zeros_like(wv), torch.ones_like(bv), "silu")
    assert torch.allclose(ones, F.silu(F.linear(x, wg, bg)), atol=1e-6)
    # gate and value are not interchangeable
    assert not torch.allclose(out, glu_oracle(x, wv, bv, wg, bg, "silu"), atol=1e-3)


def test_attention_oracle_start_position_is_a_row_window_of_full_causal_attention():
    """Causal attention of M new rows at positions s.. over N = s + M keys equals rows s.. of the ordinary (top-left
    aligned) causal attention of the whole sequence; keys beyond the horizon of the last row change nothing; and
    the element-by-element rule (key n visible to row m iff n <= m + s) holds in a scalar loop."""
    gen = torch.Generator().manual_seed(31)
    s_pos, M, D = 37, 21, 8
    N = s_pos + M
    q_all = torch.randn((1, 2, N, D), generator=gen)
    k = torch.randn((1, 2, N, D), generator=gen)
    v = torch.randn((1, 2, N, D), generator=gen)
    full = attention_oracle(q_all, k, v, 0.4, True, None)
    part = attention_oracle(q_all[:, :, s_pos:], k, v, 0.4, True, None, start_position=s_pos)
    assert torch.allclose(part, full[:, :, s_pos:], atol=1e-6)
    # extra keys behind the last visible one are ignored
    k_more = torch.cat((k, torch.randn((1, 2, 9, D), generator=gen)), dim=2)
    v_more = torch.cat((v, torch.randn((1, 2, 9, D), generator=gen)), dim=2)
    assert torch.allclose(attention_oracle(q_all[:, :, s_pos:], k_more, v_more, 0.4, True, None, start_position=s_pos), part, atol=1e-6)
    # scalar restatement of one row
    m = 5
    row = q_all[0, 1, s_pos + m]
    scores = [float(row @ k[0, 1, n]) * 0.4 for n in range(N) if n <= m + s_pos]
    w = torch.softmax(torch.tensor(scores), dim=0)
    expect = sum(w[n] * v[0, 1, n] for n in range(len(scores)))
    assert torch.allclose(part[0, 1, m], expect, atol=1e-5)


def test_e5m2_decode_oracle_against_library_and_fp16_upper_byte():
    """Every one of the 256 codes: equal to torch.float8_e5m2 widened by the library, and equal to the fp16 value whose
    upper byte is the code and whose lower byte is zero (nan compared as nan)."""
    from oracle import e5m2_decode_oracle
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    got = e5m2_decode_oracle(codes)
    lib = codes.view(torch.float8_e5m2).to(torch.float32)
    upper = (codes.to(torch.int32) << 8).to(torch.int16).view(torch.float16).to(torch.float32)
    for other in (lib, upper):
        assert torch.equal(torch.isnan(got), torch.isnan(other))
        ok = ~torch.isnan(got)
        assert torch.equal(got[ok], other[ok])
    # known values: 0x3C = 1.0, 0x40 = 2.0, 0xC5 = -5.0, 0x01 = 2^-16 (smallest subnormal), 0x7B = 57344 (largest finite)
    for code, value in ((0x3C, 1.0), (0x40, 2.0), (0xC5, -5.0), (0x01, 2.0 ** -16), (0x7B, 57344.0)):
        assert got[code].item() == value
