"""GPU parity of the fused rotary position embedding against the CPU oracle.

The reference tests its rotation against the eager complex product of its Llama model
(experimental/llama-v2/test/test_rbe.py, sizes 1..2 x 9..128 tokens x 4096 features); the cases here cover the same
idea on the half-split convention: Llama-shaped heads, strided [B,S,H,D]-backed inputs, broadcast and per-batch
tables, table dtypes, odd sizes that take the element-wise path, and the full Llama-7B prefill shape.
"""
import pytest
import torch

from kernl_amd.implementations.rotary import rotary_forward
from oracle import rotary_oracle

pytestmark = pytest.mark.gpu


def _tables(B, S, D, dtype, gen, theta=10000.0, start=0):
    inv_freq = 1.0 / (theta ** (torch.arange(0, D, 2).float() / D))
    pos = torch.arange(start, start + S).float()[None, :].expand(B, S)
    ang = pos[..., None] * inv_freq  # [B, S, D/2]
    emb = torch.cat((ang, ang), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=["fp16", "bf16", "fp32"])
@pytest.mark.parametrize("shape", [(1, 32, 2048, 128), (2, 4, 100, 64), (3, 5, 17, 32), (1, 2, 9, 6), (2, 1, 1, 128), (1, 3, 33, 80)],
                         ids=lambda s: "x".join(map(str, s)))
def test_rotary_vs_oracle(shape, dtype, close):
    gen = torch.Generator().manual_seed(0)
    B, H, S, D = shape
    # the layout a decoder hands over: [B,S,H*D] projection output viewed as [B,S,H,D] and transposed
    x = torch.randn((B, S, H, D), generator=gen).to(dtype).transpose(1, 2)
    cos, sin = _tables(1, S, D, dtype, gen)
    cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)  # [1,1,S,D]
    print(f"case {shape} {dtype}", flush=True)
    out = rotary_forward(x.cuda(), cos.cuda(), sin.cuda())
    torch.cuda.synchronize()
    assert out.dtype == dtype and out.stride() == x.stride()
    close(out, rotary_oracle(x, cos, sin), dtype, scale="magnitude", what=f"rotary {shape}")


@pytest.mark.parametrize("table_dtype", [torch.float32, torch.float16, torch.bfloat16], ids=["t-fp32", "t-fp16", "t-bf16"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
def test_rotary_table_dtypes_and_per_batch_positions(dtype, table_dtype, close):
    gen = torch.Generator().manual_seed(1)
    B, H, S, D = 3, 4, 50, 64
    x = torch.randn((B, H, S, D), generator=gen).to(dtype)
    cos, sin = _tables(B, S, D, table_dtype, gen, start=1000)
    cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)  # [B,1,S,D]
    out = rotary_forward(x.cuda(), cos.cuda(), sin.cuda())
    torch.cuda.synchronize()
    out_dtype = torch.result_type(x, cos)
    assert out.dtype == out_dtype
    close(out, rotary_oracle(x, cos, sin), torch.float16 if out_dtype == torch.float32 else out_dtype, scale="magnitude", what="rotary tables")


def test_rotary_general_tables_and_strides(close):
    """Tables with different values in the two halves and per-head entries, x with a non-unit feature stride."""
    gen = torch.Generator().manual_seed(2)
    B, H, S, D = 2, 3, 21, 16
    x = torch.randn((B, H, D, S), generator=gen).half().transpose(2, 3)  # feature stride S
    cos = torch.randn((B, H, S, D), generator=gen).half()
    sin = torch.randn((1, H, S, 2 * D), generator=gen).half()[..., ::2].expand(B, H, S, D)
    with pytest.raises(AssertionError):
        rotary_forward(x.cuda(), cos.cuda()[:, :1], sin.cuda())
    cos_b = cos[:1]
    sin_b = sin[:1]
    out = rotary_forward(x.cuda(), cos_b.cuda(), sin_b.cuda())
    torch.cuda.synchronize()
    close(out, rotary_oracle(x, cos_b, sin_b), scale="magnitude", what="rotary general")
    out = rotary_forward(x.cuda(), cos.cuda(), sin.cuda().contiguous())
    torch.cuda.synchronize()
    close(out, rotary_oracle(x, cos, sin), scale="magnitude", what="rotary per-batch per-head")


def test_rotary_round_trip_at_full_size():
    """Rotating by the angles and then by their negatives returns the input (fp16 rounding apart) at the Llama-7B
    prefill shape, where the oracle comparison above already ran once."""
    gen = torch.Generator().manual_seed(3)
    B, H, S, D = 4, 32, 2048, 128
    x = torch.randn((B, S, H, D), generator=gen).half().transpose(1, 2).cuda()
    cos, sin = _tables(1, S, D, torch.float32, gen)
    cos, sin = cos.unsqueeze(1).cuda(), sin.unsqueeze(1).cuda()
    there = rotary_forward(x, cos, sin)
    back = rotary_forward(there.half(), cos, -sin)
    torch.cuda.synchronize()
    err = (back.float() - x.float()).abs().max().item()
    assert err <= 4e-3, err


def test_rotary_argument_errors():
    x = torch.zeros((1, 2, 4, 7), dtype=torch.float16, device="cuda")
    t = torch.zeros((1, 1, 4, 7), dtype=torch.float16, device="cuda")
    with pytest.raises(AssertionError):
        rotary_forward(x, t, t)  # odd feature size
    x = torch.zeros((1, 2, 4, 8), dtype=torch.float16, device="cuda")
    t = torch.zeros((1, 1, 5, 8), dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        rotary_forward(x, t, t)  # table positions do not match
