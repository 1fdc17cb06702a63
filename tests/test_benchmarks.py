"""The three operators under the `benchmark` fixture at BASELINE's shapes, each beside eager PyTorch on the same
inputs (the way the reference's test/test_attention.py, test_linear_layer.py and test_layer_norm.py time their
kernels: `implementation` is a parameter, results of one shape form a group).  Run with
`-m gpu --benchmark-group-by group -s` to see the tables; every test also checks the value it timed."""
import pytest
import torch

from kernl_amd.implementations.attention import attention_forward, attention_reference
from kernl_amd.implementations.layer_norm import layer_norm
from kernl_amd.implementations.linear_layer import linear_layer

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def short_budgets(benchmark):
    benchmark.warmup_ms, benchmark.rep_ms = 10.0, 40.0   # the suite is a parity suite first


@pytest.mark.parametrize("implementation", ["kernl_amd", "torch"])
@pytest.mark.parametrize("shape", [(32, 12, 512, 64)], ids=["32x12x512x64"])
def test_benchmark_attention(benchmark, shape, implementation, close):
    gen = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn(shape, generator=gen, device="cuda", dtype=torch.half) for _ in range(3))
    out = torch.empty_like(q)
    fn = attention_forward if implementation == "kernl_amd" else attention_reference
    got = benchmark(fn, q, k, v, out, 0.125, False, None)
    sample = slice(0, 2)
    want = attention_reference(q[sample].float(), k[sample].float(), v[sample].float(), torch.empty_like(q[sample]).float(), 0.125, False, None)
    close(got[sample], want, what=f"benchmarked attention ({implementation})")


@pytest.mark.parametrize("implementation", ["kernl_amd", "torch"])
@pytest.mark.parametrize("shape", [(16384, 3072, 768)], ids=["16384x3072x768"])
def test_benchmark_linear_gelu(benchmark, shape, implementation, close):
    M, N, K = shape
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn((M, K), generator=gen, device="cuda", dtype=torch.half)
    w = torch.randn((N, K), generator=gen, device="cuda", dtype=torch.half) * 0.02
    b = torch.randn((N,), generator=gen, device="cuda", dtype=torch.half) * 0.02
    if implementation == "kernl_amd":
        got = benchmark(linear_layer, x, w, b, "fast_gelu")
    else:
        got = benchmark(lambda: torch.nn.functional.gelu(torch.nn.functional.linear(x, w, b), approximate="tanh"))
    want = torch.nn.functional.gelu(torch.nn.functional.linear(x[:256].float(), w.float(), b.float()), approximate="tanh")
    close(got[:256], want, what=f"benchmarked linear ({implementation})")


@pytest.mark.parametrize("implementation", ["kernl_amd", "torch"])
@pytest.mark.parametrize("shape", [(16384, 768)], ids=["16384x768"])
def test_benchmark_layer_norm(benchmark, shape, implementation, close):
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(shape, generator=gen, device="cuda", dtype=torch.half)
    w = torch.randn((shape[1],), generator=gen, device="cuda", dtype=torch.half)
    b = torch.randn((shape[1],), generator=gen, device="cuda", dtype=torch.half)
    if implementation == "kernl_amd":
        got = benchmark(layer_norm, x, w, b, 1e-5)
    else:
        got = benchmark(torch.nn.functional.layer_norm, x, (shape[1],), w, b, 1e-5)
    want = torch.nn.functional.layer_norm(x.float(), (shape[1],), w.float(), b.float(), 1.6e-5)
    close(got, want, scale="magnitude", what=f"benchmarked layer norm ({implementation})")
